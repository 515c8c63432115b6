// Implementation of the nt_compat facade on the C ABI of libntgemm.so: host tensors through the host-pointer
// entry points, device tensors (DeviceType::HIP) through the `_dev` ones on the default stream.
// Every validation happens here, before any device work, with the reference's messages.
#include "nt_compat.h"

#include "../../include/ntgemm.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <random>
#include <sstream>

namespace nt {

int64_t dtype_size(DType dt) { return ntg_dtype_size(static_cast<int>(dt)); }

const char* dtype_name(DType dt) {
    switch (dt) {
    case DType::Float16: return "Float16"; case DType::Float32: return "Float32"; case DType::Float64: return "Float64";
    case DType::BFloat16: return "BFloat16"; case DType::int8: return "int8"; case DType::int16: return "int16";
    case DType::int32: return "int32"; case DType::int64: return "int64"; case DType::uint8: return "uint8";
    case DType::uint16: return "uint16"; case DType::uint32: return "uint32"; case DType::uint64: return "uint64";
    case DType::Complex32: return "Complex32"; case DType::Complex64: return "Complex64"; case DType::Complex128: return "Complex128";
    case DType::Bool: return "Bool"; case DType::TensorObj: return "TensorObj";
    default: return "unsupported";
    }
}

namespace utils {
void throw_exception(bool ok, const std::string& message) {
    if (!ok) throw nt_error(message);
}
}  // namespace utils

std::string shape_str(const SizeRef& s) {
    std::ostringstream o;
    o << "{";
    for (size_t i = 0; i < s.size(); ++i) o << (i ? "," : "") << s[i];
    o << "}";
    return o.str();
}

static int64_t prod(const SizeRef& s, size_t from = 0, size_t to = (size_t)-1) {
    int64_t p = 1;
    for (size_t i = from; i < std::min(to, s.size()); ++i) p *= s[i];
    return p;
}

static SizeRef dense_strides(const SizeRef& shape) {
    SizeRef st(shape.size());
    int64_t acc = 1;
    for (int64_t i = (int64_t)shape.size() - 1; i >= 0; --i) { st[i] = acc; acc *= shape[i]; }
    return st;
}

// ------------------------------------------------------------------------------------------ Tensor

static void hip_check(hipError_t e, const char* what) {
    if (e != hipSuccess) throw utils::nt_error(std::string(what) + ": " + hipGetErrorString(e));
}

static std::shared_ptr<char> device_alloc(size_t bytes) {
    void* p = nullptr;
    hip_check(hipMalloc(&p, bytes), "hipMalloc");
    return std::shared_ptr<char>(static_cast<char*>(p), [](char* q) { (void)hipFree(q); });
}

// Scratch for the `_dev` convolutions and products: one buffer per thread that only grows.  All device work of this facade is
// issued on the default stream, so a later call reuses it safely after the earlier one in stream order.
static void* device_workspace(int64_t bytes) {
    static thread_local std::shared_ptr<char> buf;
    static thread_local int64_t cap = 0;
    if (bytes <= 0) return nullptr;
    if (bytes > cap) {
        hip_check(hipDeviceSynchronize(), "hipDeviceSynchronize");     // kernels may still use the smaller buffer
        buf.reset();
        buf = device_alloc((size_t)bytes);
        cap = bytes;
    }
    return buf.get();
}

// Pointer tables of a list product: copied to a device buffer this thread keeps (it only grows), through a pinned host buffer, on
// the default stream.  The copy is ordered behind the kernels of the previous call that still read the device buffer; the
// event says when the pinned buffer may be overwritten.  Nothing is allocated, freed or waited for in the steady state.
namespace {
struct TableBuffers {
    std::shared_ptr<char> dev;
    char* pinned = nullptr;
    int64_t cap = 0;
    hipEvent_t copied = nullptr;
    ~TableBuffers() {
        if (pinned) (void)hipHostFree(pinned);
        if (copied) (void)hipEventDestroy(copied);
    }
};
}  // namespace
static void* upload_table(const void* src, int64_t bytes) {
    static thread_local TableBuffers tb;
    if (bytes > tb.cap) {
        hip_check(hipDeviceSynchronize(), "hipDeviceSynchronize");     // kernels may still read the smaller table
        if (tb.pinned) { (void)hipHostFree(tb.pinned); tb.pinned = nullptr; }
        tb.dev.reset();
        tb.cap = 0;
        tb.dev = device_alloc((size_t)bytes);
        void* h = nullptr;
        hip_check(hipHostMalloc(&h, (size_t)bytes, hipHostMallocDefault), "hipHostMalloc");
        tb.pinned = static_cast<char*>(h);
        tb.cap = bytes;
        if (!tb.copied) hip_check(hipEventCreateWithFlags(&tb.copied, hipEventDisableTiming), "hipEventCreate");
    } else {
        hip_check(hipEventSynchronize(tb.copied), "hipEventSynchronize");   // the previous copy has left the pinned buffer
    }
    std::memcpy(tb.pinned, src, (size_t)bytes);
    hip_check(hipMemcpyAsync(tb.dev.get(), tb.pinned, (size_t)bytes, hipMemcpyHostToDevice, nullptr), "hipMemcpyAsync (pointer tables)");
    hip_check(hipEventRecord(tb.copied, nullptr), "hipEventRecord");
    return tb.dev.get();
}

Tensor::Tensor(SizeRef shape, DType dt, DeviceType dev) : shape_(std::move(shape)), dtype_(dt), device_(dev) {
    const int64_t es = dtype_size(dt);
    utils::throw_exception(es > 0, std::string("dtype ") + dtype_name(dt) + " has no storage in nt_compat");
    utils::throw_exception(dev == DeviceType::CPU || dev == DeviceType::HIP, "nt_compat tensors live on DeviceType::CPU or DeviceType::HIP");
    for (int64_t d : shape_) utils::throw_exception(d >= 0, "negative dimension in shape " + shape_str(shape_));
    strides_ = dense_strides(shape_);
    const size_t bytes = (size_t)std::max<int64_t>(1, prod(shape_) * es);
    if (dev == DeviceType::HIP) storage_ = device_alloc(bytes);
    else storage_ = std::shared_ptr<char>(static_cast<char*>(::operator new(bytes)), [](char* p) { ::operator delete(p); });
}

Tensor Tensor::to(DeviceType dev) const {
    utils::throw_exception(!is_null(), "cannot move a null tensor");
    utils::throw_exception(dev == DeviceType::CPU || dev == DeviceType::HIP, "nt_compat tensors live on DeviceType::CPU or DeviceType::HIP");
    if (dev == device_) return *this;
    const int64_t es = dtype_size(dtype_);
    if (dev == DeviceType::HIP) {
        const Tensor src = contiguous();
        Tensor out(shape_, dtype_, DeviceType::HIP);
        if (numel()) hip_check(hipMemcpy(out.data_ptr(), src.data_ptr(), (size_t)(numel() * es), hipMemcpyHostToDevice), "hipMemcpy to device");
        out.mutable_ = mutable_;
        return out;
    }
    // device -> host: the elements the view spans are copied as they lie, the strides are applied on the host
    int64_t span = numel() ? 1 : 0;
    for (size_t d = 0; d < shape_.size() && numel(); ++d) span += (shape_[d] - 1) * strides_[d];
    Tensor raw({std::max<int64_t>(span, 1)}, dtype_);
    if (span) hip_check(hipMemcpy(raw.data_ptr(), data_ptr(), (size_t)(span * es), hipMemcpyDeviceToHost), "hipMemcpy to host");
    Tensor out = raw;
    out.shape_ = shape_;
    out.strides_ = strides_;
    out.mutable_ = mutable_;
    return out.is_contiguous() ? out : out.clone();
}

int64_t Tensor::numel() const { return is_null() ? 0 : prod(shape_); }

bool Tensor::is_contiguous() const {
    int64_t acc = 1;
    for (int64_t i = dims() - 1; i >= 0; --i) {
        if (shape_[i] != 1 && strides_[i] != acc) return false;
        acc *= shape_[i];
    }
    return true;
}

Tensor Tensor::clone() const {
    utils::throw_exception(!is_null(), "cannot clone a null tensor");
    if (is_device()) {
        if (!is_contiguous()) return cpu().to(DeviceType::HIP);      // (strided device views are rare on this path: via the host)
        Tensor out(shape_, dtype_, DeviceType::HIP);
        if (numel()) hip_check(hipMemcpy(out.data_ptr(), data_ptr(), (size_t)(numel() * dtype_size(dtype_)), hipMemcpyDeviceToDevice), "hipMemcpy on device");
        return out;
    }
    Tensor out(shape_, dtype_);
    const int64_t es = dtype_size(dtype_), n = numel();
    if (is_contiguous()) {
        std::memcpy(out.data_ptr(), data_ptr(), (size_t)(n * es));
        return out;
    }
    const char* src = static_cast<const char*>(data_ptr());
    char* dst = static_cast<char*>(out.data_ptr());
    SizeRef idx(shape_.size(), 0);
    for (int64_t lin = 0; lin < n; ++lin) {
        int64_t off = 0;
        for (size_t d = 0; d < idx.size(); ++d) off += idx[d] * strides_[d];
        std::memcpy(dst + lin * es, src + off * es, (size_t)es);
        for (int64_t d = (int64_t)idx.size() - 1; d >= 0; --d) {
            if (++idx[d] < shape_[d]) break;
            idx[d] = 0;
        }
    }
    return out;
}

Tensor Tensor::view(SizeRef shape) const {
    utils::throw_exception(is_contiguous(), "view needs a contiguous tensor");
    int64_t known = 1, unknown = -1;
    for (size_t i = 0; i < shape.size(); ++i) {
        if (shape[i] == -1) { utils::throw_exception(unknown < 0, "only one -1 allowed in view"); unknown = (int64_t)i; }
        else known *= shape[i];
    }
    if (unknown >= 0) { utils::throw_exception(known != 0 && numel() % known == 0, "view shape does not divide numel"); shape[(size_t)unknown] = numel() / known; }
    utils::throw_exception(prod(shape) == numel(), "view of " + shape_str(shape_) + " as " + shape_str(shape) + " changes numel");
    Tensor out = *this;
    out.shape_ = shape;
    out.strides_ = dense_strides(shape);
    return out;
}

Tensor Tensor::transpose(int64_t a, int64_t b) const {
    const int64_t nd = dims();
    if (a < 0) a += nd;
    if (b < 0) b += nd;
    utils::throw_exception(a >= 0 && a < nd && b >= 0 && b < nd, "transpose dims out of range");
    Tensor out = *this;
    std::swap(out.shape_[(size_t)a], out.shape_[(size_t)b]);
    std::swap(out.strides_[(size_t)a], out.strides_[(size_t)b]);
    return out;
}

Tensor Tensor::unsqueeze_front(int64_t n) const {
    Tensor out = *this;
    for (int64_t i = 0; i < n; ++i) { out.shape_.insert(out.shape_.begin(), 1); out.strides_.insert(out.strides_.begin(), 0); }
    return out;
}

Tensor Tensor::item(int64_t i) const {
    utils::throw_exception(is_contiguous() && dims() >= 2, "item needs a contiguous tensor of matrices");
    const int64_t mat = shape_[(size_t)dims() - 1] * shape_[(size_t)dims() - 2];
    Tensor out = *this;
    out.shape_ = {shape_[(size_t)dims() - 2], shape_[(size_t)dims() - 1]};
    out.strides_ = dense_strides(out.shape_);
    out.offset_ = offset_ + i * mat * dtype_size(dtype_);
    return out;
}

TensorList Tensor::split_axis(int64_t axis) const {
    utils::throw_exception(!is_null() && is_contiguous() && dims() >= 2, "split_axis needs a contiguous tensor of two or more dimensions");
    utils::throw_exception(axis == 0, "nt_compat splits along axis 0 only");
    TensorList out;
    const int64_t per = numel() / std::max<int64_t>(shape_[0], 1);
    for (int64_t i = 0; i < shape_[0]; ++i) {
        Tensor t = *this;
        t.offset_ = offset_ + i * per * dtype_size(dtype_);
        t.shape_.assign(shape_.begin() + 1, shape_.end());
        t.strides_ = dense_strides(t.shape_);
        out.push_back(std::move(t));
    }
    return out;
}

template <class T>
static void sum_as_t(const Tensor& src, Tensor& dst, const SizeRef& tgt_padded) {
    // src contiguous with shape S; dst contiguous with shape tgt_padded (same rank, dims equal or 1)
    const SizeRef& S = src.shape();
    const int64_t n = src.numel();
    T* d = dst.data<T>();
    for (int64_t i = 0; i < dst.numel(); ++i) d[i] = T(0);
    const T* s = src.data<T>();
    const SizeRef dst_st = dense_strides(tgt_padded);
    SizeRef idx(S.size(), 0);
    for (int64_t lin = 0; lin < n; ++lin) {
        int64_t off = 0;
        for (size_t k = 0; k < S.size(); ++k) off += (tgt_padded[k] == 1 ? 0 : idx[k]) * dst_st[k];
        d[off] += s[lin];
        for (int64_t k = (int64_t)S.size() - 1; k >= 0; --k) {
            if (++idx[(size_t)k] < S[(size_t)k]) break;
            idx[(size_t)k] = 0;
        }
    }
}

// grad += in_grad with broadcasting reduced back by sum_as (nt/functional/tensor_files/operators.cpp:175-187)
Tensor Tensor::sum_leading(const SizeRef& target) const {
    Tensor src = contiguous();
    utils::throw_exception((int64_t)target.size() <= dims(), "sum_as target has more dims than the source");
    SizeRef padded(shape_.size(), 1);
    for (size_t i = 0; i < target.size(); ++i) padded[shape_.size() - target.size() + i] = target[i];
    for (size_t i = 0; i < padded.size(); ++i)
        utils::throw_exception(padded[i] == 1 || padded[i] == shape_[i], "cannot reduce " + shape_str(shape_) + " to " + shape_str(target));
    if (is_device()) {
        // Sum over leading dims only (bias and broadcast-batch gradients): ones[1, R] . src[R, T] on the device.
        size_t j = 0;
        while (j < padded.size() && padded[j] == 1) ++j;
        bool tail_equal = true;
        for (size_t i = j; i < padded.size(); ++i) tail_equal = tail_equal && padded[i] == shape_[i];
        const int64_t R = prod(shape_, 0, j), T = prod(shape_, j);
        if (!tail_equal || R == 0 || T == 0) return src.cpu().sum_leading(target).to(DeviceType::HIP);
        Tensor ones_h({1, R}, dtype_);
        switch (dtype_) {
        case DType::Float32: std::fill_n(ones_h.data<float>(), R, 1.0f); break;
        case DType::Float64: std::fill_n(ones_h.data<double>(), R, 1.0); break;
        case DType::Float16: std::fill_n(ones_h.data<uint16_t>(), R, (uint16_t)0x3c00); break;
        case DType::BFloat16: std::fill_n(ones_h.data<uint16_t>(), R, (uint16_t)0x3f80); break;
        case DType::int8: case DType::uint8: std::fill_n(ones_h.data<uint8_t>(), R, (uint8_t)1); break;
        case DType::int16: case DType::uint16: std::fill_n(ones_h.data<uint16_t>(), R, (uint16_t)1); break;
        case DType::int32: case DType::uint32: std::fill_n(ones_h.data<uint32_t>(), R, 1u); break;
        case DType::int64: case DType::uint64: std::fill_n(ones_h.data<uint64_t>(), R, (uint64_t)1); break;
        default: utils::throw_exception(false, std::string("sum_as is not available for ") + dtype_name(dtype_));
        }
        const Tensor ones = ones_h.to(DeviceType::HIP);
        Tensor out(target, dtype_, DeviceType::HIP);
        ntg_gemm_desc d;
        std::memset(&d, 0, sizeof d);
        d.dtype = static_cast<int>(dtype_); d.c_mode = NTG_C_OVERWRITE;
        d.m = 1; d.k = R; d.n = T; d.batches = 1;
        if (ntg_gemm_dev(&d, ones.data_ptr(), src.data_ptr(), out.data_ptr(), nullptr) != NTG_OK)
            throw utils::nt_error(std::string("gfx950 matmult backend: ") + ntg_last_error());
        hip_check(hipStreamSynchronize(nullptr), "hipStreamSynchronize");      // `ones` is freed on return
        return out;
    }
    Tensor out(target, dtype_);
    if (dtype_ == DType::Float32) sum_as_t<float>(src, out, padded);
    else if (dtype_ == DType::Float64) sum_as_t<double>(src, out, padded);
    else if (dtype_ == DType::int32) sum_as_t<int32_t>(src, out, padded);
    else if (dtype_ == DType::int64) sum_as_t<int64_t>(src, out, padded);
    else utils::throw_exception(false, std::string("sum_as is not available for ") + dtype_name(dtype_));
    return out;
}

// ------------------------------------------------------------------------------------------ helpers

namespace functional {

Tensor zeros(SizeRef shape, DType dt, DeviceType dev) {
    Tensor t(std::move(shape), dt, dev);
    const size_t bytes = (size_t)(t.numel() * dtype_size(dt));
    if (dev == DeviceType::HIP) { if (bytes) hip_check(hipMemset(t.data_ptr(), 0, bytes), "hipMemset"); }
    else std::memset(t.data_ptr(), 0, bytes);
    return t;
}

static uint16_t f32_to_bf16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}

// binary16 <- binary32, round to nearest even
static uint16_t f32_to_f16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) return (uint16_t)(sign | (ax > 0x7f800000u ? 0x7e00u : 0x7c00u));
    if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
    if (ax < 0x33000001u) return (uint16_t)sign;
    const int32_t e = (int32_t)(ax >> 23) - 127;
    const uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    const uint32_t shift = e < -14 ? (uint32_t)(13 + (-14 - e)) : 13u, half_exp = e < -14 ? 0u : (uint32_t)(e + 15);
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
    return (uint16_t)(sign | (half_exp == 0 ? q : ((half_exp - 1) << 10) + q));
}

Tensor randn(SizeRef shape, DType dt, uint64_t seed) {
    Tensor t(std::move(shape), dt);
    std::mt19937_64 gen(seed ? seed : 0x9e3779b97f4a7c15ull);
    std::normal_distribution<double> nd(0.0, 1.0);
    const int64_t n = t.numel();
    switch (dt) {
    case DType::Float32: for (int64_t i = 0; i < n; ++i) t.data<float>()[i] = (float)nd(gen); break;
    case DType::Float64: for (int64_t i = 0; i < n; ++i) t.data<double>()[i] = nd(gen); break;
    case DType::BFloat16: for (int64_t i = 0; i < n; ++i) t.data<uint16_t>()[i] = f32_to_bf16((float)nd(gen)); break;
    case DType::Float16: for (int64_t i = 0; i < n; ++i) t.data<uint16_t>()[i] = f32_to_f16((float)nd(gen)); break;
    case DType::Complex32: for (int64_t i = 0; i < 2 * n; ++i) t.data<uint16_t>()[i] = f32_to_f16((float)nd(gen)); break;
    case DType::Complex64: for (int64_t i = 0; i < 2 * n; ++i) t.data<float>()[i] = (float)nd(gen); break;
    case DType::Complex128: for (int64_t i = 0; i < 2 * n; ++i) t.data<double>()[i] = nd(gen); break;
    case DType::int32: for (int64_t i = 0; i < n; ++i) t.data<int32_t>()[i] = (int32_t)std::lround(nd(gen) * 4.0); break;
    case DType::int64: for (int64_t i = 0; i < n; ++i) t.data<int64_t>()[i] = (int64_t)std::lround(nd(gen) * 4.0); break;
    default: utils::throw_exception(false, std::string("randn is not available for ") + dtype_name(dt));
    }
    return t;
}

Tensor from_numpy(const std::string& path) {
    std::ifstream f(path, std::ios::binary);
    utils::throw_exception((bool)f, "cannot open " + path);
    char magic[8];
    f.read(magic, 8);
    utils::throw_exception(f && std::memcmp(magic, "\x93NUMPY", 6) == 0, path + " is not a .npy file");
    uint32_t hlen = 0;
    if (magic[6] == 1) { uint16_t h16; f.read(reinterpret_cast<char*>(&h16), 2); hlen = h16; }
    else f.read(reinterpret_cast<char*>(&hlen), 4);
    std::string hdr(hlen, ' ');
    f.read(&hdr[0], hlen);
    auto field = [&](const std::string& key) {
        size_t p = hdr.find("'" + key + "'");
        utils::throw_exception(p != std::string::npos, "npy header lacks " + key);
        return hdr.substr(hdr.find(':', p) + 1);
    };
    std::string descr = field("descr");
    descr = descr.substr(descr.find('\'') + 1);
    descr = descr.substr(0, descr.find('\''));
    utils::throw_exception(field("fortran_order").find("False") < 8, "fortran-order .npy is not supported");
    std::string shp = field("shape");
    shp = shp.substr(shp.find('(') + 1);
    shp = shp.substr(0, shp.find(')'));
    SizeRef shape;
    std::stringstream ss(shp);
    std::string tok;
    while (std::getline(ss, tok, ',')) {
        bool digit = false;
        for (char c : tok) digit |= (c >= '0' && c <= '9');
        if (digit) shape.push_back(std::stoll(tok));
    }
    DType dt;
    const std::string code = descr.substr(1);
    utils::throw_exception(descr[0] == '<' || descr[0] == '|' || descr[0] == '=', "big-endian .npy is not supported");
    if (code == "f4") dt = DType::Float32; else if (code == "f8") dt = DType::Float64; else if (code == "f2") dt = DType::Float16;
    else if (code == "i1") dt = DType::int8; else if (code == "i2") dt = DType::int16; else if (code == "i4") dt = DType::int32;
    else if (code == "i8") dt = DType::int64; else if (code == "u1") dt = DType::uint8;
    else { utils::throw_exception(false, "npy dtype " + descr + " is not supported"); dt = DType::Float32; }
    Tensor t(shape, dt);
    f.read(static_cast<char*>(t.data_ptr()), (std::streamsize)(t.numel() * dtype_size(dt)));
    utils::throw_exception((bool)f, path + " is truncated");
    return t;
}

bool allclose(const Tensor& a_, const Tensor& b_, double rtol, double atol) {
    if (a_.is_null() || b_.is_null() || a_.shape() != b_.shape() || a_.dtype() != b_.dtype()) return false;
    Tensor a = a_.cpu().contiguous(), b = b_.cpu().contiguous();
    const int64_t n = a.numel();
    auto chk = [&](auto* pa, auto* pb) {
        for (int64_t i = 0; i < n; ++i) {
            const double x = (double)pa[i], y = (double)pb[i];
            if (!(std::fabs(x - y) <= atol + rtol * std::fabs(y))) return false;
        }
        return true;
    };
    switch (a.dtype()) {
    case DType::Float32: return chk(a.data<float>(), b.data<float>());
    case DType::Float64: return chk(a.data<double>(), b.data<double>());
    case DType::int32: return chk(a.data<int32_t>(), b.data<int32_t>());
    case DType::int64: return chk(a.data<int64_t>(), b.data<int64_t>());
    default: return std::memcmp(a.data_ptr(), b.data_ptr(), (size_t)(n * dtype_size(a.dtype()))) == 0;
    }
}

static void check_status(int rc) {
    if (rc != NTG_OK) throw utils::nt_error(std::string("gfx950 matmult backend: ") + ntg_last_error());
}

// A contiguous tensor is used as is; a view whose last two dims are a transposed contiguous
// matrix flips the flag instead of copying (was_transposed_back, matmult_cpu.cpp:204-250,
// 268-274, 491-494); anything else is cloned (matmult_cpu.cpp:277-279, 471-473).
static Tensor matrix_storage(const Tensor& t, bool& trans) {
    if (t.is_contiguous()) return t;
    Tensor tt = t.transpose(-1, -2);
    if (tt.is_contiguous()) { trans = !trans; return tt; }
    return t.clone();
}

struct MatmultPlan {
    Tensor a, b;            // storage tensors (contiguous)
    bool ta, tb;
    int64_t m, k, n, nbig, na, nb;
    SizeRef out_shape;
};

static MatmultPlan plan_matmult(const Tensor& a_in, const Tensor& b_in, bool trans_a, bool trans_b, bool out_variant) {
    utils::throw_exception(!a_in.is_null() && !b_in.is_null(), "Cannot perform operation matmult on a null tensor");   // _NT_FUNCTIONAL_ALWAYS_CHECK_
    utils::throw_exception(a_in.dims() > 1 && b_in.dims() > 1,
                           "\nRuntimeError: Expected tensors to have dims greater than 1, but instead had dims of " +
                               std::to_string(a_in.dims()) + " and " + std::to_string(b_in.dims()));
    utils::throw_exception(a_in.dtype() == b_in.dtype(), std::string("Expected both tensors to have the dtype ") + dtype_name(a_in.dtype()) +
                                                             " but got " + dtype_name(a_in.dtype()) + " and " + dtype_name(b_in.dtype()));   // :868
    utils::throw_exception(dtype_size(a_in.dtype()) > 0, std::string("dtype ") + dtype_name(a_in.dtype()) + " has no matmult on this backend");
    MatmultPlan p;
    p.ta = trans_a; p.tb = trans_b;
    p.a = matrix_storage(a_in, p.ta);
    p.b = matrix_storage(b_in, p.tb);
    const SizeRef& as = p.a.shape();
    const SizeRef& bs = p.b.shape();
    const int64_t ar = as[as.size() - 2], ac = as[as.size() - 1], br = bs[bs.size() - 2], bc = bs[bs.size() - 1];
    p.m = p.ta ? ac : ar;
    p.k = p.ta ? ar : ac;
    const int64_t kb = p.tb ? bc : br;
    p.n = p.tb ? br : bc;
    utils::throw_exception(p.k == kb, "Expected dimensions -2 and -1 of shapes (" + shape_str(a_in.shape()) + "," + shape_str(b_in.shape()) +
                                          ") to be equal for matrix multiplication");   // determine_transposes, :73-90
    const size_t abd = as.size() - 2, bbd = bs.size() - 2;
    const SizeRef& big = abd >= bbd ? as : bs;
    const SizeRef& small = abd >= bbd ? bs : as;
    const size_t bigd = std::max(abd, bbd), smalld = std::min(abd, bbd);
    for (size_t i = 0; i < smalld; ++i)
        utils::throw_exception(big[bigd - smalld + i] == small[i], "Cannot multiply tensors of shapes " + shape_str(a_in.shape()) + " and " +
                                                                       shape_str(b_in.shape()) + ", outter dimensions do not match");   // :870-872
    if (out_variant && bbd > abd)
        utils::throw_exception(!p.ta && !p.tb, "Transposing a and b are not currently supported for tensors of tensors, run "
                                               "transpose_Tensors(-1, -2).clone(), and then run matrix multiplication over the tensors");   // :952
    p.nbig = prod(big, 0, bigd);
    p.na = prod(as, 0, abd);
    p.nb = prod(bs, 0, bbd);
    p.out_shape.assign(big.begin(), big.begin() + (long)bigd);
    p.out_shape.push_back(p.m);
    p.out_shape.push_back(p.n);
    return p;
}

// operands of one operation live in the same memory
static DeviceType common_device(std::initializer_list<const Tensor*> ts, const char* op) {
    DeviceType dev = DeviceType::CPU;
    bool first = true;
    for (const Tensor* t : ts) {
        if (t->is_null()) continue;
        if (first) { dev = t->device(); first = false; }
        utils::throw_exception(t->device() == dev, std::string("Expected all tensors of ") + op + " to be on the same device");
    }
    return dev;
}

// Batched product on device buffers.  Item i of the higher-rank operand pairs with item i mod count of the lower-rank
// one (and of the bias); the lower-rank batch dims equal the trailing ones of the higher-rank operand, so the items come
// in nbig / chunk consecutive chunks inside which every operand is either strided or one matrix.
static void device_gemm(int dt, int64_t es, bool ta, bool tb, int mode, int64_t m, int64_t k, int64_t n, int64_t nbig,
                        const char* A, int64_t na, const char* B, int64_t nb, char* C,
                        const char* bias = nullptr, int64_t nbias = 1, int64_t brow = 1, int64_t bcol = 1, bool relu = false) {
    int64_t chunk = nbig;
    for (int64_t cnt : {na, nb, nbias})
        if (cnt > 1 && cnt < chunk) chunk = cnt;
    for (int64_t i0 = 0; i0 < nbig; i0 += chunk) {
        ntg_gemm_desc d;
        std::memset(&d, 0, sizeof d);
        d.dtype = dt; d.transpose_a = ta; d.transpose_b = tb; d.c_mode = mode;
        d.m = m; d.k = k; d.n = n; d.batches = chunk;
        d.stride_a = na > 1 ? m * k : 0;
        d.stride_b = nb > 1 ? k * n : 0;
        d.stride_c = m * n;
        if (bias) {
            d.bias = bias + (nbias > 1 ? (i0 % nbias) * brow * bcol * es : 0);
            d.bias_batch_stride = nbias > 1 ? brow * bcol : 0;
            d.bias_row_stride = brow > 1 ? bcol : 0;
            d.bias_col_stride = bcol > 1 ? 1 : 0;
        }
        const int64_t wsb = ntg_gemm_workspace_bytes(&d);      // > 0: a faster form exists (split along k, byte planes)
        if (wsb > 0) { d.workspace = device_workspace(wsb); d.workspace_bytes = wsb; }
        const char* a_i = A + (na > 1 ? (i0 % na) * m * k * es : 0);
        const char* b_i = B + (nb > 1 ? (i0 % nb) * k * n * es : 0);
        check_status(relu ? ntg_gemm_relu_dev(&d, a_i, b_i, C + i0 * m * n * es, nullptr) : ntg_gemm_dev(&d, a_i, b_i, C + i0 * m * n * es, nullptr));
    }
}

static void run_plan(const MatmultPlan& p, Tensor& c, bool overwrite = false) {
    if (p.nbig == 0 || p.m == 0 || p.n == 0 || p.k == 0) return;
    const int64_t es = dtype_size(p.a.dtype());
    const int dt = static_cast<int>(p.a.dtype());
    const char* A = static_cast<const char*>(p.a.data_ptr());
    const char* B = static_cast<const char*>(p.b.data_ptr());
    char* C = static_cast<char*>(c.data_ptr());
    if (c.is_device()) {
        device_gemm(dt, es, p.ta, p.tb, overwrite ? NTG_C_OVERWRITE : NTG_C_ACCUMULATE, p.m, p.k, p.n, p.nbig, A, p.na, B, p.nb, C);
        return;
    }
    if (p.nbig == 1) {
        check_status(ntg_matmult(dt, A, B, C, p.m, p.k, p.k, p.n, p.ta, p.tb));
        return;
    }
    // item i of the higher-rank operand pairs with item i mod count of the lower-rank one: the
    // reference repeats the HANDLES (smaller.repeat_, :883), so the pointer tables simply repeat
    std::vector<const void*> pa((size_t)p.nbig), pb((size_t)p.nbig);
    std::vector<void*> pc((size_t)p.nbig);
    for (int64_t i = 0; i < p.nbig; ++i) {
        pa[(size_t)i] = A + (i % p.na) * p.m * p.k * es;
        pb[(size_t)i] = B + (i % p.nb) * p.k * p.n * es;
        pc[(size_t)i] = C + i * p.m * p.n * es;
    }
    check_status(ntg_matmult_batch(dt, pa.data(), pb.data(), pc.data(), p.nbig, p.m, p.k, p.k, p.n, p.ta, p.tb));
}

Tensor matmult(const Tensor& a, const Tensor& b, bool trans_a, bool trans_b) {
    MatmultPlan p = plan_matmult(a, b, trans_a, trans_b, false);
    if (common_device({&a, &b}, "matmult") == DeviceType::HIP) {
        // C = op(a).op(b) written in one pass (zeros + accumulate would read and write C once more)
        if (p.k == 0) return zeros(p.out_shape, a.dtype(), DeviceType::HIP);
        Tensor c(p.out_shape, a.dtype(), DeviceType::HIP);
        run_plan(p, c, true);
        return c;
    }
    Tensor c = zeros(p.out_shape, a.dtype());      // matmult_cpu.cpp:110, :707
    run_plan(p, c);
    return c;
}

Tensor& matmult(const Tensor& a, const Tensor& b, Tensor& c, bool trans_a, bool trans_b) {
    utils::throw_exception(!c.is_null(), "Cannot perform operation matmult on a null tensor");
    utils::throw_exception(c.is_mutable(), "Output from Matmult must be mutable");   // tensor_files/matmult.cpp:21
    MatmultPlan p = plan_matmult(a, b, trans_a, trans_b, true);
    common_device({&a, &b, &c}, "matmult");
    const SizeRef& cs = c.shape();
    const bool same = cs == p.out_shape;
    const bool same_numel = c.dims() >= 2 && c.numel() == p.nbig * p.m * p.n && cs[cs.size() - 2] == p.m && cs[cs.size() - 1] == p.n;
    utils::throw_exception(same || (p.nbig > 1 && same_numel), "Got invalid shape for output tensor " + shape_str(cs) + " expected " +
                                                                   shape_str(p.out_shape));                                         // :137-139, :807-812
    utils::throw_exception(c.is_contiguous(), "Expected output tensor for matrix multiplication to be contiguous");             // :140
    utils::throw_exception(c.dtype() == a.dtype(), std::string("Expected dtype ") + dtype_name(a.dtype()) +
                                                       " for output matrix multiplication, C dtype inputted was " + dtype_name(c.dtype()));   // :141-143
    run_plan(p, c);                                // accumulates: C += op(a).op(b)
    return c;
}

Tensor matmult_cT(const Tensor& a, const Tensor& b) { return functional::matmult(a, b, false, true); }   // tensor_files/matmult.cpp:38

// Tensors of tensors: subT_check (matmult_cpu.cpp:1556-1566), handle_dim_{n_n,n_k,k_n}_subT_matmult_std (:1240-1485).
// Every pair (a[i], b[i]) follows the N-D x K-D rule; all matrices of all pairs go out as one nt_matmult_batch, the
// lower-rank side's matrices repeated by handle (return_split_tensor_of_tensors_repeat).
Tensor matmult(const TensorList& a, const TensorList& b, bool trans_a, bool trans_b) {
    utils::throw_exception(a.size() == b.size(), "Expected both tensors to have the same number of sub-tensors, going to have these multiplied in a "
                                                 "list-like fashion, but got " + std::to_string(a.size()) + " and " + std::to_string(b.size()) + " tensors");
    utils::throw_exception(!a.empty(), "Cannot perform operation matmult on an empty list of tensors");
    const int64_t L = (int64_t)a.size();
    // the first pair fixes the shapes, the flags and every check; the others must look the same (nt_matmult_batch is uniform)
    const MatmultPlan p0 = plan_matmult(a[0], b[0], trans_a, trans_b, false);
    std::vector<const Tensor*> all;
    for (const Tensor& t : a) all.push_back(&t);
    for (const Tensor& t : b) all.push_back(&t);
    DeviceType dev = a[0].device();
    for (const Tensor* t : all) {
        utils::throw_exception(!t->is_null(), "Cannot perform operation matmult on a null tensor");
        utils::throw_exception(t->device() == dev, "Expected all tensors of matmult to be on the same device");
    }
    std::vector<Tensor> as, bs;
    for (int64_t i = 0; i < L; ++i) {
        utils::throw_exception(a[(size_t)i].shape() == a[0].shape() && b[(size_t)i].shape() == b[0].shape() && a[(size_t)i].dtype() == a[0].dtype() &&
                                   b[(size_t)i].dtype() == b[0].dtype(),
                               "Expected the sub-tensors of one list to share one shape and dtype, item " + std::to_string(i) + " differs");
        bool ta = trans_a, tb = trans_b;
        Tensor sa = matrix_storage(a[(size_t)i], ta), sb = matrix_storage(b[(size_t)i], tb);
        utils::throw_exception(ta == p0.ta && tb == p0.tb,
                               "Expected the sub-tensors of one list to share one memory layout (all contiguous or all transposed views)");
        as.push_back(sa);
        bs.push_back(sb);
    }
    SizeRef out_shape = p0.out_shape;                              // the higher-rank item's batch dims + [m, n]
    out_shape[0] *= L;                                             // bigger_shape_vec[0] *= a.numel() (:1264, :1363); pairs of plain
                                                                   // matrices: the L results stacked along the rows
    const int64_t es = dtype_size(a[0].dtype()), total = L * p0.nbig;
    const int dt = static_cast<int>(a[0].dtype());
    if (dev == DeviceType::HIP) {
        Tensor c(out_shape, a[0].dtype(), DeviceType::HIP);
        if (total == 0 || p0.m == 0 || p0.n == 0) return c;
        if (p0.k == 0) return zeros(out_shape, a[0].dtype(), DeviceType::HIP);
        std::vector<const void*> tab((size_t)(3 * total));
        for (int64_t i = 0; i < L; ++i)
            for (int64_t j = 0; j < p0.nbig; ++j) {
                const int64_t t = i * p0.nbig + j;
                tab[(size_t)t] = static_cast<const char*>(as[(size_t)i].data_ptr()) + (j % p0.na) * p0.m * p0.k * es;
                tab[(size_t)(total + t)] = static_cast<const char*>(bs[(size_t)i].data_ptr()) + (j % p0.nb) * p0.k * p0.n * es;
                tab[(size_t)(2 * total + t)] = static_cast<char*>(c.data_ptr()) + t * p0.m * p0.n * es;
            }
        ntg_gemm_desc d;
        std::memset(&d, 0, sizeof d);
        d.dtype = dt; d.transpose_a = p0.ta; d.transpose_b = p0.tb; d.c_mode = NTG_C_OVERWRITE;
        d.m = p0.m; d.k = p0.k; d.n = p0.n; d.batches = total;
        // (1) Lists made by split_axis are slices of one allocation: the matrices of an operand then lie at a constant stride
        // (or are all the same matrix) and the list is an ordinary strided batch, workspace forms included.
        auto affine = [&](const void* const* P, int64_t& stride) {
            const char* p0c = static_cast<const char*>(P[0]);
            const int64_t step = total > 1 ? static_cast<const char*>(P[1]) - p0c : 0;
            if (step < 0 || step % es != 0) return false;
            for (int64_t t = 0; t < total; ++t)
                if (static_cast<const char*>(P[t]) != p0c + t * step) return false;
            stride = step / es;
            return true;
        };
        auto with_workspace = [&](ntg_gemm_desc& q) {
            const int64_t wsb = ntg_gemm_workspace_bytes(&q);
            if (wsb > 0) { q.workspace = device_workspace(wsb); q.workspace_bytes = wsb; }
            return wsb;
        };
        if (affine(tab.data(), d.stride_a) && affine(tab.data() + total, d.stride_b)) {
            d.stride_c = p0.m * p0.n;
            with_workspace(d);
            check_status(ntg_gemm_dev(&d, tab[0], tab[(size_t)total], const_cast<void*>(tab[(size_t)(2 * total)]), nullptr));
            return c;
        }
        // (2) Any other list: where one item on its own would be given a workspace form (a split along k changes the order of
        // summation), the items go out one by one in that form, so that an item comes out bit for bit the same alone and in a
        // list (tests/src/matmult_test.cpp:108-189) ...
        {
            ntg_gemm_desc one = d;
            one.batches = 1;
            if (with_workspace(one) > 0) {
                for (int64_t t = 0; t < total; ++t)
                    check_status(ntg_gemm_dev(&one, tab[(size_t)t], tab[(size_t)(total + t)], const_cast<void*>(tab[(size_t)(2 * total + t)]), nullptr));
                return c;
            }
        }
        // (3) ... else one table batch.  The tables go to this thread's cached device buffer (upload_table), so nothing is
        // allocated, freed or waited for here; the host can see every entry, so it vouches for their alignment where that
        // holds (the facade's own allocations are 256-byte aligned).
        bool aligned = true;
        for (const void* q : tab) aligned = aligned && (reinterpret_cast<uintptr_t>(q) & 15) == 0;
        if (aligned) d.flags |= NTG_GEMM_PTRS_ALIGNED16;
        void** T = static_cast<void**>(upload_table(tab.data(), (int64_t)(tab.size() * sizeof(void*))));
        check_status(ntg_gemm_ptrs_dev(&d, T, T + total, T + 2 * total, nullptr));
        return c;
    }
    Tensor c = zeros(out_shape, a[0].dtype());
    if (total == 0 || p0.m == 0 || p0.n == 0 || p0.k == 0) return c;
    std::vector<const void*> pa((size_t)total), pb((size_t)total);
    std::vector<void*> pc((size_t)total);
    for (int64_t i = 0; i < L; ++i)
        for (int64_t j = 0; j < p0.nbig; ++j) {
            const int64_t t = i * p0.nbig + j;
            pa[(size_t)t] = static_cast<const char*>(as[(size_t)i].data_ptr()) + (j % p0.na) * p0.m * p0.k * es;
            pb[(size_t)t] = static_cast<const char*>(bs[(size_t)i].data_ptr()) + (j % p0.nb) * p0.k * p0.n * es;
            pc[(size_t)t] = static_cast<char*>(c.data_ptr()) + t * p0.m * p0.n * es;
        }
    check_status(ntg_matmult_batch(dt, pa.data(), pb.data(), pc.data(), total, p0.m, p0.k, p0.k, p0.n, p0.ta, p0.tb));
    return c;
}

static Tensor linear_impl(const Tensor& x_in, const Tensor& w_in, const Tensor& b_in, bool trans_a, bool trans_b, bool with_relu) {
    utils::throw_exception(!x_in.is_null() && !w_in.is_null() && !b_in.is_null(), "Cannot perform operation linear on a null tensor");
    utils::throw_exception(x_in.dtype() == w_in.dtype() && x_in.dtype() == b_in.dtype(), "linear expects input, weight and bias of one dtype");
    const int64_t nd = std::max({x_in.dims(), w_in.dims(), b_in.dims()});
    utils::throw_exception(nd >= 2, "Cannot perform matrix multiplication with dimensions less than 2 got " + std::to_string(nd) +
                                        " for tensor dimensions");
    // unsqueeze_as (matmult_cpu.cpp:1712-1713)
    Tensor x = x_in.unsqueeze_front(nd - x_in.dims()), w = w_in.unsqueeze_front(nd - w_in.dims());
    Tensor b = b_in.contiguous().unsqueeze_front(nd - b_in.dims());
    auto strip = [](const Tensor& t) {   // leading batch dims of 1 are dropped (:1693-1696)
        SizeRef s = t.shape();
        size_t drop = 0;
        while (s.size() - drop > 2 && s[drop] == 1) ++drop;
        SizeRef ns(s.begin() + (long)drop, s.end());
        if (t.is_contiguous()) return t.view(ns);
        return t.clone().view(ns);
    };
    x = strip(x);
    w = strip(w);
    MatmultPlan p = plan_matmult(x, w, trans_a, trans_b, false);
    const SizeRef& bs = b.shape();
    const int64_t brow = bs[bs.size() - 2], bcol = bs[bs.size() - 1];
    utils::throw_exception(brow == p.m || brow == 1, "Got invalid shape for bias (" + shape_str(b_in.shape()) +
                                                         ") to linear function expected rows to be 1 or " + std::to_string(p.m));    // :1629-1631
    utils::throw_exception(bcol == p.n || bcol == 1, "Got invalid shape for bias (" + shape_str(b_in.shape()) +
                                                         ") to linear function expected cols to be 1 or " + std::to_string(p.n));    // :1632-1634
    SizeRef bb(bs.begin(), bs.end() - 2);
    while (!bb.empty() && bb[0] == 1) bb.erase(bb.begin());
    const size_t obd = p.out_shape.size() - 2;
    utils::throw_exception(bb.size() <= obd, "Error, invalid batch shapes for linear: (" + shape_str(x_in.shape()) + ", " +
                                                 shape_str(w_in.shape()) + ", " + shape_str(b_in.shape()) + ")");
    for (size_t i = 0; i < bb.size(); ++i)
        utils::throw_exception(bb[i] == p.out_shape[obd - bb.size() + i], "Error, invalid batch shapes for linear: (" + shape_str(x_in.shape()) +
                                                                              ", " + shape_str(w_in.shape()) + ", " + shape_str(b_in.shape()) + ")");
    const int64_t nbias = prod(bb);
    const DeviceType dev = common_device({&x_in, &w_in, &b_in}, "linear");
    Tensor c(p.out_shape, x.dtype(), dev);
    if (p.nbig == 0 || p.m == 0 || p.n == 0) return c;
    const int64_t es = dtype_size(x.dtype());
    const int dt = static_cast<int>(x.dtype());
    if (dev == DeviceType::HIP) {
        device_gemm(dt, es, p.ta, p.tb, NTG_C_BIAS, p.m, p.k, p.n, p.nbig, static_cast<const char*>(p.a.data_ptr()), p.na,
                    static_cast<const char*>(p.b.data_ptr()), p.nb, static_cast<char*>(c.data_ptr()),
                    static_cast<const char*>(b.data_ptr()), nbias, brow, bcol, with_relu);
        return c;
    }
    // bias broadcast to the output is the initial accumulator (:1637-1647); fused on the device
    for (int64_t i = 0; i < p.nbig; ++i) {
        check_status(ntg_linear(dt, static_cast<const char*>(p.a.data_ptr()) + (i % p.na) * p.m * p.k * es,
                                static_cast<const char*>(p.b.data_ptr()) + (i % p.nb) * p.k * p.n * es,
                                static_cast<const char*>(b.data_ptr()) + (i % nbias) * brow * bcol * es,
                                static_cast<char*>(c.data_ptr()) + i * p.m * p.n * es, p.m, p.k, p.n, p.ta, p.tb, brow, bcol));
    }
    if (with_relu) relu_(c);
    return c;
}

Tensor linear(const Tensor& x, const Tensor& w, const Tensor& b, bool trans_a, bool trans_b) { return linear_impl(x, w, b, trans_a, trans_b, false); }
Tensor linear_relu(const Tensor& x, const Tensor& w, const Tensor& b, bool trans_a, bool trans_b) { return linear_impl(x, w, b, trans_a, trans_b, true); }

template <class T>
static void relu_host(void* data, int64_t n) {
    T* p = static_cast<T*>(data);
    for (int64_t i = 0; i < n; ++i) p[i] = p[i] > T(0) ? p[i] : T(0);
}
static void relu_host_16(void* data, int64_t n, bool bf) {
    // sign and NaN are visible in the bit pattern: negative (sign bit set, -0 included) or NaN -> +0
    uint16_t* p = static_cast<uint16_t*>(data);
    const uint16_t exp_mask = bf ? 0x7f80 : 0x7c00, man_mask = bf ? 0x007f : 0x03ff;
    for (int64_t i = 0; i < n; ++i) {
        const uint16_t v = p[i];
        const bool nan = (v & exp_mask) == exp_mask && (v & man_mask) != 0;
        if ((v & 0x8000) || nan) p[i] = 0;
    }
}

Tensor& relu_(Tensor& x) {
    utils::throw_exception(!x.is_null(), "Cannot perform operation relu_ on a null tensor");
    const DType dt = x.dtype();
    utils::throw_exception(dt == DType::Float16 || dt == DType::BFloat16 || dt == DType::Float32 || dt == DType::Float64,
                           "relu_ expects a floating dtype");
    utils::throw_exception(x.is_contiguous(), "relu_ expects a contiguous tensor");
    const int64_t n = x.numel();
    if (n == 0) return x;
    if (x.is_device()) {
        // relu_ on device memory = the product entry point with an empty k: C = max(C, 0)
        const SizeRef& sh = x.shape();
        const int64_t cols = sh.empty() ? 1 : sh.back();
        ntg_gemm_desc d;
        std::memset(&d, 0, sizeof d);
        d.dtype = static_cast<int>(dt); d.c_mode = NTG_C_ACCUMULATE;
        d.m = n / cols; d.k = 0; d.n = cols; d.batches = 1;
        check_status(ntg_gemm_relu_dev(&d, nullptr, nullptr, x.data_ptr(), nullptr));
        return x;
    }
    switch (dt) {
    case DType::Float32: relu_host<float>(x.data_ptr(), n); break;
    case DType::Float64: relu_host<double>(x.data_ptr(), n); break;
    case DType::Float16: relu_host_16(x.data_ptr(), n, false); break;
    default: relu_host_16(x.data_ptr(), n, true); break;
    }
    return x;
}

Tensor relu(const Tensor& x) {
    Tensor out = x.contiguous().clone();
    return relu_(out);
}

MatmultGrads matmult_backward(const Tensor& a, const Tensor& b, const Tensor& grad, bool trans_a, bool trans_b) {
    // nn/functional/matmult.cpp:37-62
    MatmultGrads g;
    g.da = trans_a ? functional::matmult(b, grad, trans_b, true) : functional::matmult(grad, b, false, !trans_b);
    g.db = trans_b ? functional::matmult(grad, a, true, trans_a) : functional::matmult(a, grad, !trans_a, false);
    if (g.da.shape() != a.shape()) g.da = g.da.sum_leading(a.shape());     // accumulate_gradient's broadcast reduction
    if (g.db.shape() != b.shape()) g.db = g.db.sum_leading(b.shape());
    return g;
}

LinearGrads linear_backward(const Tensor& x, const Tensor& w, const Tensor& bias, const Tensor& grad, bool trans_a, bool trans_b) {
    // nn/functional/matmult.cpp:253-275; AutoGrad.cpp:7-25 for the reductions
    MatmultGrads mg = matmult_backward(x, w, grad, trans_a, trans_b);
    LinearGrads g;
    g.dx = mg.da;
    g.dw = mg.db;
    g.db = grad.shape() == bias.shape() ? grad.clone() : grad.sum_leading(bias.shape());
    return g;
}

static void check_pair_ge(const utils::my_tuple& v, int64_t lo, const std::string& what) {
    utils::throw_exception(v.first >= lo && v.second >= lo, what);
}

Tensor unfold2d(const Tensor& x_in, utils::my_tuple k, utils::my_tuple d, utils::my_tuple p, utils::my_tuple s, bool transpose_out) {
    utils::throw_exception(!x_in.is_null(), "Cannot perform operation unfold2d on a null tensor");
    utils::throw_exception(x_in.dims() >= 3, "Expected input tensot to unfold to have dims greater than or equal to 3 but got " +
                                                 std::to_string(x_in.dims()) + "D");
    Tensor x = x_in.contiguous();
    const SizeRef& xs = x.shape();
    const int64_t H = xs[xs.size() - 2], W = xs[xs.size() - 1], C = xs[xs.size() - 3];
    const int64_t B = x.numel() / std::max<int64_t>(1, C * H * W);
    const int64_t Lr = (H + 2 * p.first - d.first * (k.first - 1) - 1) / s.first + 1;
    const int64_t Lc = (W + 2 * p.second - d.second * (k.second - 1) - 1) / s.second + 1;
    utils::throw_exception(Lr > 0 && Lc > 0 && H + 2 * p.first - d.first * (k.first - 1) - 1 >= 0 && W + 2 * p.second - d.second * (k.second - 1) - 1 >= 0,
                           "Given input with spatial size (" + std::to_string(H) + ", " + std::to_string(W) +
                               "), calculated shape of the array of sliding blocks as (" + std::to_string(Lr) + ", " + std::to_string(Lc) +
                               "), but its components must be at least one.");
    Tensor col({B, C * k.first * k.second, Lr * Lc}, x.dtype(), x.device());
    if (x.is_device())
        check_status(ntg_unfold2d_dev(static_cast<int>(x.dtype()), x.data_ptr(), col.data_ptr(), B, C, H, W, k.first, k.second, s.first, s.second,
                                      p.first, p.second, d.first, d.second, nullptr));
    else
        check_status(ntg_unfold2d(static_cast<int>(x.dtype()), x.data_ptr(), col.data_ptr(), B, C, H, W, k.first, k.second, s.first, s.second,
                                  p.first, p.second, d.first, d.second));
    if (transpose_out) return col;
    return col.transpose(-1, -2);
}

Tensor conv2d(const Tensor& image, const Tensor& kernel, utils::my_tuple s, utils::my_tuple p, utils::my_tuple d, int64_t groups) {
    utils::throw_exception(!image.is_null() && !kernel.is_null(), "Cannot perform operation conv2d on a null tensor");
    // conv.cpp:72-79
    utils::throw_exception(image.dims() >= 3, "Expected to get a 3D or greater tensor as the input for a 2d convolution, but got " +
                                                  std::to_string(image.dims()) + "D");
    utils::throw_exception(kernel.dims() == 3 || kernel.dims() == 4, "Expected to get a 4D or 3D tensor as the kernel for a 2d convolution, but got " +
                                                                         std::to_string(kernel.dims()) + "D");
    utils::throw_exception(image.dtype() == kernel.dtype(), std::string("Expected both kernel and image to have the same dtype for conv2d but got ") +
                                                                dtype_name(kernel.dtype()) + " and " + dtype_name(image.dtype()));
    utils::throw_exception(image.dtype() != DType::Bool && image.dtype() != DType::TensorObj, "Expected to get a number type for image and kernel");
    check_pair_ge(s, 1, "Conv2d stride cannot be less than 1");
    check_pair_ge(d, 1, "Conv2d dilation cannot be less than 1");
    check_pair_ge(p, 0, "Conv2d padding cannot be less than 1");
    Tensor x = image.contiguous(), w = kernel.contiguous();
    const SizeRef& xs = x.shape();
    const int64_t H = xs[xs.size() - 2], W = xs[xs.size() - 1], C = xs[xs.size() - 3];
    const int64_t B = x.numel() / std::max<int64_t>(1, C * H * W);
    const SizeRef& ws = w.shape();
    const int64_t kh = ws[ws.size() - 2], kw = ws[ws.size() - 1], Cg = ws[ws.size() - 3], O = kernel.dims() == 4 ? ws[0] : 1;
    utils::throw_exception(groups >= 1, "Conv2d groups cannot be less than 1");
    utils::throw_exception(C % groups == 0, "Expected image channels to be divisible by groups in Conv2d but got " + std::to_string(C) + " % " +
                                                std::to_string(groups) + " != 0");   // :97
    utils::throw_exception(Cg * groups == C, "Expected kernel rows times groups to be equal to rows of image Conv2d but got " + std::to_string(Cg) +
                                                 " * " + std::to_string(groups) + " != " + std::to_string(C));   // :98
    const int64_t Ro = (H + 2 * p.first - d.first * (kh - 1) - 1) / s.first + 1;
    const int64_t Co = (W + 2 * p.second - d.second * (kw - 1) - 1) / s.second + 1;
    utils::throw_exception(Ro > 0 && Co > 0, "conv2d output would be empty");
    const DeviceType dev = common_device({&image, &kernel}, "conv2d");
    Tensor out({B, O, Ro, Co}, x.dtype(), dev);
    const int dt = static_cast<int>(x.dtype());
    if (dev == DeviceType::HIP) {
        const int64_t wsb = ntg_conv2d_fast_workspace_bytes(dt, B, C, H, W, O, kh, kw, s.first, s.second, p.first, p.second, d.first, d.second, groups);
        utils::throw_exception(wsb >= 0, "conv2d output would be empty");
        check_status(ntg_conv2d_dev(dt, x.data_ptr(), w.data_ptr(), out.data_ptr(), device_workspace(wsb), wsb, B, C, H, W, O, kh, kw,
                                    s.first, s.second, p.first, p.second, d.first, d.second, groups, nullptr));
        return out;
    }
    check_status(ntg_conv2d(dt, x.data_ptr(), w.data_ptr(), out.data_ptr(), B, C, H, W, O, kh, kw, s.first, s.second,
                            p.first, p.second, d.first, d.second, groups));
    return out;
}

Tensor unfold2d_backward(const Tensor& col_in, utils::my_tuple out, utils::my_tuple k, utils::my_tuple d, utils::my_tuple p, utils::my_tuple s) {
    utils::throw_exception(!col_in.is_null(), "Cannot perform operation unfold2d_backward on a null tensor");
    utils::throw_exception(col_in.dims() == 2 || col_in.dims() == 3, "Expected to get a shape with a dimensionality of 3D or 2D, but got " +
                                                                         std::to_string(col_in.dims()) + " dimensions");   // colim_transform.cpp:594
    Tensor col = col_in.contiguous();
    const SizeRef& cs = col.shape();
    const int64_t B = col.dims() == 3 ? cs[0] : 1, rows = cs[cs.size() - 2], L = cs[cs.size() - 1];
    utils::throw_exception(rows % (k.first * k.second) == 0, "col rows are not a multiple of the kernel size");
    const int64_t C = rows / (k.first * k.second);
    const int64_t Lr = (out.first + 2 * p.first - d.first * (k.first - 1) - 1) / s.first + 1;
    const int64_t Lc = (out.second + 2 * p.second - d.second * (k.second - 1) - 1) / s.second + 1;
    utils::throw_exception(Lr > 0 && Lc > 0 && Lr * Lc == L, "Given output_size and kernel geometry do not match the number of sliding blocks");
    Tensor im({B, C, out.first, out.second}, col.dtype(), col.device());
    if (col.is_device())
        check_status(ntg_unfold2d_backward_dev(static_cast<int>(col.dtype()), col.data_ptr(), im.data_ptr(), B, C, out.first, out.second, k.first,
                                               k.second, s.first, s.second, p.first, p.second, d.first, d.second, 0, nullptr));
    else
        check_status(ntg_unfold2d_backward(static_cast<int>(col.dtype()), col.data_ptr(), im.data_ptr(), B, C, out.first, out.second, k.first,
                                           k.second, s.first, s.second, p.first, p.second, d.first, d.second, 0));
    return im;
}

ConvGrads conv2d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, utils::my_tuple s, utils::my_tuple p,
                          utils::my_tuple d, int64_t groups) {
    utils::throw_exception(!image.is_null() && !kernel.is_null() && !grad.is_null(), "Cannot perform operation conv2d backward on a null tensor");
    utils::throw_exception(image.dims() >= 3 && (kernel.dims() == 3 || kernel.dims() == 4), "conv2d backward expects an image of >= 3 dims and a 3D/4D kernel");
    utils::throw_exception(image.dtype() == kernel.dtype() && image.dtype() == grad.dtype(), "conv2d backward expects one dtype");
    Tensor x = image.contiguous(), w = kernel.contiguous(), g = grad.contiguous();
    const SizeRef& xs = x.shape();
    const int64_t H = xs[xs.size() - 2], W = xs[xs.size() - 1], C = xs[xs.size() - 3];
    const int64_t B = x.numel() / std::max<int64_t>(1, C * H * W);
    const SizeRef& ws = w.shape();
    const int64_t kh = ws[ws.size() - 2], kw = ws[ws.size() - 1], Cg = ws[ws.size() - 3], O = kernel.dims() == 4 ? ws[0] : 1;
    utils::throw_exception(groups >= 1 && C % groups == 0 && Cg * groups == C && O % groups == 0, "channels, kernel channels and filters do not fit groups");
    const int64_t Ro = (H + 2 * p.first - d.first * (kh - 1) - 1) / s.first + 1;
    const int64_t Co = (W + 2 * p.second - d.second * (kw - 1) - 1) / s.second + 1;
    utils::throw_exception(Ro > 0 && Co > 0 && g.numel() == B * O * Ro * Co, "grad does not have the shape of the convolution output");
    const DeviceType dev = common_device({&image, &kernel, &grad}, "conv2d backward");
    ConvGrads out{Tensor(image.shape(), x.dtype(), dev), Tensor(kernel.shape(), x.dtype(), dev)};
    const int dt = static_cast<int>(x.dtype());
    if (dev == DeviceType::HIP) {
        const int64_t wsb = ntg_conv2d_backward_workspace_bytes(dt, B, C, H, W, O, kh, kw, s.first, s.second, p.first, p.second, d.first, d.second, groups);
        utils::throw_exception(wsb >= 0, "conv2d backward: geometry has no output");
        check_status(ntg_conv2d_backward_dev(dt, x.data_ptr(), w.data_ptr(), g.data_ptr(), out.d_image.data_ptr(), out.d_kernel.data_ptr(),
                                             device_workspace(wsb), wsb, B, C, H, W, O, kh, kw, s.first, s.second, p.first, p.second,
                                             d.first, d.second, groups, 0, nullptr));
        return out;
    }
    check_status(ntg_conv2d_backward(dt, x.data_ptr(), w.data_ptr(), g.data_ptr(), out.d_image.data_ptr(),
                                     out.d_kernel.data_ptr(), B, C, H, W, O, kh, kw, s.first, s.second, p.first, p.second, d.first, d.second,
                                     groups, 0));
    return out;
}

// [.., C, W] -> [B, C, 1, W] (contiguous view)
static Tensor as_one_row(const Tensor& t, const char* what) {
    utils::throw_exception(!t.is_null(), std::string("Cannot perform operation ") + what + " on a null tensor");
    Tensor c = t.contiguous();
    const SizeRef& s = c.shape();
    utils::throw_exception(s.size() >= 2, std::string("Expected to get a 2D or greater tensor for ") + what + ", but got " + std::to_string(s.size()) + "D");
    const int64_t W = s[s.size() - 1], C = s[s.size() - 2];
    const int64_t B = s.size() == 2 ? 1 : c.numel() / std::max<int64_t>(1, C * W);
    return c.view({B, C, 1, W});
}

Tensor conv1d(const Tensor& image, const Tensor& kernel, int64_t stride, int64_t padding, int64_t dilation, int64_t groups) {
    utils::throw_exception(!image.is_null() && !kernel.is_null(), "Cannot perform operation conv1d on a null tensor");
    // conv.cpp:16-23
    utils::throw_exception(image.dims() >= 2, "Expected to get a 2D or greater tensor as the input for a 1d convolution, but got " + std::to_string(image.dims()) + "D");
    utils::throw_exception(kernel.dims() == 3 || kernel.dims() == 2, "Expected to get a 3D or 2D tensor as the kernel for a 1d convolution, but got " + std::to_string(kernel.dims()) + "D");
    utils::throw_exception(stride >= 1, "Conv1d stride cannot be less than 1 but got " + std::to_string(stride));
    utils::throw_exception(dilation >= 1, "Conv1d dilation cannot be less than 1 but got " + std::to_string(dilation));
    utils::throw_exception(padding >= 0, "Conv1d padding cannot be less than 1 but got " + std::to_string(padding));
    Tensor x = as_one_row(image, "conv1d"), w = as_one_row(kernel, "conv1d");
    Tensor o = functional::conv2d(x, w, {1, stride}, {0, padding}, {1, dilation}, groups);
    return o.view({o.shape()[0], o.shape()[1], o.shape()[3]});
}

ConvGrads conv1d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, int64_t stride, int64_t padding, int64_t dilation,
                          int64_t groups) {
    Tensor x = as_one_row(image, "conv1d backward"), w = as_one_row(kernel, "conv1d backward");
    ConvGrads g = functional::conv2d_backward(x, w, grad.contiguous(), {1, stride}, {0, padding}, {1, dilation}, groups);
    return {g.d_image.view(image.shape()), g.d_kernel.view(kernel.shape())};
}

Tensor conv_transpose2d(const Tensor& image, const Tensor& kernel, utils::my_tuple s, utils::my_tuple p, utils::my_tuple op, utils::my_tuple d,
                        int64_t groups) {
    utils::throw_exception(!image.is_null() && !kernel.is_null(), "Cannot perform operation conv_transpose2d on a null tensor");
    // conv.cpp:617-631
    utils::throw_exception(image.dims() >= 3, "Expected to get a 3D or greater tensor as the input for a conv2d transpose, but got " + std::to_string(image.dims()) + "D");
    utils::throw_exception(kernel.dims() == 4 || kernel.dims() == 3, "Expected to get a 4D or 3D tensor as the kernel for a conv2d transpose, but got " + std::to_string(kernel.dims()) + "D");
    utils::throw_exception(image.dtype() == kernel.dtype(), std::string("Expected both kernel and image to have the same dtype for conv2d transpose but got ") +
                                                                dtype_name(kernel.dtype()) + " and " + dtype_name(image.dtype()));
    check_pair_ge(s, 1, "Conv2d Transpose stride cannot be less than 1");
    check_pair_ge(d, 1, "Conv2d Transpose dilation cannot be less than 1");
    check_pair_ge(op, 0, "Conv2d Transpose output_padding cannot be less than 1");
    check_pair_ge(p, 0, "Conv2d Transpose padding cannot be less than 1");
    utils::throw_exception(groups > 0, "Expected groups for a convolution to be greater than 0 but got " + std::to_string(groups));
    Tensor x = image.contiguous(), w = kernel.contiguous();
    const SizeRef& xs = x.shape();
    const int64_t H = xs[xs.size() - 2], W = xs[xs.size() - 1], Cin = xs[xs.size() - 3];
    const int64_t B = x.numel() / std::max<int64_t>(1, Cin * H * W);
    const SizeRef& ws = w.shape();
    const int64_t kh = ws[ws.size() - 2], kw = ws[ws.size() - 1], Cog = ws[ws.size() - 3], Wb = kernel.dims() == 4 ? ws[0] : 1;
    utils::throw_exception(Cin == Wb, "Expected image channels to be the same as the kernel batches for conv_transpose2d but got " +
                                          shape_str(x.shape()) + " and " + shape_str(w.shape()));
    utils::throw_exception(Cin % groups == 0, "Expected image channels to be divisible by groups in Conv2d Transpose but got " + std::to_string(Cin) +
                                                  " % " + std::to_string(groups) + " != 0");
    const int64_t R = (H - 1) * s.first - 2 * p.first + d.first * (kh - 1) + 1 + op.first;
    const int64_t Cc = (W - 1) * s.second - 2 * p.second + d.second * (kw - 1) + 1 + op.second;
    utils::throw_exception(R > 0 && Cc > 0, "conv_transpose2d output would be empty");
    const DeviceType dev = common_device({&image, &kernel}, "conv_transpose2d");
    Tensor out({B, Cog * groups, R, Cc}, x.dtype(), dev);
    const int dt = static_cast<int>(x.dtype());
    if (dev == DeviceType::HIP) {
        const int64_t wsb = ntg_conv_transpose2d_workspace_bytes(dt, B, Cin, H, W, Cog * groups, kh, kw, s.first, s.second, p.first, p.second,
                                                                 d.first, d.second, op.first, op.second, groups);
        if (wsb >= 0) {
            check_status(ntg_conv_transpose2d_dev(dt, x.data_ptr(), w.data_ptr(), out.data_ptr(), device_workspace(wsb), wsb, B, Cin, H, W,
                                                  Cog * groups, kh, kw, s.first, s.second, p.first, p.second, d.first, d.second, op.first,
                                                  op.second, groups, nullptr));
            return out;
        }
        // (geometry errors are reported by the host entry point below, with its message)
    }
    check_status(ntg_conv_transpose2d(dt, x.data_ptr(), w.data_ptr(), out.data_ptr(), B, Cin, H, W, Cog * groups, kh, kw,
                                      s.first, s.second, p.first, p.second, d.first, d.second, op.first, op.second, groups));
    return out;
}

ConvGrads conv_transpose2d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, utils::my_tuple s, utils::my_tuple p,
                                    utils::my_tuple op, utils::my_tuple d, int64_t groups) {
    (void)op;   // the output size is the gradient's
    utils::throw_exception(!image.is_null() && !kernel.is_null() && !grad.is_null(), "Cannot perform operation conv_transpose2d backward on a null tensor");
    Tensor x = image.contiguous(), g = grad.contiguous();
    Tensor dx = functional::conv2d(g, kernel, s, p, d, groups);
    utils::throw_exception(dx.numel() == x.numel(), "grad does not have the shape of the transposed convolution's output");
    ConvGrads kg = functional::conv2d_backward(g, kernel, x, s, p, d, groups);
    return {dx.view(image.shape()), kg.d_kernel};
}

Tensor conv_transpose1d(const Tensor& image, const Tensor& kernel, int64_t stride, int64_t padding, int64_t output_padding, int64_t dilation,
                        int64_t groups) {
    utils::throw_exception(!image.is_null() && !kernel.is_null(), "Cannot perform operation conv_transpose1d on a null tensor");
    utils::throw_exception(image.dims() >= 2, "Expected to get a 2D or greater tensor as the input for a conv1d transpose, but got " + std::to_string(image.dims()) + "D");
    utils::throw_exception(kernel.dims() == 3 || kernel.dims() == 2, "Expected to get a 3D or 2D tensor as the kernel for a conv1d transpose, but got " + std::to_string(kernel.dims()) + "D");
    Tensor x = as_one_row(image, "conv_transpose1d"), w = as_one_row(kernel, "conv_transpose1d");
    Tensor o = functional::conv_transpose2d(x, w, {1, stride}, {0, padding}, {0, output_padding}, {1, dilation}, groups);
    return o.view({o.shape()[0], o.shape()[1], o.shape()[3]});
}

ConvGrads conv_transpose1d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, int64_t stride, int64_t padding,
                                    int64_t output_padding, int64_t dilation, int64_t groups) {
    Tensor x = as_one_row(image, "conv_transpose1d backward"), w = as_one_row(kernel, "conv_transpose1d backward");
    Tensor g = as_one_row(grad, "conv_transpose1d backward");
    ConvGrads r = functional::conv_transpose2d_backward(x, w, g, {1, stride}, {0, padding}, {0, output_padding}, {1, dilation}, groups);
    return {r.d_image.view(image.shape()), r.d_kernel.view(kernel.shape())};
}

// image [.., C, D, H, W] / kernel [O, C/g, kd, kh, kw] -> batch, channels, sizes (contiguous inputs)
struct Vol3 { int64_t B, C, size[3]; };
static Vol3 vol3(const Tensor& t, bool is_kernel, const char* what) {
    const SizeRef& s = t.shape();
    utils::throw_exception(s.size() >= 4, std::string("Expected to get a 4D or greater tensor for ") + what + ", but got " + std::to_string(s.size()) + "D");
    utils::throw_exception(!is_kernel || s.size() <= 5, std::string("Expected to get a 5D or 4D tensor as the kernel for ") + what);
    Vol3 v;
    for (int a = 0; a < 3; ++a) v.size[a] = s[s.size() - 3 + a];
    v.C = s[s.size() - 4];
    v.B = t.numel() / std::max<int64_t>(1, v.C * v.size[0] * v.size[1] * v.size[2]);
    return v;
}

Tensor conv3d(const Tensor& image, const Tensor& kernel, utils::my_n_tuple<3> s, utils::my_n_tuple<3> p, utils::my_n_tuple<3> d, int64_t groups) {
    utils::throw_exception(!image.is_null() && !kernel.is_null(), "Cannot perform operation conv3d on a null tensor");
    utils::throw_exception(image.dtype() == kernel.dtype(), "Expected both kernel and image to have the same dtype for conv3d");
    const DeviceType dev = common_device({&image, &kernel}, "conv3d");
    for (int a = 0; a < 3; ++a) {   // conv.cpp:129-131
        utils::throw_exception(s[a] >= 1, "Conv3d stride cannot be less than 1");
        utils::throw_exception(d[a] >= 1, "Conv3d dilation cannot be less than 1");
        utils::throw_exception(p[a] >= 0, "Conv3d padding cannot be less than 1");
    }
    Tensor x = image.contiguous(), w = kernel.contiguous();
    const Vol3 xv = vol3(x, false, "a 3d convolution"), wv = vol3(w, true, "a 3d convolution");
    const int64_t O = wv.B;
    utils::throw_exception(groups >= 1 && xv.C % groups == 0 && wv.C * groups == xv.C && O % groups == 0,
                           "Expected kernel rows times groups to be equal to rows of image Conv3d");
    int64_t out[3];
    for (int a = 0; a < 3; ++a) {
        out[a] = (xv.size[a] + 2 * p[a] - d[a] * (wv.size[a] - 1) - 1) / s[a] + 1;
        utils::throw_exception(out[a] > 0, "conv3d output would be empty");
    }
    Tensor y({xv.B, O, out[0], out[1], out[2]}, x.dtype(), dev);
    const int dt = static_cast<int>(x.dtype());
    if (dev == DeviceType::HIP) {
        const int64_t wsb = ntg_convnd_workspace_bytes(dt, xv.B, xv.C, O, 3, xv.size, wv.size, s.data(), p.data(), d.data(), groups, 0);
        utils::throw_exception(wsb >= 0, "conv3d output would be empty");
        check_status(ntg_convnd_dev(dt, x.data_ptr(), w.data_ptr(), y.data_ptr(), device_workspace(wsb), wsb, xv.B, xv.C, O, 3, xv.size, wv.size,
                                    s.data(), p.data(), d.data(), groups, nullptr));
        return y;
    }
    check_status(ntg_convnd(dt, x.data_ptr(), w.data_ptr(), y.data_ptr(), xv.B, xv.C, O, 3, xv.size, wv.size, s.data(), p.data(), d.data(), groups));
    return y;
}

ConvGrads conv3d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, utils::my_n_tuple<3> s, utils::my_n_tuple<3> p,
                          utils::my_n_tuple<3> d, int64_t groups) {
    utils::throw_exception(!image.is_null() && !kernel.is_null() && !grad.is_null(), "Cannot perform operation conv3d backward on a null tensor");
    const DeviceType dev = common_device({&image, &kernel, &grad}, "conv3d backward");
    Tensor x = image.contiguous(), w = kernel.contiguous(), g = grad.contiguous();
    const Vol3 xv = vol3(x, false, "conv3d backward"), wv = vol3(w, true, "conv3d backward");
    int64_t L = 1;
    for (int a = 0; a < 3; ++a) L *= (xv.size[a] + 2 * p[a] - d[a] * (wv.size[a] - 1) - 1) / s[a] + 1;
    utils::throw_exception(g.numel() == xv.B * wv.B * L, "grad does not have the shape of the convolution output");
    ConvGrads out{Tensor(image.shape(), x.dtype(), dev), Tensor(kernel.shape(), x.dtype(), dev)};
    const int dt = static_cast<int>(x.dtype());
    if (dev == DeviceType::HIP) {
        const int64_t wsb = ntg_convnd_workspace_bytes(dt, xv.B, xv.C, wv.B, 3, xv.size, wv.size, s.data(), p.data(), d.data(), groups, 1);
        utils::throw_exception(wsb >= 0, "conv3d backward: geometry has no output");
        check_status(ntg_convnd_backward_dev(dt, x.data_ptr(), w.data_ptr(), g.data_ptr(), out.d_image.data_ptr(), out.d_kernel.data_ptr(),
                                             device_workspace(wsb), wsb, xv.B, xv.C, wv.B, 3, xv.size, wv.size, s.data(), p.data(), d.data(), groups, 0, nullptr));
        return out;
    }
    check_status(ntg_convnd_backward(dt, x.data_ptr(), w.data_ptr(), g.data_ptr(), out.d_image.data_ptr(),
                                     out.d_kernel.data_ptr(), xv.B, xv.C, wv.B, 3, xv.size, wv.size, s.data(), p.data(), d.data(), groups, 0));
    return out;
}

Tensor conv_transpose3d(const Tensor& image, const Tensor& kernel, utils::my_n_tuple<3> s, utils::my_n_tuple<3> p, utils::my_n_tuple<3> op,
                        utils::my_n_tuple<3> d, int64_t groups) {
    utils::throw_exception(!image.is_null() && !kernel.is_null(), "Cannot perform operation conv_transpose3d on a null tensor");
    utils::throw_exception(image.dtype() == kernel.dtype(), "Expected both kernel and image to have the same dtype for conv3d transpose");
    const DeviceType dev = common_device({&image, &kernel}, "conv_transpose3d");
    for (int a = 0; a < 3; ++a) {   // conv.cpp:687-691
        utils::throw_exception(s[a] >= 1, "Conv3d Transpose stride cannot be less than 1");
        utils::throw_exception(d[a] >= 1, "Conv3d Transpose dilation cannot be less than 1");
        utils::throw_exception(op[a] >= 0, "Conv3d Transpose output_padding cannot be less than 1");
        utils::throw_exception(p[a] >= 0, "Conv3d Transpose padding cannot be less than 1");
    }
    utils::throw_exception(groups > 0, "Expected groups for a convolution to be greater than 0 but got " + std::to_string(groups));
    Tensor x = image.contiguous(), w = kernel.contiguous();
    const Vol3 xv = vol3(x, false, "a conv3d transpose"), wv = vol3(w, true, "a conv3d transpose");
    utils::throw_exception(xv.C == wv.B, "Expected image channels to be the same as the kernel batches for conv_transpose3d but got " +
                                             shape_str(x.shape()) + " and " + shape_str(w.shape()));
    utils::throw_exception(xv.C % groups == 0, "Expected image channels to be divisible by groups in Conv3d Transpose");
    int64_t out[3];
    for (int a = 0; a < 3; ++a) out[a] = (xv.size[a] - 1) * s[a] - 2 * p[a] + d[a] * (wv.size[a] - 1) + 1 + op[a];
    Tensor y({xv.B, wv.C * groups, out[0], out[1], out[2]}, x.dtype(), dev);
    const int dt = static_cast<int>(x.dtype());
    if (dev == DeviceType::HIP) {
        const int64_t wsb = ntg_conv_transposend_workspace_bytes(dt, xv.B, xv.C, wv.C * groups, 3, xv.size, wv.size, s.data(), p.data(), d.data(), op.data(), groups);
        utils::throw_exception(wsb >= 0, "conv_transpose3d output would be empty");
        check_status(ntg_conv_transposend_dev(dt, x.data_ptr(), w.data_ptr(), y.data_ptr(), device_workspace(wsb), wsb, xv.B, xv.C, wv.C * groups, 3,
                                              xv.size, wv.size, s.data(), p.data(), d.data(), op.data(), groups, nullptr));
        return y;
    }
    check_status(ntg_conv_transposend(dt, x.data_ptr(), w.data_ptr(), y.data_ptr(), xv.B, xv.C, wv.C * groups, 3, xv.size,
                                      wv.size, s.data(), p.data(), d.data(), op.data(), groups));
    return y;
}

ConvGrads conv_transpose3d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, utils::my_n_tuple<3> s, utils::my_n_tuple<3> p,
                                    utils::my_n_tuple<3> op, utils::my_n_tuple<3> d, int64_t groups) {
    (void)op;
    Tensor dx = functional::conv3d(grad.contiguous(), kernel, s, p, d, groups);
    utils::throw_exception(dx.numel() == image.numel(), "grad does not have the shape of the transposed convolution's output");
    ConvGrads kg = functional::conv3d_backward(grad.contiguous(), kernel, image.contiguous(), s, p, d, groups);
    return {dx.view(image.shape()), kg.d_kernel};
}

}  // namespace functional

namespace layers {

Linear::Linear(int64_t in_channels, int64_t out_channels, bool use_bias_, DType dt, uint64_t seed)
    : use_bias(use_bias_), Weight(functional::randn({in_channels, out_channels}, dt, seed)),
      Bias(use_bias_ ? functional::randn({out_channels}, dt, seed + 1) : Tensor::Null()) {
    Weight.set_mutability(false);                  // Linear.cpp:17-19
    if (use_bias) Bias.set_mutability(false);
}

Tensor Linear::forward(const Tensor& x) const {
    if (!use_bias) return functional::matmult(x, Weight);      // TensorGrad linear with a null bias, nn/functional/matmult.cpp:238-241
    return functional::linear(x, Weight, Bias);
}

functional::LinearGrads Linear::backward(const Tensor& x, const Tensor& grad) const {
    if (!use_bias) {
        functional::MatmultGrads mg = functional::matmult_backward(x, Weight, grad, false, false);
        return {mg.da, mg.db, Tensor::Null()};
    }
    return functional::linear_backward(x, Weight, Bias, grad, false, false);
}

}  // namespace layers
}  // namespace nt
