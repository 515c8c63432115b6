// nt_compat -- the reference's C++ interface for the dense matmult path, on the gfx950 backend.
//
// Mirrors, with the same names, argument meaning and error behaviour:
//   nt::functional::matmult / matmult_cT / linear   nt/functional/tensor_files/matmult.h:10-13
//   nt::functional::unfold2d                        nt/functional/tensor_files/colim_transform.cpp:565-588
//   nt::functional::conv2d                          nt/functional/tensor_files/conv.h:12
//   nt::functional::conv1d / conv_transpose1d / conv_transpose2d   nt/functional/tensor_files/conv.cpp:13-67, 538-676
//   nt::matmult / nt::linear / nt::conv2d           nt/nt.h:835-850, 369-517 (positional form of the named-argument facade)
//   nt::layers::Linear                              nt/nn/layers/Linear.h:10-20
//   gradient GEMM selection of TensorGrad linear/matmult   nt/nn/functional/matmult.cpp:37-62, 253-275
//   nt::utils::throw_exception                      nt/utils/utils.h:178-202
// nt::Tensor is reduced to what the path needs: dtype + shape + strides over ref-counted storage
// (contiguous tensors and transposed views), in host memory or -- DeviceType::HIP -- in the GPU's HBM.
// All arithmetic is done by libntgemm.so: host tensors go through the host-pointer C ABI
// (include/ntgemm.h; every call pays the PCIe copies), tensors moved to the device with
// Tensor::to(DeviceType::HIP) through the `_dev` entry points, so a chain of operations
// (Linear -> Linear, forward -> backward) never leaves HBM.  There is no CPU fallback.
#pragma once
#include <array>
#include <cstdint>
#include <initializer_list>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace nt {

// values equal the reference enum (nt/dtype/DType_enum.h:14-20); BFloat16 / uint64 are this backend's extensions
enum class DType : int {
    Float16 = 0, Float32 = 1, Float64 = 2, Float128 = 3, Complex32 = 4, Complex64 = 5, Complex128 = 6,
    int8 = 7, int16 = 8, int32 = 9, int64 = 10, int128 = 11, uint8 = 12, uint16 = 13, uint32 = 14, uint128 = 15,
    Bool = 16, TensorObj = 17, BFloat16 = 100, uint64 = 101,
    Half = Float16, Float = Float32, Double = Float64, Char = int8, Short = int16, Integer = int32, Long = int64, Byte = uint8
};
int64_t dtype_size(DType dt);
const char* dtype_name(DType dt);

namespace utils {
// thrown by every failed check; derives from std::exception like the reference's errors (test_macros.h:89)
struct nt_error : std::runtime_error { using std::runtime_error::runtime_error; };
void throw_exception(bool ok, const std::string& message);
using my_tuple = std::pair<int64_t, int64_t>;
template <size_t N> using my_n_tuple = std::array<int64_t, N>;
}  // namespace utils

using SizeRef = std::vector<int64_t>;
class Tensor;
// A list of tensors: what the reference holds as a 1-D tensor of DType::TensorObj (Tensor::split_axis,
// nt/functional/cpu/matmult_cpu.cpp:1240-1485 multiply two of them item by item)
using TensorList = std::vector<Tensor>;
std::string shape_str(const SizeRef& s);

// nt/memory/DeviceEnum.h:6-10 with the device this backend adds
enum class DeviceType : int8_t { META = -1, CPU = 0, CPUShared = 1, HIP = 2 };
constexpr DeviceType dCPU = DeviceType::CPU;
constexpr DeviceType dHIP = DeviceType::HIP;

class Tensor {
public:
    Tensor() = default;                                           // null tensor
    Tensor(SizeRef shape, DType dt, DeviceType dev = DeviceType::CPU);   // uninitialised contiguous tensor
    static Tensor Null() { return Tensor(); }

    bool is_null() const { return !storage_; }
    const SizeRef& shape() const { return shape_; }
    const SizeRef& strides() const { return strides_; }
    int64_t dims() const { return (int64_t)shape_.size(); }
    int64_t numel() const;
    DType dtype() const { return dtype_; }
    DeviceType device() const { return device_; }
    bool is_device() const { return device_ == DeviceType::HIP; }
    // copy to the other memory (contiguous result); the tensor itself when it already lives there.  Operands of one
    // operation must share a device; results live where the operands do.  data_ptr() of a device tensor is a device pointer.
    Tensor to(DeviceType dev) const;
    Tensor cpu() const { return to(DeviceType::CPU); }
    void* data_ptr() { return storage_.get() + offset_; }
    const void* data_ptr() const { return storage_.get() + offset_; }
    bool is_contiguous() const;
    bool is_mutable() const { return mutable_; }
    Tensor& set_mutability(bool m) { mutable_ = m; return *this; }

    Tensor clone() const;                                         // contiguous copy
    Tensor contiguous() const { return is_contiguous() ? *this : clone(); }
    Tensor view(SizeRef shape) const;                             // contiguous tensors only; one -1 allowed
    Tensor transpose(int64_t a, int64_t b) const;                 // strided view, no copy
    Tensor unsqueeze_front(int64_t n) const;                      // prepend n dims of 1
    Tensor item(int64_t batch_index) const;                       // i-th matrix of a contiguous [.., r, c] tensor
    TensorList split_axis(int64_t axis) const;                    // axis 0 of a contiguous tensor: its shape[0] slices, as views
    Tensor sum_leading(const SizeRef& target_shape) const;        // reduce broadcast dims back (sum_as)
    template <class T> T* data() { return reinterpret_cast<T*>(data_ptr()); }
    template <class T> const T* data() const { return reinterpret_cast<const T*>(data_ptr()); }

private:
    std::shared_ptr<char> storage_;
    int64_t offset_ = 0;        // bytes
    SizeRef shape_, strides_;   // strides in elements
    DType dtype_ = DType::Float32;
    DeviceType device_ = DeviceType::CPU;
    bool mutable_ = true;
};

namespace functional {
Tensor zeros(SizeRef shape, DType dt = DType::Float32, DeviceType dev = DeviceType::CPU);
Tensor randn(SizeRef shape, DType dt = DType::Float32, uint64_t seed = 0);   // seeded N(0,1) (the reference's randn is unseeded); complex: both parts
Tensor from_numpy(const std::string& path);                                   // .npy, C order, f2/f4/f8/i1/i2/i4/i8/u1
bool allclose(const Tensor& a, const Tensor& b, double rtol = 1e-5, double atol = 1e-8);   // compare.h:34

Tensor matmult(const Tensor& a, const Tensor& b, bool trans_a = false, bool trans_b = false);
Tensor& matmult(const Tensor& a, const Tensor& b, Tensor& c, bool trans_a = false, bool trans_b = false);
Tensor matmult_cT(const Tensor& a, const Tensor& b);
// Tensors of tensors (matmult_cpu.cpp:1240-1485, dispatched at :1576-1580): two lists of equal length are multiplied item by
// item in ONE nt_matmult_batch over all their matrices; items of one list share shape and dtype, the lower-rank side's
// matrices repeat under the higher-rank side's (the N-D x K-D rule inside every pair).  The result is one tensor: the
// higher-rank item's shape with its first dimension multiplied by the list length and the last two replaced by [m, n].
Tensor matmult(const TensorList& a, const TensorList& b, bool trans_a = false, bool trans_b = false);
Tensor linear(const Tensor& input, const Tensor& weight, const Tensor& bias, bool trans_input = false, bool trans_weight = false);
// relu = clamp(x, 0), relu_ in place (activation_functions.cpp:141-143; min_max.cpp:115-121: max(x, 0), 0 for NaN and -0);
// floating dtypes.  linear_relu(x, w, b) == relu_(linear(x, w, b)) bit for bit; on device tensors it is one launch (the
// clamp runs in the product's epilogue) -- the reference has no fused form, its layers call the two in a row.
Tensor relu(const Tensor& x);
Tensor& relu_(Tensor& x);
Tensor linear_relu(const Tensor& input, const Tensor& weight, const Tensor& bias, bool trans_input = false, bool trans_weight = false);
Tensor unfold2d(const Tensor& x, utils::my_tuple kernel_size, utils::my_tuple dilation = {1, 1}, utils::my_tuple padding = {0, 0},
                utils::my_tuple stride = {1, 1}, bool transpose_out = true);
Tensor conv2d(const Tensor& image, const Tensor& kernel, utils::my_tuple stride = {1, 1}, utils::my_tuple padding = {0, 0},
              utils::my_tuple dilation = {1, 1}, int64_t groups = 1);

// conv_dimage + conv_dkernel for dim == 2 (conv.h:17-18; conv.cpp:318-346, 444-471) and col2im
Tensor unfold2d_backward(const Tensor& col, utils::my_tuple output_size, utils::my_tuple kernel_size, utils::my_tuple dilation = {1, 1},
                         utils::my_tuple padding = {0, 0}, utils::my_tuple stride = {1, 1});
struct ConvGrads { Tensor d_image, d_kernel; };
ConvGrads conv2d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, utils::my_tuple stride = {1, 1},
                          utils::my_tuple padding = {0, 0}, utils::my_tuple dilation = {1, 1}, int64_t groups = 1);

// conv1d (conv.cpp:13-67), conv_transpose1d (:538-612), conv_transpose2d (:614-676) and their gradients.  The one-axis
// forms are the two-axis ones with a single row; a transposed convolution is the image gradient of the convolution with
// the same kernel, and its own gradients are that convolution and its kernel gradient with the operands exchanged.
Tensor conv1d(const Tensor& image, const Tensor& kernel, int64_t stride = 1, int64_t padding = 0, int64_t dilation = 1, int64_t groups = 1);
ConvGrads conv1d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, int64_t stride = 1, int64_t padding = 0,
                          int64_t dilation = 1, int64_t groups = 1);
Tensor conv_transpose2d(const Tensor& image, const Tensor& kernel, utils::my_tuple stride = {1, 1}, utils::my_tuple padding = {0, 0},
                        utils::my_tuple output_padding = {0, 0}, utils::my_tuple dilation = {1, 1}, int64_t groups = 1);
ConvGrads conv_transpose2d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, utils::my_tuple stride = {1, 1},
                                    utils::my_tuple padding = {0, 0}, utils::my_tuple output_padding = {0, 0},
                                    utils::my_tuple dilation = {1, 1}, int64_t groups = 1);
Tensor conv_transpose1d(const Tensor& image, const Tensor& kernel, int64_t stride = 1, int64_t padding = 0, int64_t output_padding = 0,
                        int64_t dilation = 1, int64_t groups = 1);
ConvGrads conv_transpose1d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, int64_t stride = 1, int64_t padding = 0,
                                    int64_t output_padding = 0, int64_t dilation = 1, int64_t groups = 1);

// conv3d (conv.cpp:122-175), conv_transpose3d (:678-745) and their gradients
Tensor conv3d(const Tensor& image, const Tensor& kernel, utils::my_n_tuple<3> stride = {1, 1, 1}, utils::my_n_tuple<3> padding = {0, 0, 0},
              utils::my_n_tuple<3> dilation = {1, 1, 1}, int64_t groups = 1);
ConvGrads conv3d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, utils::my_n_tuple<3> stride = {1, 1, 1},
                          utils::my_n_tuple<3> padding = {0, 0, 0}, utils::my_n_tuple<3> dilation = {1, 1, 1}, int64_t groups = 1);
Tensor conv_transpose3d(const Tensor& image, const Tensor& kernel, utils::my_n_tuple<3> stride = {1, 1, 1}, utils::my_n_tuple<3> padding = {0, 0, 0},
                        utils::my_n_tuple<3> output_padding = {0, 0, 0}, utils::my_n_tuple<3> dilation = {1, 1, 1}, int64_t groups = 1);
ConvGrads conv_transpose3d_backward(const Tensor& image, const Tensor& kernel, const Tensor& grad, utils::my_n_tuple<3> stride = {1, 1, 1},
                                    utils::my_n_tuple<3> padding = {0, 0, 0}, utils::my_n_tuple<3> output_padding = {0, 0, 0},
                                    utils::my_n_tuple<3> dilation = {1, 1, 1}, int64_t groups = 1);

// what the backward lambdas of TensorGrad matmult / linear compute (flags only, no transposed copies)
struct MatmultGrads { Tensor da, db; };
MatmultGrads matmult_backward(const Tensor& a, const Tensor& b, const Tensor& grad, bool trans_a, bool trans_b);
struct LinearGrads { Tensor dx, dw, db; };
LinearGrads linear_backward(const Tensor& x, const Tensor& w, const Tensor& bias, const Tensor& grad, bool trans_a, bool trans_b);
}  // namespace functional

// positional forms of the named-argument facade (nt.h:835-850)
inline Tensor matmult(const Tensor& input, const Tensor& other, bool transpose_a = false, bool transpose_b = false) {
    return functional::matmult(input, other, transpose_a, transpose_b);
}
inline Tensor& matmult(const Tensor& input, const Tensor& other, Tensor& out, bool transpose_a = false, bool transpose_b = false) {
    return functional::matmult(input, other, out, transpose_a, transpose_b);
}
inline Tensor matmult(const TensorList& input, const TensorList& other, bool transpose_a = false, bool transpose_b = false) {
    return functional::matmult(input, other, transpose_a, transpose_b);
}
inline Tensor linear(const Tensor& input, const Tensor& weight, const Tensor& bias, bool transpose_a = false, bool transpose_b = false) {
    return functional::linear(input, weight, bias, transpose_a, transpose_b);
}
inline Tensor conv2d(const Tensor& image, const Tensor& kernel, utils::my_tuple stride = {1, 1}, utils::my_tuple padding = {0, 0},
                     utils::my_tuple dilation = {1, 1}, int64_t groups = 1) {
    return functional::conv2d(image, kernel, stride, padding, dilation, groups);
}

inline Tensor conv1d(const Tensor& image, const Tensor& kernel, int64_t stride = 1, int64_t padding = 0, int64_t dilation = 1, int64_t groups = 1) {
    return functional::conv1d(image, kernel, stride, padding, dilation, groups);
}
inline Tensor conv_transpose1d(const Tensor& image, const Tensor& kernel, int64_t stride = 1, int64_t padding = 0, int64_t output_padding = 0,
                               int64_t dilation = 1, int64_t groups = 1) {
    return functional::conv_transpose1d(image, kernel, stride, padding, output_padding, dilation, groups);
}
inline Tensor conv_transpose2d(const Tensor& image, const Tensor& kernel, utils::my_tuple stride = {1, 1}, utils::my_tuple padding = {0, 0},
                               utils::my_tuple output_padding = {0, 0}, utils::my_tuple dilation = {1, 1}, int64_t groups = 1) {
    return functional::conv_transpose2d(image, kernel, stride, padding, output_padding, dilation, groups);
}

inline Tensor conv3d(const Tensor& image, const Tensor& kernel, utils::my_n_tuple<3> stride = {1, 1, 1}, utils::my_n_tuple<3> padding = {0, 0, 0},
                     utils::my_n_tuple<3> dilation = {1, 1, 1}, int64_t groups = 1) {
    return functional::conv3d(image, kernel, stride, padding, dilation, groups);
}
inline Tensor conv_transpose3d(const Tensor& image, const Tensor& kernel, utils::my_n_tuple<3> stride = {1, 1, 1},
                               utils::my_n_tuple<3> padding = {0, 0, 0}, utils::my_n_tuple<3> output_padding = {0, 0, 0},
                               utils::my_n_tuple<3> dilation = {1, 1, 1}, int64_t groups = 1) {
    return functional::conv_transpose3d(image, kernel, stride, padding, output_padding, dilation, groups);
}

namespace layers {
// Weight [in, out], Bias [out]; forward = linear(x, Weight, Bias) (Linear.cpp:10-24)
class Linear {
public:
    Linear(int64_t in_channels, int64_t out_channels, bool use_bias = true, DType dt = DType::Float32, uint64_t seed = 1);
    Linear& to(DeviceType dev) { Weight = Weight.to(dev); if (use_bias) Bias = Bias.to(dev); return *this; }
    Tensor forward(const Tensor& x) const;
    functional::LinearGrads backward(const Tensor& x, const Tensor& grad) const;
    bool use_bias;
    Tensor Weight, Bias;
};
}  // namespace layers

}  // namespace nt
