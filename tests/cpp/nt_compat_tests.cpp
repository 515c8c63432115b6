// Replays the reference's own tests for the matmult path against the nt_compat facade:
//   tests/src/matmult_test.cpp:10-107 (matmult shapes), :108-189 (batched == per item, bitwise),
//   :194-307 (linear shapes), tests/src/linear_autograd_test.cpp:126-148 (golden grads),
//   tests/src/conv_autograd_test.cpp:250-371 (golden conv2d outputs), col_im_autograd_test.cpp:77-95.
// Same structure as the reference's runner (tests/src/test_macros.h:69-93): each case is a lambda,
// a thrown exception fails the case.  `--host-only` runs the cases that never reach the device
// (argument validation must fail BEFORE any device work).  Usage: nt_compat_tests <golden dir> [--host-only]
#include "../../neurotensor_amd/nt_compat/nt_compat.h"

#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>

static int g_failed = 0, g_run = 0;

static void run_test(const char* name, const std::function<void()>& fn) {
    ++g_run;
    try {
        fn();
        std::printf("[ok]   %s\n", name);
    } catch (const std::exception& e) {
        ++g_failed;
        std::printf("[FAIL] %s: %s\n", name, e.what());
    }
}

static void expect_throw(const char* name, const std::function<void()>& fn) {
    run_test(name, [&] {
        bool threw = false;
        try { fn(); } catch (const nt::utils::nt_error&) { threw = true; }
        nt::utils::throw_exception(threw, "expected an exception");
    });
}

using nt::DType;
using nt::SizeRef;
using nt::Tensor;
namespace F = nt::functional;

// double-precision reference of op(a).op(b) for contiguous 2-D float tensors
static double max_err_vs_double(const Tensor& a, const Tensor& b, const Tensor& c, bool ta, bool tb, const float* c0 = nullptr) {
    const int64_t ar = a.shape()[0], ac = a.shape()[1], bc = b.shape()[1], br = b.shape()[0];
    const int64_t m = ta ? ac : ar, k = ta ? ar : ac, n = tb ? br : bc;
    double worst = 0;
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            double s = c0 ? c0[i * n + j] : 0.0;
            for (int64_t t = 0; t < k; ++t) {
                const double av = ta ? a.data<float>()[t * ac + i] : a.data<float>()[i * ac + t];
                const double bv = tb ? b.data<float>()[j * bc + t] : b.data<float>()[t * bc + j];
                s += av * bv;
            }
            worst = std::fmax(worst, std::fabs(s - c.data<float>()[i * n + j]));
        }
    return worst;
}

static void shape_case(const char* name, SizeRef as, SizeRef bs, bool ta, bool tb, SizeRef expect) {
    run_test(name, [&] {
        Tensor a = F::randn(as, DType::Float32, 11), b = F::randn(bs, DType::Float32, 12);
        Tensor o = nt::matmult(a, b, ta, tb);
        nt::utils::throw_exception(o.shape() == expect, "Error: Got unexpected shape for (" + nt::shape_str(as) + ") (" + nt::shape_str(bs) +
                                                            ") = (" + nt::shape_str(o.shape()) + ")");
        // values: first and last item against a double-precision loop
        const int64_t items = o.numel() / (expect[expect.size() - 1] * expect[expect.size() - 2]);
        Tensor ac = a.contiguous(), bc = b.contiguous();
        const int64_t na = ac.numel() / (as[as.size() - 1] * as[as.size() - 2]), nb = bc.numel() / (bs[bs.size() - 1] * bs[bs.size() - 2]);
        for (int64_t i : {int64_t(0), items - 1}) {
            const double err = max_err_vs_double(ac.item(i % na), bc.item(i % nb), o.item(i), ta, tb);
            nt::utils::throw_exception(err <= 1e-3, "values differ from the double-precision loop by " + std::to_string(err));
        }
    });
}

static void linear_shape_case(const char* name, SizeRef as, SizeRef bs, SizeRef bis, bool ta, bool tb, SizeRef expect) {
    run_test(name, [&] {
        Tensor a = F::randn(as, DType::Float32, 21), b = F::randn(bs, DType::Float32, 22), bi = F::randn(bis, DType::Float32, 23);
        Tensor o = nt::linear(a, b, bi, ta, tb);
        nt::utils::throw_exception(o.shape() == expect, "Error: Got unexpected shape (" + nt::shape_str(o.shape()) + ")");
        // linear == matmult + broadcast bias (bias is the initial accumulator)
        Tensor mm = nt::matmult(a, b, ta, tb);
        const int64_t n = expect[expect.size() - 1], m = expect[expect.size() - 2];
        const int64_t brow = bis.size() >= 2 ? bis[bis.size() - 2] : 1, bcol = bis[bis.size() - 1];
        for (int64_t i = 0; i < o.numel(); ++i) {
            const int64_t r = (i / n) % m, c = i % n;
            const float want = mm.data<float>()[i] + bi.data<float>()[(brow == 1 ? 0 : r) * bcol + (bcol == 1 ? 0 : c)];
            nt::utils::throw_exception(std::fabs(want - o.data<float>()[i]) <= 1e-3, "linear != matmult + bias at " + std::to_string(i));
        }
    });
}

static void host_only_cases() {
    expect_throw("matmult inner sizes differ", [] { nt::matmult(F::zeros({4, 5}), F::zeros({4, 5})); });
    expect_throw("relu of an integer tensor", [] { Tensor i32 = F::randn({4, 4}, DType::int32, 207); F::relu(i32); });
    expect_throw("matmult inner sizes differ with flags", [] { nt::matmult(F::zeros({4, 5}), F::zeros({4, 6}), true, true); });
    expect_throw("matmult 1-D operand", [] { nt::matmult(F::zeros({5}), F::zeros({5, 5})); });
    expect_throw("matmult dtype mismatch", [] { nt::matmult(F::zeros({4, 4}), F::zeros({4, 4}, DType::Float64)); });
    expect_throw("matmult batch dims do not line up", [] { nt::matmult(F::zeros({2, 3, 4, 4}), F::zeros({2, 4, 4})); });
    expect_throw("matmult null operand", [] { nt::matmult(Tensor::Null(), F::zeros({4, 4})); });
    expect_throw("matmult unsupported dtype", [] { Tensor t; nt::matmult(Tensor({2, 2}, DType::Float128), Tensor({2, 2}, DType::Float128)); });
    expect_throw("matmult out wrong shape", [] { Tensor c = F::zeros({4, 5}); nt::matmult(F::zeros({4, 4}), F::zeros({4, 4}), c); });
    expect_throw("matmult out wrong dtype", [] { Tensor c = F::zeros({4, 4}, DType::Float64); nt::matmult(F::zeros({4, 4}), F::zeros({4, 4}), c); });
    expect_throw("matmult out immutable", [] { Tensor c = F::zeros({4, 4}); c.set_mutability(false); nt::matmult(F::zeros({4, 4}), F::zeros({4, 4}), c); });
    expect_throw("matmult out not contiguous", [] { Tensor c = F::zeros({4, 4}).transpose(0, 1); nt::matmult(F::zeros({4, 4}), F::zeros({4, 4}), c); });
    expect_throw("matmult out with flags on lower-rank a", [] { Tensor c = F::zeros({3, 4, 4}); nt::matmult(F::zeros({4, 4}), F::zeros({3, 4, 4}), c, true, false); });
    expect_throw("linear bias rows", [] { nt::linear(F::zeros({4, 5}), F::zeros({5, 6}), F::zeros({2, 6})); });
    expect_throw("linear bias cols", [] { nt::linear(F::zeros({4, 5}), F::zeros({5, 6}), F::zeros({5})); });
    expect_throw("conv2d kernel dims", [] { nt::conv2d(F::zeros({1, 3, 8, 8}), F::zeros({3, 3})); });
    expect_throw("conv2d groups", [] { nt::conv2d(F::zeros({1, 3, 8, 8}), F::zeros({4, 3, 3, 3}), {1, 1}, {0, 0}, {1, 1}, 2); });
    expect_throw("conv2d stride", [] { nt::conv2d(F::zeros({1, 3, 8, 8}), F::zeros({4, 3, 3, 3}), {0, 1}); });
    expect_throw("conv3d stride", [] { nt::conv3d(F::zeros({1, 3, 4, 8, 8}), F::zeros({4, 3, 3, 3, 3}), {1, 0, 1}); });
    expect_throw("conv3d groups", [] { nt::conv3d(F::zeros({1, 3, 4, 8, 8}), F::zeros({4, 3, 3, 3, 3}), {1, 1, 1}, {0, 0, 0}, {1, 1, 1}, 2); });
    expect_throw("conv1d image dims", [] { nt::conv1d(F::zeros({8}), F::zeros({4, 3, 3})); });
    expect_throw("conv1d stride", [] { nt::conv1d(F::zeros({1, 3, 8}), F::zeros({4, 3, 3}), 0); });
    expect_throw("conv_transpose2d channels", [] { nt::conv_transpose2d(F::zeros({1, 3, 8, 8}), F::zeros({4, 3, 3, 3})); });
    expect_throw("conv_transpose2d output_padding", [] { nt::conv_transpose2d(F::zeros({1, 3, 8, 8}), F::zeros({3, 4, 3, 3}), {1, 1}, {0, 0}, {-1, 0}); });
    expect_throw("unfold2d empty", [] { F::unfold2d(F::zeros({1, 1, 2, 2}), {5, 5}); });
    run_test("tensor views", [] {
        Tensor a = F::randn({3, 4, 5}, DType::Float32, 5);
        Tensor t = a.transpose(-1, -2);
        nt::utils::throw_exception(!t.is_contiguous() && t.shape() == SizeRef({3, 5, 4}), "transpose view");
        Tensor c = t.clone();
        nt::utils::throw_exception(c.is_contiguous() && c.data<float>()[1] == a.data<float>()[5], "clone of a strided view");
        nt::utils::throw_exception(F::allclose(c.transpose(-1, -2), a), "double transpose");
        Tensor s = a.sum_leading({5});
        float want = 0;
        for (int i = 0; i < 12; ++i) want += a.data<float>()[i * 5 + 2];
        nt::utils::throw_exception(std::fabs(s.data<float>()[2] - want) < 1e-5, "sum_as");
    });
}

static void device_cases(const std::string& g) {
    shape_case("matmult 2d", {30, 30}, {30, 30}, false, false, {30, 30});
    shape_case("matmult 2d Ta", {30, 14}, {30, 30}, true, false, {14, 30});
    shape_case("matmult 2d Tb", {30, 30}, {14, 30}, false, true, {30, 14});
    shape_case("matmult 2d T(a, b)", {30, 14}, {14, 30}, true, true, {14, 14});
    shape_case("matmult 3d", {10, 30, 30}, {10, 30, 30}, false, false, {10, 30, 30});
    shape_case("matmult 3d Ta", {10, 30, 14}, {10, 30, 30}, true, false, {10, 14, 30});
    shape_case("matmult 3d Tb", {10, 30, 30}, {10, 14, 30}, false, true, {10, 30, 14});
    shape_case("matmult 3d T(a, b)", {10, 30, 14}, {10, 14, 30}, true, true, {10, 14, 14});
    shape_case("matmult 3d bigger A", {5, 10, 30, 30}, {10, 30, 30}, false, false, {5, 10, 30, 30});
    shape_case("matmult 3d Ta bigger A", {5, 10, 30, 14}, {10, 30, 30}, true, false, {5, 10, 14, 30});
    shape_case("matmult 3d Tb bigger A", {5, 10, 30, 30}, {10, 14, 30}, false, true, {5, 10, 30, 14});
    shape_case("matmult 3d T(a, b) bigger A", {5, 10, 30, 14}, {10, 14, 30}, true, true, {5, 10, 14, 14});
    shape_case("matmult 3d bigger B", {10, 30, 30}, {5, 10, 30, 30}, false, false, {5, 10, 30, 30});
    shape_case("matmult 3d Ta bigger B", {10, 30, 14}, {5, 10, 30, 30}, true, false, {5, 10, 14, 30});
    shape_case("matmult 3d Tb bigger B", {10, 30, 30}, {5, 10, 14, 30}, false, true, {5, 10, 30, 14});
    shape_case("matmult 3d T(a, b) bigger B", {10, 30, 14}, {5, 10, 14, 30}, true, true, {5, 10, 14, 14});

    run_test("matmult batched == per item (bitwise)", [] {
        Tensor a = F::randn({5, 2, 3, 4}, DType::Float32, 31), b = F::randn({5, 2, 4, 3}, DType::Float32, 32);
        Tensor o = nt::matmult(a, b);
        for (int64_t i = 0; i < 10; ++i) {
            Tensor oi = nt::matmult(a.item(i).clone(), b.item(i).clone());
            nt::utils::throw_exception(std::memcmp(oi.data_ptr(), o.item(i).data_ptr(), 9 * sizeof(float)) == 0, "item differs");
        }
    });
    // tests/src/matmult_test.cpp:108-189: two lists of tensors multiplied item by item in one batch == per-item products, bit for bit
    struct ListCase { const char* name; SizeRef as, bs; bool ta, tb; SizeRef view; };
    for (const ListCase& lc : {ListCase{"matmult tensors (no bigger)", {5, 2, 3, 4}, {5, 2, 4, 3}, false, false, {5, 2, 3, 3}},
                               ListCase{"matmult tensors Ta", {5, 2, 4, 3}, {5, 2, 4, 3}, true, false, {5, 2, 3, 3}},
                               ListCase{"matmult tensors Tb", {5, 2, 4, 3}, {5, 2, 4, 3}, false, true, {5, 2, 4, 4}},
                               ListCase{"matmult tensors Ta (bigger a)", {5, 2, 4, 3}, {5, 4, 3}, true, false, {5, 2, 3, 3}},
                               ListCase{"matmult tensors Tb (bigger a)", {5, 2, 4, 3}, {5, 4, 3}, false, true, {5, 2, 4, 4}},
                               ListCase{"matmult tensors T(a, b) (bigger b)", {5, 4, 3}, {5, 2, 6, 4}, true, true, {5, 2, 3, 6}}}) {
        run_test(lc.name, [&] {
            nt::TensorList a = F::randn(lc.as, DType::Float32, 51).split_axis(0), b = F::randn(lc.bs, DType::Float32, 52).split_axis(0);
            Tensor o = nt::matmult(a, b, lc.ta, lc.tb);
            SizeRef flat = lc.view;
            flat.erase(flat.begin());
            flat[0] *= 5;
            nt::utils::throw_exception(o.shape() == flat, "Error: Got unexpected shape (" + nt::shape_str(o.shape()) + ")");
            Tensor ov = o.view(lc.view);
            const int64_t per = ov.numel() / 5;
            for (int64_t i = 0; i < 5; ++i) {
                Tensor o1 = nt::matmult(a[(size_t)i], b[(size_t)i], lc.ta, lc.tb);
                nt::utils::throw_exception(o1.numel() == per && std::memcmp(o1.data_ptr(), static_cast<const char*>(ov.data_ptr()) + i * per * 4, (size_t)per * 4) == 0,
                                           "Error tensors did not match at index " + std::to_string(i));
            }
        });
    }
    run_test("matmult tensors: list errors", [] {
        nt::TensorList a = F::randn({3, 4, 5}, DType::Float32, 53).split_axis(0), b = F::randn({2, 5, 4}, DType::Float32, 54).split_axis(0);
        bool threw = false;
        try { nt::matmult(a, b); } catch (const nt::utils::nt_error&) { threw = true; }
        nt::utils::throw_exception(threw, "lists of different lengths must be rejected");
        nt::TensorList c = F::randn({3, 6, 4}, DType::Float32, 55).split_axis(0);
        threw = false;
        try { nt::matmult(a, c); } catch (const nt::utils::nt_error&) { threw = true; }
        nt::utils::throw_exception(threw, "inner sizes that differ must be rejected");
    });
    // tests/src/conv_test.cpp:192-213: conv2d over every floating and complex dtype
    run_test("conv2d dtype sweep (floating and complex)", [] {
        for (DType dt : {DType::Float32, DType::Float64, DType::Float16, DType::BFloat16, DType::Complex32, DType::Complex64, DType::Complex128}) {
            Tensor x = F::randn({1, 3, 16, 16}, dt, 61), w = F::randn({4, 3, 3, 3}, dt, 62);
            Tensor y = nt::conv2d(x, w, {1, 1}, {1, 1});
            nt::utils::throw_exception(!x.is_null() && !y.is_null() && y.shape() == SizeRef({1, 4, 16, 16}) && y.dtype() == dt,
                                       std::string("Error x was made null after conv2d call for ") + nt::dtype_name(dt));
        }
        // Complex64: the reference's lane-wise product = a real convolution of the real parts and one of the imaginary parts
        Tensor x = F::randn({2, 3, 9, 8}, DType::Complex64, 63), w = F::randn({4, 3, 3, 3}, DType::Complex64, 64);
        Tensor y = nt::conv2d(x, w, {1, 1}, {1, 1});
        for (int part = 0; part < 2; ++part) {
            Tensor xr({2, 3, 9, 8}, DType::Float32), wr({4, 3, 3, 3}, DType::Float32);
            for (int64_t i = 0; i < xr.numel(); ++i) xr.data<float>()[i] = x.data<float>()[2 * i + part];
            for (int64_t i = 0; i < wr.numel(); ++i) wr.data<float>()[i] = w.data<float>()[2 * i + part];
            Tensor yr = nt::conv2d(xr, wr, {1, 1}, {1, 1});
            for (int64_t i = 0; i < yr.numel(); ++i)
                nt::utils::throw_exception(std::fabs(yr.data<float>()[i] - y.data<float>()[2 * i + part]) <= 1e-4, "complex conv2d plane differs from the real convolution");
        }
        Tensor a = F::randn({7, 9}, DType::Complex128, 65), b = F::randn({9, 5}, DType::Complex128, 66);
        Tensor o = nt::matmult(a, b);
        for (int64_t i = 0; i < 7; ++i)
            for (int64_t j = 0; j < 5; ++j)
                for (int part = 0; part < 2; ++part) {
                    double sum = 0;
                    for (int64_t t = 0; t < 9; ++t) sum = std::fma(a.data<double>()[2 * (i * 9 + t) + part], b.data<double>()[2 * (t * 5 + j) + part], sum);
                    nt::utils::throw_exception(o.data<double>()[2 * (i * 5 + j) + part] == sum, "Complex128 matmult is the lane-wise fused chain, bit for bit");
                }
    });
    // tests/src/conv_test.cpp:175-189, :216-279: conv1d, conv3d and the transposed convolutions over every floating and complex dtype
    run_test("conv1d / conv3d / conv_transpose1d / 2d / 3d dtype sweep (floating and complex)", [] {
        for (DType dt : {DType::Float32, DType::Float64, DType::Float16, DType::BFloat16, DType::Complex32, DType::Complex64, DType::Complex128}) {
            const std::string name = nt::dtype_name(dt);
            Tensor x1 = F::randn({1, 3, 10}, dt, 71), w1 = F::randn({2, 3, 3}, dt, 72);
            Tensor y1 = nt::conv1d(x1, w1, 1, 1);
            nt::utils::throw_exception(!x1.is_null() && y1.shape() == SizeRef({1, 2, 10}) && y1.dtype() == dt, "conv1d for " + name);
            Tensor x3 = F::randn({1, 3, 8, 8, 8}, dt, 73), w3 = F::randn({4, 3, 3, 3, 3}, dt, 74);
            Tensor y3 = nt::conv3d(x3, w3, {1, 1, 1}, {1, 1, 1});
            nt::utils::throw_exception(!x3.is_null() && y3.shape() == SizeRef({1, 4, 8, 8, 8}) && y3.dtype() == dt, "conv3d for " + name);
            Tensor xt1 = F::randn({1, 3, 10}, dt, 75), wt1 = F::randn({3, 2, 3}, dt, 76);
            Tensor yt1 = nt::conv_transpose1d(xt1, wt1, 1, 1);
            nt::utils::throw_exception(!xt1.is_null() && yt1.shape() == SizeRef({1, 2, 10}) && yt1.dtype() == dt, "conv_transpose1d for " + name);
            Tensor xt2 = F::randn({1, 3, 16, 16}, dt, 77), wt2 = F::randn({3, 4, 3, 3}, dt, 78);
            Tensor yt2 = nt::conv_transpose2d(xt2, wt2, {1, 1}, {1, 1});
            nt::utils::throw_exception(!xt2.is_null() && yt2.shape() == SizeRef({1, 4, 16, 16}) && yt2.dtype() == dt, "conv_transpose2d for " + name);
            Tensor xt3 = F::randn({1, 3, 8, 8, 8}, dt, 79), wt3 = F::randn({3, 4, 3, 3, 3}, dt, 80);
            Tensor yt3 = nt::conv_transpose3d(xt3, wt3, {1, 1, 1}, {1, 1, 1});
            nt::utils::throw_exception(!xt3.is_null() && yt3.shape() == SizeRef({1, 4, 8, 8, 8}) && yt3.dtype() == dt, "conv_transpose3d for " + name);
        }
        // Complex64 conv3d and conv_transpose2d: every plane is the real operation on that plane (the reference's lane-wise product)
        Tensor x = F::randn({2, 4, 4, 5, 6}, DType::Complex64, 81), w = F::randn({6, 2, 2, 3, 2}, DType::Complex64, 82);
        Tensor y = nt::conv3d(x, w, {1, 2, 1}, {1, 0, 1}, {1, 1, 1}, 2);
        Tensor xt = F::randn({2, 4, 5, 6}, DType::Complex64, 83), wt = F::randn({4, 3, 3, 2}, DType::Complex64, 84);
        Tensor yt = nt::conv_transpose2d(xt, wt, {2, 2}, {1, 1}, {1, 1}, {1, 1}, 2);
        auto plane = [](const Tensor& t, int part) {
            Tensor r(t.shape(), DType::Float32);
            for (int64_t i = 0; i < r.numel(); ++i) r.data<float>()[i] = t.data<float>()[2 * i + part];
            return r;
        };
        for (int part = 0; part < 2; ++part) {
            Tensor yr = nt::conv3d(plane(x, part), plane(w, part), {1, 2, 1}, {1, 0, 1}, {1, 1, 1}, 2);
            for (int64_t i = 0; i < yr.numel(); ++i)
                nt::utils::throw_exception(std::fabs(yr.data<float>()[i] - y.data<float>()[2 * i + part]) <= 1e-4, "complex conv3d plane differs from the real convolution");
            Tensor ytr = nt::conv_transpose2d(plane(xt, part), plane(wt, part), {2, 2}, {1, 1}, {1, 1}, {1, 1}, 2);
            for (int64_t i = 0; i < ytr.numel(); ++i)
                nt::utils::throw_exception(std::fabs(ytr.data<float>()[i] - yt.data<float>()[2 * i + part]) <= 1e-4, "complex conv_transpose2d plane differs from the real one");
        }
    });
    run_test("matmult transposed view == flag (no copy)", [] {
        Tensor a = F::randn({6, 40, 30}, DType::Float32, 33), b = F::randn({6, 20, 30}, DType::Float32, 34);
        Tensor o1 = nt::matmult(a, b, false, true);
        Tensor o2 = nt::matmult(a, b.transpose(-1, -2));
        nt::utils::throw_exception(std::memcmp(o1.data_ptr(), o2.data_ptr(), (size_t)o1.numel() * 4) == 0, "view and flag disagree");
    });
    run_test("matmult out= accumulates", [] {
        Tensor a = F::randn({33, 17}, DType::Float32, 35), b = F::randn({17, 29}, DType::Float32, 36);
        Tensor c0 = F::randn({33, 29}, DType::Float32, 37), c = c0.clone();
        nt::matmult(a, b, c);
        nt::utils::throw_exception(max_err_vs_double(a, b, c, false, false, c0.data<float>()) <= 1e-3, "C += A.B");
    });
    run_test("matmult int32 / float64 / int64 values", [] {
        Tensor a = F::randn({19, 23}, DType::int32, 41), b = F::randn({23, 7}, DType::int32, 42);
        Tensor o = nt::matmult(a, b);
        for (int64_t i = 0; i < 19; ++i)
            for (int64_t j = 0; j < 7; ++j) {
                int64_t s = 0;
                for (int64_t t = 0; t < 23; ++t) s += (int64_t)a.data<int32_t>()[i * 23 + t] * b.data<int32_t>()[t * 7 + j];
                nt::utils::throw_exception(o.data<int32_t>()[i * 7 + j] == (int32_t)s, "int32 result not exact");
            }
        Tensor x = F::randn({12, 40}, DType::Float64, 43), y = F::randn({40, 9}, DType::Float64, 44);
        Tensor z = nt::matmult(x, y);
        double worst = 0;
        for (int64_t i = 0; i < 12; ++i)
            for (int64_t j = 0; j < 9; ++j) {
                double s = 0;
                for (int64_t t = 0; t < 40; ++t) s += x.data<double>()[i * 40 + t] * y.data<double>()[t * 9 + j];
                worst = std::fmax(worst, std::fabs(s - z.data<double>()[i * 9 + j]));
            }
        nt::utils::throw_exception(worst <= 1e-12, "float64 result off by " + std::to_string(worst));
    });

    linear_shape_case("linear 2d", {30, 30}, {30, 30}, {30}, false, false, {30, 30});
    linear_shape_case("linear 2d Ta", {30, 14}, {30, 30}, {30}, true, false, {14, 30});
    linear_shape_case("linear 2d Tb", {30, 30}, {14, 30}, {30, 14}, false, true, {30, 14});
    linear_shape_case("linear 2d T(a, b)", {30, 14}, {14, 30}, {14, 14}, true, true, {14, 14});
    linear_shape_case("linear 3d", {10, 30, 30}, {10, 30, 30}, {30, 30}, false, false, {10, 30, 30});
    linear_shape_case("linear 3d Ta", {10, 30, 14}, {10, 30, 30}, {14, 30}, true, false, {10, 14, 30});
    linear_shape_case("linear 3d Tb", {10, 30, 30}, {10, 14, 30}, {30, 14}, false, true, {10, 30, 14});
    linear_shape_case("linear 3d T(a, b)", {10, 30, 14}, {10, 14, 30}, {14, 14}, true, true, {10, 14, 14});
    linear_shape_case("linear 3d bigger A", {5, 10, 30, 30}, {10, 30, 30}, {30, 30}, false, false, {5, 10, 30, 30});
    linear_shape_case("linear 3d Ta bigger A", {5, 10, 30, 14}, {10, 30, 30}, {14, 30}, true, false, {5, 10, 14, 30});
    linear_shape_case("linear 3d Tb bigger A", {5, 10, 30, 30}, {10, 14, 30}, {30, 14}, false, true, {5, 10, 30, 14});
    linear_shape_case("linear 3d T(a, b) bigger A", {5, 10, 30, 14}, {10, 14, 30}, {14, 14}, true, true, {5, 10, 14, 14});
    linear_shape_case("linear 3d bigger B", {10, 30, 30}, {5, 10, 30, 30}, {30, 30}, false, false, {5, 10, 30, 30});
    linear_shape_case("linear 3d Ta bigger B", {10, 30, 14}, {5, 10, 30, 30}, {14, 30}, true, false, {5, 10, 14, 30});
    linear_shape_case("linear 3d Tb bigger B", {10, 30, 30}, {5, 10, 14, 30}, {30, 14}, false, true, {5, 10, 30, 14});
    linear_shape_case("linear 3d T(a, b) bigger B", {10, 30, 14}, {5, 10, 14, 30}, {14, 14}, true, true, {5, 10, 14, 14});

    run_test("Linear Autograd test (golden)", [&] {
        Tensor x = F::from_numpy(g + "/linear_input.npy"), grad = F::from_numpy(g + "/linear_grad.npy");
        Tensor w = F::from_numpy(g + "/linear_weight.npy"), b = F::from_numpy(g + "/linear_bias.npy");
        Tensor o = nt::linear(x, w, b, false, true);
        nt::utils::throw_exception(o.shape() == SizeRef({3, 4, 3}), "forward shape");
        F::LinearGrads gr = F::linear_backward(x, w, b, grad, false, true);
        nt::utils::throw_exception(F::allclose(gr.dx, F::from_numpy(g + "/linear_xgrad.npy"), 1e-5, 1e-6) &&
                                       F::allclose(gr.dw, F::from_numpy(g + "/linear_wgrad.npy"), 1e-5, 1e-6) &&
                                       F::allclose(gr.db, F::from_numpy(g + "/linear_bgrad.npy"), 1e-5, 1e-6),
                                   "Error, grads do not match");
    });
    run_test("layers::Linear forward/backward", [] {
        nt::layers::Linear lin(20, 12);
        Tensor x = F::randn({7, 20}, DType::Float32, 51), gy = F::randn({7, 12}, DType::Float32, 52);
        Tensor y = lin.forward(x);
        nt::utils::throw_exception(y.shape() == SizeRef({7, 12}), "forward shape");
        Tensor mm = nt::matmult(x, lin.Weight);
        for (int64_t i = 0; i < y.numel(); ++i)
            nt::utils::throw_exception(std::fabs(y.data<float>()[i] - mm.data<float>()[i] - lin.Bias.data<float>()[i % 12]) <= 1e-4, "forward value");
        F::LinearGrads gr = lin.backward(x, gy);
        nt::utils::throw_exception(gr.dx.shape() == x.shape() && gr.dw.shape() == lin.Weight.shape() && gr.db.shape() == lin.Bias.shape(), "grad shapes");
        nt::utils::throw_exception(max_err_vs_double(gy, lin.Weight, gr.dx, false, true) <= 1e-3, "dX = dY.W^T");
        nt::utils::throw_exception(max_err_vs_double(x, gy, gr.dw, true, false) <= 1e-3, "dW = X^T.dY");
    });
    for (const char* sfx : {"", "_batched", "_grouped", "_grouped_batched"}) {
        const std::string name = std::string("conv2d golden") + sfx;
        run_test(name.c_str(), [&] {
            const bool grouped = std::strstr(sfx, "grouped") != nullptr;
            Tensor x = F::from_numpy(g + "/conv2d_input" + sfx + ".npy"), w = F::from_numpy(g + "/conv2d_weight" + sfx + ".npy");
            Tensor want = F::from_numpy(g + "/conv2d_output" + sfx + ".npy");
            const int64_t pad = grouped ? 0 : 1;
            Tensor o = nt::conv2d(x, w, {1, 1}, {pad, pad}, {1, 1}, grouped ? 2 : 1);
            nt::utils::throw_exception(o.shape() == want.shape(), "output shape " + nt::shape_str(o.shape()));
            nt::utils::throw_exception(F::allclose(o, want, 1e-4, 1e-4), "conv2d output differs from the fixture");
            // xgrad / wgrad of the same test case (conv_dimage, conv_dkernel)
            F::ConvGrads gr = F::conv2d_backward(x, w, F::from_numpy(g + "/conv2d_grad" + sfx + ".npy"), {1, 1}, {pad, pad}, {1, 1}, grouped ? 2 : 1);
            nt::utils::throw_exception(F::allclose(gr.d_image, F::from_numpy(g + "/conv2d_xgrad" + sfx + ".npy"), 1e-4, 1e-4), "xgrad differs from the fixture");
            nt::utils::throw_exception(F::allclose(gr.d_kernel, F::from_numpy(g + "/conv2d_wgrad" + sfx + ".npy"), 1e-4, 1e-3), "wgrad differs from the fixture");
        });
    }
    // tests/src/conv_autograd_test.cpp:125-247 (conv1d), :555-716 (conv_transpose1d), :720-846 (conv_transpose2d)
    auto close = [](const Tensor& a, const Tensor& b, const char* what) {
        nt::utils::throw_exception(a.shape() == b.shape(), std::string(what) + " shape " + nt::shape_str(a.shape()));
        nt::utils::throw_exception(F::allclose(a, b, 1e-4, 1e-3), std::string(what) + " differs from the fixture");
    };
    auto fixture = [&](const std::string& fam, const char* part, const char* sfx) { return F::from_numpy(g + "/" + fam + "_" + part + sfx + ".npy"); };
    for (const char* sfx : {"", "_batched", "_grouped", "_grouped_batched"}) {
        run_test((std::string("conv1d golden") + sfx).c_str(), [&] {
            const bool grouped = std::strstr(sfx, "grouped") != nullptr;
            Tensor x = fixture("conv1d", "input", sfx), w = fixture("conv1d", "weight", sfx);
            Tensor o = nt::conv1d(x, w, 1, grouped ? 0 : 1, 1, grouped ? 2 : 1);
            close(o, fixture("conv1d", "output", sfx), "conv1d output");
            F::ConvGrads gr = F::conv1d_backward(x, w, fixture("conv1d", "grad", sfx), 1, grouped ? 0 : 1, 1, grouped ? 2 : 1);
            close(gr.d_image, fixture("conv1d", "xgrad", sfx), "conv1d xgrad");
            close(gr.d_kernel, fixture("conv1d", "wgrad", sfx), "conv1d wgrad");
        });
    }
    struct TCase { const char* sfx; int64_t stride, padding, output_padding, groups; };
    for (const TCase& c : {TCase{"", 2, 0, 1, 1}, TCase{"_grouped", 1, 1, 0, 2}, TCase{"_grouped_bigger", 1, 1, 0, 5}, TCase{"_batched", 2, 1, 1, 1},
                           TCase{"_grouped_batched", 1, 1, 0, 2}}) {
        run_test((std::string("conv_transpose1d golden") + c.sfx).c_str(), [&] {
            Tensor x = fixture("conv_transpose1d", "input", c.sfx), w = fixture("conv_transpose1d", "weight", c.sfx);
            Tensor o = nt::conv_transpose1d(x, w, c.stride, c.padding, c.output_padding, 1, c.groups);
            close(o, fixture("conv_transpose1d", "output", c.sfx), "conv_transpose1d output");
            F::ConvGrads gr = F::conv_transpose1d_backward(x, w, fixture("conv_transpose1d", "grad", c.sfx), c.stride, c.padding, c.output_padding, 1, c.groups);
            close(gr.d_image, fixture("conv_transpose1d", "xgrad", c.sfx), "conv_transpose1d xgrad");
            close(gr.d_kernel, fixture("conv_transpose1d", "wgrad", c.sfx), "conv_transpose1d wgrad");
        });
    }
    for (const TCase& c : {TCase{"", 2, 0, 1, 1}, TCase{"_grouped", 1, 1, 0, 5}, TCase{"_batched", 2, 1, 1, 1}, TCase{"_grouped_batched", 1, 1, 0, 2}}) {
        run_test((std::string("conv_transpose2d golden") + c.sfx).c_str(), [&] {
            Tensor x = fixture("conv_transpose2d", "input", c.sfx), w = fixture("conv_transpose2d", "weight", c.sfx);
            Tensor o = nt::conv_transpose2d(x, w, {c.stride, c.stride}, {c.padding, c.padding}, {c.output_padding, c.output_padding}, {1, 1}, c.groups);
            close(o, fixture("conv_transpose2d", "output", c.sfx), "conv_transpose2d output");
            F::ConvGrads gr = F::conv_transpose2d_backward(x, w, fixture("conv_transpose2d", "grad", c.sfx), {c.stride, c.stride}, {c.padding, c.padding},
                                                           {c.output_padding, c.output_padding}, {1, 1}, c.groups);
            close(gr.d_image, fixture("conv_transpose2d", "xgrad", c.sfx), "conv_transpose2d xgrad");
            close(gr.d_kernel, fixture("conv_transpose2d", "wgrad", c.sfx), "conv_transpose2d wgrad");
        });
    }
    // tests/src/conv_autograd_test.cpp:375-497 (conv3d), :847-971 (conv_transpose3d)
    for (const char* sfx : {"", "_batched", "_grouped", "_grouped_batched"}) {
        run_test((std::string("conv3d golden") + sfx).c_str(), [&] {
            const bool grouped = std::strstr(sfx, "grouped") != nullptr;
            const int64_t pad = grouped ? 0 : 1, groups = grouped ? 2 : 1;
            Tensor x = fixture("conv3d", "input", sfx), w = fixture("conv3d", "weight", sfx);
            Tensor o = nt::conv3d(x, w, {1, 1, 1}, {pad, pad, pad}, {1, 1, 1}, groups);
            close(o, fixture("conv3d", "output", sfx), "conv3d output");
            F::ConvGrads gr = F::conv3d_backward(x, w, fixture("conv3d", "grad", sfx), {1, 1, 1}, {pad, pad, pad}, {1, 1, 1}, groups);
            close(gr.d_image, fixture("conv3d", "xgrad", sfx), "conv3d xgrad");
            close(gr.d_kernel, fixture("conv3d", "wgrad", sfx), "conv3d wgrad");
        });
    }
    for (const TCase& c : {TCase{"", 2, 0, 1, 1}, TCase{"_grouped_batched", 1, 1, 0, 2}}) {
        run_test((std::string("conv_transpose3d golden") + c.sfx).c_str(), [&] {
            Tensor x = fixture("conv_transpose3d", "input", c.sfx), w = fixture("conv_transpose3d", "weight", c.sfx);
            const nt::utils::my_n_tuple<3> s{c.stride, c.stride, c.stride}, p{c.padding, c.padding, c.padding},
                op{c.output_padding, c.output_padding, c.output_padding}, d{1, 1, 1};
            Tensor o = nt::conv_transpose3d(x, w, s, p, op, d, c.groups);
            close(o, fixture("conv_transpose3d", "output", c.sfx), "conv_transpose3d output");
            F::ConvGrads gr = F::conv_transpose3d_backward(x, w, fixture("conv_transpose3d", "grad", c.sfx), s, p, op, d, c.groups);
            close(gr.d_image, fixture("conv_transpose3d", "xgrad", c.sfx), "conv_transpose3d xgrad");
            close(gr.d_kernel, fixture("conv_transpose3d", "wgrad", c.sfx), "conv_transpose3d wgrad");
        });
    }
    run_test("unfold2d golden", [&] {
        Tensor x = F::from_numpy(g + "/unfold_input.npy"), want = F::from_numpy(g + "/unfold_output.npy");
        Tensor col = F::unfold2d(x, {3, 2}, {1, 2}, {1, 1}, {2, 2}, true);
        nt::utils::throw_exception(col.shape() == SizeRef({1, 18, 16}) && std::memcmp(col.data_ptr(), want.data_ptr(), 18 * 16 * 4) == 0, "unfold output");
        Tensor gi = F::unfold2d_backward(F::from_numpy(g + "/unfold_grad.npy"), {8, 8}, {3, 2}, {1, 2}, {1, 1}, {2, 2});
        nt::utils::throw_exception(F::allclose(gi, F::from_numpy(g + "/unfold_input_grad.npy"), 1e-5, 1e-6), "unfold input grad");
    });
}

// Tensors moved to the GPU with to(DeviceType::HIP): every operation stays in HBM and must give what the same
// operation gives on host tensors (the same kernels run either way; only the copies differ).
static void device_resident_cases(const std::string& g) {
    using nt::DeviceType;
    // integers bit for bit; floating results within rounding (strided batches and pointer tables may take different kernels)
    auto same_bits = [](const Tensor& dev, const Tensor& host, const char* what) {
        nt::utils::throw_exception(dev.device() == DeviceType::HIP, std::string(what) + ": result left the device");
        Tensor h = dev.cpu();
        nt::utils::throw_exception(h.shape() == host.shape() && h.dtype() == host.dtype(), std::string(what) + ": shape / dtype");
        bool ok;
        if (host.dtype() == DType::BFloat16) {
            auto f = [](uint16_t v) { uint32_t u = (uint32_t)v << 16; float x; std::memcpy(&x, &u, 4); return x; };
            ok = true;
            for (int64_t i = 0; i < host.numel(); ++i) {
                const float x = f(h.data<uint16_t>()[i]), y = f(host.data<uint16_t>()[i]);
                ok = ok && std::fabs(x - y) <= 0.02f * (1.0f + std::fabs(y));
            }
        } else if (host.dtype() == DType::Float32 || host.dtype() == DType::Float64) {
            ok = F::allclose(h, host, 1e-4, 1e-4);
        } else {
            ok = std::memcmp(h.data_ptr(), host.data_ptr(), (size_t)(host.numel() * nt::dtype_size(host.dtype()))) == 0;
        }
        nt::utils::throw_exception(ok, std::string(what) + ": device and host results differ");
    };
    run_test("device tensor round trip, views, clone, zeros", [] {
        Tensor a = F::randn({3, 7, 5}, DType::Float32, 71);
        Tensor d = a.to(DeviceType::HIP);
        nt::utils::throw_exception(d.is_device() && d.to(DeviceType::HIP).data_ptr() == d.data_ptr(), "to(same device) must not copy");
        nt::utils::throw_exception(F::allclose(d, a, 0, 0), "round trip");
        nt::utils::throw_exception(F::allclose(d.transpose(-1, -2).cpu(), a.transpose(-1, -2).clone(), 0, 0), "strided view to host");
        nt::utils::throw_exception(F::allclose(d.transpose(-1, -2).clone(), a.transpose(-1, -2).clone(), 0, 0), "clone of a strided device view");
        nt::utils::throw_exception(F::allclose(d.item(2).clone(), a.item(2).clone(), 0, 0), "item");
        nt::utils::throw_exception(F::allclose(F::zeros({4, 3}, DType::Float32, DeviceType::HIP), F::zeros({4, 3}), 0, 0), "zeros");
        nt::utils::throw_exception(F::allclose(d.sum_leading({5}), a.sum_leading({5}), 1e-5, 1e-5), "sum_as over leading dims");
        nt::utils::throw_exception(F::allclose(d.sum_leading({7, 1}), a.sum_leading({7, 1}), 1e-5, 1e-5), "sum_as over an inner dim");
    });
    expect_throw("matmult of a host and a device tensor", [] {
        nt::matmult(F::zeros({4, 4}), F::zeros({4, 4}, DType::Float32, DeviceType::HIP));
    });
    expect_throw("linear with the bias on the other device", [] {
        nt::linear(F::zeros({4, 4}, DType::Float32, DeviceType::HIP), F::zeros({4, 4}, DType::Float32, DeviceType::HIP), F::zeros({4}));
    });
    for (DType dt : {DType::Float32, DType::Float64, DType::BFloat16, DType::int32}) {
        run_test((std::string("device matmult / linear == host, ") + nt::dtype_name(dt)).c_str(), [&] {
            Tensor a = F::randn({5, 2, 33, 20}, dt, 81), b = F::randn({2, 20, 17}, dt, 82), a2 = F::randn({2, 20, 33}, dt, 83);
            Tensor bb = F::randn({5, 2, 20, 17}, dt, 87);
            Tensor da = a.to(DeviceType::HIP), db = b.to(DeviceType::HIP), da2 = a2.to(DeviceType::HIP), dbb = bb.to(DeviceType::HIP);
            same_bits(nt::matmult(da, db), nt::matmult(a, b), "bigger A");
            same_bits(nt::matmult(da2, dbb, true, false), nt::matmult(a2, bb, true, false), "bigger B, transpose_a");
            same_bits(nt::matmult(da, db.transpose(-1, -2).clone(), false, true), nt::matmult(a, b.transpose(-1, -2).clone(), false, true), "transpose_b");
            same_bits(nt::matmult(da, db.transpose(-1, -2).clone().transpose(-1, -2)), nt::matmult(a, b), "transposed device view == flag");
            Tensor c = F::randn({5, 2, 33, 17}, dt, 84), dc = c.to(DeviceType::HIP);
            nt::matmult(a, b, c);
            nt::matmult(da, db, dc);
            same_bits(dc, c, "out= accumulates on the device");
            if (dt != DType::int32) {
                Tensor bias = F::randn({17}, dt, 85), bias2 = F::randn({2, 33, 1}, dt, 86);
                same_bits(nt::linear(da, db, bias.to(DeviceType::HIP)), nt::linear(a, b, bias), "linear, bias [n]");
                same_bits(nt::linear(da, db, bias2.to(DeviceType::HIP)), nt::linear(a, b, bias2), "linear, bias [2, m, 1]");
            }
        });
    }
    run_test("Linear -> Linear forward and backward without leaving the device", [] {
        nt::layers::Linear l1(64, 48, true, DType::Float32, 91), l2(48, 24, true, DType::Float32, 93);
        Tensor x = F::randn({6, 10, 64}, DType::Float32, 95), gy = F::randn({6, 10, 24}, DType::Float32, 96);
        Tensor h = l1.forward(x), y = l2.forward(h);
        F::LinearGrads g2 = l2.backward(h, gy), g1 = l1.backward(x, g2.dx);
        nt::layers::Linear d1 = l1, d2 = l2;
        d1.to(DeviceType::HIP); d2.to(DeviceType::HIP);
        Tensor dx = x.to(DeviceType::HIP), dgy = gy.to(DeviceType::HIP);
        Tensor dh = d1.forward(dx), dy = d2.forward(dh);
        F::LinearGrads dg2 = d2.backward(dh, dgy), dg1 = d1.backward(dx, dg2.dx);
        nt::utils::throw_exception(dy.is_device() && dg1.dx.is_device() && dg1.dw.is_device() && dg1.db.is_device(), "results left the device");
        nt::utils::throw_exception(F::allclose(dy, y, 1e-4, 1e-4), "forward");
        nt::utils::throw_exception(F::allclose(dg1.dx, g1.dx, 1e-4, 1e-4) && F::allclose(dg2.dw, g2.dw, 1e-4, 1e-3), "dx / dw of the chain");
        // dW of a batched input and db are sums over the leading dims: one GEMM with a row of ones on the device
        nt::utils::throw_exception(F::allclose(dg1.dw, g1.dw, 1e-4, 1e-3) && F::allclose(dg1.db, g1.db, 1e-4, 1e-3) &&
                                       F::allclose(dg2.db, g2.db, 1e-4, 1e-3), "reduced gradients");
    });
    run_test("Linear -> ReLU -> Linear: relu_(linear) in one launch == the two in a row, bit for bit, four dtypes", [&] {
        for (DType dt : {DType::Float32, DType::Float64, DType::Float16, DType::BFloat16}) {
            Tensor x = F::randn({3, 40, 64}, dt, 201), w = F::randn({64, 72}, dt, 202), b = F::randn({72}, dt, 203);
            Tensor w2 = F::randn({72, 24}, dt, 204), b2 = F::randn({24}, dt, 205);
            // host: the reference's order of calls
            Tensor h = nt::linear(x, w, b);
            Tensor hr = F::relu(h);
            Tensor y = nt::linear(hr, w2, b2);
            nt::utils::throw_exception(!F::allclose(h, hr, 0, 0), "relu changed nothing");
            nt::utils::throw_exception(F::allclose(F::linear_relu(x, w, b), hr, 0, 0), "host linear_relu");
            // device: fused epilogue, relu_ in place on device memory, and the chain
            Tensor dx = x.to(DeviceType::HIP), dw = w.to(DeviceType::HIP), db = b.to(DeviceType::HIP);
            Tensor dfused = F::linear_relu(dx, dw, db);
            nt::utils::throw_exception(dfused.is_device(), "result left the device");
            same_bits(dfused, hr, "device linear_relu == relu(linear) on the host");
            Tensor dh = nt::linear(dx, dw, db);
            same_bits(F::relu_(dh), hr, "device relu_ in place");
            same_bits(nt::linear(dfused, w2.to(DeviceType::HIP), b2.to(DeviceType::HIP)), y, "second layer on the clamped activations");
        }
        // NaN and -0 become +0 (max(x, 0) returns its second operand for both)
        Tensor t = F::randn({2, 8}, DType::Float32, 206);
        float* p = static_cast<float*>(t.data_ptr());
        p[0] = std::nanf(""); p[1] = -0.0f; p[2] = -3.5f; p[3] = 2.25f;
        Tensor r = F::relu(t), dr = F::relu(t.to(DeviceType::HIP));
        const float* q = static_cast<const float*>(r.data_ptr());
        uint32_t b0, b1;
        std::memcpy(&b0, q, 4); std::memcpy(&b1, q + 1, 4);
        nt::utils::throw_exception(b0 == 0 && b1 == 0 && q[2] == 0.0f && q[3] == 2.25f, "relu of NaN / -0 / negative / positive");
        same_bits(dr, r, "device relu of NaN and -0");
    });
    run_test("two Linear layers on 2048 rows: host tensors against device tensors (timing printed)", [] {
        nt::layers::Linear l1(1024, 1024, true, DType::Float32, 97), l2(1024, 1024, true, DType::Float32, 98);
        Tensor x = F::randn({2048, 1024}, DType::Float32, 99);
        auto now = [] { return std::chrono::steady_clock::now(); };
        auto ms = [](auto a, auto b) { return std::chrono::duration<double, std::milli>(b - a).count(); };
        Tensor y = l2.forward(l1.forward(x));                       // warm-up (library load, clocks)
        auto t0 = now();
        for (int i = 0; i < 5; ++i) y = l2.forward(l1.forward(x));
        const double host_ms = ms(t0, now()) / 5;
        nt::layers::Linear d1 = l1, d2 = l2;
        d1.to(DeviceType::HIP); d2.to(DeviceType::HIP);
        Tensor dx = x.to(DeviceType::HIP);
        Tensor dy = d2.forward(d1.forward(dx));
        Tensor first = dy.cpu();
        t0 = now();
        for (int i = 0; i < 50; ++i) dy = d2.forward(d1.forward(dx));
        Tensor last = dy.cpu();                                      // (waits for the stream)
        const double dev_ms = ms(t0, now()) / 50;
        std::printf("       host tensors %.3f ms per chain (PCIe copies in every call), device tensors %.3f ms\n", host_ms, dev_ms);
        nt::utils::throw_exception(F::allclose(last, y, 1e-4, 1e-3) && F::allclose(first, last, 0, 0), "chain result");
    });
    for (const char* sfx : {"", "_grouped_batched"}) {
        run_test((std::string("device conv2d forward / backward == golden") + sfx).c_str(), [&] {
            const bool grouped = std::strstr(sfx, "grouped") != nullptr;
            const int64_t pad = grouped ? 0 : 1, groups = grouped ? 2 : 1;
            auto fx = [&](const char* part) { return F::from_numpy(g + "/conv2d_" + part + sfx + ".npy"); };
            Tensor x = fx("input").to(DeviceType::HIP), w = fx("weight").to(DeviceType::HIP);
            Tensor o = nt::conv2d(x, w, {1, 1}, {pad, pad}, {1, 1}, groups);
            nt::utils::throw_exception(o.is_device() && F::allclose(o, fx("output"), 1e-4, 1e-4), "conv2d output");
            F::ConvGrads gr = F::conv2d_backward(x, w, fx("grad").to(DeviceType::HIP), {1, 1}, {pad, pad}, {1, 1}, groups);
            nt::utils::throw_exception(gr.d_image.is_device() && F::allclose(gr.d_image, fx("xgrad"), 1e-4, 1e-4), "conv2d xgrad");
            nt::utils::throw_exception(F::allclose(gr.d_kernel, fx("wgrad"), 1e-4, 1e-3), "conv2d wgrad");
        });
    }
    run_test("device tensors of tensors == host, bit for bit", [&] {
        Tensor A = F::randn({5, 2, 40, 30}, DType::Float32, 111), B = F::randn({5, 40, 24}, DType::Float32, 112);
        nt::TensorList a = A.split_axis(0), b = B.split_axis(0);
        nt::TensorList da = A.to(DeviceType::HIP).split_axis(0), db = B.to(DeviceType::HIP).split_axis(0);
        Tensor o = nt::matmult(a, b, true, false), dout = nt::matmult(da, db, true, false);
        nt::utils::throw_exception(dout.is_device() && dout.shape() == SizeRef({10, 30, 24}), "shape of the device result");
        same_bits(dout, o, "list product");
    });
    run_test("device lists of separately allocated tensors: every item == the pair alone, bit for bit", [&] {
        // the reference's list test (tests/src/matmult_test.cpp:108-189) on lists that are NOT slices of one allocation, at
        // sizes where an item alone is split along k (64 x 4096 x 64: its items then go out one by one) and where it is not
        // (a pointer-table batch); two rounds, so the cached tables are reused
        for (int round = 0; round < 2; ++round)
            for (const SizeRef& mkn : {SizeRef{64, 4096, 64}, SizeRef{96, 200, 72}, SizeRef{16, 512, 128}}) {
                nt::TensorList da, db;
                for (int i = 0; i < 4; ++i) {
                    da.push_back(F::randn({mkn[0], mkn[1]}, DType::Float32, 300 + i + 10 * round).to(DeviceType::HIP));
                    db.push_back(F::randn({mkn[1], mkn[2]}, DType::Float32, 400 + i + 10 * round).to(DeviceType::HIP));
                }
                nt::TensorList shuffled_a = {da[2], da[0], da[3], da[0]}, shuffled_b = {db[2], db[1], db[3], db[0]};
                Tensor o = nt::matmult(shuffled_a, shuffled_b);
                nt::utils::throw_exception(o.is_device() && o.shape() == SizeRef({4 * mkn[0], mkn[2]}), "shape of the list result");
                Tensor oh = o.cpu();
                const int ia[4] = {2, 0, 3, 0}, ib[4] = {2, 1, 3, 0};
                for (int i = 0; i < 4; ++i) {
                    Tensor one = nt::matmult(da[(size_t)ia[i]], db[(size_t)ib[i]]).cpu();
                    const size_t bytes = (size_t)(mkn[0] * mkn[2]) * sizeof(float);
                    nt::utils::throw_exception(std::memcmp(static_cast<const char*>(oh.data_ptr()) + (size_t)i * bytes, one.data_ptr(), bytes) == 0,
                                               "item " + std::to_string(i) + " of the list differs from the pair alone");
                }
            }
    });
    run_test("device conv2d (channels-last path), conv1d, conv_transpose2d, unfold2d, conv3d == host", [&] {
        Tensor x = F::randn({3, 32, 9, 11}, DType::Float32, 101), w = F::randn({24, 16, 3, 3}, DType::Float32, 102);
        Tensor dx = x.to(DeviceType::HIP), dw = w.to(DeviceType::HIP);
        nt::utils::throw_exception(F::allclose(nt::conv2d(dx, dw, {1, 1}, {1, 1}, {1, 1}, 2), nt::conv2d(x, w, {1, 1}, {1, 1}, {1, 1}, 2), 1e-5, 1e-5), "conv2d");
        Tensor x1 = F::randn({4, 6, 40}, DType::Float32, 103), w1 = F::randn({8, 3, 5}, DType::Float32, 104);
        same_bits(nt::conv1d(x1.to(DeviceType::HIP), w1.to(DeviceType::HIP), 2, 2, 1, 2), nt::conv1d(x1, w1, 2, 2, 1, 2), "conv1d");
        Tensor xt = F::randn({2, 6, 7, 5}, DType::Float32, 105), wt = F::randn({6, 4, 3, 3}, DType::Float32, 106);
        nt::utils::throw_exception(F::allclose(nt::conv_transpose2d(xt.to(DeviceType::HIP), wt.to(DeviceType::HIP), {2, 2}, {1, 1}, {1, 1}, {1, 1}, 2),
                                               nt::conv_transpose2d(xt, wt, {2, 2}, {1, 1}, {1, 1}, {1, 1}, 2), 1e-5, 1e-5), "conv_transpose2d");
        same_bits(F::unfold2d(dx, {3, 2}, {1, 2}, {1, 1}, {2, 2}, true), F::unfold2d(x, {3, 2}, {1, 2}, {1, 1}, {2, 2}, true), "unfold2d");
        Tensor x3 = F::randn({2, 4, 5, 6, 7}, DType::Float32, 107), w3 = F::randn({6, 4, 2, 3, 2}, DType::Float32, 108);
        same_bits(nt::conv3d(x3.to(DeviceType::HIP), w3.to(DeviceType::HIP)), nt::conv3d(x3, w3), "conv3d");
    });
    run_test("device conv3d family stays in HBM: forward, gradients, transposed == host", [&] {
        Tensor x3 = F::randn({2, 4, 5, 6, 7}, DType::Float32, 121), w3 = F::randn({6, 2, 2, 3, 2}, DType::Float32, 122);
        Tensor dx3 = x3.to(DeviceType::HIP), dw3 = w3.to(DeviceType::HIP);
        Tensor y = nt::conv3d(x3, w3, {1, 2, 1}, {1, 0, 1}, {1, 1, 2}, 2), dy = nt::conv3d(dx3, dw3, {1, 2, 1}, {1, 0, 1}, {1, 1, 2}, 2);
        nt::utils::throw_exception(dy.is_device() && F::allclose(dy, y, 1e-5, 1e-5), "conv3d (strided, dilated, grouped)");
        Tensor g = F::randn(y.shape(), DType::Float32, 123);
        F::ConvGrads hg = F::conv3d_backward(x3, w3, g, {1, 2, 1}, {1, 0, 1}, {1, 1, 2}, 2);
        F::ConvGrads dg = F::conv3d_backward(dx3, dw3, g.to(DeviceType::HIP), {1, 2, 1}, {1, 0, 1}, {1, 1, 2}, 2);
        nt::utils::throw_exception(dg.d_image.is_device() && dg.d_kernel.is_device() && F::allclose(dg.d_image, hg.d_image, 1e-4, 1e-4) &&
                                       F::allclose(dg.d_kernel, hg.d_kernel, 1e-4, 1e-3), "conv3d gradients");
        Tensor xt = F::randn({2, 6, 3, 4, 5}, DType::Float32, 124), wt = F::randn({6, 2, 2, 3, 3}, DType::Float32, 125);
        Tensor yt = nt::conv_transpose3d(xt, wt, {2, 1, 2}, {0, 1, 1}, {1, 0, 1}, {1, 1, 1}, 2);
        Tensor dyt = nt::conv_transpose3d(xt.to(DeviceType::HIP), wt.to(DeviceType::HIP), {2, 1, 2}, {0, 1, 1}, {1, 0, 1}, {1, 1, 1}, 2);
        nt::utils::throw_exception(dyt.is_device() && F::allclose(dyt, yt, 1e-5, 1e-5), "conv_transpose3d");
    });
}

int main(int argc, char** argv) {
    if (argc < 2) { std::fprintf(stderr, "usage: %s <golden dir> [--host-only]\n", argv[0]); return 2; }
    const bool host_only = argc > 2 && std::strcmp(argv[2], "--host-only") == 0;
    host_only_cases();
    if (!host_only) { device_cases(argv[1]); device_resident_cases(argv[1]); }
    std::printf("%d cases, %d failed\n", g_run, g_failed);
    return g_failed ? 1 : 0;
}
