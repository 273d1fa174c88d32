// Test infrastructure: the reference's ComputeBackend interface (include/quant/backend.h:77-108) subclassed for
// BackendType::GPU_HIP over this library's tfq::HipBackend operators, compiled against the reference's own headers
// and Tensor where the reference tree is present (oracle/Makefile, target ref_backend), with C entry points that
// build reference Tensors around caller buffers and call the subclass through a ComputeBackend pointer.  The class
// is the glue a maintainer adds next to the reference's other backends; the tests drive it on a GPU and compare
// with numpy.  Nothing here is linked into the shipped library.
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>

#include "quant/backend.h"
#include "../include/tfq.h"
#include "../include/tfq_shims.hpp"

namespace {

using quant::Shape;
using quant::Tensor;
using quant::backend::BackendType;
using quant::backend::ComputeBackend;

class Gfx950Backend : public ComputeBackend {
public:
    BackendType type() const override { return BackendType::GPU_HIP; }
    const char* name() const override { return tfq::HipBackend::name(); }
    void gemm(float alpha, const Tensor& A, const Tensor& B, float beta, Tensor& C) override {
        check(tfq::HipBackend::gemm(alpha, A.data<float>(), B.data<float>(), beta, C.data<float>(), A.dim(0), B.dim(1), A.dim(1)));
    }
    void gemv(float alpha, const Tensor& A, const Tensor& x, float beta, Tensor& y) override {
        check(tfq::HipBackend::gemv(alpha, A.data<float>(), x.data<float>(), beta, y.data<float>(), A.dim(0), A.dim(1)));
    }
    void softmax(const Tensor& x, Tensor& y, int axis) override {
        if (axis < 0) axis += x.rank();
        int64_t outer = 1, inner = 1;
        for (int i = 0; i < axis; ++i) outer *= x.dim(i);
        for (int i = axis + 1; i < x.rank(); ++i) inner *= x.dim(i);
        check(tfq::HipBackend::softmax(x.data<float>(), y.data<float>(), outer, x.dim(axis), inner));
    }
    void layer_norm(const Tensor& x, const Tensor& gamma, const Tensor& beta, float eps, Tensor& y) override {
        const int64_t n = x.dim(x.rank() - 1);
        check(tfq::HipBackend::layer_norm(x.data<float>(), gamma.data<float>(), beta.data<float>(), eps, y.data<float>(), x.numel() / n, n));
    }
    void rms_norm(const Tensor& x, const Tensor& gamma, float eps, Tensor& y) override {
        const int64_t n = x.dim(x.rank() - 1);
        check(tfq::HipBackend::rms_norm(x.data<float>(), gamma.data<float>(), eps, y.data<float>(), x.numel() / n, n));
    }
    void relu(const Tensor& x, Tensor& y) override { check(tfq::HipBackend::relu(x.data<float>(), y.data<float>(), x.numel())); }
    void gelu(const Tensor& x, Tensor& y) override { check(tfq::HipBackend::gelu(x.data<float>(), y.data<float>(), x.numel())); }
    void silu(const Tensor& x, Tensor& y) override { check(tfq::HipBackend::silu(x.data<float>(), y.data<float>(), x.numel())); }
    void add(const Tensor& a, const Tensor& b, Tensor& c) override {
        check(tfq::HipBackend::add(a.data<float>(), b.data<float>(), c.data<float>(), a.numel()));
    }
    void mul(const Tensor& a, const Tensor& b, Tensor& c) override {
        check(tfq::HipBackend::mul(a.data<float>(), b.data<float>(), c.data<float>(), a.numel()));
    }
    void scale(float s, const Tensor& x, Tensor& y) override { check(tfq::HipBackend::scale(s, x.data<float>(), y.data<float>(), x.numel())); }
    void copy(const Tensor& src, Tensor& dst) override { std::memcpy(dst.data(), src.data(), src.size_bytes()); }
    void fill(Tensor& t, float val) override { t.fill(val); }
    void zero(Tensor& t) override { t.zero_(); }
    bool is_available() const override { return tfq::HipBackend::is_available(); }
    int64_t memory_free() const override { return tfq::HipBackend::memory_free(); }
    int64_t memory_total() const override { return tfq::HipBackend::memory_total(); }
    void synchronize() override { tfq::HipBackend::synchronize(); }

private:
    static void check(bool ok) {
        if (!ok) throw std::runtime_error(std::string("[REAL-ONLY] ") + tfq_last_error());
    }
};

ComputeBackend* backend() {
    static Gfx950Backend b;
    return &b;  // every call below goes through the base-class pointer, as the reference's callers do
}

Tensor from(const float* p, Shape s) {
    Tensor t(s);
    std::memcpy(t.data(), p, t.size_bytes());
    return t;
}

// runs f, copies `out` back; 1 on success, 0 when the backend threw
template <class F>
int run(Tensor& out, float* dst, F f) {
    try {
        f();
    } catch (const std::exception&) {
        return 0;
    }
    std::memcpy(dst, out.data(), out.size_bytes());
    return 1;
}

}  // namespace

extern "C" {

const char* refglue_name() { return backend()->name(); }
int refglue_is_gpu_hip() { return backend()->type() == BackendType::GPU_HIP; }
int refglue_available() { return backend()->is_available(); }
long long refglue_memory_total() { return backend()->memory_total(); }

int refglue_gemm(float alpha, const float* A, const float* B, float beta, float* C, long long M, long long N, long long K) {
    Tensor a = from(A, Shape(M, K)), b = from(B, Shape(K, N)), c = from(C, Shape(M, N));
    return run(c, C, [&] { backend()->gemm(alpha, a, b, beta, c); });
}
int refglue_gemv(float alpha, const float* A, const float* x, float beta, float* y, long long M, long long N) {
    Tensor a = from(A, Shape(M, N)), xv = from(x, Shape(N)), yv = from(y, Shape(M));
    return run(yv, y, [&] { backend()->gemv(alpha, a, xv, beta, yv); });
}
int refglue_softmax(const float* x, float* y, long long d0, long long d1, long long d2, int axis) {
    Tensor xv = from(x, Shape(d0, d1, d2)), yv{Shape(d0, d1, d2)};
    return run(yv, y, [&] { backend()->softmax(xv, yv, axis); });
}
int refglue_layer_norm(const float* x, const float* gamma, const float* beta, float eps, float* y, long long rows, long long n) {
    Tensor xv = from(x, Shape(rows, n)), g = from(gamma, Shape(n)), b = from(beta, Shape(n)), yv{Shape(rows, n)};
    return run(yv, y, [&] { backend()->layer_norm(xv, g, b, eps, yv); });
}
int refglue_rms_norm(const float* x, const float* gamma, float eps, float* y, long long rows, long long n) {
    Tensor xv = from(x, Shape(rows, n)), g = from(gamma, Shape(n)), yv{Shape(rows, n)};
    return run(yv, y, [&] { backend()->rms_norm(xv, g, eps, yv); });
}
// op: 0 relu, 1 gelu, 2 silu, 3 scale by s
int refglue_unary(int op, float s, const float* x, float* y, long long n) {
    Tensor xv = from(x, Shape(n)), yv{Shape(n)};
    return run(yv, y, [&] {
        if (op == 0) backend()->relu(xv, yv);
        else if (op == 1) backend()->gelu(xv, yv);
        else if (op == 2) backend()->silu(xv, yv);
        else backend()->scale(s, xv, yv);
    });
}
// op: 0 add, 1 mul
int refglue_binary(int op, const float* a, const float* b, float* c, long long n) {
    Tensor av = from(a, Shape(n)), bv = from(b, Shape(n)), cv{Shape(n)};
    return run(cv, c, [&] {
        if (op == 0) backend()->add(av, bv, cv);
        else backend()->mul(av, bv, cv);
    });
}

}  // extern "C"
