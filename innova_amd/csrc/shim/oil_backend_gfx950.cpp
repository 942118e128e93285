// oil_backend_gfx950.cpp -- the gfx950 device behind the reference's backend dispatch: a backend::ComputeBackend
// (include/oil/backend.h:49-80) whose operations run as HIP kernels of liboilhip, the two free functions the
// patched factory and hardware probe call (include/oil_backend_gfx950.patch: BackendType::GPU_HIP_GFX950, the case in
// ComputeBackend::create, src/backend.cpp:446-463, the flag in probe_hardware, :672-730, and the rule in
// select_optimal_backend, :732-786).
//
// Built only inside the reference tree, with that patch applied and OIL_USE_HIP_GFX950 defined, and linked with
// liboilhip.so.  Operands are host tensors, as for every backend of the reference: each call uploads, runs on the
// device and downloads, like GPUDirectXBackend::gemm (src/backend.cpp:286-318).  There is no CPU fallback: a failed
// device call throws oil::Error.
#include "oil/backend.h"

#include <hip/hip_runtime.h>

#include <string>

#include "oilhip.h"

namespace oil {
namespace backend {
namespace {

void ok(int rc, const char* what) {
    if (rc != OILHIP_OK) throw Error(std::string(what) + ": " + oilhip_last_error());
}
void hip_ok(hipError_t e, const char* what) {
    if (e != hipSuccess) throw Error(std::string(what) + ": " + hipGetErrorString(e));
}

// Device copy of a host tensor's floats (or room for a result).
class Dev {
public:
    Dev(const Tensor& t, bool upload) : n_((size_t)t.numel()) {
        if (n_ == 0) return;
        hip_ok(hipMalloc(&p_, n_ * sizeof(float)), "hipMalloc");
        if (upload) hip_ok(hipMemcpy(p_, t.data<float>(), n_ * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy H2D");
    }
    ~Dev() { if (p_) (void)hipFree(p_); }
    Dev(const Dev&) = delete;
    Dev& operator=(const Dev&) = delete;
    float* get() const { return p_; }
    void to(Tensor& t) const {
        if (n_) hip_ok(hipMemcpy(t.data<float>(), p_, n_ * sizeof(float), hipMemcpyDeviceToHost), "hipMemcpy D2H");
    }
private:
    float* p_ = nullptr;
    size_t n_;
};

class Gfx950Backend final : public ComputeBackend {
public:
    BackendType type() const override { return BackendType::GPU_HIP_GFX950; }
    const char* name() const override { return "hip-gfx950"; }

    // shape rules of math::gemm (src/math.cpp:72-80)
    void gemm(float alpha, const Tensor& A, const Tensor& B, float beta, Tensor& C) override {
        OIL_CHECK(A.rank() == 2 && B.rank() == 2 && C.rank() == 2, "gemm operands must be 2D");
        const int64_t M = A.dim(0), K = A.dim(1), N = B.dim(1);
        OIL_CHECK(B.dim(0) == K, "gemm A cols != B rows");
        OIL_CHECK(C.dim(0) == M && C.dim(1) == N, "gemm C shape mismatch");
        Dev a(A, true), b(B, true), c(C, beta != 0.0f);
        ok(oilhip_dense_gemm_f32(alpha, a.get(), b.get(), beta, c.get(), M, N, K, nullptr), "gemm");
        c.to(C);
    }
    // src/math.cpp:50-57
    void gemv(float alpha, const Tensor& A, const Tensor& x, float beta, Tensor& y) override {
        OIL_CHECK(A.rank() == 2 && x.rank() == 1 && y.rank() == 1, "gemv expects a 2D matrix and 1D vectors");
        const int64_t M = A.dim(0), N = A.dim(1);
        OIL_CHECK(x.numel() == N, "gemv x size != A cols");
        OIL_CHECK(y.numel() == M, "gemv y size != A rows");
        Dev a(A, true), dx(x, true), dy(y, beta != 0.0f);
        ok(oilhip_dense_gemv_f32(alpha, a.get(), dx.get(), beta, dy.get(), M, N, nullptr), "gemv");
        dy.to(y);
    }
    // src/math.cpp:205-221
    void softmax(const Tensor& x, Tensor& y, int axis) override {
        OIL_CHECK(x.numel() == y.numel(), "softmax shape mismatch");
        const int rank = x.rank();
        if (axis < 0) axis += rank;
        OIL_CHECK(axis >= 0 && axis < rank, "softmax axis out of range");
        int64_t outer = 1, inner = 1;
        for (int i = 0; i < axis; ++i) outer *= x.dim(i);
        for (int i = axis + 1; i < rank; ++i) inner *= x.dim(i);
        Dev dx(x, true), dy(y, false);
        ok(oilhip_dense_softmax_f32(dx.get(), dy.get(), outer, x.dim(axis), inner, nullptr), "softmax");
        dy.to(y);
    }
    // src/math.cpp:146-153
    void layer_norm(const Tensor& x, const Tensor& gamma, const Tensor& beta, float eps, Tensor& y) override {
        OIL_CHECK(x.numel() == y.numel(), "layer_norm shape mismatch");
        OIL_CHECK(x.rank() >= 1, "layer_norm needs at least one dimension");
        const int64_t n = x.dim(x.rank() - 1);
        OIL_CHECK(gamma.numel() == n, "layer_norm gamma dim mismatch");
        OIL_CHECK(beta.numel() == n, "layer_norm beta dim mismatch");
        Dev dx(x, true), g(gamma, true), b(beta, true), dy(y, false);
        ok(oilhip_dense_norm_f32(0, dx.get(), g.get(), b.get(), eps, dy.get(), n ? x.numel() / n : 0, n, nullptr), "layer_norm");
        dy.to(y);
    }
    // src/math.cpp:180-185
    void rms_norm(const Tensor& x, const Tensor& gamma, float eps, Tensor& y) override {
        OIL_CHECK(x.numel() == y.numel(), "rms_norm shape mismatch");
        OIL_CHECK(x.rank() >= 1, "rms_norm needs at least one dimension");
        const int64_t n = x.dim(x.rank() - 1);
        OIL_CHECK(gamma.numel() == n, "rms_norm gamma dim mismatch");
        Dev dx(x, true), g(gamma, true), dy(y, false);
        ok(oilhip_dense_norm_f32(1, dx.get(), g.get(), nullptr, eps, dy.get(), n ? x.numel() / n : 0, n, nullptr), "rms_norm");
        dy.to(y);
    }

    void relu(const Tensor& x, Tensor& y) override { unary(0, 0.0f, x, y, "relu shape mismatch"); }
    void gelu(const Tensor& x, Tensor& y) override { unary(1, 0.0f, x, y, "gelu shape mismatch"); }
    void silu(const Tensor& x, Tensor& y) override { unary(2, 0.0f, x, y, "silu shape mismatch"); }
    void add(const Tensor& a, const Tensor& b, Tensor& c) override { binary(3, a, b, c, "add shape mismatch"); }
    void mul(const Tensor& a, const Tensor& b, Tensor& c) override { binary(4, a, b, c, "mul shape mismatch"); }
    void scale(float s, const Tensor& x, Tensor& y) override { unary(5, s, x, y, "scale shape mismatch"); }

    // host tensors: these move or set host memory, as in every backend of the reference (src/backend.cpp:64-66)
    void copy(const Tensor& src, Tensor& dst) override { dst.copy_from(src); }
    void fill(Tensor& t, float val) override { t.fill(val); }
    void zero(Tensor& t) override { t.zero_(); }

    bool is_available() const override { return is_hip_gfx950_available(); }
    int64_t memory_free() const override {
        size_t f = 0, t = 0;
        return hipMemGetInfo(&f, &t) == hipSuccess ? (int64_t)f : 0;
    }
    int64_t memory_total() const override {
        size_t f = 0, t = 0;
        return hipMemGetInfo(&f, &t) == hipSuccess ? (int64_t)t : 0;
    }
    void synchronize() override { hip_ok(hipDeviceSynchronize(), "hipDeviceSynchronize"); }

private:
    void unary(int op, float s, const Tensor& x, Tensor& y, const char* mismatch) {
        OIL_CHECK(x.numel() == y.numel(), mismatch);
        Dev dx(x, true), dy(y, false);
        ok(oilhip_dense_map_f32(op, dx.get(), nullptr, s, dy.get(), x.numel(), nullptr), "elementwise");
        dy.to(y);
    }
    void binary(int op, const Tensor& a, const Tensor& b, Tensor& c, const char* mismatch) {
        OIL_CHECK(a.numel() == b.numel() && b.numel() == c.numel(), mismatch);
        Dev da(a, true), db(b, true), dc(c, false);
        ok(oilhip_dense_map_f32(op, da.get(), db.get(), 0.0f, dc.get(), a.numel(), nullptr), "elementwise");
        dc.to(c);
    }
};

}  // namespace

bool is_hip_gfx950_available() {
    int gfx = 0;
    return oilhip_probe(&gfx, nullptr, nullptr, nullptr, 0) == OILHIP_OK && gfx == 950;
}

ComputeBackend* create_gfx950_backend(const BackendConfig& cfg) {
    if (!is_hip_gfx950_available()) return nullptr;
    if (cfg.device_id != 0) {
        int count = 0;
        if (hipGetDeviceCount(&count) != hipSuccess || cfg.device_id < 0 || cfg.device_id >= count) return nullptr;
        if (hipSetDevice((int)cfg.device_id) != hipSuccess) return nullptr;
    }
    return new Gfx950Backend();
}

}  // namespace backend
}  // namespace oil
