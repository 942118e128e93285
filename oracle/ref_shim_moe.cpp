// ref_shim_moe.cpp -- C entry points over the reference's mixture-of-experts routing and batched
// dispatch (src/moe_variants.cpp:97-134,767-827), compiled from the reference's own sources.
// Only the functions reachable from these entry points are kept (function sections + section
// garbage collection + the export list in ref_exports.map), so the rest of those translation
// units needs nothing else from the reference build.  TEST INFRASTRUCTURE ONLY.
#include "oil/moe_variants.h"

#include <cstdint>
#include <cstring>
#include <vector>

extern "C" {

void ref_softmax_topk(const float* logits, int64_t T, int64_t E, int64_t k, float* probs, int64_t* idx, float* w) {
    oil::Tensor l({T, E});
    std::memcpy(l.data<float>(), logits, (size_t)(T * E) * 4);
    oil::Tensor io, wo;
    oil::Tensor p = oil::moe::softmax_with_topk(l, k, io, wo);
    std::memcpy(probs, p.data<float>(), (size_t)(T * E) * 4);
    std::memcpy(idx, io.data<int64_t>(), (size_t)(T * k) * 8);
    std::memcpy(w, wo.data<float>(), (size_t)(T * k) * 4);
}

// Experts as row-major matrices gate/up [F][D], down [D][F] with Y = X W^T.  Linear::forward hands its
// weight buffer to kernel::scalar_gemm as B[K][N] (src/transformer.cpp:61-69, src/kernel_gemm.cpp:13-23),
// so each buffer receives the transposed matrix; biases stay zero.
void ref_moe_dispatch(const float* x, const float* const* gate, const float* const* up, const float* const* down,
                      const int64_t* indices, const float* weights, int64_t T, int64_t K, int64_t E, int64_t D,
                      int64_t F, float* out, float* z_loss, int64_t* dropped) {
    auto fill = [](oil::Linear& lin, const float* W, int64_t N, int64_t Kd) {      // W [N][Kd]
        float* b = lin.weight.data<float>();
        for (int64_t n = 0; n < N; ++n)
            for (int64_t k = 0; k < Kd; ++k) b[k * N + n] = W[n * Kd + k];
        std::memset(lin.bias.data<float>(), 0, (size_t)N * 4);
    };
    std::vector<oil::moe::ExpertFFN> experts;
    for (int64_t e = 0; e < E; ++e) {
        experts.emplace_back(D, F, oil::Activation::SiLU);
        fill(experts.back().gate_proj, gate[e], F, D);
        fill(experts.back().up_proj, up[e], F, D);
        fill(experts.back().down_proj, down[e], D, F);
    }
    oil::Tensor xt({T, D});
    std::memcpy(xt.data<float>(), x, (size_t)(T * D) * 4);
    oil::Tensor o = oil::moe::moe_dispatch_batched(xt, experts, indices, weights, T, K, E, D, z_loss, dropped);
    std::memcpy(out, o.data<float>(), (size_t)(T * D) * 4);
}

}  // extern "C"
