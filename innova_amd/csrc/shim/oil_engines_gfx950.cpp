// oil_engines_gfx950.cpp -- the engine classes' matmul and dequantize members (include/oil/oil_engines.h) and the
// SPARK lookup kernels (include/oil/kernel.h:11-18) with their bodies on the gfx950 device.
//
// Built only inside the reference tree, in place of the same definitions in src/oil_engines_{oil8,oil4,oil2,oil1,
// spark,fp}.cpp and src/kernel_tl.cpp (which a build with OIL_USE_HIP_GFX950 leaves out), and linked with
// liboilhip_shims.so.  Signatures are the reference's own: this file includes its headers and defines its members.
// Results are the CPU bodies' bit for bit (same contraction order, fused multiply-adds as the reference's -mfma build).
#include "oil/kernel.h"
#include "oil/oil_engines.h"

#include "oilhip_shims.hpp"

namespace oil {
namespace engines {

// include/oil/oil_engines.h:48-49,43-44; CPU bodies src/oil_engines_oil8.cpp:171-183,197-216,121-134
Tensor OIL8Engine::dequant_tensor(const uint8_t* indices, int64_t n) const {
    Tensor out({n});
    gfx950::engine_dequant(8, indices, codebook_.data(), n, nullptr, 0, out.data<float>());
    return out;
}
Tensor OIL8Engine::quant_gemm(const Tensor& a, const uint8_t* b_idx, int64_t M, int64_t N, int64_t K) const {
    Tensor C({M, N});
    C.zero_();
    gfx950::engine_quant_gemm(8, a.data<float>(), b_idx, codebook_.data(), C.data<float>(), M, N, K);
    return C;
}
void OIL8Engine::dequantize_per_block(const uint8_t* indices, const float* scales, int64_t n, int64_t block_size,
                                      float* out) const {
    gfx950::engine_dequant(8, indices, codebook_.data(), n, scales, block_size, out);
}

// include/oil/oil_engines.h:77-78,72-73; CPU bodies src/oil_engines_oil4.cpp:205-220,238-261,136-150
Tensor OIL4Engine::dequant_tensor(const uint8_t* indices, int64_t n) const {
    Tensor out({n});
    gfx950::engine_dequant(4, indices, codebook_.data(), n, nullptr, 0, out.data<float>());
    return out;
}
Tensor OIL4Engine::quant_gemm(const Tensor& a, const uint8_t* b_idx, int64_t M, int64_t N, int64_t K) const {
    Tensor C({M, N});
    C.zero_();
    gfx950::engine_quant_gemm(4, a.data<float>(), b_idx, codebook_.data(), C.data<float>(), M, N, K);
    return C;
}
void OIL4Engine::dequantize_per_block(const uint8_t* indices, const float* scales, int64_t n, int64_t block_size,
                                      float* out) const {
    gfx950::engine_dequant(4, indices, codebook_.data(), n, scales, block_size, out);
}

// include/oil/oil_engines.h:150-151; CPU bodies src/oil_engines_oil2.cpp:184-193,210-229
Tensor OIL2Engine::dequant_tensor(const uint8_t* indices, int64_t n) const {
    Tensor out({n});
    gfx950::engine_dequant(2, indices, codebook_.data(), n, nullptr, 0, out.data<float>());
    return out;
}
Tensor OIL2Engine::quant_gemm(const Tensor& a, const uint8_t* b_idx, int64_t M, int64_t N, int64_t K) const {
    Tensor C({M, N});
    C.zero_();
    gfx950::engine_quant_gemm(2, a.data<float>(), b_idx, codebook_.data(), C.data<float>(), M, N, K);
    return C;
}

// include/oil/oil_engines.h:123; CPU body src/oil_engines_oil1.cpp:61-82 (the scale argument is unused there too)
Tensor Oil1Engine::quant_gemm(const Tensor& a, const Tensor& b_packed, float, int64_t M, int64_t N, int64_t K) {
    Tensor C({M, N});
    C.zero_();
    gfx950::engine_dense_gemm(1, a.data<float>(), b_packed.data<float>(), nullptr, 32, C.data<float>(), M, N, K);
    return C;
}
// include/oil/oil_engines.h:103; CPU body src/oil_engines_spark.cpp:154-186
Tensor SparkEngine::quant_gemm(const Tensor& a, const Tensor& b_packed, const Tensor& b_scales, int64_t M, int64_t N,
                               int64_t K) {
    Tensor C({M, N});
    C.zero_();
    gfx950::engine_dense_gemm(3, a.data<float>(), b_packed.data(), b_scales.data<float>(), block_size_, C.data<float>(), M, N, K);
    return C;
}
// include/oil/oil_engines.h:167,183; CPU bodies src/oil_engines_fp.cpp:433-451,531-547
Tensor OIL16Engine::quant_gemm(const Tensor& a, const Tensor& b_packed, int64_t M, int64_t N, int64_t K) const {
    Tensor C({M, N});
    C.zero_();
    gfx950::engine_dense_gemm(16, a.data<float>(), b_packed.data(), nullptr, 0, C.data<float>(), M, N, K);
    return C;
}
Tensor OIL32Engine::quant_gemm(const Tensor& a, const Tensor& b_packed, int64_t M, int64_t N, int64_t K) const {
    Tensor C({M, N});
    C.zero_();
    gfx950::engine_dense_gemm(32, a.data<float>(), b_packed.data(), nullptr, 0, C.data<float>(), M, N, K);
    return C;
}

}  // namespace engines

namespace kernel {

// include/oil/kernel.h:11-12,17-18; CPU bodies src/kernel_tl.cpp:32-90,124-184
void tl1_gemm(const Tensor& weights, const Tensor& activations, Tensor& output, int M, int N, int K) {
    gfx950::tl_gemm(1, weights.data<uint8_t>(), activations.data<float>(), output.data<float>(), M, N, K);
}
void tl2_gemm(const Tensor& weights, const Tensor& activations, Tensor& output, int M, int N, int K) {
    gfx950::tl_gemm(2, weights.data<uint8_t>(), activations.data<float>(), output.data<float>(), M, N, K);
}

}  // namespace kernel
}  // namespace oil
