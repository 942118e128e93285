// ref_shim.cpp -- C entry points onto the *compiled reference* (checker only).
//
// This file contains no reference code: it includes the reference's public
// headers from the reference tree and forwards to its functions so that the
// Python tests and the fixture generator can call them through ctypes.  It is
// linked only into oracle/_ref/liboilref*.so, which is built only where the
// reference tree is present, and is never part of the product.
#include "oil/block_codec.h"
#include "oil/kernel.h"
#include "oil/kernel_production.h"
#include "oil/oil_engines.h"
#include "oil/types.h"

#include <cstdint>
#include <cstring>
#include <vector>

namespace oil {
// internal linkage in block_codec.cpp; reached through the public pair below
}

extern "C" {

// include/oil/block_codec.h:55-56
int ref_quantize_block(int fmt, const float* w, int n,
                       uint8_t* idx, size_t idx_cap, size_t* idx_len,
                       uint8_t* cb, size_t cb_cap, size_t* cb_len) {
    std::vector<uint8_t> vi, vc;
    const bool ok = oil::quantize_block_all((oil::Format)fmt, w, n, vi, vc);
    *idx_len = vi.size();
    *cb_len = vc.size();
    if (vi.size() > idx_cap || vc.size() > cb_cap) return -1;
    if (!vi.empty()) std::memcpy(idx, vi.data(), vi.size());
    if (!vc.empty()) std::memcpy(cb, vc.data(), vc.size());
    return ok ? 1 : 0;
}

// include/oil/block_codec.h:60-63
void ref_dequantize_block(int fmt, const uint8_t* idx, size_t idx_bytes,
                          const uint8_t* cb, size_t cb_bytes, uint32_t nw, float* out) {
    oil::dequantize_block_all((oil::Format)fmt, idx, idx_bytes, cb, cb_bytes, nw, out);
}

float ref_format_bpw(int fmt) { return oil::format_bpw((oil::Format)fmt); }

// include/oil/kernel.h:24-32
void ref_oil8_gemm(const uint8_t* idx, const float* cb, const float* act, float* out,
                   int M, int N, int K) {
    oil::kernel::oil8_gemm(idx, cb, act, out, M, N, K);
}
void ref_oil4_gemm(const uint8_t* packed, const uint16_t* cb, const float* act, float* out,
                   int M, int N, int K) {
    oil::kernel::oil4_gemm(packed, cb, act, out, M, N, K);
}

// include/oil/kernel_production.h:25-52
void ref_gemv_spark(const uint8_t* w, float scale, const float* x, float* y, int M, int K) {
    oil::adapters::prod::gemv_spark_tiled(w, scale, x, y, M, K);
}
void ref_gemv_oil4(const uint8_t* w, const uint16_t* cb, float scale, const float* x, float* y,
                   int M, int K) {
    oil::adapters::prod::gemv_oil4_tiled(w, cb, scale, x, y, M, K);
}
void ref_gemv_oil8(const uint8_t* w, const float* cb, float scale, const float* x, float* y,
                   int M, int K) {
    oil::adapters::prod::gemv_oil8_tiled(w, cb, scale, x, y, M, K);
}
void ref_gemv_oil4_batch(const uint8_t* w, const uint16_t* cb, float scale, const float* X,
                         float* Y, int M, int N, int K) {
    oil::adapters::prod::gemv_oil4_batch(w, cb, scale, X, Y, M, N, K);
}

// include/oil/oil_engines.h:34-187: engines with their default codebooks.
// bits selects OIL8Engine / OIL4Engine / OIL2Engine.  cb_out receives the
// engine's codebook (256 / 16 / 4 floats).
int ref_engine_codebook(int bits, float* cb_out) {
    if (bits == 8) { oil::engines::OIL8Engine e; std::memcpy(cb_out, e.codebook().data(), e.codebook().size() * 4); return (int)e.codebook().size(); }
    if (bits == 4) { oil::engines::OIL4Engine e; std::memcpy(cb_out, e.codebook().data(), e.codebook().size() * 4); return (int)e.codebook().size(); }
    if (bits == 2) { oil::engines::OIL2Engine e; std::memcpy(cb_out, e.codebook().data(), e.codebook().size() * 4); return (int)e.codebook().size(); }
    return 0;
}

void ref_engine_quant_gemm(int bits, const float* A, const uint8_t* b_idx, float* C,
                           int64_t M, int64_t N, int64_t K) {
    oil::Tensor a({M, K});
    std::memcpy(a.data<float>(), A, (size_t)(M * K) * 4);
    oil::Tensor c;
    if (bits == 8) { oil::engines::OIL8Engine e; c = e.quant_gemm(a, b_idx, M, N, K); }
    else if (bits == 4) { oil::engines::OIL4Engine e; c = e.quant_gemm(a, b_idx, M, N, K); }
    else { oil::engines::OIL2Engine e; c = e.quant_gemm(a, b_idx, M, N, K); }
    std::memcpy(C, c.data<float>(), (size_t)(M * N) * 4);
}

}  // extern "C"
