// generic_kernels.hip -- the all-format kernels: bit-exact tensor dequantize and a
// GEMV/GEMM that decodes every weight through decode_weight().  They cover every
// wire format, mixed-format rows and ragged tail blocks; the specialised kernels
// (gemv_oil4.hip, ...) take over for the shapes that matter for throughput.
#include "common.h"

namespace oilhip {
namespace {

// One workgroup per block, one thread per weight (strided for blocks > 256).
// Mirrors OILReader::read_tensor's loop over dequantize_block_all
// (src/oil_format.cpp:464-477).
__global__ void __launch_bounds__(256)
dequant_kernel(const uint8_t* __restrict__ payload, const DevBlock* __restrict__ blocks,
               const uint64_t* __restrict__ out_off, const DecodeTables* __restrict__ T,
               float* __restrict__ out, uint32_t nblocks, uint32_t uniform_nw) {
    for (uint32_t b = blockIdx.x; b < nblocks; b += gridDim.x) {
        const DevBlock d = blocks[b];
        const uint8_t* cb = payload + (size_t)d.off16 * 16;
        const uint8_t* idx = cb + d.cb_bytes;
        float* o = out + (out_off ? out_off[b] : (uint64_t)b * uniform_nw);
        for (uint32_t i = threadIdx.x; i < d.nw; i += 256)
            o[i] = decode_weight(d.fmt, cb, d.cb_bytes, idx, d.idx_bytes, d.nw, i, T);
    }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Y[m][row] = sum_k W[row][k] * X[m][k] for MB batch rows at a time; one
// workgroup per output row, thread t owns weight t of every block in the row
// (Qwen35Engine::gemm, src/adapters/tools/qwen35_engine.cpp:66-81).
template <int MB>
__global__ void __launch_bounds__(256)
gemv_generic_kernel(const uint8_t* __restrict__ payload, const DevBlock* __restrict__ blocks,
                    const DecodeTables* __restrict__ T, const float* __restrict__ x,
                    float* __restrict__ y, uint32_t rows, uint32_t cols, int M, int m0) {
    __shared__ float part[MB][4];
    const uint32_t row = blockIdx.x, t = threadIdx.x, bpr = cols >> 8;
    float acc[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) acc[b] = 0.0f;
    for (uint32_t k = 0; k < bpr; ++k) {
        const DevBlock d = blocks[(size_t)row * bpr + k];
        const uint8_t* cb = payload + (size_t)d.off16 * 16;
        const float v = decode_weight(d.fmt, cb, d.cb_bytes, cb + d.cb_bytes, d.idx_bytes, 256, t, T);
#pragma unroll
        for (int b = 0; b < MB; ++b)
            if (m0 + b < M) acc[b] = __fmaf_rn(v, x[(size_t)(m0 + b) * cols + (size_t)k * 256 + t], acc[b]);
    }
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const float s = wave_sum(acc[b]);
        if ((t & 63) == 0) part[b][t >> 6] = s;
    }
    __syncthreads();
    if (t < MB && m0 + (int)t < M)
        y[(size_t)(m0 + t) * rows + row] = (part[t][0] + part[t][1]) + (part[t][2] + part[t][3]);
}

// Mean squared error of one decoded block against the original weights it encodes:
// FormatRegistry::measure_mse (src/format_registry.cpp:281-289) over dequantize_block_all,
// one thread per block, double accumulation in index order with the fused multiply-add the
// reference build uses, rounded to float at the end.
__global__ void __launch_bounds__(64)
block_mse_kernel(const uint8_t* __restrict__ payload, const DevBlock* __restrict__ blocks,
                 const DecodeTables* __restrict__ T, const float* __restrict__ orig,
                 const uint64_t* __restrict__ start, float* __restrict__ out, uint32_t nblocks) {
    const uint32_t b = blockIdx.x * 64 + threadIdx.x;
    if (b >= nblocks) return;
    const DevBlock d = blocks[b];
    const uint8_t* cb = payload + (size_t)d.off16 * 16;
    const float* o = orig + start[b];
    double s = 0.0;
    for (uint32_t i = 0; i < d.nw; ++i) {
        const double diff = (double)o[i] - (double)decode_weight(d.fmt, cb, d.cb_bytes, cb + d.cb_bytes, d.idx_bytes, d.nw, i, T);
        s = fma(diff, diff, s);
    }
    out[b] = (float)(s / (double)d.nw);
}

}  // namespace

int launch_block_mse(const oilhip_weights& w, const float* d_orig, const uint64_t* d_start, float* d_out, hipStream_t s) {
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    if (w.nblocks == 0) return OILHIP_OK;
    hipLaunchKernelGGL(block_mse_kernel, dim3((w.nblocks + 63) / 64), dim3(64), 0, s, w.d_payload, w.d_blocks, T,
                       d_orig, d_start, d_out, w.nblocks);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int launch_dequant(const oilhip_weights& w, float* d_out, hipStream_t s) {
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    if (w.nblocks == 0) return OILHIP_OK;
    const uint32_t grid = w.nblocks < (1u << 20) ? w.nblocks : (1u << 20);
    hipLaunchKernelGGL(dequant_kernel, dim3(grid), dim3(256), 0, s, w.d_payload, w.d_blocks,
                       w.d_out_off, T, d_out, w.nblocks, 256u);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int launch_gemv_generic(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s) {
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    constexpr int MB = 4;
    for (int m0 = 0; m0 < M; m0 += MB) {
        hipLaunchKernelGGL(gemv_generic_kernel<MB>, dim3((uint32_t)w.rows), dim3(256), 0, s,
                           w.d_payload, w.d_blocks, T, d_x, d_y, (uint32_t)w.rows, (uint32_t)w.cols, M, m0);
        OILHIP_HIP(hipGetLastError());
    }
    return OILHIP_OK;
}

}  // namespace oilhip
