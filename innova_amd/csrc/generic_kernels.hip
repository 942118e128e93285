// generic_kernels.hip -- the all-format kernels: bit-exact tensor dequantize and a
// GEMV/GEMM that decodes every weight through decode_weight().  They cover every
// wire format, mixed-format rows and ragged tail blocks; the specialised kernels
// (gemv_oil4.hip, ...) take over for the shapes that matter for throughput.
#include <algorithm>

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

// Full OIL2 / OIL4 / OIL8 blocks of one format, laid out back to back at a regular stride (`blocks` null) or wherever
// their descriptors say (tensors stored as window streams): a wavefront per block, lane l decodes
// weights 4l .. 4l+3 from two dwords and stores one float4, so a block is one coalesced 1 KB store.  Values are
// formed exactly as decode_weight forms them: level (literal table / host-built table) times the FP16 scale widened
// by the integer rule; slot weights are 0.
template <int BITS>
__global__ void __launch_bounds__(256)
dequant_lattice_kernel(const uint8_t* __restrict__ base, uint32_t stride, const DevBlock* __restrict__ blocks,
                       const DecodeTables* __restrict__ T, float* __restrict__ out, uint32_t nblocks) {
    __shared__ float lv[256];
    if (BITS == 8) lv[threadIdx.x] = T->lv8[threadIdx.x];
    else if (BITS == 4 && threadIdx.x < 16) lv[threadIdx.x] = kLv4[threadIdx.x];
    else if (BITS == 2 && threadIdx.x < 4) lv[threadIdx.x] = kLv2[threadIdx.x];
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    for (uint32_t b = blockIdx.x * 4u + wave; b < nblocks; b += gridDim.x * 4u) {
        const uint32_t* q = reinterpret_cast<const uint32_t*>(base + (blocks ? (size_t)blocks[b].off16 * 16u : (size_t)b * stride));
        const float scale = half_bits_to_float(q[0] & 0xFFFFu);
        // first code bit of weight 4l: 16 + BITS * (4l - slots before it); one slot per 16*BITS weights
        const uint32_t i0 = 4u * lane;
        const uint32_t bit = 16u + BITS * (i0 - i0 / (16u * BITS));
        const uint32_t lo = q[bit >> 5], hi = q[(bit >> 5) + 1u];            // hi may be the first dword after the block: unused bits
        const uint32_t v = __builtin_amdgcn_alignbit(hi, lo, bit & 31u);
        const bool last_is_slot = ((i0 + 4u) % (16u * BITS)) == 0u;
        float4 o;
        if (BITS == 2) {
            o.x = lv[v & 3u] * scale; o.y = lv[(v >> 2) & 3u] * scale; o.z = lv[(v >> 4) & 3u] * scale;
            o.w = last_is_slot ? 0.0f : lv[(v >> 6) & 3u] * scale;
        } else if (BITS == 4) {
            o.x = lv[v & 15u] * scale; o.y = lv[(v >> 4) & 15u] * scale; o.z = lv[(v >> 8) & 15u] * scale;
            o.w = last_is_slot ? 0.0f : lv[(v >> 12) & 15u] * scale;
        } else {
            o.x = lv[v & 255u] * scale; o.y = lv[(v >> 8) & 255u] * scale; o.z = lv[(v >> 16) & 255u] * scale;
            o.w = last_is_slot ? 0.0f : lv[v >> 24] * scale;
        }
        reinterpret_cast<float4*>(out + (size_t)b * 256u)[lane] = o;
    }
}

// Full OIL1 (FMT 0: eight FP16 run means, 16 bytes) and SPARK_Q0 (FMT 1: per run of 32 an FP16 scale and 32 sign
// bits, 48 bytes) blocks, back to back or by descriptor as above; lane l stores weights 4l .. 4l+3 of its wavefront's block.
template <int FMT>
__global__ void __launch_bounds__(256)
dequant_runs_kernel(const uint8_t* __restrict__ base, uint32_t stride, const DevBlock* __restrict__ blocks,
                    float* __restrict__ out, uint32_t nblocks) {
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t run = lane >> 3, j0 = 4u * (lane & 7u);
    for (uint32_t b = blockIdx.x * 4u + wave; b < nblocks; b += gridDim.x * 4u) {
        const uint16_t* h = reinterpret_cast<const uint16_t*>(base + (blocks ? (size_t)blocks[b].off16 * 16u : (size_t)b * stride));
        float4 o;
        if (FMT == 0) {
            const float m = half_bits_to_float(h[run]);
            o = make_float4(m, m, m, m);
        } else {
            const float sc = half_bits_to_float(h[3u * run]);
            const uint32_t bits = ((uint32_t)h[3u * run + 1u] | ((uint32_t)h[3u * run + 2u] << 16)) >> j0;
            o = make_float4((bits & 1u) ? sc : -sc, (bits & 2u) ? sc : -sc, (bits & 4u) ? sc : -sc, (bits & 8u) ? sc : -sc);
        }
        reinterpret_cast<float4*>(out + (size_t)b * 256u)[lane] = o;
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
    // one format, full blocks: regular stride, or (window streams) the place of every block from its descriptor
    const bool by_stride = w.uniform_stride > 0 && (w.uniform_base & 3u) == 0 && (w.uniform_stride & 3u) == 0;
    const bool by_desc = w.seg.nstreams > 0 && w.seg.nf == 1;
    if (w.all_full && w.uniform_fmt >= 0 && !w.d_out_off && (by_stride || by_desc)) {
        const uint32_t g = std::min<uint32_t>((w.nblocks + 3u) / 4u, (uint32_t)device_cu_count() * 16u);
        const uint8_t* base = w.d_payload + (by_stride ? w.uniform_base : 0u);
        const DevBlock* bl = by_stride ? nullptr : w.d_blocks;
        const int f = w.uniform_fmt;
        const uint32_t st = by_stride ? w.uniform_stride : w.seg.stride[0];
        const uint32_t cb = by_stride ? w.uniform_cb : w.seg.cb_bytes[0];
        bool done = true;
        if (f == OILHIP_OIL4 && st == 128 && cb == 0)
            hipLaunchKernelGGL(dequant_lattice_kernel<4>, dim3(g), dim3(256), 0, s, base, st, bl, T, d_out, w.nblocks);
        else if (f == OILHIP_OIL8 && st == 256 && cb == 0)
            hipLaunchKernelGGL(dequant_lattice_kernel<8>, dim3(g), dim3(256), 0, s, base, st, bl, T, d_out, w.nblocks);
        else if (f == OILHIP_OIL2 && st == 64 && cb == 0)
            hipLaunchKernelGGL(dequant_lattice_kernel<2>, dim3(g), dim3(256), 0, s, base, st, bl, T, d_out, w.nblocks);
        else if (f == OILHIP_OIL1 && st == 16 && cb == 16)
            hipLaunchKernelGGL(dequant_runs_kernel<0>, dim3(g), dim3(256), 0, s, base, st, bl, d_out, w.nblocks);
        else if (f == OILHIP_SPARK_Q0 && st == 48 && cb == 0)
            hipLaunchKernelGGL(dequant_runs_kernel<1>, dim3(g), dim3(256), 0, s, base, st, bl, d_out, w.nblocks);
        else
            done = false;
        if (done) {
            OILHIP_HIP(hipGetLastError());
            return OILHIP_OK;
        }
    }
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
