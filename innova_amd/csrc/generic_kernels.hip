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

// ---- full 256-weight blocks of nominal size: a wavefront per block, lane l decodes weights 4l .. 4l+3 and stores one
// float4, so a block is one coalesced 1 KB store.  Every value is formed exactly as decode_weight forms it (level
// from the literal / host-built tables times the FP16 scale widened by the integer rule, one fused multiply-add for
// the grouped formats, scale == 0 -> zero point, slots 0).  Blocks sit back to back at a regular stride (`blocks`
// null) or wherever their descriptors say (tensors stored as window streams).
struct FullTables { const float* lv8; const float* t255; const float* q127; const float* lv4; const float* lv2; };   // LDS copies


template <int FMT>
__device__ __forceinline__ float4 decode_full4(const uint8_t* __restrict__ p, uint32_t lane, const FullTables& L) {
    const uint32_t* q = reinterpret_cast<const uint32_t*>(p);
    const uint32_t i0 = 4u * lane;
    if constexpr (FMT == 2 || FMT == 3 || FMT == 4) {                      // OIL2 / OIL4 / OIL8 (src/block_codec.cpp:173-182)
        constexpr uint32_t BITS = FMT == 2 ? 2u : (FMT == 3 ? 4u : 8u);
        const float* lv = FMT == 2 ? L.lv2 : (FMT == 3 ? L.lv4 : L.lv8);
        const float scale = half_bits_to_float(q[0] & 0xFFFFu);
        // first code bit of weight 4l: 16 + BITS * (4l - slots before it); one slot per 16*BITS weights
        const uint32_t bit = 16u + BITS * (i0 - i0 / (16u * BITS));
        const uint32_t lo = q[bit >> 5], hi = q[(bit >> 5) + 1u];            // hi may be the first dword after the block: unused bits
        const uint32_t v = __builtin_amdgcn_alignbit(hi, lo, bit & 31u);
        const bool last_is_slot = ((i0 + 4u) % (16u * BITS)) == 0u;
        constexpr uint32_t mask = (1u << BITS) - 1u;
        return make_float4(lv[v & mask] * scale, lv[(v >> BITS) & mask] * scale, lv[(v >> (2u * BITS)) & mask] * scale,
                           last_is_slot ? 0.0f : lv[(v >> (3u * BITS)) & mask] * scale);
    } else if constexpr (FMT == 0) {                                       // OIL1: eight FP16 run means (:615-626)
        const float m = half_bits_to_float(reinterpret_cast<const uint16_t*>(p)[lane >> 3]);
        return make_float4(m, m, m, m);
    } else if constexpr (FMT == 1) {                                       // SPARK_Q0: per run FP16 scale + 32 sign bits (:643-654)
        const uint16_t* h = reinterpret_cast<const uint16_t*>(p);
        const uint32_t run = lane >> 3, j0 = 4u * (lane & 7u);
        const float sc = half_bits_to_float(h[3u * run]);
        const uint32_t bits = ((uint32_t)h[3u * run + 1u] | ((uint32_t)h[3u * run + 2u] << 16)) >> j0;
        return make_float4((bits & 1u) ? sc : -sc, (bits & 2u) ? sc : -sc, (bits & 4u) ? sc : -sc, (bits & 8u) ? sc : -sc);
    } else if constexpr (FMT == 5 || FMT == 12) {                          // OIL16 / OIL16_GRP: 512 bytes of FP16 (:588-596)
        const uint32_t a = q[2u * lane], c = q[2u * lane + 1u];
        return make_float4(half_bits_to_float(a & 0xFFFFu), half_bits_to_float(a >> 16), half_bits_to_float(c & 0xFFFFu),
                           half_bits_to_float(c >> 16));
    } else if constexpr (FMT == 6) {                                       // OIL32: raw FP32 (:585-587)
        const uint4 v = reinterpret_cast<const uint4*>(p)[lane];
        return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
    } else if constexpr (FMT == 7) {                                       // OIL1_GRP: scale, 240 sign bits, every 16th weight a slot (:627-642)
        const float scale = half_bits_to_float(q[0] & 0xFFFFu);
        const uint32_t bit = 16u + i0 - i0 / 16u;
        const uint32_t v = __builtin_amdgcn_alignbit(q[(bit >> 5) + 1u], q[bit >> 5], bit & 31u);
        const bool last_is_slot = ((i0 + 4u) & 15u) == 0u;
        return make_float4((v & 1u) ? scale : -scale, (v & 2u) ? scale : -scale, (v & 4u) ? scale : -scale,
                           last_is_slot ? 0.0f : ((v & 8u) ? scale : -scale));
    } else if constexpr (FMT == 8) {                                       // SPARK_Q0_GRP: scale, 256 signs, 112 refinement bits (:655-676)
        const float scale = half_bits_to_float(q[0] & 0xFFFFu);
        const uint32_t sbit = 16u + i0;                                    // four signs inside one dword
        const uint32_t sg = q[sbit >> 5] >> (sbit & 31u);
        float r[4];
#pragma unroll
        for (uint32_t e = 0; e < 4u; ++e) {
            const uint32_t i = i0 + e;
            float mag = scale;
            if (((i + 1u) * 112u) / 256u != (i * 112u) / 256u) {           // a refined position (is_slot with 112 of 256)
                const uint32_t rpos = 16u + 256u + (i * 112u) / 256u;
                mag = __fmul_rn(scale, ((q[rpos >> 5] >> (rpos & 31u)) & 1u) ? 1.893f : 0.567f);
            }
            r[e] = ((sg >> e) & 1u) ? mag : -mag;
        }
        return make_float4(r[0], r[1], r[2], r[3]);
    } else if constexpr (FMT == 9 || FMT == 10 || FMT == 11) {             // grouped lattice: 4 x {FP16 zp, FP16 scale, 64 codes} (:308-331)
        constexpr uint32_t bits = FMT == 9 ? 2u : (FMT == 10 ? 4u : 8u), gbytes = 4u + 8u * bits;
        const float* lv = FMT == 9 ? L.lv2 : (FMT == 10 ? L.lv4 : L.t255);
        const uint32_t g = lane >> 4, j0 = 4u * (lane & 15u);              // group, first weight of the lane inside it
        const uint32_t hdr = *reinterpret_cast<const uint32_t*>(p + g * gbytes);
        const float zp = half_bits_to_float(hdr & 0xFFFFu), sc = half_bits_to_float(hdr >> 16);
        const uint32_t cbit = j0 * bits;                                   // 4 codes: 8, 16 or 32 bits inside one dword
        const uint32_t v = *reinterpret_cast<const uint32_t*>(p + g * gbytes + 4u + (cbit >> 5) * 4u) >> (cbit & 31u);
        float r[4];
#pragma unroll
        for (uint32_t e = 0; e < 4u; ++e)
            r[e] = sc == 0.0f ? zp : __fmaf_rn(lv[(v >> (e * bits)) & ((1u << bits) - 1u)], sc, zp);
        return make_float4(r[0], r[1], r[2], r[3]);
    } else {                                                               // SPARK_SPARSE / _GRP: header + 20 records, later ones win (:677-716)
        const uint4* p4 = reinterpret_cast<const uint4*>(p);
        const uint4 v0 = p4[0], v1 = p4[1], v2 = p4[2], v3 = p4[3];
        const uint32_t d[16] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w, v2.x, v2.y, v2.z, v2.w, v3.x, v3.y, v3.z, v3.w};
        float s0, s1;
        bool dead;
        if (FMT == 13) { s0 = s1 = __uint_as_float(d[0]); dead = s0 == 0.0f; }
        else { s0 = half_bits_to_float(d[0] & 0xFFFFu); s1 = half_bits_to_float(d[0] >> 16); dead = s0 == 0.0f && s1 == 0.0f; }
        float r[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int k = 0; k < 20; ++k) {
            const int o = 4 + 3 * k;                                       // byte offset of record k
            const uint32_t lo = d[o >> 2], hi = d[(o >> 2) + ((o & 3) ? 1 : 0)];
            const uint32_t rec = __builtin_amdgcn_alignbyte(hi, lo, o & 3) & 0xFFFFFFu;
            const uint32_t rel = rec & 0xFFFFu, e = rel - i0;
            const float val = L.q127[rec >> 16] * (rel < 128u ? s0 : s1);
#pragma unroll
            for (uint32_t t = 0; t < 4u; ++t) r[t] = e == t ? val : r[t];
        }
        return dead ? make_float4(0.0f, 0.0f, 0.0f, 0.0f) : make_float4(r[0], r[1], r[2], r[3]);
    }
}

#define OILHIP_ALL_FORMATS(X) X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14)

// FMT >= 0: every block has that format; FMT < 0: each block's format from its descriptor (tensors that mix formats)
// BF16: the blocks [b0, b0 + nblocks) as bf16 (each FP32 value rounded once, to nearest even), for the prefill GEMM
template <int FMT, bool BF16 = false>
__global__ void __launch_bounds__(256)
dequant_full_kernel(const uint8_t* __restrict__ base, uint32_t stride, const DevBlock* __restrict__ blocks,
                    const DecodeTables* __restrict__ T, void* __restrict__ out_, uint32_t nblocks, uint32_t b0 = 0) {
    __shared__ float tb[256 * 3 + 20];
    {
        const uint32_t t = threadIdx.x;
        tb[t] = T->lv8[t]; tb[256 + t] = T->t255[t]; tb[512 + t] = T->q127[t];
        if (t < 16) tb[768 + t] = kLv4[t];
        if (t < 4) tb[784 + t] = kLv2[t];
    }
    __syncthreads();
    const FullTables L{tb, tb + 256, tb + 512, tb + 768, tb + 784};
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    for (uint32_t bi = blockIdx.x * 4u + wave; bi < nblocks; bi += gridDim.x * 4u) {
        const uint32_t b = b0 + bi;
        const uint8_t* p = base + (blocks ? (size_t)blocks[b].off16 * 16u : (size_t)b * stride);
        float4 o = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if constexpr (FMT >= 0) {
            o = decode_full4<FMT>(p, lane, L);
        } else {
            const int f = __builtin_amdgcn_readfirstlane((int)blocks[b].fmt);
#define OILHIP_CASE(F) case F: o = decode_full4<F>(p, lane, L); break;
            switch (f) { OILHIP_ALL_FORMATS(OILHIP_CASE) default: break; }
#undef OILHIP_CASE
        }
        if constexpr (BF16) {
            typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
            const bf2 lo = bf2{(__bf16)o.x, (__bf16)o.y}, hi = bf2{(__bf16)o.z, (__bf16)o.w};
            reinterpret_cast<uint2*>(static_cast<uint16_t*>(out_) + (size_t)bi * 256u)[lane] =
                make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
        } else {
            reinterpret_cast<float4*>(static_cast<float*>(out_) + (size_t)bi * 256u)[lane] = o;
        }
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

// full blocks of nominal size: one format at a regular stride (1), or (window streams, one format or several) the place
// and format of every block from its descriptor (2); 0: neither
static int full_block_layout(const oilhip_weights& w) {
    if (!w.all_full || w.d_out_off) return 0;
    const bool by_stride = w.uniform_fmt >= 0 && w.uniform_stride > 0 && (w.uniform_base & 3u) == 0 &&
                           w.uniform_stride == full_block_bytes(w.uniform_fmt) &&
                           w.uniform_cb == full_block_cb_bytes(w.uniform_fmt) &&
                           w.uniform_cb + w.uniform_idx == w.uniform_stride;
    if (by_stride) return 1;
    bool by_desc = w.seg.nstreams > 0;
    for (uint32_t i = 0; by_desc && i < w.seg.nf; ++i)
        by_desc = w.seg.cb_bytes[i] == full_block_cb_bytes((int)w.seg.fmt[i]) &&
                  w.seg.cb_bytes[i] + w.seg.idx_bytes[i] == full_block_bytes((int)w.seg.fmt[i]);
    return by_desc ? 2 : 0;
}

bool dequant_bf16_blocks_covers(const oilhip_weights& w) { return full_block_layout(w) != 0; }

// The blocks [b0, b0 + nb) decoded to bf16 at d_out (nb * 256 values).  Returns 1 when the tensor's blocks are not
// full blocks of nominal size.
int launch_dequant_bf16_blocks(const oilhip_weights& w, uint32_t b0, uint32_t nb, uint16_t* d_out, hipStream_t s) {
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    const int layout = full_block_layout(w);
    if (!layout) return 1;
    if (nb == 0) return OILHIP_OK;
    const uint32_t g = std::min<uint32_t>((nb + 3u) / 4u, (uint32_t)device_cu_count() * 16u);
    const bool by_stride = layout == 1;
    const uint8_t* base = w.d_payload + (by_stride ? w.uniform_base : 0u);
    const DevBlock* bl = by_stride ? nullptr : w.d_blocks;
    const int f = by_stride || w.seg.nf == 1 ? w.uniform_fmt : -1;
#define OILHIP_CASE(F) case F: hipLaunchKernelGGL((dequant_full_kernel<F, true>), dim3(g), dim3(256), 0, s, base, w.uniform_stride, bl, T, (void*)d_out, nb, b0); break;
    switch (f) {
        OILHIP_ALL_FORMATS(OILHIP_CASE)
        default: hipLaunchKernelGGL((dequant_full_kernel<-1, true>), dim3(g), dim3(256), 0, s, base, 0u, bl, T, (void*)d_out, nb, b0); break;
    }
#undef OILHIP_CASE
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int launch_dequant(const oilhip_weights& w, float* d_out, hipStream_t s) {
    const DecodeTables* T = nullptr;
    if (int rc = get_tables(&T)) return rc;
    if (w.nblocks == 0) return OILHIP_OK;
    {
        const uint32_t g = std::min<uint32_t>((w.nblocks + 3u) / 4u, (uint32_t)device_cu_count() * 16u);
        const int layout = full_block_layout(w);
        const bool by_stride = layout == 1;
        if (layout) {
            const uint8_t* base = w.d_payload + (by_stride ? w.uniform_base : 0u);
            const DevBlock* bl = by_stride ? nullptr : w.d_blocks;
            const int f = by_stride || w.seg.nf == 1 ? w.uniform_fmt : -1;
#define OILHIP_CASE(F) case F: hipLaunchKernelGGL((dequant_full_kernel<F, false>), dim3(g), dim3(256), 0, s, base, w.uniform_stride, bl, T, (void*)d_out, w.nblocks, 0u); break;
            switch (f) {
                OILHIP_ALL_FORMATS(OILHIP_CASE)
                default: hipLaunchKernelGGL((dequant_full_kernel<-1, false>), dim3(g), dim3(256), 0, s, base, 0u, bl, T, (void*)d_out, w.nblocks, 0u); break;
            }
#undef OILHIP_CASE
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
