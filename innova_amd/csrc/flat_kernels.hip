// flat_kernels.hip -- the reference's flat-codebook matmul entry points on the
// device: one caller-supplied codebook, plain row-major index matrices.
//   oil::kernel::oil8_gemm / oil4_gemm          src/kernel_oil8.cpp, src/kernel_oil4.cpp
//   oil::adapters::prod::gemv_{spark,oil4,oil8} src/kernel_production.cpp:79-128,345-364
//   oil::engines::OIL{8,4,2}Engine::quant_gemm  src/oil_engines_oil{8,4,2}.cpp
// One workgroup of 256 threads per output row; the codebook sits in LDS; thread t
// walks k = t, t+256, ... so index bytes are read coalesced.
#include <algorithm>

#include "common.h"

namespace oilhip {
namespace {

constexpr int MBF = 4;   // activation rows per pass

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// Sum acc[0..MBF) over the 256 threads; thread b < MBF returns the total of acc[b].
__device__ __forceinline__ float block_sums(const float (&acc)[MBF], float (*part)[4]) {
    const uint32_t t = threadIdx.x;
#pragma unroll
    for (int b = 0; b < MBF; ++b) {
        const float s = wave_sum(acc[b]);
        if ((t & 63) == 0) part[b][t >> 6] = s;
    }
    __syncthreads();
    float r = 0.0f;
    if (t < MBF) r = (part[t][0] + part[t][1]) + (part[t][2] + part[t][3]);
    __syncthreads();
    return r;
}

// FP16 codebook entry exactly as fp16_to_float (src/kernel_oil4.cpp:15-29).
__device__ __forceinline__ float flat_half(uint16_t h) {
    const uint32_t e = (h >> 10) & 31u, m = h & 0x3FFu;
    if (e == 31u && m != 0u) return __uint_as_float(0x7FC00000u);
    return half_bits_to_float(h);
}

// mode 0: oil8_gemm  -- weights row n (K bytes),        activations row m, out[m*N+n]
// mode 1: prod oil8  -- weights row n (K bytes),        activations row m, out[m*N+n] * scale
__global__ void __launch_bounds__(256)
flat8_kernel(const uint8_t* __restrict__ idx, const float* __restrict__ cb, const float* __restrict__ act,
             float* __restrict__ out, int M, int N, int K, float scale) {
    __shared__ float c[256];
    __shared__ float part[MBF][4];
    const uint32_t t = threadIdx.x, n = blockIdx.x;
    c[t] = cb[t];
    __syncthreads();
    const uint8_t* w = idx + (size_t)n * K;
    for (int m0 = 0; m0 < M; m0 += MBF) {
        float acc[MBF] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int k = t; k < K; k += 256) {
            const float v = c[w[k]];
#pragma unroll
            for (int b = 0; b < MBF; ++b)
                if (m0 + b < M) acc[b] = __fmaf_rn(v, act[(size_t)(m0 + b) * K + k], acc[b]);
        }
        const float r = block_sums(acc, part);
        if (t < MBF && m0 + (int)t < M) out[(size_t)(m0 + t) * N + n] = r * scale;
    }
}

// oil4_gemm: one workgroup per (m, n) pair; the pair's K nibbles start at nibble
// (m*N+n)*K rounded down to a byte, activations are row n (src/kernel_oil4.cpp:38-56).
__global__ void __launch_bounds__(256)
flat4_pair_kernel(const uint8_t* __restrict__ packed, const uint16_t* __restrict__ cb16,
                  const float* __restrict__ act, float* __restrict__ out, int N, int K) {
    __shared__ float c[16];
    __shared__ float part[MBF][4];
    const uint32_t t = threadIdx.x;
    const uint64_t pair = blockIdx.x;
    if (t < 16) c[t] = flat_half(cb16[t]);
    __syncthreads();
    const uint8_t* w = packed + (pair * (uint64_t)K) / 2;
    const float* a = act + (pair % (uint64_t)N) * (uint64_t)K;
    float acc[MBF] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int k = t; k < K; k += 256) {
        const uint32_t byte = w[k >> 1];
        acc[0] = __fmaf_rn(c[(k & 1) ? (byte >> 4) : (byte & 15u)], a[k], acc[0]);
    }
    const float r = block_sums(acc, part);
    if (t == 0) out[pair] = r;
}

// prod gemv over packed rows: BITS = 4 (two codes per byte, FP16 codebook) or
// BITS = 2 (SPARK ternary: 0 -> -1, 1 -> 0, 2 and 3 -> +1).  Row m of W against
// activation row b; Y[b*M + m] = scale * dot.
template <int BITS>
__global__ void __launch_bounds__(256)
prod_packed_kernel(const uint8_t* __restrict__ wq, const uint16_t* __restrict__ cb16, float scale,
                   const float* __restrict__ x, float* __restrict__ y, int M, int K, int batch) {
    __shared__ float c[16];
    __shared__ float part[MBF][4];
    const uint32_t t = threadIdx.x, m = blockIdx.x;
    if (BITS == 4 && t < 16) c[t] = flat_half(cb16[t]);
    __syncthreads();
    constexpr int PER = 8 / BITS;
    const uint8_t* row = wq + (size_t)m * ((K + PER - 1) / PER);
    for (int b0 = 0; b0 < batch; b0 += MBF) {
        float acc[MBF] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int k = t; k < K; k += 256) {
            const uint32_t code = (row[k / PER] >> ((k % PER) * BITS)) & ((1u << BITS) - 1u);
            const float v = BITS == 4 ? c[code] : (code == 0 ? -1.0f : (code == 1 ? 0.0f : 1.0f));
#pragma unroll
            for (int b = 0; b < MBF; ++b)
                if (b0 + b < batch) acc[b] = __fmaf_rn(v, x[(size_t)(b0 + b) * K + k], acc[b]);
        }
        const float r = block_sums(acc, part);
        if (t < MBF && b0 + (int)t < batch) y[(size_t)(b0 + t) * M + m] = r * scale;
    }
}

// Engine layout: codes packed along the flat [K][N] index; thread per output column
// n, sequential in k like the reference loop (terms with A == 0 are skipped).
template <int BITS>
__global__ void __launch_bounds__(64)
engine_kernel(const float* __restrict__ A, const uint8_t* __restrict__ bq, const float* __restrict__ cb,
              float* __restrict__ C, long long M, long long N, long long K) {
    // One wavefront per 64 outputs of a row of C: the chain of every output stays one thread's k-ordered FMA
    // sequence (bit-identical to the reference loop), so the only parallelism is across outputs; what can be taken
    // off the chain is taken off: the codes of 32 steps are fetched together, A[m][k] is wave-uniform and read
    // through the scalar cache, and the codebook sits in LDS in 8 copies.
    __shared__ float c[(1 << BITS) * 8];
    for (int i = threadIdx.x; i < (1 << BITS) * 8; i += 64) c[i] = cb[i >> 3];
    __syncthreads();
    const long long n = (long long)blockIdx.x * 64 + threadIdx.x;
    const long long m = blockIdx.y;
    const bool live = n < N;
    const long long nn = live ? n : N - 1;                // idle lanes follow the last column and store nothing
    constexpr int PER = 8 / BITS;
    constexpr int UN = 32;
    const float* a_row = A + m * K;
    const uint32_t copy = threadIdx.x & 7u;
    float acc = 0.0f;
    long long k = 0;
    uint8_t raw[UN], nxt[UN];
    auto fetch = [&](uint8_t (&dst)[UN], long long k0) {
#pragma unroll
        for (int j = 0; j < UN; ++j) dst[j] = bq[((unsigned long long)(k0 + j) * (unsigned long long)N + (unsigned long long)nn) / PER];
    };
    if (K >= UN) fetch(raw, 0);
    for (; k + UN <= K; k += UN) {
        const bool more = k + 2 * UN <= K;
        if (more) fetch(nxt, k + UN);                     // the next 32 steps fly while these are folded in
        float lv[UN];
#pragma unroll
        for (int j = 0; j < UN; ++j) {                    // look-ups off the chain: none of them depends on acc
            const uint32_t sub = (uint32_t)((unsigned long long)(k + j) * (unsigned long long)N + (unsigned long long)nn) & (uint32_t)(PER - 1);
            const uint32_t code = ((uint32_t)raw[j] >> (sub * BITS)) & ((1u << BITS) - 1u);
            lv[j] = c[code * 8u + copy];
        }
#pragma unroll
        for (int j = 0; j < UN; ++j) {
            const float a = a_row[k + j];
            const float t = __fmaf_rn(a, lv[j], acc);
            acc = a != 0.0f ? t : acc;                    // the reference skips the term, 0 * inf must not reach acc
        }
        if (more) {
#pragma unroll
            for (int j = 0; j < UN; ++j) raw[j] = nxt[j];
        }
    }
    for (; k < K; ++k) {
        const float a = a_row[k];
        if (a == 0.0f) continue;
        const long long flat = k * N + nn;
        const uint32_t code = (bq[flat / PER] >> ((flat % PER) * BITS)) & ((1u << BITS) - 1u);
        acc = __fmaf_rn(a, c[code * 8u + copy], acc);
    }
    if (live) C[m * N + n] = acc;
}

// engine_kernel<8> for N a multiple of 4: the same k-ordered chain per output, fed differently.  A wavefront per 64
// outputs leaves most of the chip idle and a single wavefront issues one instruction at a time, so the time is the
// instruction count per k step.  The four lanes of a quad own four neighbouring columns, whose codes of one k step
// share a dword: lane q of the quad loads the dword of step 4i + q and the quad passes the dwords round with DPP
// (8 loads per lane and 32 steps instead of 32 byte loads, three batches of 32 steps in flight); the look-up address
// is one v_perm_b32 (entry v of lane l at byte v*256 + l*4 of a 64 KB table); the levels of batch b+1 are looked up
// before the chain of batch b runs.  A batch without a zero in A (the usual case) is 32 bare FMAs; one with a zero
// keeps the reference's skip as a select behind every FMA, so the result is the reference's bit for bit either way.
__global__ void __launch_bounds__(64)
engine8_quad_kernel(const float* __restrict__ A, const uint8_t* __restrict__ bq, const float* __restrict__ cb,
                    float* __restrict__ C, long long M, long long N, long long K) {
    __shared__ float c[256 * 64];
    {
        const float mine[4] = {cb[threadIdx.x], cb[64 + threadIdx.x], cb[128 + threadIdx.x], cb[192 + threadIdx.x]};
#pragma unroll
        for (int part = 0; part < 4; ++part)
            for (int v = 0; v < 64; ++v)
                c[(part * 64 + v) * 64 + threadIdx.x] = __shfl(mine[part], v);
    }
    __syncthreads();
    const long long n = (long long)blockIdx.x * 64 + threadIdx.x;
    const long long m = blockIdx.y;
    const bool live = n < N;                               // N % 4 == 0: a quad is live or idle as a whole
    const uint32_t sub = threadIdx.x & 3u, lane = threadIdx.x;
    const unsigned long long n4 = (unsigned long long)(live ? n - sub : N - 4);
    const float* a_row = A + m * K;
    constexpr int UN = 32, NB = 4;
    const long long nb = K / UN;                           // full batches
    const uint32_t lanebase = lane * 4u, sel = 0x0C0C0000u | ((4u + sub) << 8);
    uint32_t dw[NB][8];
    float av[NB];                                          // lane j < 32: A[m][32 b + j], for the zero test
    auto clampb = [&](long long b) { return b < nb ? b : nb - 1; };
    // a lane's byte offset inside a k step's row pair: uniform 64-bit bases, 32-bit lane offsets (N < 2^29)
    const uint32_t lane_off = sub * (uint32_t)N + (uint32_t)n4;
    auto fetch = [&](int slot, long long b) {              // batch b, clamped to the last one: issued unconditionally
        const unsigned long long k0 = (unsigned long long)clampb(b) * UN;
        const uint8_t* ub = bq + k0 * (unsigned long long)N;                 // uniform
#pragma unroll
        for (int i = 0; i < 8; ++i) dw[slot][i] = *reinterpret_cast<const uint32_t*>(ub + 4ull * i * (unsigned long long)N + lane_off);
        av[slot] = a_row[k0 + (lane & 31u)];
    };
    float lv[2][UN];
    auto lookup = [&](int slot, int set) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int v = (int)dw[slot][i];
            const uint32_t qs[4] = {(uint32_t)__builtin_amdgcn_mov_dpp(v, 0x00, 0xF, 0xF, true),     // quad_perm [0,0,0,0]
                                    (uint32_t)__builtin_amdgcn_mov_dpp(v, 0x55, 0xF, 0xF, true),     // [1,1,1,1]
                                    (uint32_t)__builtin_amdgcn_mov_dpp(v, 0xAA, 0xF, 0xF, true),     // [2,2,2,2]
                                    (uint32_t)__builtin_amdgcn_mov_dpp(v, 0xFF, 0xF, 0xF, true)};    // [3,3,3,3]
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t addr = __builtin_amdgcn_perm(qs[q], lanebase, sel);
                lv[set][4 * i + q] = *reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(c) + addr);
            }
        }
    };
    float acc = 0.0f;
    auto chain = [&](const float (&a)[UN], int slot, int set) {
        const bool any_zero = __ballot(av[slot] == 0.0f) != 0ull;         // uniform
        if (!any_zero) {
#pragma unroll
            for (int j = 0; j < UN; ++j) acc = __fmaf_rn(a[j], lv[set][j], acc);
        } else {
#pragma unroll
            for (int j = 0; j < UN; ++j) {
                const float t = __fmaf_rn(a[j], lv[set][j], acc);
                acc = a[j] != 0.0f ? t : acc;              // the reference skips the term
            }
        }
    };
    if (nb > 0) {
#pragma unroll
        for (int u = 0; u < NB - 1; ++u) fetch(u, u);
        lookup(0, 0);
        for (long long b = 0; b < nb; b += NB) {
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                if (b + u < nb) {
                    float a[UN];                           // A[m][32 (b+u) ..], uniform: requested before the look-ups
#pragma unroll
                    for (int j = 0; j < UN; ++j) a[j] = a_row[(b + u) * UN + j];
                    fetch((u + NB - 1) % NB, b + u + NB - 1);
                    lookup((u + 1) % NB, (u + 1) & 1);     // batch b+u+1 (past the end: the clamped copy, never folded in)
                    chain(a, u, u & 1);
                }
            }
        }
    }
    const unsigned long long nn = n4 + sub;
    for (long long k = nb * UN; k < K; ++k) {
        const float a = a_row[k];
        if (a == 0.0f) continue;
        acc = __fmaf_rn(a, c[(uint32_t)bq[(unsigned long long)k * (unsigned long long)N + nn] * 64u + lane], acc);
    }
    if (live) C[m * N + n] = acc;
}

// The engines whose B operand is not a codebook index: kind 1 = Oil1Engine (one float per 32 flat positions,
// src/oil_engines_oil1.cpp:61-82), 3 = SparkEngine (2-bit codes: 2 -> +s, 0 -> -s, else 0, with s = a * scale of
// the flat position's block, src/oil_engines_spark.cpp:154-186), 16 = OIL16Engine (FP16 widened as
// math::vec_fp16_to_fp32 does, src/math.cpp:509-526; src/oil_engines_fp.cpp:433-451), 32 = OIL32Engine (:531-547).
// Terms with a == 0 are skipped and k runs in ascending order, as in the reference loops.
template <int KIND>
__global__ void __launch_bounds__(64)
engine_dense_kernel(const float* __restrict__ A, const void* __restrict__ B, const float* __restrict__ scales,
                    long long block, float* __restrict__ C, long long M, long long N, long long K) {
    // Same frame as engine_kernel: a wavefront per 64 outputs, the operand of 32 steps fetched together and one
    // batch ahead, the k-ordered chain of every output untouched.
    const long long n = (long long)blockIdx.x * 64 + threadIdx.x;
    const long long m = blockIdx.y;
    const bool live = n < N;
    const unsigned long long nn = (unsigned long long)(live ? n : N - 1);
    constexpr int UN = KIND == 3 ? 16 : 32;              // kind 3 fetches two operands per step
    const float* a_row = A + m * K;
    struct Term { float b; float s; };                   // kind 3: b = +1 / -1 / 0 by code, s = scale of the flat position's block
    // kind 3: block index and offset of the next flat position to be fetched (fetches go through k in order)
    const unsigned long long ublock = block > 0 ? (unsigned long long)block : 1ull;
    unsigned long long fq = nn / ublock, fr = nn % ublock;
    const unsigned long long dq = (unsigned long long)N / ublock, dr = (unsigned long long)N % ublock;
    auto fetch_one = [&](long long kk) {
        const unsigned long long flat = (unsigned long long)kk * (unsigned long long)N + nn;
        Term t{0.0f, 1.0f};
        if (KIND == 1) t.b = reinterpret_cast<const float*>(B)[flat / 32];
        else if (KIND == 32) t.b = reinterpret_cast<const float*>(B)[flat];
        else if (KIND == 16) t.b = __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(B)[flat]);   // raw half, widened later
        else {
            t.s = scales[fq];
            t.b = __uint_as_float((uint32_t)((reinterpret_cast<const uint8_t*>(B)[flat / 4] >> ((flat % 4) * 2)) & 3u));
            fq += dq; fr += dr;
            if (fr >= ublock) { fr -= ublock; ++fq; }
        }
        return t;
    };
    auto widen = [](float raw) {                          // math::vec_fp16_to_fp32: -0 widens to +0; selects only
        const uint32_t h = __float_as_uint(raw);
        const uint32_t sg = (h & 0x8000u) << 16, e = (h >> 10) & 31u, mt = h & 0x3FFu;
        const uint32_t normal = sg | ((e + 112u) << 23) | (mt << 13);
        const uint32_t infnan = sg | 0x7F800000u | (mt << 13);
        const uint32_t sub = sg | __float_as_uint(__uint2float_rn(mt) * 0x1p-24f);      // exact
        const uint32_t r = e == 31u ? infnan : (e != 0u ? normal : sub);
        return (h & 0x7FFFu) == 0u ? 0.0f : __uint_as_float(r);
    };
    auto fold = [&](float acc, float a, const Term& t) {
        if (KIND == 1 || KIND == 32) {
            const float r = __fmaf_rn(a, t.b, acc);
            return a != 0.0f ? r : acc;
        } else if (KIND == 16) {
            const float r = __fmaf_rn(a, t.b, acc);                                  // widened before the chain starts
            return a != 0.0f ? r : acc;
        } else {
            const float s = __fmul_rn(a, t.s);                                       // a product, then a sum: no fused form here
            const uint32_t code = __float_as_uint(t.b);
            const float r = code == 2u ? __fadd_rn(acc, s) : (code == 0u ? __fsub_rn(acc, s) : acc);
            return a != 0.0f ? r : acc;
        }
    };
    float acc = 0.0f;
    long long k = 0;
    Term cur[UN], nxt[UN];
    if (K >= UN) {
#pragma unroll
        for (int j = 0; j < UN; ++j) cur[j] = fetch_one(j);
    }
    for (; k + UN <= K; k += UN) {
        const bool more = k + 2 * UN <= K;
        if (more) {
#pragma unroll
            for (int j = 0; j < UN; ++j) nxt[j] = fetch_one(k + UN + j);
        }
        if (KIND == 16) {
#pragma unroll
            for (int j = 0; j < UN; ++j) cur[j].b = widen(cur[j].b);
        }
#pragma unroll
        for (int j = 0; j < UN; ++j) acc = fold(acc, a_row[k + j], cur[j]);
        if (more) {
#pragma unroll
            for (int j = 0; j < UN; ++j) cur[j] = nxt[j];
        }
    }
    for (; k < K; ++k) {
        Term t = fetch_one(k);
        if (KIND == 16) t.b = widen(t.b);
        acc = fold(acc, a_row[k], t);
    }
    if (live) C[m * N + n] = acc;
}

// OIL{8,4,2}Engine::dequant_tensor (src/oil_engines_oil8.cpp:171-183, oil4.cpp:205-220, oil2.cpp:184-193): packed
// codes -> codebook values; with scales, OIL8Engine / OIL4Engine::dequantize_per_block (oil8.cpp:121-134:
// cb[i] * scale; oil4.cpp:136-150: cb[i] * half_range + center, one multiply-add in the reference build) over
// one index byte per weight.
__global__ void __launch_bounds__(256)
engine_dequant_kernel(int bits, const uint8_t* __restrict__ idx, const float* __restrict__ cb, long long n,
                      const float* __restrict__ scales, long long block, float* __restrict__ out) {
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
        if (!scales) {
            const int per = 8 / bits;
            const uint32_t code = (idx[i / per] >> ((i % per) * bits)) & ((1u << bits) - 1u);
            out[i] = cb[code];
        } else if (bits == 8) {
            out[i] = cb[idx[i]] * scales[i / block];
        } else {
            const long long b = i / block;
            out[i] = __fmaf_rn(cb[idx[i] & 15u], scales[2 * b + 1], scales[2 * b]);
        }
    }
}

// Negative sizes are errors; an empty output (M or N zero) needs no pointers at all.
int check(const void* a, const void* b, const void* c, const void* d, long long M, long long N, long long K) {
    if (M < 0 || N < 0 || K < 0) return fail(OILHIP_E_ARG, "negative dimension");
    if (M == 0 || N == 0) return OILHIP_OK;
    if (!a || !b || !c || !d) return fail(OILHIP_E_ARG, "null argument");
    return OILHIP_OK;
}

}  // namespace
}  // namespace oilhip

using namespace oilhip;

extern "C" {

int oilhip_flat_oil8_gemm(const uint8_t* d_idx, const float* d_cb, const float* d_act, float* d_out,
                          int M, int N, int K, void* stream) {
    if (int rc = check(d_idx, d_cb, d_act, d_out, M, N, K)) return rc;
    if (M == 0 || N == 0) return OILHIP_OK;
    if (M <= 4) {                                     // decode shapes: the register-resident kernel
        const int rc = launch_gemv_flat8(d_idx, d_cb, d_act, d_out, M, N, K, 1.0f, (hipStream_t)stream);
        if (rc <= 0) return rc;
    }
    hipLaunchKernelGGL(flat8_kernel, dim3(N), dim3(256), 0, (hipStream_t)stream, d_idx, d_cb, d_act, d_out, M, N, K, 1.0f);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int oilhip_flat_oil4_gemm(const uint8_t* d_packed, const uint16_t* d_cb16, const float* d_act, float* d_out,
                          int M, int N, int K, void* stream) {
    if (int rc = check(d_packed, d_cb16, d_act, d_out, M, N, K)) return rc;
    if (M == 0 || N == 0) return OILHIP_OK;
    if ((long long)M * N > 0x7FFFFFFFll) return fail(OILHIP_E_ARG, "M*N exceeds the grid limit");
    hipLaunchKernelGGL(flat4_pair_kernel, dim3((uint32_t)((long long)M * N)), dim3(256), 0, (hipStream_t)stream,
                       d_packed, d_cb16, d_act, d_out, N, K);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int oilhip_prod_gemv_spark(const uint8_t* d_w, float scale, const float* d_x, float* d_y,
                           int M, int K, int batch, void* stream) {
    if (int rc = check(d_w, d_x, d_y, d_y, M, batch, K)) return rc;
    if (M == 0 || batch == 0) return OILHIP_OK;
    hipLaunchKernelGGL(prod_packed_kernel<2>, dim3(M), dim3(256), 0, (hipStream_t)stream, d_w,
                       (const uint16_t*)nullptr, scale, d_x, d_y, M, K, batch);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int oilhip_prod_gemv_oil4(const uint8_t* d_w, const uint16_t* d_cb16, float scale, const float* d_x,
                          float* d_y, int M, int K, int batch, void* stream) {
    if (int rc = check(d_w, d_cb16, d_x, d_y, M, batch, K)) return rc;
    if (M == 0 || batch == 0) return OILHIP_OK;
    if (batch <= 2) {                                 // decode: the register-resident kernel, one activation row per launch
        int rc = 0;
        for (int b = 0; b < batch && rc == 0; ++b)
            rc = launch_gemv_flat4(d_w, d_cb16, scale, d_x + (size_t)b * K, d_y + (size_t)b * M, M, K, (hipStream_t)stream);
        if (rc <= 0) return rc;
    }
    hipLaunchKernelGGL(prod_packed_kernel<4>, dim3(M), dim3(256), 0, (hipStream_t)stream, d_w, d_cb16, scale,
                       d_x, d_y, M, K, batch);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

// Y[b*M + m]: the flat OIL8 kernel with (rows = M weight rows, batch = activation rows).
int oilhip_prod_gemv_oil8(const uint8_t* d_w, const float* d_cb, float scale, const float* d_x, float* d_y,
                          int M, int K, int batch, void* stream) {
    if (int rc = check(d_w, d_cb, d_x, d_y, M, batch, K)) return rc;
    if (M == 0 || batch == 0) return OILHIP_OK;
    if (batch <= 4) {
        const int rc = launch_gemv_flat8(d_w, d_cb, d_x, d_y, batch, M, K, scale, (hipStream_t)stream);
        if (rc <= 0) return rc;
    }
    hipLaunchKernelGGL(flat8_kernel, dim3(M), dim3(256), 0, (hipStream_t)stream, d_w, d_cb, d_x, d_y, batch, M, K, scale);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

// profile_gemv_{spark,oil4,oil8} (src/kernel_production.cpp:433-485): `repeats` launches of the tiled GEMV between two
// events on `stream`; waits for them.  Not capturable.
int oilhip_profile_gemv(int kind, const uint8_t* d_w, const void* d_cb, float scale, const float* d_x, float* d_y,
                        int M, int K, int repeats, oilhip_kernel_perf_t* out, void* stream) {
    if (!out) return fail(OILHIP_E_ARG, "profile_gemv: null result");
    if (kind != 0 && kind != 4 && kind != 8) return fail(OILHIP_E_ARG, "profile_gemv: kind must be 0 (SPARK), 4 (OIL4) or 8 (OIL8)");
    if (repeats < 1) repeats = 1;
    auto run = [&]() {
        return kind == 0 ? oilhip_prod_gemv_spark(d_w, scale, d_x, d_y, M, K, 1, stream)
             : kind == 4 ? oilhip_prod_gemv_oil4(d_w, static_cast<const uint16_t*>(d_cb), scale, d_x, d_y, M, K, 1, stream)
                         : oilhip_prod_gemv_oil8(d_w, static_cast<const float*>(d_cb), scale, d_x, d_y, M, K, 1, stream);
    };
    if (int rc = run()) return rc;                    // first-use set-up stays outside the timed launches
    auto s = static_cast<hipStream_t>(stream);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    OILHIP_HIP(hipEventCreate(&e0));
    if (hipError_t e = hipEventCreate(&e1); e != hipSuccess) {
        (void)hipEventDestroy(e0);
        return fail(OILHIP_E_DEVICE, std::string("hipEventCreate: ") + hipGetErrorString(e));
    }
    int rc = OILHIP_OK;
    float ms = 0.f;
    hipError_t he = hipEventRecord(e0, s);
    for (int r = 0; r < repeats && rc == OILHIP_OK && he == hipSuccess; ++r) rc = run();
    if (he == hipSuccess) he = hipEventRecord(e1, s);
    if (he == hipSuccess) he = hipEventSynchronize(e1);
    if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != OILHIP_OK) return rc;
    if (he != hipSuccess) return fail(OILHIP_E_DEVICE, std::string("profile_gemv: ") + hipGetErrorString(he));
    int dev = 0, khz = 0;
    OILHIP_HIP(hipGetDevice(&dev));
    OILHIP_HIP(hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, dev));
    const double sec = (double)ms * 1e-3 / repeats;
    const uint64_t m = (uint64_t)(M > 0 ? M : 0), k = (uint64_t)(K > 0 ? K : 0);
    out->cycles = (uint64_t)(sec * (double)khz * 1e3);            // shader clocks at the device's peak frequency
    out->bytes_read = kind == 0 ? m * k * 2 : kind == 4 ? m * k / 2 + m * k * 4 : m * k + m * 1024;   // the reference's formulas
    out->bytes_written = m * 4;
    out->gflops = sec > 0.0 ? 2.0 * (double)m * (double)k / (sec * 1.0e9) : 0.0;
    return OILHIP_OK;
}

int oilhip_engine_quant_gemm(int bits, const float* d_a, const uint8_t* d_b, const float* d_cb, float* d_c,
                             int64_t M, int64_t N, int64_t K, void* stream) {
    if (int rc = check(d_a, d_b, d_cb, d_c, M, N, K)) return rc;
    if (bits != 2 && bits != 4 && bits != 8) return fail(OILHIP_E_ARG, "bits must be 2, 4 or 8");
    if (M == 0 || N == 0) return OILHIP_OK;
    if (M > 65535) return fail(OILHIP_E_ARG, "M exceeds the grid limit");
    const dim3 grid((uint32_t)((N + 63) / 64), (uint32_t)M);
    hipStream_t s = (hipStream_t)stream;
    if (bits == 8 && (N & 3) == 0 && N < (1ll << 29) && (reinterpret_cast<uintptr_t>(d_b) & 3u) == 0)
        hipLaunchKernelGGL(engine8_quad_kernel, grid, dim3(64), 0, s, d_a, d_b, d_cb, d_c, M, N, K);
    else if (bits == 8) hipLaunchKernelGGL(engine_kernel<8>, grid, dim3(64), 0, s, d_a, d_b, d_cb, d_c, M, N, K);
    else if (bits == 4) hipLaunchKernelGGL(engine_kernel<4>, grid, dim3(64), 0, s, d_a, d_b, d_cb, d_c, M, N, K);
    else hipLaunchKernelGGL(engine_kernel<2>, grid, dim3(64), 0, s, d_a, d_b, d_cb, d_c, M, N, K);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int oilhip_engine_dequant(int bits, const uint8_t* d_idx, const float* d_cb, int64_t n, const float* d_scales,
                          int64_t block, float* d_out, void* stream) {
    if (n < 0) return fail(OILHIP_E_ARG, "negative length");
    if (n == 0) return OILHIP_OK;
    if (!d_idx || !d_cb || !d_out) return fail(OILHIP_E_ARG, "null argument");
    if (bits != 2 && bits != 4 && bits != 8) return fail(OILHIP_E_ARG, "bits must be 2, 4 or 8");
    if (d_scales && (bits == 2 || block <= 0)) return fail(OILHIP_E_ARG, "per-block dequantize exists for 4 and 8 bits with a positive block size");
    const uint32_t grid = (uint32_t)std::min<int64_t>((n + 255) / 256, 65535);
    hipLaunchKernelGGL(engine_dequant_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, bits, d_idx, d_cb, (long long)n,
                       d_scales, (long long)block, d_out);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

int oilhip_engine_dense_gemm(int kind, const float* d_a, const void* d_b, const float* d_scales, int64_t block,
                             float* d_c, int64_t M, int64_t N, int64_t K, void* stream) {
    if (int rc = check(d_a, d_b, d_c, d_c, M, N, K)) return rc;
    if (kind != 1 && kind != 3 && kind != 16 && kind != 32) return fail(OILHIP_E_ARG, "kind must be 1, 3, 16 or 32");
    if (M == 0 || N == 0) return OILHIP_OK;
    if (kind == 3 && (!d_scales || block <= 0)) return fail(OILHIP_E_ARG, "the SPARK engine needs scales and a block size");
    if (M > 65535) return fail(OILHIP_E_ARG, "M exceeds the grid limit");
    const dim3 grid((uint32_t)((N + 63) / 64), (uint32_t)M);
    hipStream_t s = (hipStream_t)stream;
    if (kind == 1) hipLaunchKernelGGL(engine_dense_kernel<1>, grid, dim3(64), 0, s, d_a, d_b, d_scales, (long long)block, d_c, M, N, K);
    else if (kind == 3) hipLaunchKernelGGL(engine_dense_kernel<3>, grid, dim3(64), 0, s, d_a, d_b, d_scales, (long long)block, d_c, M, N, K);
    else if (kind == 16) hipLaunchKernelGGL(engine_dense_kernel<16>, grid, dim3(64), 0, s, d_a, d_b, d_scales, (long long)block, d_c, M, N, K);
    else hipLaunchKernelGGL(engine_dense_kernel<32>, grid, dim3(64), 0, s, d_a, d_b, d_scales, (long long)block, d_c, M, N, K);
    OILHIP_HIP(hipGetLastError());
    return OILHIP_OK;
}

}  // extern "C"
