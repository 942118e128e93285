// run_decode.h -- one run of 32 consecutive weights of a full 256-weight block, per wire format, in two halves:
// fetch_run<FMT> issues the loads of the run's bytes into a few registers, expand_run<FMT> turns them into 32
// FP32 weights.  Keeping the halves apart lets a kernel fetch several runs before it expands the first.  Bit
// layouts follow dequantize_block_all for nw = 256 (src/block_codec.cpp:576-720): dequant_lattice (:173-182),
// dequant_grouped_lattice (:308-331), OIL1 (:615-626), OIL1_GRP (:627-642), SPARK_Q0 (:643-654), OIL16 / OIL32
// (:585-596).  SPARK_Q0_GRP and the sparse formats go through decode_weight, weight by weight.
#pragma once
#include <hip/hip_fp16.h>

#include "block_decode.h"

namespace oilhip {

struct LdsTables { const float* lv2; const float* lv4; const float* lv8; const float* t255; };   // copies in LDS

// FP16 bits -> FP32 through the hardware conversion: the same value as f16_to_f32 (src/block_codec.cpp:61-84) for
// every finite input and infinity (NaN payloads, which the bit-exact dequantization keeps, do not matter in a dot product)
__device__ __forceinline__ float f16_bits(uint32_t h) { return __half2float(__ushort_as_half((unsigned short)(h & 0xFFFFu))); }

// 32-bit window starting `sh` bits into the dword pair (lo, hi)
__device__ __forceinline__ uint32_t funnel(uint32_t lo, uint32_t hi, uint32_t sh) {
    return __builtin_amdgcn_alignbit(hi, lo, sh);       // (hi:lo >> (sh & 31)) low dword
}

// registers a fetched run occupies
__host__ __device__ constexpr int run_raw_dwords(int fmt) {
    return fmt == 0 ? 1 : fmt == 1 ? 2 : fmt == 2 ? 4 : fmt == 3 ? 6 : fmt == 4 ? 10 : fmt == 5 || fmt == 12 ? 16
         : fmt == 6 ? 32 : fmt == 7 ? 3 : fmt == 9 ? 3 : fmt == 10 ? 5 : fmt == 11 ? 9 : 1;
}

// steps of 8 blocks the segmented GEMV fetches together for a format (few registers per run: more steps)
__host__ __device__ constexpr int seg_batch_steps(int fmt) {
    return run_raw_dwords(fmt) <= 3 ? 4 : (run_raw_dwords(fmt) <= 10 ? 2 : 1);
}

__host__ __device__ constexpr int lattice_bits(int fmt) { return fmt == 2 || fmt == 9 ? 2 : (fmt == 3 || fmt == 10 ? 4 : 8); }

// cb: start of the block's payload (codebook channel, then index channel); r: run 0..7 of the block
template <int FMT>
__device__ __forceinline__ void fetch_run(const uint8_t* __restrict__ cb, uint32_t cb_bytes, uint32_t r,
                                          uint32_t (&raw)[run_raw_dwords(FMT)]) {
    const uint8_t* idx = cb + cb_bytes;
    if constexpr (FMT == 0) {
        raw[0] = *reinterpret_cast<const uint16_t*>(cb + 2 * r);
    } else if constexpr (FMT == 1) {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(idx + 6 * r);
        raw[0] = p[0];
        raw[1] = (uint32_t)p[1] | ((uint32_t)p[2] << 16);
    } else if constexpr (FMT == 2 || FMT == 3 || FMT == 4) {
        constexpr uint32_t bits = lattice_bits(FMT), period = 16u * bits;
        const uint32_t b0 = 16u + bits * (32u * r - (32u * r) / period);
        const uint32_t* q = reinterpret_cast<const uint32_t*>(idx) + (b0 >> 5);
        raw[0] = *reinterpret_cast<const uint16_t*>(idx);
#pragma unroll
        for (int j = 0; j < run_raw_dwords(FMT) - 1; ++j) raw[1 + j] = q[j];
    } else if constexpr (FMT == 9 || FMT == 10 || FMT == 11) {
        constexpr uint32_t bits = lattice_bits(FMT), gbytes = 4u + 8u * bits;
        const uint8_t* g = idx + (r >> 1) * gbytes;
        raw[0] = *reinterpret_cast<const uint32_t*>(g);
        const uint32_t* q = reinterpret_cast<const uint32_t*>(g + 4 + (r & 1u) * 4u * bits);
#pragma unroll
        for (int j = 0; j < (int)bits; ++j) raw[1 + j] = q[j];
    } else if constexpr (FMT == 5 || FMT == 12) {
        const uint32_t* q = reinterpret_cast<const uint32_t*>(idx + 64 * r);
#pragma unroll
        for (int j = 0; j < 16; ++j) raw[j] = q[j];
    } else if constexpr (FMT == 6) {
        const uint32_t* q = reinterpret_cast<const uint32_t*>(idx + 128 * r);
#pragma unroll
        for (int j = 0; j < 32; ++j) raw[j] = q[j];
    } else if constexpr (FMT == 7) {
        const uint32_t b0 = 16u + 30u * r;                                     // 30 coded weights per run
        const uint32_t* q = reinterpret_cast<const uint32_t*>(idx) + (b0 >> 5);
        raw[0] = *reinterpret_cast<const uint16_t*>(idx);
        raw[1] = q[0];
        raw[2] = q[1];
    } else {
        raw[0] = 0;
    }
}

// OIL1 has no per-weight form: the caller multiplies the run's mean with the sum of the run's activations.
__device__ __forceinline__ float oil1_mean(const uint32_t (&raw)[1]) { return f16_bits(raw[0]); }

template <int FMT>
__device__ __forceinline__ void expand_run(const uint32_t (&raw)[run_raw_dwords(FMT)], const uint8_t* __restrict__ cb,
                                           uint32_t cb_bytes, uint32_t idx_bytes, uint32_t r,
                                           const DecodeTables* __restrict__ T, const LdsTables& L, float (&w)[32]) {
    static_assert(FMT != 0, "OIL1 runs are a mean, see oil1_mean");
    if constexpr (FMT == 1) {
        const uint32_t sbits = __float_as_uint(f16_bits(raw[0]));
        const uint32_t neg = ~raw[1];                                              // bit set -> weight is -scale
#pragma unroll
        for (int k = 0; k < 32; ++k)    // magnitude of the scale, sign from bit k
            w[k] = __uint_as_float((sbits & 0x7FFFFFFFu) | (((neg << (31 - k)) & 0x80000000u) ^ (sbits & 0x80000000u)));
    } else if constexpr (FMT == 2 || FMT == 3 || FMT == 4) {
        constexpr uint32_t bits = lattice_bits(FMT), period = 16u * bits;
        const uint32_t b0 = 16u + bits * (32u * r - (32u * r) / period);
        const bool last_is_slot = ((32u * (r + 1)) % period) == 0u;
        const float scale = f16_bits(raw[0]);
        const uint32_t sh = b0 & 31u;
        constexpr int per = 32 / (int)bits;                                        // weights per dword
#pragma unroll
        for (int j = 0; j < run_raw_dwords(FMT) - 2; ++j) {
            const uint32_t v = funnel(raw[1 + j], raw[2 + j], sh);
#pragma unroll
            for (int e = 0; e < per; ++e) {
                const uint32_t q = (v >> (bits * e)) & ((1u << bits) - 1u);
                w[per * j + e] = (bits == 2u ? L.lv2[q] : bits == 4u ? L.lv4[q] : L.lv8[q]) * scale;
            }
        }
        if (last_is_slot) w[31] = 0.0f;
    } else if constexpr (FMT == 9 || FMT == 10 || FMT == 11) {
        constexpr uint32_t bits = lattice_bits(FMT);
        const float zp = f16_bits(raw[0]), sc = f16_bits(raw[0] >> 16);
        constexpr int per = 32 / (int)bits;
        if (sc == 0.0f) {
#pragma unroll
            for (int k = 0; k < 32; ++k) w[k] = zp;
        } else {
#pragma unroll
            for (int j = 0; j < (int)bits; ++j) {
                const uint32_t v = raw[1 + j];
#pragma unroll
                for (int e = 0; e < per; ++e) {
                    const uint32_t q = (v >> (bits * e)) & ((1u << bits) - 1u);
                    w[per * j + e] = __fmaf_rn(bits == 2u ? L.lv2[q] : bits == 4u ? L.lv4[q] : L.t255[q], sc, zp);
                }
            }
        }
    } else if constexpr (FMT == 5 || FMT == 12) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            w[2 * j] = f16_bits(raw[j]);
            w[2 * j + 1] = f16_bits(raw[j] >> 16);
        }
    } else if constexpr (FMT == 6) {
#pragma unroll
        for (int k = 0; k < 32; ++k) w[k] = __uint_as_float(raw[k]);
    } else if constexpr (FMT == 7) {
        const float scale = f16_bits(raw[0]);
        const uint32_t v = funnel(raw[1], raw[2], (16u + 30u * r) & 31u);
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const int code = k - (k >= 15 ? 1 : 0);                                // weights 15 and 31 of a run are slots
            w[k] = (k == 15 || k == 31) ? 0.0f : (((v >> code) & 1u) ? scale : -scale);
        }
    } else {
        for (int k = 0; k < 32; ++k)
            w[k] = decode_weight((uint32_t)FMT, cb, cb_bytes, cb + cb_bytes, idx_bytes, 256u, 32u * r + (uint32_t)k, T);
    }
}

// ---- dot product of one run with MB activation rows, without expanding the weights ---------------------------------
// The lattice and grouped formats factor the per-block (per-group) scale out of the sum:
//   lattice  w = L[q] * scale        -> dot = scale * sum L[q] x
//   grouped  w = L[q] * sc + zp      -> dot = sc * sum L[q] x + zp * sum x      (sc == 0 gives zp * sum x as well)
// so the inner loop needs the bare levels only: one look-up in a 16- or 4-entry LDS table (every entry in a bank of its
// own, lanes that want the same entry share the read) and one FMA per weight.  The 8-bit levels are affine in q
// (-8 + 16 q / 255 and q / 255), so a run is sum q x plus a multiple of sum x.  Rounding differs from level * scale
// rounded per weight (src/block_codec.cpp:173-182, 308-331) in the last bits only; the bit-exact form stays with
// expand_run / decode_weight.  The two tables sit at the start of the kernel's LDS.
constexpr uint32_t kLv4Off = 0;            // 16 floats
constexpr uint32_t kLv2Off = 64;           // 4 floats
constexpr uint32_t kLevelTabBytes = 128;

typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const float lds_cf;
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void build_level_tables(float* lds0, uint32_t tid) {
    if (tid < 16u) lds0[kLv4Off / 4 + tid] = kLv4[tid];
    if (tid < 4u) lds0[kLv2Off / 4 + tid] = kLv2[tid];
}

// formats dot_run covers (the others go through expand_run)
__host__ __device__ constexpr bool has_dot_run(int fmt) {
    return fmt == 2 || fmt == 3 || fmt == 4 || fmt == 5 || fmt == 7 || fmt == 9 || fmt == 10 || fmt == 11 || fmt == 12;
}

// sum over the run of L[q_k] * x_k for a 4-bit payload: d = the run's 4 dwords, LSB-first nibbles
template <int MB>
__device__ __forceinline__ void dot_nibbles(const uint32_t (&d)[4], const f32x4_t (&xv)[MB][8], float (&s)[MB]) {
    float lv[32];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t off = e == 0 ? (d[j] << 2) & 0x3Cu : (d[j] >> (4 * e - 2)) & 0x3Cu;      // 4 * nibble e
            lv[8 * j + e] = *(lds_cf*)(uintptr_t)(kLv4Off + off);
        }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            a0 = __fmaf_rn(lv[4 * c], xv[m][c].x, a0);
            a1 = __fmaf_rn(lv[4 * c + 1], xv[m][c].y, a1);
            a0 = __fmaf_rn(lv[4 * c + 2], xv[m][c].z, a0);
            a1 = __fmaf_rn(lv[4 * c + 3], xv[m][c].w, a1);
        }
        s[m] = a0 + a1;
    }
}

// the same for a 2-bit payload: d = the run's 2 dwords
template <int MB>
__device__ __forceinline__ void dot_crumbs(const uint32_t (&d)[2], const f32x4_t (&xv)[MB][8], float (&s)[MB]) {
    float lv[32];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const uint32_t off = e == 0 ? (d[j] << 2) & 0xCu : (d[j] >> (2 * e - 2)) & 0xCu;        // 4 * field e
            lv[16 * j + e] = *(lds_cf*)(uintptr_t)(kLv2Off + off);
        }
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            a0 = __fmaf_rn(lv[4 * c], xv[m][c].x, a0);
            a1 = __fmaf_rn(lv[4 * c + 1], xv[m][c].y, a1);
            a0 = __fmaf_rn(lv[4 * c + 2], xv[m][c].z, a0);
            a1 = __fmaf_rn(lv[4 * c + 3], xv[m][c].w, a1);
        }
        s[m] = a0 + a1;
    }
}

// sum q_k * x_k for an 8-bit payload: d = the run's 8 dwords
template <int MB>
__device__ __forceinline__ void dot_bytes(const uint32_t (&d)[8], const f32x4_t (&xv)[MB][8], float (&s)[MB]) {
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        float a0 = 0.f, a1 = 0.f;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            a0 = __fmaf_rn((float)(d[c] & 0xFFu), xv[m][c].x, a0);
            a1 = __fmaf_rn((float)((d[c] >> 8) & 0xFFu), xv[m][c].y, a1);
            a0 = __fmaf_rn((float)((d[c] >> 16) & 0xFFu), xv[m][c].z, a0);
            a1 = __fmaf_rn((float)(d[c] >> 24), xv[m][c].w, a1);
        }
        s[m] = a0 + a1;
    }
}

// part[m] = dot product of the run with activation row m.  xv: the run's 32 activations per row (modified in place
// where a slot weight has to drop out), xsum: their sum per row.
template <int FMT, int MB>
__device__ __forceinline__ void dot_run(const uint32_t (&raw)[run_raw_dwords(FMT)], uint32_t r, f32x4_t (&xv)[MB][8],
                                        const float (&xsum)[MB], float (&part)[MB]) {
    static_assert(has_dot_run(FMT), "format has no closed-form run");
    if constexpr (FMT == 2 || FMT == 3 || FMT == 4) {
        constexpr uint32_t bits = lattice_bits(FMT), period = 16u * bits;
        const uint32_t sh = (16u + bits * (32u * r - (32u * r) / period)) & 31u;
        const bool last_is_slot = ((32u * (r + 1)) % period) == 0u;         // the run's last weight owns no bits: 0.0f
        const float scale = f16_bits(raw[0]);
        float x31[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            x31[m] = last_is_slot ? xv[m][7].w : 0.f;
            xv[m][7].w = last_is_slot ? 0.f : xv[m][7].w;
        }
        constexpr int ND = run_raw_dwords(FMT) - 2;
        uint32_t d[ND];
#pragma unroll
        for (int j = 0; j < ND; ++j) d[j] = funnel(raw[1 + j], raw[2 + j], sh);
        float s[MB];
        if constexpr (FMT == 3) dot_nibbles<MB>(d, xv, s);
        else if constexpr (FMT == 2) dot_crumbs<MB>(d, xv, s);
        else dot_bytes<MB>(d, xv, s);
#pragma unroll
        for (int m = 0; m < MB; ++m)    // level(q) = -8 + 16 q / 255 = (16 / 255) (q - 127.5) for the 8-bit lattice
            part[m] = FMT == 4 ? scale * (16.0f / 255.0f) * (s[m] - 127.5f * (xsum[m] - x31[m])) : scale * s[m];
    } else if constexpr (FMT == 9 || FMT == 10 || FMT == 11) {
        const float zp = f16_bits(raw[0]), sc = f16_bits(raw[0] >> 16);
        constexpr int ND = (int)lattice_bits(FMT);
        uint32_t d[ND];
#pragma unroll
        for (int j = 0; j < ND; ++j) d[j] = raw[1 + j];
        float s[MB];
        if constexpr (FMT == 10) dot_nibbles<MB>(d, xv, s);
        else if constexpr (FMT == 9) dot_crumbs<MB>(d, xv, s);
        else dot_bytes<MB>(d, xv, s);
#pragma unroll
        for (int m = 0; m < MB; ++m)
            part[m] = __fmaf_rn(FMT == 11 ? sc * (1.0f / 255.0f) : sc, s[m], zp * xsum[m]);
    } else if constexpr (FMT == 5 || FMT == 12) {                        // FP16 weights, two per dword
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            float a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const f16x2_t p0 = __builtin_bit_cast(f16x2_t, raw[2 * c]), p1 = __builtin_bit_cast(f16x2_t, raw[2 * c + 1]);
                a0 = __fmaf_rn((float)p0[0], xv[m][c].x, a0);
                a1 = __fmaf_rn((float)p0[1], xv[m][c].y, a1);
                a0 = __fmaf_rn((float)p1[0], xv[m][c].z, a0);
                a1 = __fmaf_rn((float)p1[1], xv[m][c].w, a1);
            }
            part[m] = a0 + a1;
        }
    } else {                                                             // OIL1_GRP: block scale, 30 sign bits per run
        // weights 15 and 31 of a run are slots (0.0f); weight k < 15 has bit k of the run's field, weight 16 + k bit 15 + k
        const uint32_t v = funnel(raw[1], raw[2], (16u + 30u * r) & 31u);
        const uint32_t s16 = raw[0] & 0xFFFFu, mag = s16 & 0x7FFFu;
        uint32_t mag2 = mag | (mag << 16);
        asm volatile("" : "+v"(mag2));
        const uint32_t two = (v & 0x7FFFu) | ((v >> 15) << 16);            // bit k -> low half, bit 15 + k -> high half
        const uint32_t negm = ~two ^ (0u - (s16 >> 15));
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            float a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int k = 0; k < 15; ++k) {
                const f16x2_t p = __builtin_bit_cast(f16x2_t, ((negm << (15 - k)) & 0x80008000u) | mag2);
                const float xl = k % 4 == 0 ? xv[m][k / 4].x : k % 4 == 1 ? xv[m][k / 4].y : k % 4 == 2 ? xv[m][k / 4].z : xv[m][k / 4].w;
                const float xh = k % 4 == 0 ? xv[m][4 + k / 4].x : k % 4 == 1 ? xv[m][4 + k / 4].y : k % 4 == 2 ? xv[m][4 + k / 4].z : xv[m][4 + k / 4].w;
                a0 = __fmaf_rn((float)p[0], xl, a0);
                a1 = __fmaf_rn((float)p[1], xh, a1);
            }
            part[m] = a0 + a1;
        }
    }
}

}  // namespace oilhip
