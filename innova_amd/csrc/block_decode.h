// block_decode.h -- random-access, bit-exact decode of one weight of one .oil
// block on the device.  This is the general path: every format, any block
// length, payloads of any (even truncated) size.  It reproduces
// dequantize_block_all (src/block_codec.cpp:576-720) value for value:
//   * bits past the end of the payload read as zero (BitReader::get, :108-116);
//   * lattice formats are one FP32 multiply; grouped lattice formats are one
//     fused multiply-add (the reference build contracts level*scale+zp);
//   * halves widen with the exact integer rule of f16_to_f32 (:61-84), NaN
//     payload bits included.
// The specialised GEMV/GEMM kernels use their own vectorised decoders and are
// tested against this one.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace oilhip {

// Device descriptor of one block (16 bytes).  Payload of block b starts at
// byte off16*16 of the payload buffer: cb_bytes of codebook channel followed
// immediately by idx_bytes of index channel.
struct DevBlock {
    uint32_t off16;
    uint32_t idx_bytes;
    uint32_t nw;
    uint16_t cb_bytes;
    uint8_t fmt;
    uint8_t pad;
};
static_assert(sizeof(DevBlock) == 16, "descriptor is 16 bytes");

// Lookup tables built on the host with the reference's exact expressions and
// copied to the device once (see tables.cpp).
struct DecodeTables {
    float lv8[256];     // -8 + (16*q)/255            (block_codec.cpp:131)
    float t255[256];    // q / 255                    (:326)
    float t1275[256];   // q / 127.5 - 1              (:338,349)
    float q127[256];    // (int8)q / 127              (:690,713)
};

__device__ __constant__ const float kLv2[4] = {-1.5104f, -0.4528f, 0.4528f, 1.5104f};
__device__ __constant__ const float kLv4[16] = {
    -2.7178f, -2.0522f, -1.5995f, -1.2392f, -0.9275f, -0.6508f, -0.3976f, -0.1260f,
    0.1260f,  0.3976f,  0.6508f,  0.9275f,  1.2392f,  1.5995f,  2.0522f,  2.7178f};

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
    const uint32_t s = (h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 0x3FFu;
    if (e == 31u) return __uint_as_float(s | 0x7F800000u | (m << 13));
    if (e != 0u) return __uint_as_float(s | ((e + 112u) << 23) | (m << 13));
    return __uint_as_float(s | __float_as_uint(__uint2float_rn(m) * 0x1p-24f));   // exact
}

// `count` (<= 16) bits starting at bit `pos`, LSB first; bytes >= nbytes read as 0.
__device__ __forceinline__ uint32_t bits_at(const uint8_t* __restrict__ p, uint32_t nbytes,
                                            uint64_t pos, int count) {
    const uint64_t byte = pos >> 3;
    uint32_t v = 0;
    if (byte < nbytes) v = p[byte];
    if (byte + 1 < nbytes) v |= (uint32_t)p[byte + 1] << 8;
    if (byte + 2 < nbytes) v |= (uint32_t)p[byte + 2] << 16;
    return (v >> (uint32_t)(pos & 7u)) & ((1u << count) - 1u);
}

// is_slot (block_codec.cpp:122-126) and the number of slots before index i.
__device__ __forceinline__ bool slot_at(uint64_t i, uint64_t n, uint64_t count) {
    if (count == 0 || n == 0) return false;
    return ((i + 1) * count) / n != (i * count) / n;
}
__device__ __forceinline__ uint64_t slots_before(uint64_t i, uint64_t n, uint64_t count) {
    if (count == 0 || n == 0) return 0;
    return count >= n ? i : (i * count) / n;
}

__device__ __forceinline__ float lattice_level(int bits, uint32_t q, const DecodeTables* __restrict__ T) {
    if (bits == 2) return kLv2[q & 3u];
    if (bits == 4) return kLv4[q & 15u];
    return T->lv8[q & 255u];
}

__device__ inline float decode_weight(uint32_t fmt, const uint8_t* __restrict__ cb, uint32_t cb_bytes,
                                      const uint8_t* __restrict__ idx, uint32_t idx_bytes,
                                      uint32_t nw, uint32_t i,
                                      const DecodeTables* __restrict__ T) {
    const uint32_t n = nw < (1u << 24) ? nw : (1u << 24);
    if (i >= n) return 0.0f;
    switch (fmt) {
        case 6: {  // OIL32
            if ((uint64_t)idx_bytes < (uint64_t)n * 4) return 0.0f;
            const uint8_t* q = idx + (size_t)i * 4;
            return __uint_as_float((uint32_t)q[0] | ((uint32_t)q[1] << 8) | ((uint32_t)q[2] << 16) |
                                   ((uint32_t)q[3] << 24));
        }
        case 5: case 12: {  // OIL16, OIL16_GRP
            const uint64_t o = (uint64_t)i * 2;
            if (o + 1 >= idx_bytes) return 0.0f;
            return half_bits_to_float((uint32_t)idx[o] | ((uint32_t)idx[o + 1] << 8));
        }
        case 2: case 3: case 4: {  // OIL2, OIL4, OIL8
            const int bits = fmt == 2 ? 2 : (fmt == 3 ? 4 : 8);
            const uint32_t slots = 16u / bits;
            if (slot_at(i, n, slots)) return 0.0f;
            const float scale = half_bits_to_float(bits_at(idx, idx_bytes, 0, 16));
            const uint64_t pos = 16 + (uint64_t)bits * (i - slots_before(i, n, slots));
            return lattice_level(bits, bits_at(idx, idx_bytes, pos, bits), T) * scale;
        }
        case 9: case 10: case 11: {  // OIL2_GRP, OIL4_GRP, OIL8_GRP
            const int bits = fmt == 9 ? 2 : (fmt == 10 ? 4 : 8);
            const bool wide = bits == 8;
            const uint32_t nfull = n / 64;
            const uint64_t gbits = 32 + 64 * (uint64_t)bits;
            if (nfull == 0) {
                if (n < 8) {
                    const uint32_t q = bits_at(idx, idx_bytes, (uint64_t)i * bits, bits);
                    return wide ? T->t1275[q] : lattice_level(bits, q, T);
                }
                const float sc = half_bits_to_float(bits_at(idx, idx_bytes, 0, 16));
                if (sc == 0.0f) return 0.0f;
                const uint32_t q = bits_at(idx, idx_bytes, 16 + (uint64_t)i * bits, bits);
                return (wide ? T->t1275[q] : lattice_level(bits, q, T)) * sc;
            }
            uint32_t g = i / 64;
            uint64_t pos;
            if (g < nfull) {
                pos = g * gbits + 32 + (uint64_t)(i % 64) * bits;
            } else {                                  // partial tail reuses the last full group
                pos = nfull * gbits + (uint64_t)(i - nfull * 64) * bits;
                g = nfull - 1;
            }
            const float zp = half_bits_to_float(bits_at(idx, idx_bytes, g * gbits, 16));
            const float sc = half_bits_to_float(bits_at(idx, idx_bytes, g * gbits + 16, 16));
            if (sc == 0.0f) return zp;
            const uint32_t q = bits_at(idx, idx_bytes, pos, bits);
            return __fmaf_rn(wide ? T->t255[q] : lattice_level(bits, q, T), sc, zp);
        }
        case 0: {  // OIL1: FP16 mean per run of 32, in the codebook channel
            const uint64_t o = (uint64_t)(i / 32) * 2;
            if (o + 1 >= cb_bytes) return 0.0f;
            return half_bits_to_float((uint32_t)cb[o] | ((uint32_t)cb[o + 1] << 8));
        }
        case 7: {  // OIL1_GRP
            if (n < 32) return bits_at(idx, idx_bytes, i, 1) ? 1.0f : -1.0f;
            if (slot_at(i, n, 16)) return 0.0f;
            const float scale = half_bits_to_float(bits_at(idx, idx_bytes, 0, 16));
            return bits_at(idx, idx_bytes, 16 + (i - slots_before(i, n, 16)), 1) ? scale : -scale;
        }
        case 1: {  // SPARK_Q0: per 32 weights an FP16 scale (full sub-blocks only) + 32 signs
            const uint32_t s = i / 32, j = i % 32;
            const uint64_t base = (uint64_t)s * 48;
            if ((uint64_t)s * 32 + 32 <= n) {
                const float scale = half_bits_to_float(bits_at(idx, idx_bytes, base, 16));
                return bits_at(idx, idx_bytes, base + 16 + j, 1) ? scale : -scale;
            }
            return bits_at(idx, idx_bytes, base + j, 1) ? 1.0f : -1.0f;
        }
        case 8: {  // SPARK_Q0_GRP: scale, n signs, then refinement bits
            if (n < 32) return bits_at(idx, idx_bytes, i, 1) ? 1.0f : -1.0f;
            const float scale = half_bits_to_float(bits_at(idx, idx_bytes, 0, 16));
            const uint32_t refined = n / 2 - 16;
            float mag = scale;
            if (slot_at(i, n, refined)) {
                const uint64_t rpos = 16 + (uint64_t)n + slots_before(i, n, refined);
                mag = scale * (bits_at(idx, idx_bytes, rpos, 1) ? 1.893f : 0.567f);
            }
            return bits_at(idx, idx_bytes, 16 + (uint64_t)i, 1) ? mag : -mag;
        }
        case 13: case 14: {  // SPARK_SPARSE, SPARK_SPARSE_GRP: later records win
            const bool grouped = fmt == 14;
            if (idx_bytes < (grouped ? 7u : 4u)) return 0.0f;
            float s0, s1;
            if (!grouped) {
                s0 = s1 = __uint_as_float((uint32_t)idx[0] | ((uint32_t)idx[1] << 8) |
                                          ((uint32_t)idx[2] << 16) | ((uint32_t)idx[3] << 24));
                if (s0 == 0.0f) return 0.0f;
            } else {
                s0 = half_bits_to_float((uint32_t)idx[0] | ((uint32_t)idx[1] << 8));
                s1 = half_bits_to_float((uint32_t)idx[2] | ((uint32_t)idx[3] << 8));
                if (s0 == 0.0f && s1 == 0.0f) return 0.0f;
            }
            const uint32_t records = (idx_bytes - 4) / 3;
            float v = 0.0f;
            for (uint32_t r = 0; r < records; ++r) {
                const uint8_t* rec = idx + 4 + 3 * (size_t)r;
                const uint32_t rel = (uint32_t)rec[0] | ((uint32_t)rec[1] << 8);
                if (rel == i) v = T->q127[rec[2]] * ((rel < n / 2) ? s0 : s1);
            }
            return v;
        }
        default: return 0.0f;
    }
}

}  // namespace oilhip
