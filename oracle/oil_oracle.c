/*
 * oil_oracle.c -- CPU oracle for the OIL quantized-weight matmul path.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels (tests, smoke,
 * cpu_baseline).  Nothing in the product path may link or call this file.
 *
 * Pinning status (what proves each function right):
 *   orc_f32_to_f16 / orc_f16_to_f32      exhaustive (all 65536 halves) and sampled
 *                                        floats against the compiled reference;
 *                                        golden fixture.
 *   orc_quantize_block, orc_dequantize_block
 *                                        byte/bit identity with the compiled
 *                                        reference on the committed golden
 *                                        fixture (15 formats x full and tail
 *                                        sizes) and on fresh random blocks when
 *                                        the reference build is present; the
 *                                        reference tests' own invariants
 *                                        (payload sizes, zero block, sign
 *                                        preservation, OIL32 bitwise).
 *   orc_block_gemm_*                     brute-force double dot of decoded
 *                                        weights; golden fixture made with the
 *                                        reference's dequantize_block_all.
 *   orc_oil4_gemm / orc_oil8_gemm        compiled reference (AVX2 order is
 *                                        bit-identical); identity-codebook case
 *                                        reduces to a plain matrix product.
 *   orc_gemv_*                           compiled reference built without SIMD
 *                                        flags (its scalar bodies).
 *   orc_engine_quant_gemm                compiled reference engines.
 *   orc_tl_gemm                          compiled reference (golden fixture incl.
 *                                        the shape of tests/test_protected.cpp:177-
 *                                        192); plain integer matrix product when
 *                                        no pair sum leaves int8 (brute force).
 *
 * Compile with -ffp-contract=off: fusions the reference build performs are
 * written out as fmaf()/fma() below.
 */
#define _GNU_SOURCE
#include "oil_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

/* ------------------------------------------------------------------ tables */
/* src/block_codec.cpp:14-23 */
static const float LV2[4] = { -1.5104f, -0.4528f, 0.4528f, 1.5104f };
static const float LV4[16] = {
    -2.7178f, -2.0522f, -1.5995f, -1.2392f, -0.9275f, -0.6508f, -0.3976f, -0.1260f,
     0.1260f,  0.3976f,  0.6508f,  0.9275f,  1.2392f,  1.5995f,  2.0522f,  2.7178f };

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* --------------------------------------------------------------- half <-> float */
/* src/block_codec.cpp:26-59: round to nearest even; anything with unbiased
 * exponent above 15 (NaN included) becomes infinity; magnitudes below 2^-24
 * flush to signed zero. */
uint16_t orc_f32_to_f16(float v) {
    const uint32_t u = f2u(v);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    int e = (int)((u >> 23) & 0xFFu) - 127;
    if (e > 15) return (uint16_t)(sign | 0x7C00u);
    if (e < -24) return sign;
    const uint32_t sig = (u & 0x7FFFFFu) | 0x800000u;
    const int drop = (e >= -14) ? 13 : (-e - 1);      /* bits shifted out */
    uint32_t q = sig >> drop;
    const uint32_t rem = sig & ((1u << drop) - 1u);
    const uint32_t half = 1u << (drop - 1);
    if (rem > half || (rem == half && (q & 1u))) q += 1u;
    if (e >= -14) {
        if (q >= 0x800u) { q >>= 1; e += 1; if (e > 15) return (uint16_t)(sign | 0x7C00u); }
        return (uint16_t)(sign | (uint32_t)((e + 15) << 10) | (q & 0x3FFu));
    }
    return (uint16_t)(sign | q);   /* q == 0x400 is the smallest normal */
}

/* src/block_codec.cpp:61-84 */
float orc_f16_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    const uint32_t m = h & 0x3FFu;
    if (e == 31u) return u2f(sign | 0x7F800000u | (m << 13));
    if (e != 0u) return u2f(sign | ((e + 112u) << 23) | (m << 13));
    /* zero / subnormal: m * 2^-24 is exact in binary32 */
    return u2f(sign | f2u((float)m * 0x1p-24f));
}

/* src/kernel_oil4.cpp:15-29 (identical values; NaN payloads collapse to NAN) */
float orc_flat_fp16_to_float(uint16_t h) {
    const uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 31u && m != 0u) return NAN;
    return orc_f16_to_f32(h);
}

float orc_format_bpw(int fmt) {
    switch (fmt) {
        case ORC_OIL1: case ORC_OIL1_GRP: return 1.0f;
        case ORC_SPARK_Q0: case ORC_SPARK_Q0_GRP: return 1.5f;
        case ORC_OIL2: case ORC_SPARK_SPARSE: case ORC_SPARK_SPARSE_GRP: return 2.0f;
        case ORC_OIL2_GRP: return 2.5f;
        case ORC_OIL4: return 4.0f;
        case ORC_OIL4_GRP: return 4.5f;
        case ORC_OIL8: return 8.0f;
        case ORC_OIL8_GRP: return 8.5f;
        case ORC_OIL16: case ORC_OIL16_GRP: return 16.0f;
        case ORC_OIL32: return 32.0f;
        default: return 0.0f;
    }
}

/* ------------------------------------------------------------ bit streams */
/* LSB-first fields (src/block_codec.cpp:86-118).  Bits past the end of the
 * buffer read as zero and writes past the end are dropped. */
static uint32_t bits_get(const uint8_t* p, size_t nbytes, size_t pos, int count) {
    uint32_t r = 0;
    for (int i = 0; i < count; ++i) {
        const size_t b = pos + (size_t)i;
        if ((b >> 3) >= nbytes) break;
        r |= (uint32_t)((p[b >> 3] >> (b & 7u)) & 1u) << i;
    }
    return r;
}

static void bits_put(uint8_t* p, size_t nbytes, size_t pos, uint32_t value, int count) {
    for (int i = 0; i < count; ++i) {
        const size_t b = pos + (size_t)i;
        if ((b >> 3) >= nbytes) return;
        if ((value >> i) & 1u) p[b >> 3] |= (uint8_t)(1u << (b & 7u));
    }
}

/* src/block_codec.cpp:122-126: `count` positions spread evenly over `group`. */
static int slot_at(int64_t i, int64_t group, int count) {
    if (count <= 0 || group <= 0) return 0;
    return ((i + 1) * count) / group != (i * count) / group;
}

/* src/block_codec.cpp:128-132.  8-bit: multiply, divide, add, each rounded. */
static float lattice_level(int bits, uint32_t idx) {
    if (bits == 2) return LV2[idx > 3u ? 3u : idx];
    if (bits == 4) return LV4[idx > 15u ? 15u : idx];
    if (idx > 255u) idx = 255u;
    const float num = 16.0f * (float)idx;
    const float quo = num / 255.0f;
    return -8.0f + quo;
}

/* src/block_codec.cpp:134-147: ties keep the lower index. */
static uint32_t lattice_nearest(float v, int bits) {
    if (bits == 8) {
        float c = v < 8.0f ? v : 8.0f;            /* min(8, v): NaN -> 8 as std::min does */
        c = c > -8.0f ? c : -8.0f;
        const float t = (c + 8.0f) * 255.0f;
        return (uint32_t)lroundf(t / 16.0f);
    }
    const int count = bits == 2 ? 4 : 16;
    uint32_t best = 0;
    float bd = fabsf(v - lattice_level(bits, 0));
    for (int i = 1; i < count; ++i) {
        const float d = fabsf(v - lattice_level(bits, (uint32_t)i));
        if (d < bd) { bd = d; best = (uint32_t)i; }
    }
    return best;
}

/* src/block_codec.cpp:149-154; the double product-sum is fused in the reference build. */
static float rms_of(const float* w, int n) {
    if (n <= 0) return 0.0f;
    double s = 0.0;
    for (int i = 0; i < n; ++i) s = fma((double)w[i], (double)w[i], s);
    return (float)sqrt(s / (double)n);
}

/* -------------------------------------------------------------- payload sizes */
static size_t grp_hdr_bits(int n) {
    const int nfull = n / 64;
    if (nfull == 0) return n < 8 ? 0u : 16u;
    return (size_t)nfull * 32u;
}

size_t orc_max_payload_bytes(int fmt, int n) {
    if (n <= 0) return 0;
    const size_t N = (size_t)n;
    switch (fmt) {
        case ORC_OIL32: return N * 4;
        case ORC_OIL16: case ORC_OIL16_GRP: return N * 2;
        case ORC_OIL8: return N;
        case ORC_OIL4: return (N * 4 + 7) / 8;
        case ORC_OIL2: return (N * 2 + 7) / 8;
        case ORC_OIL8_GRP: return (grp_hdr_bits(n) + N * 8 + 7) / 8;
        case ORC_OIL4_GRP: return (grp_hdr_bits(n) + N * 4 + 7) / 8;
        case ORC_OIL2_GRP: return (grp_hdr_bits(n) + N * 2 + 7) / 8;
        case ORC_OIL1: return ((N + 31) / 32) * 2;
        case ORC_OIL1_GRP: return (N + 7) / 8;
        case ORC_SPARK_Q0: return (N * 3 + 15) / 16;
        case ORC_SPARK_Q0_GRP: return n < 32 ? (N + 7) / 8 : (N * 3 + 15) / 16;
        case ORC_SPARK_SPARSE: {
            const size_t budget = N / 4;
            if (budget < 4) return 0;
            size_t keep = (budget - 4) / 3; if (keep > 20) keep = 20;
            return 4 + keep * 3;
        }
        case ORC_SPARK_SPARSE_GRP: {
            const size_t budget = N / 4;
            if (budget < 8) return 0;
            return 4 + ((budget - 4) / 3) * 3;
        }
        default: return 0;
    }
}

/* ------------------------------------------------------------------- encode */
/* src/block_codec.cpp:157-171 */
static size_t enc_lattice(const float* w, int n, int bits, uint8_t* out) {
    const size_t nbytes = ((size_t)bits * (size_t)n + 7) / 8;
    memset(out, 0, nbytes);
    const int slots = 16 / bits;
    const float scale = rms_of(w, n);
    size_t pos = 0;
    bits_put(out, nbytes, pos, orc_f32_to_f16(scale), 16); pos += 16;
    const float s = (scale <= 1e-12f) ? 0.0f : scale;
    for (int i = 0; i < n; ++i) {
        if (slot_at(i, n, slots)) continue;
        const float t = (s == 0.0f) ? 0.0f : w[i] / s;
        bits_put(out, nbytes, pos, lattice_nearest(t, bits), bits); pos += (size_t)bits;
    }
    return nbytes;
}

static uint32_t clamp255(long v) { return (uint32_t)v > 255u ? 255u : (uint32_t)v; }

/* src/block_codec.cpp:191-306 */
static size_t enc_grouped(const float* w, int n, int bits, uint8_t* out) {
    const int nfull = n / 64;
    const size_t nbytes = (grp_hdr_bits(n) + (size_t)n * (size_t)bits + 7) / 8;
    memset(out, 0, nbytes);
    size_t pos = 0;
    float pzp = 0.0f, psc = 1.0f;
    const int wide = (bits == 8);
    for (int g = 0; g < nfull; ++g) {
        const float* x = w + g * 64;
        float zp, sc;
        if (wide) {
            float lo = x[0], hi = x[0];
            for (int i = 1; i < 64; ++i) { if (x[i] < lo) lo = x[i]; if (x[i] > hi) hi = x[i]; }
            zp = lo; sc = hi - lo;
        } else {
            double mu = 0.0, ss = 0.0;
            for (int i = 0; i < 64; ++i) mu += x[i];
            mu /= 64.0;
            for (int i = 0; i < 64; ++i) { const double d = (double)x[i] - mu; ss = fma(d, d, ss); }
            zp = (float)mu;
            sc = (ss > 0.0) ? (float)sqrt(ss / 64.0) : 0.0f;
        }
        bits_put(out, nbytes, pos, orc_f32_to_f16(zp), 16); pos += 16;
        bits_put(out, nbytes, pos, orc_f32_to_f16(sc), 16); pos += 16;
        pzp = zp; psc = sc;
        if (sc == 0.0f) { pos += (size_t)64 * (size_t)bits; continue; }
        for (int i = 0; i < 64; ++i) {
            uint32_t q;
            if (wide) {
                const float t = (x[i] - zp) / sc;
                q = clamp255(lroundf(t * 255.0f));
            } else {
                q = lattice_nearest((float)(((double)x[i] - (double)zp) / (double)sc), bits);
            }
            bits_put(out, nbytes, pos, q, bits); pos += (size_t)bits;
        }
    }
    const int t0 = nfull * 64;
    if (n - t0 <= 0) return nbytes;
    if (nfull == 0) {
        if (n < 8) {                       /* headerless: implicit scale 1, zp 0 */
            for (int i = 0; i < n; ++i) {
                const uint32_t q = wide ? clamp255(lroundf((w[i] + 1.0f) * 127.5f))
                                        : lattice_nearest(w[i], bits);
                bits_put(out, nbytes, pos, q, bits); pos += (size_t)bits;
            }
            return nbytes;
        }
        float sc;                          /* scale-only header */
        if (wide) {
            sc = fabsf(w[0]);
            for (int i = 1; i < n; ++i) { const float a = fabsf(w[i]); if (sc < a) sc = a; }
        } else {
            double ss = 0.0;
            for (int i = 0; i < n; ++i) ss = fma((double)w[i], (double)w[i], ss);
            sc = (ss > 0.0) ? (float)sqrt(ss / (double)n) : 0.0f;
        }
        bits_put(out, nbytes, pos, orc_f32_to_f16(sc), 16); pos += 16;
        if (sc == 0.0f) return nbytes;
        for (int i = 0; i < n; ++i) {
            const uint32_t q = wide ? clamp255(lroundf((w[i] / sc + 1.0f) * 127.5f))
                                    : lattice_nearest(w[i] / sc, bits);
            bits_put(out, nbytes, pos, q, bits); pos += (size_t)bits;
        }
        return nbytes;
    }
    for (int i = t0; i < n; ++i) {         /* tail reuses the last full group's zp/scale */
        uint32_t q = 0;
        if (psc != 0.0f) {
            if (wide) {
                const float t = (w[i] - pzp) / psc;
                q = clamp255(lroundf(t * 255.0f));
            } else {
                q = lattice_nearest((float)(((double)w[i] - (double)pzp) / (double)psc), bits);
            }
        }
        bits_put(out, nbytes, pos, q, bits); pos += (size_t)bits;
    }
    return nbytes;
}

/* stable "k largest magnitudes first" as std::partial_sort with a > comparator
 * leaves them is NOT specified for ties; the reference uses libstdc++'s heap
 * based partial_sort, restated here so equal magnitudes land in the same order. */
typedef struct { float a; int i; } mag_t;

static void heap_sift(mag_t* h, int len, int hole, mag_t v) {
    /* libstdc++ __adjust_heap with comp(a,b) = a.a > b.a (so the heap top is the smallest) */
    const int top = hole;
    int child = hole;
    while (child < (len - 1) / 2) {
        child = 2 * (child + 1);
        if (h[child].a > h[child - 1].a) child--;
        h[hole] = h[child];
        hole = child;
    }
    if ((len & 1) == 0 && child == (len - 2) / 2) {
        child = 2 * (child + 1);
        h[hole] = h[child - 1];
        hole = child - 1;
    }
    int parent = (hole - 1) / 2;           /* __push_heap */
    while (hole > top && h[parent].a > v.a) {
        h[hole] = h[parent];
        hole = parent;
        parent = (hole - 1) / 2;
    }
    h[hole] = v;
}

static void top_k_by_magnitude(mag_t* m, int n, int k) {
    if (k <= 0) return;
    if (k > n) k = n;
    /* make_heap on [0,k) */
    if (k >= 2) {
        for (int parent = (k - 2) / 2; ; --parent) {
            mag_t v = m[parent];
            heap_sift(m, k, parent, v);
            if (parent == 0) break;
        }
    }
    /* heap_select: anything after k that beats the top replaces it */
    for (int i = k; i < n; ++i) {
        if (m[i].a > m[0].a) {
            mag_t v = m[i];
            m[i] = m[0];
            heap_sift(m, k, 0, v);
        }
    }
    /* sort_heap */
    for (int last = k - 1; last > 0; --last) {
        mag_t v = m[last];
        m[last] = m[0];
        heap_sift(m, last, 0, v);
    }
}

int orc_quantize_block(int fmt, const float* w, int n,
                       uint8_t* idx, size_t idx_cap, size_t* idx_len,
                       uint8_t* cb, size_t cb_cap, size_t* cb_len) {
    if (idx_len) *idx_len = 0;
    if (cb_len) *cb_len = 0;
    if (!w || n <= 0 || !idx_len || !cb_len) return 0;
    if (fmt < 0 || fmt >= ORC_NUM_FORMATS) return 0;
    const size_t need = orc_max_payload_bytes(fmt, n);
    if (fmt == ORC_OIL1) { if (cb_cap < need || !cb) return 0; }
    else if (need > 0 && (idx_cap < need || !idx)) return 0;

    switch (fmt) {
        case ORC_OIL32:
            memcpy(idx, w, (size_t)n * 4); *idx_len = (size_t)n * 4; return 1;
        case ORC_OIL16: case ORC_OIL16_GRP:
            for (int i = 0; i < n; ++i) {
                const uint16_t h = orc_f32_to_f16(w[i]);
                idx[2 * i] = (uint8_t)(h & 0xFF); idx[2 * i + 1] = (uint8_t)(h >> 8);
            }
            *idx_len = (size_t)n * 2; return 1;
        case ORC_OIL8: *idx_len = enc_lattice(w, n, 8, idx); return 1;
        case ORC_OIL4: *idx_len = enc_lattice(w, n, 4, idx); return 1;
        case ORC_OIL2: *idx_len = enc_lattice(w, n, 2, idx); return 1;
        case ORC_OIL8_GRP: *idx_len = enc_grouped(w, n, 8, idx); return 1;
        case ORC_OIL4_GRP: *idx_len = enc_grouped(w, n, 4, idx); return 1;
        case ORC_OIL2_GRP: *idx_len = enc_grouped(w, n, 2, idx); return 1;
        case ORC_OIL1: {                              /* :406-420 */
            const int runs = (n + 31) / 32;
            for (int r = 0; r < runs; ++r) {
                const int a = r * 32, b = (a + 32 < n) ? a + 32 : n;
                double s = 0.0;
                for (int i = a; i < b; ++i) s += w[i];
                const uint16_t h = orc_f32_to_f16((float)(s / (double)(b - a)));
                cb[2 * r] = (uint8_t)(h & 0xFF); cb[2 * r + 1] = (uint8_t)(h >> 8);
            }
            *cb_len = (size_t)runs * 2; return 1;
        }
        case ORC_OIL1_GRP: {                          /* :421-443 */
            const size_t nb = ((size_t)n + 7) / 8;
            memset(idx, 0, nb);
            size_t pos = 0;
            if (n >= 32) { bits_put(idx, nb, 0, orc_f32_to_f16(rms_of(w, n)), 16); pos = 16; }
            for (int i = 0; i < n; ++i) {
                if (n >= 32 && slot_at(i, n, 16)) continue;
                bits_put(idx, nb, pos, w[i] >= 0.0f ? 1u : 0u, 1); pos++;
            }
            *idx_len = nb; return 1;
        }
        case ORC_SPARK_Q0: {                          /* :444-458 */
            const size_t nb = ((size_t)n * 3 + 15) / 16;
            memset(idx, 0, nb);
            size_t pos = 0;
            for (int a = 0; a < n; a += 32) {
                const int b = (a + 32 < n) ? a + 32 : n;
                if (b - a == 32) { bits_put(idx, nb, pos, orc_f32_to_f16(rms_of(w + a, 32)), 16); pos += 16; }
                for (int i = a; i < b; ++i) { bits_put(idx, nb, pos, w[i] >= 0.0f ? 1u : 0u, 1); pos++; }
            }
            *idx_len = nb; return 1;
        }
        case ORC_SPARK_Q0_GRP: {                      /* :459-483 */
            if (n < 32) {
                const size_t nb = ((size_t)n + 7) / 8;
                memset(idx, 0, nb);
                for (int i = 0; i < n; ++i) bits_put(idx, nb, (size_t)i, w[i] >= 0.0f ? 1u : 0u, 1);
                *idx_len = nb; return 1;
            }
            const size_t nb = ((size_t)n * 3 + 15) / 16;
            memset(idx, 0, nb);
            const float scale = rms_of(w, n);
            size_t pos = 0;
            bits_put(idx, nb, pos, orc_f32_to_f16(scale), 16); pos += 16;
            for (int i = 0; i < n; ++i) { bits_put(idx, nb, pos, w[i] >= 0.0f ? 1u : 0u, 1); pos++; }
            const int refined = (n / 2 - 16) > 0 ? (n / 2 - 16) : 0;
            const float thr = scale * 1.23f;
            for (int i = 0; i < n; ++i) {
                if (!slot_at(i, n, refined)) continue;
                bits_put(idx, nb, pos, fabsf(w[i]) > thr ? 1u : 0u, 1); pos++;
            }
            *idx_len = nb; return 1;
        }
        case ORC_SPARK_SPARSE: case ORC_SPARK_SPARSE_GRP: {   /* :484-570 */
            const int grouped = (fmt == ORC_SPARK_SPARSE_GRP);
            const size_t budget = (size_t)n / 4;
            if (budget < (grouped ? 8u : 4u)) return 1;
            int keep = (int)((budget - 4) / 3);
            if (!grouped && keep > 20) keep = 20;
            if (grouped && keep <= 0) return 1;
            const int half = n / 2;
            mag_t* m = (mag_t*)malloc(sizeof(mag_t) * (size_t)n);
            if (!m) return 0;
            float s0 = 0.0f, s1 = 0.0f;
            for (int i = 0; i < n; ++i) {
                const float a = fabsf(w[i]);
                m[i].a = a; m[i].i = i;
                if (!grouped || i < half) { if (s0 < a) s0 = a; } else { if (s1 < a) s1 = a; }
            }
            if (!grouped) {
                if (s0 <= 1e-12f) { memset(idx, 0, 4); *idx_len = 4; free(m); return 1; }
            } else {
                if (s0 <= 1e-12f) s0 = 1.0f;
                if (s1 <= 1e-12f) s1 = 1.0f;
            }
            if (keep > 0) top_k_by_magnitude(m, n, keep);
            if (!grouped) {
                const uint32_t sb = f2u(s0);
                idx[0] = (uint8_t)sb; idx[1] = (uint8_t)(sb >> 8);
                idx[2] = (uint8_t)(sb >> 16); idx[3] = (uint8_t)(sb >> 24);
            } else {
                const uint16_t h0 = orc_f32_to_f16(s0), h1 = orc_f32_to_f16(s1);
                idx[0] = (uint8_t)h0; idx[1] = (uint8_t)(h0 >> 8);
                idx[2] = (uint8_t)h1; idx[3] = (uint8_t)(h1 >> 8);
            }
            for (int r = 0; r < keep; ++r) {
                const int at = m[r].i;
                const float s = (!grouped || at < half) ? s0 : s1;
                long q = lroundf(w[at] / s * 127.0f);
                if (q < -127) q = -127;
                if (q > 127) q = 127;
                uint8_t* rec = idx + 4 + 3 * (size_t)r;
                rec[0] = (uint8_t)(at & 0xFF); rec[1] = (uint8_t)((at >> 8) & 0xFF);
                rec[2] = (uint8_t)(int8_t)q;
            }
            *idx_len = 4 + 3 * (size_t)keep;
            free(m);
            return 1;
        }
        default: return 0;
    }
}

/* ------------------------------------------------------------------- decode */
/* src/block_codec.cpp:173-182 */
static void dec_lattice(const uint8_t* p, size_t nb, int n, int bits, float* out) {
    const int slots = 16 / bits;
    const float scale = orc_f16_to_f32((uint16_t)bits_get(p, nb, 0, 16));
    size_t pos = 16;
    for (int i = 0; i < n; ++i) {
        if (slot_at(i, n, slots)) { out[i] = 0.0f; continue; }
        const uint32_t q = bits_get(p, nb, pos, bits); pos += (size_t)bits;
        out[i] = lattice_level(bits, q) * scale;
    }
}

/* src/block_codec.cpp:308-364; level*scale+zp is a single fused operation in
 * the reference build, as is zp + t*scale for the 8-bit form. */
static void dec_grouped(const uint8_t* p, size_t nb, int bits, int n, float* out) {
    const int nfull = n / 64;
    const int wide = (bits == 8);
    size_t pos = 0;
    float pzp = 0.0f, psc = 1.0f;
    for (int g = 0; g < nfull; ++g) {
        const float zp = orc_f16_to_f32((uint16_t)bits_get(p, nb, pos, 16)); pos += 16;
        const float sc = orc_f16_to_f32((uint16_t)bits_get(p, nb, pos, 16)); pos += 16;
        pzp = zp; psc = sc;
        float* o = out + g * 64;
        for (int i = 0; i < 64; ++i) {
            const uint32_t q = bits_get(p, nb, pos, bits); pos += (size_t)bits;
            if (sc == 0.0f) o[i] = zp;
            else if (wide) o[i] = fmaf((float)q / 255.0f, sc, zp);
            else o[i] = fmaf(lattice_level(bits, q), sc, zp);
        }
    }
    const int t0 = nfull * 64;
    if (n - t0 <= 0) return;
    if (nfull == 0) {
        if (n < 8) {
            for (int i = 0; i < n; ++i) {
                const uint32_t q = bits_get(p, nb, pos, bits); pos += (size_t)bits;
                out[i] = wide ? ((float)q / 127.5f - 1.0f) : lattice_level(bits, q);
            }
            return;
        }
        const float sc = orc_f16_to_f32((uint16_t)bits_get(p, nb, pos, 16)); pos += 16;
        for (int i = 0; i < n; ++i) {
            const uint32_t q = bits_get(p, nb, pos, bits); pos += (size_t)bits;
            if (sc == 0.0f) out[i] = 0.0f;
            else out[i] = wide ? ((float)q / 127.5f - 1.0f) * sc : lattice_level(bits, q) * sc;
        }
        return;
    }
    for (int i = t0; i < n; ++i) {
        const uint32_t q = bits_get(p, nb, pos, bits); pos += (size_t)bits;
        if (psc == 0.0f) out[i] = pzp;
        else if (wide) out[i] = fmaf((float)q / 255.0f, psc, pzp);
        else out[i] = fmaf(lattice_level(bits, q), psc, pzp);
    }
}

void orc_dequantize_block(int fmt, const uint8_t* idx, size_t idx_bytes,
                          const uint8_t* cb, size_t cb_bytes,
                          uint32_t nw, float* out) {
    if (!out || nw == 0) return;
    for (uint32_t i = 0; i < nw; ++i) out[i] = 0.0f;
    const int n = (int)(nw < (1u << 24) ? nw : (1u << 24));
    switch (fmt) {
        case ORC_OIL32:
            if (idx_bytes >= (size_t)n * 4) memcpy(out, idx, (size_t)n * 4);
            return;
        case ORC_OIL16: case ORC_OIL16_GRP:
            for (int i = 0; i < n; ++i) {
                const size_t o = (size_t)i * 2;
                if (o + 1 >= idx_bytes) break;
                out[i] = orc_f16_to_f32((uint16_t)(idx[o] | (idx[o + 1] << 8)));
            }
            return;
        case ORC_OIL8: dec_lattice(idx, idx_bytes, n, 8, out); return;
        case ORC_OIL4: dec_lattice(idx, idx_bytes, n, 4, out); return;
        case ORC_OIL2: dec_lattice(idx, idx_bytes, n, 2, out); return;
        case ORC_OIL8_GRP: dec_grouped(idx, idx_bytes, 8, n, out); return;
        case ORC_OIL4_GRP: dec_grouped(idx, idx_bytes, 4, n, out); return;
        case ORC_OIL2_GRP: dec_grouped(idx, idx_bytes, 2, n, out); return;
        case ORC_OIL1:                                 /* :615-626 */
            for (int r = 0; r * 32 < n; ++r) {
                const size_t o = (size_t)r * 2;
                if (o + 1 >= cb_bytes) break;
                const float mean = orc_f16_to_f32((uint16_t)(cb[o] | (cb[o + 1] << 8)));
                const int a = r * 32, b = (a + 32 < n) ? a + 32 : n;
                for (int i = a; i < b; ++i) out[i] = mean;
            }
            return;
        case ORC_OIL1_GRP: {                           /* :627-642 */
            if (n < 32) {
                for (int i = 0; i < n; ++i)
                    out[i] = bits_get(idx, idx_bytes, (size_t)i, 1) ? 1.0f : -1.0f;
                return;
            }
            const float scale = orc_f16_to_f32((uint16_t)bits_get(idx, idx_bytes, 0, 16));
            size_t pos = 16;
            for (int i = 0; i < n; ++i) {
                if (slot_at(i, n, 16)) { out[i] = 0.0f; continue; }
                out[i] = bits_get(idx, idx_bytes, pos++, 1) ? scale : -scale;
            }
            return;
        }
        case ORC_SPARK_Q0: {                           /* :643-654 */
            size_t pos = 0;
            for (int a = 0; a < n; a += 32) {
                const int b = (a + 32 < n) ? a + 32 : n;
                float scale = 1.0f;
                if (b - a == 32) { scale = orc_f16_to_f32((uint16_t)bits_get(idx, idx_bytes, pos, 16)); pos += 16; }
                for (int i = a; i < b; ++i)
                    out[i] = bits_get(idx, idx_bytes, pos++, 1) ? scale : -scale;
            }
            return;
        }
        case ORC_SPARK_Q0_GRP: {                       /* :655-676 */
            if (n < 32) {
                for (int i = 0; i < n; ++i)
                    out[i] = bits_get(idx, idx_bytes, (size_t)i, 1) ? 1.0f : -1.0f;
                return;
            }
            const float scale = orc_f16_to_f32((uint16_t)bits_get(idx, idx_bytes, 0, 16));
            const int refined = (n / 2 - 16) > 0 ? (n / 2 - 16) : 0;
            size_t rpos = 16 + (size_t)n;              /* refinement bits follow all signs */
            for (int i = 0; i < n; ++i) {
                float mag = scale;
                if (slot_at(i, n, refined))
                    mag = scale * (bits_get(idx, idx_bytes, rpos++, 1) ? 1.893f : 0.567f);
                out[i] = bits_get(idx, idx_bytes, 16 + (size_t)i, 1) ? mag : -mag;
            }
            return;
        }
        case ORC_SPARK_SPARSE: case ORC_SPARK_SPARSE_GRP: {   /* :677-716 */
            const int grouped = (fmt == ORC_SPARK_SPARSE_GRP);
            if (idx_bytes < (grouped ? 7u : 4u)) return;
            float s0, s1;
            if (!grouped) {
                s0 = s1 = u2f((uint32_t)idx[0] | ((uint32_t)idx[1] << 8) |
                              ((uint32_t)idx[2] << 16) | ((uint32_t)idx[3] << 24));
                if (s0 == 0.0f) return;
            } else {
                s0 = orc_f16_to_f32((uint16_t)(idx[0] | (idx[1] << 8)));
                s1 = orc_f16_to_f32((uint16_t)(idx[2] | (idx[3] << 8)));
                if (s0 == 0.0f && s1 == 0.0f) return;
            }
            const size_t records = (idx_bytes - 4) / 3;
            const int half = n / 2;
            for (size_t r = 0; r < records; ++r) {
                const uint8_t* rec = idx + 4 + 3 * r;
                const uint32_t rel = (uint32_t)rec[0] | ((uint32_t)rec[1] << 8);
                const float qf = (float)(int8_t)rec[2] / 127.0f;
                if (rel < (uint32_t)n) out[rel] = qf * (((int)rel < half) ? s0 : s1);
            }
            return;
        }
        default: return;
    }
}

/* ------------------------------------------------------------ tensor encode */
typedef struct {
    const uint8_t* fmts; const float* w; uint64_t numel; uint32_t b0, b1;
    uint8_t* tmp; size_t stride; uint32_t* ilen; uint32_t* clen; int ok;
} qjob_t;

static void* quant_worker(void* arg) {
    qjob_t* j = (qjob_t*)arg;
    for (uint32_t b = j->b0; b < j->b1; ++b) {
        const uint64_t at = (uint64_t)b * 256;
        const int n = (int)((j->numel - at) < 256 ? (j->numel - at) : 256);
        uint8_t* slot = j->tmp + (size_t)b * j->stride;
        size_t il = 0, cl = 0;
        /* codebook channel first in the slot, index channel after it */
        uint8_t cbuf[32];
        if (!orc_quantize_block(j->fmts[b], j->w + at, n, slot + 32, j->stride - 32, &il,
                                cbuf, sizeof cbuf, &cl)) { j->ok = 0; return NULL; }
        memcpy(slot, cbuf, cl);
        j->ilen[b] = (uint32_t)il; j->clen[b] = (uint32_t)cl;
    }
    return NULL;
}

uint64_t orc_quantize_tensor(const uint8_t* fmts, uint32_t nblocks,
                             const float* w, uint64_t numel, uint32_t align,
                             uint8_t* payload, uint64_t cap, orc_block_t* blocks,
                             int threads) {
    if (!fmts || !w || nblocks == 0 || align == 0) return 0;
    if ((uint64_t)nblocks * 256 < numel || (uint64_t)(nblocks - 1) * 256 >= numel) return 0;
    size_t stride = 0; uint64_t bound = 0;
    for (uint32_t b = 0; b < nblocks; ++b) {
        if (fmts[b] >= ORC_NUM_FORMATS) return 0;
        const size_t m = orc_max_payload_bytes(fmts[b], 256);
        if (m > stride) stride = m;
        bound += (m + align - 1) / align * align;
    }
    if (!payload) return bound;
    if (!blocks) return 0;
    stride += 32;
    uint8_t* tmp = (uint8_t*)malloc((size_t)nblocks * stride);
    uint32_t* ilen = (uint32_t*)malloc(sizeof(uint32_t) * nblocks);
    uint32_t* clen = (uint32_t*)malloc(sizeof(uint32_t) * nblocks);
    if (!tmp || !ilen || !clen) { free(tmp); free(ilen); free(clen); return 0; }
    if (threads <= 0) { long hc = sysconf(_SC_NPROCESSORS_ONLN); threads = hc < 1 ? 1 : (hc > 16 ? 16 : (int)hc); }
    if (threads > 64) threads = 64;
    if ((uint32_t)threads > nblocks) threads = (int)nblocks;
    pthread_t tid[64]; qjob_t job[64];
    const uint32_t chunk = (nblocks + (uint32_t)threads - 1) / (uint32_t)threads;
    int started = 0;
    for (int t = 0; t < threads; ++t) {
        const uint32_t b0 = (uint32_t)t * chunk, b1 = b0 + chunk < nblocks ? b0 + chunk : nblocks;
        if (b0 >= b1) continue;
        job[started] = (qjob_t){ fmts, w, numel, b0, b1, tmp, stride, ilen, clen, 1 };
        pthread_create(&tid[started], NULL, quant_worker, &job[started]);
        started++;
    }
    int ok = 1;
    for (int t = 0; t < started; ++t) { pthread_join(tid[t], NULL); ok &= job[t].ok; }
    uint64_t off = 0;
    for (uint32_t b = 0; ok && b < nblocks; ++b) {
        off = (off + align - 1) / align * align;
        const uint64_t at = (uint64_t)b * 256;
        if (off + clen[b] + ilen[b] > cap) { ok = 0; break; }
        const uint8_t* slot = tmp + (size_t)b * stride;
        memcpy(payload + off, slot, clen[b]);
        memcpy(payload + off + clen[b], slot + 32, ilen[b]);
        blocks[b].cb_off = off; blocks[b].idx_off = off + clen[b];
        blocks[b].cb_bytes = clen[b]; blocks[b].idx_bytes = ilen[b];
        blocks[b].nw = (uint32_t)((numel - at) < 256 ? (numel - at) : 256);
        blocks[b].fmt = fmts[b]; memset(blocks[b].pad_, 0, 3);
        off += clen[b] + ilen[b];
    }
    free(tmp); free(ilen); free(clen);
    return ok ? off : 0;
}

/* ------------------------------------------------------- block-decode consumer */
void orc_dequant_blocks(const uint8_t* payload, const orc_block_t* blocks,
                        uint32_t nblocks, float* out) {
    for (uint32_t b = 0; b < nblocks; ++b) {
        const orc_block_t* d = &blocks[b];
        orc_dequantize_block(d->fmt, payload + d->idx_off, d->idx_bytes,
                             payload + d->cb_off, d->cb_bytes, d->nw, out);
        out += d->nw;
    }
}

typedef struct {
    const uint8_t* payload; const orc_block_t* blocks;
    uint32_t rows, cols; const float* X; float* Y; int B; int wide;
    uint32_t r0, r1;
} gemm_job_t;

static void* gemm_worker(void* arg) {
    gemm_job_t* j = (gemm_job_t*)arg;
    const uint32_t bpr = j->cols / 256;
    float sc[256];
    float* accf = (float*)calloc((size_t)j->B, sizeof(float));
    double* accd = (double*)calloc((size_t)j->B, sizeof(double));
    for (uint32_t r = j->r0; r < j->r1; ++r) {
        for (int b = 0; b < j->B; ++b) { accf[b] = 0.0f; accd[b] = 0.0; }
        for (uint32_t k = 0; k < bpr; ++k) {
            const orc_block_t* d = &j->blocks[(size_t)r * bpr + k];
            for (int i = 0; i < 256; ++i) sc[i] = 0.0f;       /* qwen35_engine.cpp:18 */
            orc_dequantize_block(d->fmt, j->payload + d->idx_off, d->idx_bytes,
                                 j->payload + d->cb_off, d->cb_bytes, 256, sc);
            for (int b = 0; b < j->B; ++b) {
                const float* x = j->X + (size_t)b * j->cols + (size_t)k * 256;
                if (j->wide) {
                    double a = 0.0;
                    for (int i = 0; i < 256; ++i) a += (double)sc[i] * (double)x[i];
                    accd[b] += a;
                } else {
                    float a = 0.0f;
                    for (int i = 0; i < 256; ++i) a = fmaf(sc[i], x[i], a);
                    accf[b] += a;
                }
            }
        }
        for (int b = 0; b < j->B; ++b)
            j->Y[(size_t)b * j->rows + r] = j->wide ? (float)accd[b] : accf[b];
    }
    free(accf); free(accd);
    return NULL;
}

static void block_gemm(const uint8_t* payload, const orc_block_t* blocks,
                       uint32_t rows, uint32_t cols, const float* X, float* Y,
                       int B, int threads, int wide) {
    if (threads <= 0) {
        long hc = sysconf(_SC_NPROCESSORS_ONLN);
        threads = hc < 1 ? 1 : (hc > 8 ? 8 : (int)hc);
    }
    if (threads > 64) threads = 64;
    if ((uint32_t)threads > rows) threads = rows ? (int)rows : 1;
    const uint32_t chunk = (rows + (uint32_t)threads - 1) / (uint32_t)threads;
    pthread_t tid[64]; gemm_job_t job[64];
    int started = 0;
    for (int t = 0; t < threads; ++t) {
        const uint32_t r0 = (uint32_t)t * chunk;
        const uint32_t r1 = r0 + chunk < rows ? r0 + chunk : rows;
        if (r0 >= r1) continue;
        job[started] = (gemm_job_t){ payload, blocks, rows, cols, X, Y, B, wide, r0, r1 };
        if (threads == 1) { gemm_worker(&job[started]); return; }
        pthread_create(&tid[started], NULL, gemm_worker, &job[started]);
        started++;
    }
    for (int t = 0; t < started; ++t) pthread_join(tid[t], NULL);
}

void orc_block_gemm_f32(const uint8_t* payload, const orc_block_t* blocks,
                        uint32_t rows, uint32_t cols, const float* X, float* Y,
                        int B, int threads) {
    block_gemm(payload, blocks, rows, cols, X, Y, B, threads, 0);
}

void orc_block_gemm_f64(const uint8_t* payload, const orc_block_t* blocks,
                        uint32_t rows, uint32_t cols, const float* X, float* Y,
                        int B, int threads) {
    block_gemm(payload, blocks, rows, cols, X, Y, B, threads, 1);
}

/* ------------------------------------------------------------- flat kernels */
/* The AVX2 paths keep 8 lane accumulators, fold lanes (l, l+4), then hadd
 * twice: ((a0+a4)+(a1+a5)) + ((a2+a6)+(a3+a7)); a scalar tail follows. */
static float fold8(const float a[8]) {
    const float s0 = a[0] + a[4], s1 = a[1] + a[5], s2 = a[2] + a[6], s3 = a[3] + a[7];
    return (s0 + s1) + (s2 + s3);
}

void orc_oil8_gemm(const uint8_t* idx, const float* cb, const float* act,
                   float* out, int M, int N, int K, int order) {
    for (int m = 0; m < M; ++m) {
        const float* a = act + (int64_t)m * K;
        for (int n = 0; n < N; ++n) {
            const uint8_t* w = idx + (int64_t)n * K;
            float r;
            if (order == 2) {
                double s = 0.0;
                for (int k = 0; k < K; ++k) s += (double)cb[w[k]] * (double)a[k];
                r = (float)s;
            } else if (order == 1) {
                float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                int k = 0;
                for (; k + 8 <= K; k += 8)
                    for (int l = 0; l < 8; ++l) acc[l] = fmaf(cb[w[k + l]], a[k + l], acc[l]);
                r = fold8(acc);
                for (; k < K; ++k) r = fmaf(cb[w[k]], a[k], r);
            } else {
                r = 0.0f;
                for (int k = 0; k < K; ++k) r = fmaf(cb[w[k]], a[k], r);
            }
            out[(int64_t)m * N + n] = r;
        }
    }
}

static inline unsigned nib_at(const uint8_t* row, int k) {
    return (k & 1) ? (row[k >> 1] >> 4) & 0xFu : row[k >> 1] & 0xFu;
}

void orc_oil4_gemm(const uint8_t* packed, const uint16_t* cb16, const float* act,
                   float* out, int M, int N, int K, int order) {
    float c[16];
    for (int i = 0; i < 16; ++i) c[i] = orc_flat_fp16_to_float(cb16[i]);
    for (int m = 0; m < M; ++m) {
        for (int n = 0; n < N; ++n) {
            const uint8_t* w = packed + ((int64_t)m * N + n) * K / 2;
            const float* a = act + (int64_t)n * K;
            float r;
            if (order == 2) {
                double s = 0.0;
                for (int k = 0; k < K; ++k) s += (double)c[nib_at(w, k)] * (double)a[k];
                r = (float)s;
            } else if (order == 1) {
                float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                int k = 0;
                for (; k + 16 <= K; k += 16) {
                    for (int l = 0; l < 8; ++l) acc[l] = fmaf(c[nib_at(w, k + l)], a[k + l], acc[l]);
                    for (int l = 0; l < 8; ++l) acc[l] = fmaf(c[nib_at(w, k + 8 + l)], a[k + 8 + l], acc[l]);
                }
                r = fold8(acc);
                for (; k < K; ++k) r = fmaf(c[nib_at(w, k)], a[k], r);
            } else {
                r = 0.0f;
                for (int k = 0; k < K; ++k) r = fmaf(c[nib_at(w, k)], a[k], r);
            }
            out[(int64_t)m * N + n] = r;
        }
    }
}

/* --------------------------------------------------------- production GEMVs */
static inline float mac(float v, float x, float s, int mode) {
    if (mode == 2) { const float p = v * x; return s + p; }
    return fmaf(v, x, s);
}

void orc_gemv_spark(const uint8_t* w, float scale, const float* x, float* y,
                    int M, int K, int mode) {
    const int as_double = (mode == 1);
    const int stride = (K + 3) / 4;
    for (int m = 0; m < M; ++m) {
        const uint8_t* row = w + (int64_t)m * stride;
        float sf = 0.0f; double sd = 0.0;
        for (int k = 0; k < K; ++k) {
            const int code = (row[k >> 2] >> ((k & 3) * 2)) & 3;
            const float v = code == 0 ? -1.0f : (code == 1 ? 0.0f : 1.0f);
            if (as_double) sd += (double)v * (double)x[k]; else sf = mac(v, x[k], sf, mode);
        }
        y[m] = as_double ? (float)(sd * (double)scale) : sf * scale;
    }
}

void orc_gemv_oil4(const uint8_t* w, const uint16_t* cb16, float scale,
                   const float* x, float* y, int M, int K, int mode) {
    const int as_double = (mode == 1);
    float c[16];
    for (int i = 0; i < 16; ++i) c[i] = orc_flat_fp16_to_float(cb16[i]);
    const int stride = (K + 1) / 2;
    for (int m = 0; m < M; ++m) {
        const uint8_t* row = w + (int64_t)m * stride;
        float sf = 0.0f; double sd = 0.0;
        for (int k = 0; k < K; ++k) {
            const float v = c[nib_at(row, k)];
            if (as_double) sd += (double)v * (double)x[k]; else sf = mac(v, x[k], sf, mode);
        }
        y[m] = as_double ? (float)(sd * (double)scale) : sf * scale;
    }
}

void orc_gemv_oil8(const uint8_t* w, const float* cb, float scale,
                   const float* x, float* y, int M, int K, int mode) {
    const int as_double = (mode == 1);
    for (int m = 0; m < M; ++m) {
        const uint8_t* row = w + (int64_t)m * K;
        float sf = 0.0f; double sd = 0.0;
        for (int k = 0; k < K; ++k) {
            const float v = cb[row[k]];
            if (as_double) sd += (double)v * (double)x[k]; else sf = mac(v, x[k], sf, mode);
        }
        y[m] = as_double ? (float)(sd * (double)scale) : sf * scale;
    }
}

/* ------------------------------------------------------------ engine layout */
void orc_engine_quant_gemm(int bits, const float* A, const uint8_t* b_idx,
                           const float* cb, float* C,
                           int64_t M, int64_t N, int64_t K, int as_double) {
    const int per = 8 / bits;                 /* codes per byte */
    const unsigned mask = (1u << bits) - 1u;
    double* acc = as_double ? (double*)calloc((size_t)N, sizeof(double)) : NULL;
    for (int64_t m = 0; m < M; ++m) {
        float* c = C + m * N;
        for (int64_t n = 0; n < N; ++n) c[n] = 0.0f;
        if (acc) for (int64_t n = 0; n < N; ++n) acc[n] = 0.0;
        for (int64_t k = 0; k < K; ++k) {
            const float a = A[m * K + k];
            if (a == 0.0f) continue;
            for (int64_t n = 0; n < N; ++n) {
                const int64_t flat = k * N + n;
                unsigned code = (b_idx[flat / per] >> ((flat % per) * bits)) & mask;
                if (bits == 4 && code >= 16u) code = 0;
                if (acc) acc[n] += (double)a * (double)cb[code];
                else c[n] = fmaf(a, cb[code], c[n]);
            }
        }
        if (acc) for (int64_t n = 0; n < N; ++n) c[n] = (float)acc[n];
    }
    free(acc);
}

/* ------------------------------------------------------------------ mixture of experts */
void orc_softmax_topk(const float* logits, int64_t T, int64_t E, int64_t k,
                      float* probs, int64_t* indices, float* weights) {
    mag_t* sc = (mag_t*)malloc((size_t)E * sizeof(mag_t));
    for (int64_t t = 0; t < T; ++t) {
        const float* l = logits + t * E;
        float* p = probs + t * E;
        float maxv = l[0];
        for (int64_t e = 1; e < E; ++e) if (l[e] > maxv) maxv = l[e];
        float sum = 0.0f;
        for (int64_t e = 0; e < E; ++e) { const float v = expf(l[e] - maxv); p[e] = v; sum += v; }
        const float inv = 1.0f / sum;
        for (int64_t e = 0; e < E; ++e) p[e] *= inv;
        for (int64_t e = 0; e < E; ++e) { sc[e].a = p[e]; sc[e].i = (int)e; }
        top_k_by_magnitude(sc, (int)E, (int)k);
        for (int64_t j = 0; j < k; ++j) { indices[t * k + j] = sc[j].i; weights[t * k + j] = sc[j].a; }
    }
    free(sc);
}

/* Y[nt][N] = X[nt][Kd] W[N][Kd]^T */
static void moe_matmul(const float* X, const float* W, float* Y, int64_t nt, int64_t N, int64_t Kd, int as_double) {
    for (int64_t m = 0; m < nt; ++m)
        for (int64_t n = 0; n < N; ++n) {
            const float* xr = X + m * Kd;
            const float* wr = W + n * Kd;
            if (as_double) {
                double acc = 0.0;
                for (int64_t k = 0; k < Kd; ++k) acc += (double)xr[k] * (double)wr[k];
                Y[m * N + n] = (float)acc;
            } else {
                float acc = 0.0f;
                for (int64_t k = 0; k < Kd; ++k) acc = fmaf(xr[k], wr[k], acc);
                Y[m * N + n] = acc;
            }
        }
}

void orc_moe_dispatch(const float* x, const float* const* gate, const float* const* up,
                      const float* const* down, const int64_t* indices, const float* weights,
                      int64_t T, int64_t K, int64_t E, int64_t D, int64_t F,
                      float* out, float* z_loss, int64_t* dropped, int as_double) {
    double* wide = as_double ? (double*)calloc((size_t)(T * D), sizeof(double)) : NULL;
    memset(out, 0, (size_t)(T * D) * sizeof(float));
    float zl = 0.0f;
    int64_t drop = 0;
    int64_t* toks = (int64_t*)malloc((size_t)(T * K + 1) * sizeof(int64_t));
    for (int64_t e = 0; e < E; ++e) {
        int64_t nt = 0;
        for (int64_t t = 0; t < T; ++t)
            for (int64_t k = 0; k < K; ++k)
                if (indices[t * K + k] == e) toks[nt++] = t;
        if (nt == 0) continue;
        float* bi = (float*)malloc((size_t)(nt * D) * sizeof(float));
        float* g = (float*)malloc((size_t)(nt * F) * sizeof(float));
        float* u = (float*)malloc((size_t)(nt * F) * sizeof(float));
        float* bo = (float*)malloc((size_t)(nt * D) * sizeof(float));
        for (int64_t i = 0; i < nt; ++i) memcpy(bi + i * D, x + toks[i] * D, (size_t)D * sizeof(float));
        moe_matmul(bi, gate[e], g, nt, F, D, as_double);
        moe_matmul(bi, up[e], u, nt, F, D, as_double);
        for (int64_t i = 0; i < nt * F; ++i) { const float v = g[i]; g[i] = (v / (1.0f + expf(-v))) * u[i]; }
        moe_matmul(g, down[e], bo, nt, D, F, as_double);
        for (int64_t i = 0; i < nt; ++i) {
            const int64_t t = toks[i];
            float wgt = 0.0f;
            for (int64_t k = 0; k < K; ++k) if (indices[t * K + k] == e) { wgt = weights[t * K + k]; break; }
            if (wgt <= 0.0f) { drop++; continue; }
            for (int64_t d = 0; d < D; ++d) {
                const float v = wgt * bo[i * D + d];
                if (as_double) wide[t * D + d] += (double)wgt * (double)bo[i * D + d];
                else out[t * D + d] += v;
                zl = fmaf(v, v, zl);
            }
        }
        free(bi); free(g); free(u); free(bo);
    }
    if (as_double) { for (int64_t i = 0; i < T * D; ++i) out[i] = (float)wide[i]; free(wide); }
    free(toks);
    if (z_loss) *z_loss = zl;
    if (dropped) *dropped = drop;
}

/* ------------------------------------------------------------------ dense / sign-coded engines */
static float widen_fp16_engine(uint16_t h) {          /* src/math.cpp:509-526 */
    const uint32_t sign = (uint32_t)(h >> 15) << 31;
    const int32_t e = (h >> 10) & 0x1F;
    const uint32_t mant = h & 0x03FF;
    uint32_t bits;
    float out;
    if (e == 0) {
        if (mant == 0) return 0.0f;
        return (sign ? -1.0f : 1.0f) * ((float)mant / 1024.0f) * 1.5258789e-5f;
    }
    bits = e == 31 ? (sign | 0x7F800000u | (mant << 13)) : (sign | ((uint32_t)(e + 112) << 23) | (mant << 13));
    memcpy(&out, &bits, 4);
    return out;
}

void orc_engine_dense_gemm(int kind, const float* A, const void* B, const float* scales, int64_t block,
                           float* C, int64_t M, int64_t N, int64_t K) {
    for (int64_t i = 0; i < M * N; ++i) C[i] = 0.0f;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) {
            const float a = A[m * K + k];
            if (a == 0.0f) continue;
            for (int64_t n = 0; n < N; ++n) {
                const int64_t flat = k * N + n;
                float* c = &C[m * N + n];
                if (kind == 1) *c = fmaf(a, ((const float*)B)[flat / 32], *c);
                else if (kind == 32) *c = fmaf(a, ((const float*)B)[flat], *c);
                else if (kind == 16) *c = fmaf(a, widen_fp16_engine(((const uint16_t*)B)[flat]), *c);
                else {
                    const float s = a * scales[flat / block];
                    const unsigned code = (((const uint8_t*)B)[flat / 4] >> ((flat % 4) * 2)) & 3u;
                    if (code == 2u) *c += s;
                    else if (code == 0u) *c -= s;
                }
            }
        }
}

/* ------------------------------------------------------------------ decode-step pieces */
void orc_rmsnorm(const float* x, const float* w, int n, float* out) {
    float s = 0.0f;
    for (int i = 0; i < n; ++i) s = fmaf(x[i], x[i], s);
    const float r = 1.0f / sqrtf(s / (float)n + 1e-6f);
    for (int i = 0; i < n; ++i) out[i] = x[i] * r * (1.0f + w[i]);
}

void orc_swiglu(const float* g, const float* u, int64_t n, float* h) {
    for (int64_t i = 0; i < n; ++i) {
        const float v = g[i];
        h[i] = (v * (1.0f / (1.0f + expf(-v)))) * u[i];
    }
}

/* ---- OIL4 KV cache (src/kv_cache_oil4.cpp, src/codebook.cpp:16-64) ------------------------------------------ */
uint16_t orc_kv_float_to_half(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const int32_t e = (int32_t)((u >> 23) & 0xFFu) - 127 + 15;
    uint32_t mant = u & 0x007FFFFFu;
    if (e <= 0) {
        if (e < -10) return sign;
        mant = (mant | 0x00800000u) >> (1 - e);
        return (uint16_t)(sign | (uint16_t)(mant >> 13));
    }
    if (e >= 31) return (uint16_t)(sign | 0x7C00u | (mant != 0 ? 0x0200u : 0u));
    return (uint16_t)(sign | ((uint16_t)e << 10) | (uint16_t)(mant >> 13));
}

float orc_kv_half_to_float(uint16_t h) {
    const uint32_t sign = h & 0x8000u;
    int32_t e = (h >> 10) & 0x1F;
    uint16_t mant = h & 0x03FFu;
    uint32_t f;
    if (e == 0) {
        if (mant == 0) {
            f = sign << 16;
        } else {
            int shift = 10;
            while ((mant & 0x0400u) == 0) { mant = (uint16_t)(mant << 1); shift--; }
            e = 1 - shift + 127 - 15;
            /* the reference keeps the shifted mantissa in a uint16_t: only bits 13-15 survive (codebook.cpp:52) */
            f = (sign << 16) | ((uint32_t)e << 23) | (((uint32_t)(mant & 0x03FFu) << 13) & 0xFFFFu);
        }
    } else if (e == 31) {
        f = (sign << 16) | 0x7F800000u | ((uint32_t)mant << 13);
    } else {
        f = (sign << 16) | ((uint32_t)(e - 15 + 127) << 23) | ((uint32_t)mant << 13);
    }
    float r;
    memcpy(&r, &f, 4);
    return r;
}

static int kv_cmp_float(const void* a, const void* b) {
    const float x = *(const float*)a, y = *(const float*)b;
    return x < y ? -1 : (x > y ? 1 : 0);
}

static int kv_nearest(const float* cen, float x) {
    float best = fabsf(x - cen[0]);
    int bi = 0;
    for (int c = 1; c < 16; ++c) {
        const float d = fabsf(x - cen[c]);
        if (d < best) { best = d; bi = c; }
    }
    return bi;
}

void orc_kv_quantize_block(const float* src, int64_t n, uint16_t* cb16, uint8_t* codes) {
    if (n == 0) return;
    float lo = src[0], hi = src[0];
    for (int64_t i = 1; i < n; ++i) {
        if (src[i] < lo) lo = src[i];
        if (src[i] > hi) hi = src[i];
    }
    if (hi - lo < 1e-10f) {
        for (int64_t i = 0; i < n; ++i) codes[i] = 8;
        for (int c = 0; c < 16; ++c) cb16[c] = orc_kv_float_to_half(lo);
        return;
    }
    float cen[16];
    for (int c = 0; c < 16; ++c) cen[c] = lo + (hi - lo) * ((float)c + 0.5f) / 16.0f;
    float sorted[4096];
    const int64_t m = n > 4096 ? 4096 : n;
    memcpy(sorted, src, (size_t)m * 4);
    qsort(sorted, (size_t)m, 4, kv_cmp_float);          /* values only: any correct sort gives the same array up to -0/+0 and NaN order */
    for (int it = 0; it < 20; ++it) {
        float sums[16] = {0};
        int counts[16] = {0};
        for (int64_t i = 0; i < m; ++i) {
            const int b = kv_nearest(cen, sorted[i]);
            sums[b] += sorted[i];
            counts[b]++;
        }
        for (int c = 0; c < 16; ++c)
            if (counts[c] > 0) cen[c] = sums[c] / (float)counts[c];
    }
    for (int64_t i = 0; i < n; ++i) codes[i] = (uint8_t)kv_nearest(cen, src[i]);
    for (int c = 0; c < 16; ++c) cb16[c] = orc_kv_float_to_half(cen[c]);
}

static int64_t kv_block(int64_t block) { return block == 32 || block == 64 || block == 128 ? block : 64; }

void orc_kv_append(uint8_t* k_idx, uint8_t* v_idx, uint16_t* k_cb, uint16_t* v_cb, int64_t idx_bytes,
                   int64_t max_seq, int64_t per_token, int64_t block, int64_t pos,
                   const float* k, const float* v, int64_t seq_len) {
    block = kv_block(block);
    const int64_t ibpb = (block + 1) / 2;
    uint8_t codes[128], packed[64];
    uint16_t cb[16];
    for (int64_t s = 0; s < seq_len && pos + s < max_seq; ++s) {
        int64_t left = per_token, src = s * per_token, flat = (pos + s) * per_token;
        while (left > 0) {
            const int64_t blk = flat / block, off = flat % block;
            const int64_t chunk = left < block - off ? left : block - off;
            const int64_t at = blk * ibpb + off / 2;
            for (int pass = 0; pass < 2; ++pass) {
                orc_kv_quantize_block((pass ? v : k) + src, chunk, cb, codes);
                const int64_t nbytes = (chunk + 1) / 2;
                for (int64_t i = 0; i < nbytes; ++i) {
                    const uint8_t lo4 = codes[2 * i] & 0x0F;
                    const uint8_t hi4 = (2 * i + 1) < chunk ? (codes[2 * i + 1] & 0x0F) : 0;
                    packed[i] = (uint8_t)(lo4 | (hi4 << 4));
                }
                int64_t put = nbytes;
                if (at + put > idx_bytes) put = idx_bytes - at;
                if (put > 0) memcpy((pass ? v_idx : k_idx) + at, packed, (size_t)put);
                if (pass || off == 0 || pos == 0) memcpy((pass ? v_cb : k_cb) + blk * 16, cb, 32);
            }
            left -= chunk; src += chunk; flat += chunk;
        }
    }
}

void orc_kv_get_range(const uint8_t* idx, const uint16_t* cb, int64_t idx_bytes, int64_t per_token, int64_t block,
                      int64_t start, int64_t len, float* out) {
    block = kv_block(block);
    const int64_t ibpb = (block + 1) / 2;
    for (int64_t s = 0; s < len; ++s) {
        int64_t left = per_token, flat = (start + s) * per_token, dst = s * per_token;
        while (left > 0) {
            const int64_t blk = flat / block, off = flat % block;
            const int64_t chunk = left < block - off ? left : block - off;
            const int64_t at = blk * ibpb + off / 2;
            for (int64_t i = 0; i < chunk; ++i) {
                const int64_t b = at + i / 2;
                const uint8_t byte = b < idx_bytes ? idx[b] : 0;
                const uint8_t code = (i & 1) ? (uint8_t)(byte >> 4) : (uint8_t)(byte & 0x0F);
                out[dst + i] = orc_kv_half_to_float(cb[blk * 16 + code]);
            }
            left -= chunk; flat += chunk; dst += chunk;
        }
    }
}

/* ------------------------------------------------------------ SPARK lookup kernels */
/* src/kernel_tl.cpp:32-90 (TL1) and :124-184 (TL2). */
void orc_tl_gemm(int kind, const uint8_t* w, const float* a, float* out, int M, int N, int K) {
    if (M <= 0 || N <= 0 || K < 0) return;
    const size_t row_bytes = kind == 1 ? (size_t)((K + 3) / 4) : (size_t)(((K + 11) / 12) * 3);
    int8_t* q = (int8_t*)malloc((size_t)N * (size_t)(K > 0 ? K : 1));
    float* scales = (float*)malloc(sizeof(float) * (size_t)N);
    for (int n = 0; n < N; ++n) {                          /* :39-50 / :131-143 */
        float mx = 0.f;
        for (int k = 0; k < K; ++k) { const float v = fabsf(a[(size_t)n * K + k]); if (v > mx) mx = v; }
        if (mx < 1e-10f) mx = 1e-10f;
        scales[n] = 127.0f / mx;
        for (int k = 0; k < K; ++k) q[(size_t)n * K + k] = (int8_t)roundf(a[(size_t)n * K + k] * scales[n]);
    }
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            const uint8_t* wr = w + ((size_t)m * N + n) * row_bytes;
            const int8_t* ar = q + (size_t)n * K;
            int64_t total = 0;
            for (int k = 0; k < K; ++k) {
                const int c = (wr[k / 4] >> ((k % 4) * 2)) & 3;   /* 0 -> -1, 1 -> 0, else +1 (:68-71, :112-117) */
                const int wv = c == 0 ? -1 : (c == 1 ? 0 : 1);
                if (kind == 1 && k + 1 < K && (k & 1) == 0) {     /* pair sum stored as int8 (:22-24) */
                    const int c1 = (wr[k / 4] >> ((k % 4) * 2 + 2)) & 3;
                    const int w1 = c1 == 0 ? -1 : (c1 == 1 ? 0 : 1);
                    int sum = (int)ar[k] * wv + (int)ar[k + 1] * w1;
                    if (sum < -128) sum = -128;
                    if (sum > 127) sum = 127;
                    total += sum;
                    ++k;
                } else {
                    total += (int)ar[k] * wv;                     /* odd tail of TL1 (:75-81); every term of TL2 */
                }
            }
            if (kind == 1) total = (int32_t)total;
            out[(size_t)m * N + n] = (float)total / scales[n];
        }
    free(q);
    free(scales);
}
