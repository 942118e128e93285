// host_codec.cpp -- host-side OIL block quantizer (the producer of block
// payloads).  In the reference the quantizer is CPU code as well
// (quantize_block_all, src/block_codec.cpp:368-574); it is not part of the
// accelerated decode path.  The reference build fuses a*b+c (its -mfma flag
// with the compiler's default contraction), so sums of products below use
// std::fma explicitly and this file is compiled with -ffp-contract=off.
#include <algorithm>
#include <array>
#include <cmath>
#include <cstring>
#include <span>
#include <thread>
#include <utility>
#include <vector>

#include "../../include/oilhip.h"

namespace oilhip {
int fail(int code, const std::string& msg);
}

namespace {

constexpr std::array<float, 4> kL2 = {-1.5104f, -0.4528f, 0.4528f, 1.5104f};
constexpr std::array<float, 16> kL4 = {-2.7178f, -2.0522f, -1.5995f, -1.2392f, -0.9275f, -0.6508f,
                                       -0.3976f, -0.1260f, 0.1260f,  0.3976f,  0.6508f,  0.9275f,
                                       1.2392f,  1.5995f,  2.0522f,  2.7178f};

// block_codec.cpp:26-59 -- round to nearest even, overflow and NaN to infinity,
// magnitudes under 2^-24 to signed zero.
uint16_t to_half(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    const uint32_t sgn = (u >> 16) & 0x8000u;
    int ex = int((u >> 23) & 0xFF) - 127;
    if (ex > 15) return uint16_t(sgn | 0x7C00u);
    if (ex < -24) return uint16_t(sgn);
    const uint32_t sig = (u & 0x7FFFFFu) | 0x800000u;
    const int cut = ex >= -14 ? 13 : -ex - 1;
    uint32_t keep = sig >> cut;
    const uint32_t lost = sig & ((1u << cut) - 1u), mid = 1u << (cut - 1);
    keep += (lost > mid) || (lost == mid && (keep & 1u));
    if (ex < -14) return uint16_t(sgn | keep);
    if (keep >= 0x800u) {
        keep >>= 1;
        if (++ex > 15) return uint16_t(sgn | 0x7C00u);
    }
    return uint16_t(sgn | uint32_t(ex + 15) << 10 | (keep & 0x3FFu));
}

// LSB-first bit sink over a fixed-size byte span (block_codec.cpp:87-100).
class BitSink {
public:
    explicit BitSink(std::span<uint8_t> out) : out_(out) { std::fill(out.begin(), out.end(), uint8_t{0}); }
    void put(uint32_t v, int n) {
        for (int i = 0; i < n; ++i, ++at_)
            if ((at_ >> 3) < out_.size() && ((v >> i) & 1u)) out_[at_ >> 3] |= uint8_t(1u << (at_ & 7));
    }
    void skip(size_t n) { at_ += n; }
private:
    std::span<uint8_t> out_;
    size_t at_ = 0;
};

bool is_slot(long long i, long long n, int count) {   // block_codec.cpp:122-126
    return count > 0 && n > 0 && ((i + 1) * count) / n != (i * count) / n;
}

template <size_t N>
uint32_t nearest(float v, const std::array<float, N>& lv) {   // :139-146, ties keep the lower index
    uint32_t best = 0;
    float bd = std::fabs(v - lv[0]);
    for (uint32_t i = 1; i < N; ++i) {
        const float d = std::fabs(v - lv[i]);
        if (d < bd) { bd = d; best = i; }
    }
    return best;
}

uint32_t nearest_level(float v, int bits) {
    if (bits == 2) return nearest(v, kL2);
    if (bits == 4) return nearest(v, kL4);
    const float c = std::max(-8.0f, std::min(8.0f, v));
    return uint32_t(std::lround((c + 8.0f) * 255.0f / 16.0f));
}

float rms(std::span<const float> w) {   // :149-154
    if (w.empty()) return 0.0f;
    double s = 0.0;
    for (float x : w) s = std::fma(double(x), double(x), s);
    return float(std::sqrt(s / double(w.size())));
}

uint32_t cap255(long v) { return uint32_t(v) > 255u ? 255u : uint32_t(v); }

size_t grp_header_bits(int n) { return n < 64 ? (n < 8 ? 0u : 16u) : size_t(n / 64) * 32u; }

size_t payload_bound(int fmt, int n) {
    if (n <= 0) return 0;
    const size_t N = size_t(n);
    switch (fmt) {
        case OILHIP_OIL32: return N * 4;
        case OILHIP_OIL16: case OILHIP_OIL16_GRP: return N * 2;
        case OILHIP_OIL8: return N;
        case OILHIP_OIL4: return (N * 4 + 7) / 8;
        case OILHIP_OIL2: return (N * 2 + 7) / 8;
        case OILHIP_OIL8_GRP: return (grp_header_bits(n) + N * 8 + 7) / 8;
        case OILHIP_OIL4_GRP: return (grp_header_bits(n) + N * 4 + 7) / 8;
        case OILHIP_OIL2_GRP: return (grp_header_bits(n) + N * 2 + 7) / 8;
        case OILHIP_OIL1: return ((N + 31) / 32) * 2;
        case OILHIP_OIL1_GRP: return (N + 7) / 8;
        case OILHIP_SPARK_Q0: return (N * 3 + 15) / 16;
        case OILHIP_SPARK_Q0_GRP: return n < 32 ? (N + 7) / 8 : (N * 3 + 15) / 16;
        case OILHIP_SPARK_SPARSE: return N / 4 < 4 ? 0 : 4 + std::min<size_t>(20, (N / 4 - 4) / 3) * 3;
        case OILHIP_SPARK_SPARSE_GRP: return N / 4 < 8 ? 0 : 4 + ((N / 4 - 4) / 3) * 3;
        default: return 0;
    }
}

size_t encode_lattice(std::span<const float> w, int bits, uint8_t* out) {   // :157-171
    const int n = int(w.size());
    const size_t bytes = (size_t(bits) * n + 7) / 8;
    BitSink sink({out, bytes});
    const float scale = rms(w);
    sink.put(to_half(scale), 16);
    const float s = scale <= 1e-12f ? 0.0f : scale;
    for (int i = 0; i < n; ++i) {
        if (is_slot(i, n, 16 / bits)) continue;
        sink.put(nearest_level(s == 0.0f ? 0.0f : w[i] / s, bits), bits);
    }
    return bytes;
}

size_t encode_grouped(std::span<const float> w, int bits, uint8_t* out) {   // :191-306
    const int n = int(w.size()), full = n / 64;
    const bool wide = bits == 8;
    const size_t bytes = (grp_header_bits(n) + size_t(n) * bits + 7) / 8;
    BitSink sink({out, bytes});
    auto code = [&](float v, float zp, float sc) -> uint32_t {
        if (wide) return cap255(std::lround((v - zp) / sc * 255.0f));
        return nearest_level(float((double(v) - zp) / double(sc)), bits);
    };
    float pzp = 0.0f, psc = 1.0f;
    for (int g = 0; g < full; ++g) {
        const auto grp = w.subspan(size_t(g) * 64, 64);
        float zp, sc;
        if (wide) {
            const auto [lo, hi] = std::minmax_element(grp.begin(), grp.end());
            zp = *lo;
            sc = *hi - *lo;
        } else {
            double mu = 0.0, ss = 0.0;
            for (float x : grp) mu += x;
            mu /= 64.0;
            for (float x : grp) { const double d = double(x) - mu; ss = std::fma(d, d, ss); }
            zp = float(mu);
            sc = ss > 0.0 ? float(std::sqrt(ss / 64.0)) : 0.0f;
        }
        sink.put(to_half(zp), 16);
        sink.put(to_half(sc), 16);
        pzp = zp;
        psc = sc;
        if (sc == 0.0f) { sink.skip(size_t(64) * bits); continue; }
        for (float x : grp) sink.put(code(x, zp, sc), bits);
    }
    const auto tail = w.subspan(size_t(full) * 64);
    if (tail.empty()) return bytes;
    if (full > 0) {                               // partial tail reuses the last group's zp/scale
        for (float x : tail) sink.put(psc == 0.0f ? 0u : code(x, pzp, psc), bits);
        return bytes;
    }
    if (n < 8) {                                  // headerless: implicit scale 1, zero-point 0
        for (float x : tail)
            sink.put(wide ? cap255(std::lround((x + 1.0f) * 127.5f)) : nearest_level(x, bits), bits);
        return bytes;
    }
    float sc;
    if (wide) {
        sc = std::fabs(tail[0]);
        for (float x : tail.subspan(1)) sc = std::max(sc, std::fabs(x));
    } else {
        double ss = 0.0;
        for (float x : tail) ss = std::fma(double(x), double(x), ss);
        sc = ss > 0.0 ? float(std::sqrt(ss / double(n))) : 0.0f;
    }
    sink.put(to_half(sc), 16);
    if (sc == 0.0f) return bytes;
    for (float x : tail)
        sink.put(wide ? cap255(std::lround((x / sc + 1.0f) * 127.5f)) : nearest_level(x / sc, bits), bits);
    return bytes;
}

size_t encode_sparse(std::span<const float> w, bool grouped, uint8_t* out) {   // :484-570
    const int n = int(w.size());
    const size_t budget = size_t(n) / 4;
    if (budget < (grouped ? 8u : 4u)) return 0;
    int keep = int((budget - 4) / 3);
    if (!grouped) keep = std::min(keep, 20);
    if (grouped && keep <= 0) return 0;
    const int half = n / 2;
    std::vector<std::pair<float, int>> mag(static_cast<size_t>(n));
    float s0 = 0.0f, s1 = 0.0f;
    for (int i = 0; i < n; ++i) {
        const float a = std::fabs(w[i]);
        mag[size_t(i)] = {a, i};
        float& top = (!grouped || i < half) ? s0 : s1;
        top = std::max(top, a);
    }
    if (!grouped) {
        if (s0 <= 1e-12f) { std::memset(out, 0, 4); return 4; }
        std::memcpy(out, &s0, 4);
    } else {
        if (s0 <= 1e-12f) s0 = 1.0f;
        if (s1 <= 1e-12f) s1 = 1.0f;
        const uint16_t h0 = to_half(s0), h1 = to_half(s1);
        out[0] = uint8_t(h0); out[1] = uint8_t(h0 >> 8); out[2] = uint8_t(h1); out[3] = uint8_t(h1 >> 8);
    }
    if (keep > 0)   // same call as the reference: equal magnitudes land where libstdc++'s heap puts them
        std::partial_sort(mag.begin(), mag.begin() + keep, mag.end(),
                          [](const auto& a, const auto& b) { return a.first > b.first; });
    for (int r = 0; r < keep; ++r) {
        const int at = mag[size_t(r)].second;
        const float s = (!grouped || at < half) ? s0 : s1;
        const int q = std::clamp(int(std::lround(w[at] / s * 127.0f)), -127, 127);
        uint8_t* rec = out + 4 + 3 * size_t(r);
        rec[0] = uint8_t(at); rec[1] = uint8_t(at >> 8); rec[2] = uint8_t(int8_t(q));
    }
    return 4 + 3 * size_t(keep);
}

// Encodes one block; returns false for an unknown format.  cb receives the OIL1
// run means, idx everything else.
bool encode_block(int fmt, std::span<const float> w, uint8_t* idx, size_t& il, uint8_t* cb, size_t& cl) {
    const int n = int(w.size());
    il = cl = 0;
    auto sign_bit = [](float v) { return v >= 0.0f ? 1u : 0u; };
    switch (fmt) {
        case OILHIP_OIL32: std::memcpy(idx, w.data(), size_t(n) * 4); il = size_t(n) * 4; return true;
        case OILHIP_OIL16: case OILHIP_OIL16_GRP:
            for (int i = 0; i < n; ++i) { const uint16_t h = to_half(w[i]); idx[2 * i] = uint8_t(h); idx[2 * i + 1] = uint8_t(h >> 8); }
            il = size_t(n) * 2; return true;
        case OILHIP_OIL8: il = encode_lattice(w, 8, idx); return true;
        case OILHIP_OIL4: il = encode_lattice(w, 4, idx); return true;
        case OILHIP_OIL2: il = encode_lattice(w, 2, idx); return true;
        case OILHIP_OIL8_GRP: il = encode_grouped(w, 8, idx); return true;
        case OILHIP_OIL4_GRP: il = encode_grouped(w, 4, idx); return true;
        case OILHIP_OIL2_GRP: il = encode_grouped(w, 2, idx); return true;
        case OILHIP_OIL1:                                       // :406-420
            for (int a = 0, r = 0; a < n; a += 32, ++r) {
                const auto run = w.subspan(size_t(a), size_t(std::min(32, n - a)));
                double s = 0.0;
                for (float x : run) s += x;
                const uint16_t h = to_half(float(s / double(run.size())));
                cb[2 * r] = uint8_t(h); cb[2 * r + 1] = uint8_t(h >> 8);
                cl += 2;
            }
            return true;
        case OILHIP_OIL1_GRP: {                                 // :421-443
            il = (size_t(n) + 7) / 8;
            BitSink sink({idx, il});
            if (n >= 32) sink.put(to_half(rms(w)), 16);
            for (int i = 0; i < n; ++i)
                if (n < 32 || !is_slot(i, n, 16)) sink.put(sign_bit(w[i]), 1);
            return true;
        }
        case OILHIP_SPARK_Q0: {                                 // :444-458
            il = (size_t(n) * 3 + 15) / 16;
            BitSink sink({idx, il});
            for (int a = 0; a < n; a += 32) {
                const auto run = w.subspan(size_t(a), size_t(std::min(32, n - a)));
                if (run.size() == 32) sink.put(to_half(rms(run)), 16);
                for (float x : run) sink.put(sign_bit(x), 1);
            }
            return true;
        }
        case OILHIP_SPARK_Q0_GRP: {                             // :459-483
            if (n < 32) {
                il = (size_t(n) + 7) / 8;
                BitSink sink({idx, il});
                for (float x : w) sink.put(sign_bit(x), 1);
                return true;
            }
            il = (size_t(n) * 3 + 15) / 16;
            BitSink sink({idx, il});
            const float scale = rms(w);
            sink.put(to_half(scale), 16);
            for (float x : w) sink.put(sign_bit(x), 1);
            const float thr = scale * 1.23f;
            for (int i = 0; i < n; ++i)
                if (is_slot(i, n, n / 2 - 16)) sink.put(std::fabs(w[i]) > thr ? 1u : 0u, 1);
            return true;
        }
        case OILHIP_SPARK_SPARSE: il = encode_sparse(w, false, idx); return true;
        case OILHIP_SPARK_SPARSE_GRP: il = encode_sparse(w, true, idx); return true;
        default: return false;
    }
}

}  // namespace

extern "C" {

size_t oilhip_payload_bound(int fmt, int n) { return payload_bound(fmt, n); }

int oilhip_quantize_block(int fmt, const float* w, int n, uint8_t* idx, size_t idx_cap, size_t* idx_len,
                          uint8_t* cb, size_t cb_cap, size_t* cb_len) {
    if (!w || n <= 0 || !idx_len || !cb_len) return oilhip::fail(OILHIP_E_ARG, "quantize_block: bad arguments");
    if (fmt < 0 || fmt >= OILHIP_NUM_FORMATS) return oilhip::fail(OILHIP_E_ARG, "quantize_block: unknown format");
    const size_t need = payload_bound(fmt, n);
    if (fmt == OILHIP_OIL1 ? (cb_cap < need || !cb) : (need > 0 && (idx_cap < need || !idx)))
        return oilhip::fail(OILHIP_E_ARG, "quantize_block: output buffer too small");
    encode_block(fmt, {w, size_t(n)}, idx, *idx_len, cb, *cb_len);
    return OILHIP_OK;
}

int oilhip_quantize_tensor(const uint8_t* fmts, uint32_t nblocks, const float* w, uint64_t numel,
                           uint8_t* payload, uint64_t cap, oilhip_block_t* blocks, uint64_t* total, int threads) {
    if (!fmts || !w || !total || nblocks == 0) return oilhip::fail(OILHIP_E_ARG, "quantize_tensor: bad arguments");
    if (uint64_t(nblocks) * 256 < numel || uint64_t(nblocks - 1) * 256 >= numel)
        return oilhip::fail(OILHIP_E_ARG, "quantize_tensor: nblocks does not match numel");
    size_t widest = 0;
    uint64_t bound = 0;
    for (uint32_t b = 0; b < nblocks; ++b) {
        if (fmts[b] >= OILHIP_NUM_FORMATS) return oilhip::fail(OILHIP_E_ARG, "quantize_tensor: unknown format");
        const size_t m = payload_bound(fmts[b], 256);
        widest = std::max(widest, m);
        bound += (m + 15) & ~size_t(15);
    }
    if (!payload) { *total = bound; return OILHIP_OK; }
    if (!blocks) return oilhip::fail(OILHIP_E_ARG, "quantize_tensor: blocks is null");
    struct Enc { uint32_t il, cl; };
    const size_t stride = widest + 32;             // [32 bytes codebook channel][index channel]
    std::vector<uint8_t> tmp(size_t(nblocks) * stride);
    std::vector<Enc> len(nblocks);
    if (threads <= 0) threads = int(std::max(1u, std::thread::hardware_concurrency()));
    threads = int(std::min<uint32_t>(uint32_t(std::min(threads, 64)), nblocks));
    auto work = [&](uint32_t b0, uint32_t b1) {
        for (uint32_t b = b0; b < b1; ++b) {
            const uint64_t at = uint64_t(b) * 256;
            const size_t n = size_t(std::min<uint64_t>(256, numel - at));
            size_t il = 0, cl = 0;
            uint8_t* slot = tmp.data() + size_t(b) * stride;
            encode_block(fmts[b], {w + at, n}, slot + 32, il, slot, cl);
            len[b] = {uint32_t(il), uint32_t(cl)};
        }
    };
    std::vector<std::thread> pool;
    const uint32_t chunk = (nblocks + uint32_t(threads) - 1) / uint32_t(threads);
    for (int t = 1; t < threads; ++t) {
        const uint32_t b0 = uint32_t(t) * chunk, b1 = std::min(nblocks, b0 + chunk);
        if (b0 < b1) pool.emplace_back(work, b0, b1);
    }
    work(0, std::min(nblocks, chunk));
    for (auto& th : pool) th.join();
    uint64_t off = 0;
    for (uint32_t b = 0; b < nblocks; ++b) {
        off = (off + 15) & ~uint64_t(15);
        if (off + len[b].cl + len[b].il > cap) return oilhip::fail(OILHIP_E_ARG, "quantize_tensor: payload buffer too small");
        const uint8_t* slot = tmp.data() + size_t(b) * stride;
        std::memcpy(payload + off, slot, len[b].cl);
        std::memcpy(payload + off + len[b].cl, slot + 32, len[b].il);
        const uint64_t at = uint64_t(b) * 256;
        blocks[b] = oilhip_block_t{off, off + len[b].cl, len[b].cl, len[b].il,
                                   uint32_t(std::min<uint64_t>(256, numel - at)), fmts[b], {0, 0, 0}};
        off += len[b].cl + len[b].il;
    }
    *total = off;
    return OILHIP_OK;
}

}  // extern "C"
