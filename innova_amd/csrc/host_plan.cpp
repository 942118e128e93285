// host_plan.cpp -- host-side format routing: which wire format each 256-weight block gets.
// Producer-side logic (it decides what the quantizer writes); the reference runs it on the
// CPU as well.  Counterparts:
//   FormatPlanner::score_importance / score_importance_fisher   src/format_planner.cpp:12-61
//   FormatPlanner::compute_format_mix / allocate / estimate_bpw src/format_planner.cpp:63-122,133-332
//   FormatRegistry singles and mixes                            src/format_registry.cpp:19-101
//   FormatRegistry::allocate_mix_blocks                         src/format_registry.cpp:477-599
// The adaptive mix allocator needs the reconstruction error of every candidate format on
// every block; those decodes run on the GPU (block_mse in generic_kernels.hip), only the
// greedy benefit-per-byte walk stays on the host.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <numeric>
#include <queue>
#include <string>
#include <vector>

#include <hip/hip_runtime.h>

#include "common.h"

namespace oilhip {
int launch_block_mse(const oilhip_weights& w, const float* d_orig, const uint64_t* d_start, float* d_out, hipStream_t s);
}

namespace {

struct Single { uint8_t fmt; float bpw; };
// registry order matters: the closest single is the first one at minimal distance
constexpr Single kSingles[15] = {
    {OILHIP_OIL1, 1.0f}, {OILHIP_OIL2, 2.0f}, {OILHIP_OIL4, 4.0f}, {OILHIP_OIL8, 8.0f}, {OILHIP_OIL16, 16.0f},
    {OILHIP_OIL32, 32.0f}, {OILHIP_OIL1_GRP, 1.0f}, {OILHIP_OIL2_GRP, 2.5f}, {OILHIP_OIL4_GRP, 4.5f},
    {OILHIP_OIL8_GRP, 8.5f}, {OILHIP_OIL16_GRP, 16.0f}, {OILHIP_SPARK_SPARSE, 2.0f},
    {OILHIP_SPARK_SPARSE_GRP, 2.0f}, {OILHIP_SPARK_Q0, 1.5f}, {OILHIP_SPARK_Q0_GRP, 1.5f}};

struct Mix { int tiers; uint8_t fmt[4]; float ratio[4]; float bpw; };
constexpr Mix kTwoMixes[9] = {
    {2, {OILHIP_OIL8, OILHIP_OIL2, OILHIP_OIL2, OILHIP_OIL2}, {0.01f, 0.99f, 0, 0}, 2.06f},
    {2, {OILHIP_OIL8, OILHIP_OIL4, OILHIP_OIL4, OILHIP_OIL4}, {0.05f, 0.95f, 0, 0}, 4.20f},
    {2, {OILHIP_OIL4, OILHIP_OIL2, OILHIP_OIL2, OILHIP_OIL2}, {0.10f, 0.90f, 0, 0}, 2.20f},
    {2, {OILHIP_OIL8, OILHIP_OIL2, OILHIP_OIL2, OILHIP_OIL2}, {0.10f, 0.90f, 0, 0}, 2.60f},
    {2, {OILHIP_SPARK_Q0, OILHIP_OIL8, OILHIP_OIL8, OILHIP_OIL8}, {0.05f, 0.95f, 0, 0}, 7.675f},
    {2, {OILHIP_OIL16, OILHIP_OIL4, OILHIP_OIL4, OILHIP_OIL4}, {0.01f, 0.99f, 0, 0}, 4.12f},
    {2, {OILHIP_OIL16, OILHIP_OIL8, OILHIP_OIL8, OILHIP_OIL8}, {0.05f, 0.95f, 0, 0}, 8.40f},
    {2, {OILHIP_OIL32, OILHIP_OIL8, OILHIP_OIL8, OILHIP_OIL8}, {0.01f, 0.99f, 0, 0}, 8.24f},
    {4, {OILHIP_OIL8_GRP, OILHIP_OIL4_GRP, OILHIP_OIL2_GRP, OILHIP_OIL1_GRP}, {0.01f, 0.02f, 0.52f, 0.45f}, 1.925f}};   // SPARK_MIX_Q0
constexpr Mix kFourMixes[3] = {
    {4, {OILHIP_OIL16, OILHIP_OIL8, OILHIP_OIL4, OILHIP_OIL2}, {0.01f, 0.05f, 0.24f, 0.70f}, 2.92f},
    {4, {OILHIP_OIL32, OILHIP_OIL16, OILHIP_OIL8, OILHIP_OIL4}, {0.01f, 0.05f, 0.24f, 0.70f}, 5.84f},
    {4, {OILHIP_OIL32, OILHIP_OIL8_GRP, OILHIP_OIL2_GRP, OILHIP_OIL1_GRP}, {0.01f, 0.01f, 0.46f, 0.52f}, 2.075f}};  // QUAD_SPARK_Q1

float wire_bpw(int fmt) {                      // include/oil/types.h:57-82
    for (const Single& s : kSingles) if (s.fmt == fmt) return s.bpw;
    return 0.0f;
}

template <size_t N>
const Mix& closest_mix(const Mix (&mixes)[N], float target, float& diff) {
    size_t best = 0;
    diff = 1e9f;
    for (size_t i = 0; i < N; ++i) {
        const float d = std::fabs(mixes[i].bpw - target);
        if (d < diff) { diff = d; best = i; }
    }
    return mixes[best];
}

// blocks by descending importance; std::sort with the reference's comparator so equal scores
// land where the same library puts them
std::vector<int> importance_order(int nb, const float* scores, int64_t nscores) {
    std::vector<int> order((size_t)nb);
    std::iota(order.begin(), order.end(), 0);
    if (scores && nscores > 0)
        std::sort(order.begin(), order.end(), [&](int a, int b) {
            const float sa = a < nscores ? scores[a] : 0, sb = b < nscores ? scores[b] : 0;
            return sa > sb;
        });
    return order;
}

// src/format_planner.cpp:63-122: block counts per precision for a plain target
void ladder_counts(int nb, float t, int (&c)[7]) {   // c = {32, 16, 8, 4, 2, spark, 1}
    float f[7] = {0, 0, 0, 0, 0, 0, 0};
    if (t >= 32.0f) f[0] = 1.0f;
    else if (t >= 16.0f) { f[0] = (t - 16.0f) / 16.0f; f[1] = 1.0f - f[0]; }
    else if (t >= 8.0f) { f[1] = (t - 8.0f) / 8.0f; f[2] = 1.0f - f[1]; }
    else if (t >= 4.0f) { f[2] = (t - 4.0f) / 4.0f; f[3] = 1.0f - f[2]; }
    else if (t >= 2.0f) { f[3] = (t - 2.0f) / 2.0f; f[4] = 1.0f - f[3]; }
    else if (t >= 1.0f) { f[5] = (t - 1.0f) / 1.0f; f[6] = 1.0f - f[5]; }
    else f[6] = 1.0f;
    int total = 0;
    for (int i = 0; i < 7; ++i) { c[i] = (int)std::round(f[i] * (double)nb); total += c[i]; }
    const int diff = nb - total;
    if (diff > 0) c[6] += diff;
    else if (diff < 0) {
        if (c[6] >= -diff) c[6] += diff;
        else { c[6] = 0; c[5] = std::max(0, c[5] + diff); }
    }
    int left = nb;
    for (int i = 0; i < 6; ++i) { c[i] = std::min(c[i], left); left -= c[i]; }
    c[6] = std::max(0, left);
}

}  // namespace

extern "C" {

int oilhip_score_importance(const float* w, const float* aux, int64_t n, int block_size, int fisher,
                            float* scores, int64_t nblocks) {
    if (!w || !scores || n <= 0 || block_size <= 0) return oilhip::fail(OILHIP_E_ARG, "score_importance: bad arguments");
    if (nblocks != (n + block_size - 1) / block_size) return oilhip::fail(OILHIP_E_ARG, "score_importance: nblocks mismatch");
    if (fisher && !aux) return oilhip::fail(OILHIP_E_ARG, "score_importance: the Fisher metric needs gradients");
    for (int64_t b = 0; b < nblocks; ++b) {
        const int64_t a = b * block_size, e = std::min<int64_t>(a + block_size, n);
        double s = 0;
        if (fisher) {
            for (int64_t i = a; i < e; ++i) { const float g = aux[i]; s += (double)(g * g); }
            s = std::sqrt(s / (double)(e - a)) * (double)std::fabs(w[a]);
        } else {
            for (int64_t i = a; i < e; ++i)
                s = std::fma((double)std::fabs(w[i]), (double)(aux ? std::fabs(aux[i]) : 1.0f), s);   // fused in the reference build
            s /= (double)(e - a);
        }
        scores[b] = (float)s;
    }
    return OILHIP_OK;
}

int oilhip_plan_formats(float target_bpw, const float* scores, int64_t nscores, int num_blocks,
                        uint8_t* fmts, float* achieved_bpw, int* uses_mix, int* counts7) {
    if (num_blocks < 0 || (num_blocks > 0 && !fmts)) return oilhip::fail(OILHIP_E_ARG, "plan_formats: bad arguments");
    float single_diff = 1e9f;
    for (const Single& s : kSingles) single_diff = std::min(single_diff, std::fabs(s.bpw - target_bpw));
    float two_diff, four_diff;
    const Mix& two = closest_mix(kTwoMixes, target_bpw, two_diff);
    const Mix& four = closest_mix(kFourMixes, target_bpw, four_diff);
    const bool use_two = two_diff < single_diff && two_diff < four_diff;
    const bool use_four = four_diff < single_diff && four_diff < two_diff;
    const std::vector<int> order = importance_order(num_blocks, scores, nscores);
    if (use_two || use_four) {
        const Mix& m = use_four ? four : two;
        int cnt[4] = {0, 0, 0, 0}, used = 0;
        for (int t = 0; t < m.tiers - 1; ++t) { cnt[t] = (int)std::round(m.ratio[t] * (double)num_blocks); used += cnt[t]; }
        cnt[m.tiers - 1] = std::max(0, num_blocks - used);
        for (int i = 0; i < num_blocks; ++i) {
            int tier = 0, cum = 0;
            for (int t = 0; t < m.tiers; ++t) {
                if (i < cum + cnt[t]) { tier = t; break; }
                cum += cnt[t];
            }
            fmts[order[(size_t)i]] = m.fmt[tier];
        }
    } else {
        int c[7];
        ladder_counts(num_blocks, target_bpw, c);
        static const uint8_t f[7] = {OILHIP_OIL32, OILHIP_OIL16, OILHIP_OIL8, OILHIP_OIL4, OILHIP_OIL2, OILHIP_SPARK_Q0, OILHIP_OIL1};
        for (int i = 0; i < num_blocks; ++i) {
            int tier = 6, cum = 0;
            for (int t = 0; t < 6; ++t) {
                cum += c[t];
                if (i < cum) { tier = t; break; }
            }
            fmts[order[(size_t)i]] = f[tier];
        }
    }
    if (uses_mix) *uses_mix = (use_two || use_four) ? 1 : 0;
    if (counts7) {
        std::memset(counts7, 0, 7 * sizeof(int));
        for (int i = 0; i < num_blocks; ++i) {
            switch (fmts[i]) {   // src/format_planner.cpp:236-249
                case OILHIP_OIL32: counts7[0]++; break;
                case OILHIP_OIL16: case OILHIP_OIL16_GRP: counts7[1]++; break;
                case OILHIP_OIL8: case OILHIP_OIL8_GRP: counts7[2]++; break;
                case OILHIP_OIL4: case OILHIP_OIL4_GRP: counts7[3]++; break;
                case OILHIP_OIL2: case OILHIP_OIL2_GRP: counts7[4]++; break;
                case OILHIP_SPARK_Q0: case OILHIP_SPARK_Q0_GRP: case OILHIP_SPARK_SPARSE: case OILHIP_SPARK_SPARSE_GRP: counts7[5]++; break;
                default: counts7[6]++; break;
            }
        }
    }
    if (achieved_bpw) {
        float total = 0;
        for (int i = 0; i < num_blocks; ++i) total += wire_bpw(fmts[i]);
        *achieved_bpw = num_blocks ? total / (float)num_blocks : 0.0f;
    }
    return OILHIP_OK;
}

int oilhip_mix_allocate(const uint8_t* tier_fmts, int num_tiers, float effective_bpw, const float* data, int64_t n,
                        int block_size, int64_t rows, int64_t cols, uint8_t* fmts_out, int64_t* starts_out,
                        int64_t* lens_out, int64_t cap, int64_t* nblocks_out) {
    if (!tier_fmts || num_tiers <= 0 || !data || n <= 0 || !nblocks_out)
        return oilhip::fail(OILHIP_E_ARG, "mix_allocate: bad arguments");
    const int bs = block_size > 0 ? block_size : 256;
    std::vector<uint8_t> ladder(tier_fmts, tier_fmts + std::min(num_tiers, 4));
    for (uint8_t f : ladder) if (f >= OILHIP_NUM_FORMATS) return oilhip::fail(OILHIP_E_ARG, "mix_allocate: unknown format");
    std::sort(ladder.begin(), ladder.end(), [](uint8_t a, uint8_t b) { return wire_bpw(a) < wire_bpw(b); });
    ladder.erase(std::unique(ladder.begin(), ladder.end()), ladder.end());
    const int T = (int)ladder.size();
    std::vector<int64_t> seg_start, seg_len;
    if (rows > 0 && cols > 0 && cols < bs) {                 // narrow rank-2 tensors: one block per row
        const int64_t r = n / cols;
        for (int64_t i = 0; i < r; ++i) { seg_start.push_back(i * cols); seg_len.push_back(cols); }
        if (r * cols < n) { seg_start.push_back(r * cols); seg_len.push_back(n - r * cols); }
    } else {
        for (int64_t a = 0; a < n; a += bs) { seg_start.push_back(a); seg_len.push_back(std::min<int64_t>(bs, n - a)); }
    }
    const int64_t nb = (int64_t)seg_start.size();
    *nblocks_out = nb;
    if (!fmts_out) return OILHIP_OK;                          // size query
    if (cap < nb) return oilhip::fail(OILHIP_E_ARG, "mix_allocate: output arrays too small");

    // every candidate encoding of every block, decoded and compared on the device
    std::vector<uint8_t> pay;
    std::vector<oilhip_block_t> desc((size_t)(nb * T));
    std::vector<uint64_t> starts((size_t)(nb * T));
    std::vector<int64_t> bytes((size_t)(nb * T));
    std::vector<uint8_t> ibuf, cbuf;
    for (int64_t b = 0; b < nb; ++b)
        for (int t = 0; t < T; ++t) {
            const int len = (int)seg_len[(size_t)b];
            ibuf.resize(std::max<size_t>(16, oilhip_payload_bound(ladder[(size_t)t], len)));
            cbuf.resize(2 * ((size_t)len + 31) / 32 + 2);
            size_t il = 0, cl = 0;
            if (oilhip_quantize_block(ladder[(size_t)t], data + seg_start[(size_t)b], len, ibuf.data(), ibuf.size(), &il,
                                      cbuf.data(), cbuf.size(), &cl) != OILHIP_OK) return OILHIP_E_ARG;
            const size_t j = (size_t)(b * T + t);
            desc[j] = oilhip_block_t{pay.size(), pay.size() + cl, (uint32_t)cl, (uint32_t)il, (uint32_t)len, ladder[(size_t)t], {0, 0, 0}};
            pay.insert(pay.end(), cbuf.begin(), cbuf.begin() + (long)cl);
            pay.insert(pay.end(), ibuf.begin(), ibuf.begin() + (long)il);
            starts[j] = (uint64_t)seg_start[(size_t)b];
            bytes[j] = (int64_t)(il + cl);
        }
    uint64_t total_nw = 0;
    for (const auto& d : desc) total_nw += d.nw;
    oilhip_weights* h = nullptr;
    if (int rc = oilhip_weights_create(pay.data(), pay.size(), desc.data(), (uint32_t)desc.size(), 1, total_nw, &h)) return rc;
    std::vector<float> mse((size_t)(nb * T));
    float *d_data = nullptr, *d_mse = nullptr;
    uint64_t* d_start = nullptr;
    int rc = OILHIP_OK;
    auto hip = [&](hipError_t e) { if (e != hipSuccess && rc == OILHIP_OK) rc = oilhip::fail(OILHIP_E_DEVICE, hipGetErrorString(e)); };
    hip(hipMalloc(&d_data, (size_t)n * 4));
    hip(hipMalloc(&d_mse, mse.size() * 4));
    hip(hipMalloc(&d_start, starts.size() * 8));
    if (rc == OILHIP_OK) {
        hip(hipMemcpy(d_data, data, (size_t)n * 4, hipMemcpyHostToDevice));
        hip(hipMemcpy(d_start, starts.data(), starts.size() * 8, hipMemcpyHostToDevice));
        if (rc == OILHIP_OK) rc = oilhip::launch_block_mse(*h, d_data, d_start, d_mse, nullptr);
        hip(hipMemcpy(mse.data(), d_mse, mse.size() * 4, hipMemcpyDeviceToHost));
    }
    if (d_data) (void)hipFree(d_data);
    if (d_mse) (void)hipFree(d_mse);
    if (d_start) (void)hipFree(d_start);
    oilhip_weights_destroy(h);
    if (rc != OILHIP_OK) return rc;

    // greedy upgrades by error reduction per added byte under the hard byte budget
    const int64_t budget = (int64_t)std::ceil((double)effective_bpw * (double)n / 8.0);
    std::vector<int> state((size_t)nb, 0);
    int64_t used = 0;
    for (int64_t b = 0; b < nb; ++b) used += bytes[(size_t)(b * T)];
    struct Cand { float ratio; int64_t b; int t; };
    auto worse = [](const Cand& a, const Cand& c) { return a.ratio != c.ratio ? a.ratio < c.ratio : a.t < c.t; };
    std::priority_queue<Cand, std::vector<Cand>, decltype(worse)> pq(worse);
    auto offer = [&](int64_t b, int t) {
        const int cur = state[(size_t)b];
        if (t <= cur || t >= T) return;
        const int64_t added = bytes[(size_t)(b * T + t)] - bytes[(size_t)(b * T + cur)];
        if (added <= 0 || used + added > budget) return;
        const float gain = mse[(size_t)(b * T + cur)] - mse[(size_t)(b * T + t)];
        if (!(gain > 0.0f)) return;
        pq.push({gain / (float)added, b, t});
    };
    for (int64_t b = 0; b < nb; ++b) for (int t = 1; t < T; ++t) offer(b, t);
    while (!pq.empty()) {
        const Cand c = pq.top();
        pq.pop();
        const int cur = state[(size_t)c.b];
        if (c.t <= cur || c.t >= T) continue;
        const int64_t added = bytes[(size_t)(c.b * T + c.t)] - bytes[(size_t)(c.b * T + cur)];
        if (added <= 0 || used + added > budget) continue;
        if (!(mse[(size_t)(c.b * T + cur)] - mse[(size_t)(c.b * T + c.t)] > 0.0f)) continue;
        used += added;
        state[(size_t)c.b] = c.t;
        for (int t = c.t + 1; t < T; ++t) offer(c.b, t);
    }
    for (int64_t b = 0; b < nb; ++b) {
        fmts_out[b] = ladder[(size_t)state[(size_t)b]];
        if (starts_out) starts_out[b] = seg_start[(size_t)b];
        if (lens_out) lens_out[b] = seg_len[(size_t)b];
    }
    return OILHIP_OK;
}

}  // extern "C"
