// moe.hip -- mixture-of-experts step over quantized experts: routing on the host, batched expert
// feed-forward on the device.  Counterparts: softmax_with_topk (src/moe_variants.cpp:97-134),
// moe_dispatch_batched (:767-827) and ExpertFFN::forward with SiLU (:77-91), with each expert's
// three projections held as .oil tensors (Y = X W^T, no bias) instead of dense FP32 Linear layers.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <utility>
#include <vector>

#include "common.h"

namespace oilhip {
namespace {

__global__ void __launch_bounds__(256) fill_zero_kernel(float* __restrict__ p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) p[i] = 0.0f;
}

// three ranges in one launch (what a grouped step needs cleared before its first kernel)
__global__ void __launch_bounds__(256) fill_zero3_kernel(float* __restrict__ a, size_t na, float* __restrict__ b, size_t nb,
                                                         float* __restrict__ c, size_t nc) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < na + nb + nc; i += (size_t)gridDim.x * 256) {
        if (i < na) a[i] = 0.0f;
        else if (i < na + nb) b[i - na] = 0.0f;
        else c[i - na - nb] = 0.0f;
    }
}

// h = silu(g) * u, silu(v) = v / (1 + exp(-v))  (src/math.cpp:117-126)
__global__ void __launch_bounds__(256) swiglu_kernel(float* __restrict__ g, const float* __restrict__ u, size_t n) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
        const float v = g[i];
        g[i] = (v / (1.0f + expf(-v))) * u[i];
    }
}

// x rows picked by tok[] into a dense [nt][D] batch (experts in formats without a gathering kernel)
__global__ void __launch_bounds__(256) gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ tok,
                                                          float* __restrict__ out, uint32_t D) {
    const float* src = x + (size_t)tok[blockIdx.x] * D;
    float* dst = out + (size_t)blockIdx.x * D;
    for (uint32_t d = threadIdx.x; d < D; d += 256) dst[d] = src[d];
}

// out[tok[i]][d] += wgt[i] * o[i][d] in list order (one thread per column walks the expert's rows, so a
// token listed twice is added twice, in order); the squared contributions feed the z-loss sum.
__global__ void __launch_bounds__(256) combine_kernel(const float* __restrict__ o, const int* __restrict__ tok,
                                                      const float* __restrict__ wgt, int nt, uint32_t D,
                                                      float* __restrict__ out, double* __restrict__ zacc) {
    __shared__ double part[4];
    const uint32_t d = blockIdx.x * 256 + threadIdx.x;
    double z = 0.0;
    if (d < D) {
        for (int i = 0; i < nt; ++i) {
            const float w = wgt[i];
            if (!(w > 0.0f)) continue;
            const float v = w * o[(size_t)i * D + d];
            out[(size_t)tok[i] * D + d] += v;
            z += (double)v * (double)v;
        }
    }
    for (int off = 32; off > 0; off >>= 1) z += __shfl_xor(z, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = z;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(zacc, (part[0] + part[1]) + (part[2] + part[3]));
}

// The same for a list without repeated tokens (what top-k routing produces): every (row, column) of the list has an
// output element of its own, so the rows go side by side, blockIdx.y = list entry.
__global__ void __launch_bounds__(256) combine_distinct_kernel(const float* __restrict__ o, const int* __restrict__ tok,
                                                               const float* __restrict__ wgt, uint32_t D,
                                                               float* __restrict__ out, double* __restrict__ zacc) {
    __shared__ double part[4];
    const uint32_t d = blockIdx.x * 256 + threadIdx.x, i = blockIdx.y;
    const float w = wgt[i];
    double z = 0.0;
    if (d < D && w > 0.0f) {
        const float v = w * o[(size_t)i * D + d];
        out[(size_t)tok[i] * D + d] += v;
        z = (double)v * (double)v;
    }
    for (int off = 32; off > 0; off >>= 1) z += __shfl_xor(z, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = z;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(zacc, (part[0] + part[1]) + (part[2] + part[3]));
}

// The grouped path's combine: every token's contributions in the order the reference adds them (ascending expert,
// then list order), out[t][d] written once.  The lists travel by value with the launch.
constexpr int kMaxPairs = 448;
struct CombineLists {
    int K;
    int16_t pair[kMaxPairs];    // pair[t * K + k]: row of o behind the k-th contribution of token t, or -1
    uint8_t nparts[kMaxPairs];  // nparts[row of o]: K parts of that row left in `parts` by the down projection (0: the row is in o)
    float wgt[kMaxPairs];       // its weight (<= 0: dropped)
};

static_assert(sizeof(CombineLists) <= 3584, "the lists travel in the kernel arguments (4 KB with the other arguments)");

// zacc == nullptr: the caller does not want the z-loss, and the workgroups skip their atomic on its one address.
// Rows whose down projection was cut into three or more K parts arrive as those parts (parts[p * pstride + row * D + d])
// and are summed here in ascending part order: the sum does not depend on the order in which workgroups ran.
__global__ void __launch_bounds__(256) combine_grouped_kernel(const float* __restrict__ o, const float* __restrict__ parts, uint32_t pstride,
                                                              uint32_t D, float* __restrict__ out, double* __restrict__ zacc,
                                                              const CombineLists L) {
    __shared__ double part[4];
    const uint32_t d = blockIdx.x * 256 + threadIdx.x, t = blockIdx.y;
    double z = 0.0;
    if (d < D) {
        float sum = 0.0f;
        for (int k = 0; k < L.K; ++k) {
            const int i = L.pair[t * L.K + k];
            const float w = L.wgt[t * L.K + k];
            if (i < 0 || !(w > 0.0f)) continue;
            float y = 0.0f;
            const uint32_t np = L.nparts[i];
            if (np == 0u) y = o[(size_t)i * D + d];
            for (uint32_t p = 0; p < np; ++p) y += parts[(size_t)p * pstride + (size_t)i * D + d];
            const float v = w * y;
            sum += v;
            z += (double)v * (double)v;
        }
        out[(size_t)t * D + d] = sum;
    }
    if (!zacc) return;                                     // uniform over the grid
    for (int off = 32; off > 0; off >>= 1) z += __shfl_xor(z, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = z;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(zacc, (part[0] + part[1]) + (part[2] + part[3]));
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

struct Workspace {
    int* tok; float* wgt; float* g; float* u; float* o; float* xg; float* parts; double* z; uint8_t* batch;
    size_t bytes, batch_bytes;
};

constexpr int kChunk = 16;      // expert batches per grouped launch (gate and up together are 32 tensors)

// scratch of one grouped launch: the larger of the gate/up side (rows F, cols D) and the down side (rows D, cols F)
size_t batch_scratch_bytes(int64_t D, int64_t F) {
    return std::max(gemv_oil4_multi_batches_bytes(kChunk, (uint64_t)F, (uint64_t)D, true), gemv_oil4_multi_batches_bytes(kChunk, (uint64_t)D, (uint64_t)F, false));
}

// the most K parts a row of F weights is cut into, over the pass sizes; 0 when no pass size cuts it in three or more
uint32_t down_parts_max(int64_t F) {
    uint32_t m = 0;
    for (int kind = 0; kind < 3; ++kind) m = std::max(m, gemv_oil4_multi_parts(kind, (uint64_t)F));
    return m > 2u ? m : 0u;
}

Workspace carve(void* base, int64_t pairs, int64_t D, int64_t F) {
    Workspace w{};
    uint8_t* p = (uint8_t*)base;
    size_t off = 0;
    auto take = [&](size_t n) { uint8_t* r = p ? p + off : nullptr; off += align256(n); return r; };
    w.z = (double*)take(8);
    w.tok = (int*)take((size_t)pairs * 4);
    w.wgt = (float*)take((size_t)pairs * 4);
    w.g = (float*)take((size_t)pairs * F * 4);
    w.u = (float*)take((size_t)pairs * F * 4);
    w.o = (float*)take((size_t)pairs * D * 4);
    w.xg = (float*)take((size_t)pairs * D * 4);
    w.batch_bytes = (D % 256 == 0 && F % 256 == 0 && D <= 32768 && F <= 32768) ? batch_scratch_bytes(D, F) : 0;
    w.batch = take(w.batch_bytes);
    // K parts of the down projections' outputs (rows of F weights cut into three or more parts), summed by the combine
    w.parts = (float*)take(w.batch_bytes ? (size_t)down_parts_max(F) * pairs * D * 4 : 0);
    w.bytes = off;
    return w;
}

// one projection of an expert batch: Y[nt][rows] from rows tok[] of X (or X itself when tok is null)
int expert_gemv(const oilhip_weights& w, const float* d_x, const int* d_tok, float* d_y, int nt, uint32_t xrows,
                float* d_gather, hipStream_t s) {
    if (plain_oil4(w)) {
        const int rc = launch_gemv_oil4_multi(w, d_x, d_tok, d_y, nt, (uint32_t)w.cols, (uint32_t)w.rows, xrows, s);
        if (rc <= 0) return rc;
    }
    const float* xin = d_x;
    if (d_tok) {
        hipLaunchKernelGGL(gather_rows_kernel, dim3((uint32_t)nt), dim3(256), 0, s, d_x, d_tok, d_gather, (uint32_t)w.cols);
        OILHIP_HIP(hipGetLastError());
        xin = d_gather;
    }
    return oilhip_gemv_f32(&w, xin, d_y, nt, s);      // every other format and mixed rows: the decode GEMV's own routing
}

}  // namespace
}  // namespace oilhip

using namespace oilhip;

extern "C" {

int oilhip_moe_route(const float* logits, int64_t T, int64_t E, int64_t k, float* probs, int64_t* indices, float* weights) {
    if (!logits || !probs || !indices || !weights || T < 0 || E <= 0 || k <= 0 || k > E)
        return fail(OILHIP_E_ARG, "moe_route: bad arguments");
    std::vector<std::pair<float, int64_t>> scored;
    for (int64_t t = 0; t < T; ++t) {
        const float* l = logits + t * E;
        float* p = probs + t * E;
        float maxv = l[0];
        for (int64_t e = 1; e < E; ++e) if (l[e] > maxv) maxv = l[e];
        float sum = 0.0f;
        for (int64_t e = 0; e < E; ++e) { const float v = std::exp(l[e] - maxv); p[e] = v; sum += v; }
        const float inv = 1.0f / sum;
        for (int64_t e = 0; e < E; ++e) p[e] *= inv;
        scored.clear();
        for (int64_t e = 0; e < E; ++e) scored.push_back({p[e], e});
        std::partial_sort(scored.begin(), scored.begin() + k, scored.end(),
                          [](const auto& a, const auto& b) { return a.first > b.first; });
        for (int64_t j = 0; j < k; ++j) { indices[t * k + j] = scored[(size_t)j].second; weights[t * k + j] = scored[(size_t)j].first; }
    }
    return OILHIP_OK;
}

size_t oilhip_moe_workspace_bytes(int64_t T, int64_t K, int64_t D, int64_t F) {
    if (T <= 0 || K <= 0 || D <= 0 || F <= 0) return 0;
    return carve(nullptr, T * K, D, F).bytes;
}

int oilhip_moe_forward(const oilhip_weights* const* gate, const oilhip_weights* const* up,
                       const oilhip_weights* const* down, int E, const float* d_x, const int64_t* indices,
                       const float* weights, int64_t T, int64_t K, float* d_out, void* d_workspace,
                       size_t workspace_bytes, float* z_loss, int64_t* dropped, void* stream) {
    if (!gate || !up || !down || E <= 0 || !d_x || !indices || !weights || T <= 0 || K <= 0 || !d_out || !d_workspace)
        return fail(OILHIP_E_ARG, "moe_forward: bad arguments");
    for (int e = 0; e < E; ++e)
        if (!gate[e] || !up[e] || !down[e]) return fail(OILHIP_E_ARG, "moe_forward: null expert tensor");
    const int64_t D = (int64_t)gate[0]->cols, F = (int64_t)gate[0]->rows;
    for (int e = 0; e < E; ++e) {
        if ((int64_t)gate[e]->cols != D || (int64_t)gate[e]->rows != F || (int64_t)up[e]->cols != D || (int64_t)up[e]->rows != F ||
            (int64_t)down[e]->cols != F || (int64_t)down[e]->rows != D)
            return fail(OILHIP_E_ARG, "moe_forward: expert " + std::to_string(e) + " has mismatched shapes");
        for (const oilhip_weights* w : {gate[e], up[e], down[e]})
            if (!w->all_full || (w->cols & 255)) return fail(OILHIP_E_ARG, "moe_forward: expert tensors need full 256-weight blocks");
    }
    if (T * K > 0x7FFFFFFF || T > 0x7FFFFFFF) return fail(OILHIP_E_ARG, "moe_forward: too many (token, expert) pairs");
    const Workspace ws = carve(d_workspace, T * K, D, F);
    if (workspace_bytes < ws.bytes) return fail(OILHIP_E_ARG, "moe_forward: workspace too small");
    hipStream_t s = (hipStream_t)stream;

    // tokens per expert in ascending token order, each with the weight of its first matching slot
    std::vector<int> tok;
    std::vector<float> wgt;
    std::vector<int> begin((size_t)E + 1, 0);
    int64_t drop = 0;
    for (int e = 0; e < E; ++e) {
        begin[(size_t)e] = (int)tok.size();
        for (int64_t t = 0; t < T; ++t)
            for (int64_t k = 0; k < K; ++k)
                if (indices[t * K + k] == e) {
                    float w = 0.0f;
                    for (int64_t k2 = 0; k2 < K; ++k2) if (indices[t * K + k2] == e) { w = weights[t * K + k2]; break; }
                    if (!(w > 0.0f)) drop++;
                    tok.push_back((int)t);
                    wgt.push_back(w);
                }
    }
    begin[(size_t)E] = (int)tok.size();
    // a list is in ascending token order, so a token listed twice sits next to itself
    std::vector<char> distinct((size_t)E, 1);
    for (int e = 0; e < E; ++e)
        for (int i = begin[(size_t)e] + 1; i < begin[(size_t)e + 1]; ++i)
            if (tok[(size_t)i] == tok[(size_t)i - 1]) distinct[(size_t)e] = 0;
    if (dropped) *dropped = drop;
    // ---- grouped path: uniform OIL4 experts, lists small enough to travel with the launches ---------------------
    // Per chunk of expert batches (passes of 32, 16 and 8 tokens side by side): one launch that splits the gathered
    // activations, one launch over the gate and up projections of all those experts, one that forms silu(gate) * up
    // while splitting it, one over their down projections; then one combine.  No copy, no synchronisation: the step can
    // be captured.
    bool grouped = ws.batch_bytes > 0 && (int64_t)tok.size() <= kMaxPairs && T * K <= kMaxPairs && !tok.empty();
    for (int e = 0; e < E && grouped; ++e) grouped = plain_oil4(*gate[e]) && plain_oil4(*up[e]) && plain_oil4(*down[e]);
    if (grouped) {
        const int64_t pairs = (int64_t)tok.size();
        // the z-loss accumulator and the slab counters at the start of the batch workspace start at zero (every launch
        // leaves the counters at zero again); outputs that row parts add into are cleared by the launch that splits
        // the activations
        // (the launch is skipped when nothing needs it: no z-loss asked for, and no launch of the step counts arrivals --
        // the gate/up rows are cut in at most two parts and the down projections leave their parts to the combine)
        const bool parts_mode = gemv_oil4_multi_ordered() && down_parts_max(F) > 0u;
        const bool counters = gemv_oil4_multi_ordered() && (down_parts_max(D) > 0u || (down_parts_max(F) > 0u && !parts_mode));
        if (z_loss || counters) {
            hipLaunchKernelGGL(fill_zero3_kernel, dim3(64), dim3(256), 0, s, ws.g, (size_t)0, (float*)ws.z, (size_t)2, (float*)ws.batch,
                               kGemvBatchCounterBytes / 4);
            OILHIP_HIP(hipGetLastError());
        }
        // down projections cut into three or more K parts leave the parts to the combine (parts_mode: ordered sums; with
        // the atomic sums switched on they add into their outputs instead)
        struct Batch { int e, pair0, m, kind; };
        std::vector<Batch> batches;
        for (int pass = 2; pass >= 0; --pass)                     // the longest passes first: they end last
            for (int e = 0; e < E; ++e) {
                int n = begin[(size_t)e + 1] - begin[(size_t)e], pos = begin[(size_t)e];
                while (n > 0) {
                    // more than 16 tokens: a pass of 32 (its table reads serve two token tiles: 1.36 times the cost of a
                    // pass of 16); then what is left as a pass of 16 or of 8
                    const int take = n > 32 ? 32 : n, kind = take <= 8 ? 0 : take <= 16 ? 1 : 2;
                    if (kind == pass) batches.push_back(Batch{e, pos, take, kind});
                    pos += take; n -= take;
                }
            }
        // all pass sizes of a chunk of batches share one launch per side: one launch that splits the gathered
        // activations, one over the gate and up projections, one that forms silu(gate) * up while splitting it, one
        // over the down projections
        for (size_t c0 = 0; c0 < batches.size(); c0 += kChunk) {
            const int nb = (int)std::min<size_t>(kChunk, batches.size() - c0);
            const oilhip_weights *wg[kChunk], *wu[kChunk], *wd[kChunk];
            float *yg[kChunk], *yu[kChunk], *yo[kChunk];
            int Mb[kChunk], r0[kChunk], kd[kChunk];
            for (int b = 0; b < nb; ++b) {
                const Batch& B = batches[c0 + b];
                wg[b] = gate[B.e]; wu[b] = up[B.e]; wd[b] = down[B.e];
                yg[b] = ws.g + (size_t)B.pair0 * F; yu[b] = ws.u + (size_t)B.pair0 * F; yo[b] = ws.o + (size_t)B.pair0 * D;
                Mb[b] = B.m; r0[b] = B.pair0; kd[b] = B.kind;
            }
            int rc = launch_gemv_oil4_multi_batches(nb, kd, wg, yg, wu, yu, Mb, r0, tok.data(), (int)tok.size(), d_x, nullptr,
                                                    (uint32_t)D, (uint32_t)T, (uint32_t)F, ws.batch, ws.batch_bytes, s, true);
            if (rc == 0)
                rc = launch_gemv_oil4_multi_batches(nb, kd, wd, yo, nullptr, nullptr, Mb, r0, nullptr, 0, ws.g, ws.u,
                                                    (uint32_t)F, (uint32_t)pairs, (uint32_t)D, ws.batch, ws.batch_bytes, s, true,
                                                    parts_mode ? ws.parts : nullptr, (uint32_t)pairs);
            if (rc < 0) return rc;
            if (rc == 1) return fail(OILHIP_E_ARG, "moe_forward: the grouped launch refused a shape it was planned for");
        }
        CombineLists L{};
        L.K = (int)K;
        for (int64_t i = 0; i < T * K; ++i) { L.pair[i] = -1; L.wgt[i] = 0.0f; }
        for (const Batch& B : batches) {
            const uint32_t np = parts_mode ? gemv_oil4_multi_parts(B.kind, (uint64_t)F) : 0u;
            for (int m = 0; m < B.m; ++m) L.nparts[B.pair0 + m] = (uint8_t)(np > 2u ? np : 0u);
        }
        std::vector<int> filled((size_t)T, 0);
        for (int e = 0; e < E; ++e)                      // ascending expert, list order: the order of the reference's additions
            for (int i = begin[(size_t)e]; i < begin[(size_t)e + 1]; ++i) {
                const int t = tok[(size_t)i];
                L.pair[t * K + filled[(size_t)t]] = (int16_t)i;
                L.wgt[t * K + filled[(size_t)t]] = wgt[(size_t)i];
                filled[(size_t)t]++;
            }
        hipLaunchKernelGGL(combine_grouped_kernel, dim3((uint32_t)((D + 255) / 256), (uint32_t)T), dim3(256), 0, s, ws.o, ws.parts,
                           (uint32_t)(pairs * D), (uint32_t)D, d_out, z_loss ? ws.z : (double*)nullptr, L);
        OILHIP_HIP(hipGetLastError());
        if (z_loss) {
            double z = 0.0;
            OILHIP_HIP(hipMemcpyAsync(&z, ws.z, 8, hipMemcpyDeviceToHost, s));
            OILHIP_HIP(hipStreamSynchronize(s));
            *z_loss = (float)z;
        }
        return OILHIP_OK;
    }
    if (!tok.empty()) {
        OILHIP_HIP(hipMemcpyAsync(ws.tok, tok.data(), tok.size() * 4, hipMemcpyHostToDevice, s));
        OILHIP_HIP(hipMemcpyAsync(ws.wgt, wgt.data(), wgt.size() * 4, hipMemcpyHostToDevice, s));
        OILHIP_HIP(hipStreamSynchronize(s));          // the host vectors go out of scope
    }
    hipLaunchKernelGGL(fill_zero_kernel, dim3(256), dim3(256), 0, s, d_out, (size_t)(T * D));
    hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(256), 0, s, (float*)ws.z, (size_t)2);
    OILHIP_HIP(hipGetLastError());
    for (int e = 0; e < E; ++e) {
        const int b = begin[(size_t)e], nt = begin[(size_t)e + 1] - b;
        if (nt == 0) continue;
        // gate and up read the same gathered activations: uniform OIL4 experts split them once per pass for both
        int both = 1;
        if (plain_oil4(*gate[e]))
            both = launch_gemv_oil4_multi(*gate[e], d_x, ws.tok + b, ws.g, nt, (uint32_t)D, (uint32_t)F, (uint32_t)T, s, up[e], ws.u,
                                          (uint32_t)F);
        if (both < 0) return both;
        if (both == 1) {
            if (int rc = expert_gemv(*gate[e], d_x, ws.tok + b, ws.g, nt, (uint32_t)T, ws.xg, s)) return rc;
            if (int rc = expert_gemv(*up[e], d_x, ws.tok + b, ws.u, nt, (uint32_t)T, ws.xg, s)) return rc;
        }
        // silu(gate) * up: formed while the down projection's activations are split (uniform OIL4), or by a kernel of its own
        int fused = 1;
        if (plain_oil4(*down[e]))
            fused = launch_gemv_oil4_multi(*down[e], ws.g, nullptr, ws.o, nt, (uint32_t)F, (uint32_t)D, (uint32_t)nt, s, nullptr, nullptr, 0,
                                           ws.u);
        if (fused < 0) return fused;
        if (fused == 1) {
            const size_t n = (size_t)nt * (size_t)F;
            hipLaunchKernelGGL(swiglu_kernel, dim3((uint32_t)std::min<size_t>((n + 255) / 256, 4096)), dim3(256), 0, s, ws.g, ws.u, n);
            OILHIP_HIP(hipGetLastError());
            if (int rc = expert_gemv(*down[e], ws.g, nullptr, ws.o, nt, (uint32_t)nt, ws.xg, s)) return rc;
        }
        if (distinct[(size_t)e])
            hipLaunchKernelGGL(combine_distinct_kernel, dim3((uint32_t)((D + 255) / 256), (uint32_t)nt), dim3(256), 0, s, ws.o, ws.tok + b,
                               ws.wgt + b, (uint32_t)D, d_out, ws.z);
        else
            hipLaunchKernelGGL(combine_kernel, dim3((uint32_t)((D + 255) / 256)), dim3(256), 0, s, ws.o, ws.tok + b, ws.wgt + b, nt,
                               (uint32_t)D, d_out, ws.z);
        OILHIP_HIP(hipGetLastError());
    }
    if (dropped) *dropped = drop;
    if (z_loss) {
        double z = 0.0;
        OILHIP_HIP(hipMemcpyAsync(&z, ws.z, 8, hipMemcpyDeviceToHost, s));
        OILHIP_HIP(hipStreamSynchronize(s));
        *z_loss = (float)z;
    }
    return OILHIP_OK;
}

}  // extern "C"
