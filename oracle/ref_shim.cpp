// ref_shim.cpp -- C entry points onto the *compiled reference* (checker only).
//
// This file contains no reference code: it includes the reference's public
// headers from the reference tree and forwards to its functions so that the
// Python tests and the fixture generator can call them through ctypes.  It is
// linked only into oracle/_ref/liboilref*.so, which is built only where the
// reference tree is present, and is never part of the product.
#include "oil/block_codec.h"
#include "oil/format_planner.h"
#include "oil/format_registry.h"
#include "oil/oil_format.h"
#include "oil/kernel.h"
#include "oil/kernel_production.h"
#include "oil/oil_engines.h"
#include "oil/kv_cache_oil4.h"
#include "oil/codebook.h"
#include "oil/types.h"

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <algorithm>
#include <string>
#include <vector>

namespace oil {
// internal linkage in block_codec.cpp; reached through the public pair below
}

extern "C" {

// include/oil/block_codec.h:55-56
int ref_quantize_block(int fmt, const float* w, int n,
                       uint8_t* idx, size_t idx_cap, size_t* idx_len,
                       uint8_t* cb, size_t cb_cap, size_t* cb_len) {
    std::vector<uint8_t> vi, vc;
    const bool ok = oil::quantize_block_all((oil::Format)fmt, w, n, vi, vc);
    *idx_len = vi.size();
    *cb_len = vc.size();
    if (vi.size() > idx_cap || vc.size() > cb_cap) return -1;
    if (!vi.empty()) std::memcpy(idx, vi.data(), vi.size());
    if (!vc.empty()) std::memcpy(cb, vc.data(), vc.size());
    return ok ? 1 : 0;
}

// include/oil/block_codec.h:60-63
void ref_dequantize_block(int fmt, const uint8_t* idx, size_t idx_bytes,
                          const uint8_t* cb, size_t cb_bytes, uint32_t nw, float* out) {
    oil::dequantize_block_all((oil::Format)fmt, idx, idx_bytes, cb, cb_bytes, nw, out);
}

float ref_format_bpw(int fmt) { return oil::format_bpw((oil::Format)fmt); }

// include/oil/kernel.h:24-32
void ref_oil8_gemm(const uint8_t* idx, const float* cb, const float* act, float* out,
                   int M, int N, int K) {
    oil::kernel::oil8_gemm(idx, cb, act, out, M, N, K);
}
void ref_oil4_gemm(const uint8_t* packed, const uint16_t* cb, const float* act, float* out,
                   int M, int N, int K) {
    oil::kernel::oil4_gemm(packed, cb, act, out, M, N, K);
}

// include/oil/kernel_production.h:25-52
void ref_gemv_spark(const uint8_t* w, float scale, const float* x, float* y, int M, int K) {
    oil::adapters::prod::gemv_spark_tiled(w, scale, x, y, M, K);
}
void ref_gemv_oil4(const uint8_t* w, const uint16_t* cb, float scale, const float* x, float* y,
                   int M, int K) {
    oil::adapters::prod::gemv_oil4_tiled(w, cb, scale, x, y, M, K);
}
void ref_gemv_oil8(const uint8_t* w, const float* cb, float scale, const float* x, float* y,
                   int M, int K) {
    oil::adapters::prod::gemv_oil8_tiled(w, cb, scale, x, y, M, K);
}
void ref_gemv_oil4_batch(const uint8_t* w, const uint16_t* cb, float scale, const float* X,
                         float* Y, int M, int N, int K) {
    oil::adapters::prod::gemv_oil4_batch(w, cb, scale, X, Y, M, N, K);
}

// include/oil/oil_engines.h:34-187: engines with their default codebooks.
// bits selects OIL8Engine / OIL4Engine / OIL2Engine.  cb_out receives the
// engine's codebook (256 / 16 / 4 floats).
int ref_engine_codebook(int bits, float* cb_out) {
    if (bits == 8) { oil::engines::OIL8Engine e; std::memcpy(cb_out, e.codebook().data(), e.codebook().size() * 4); return (int)e.codebook().size(); }
    if (bits == 4) { oil::engines::OIL4Engine e; std::memcpy(cb_out, e.codebook().data(), e.codebook().size() * 4); return (int)e.codebook().size(); }
    if (bits == 2) { oil::engines::OIL2Engine e; std::memcpy(cb_out, e.codebook().data(), e.codebook().size() * 4); return (int)e.codebook().size(); }
    return 0;
}

void ref_engine_quant_gemm(int bits, const float* A, const uint8_t* b_idx, float* C,
                           int64_t M, int64_t N, int64_t K) {
    oil::Tensor a({M, K});
    std::memcpy(a.data<float>(), A, (size_t)(M * K) * 4);
    oil::Tensor c;
    if (bits == 8) { oil::engines::OIL8Engine e; c = e.quant_gemm(a, b_idx, M, N, K); }
    else if (bits == 4) { oil::engines::OIL4Engine e; c = e.quant_gemm(a, b_idx, M, N, K); }
    else { oil::engines::OIL2Engine e; c = e.quant_gemm(a, b_idx, M, N, K); }
    std::memcpy(C, c.data<float>(), (size_t)(M * N) * 4);
}

// include/oil/format_planner.h:44-78.  aux = calibration activations (fisher 0, may be null)
// or gradients (fisher 1).
void ref_score_importance(const float* w, const float* aux, int64_t n, int block_size, int fisher, float* scores) {
    oil::Tensor wt({n}), at;
    std::memcpy(wt.data<float>(), w, (size_t)n * 4);
    if (aux) { at = oil::Tensor({n}); std::memcpy(at.data<float>(), aux, (size_t)n * 4); }
    oil::FormatPlanner pl(1.5f);
    pl.score_importance(wt, at, block_size, fisher ? oil::ImportanceMetric::FISHER_DIAG : oil::ImportanceMetric::MAGNITUDE);
    std::memcpy(scores, pl.importance_scores().data(), pl.importance_scores().size() * 4);
}

// FormatPlanner::allocate with scores planted through score_importance on |w| = score, a = null
// (mean of one weight per block reproduces the score exactly with block_size 1).
void ref_plan_allocate(float target, const float* scores, int64_t nscores, int nb, uint8_t* fmts,
                       float* achieved, float* estimated, int* uses_mix, int* counts7) {
    oil::FormatPlanner pl(target);
    if (scores && nscores > 0) {
        oil::Tensor wt({nscores}), at;
        std::memcpy(wt.data<float>(), scores, (size_t)nscores * 4);
        pl.score_importance(wt, at, 1, oil::ImportanceMetric::MAGNITUDE);
    }
    oil::FormatPlan plan = pl.allocate(nb, 256);
    for (int i = 0; i < nb; ++i) fmts[i] = (uint8_t)plan.blocks[(size_t)i].assigned_format;
    *achieved = plan.achieved_bpw;
    *estimated = oil::FormatPlanner::estimate_bpw(plan);
    *uses_mix = plan.uses_mix ? 1 : 0;
    counts7[0] = plan.num_oil32_blocks; counts7[1] = plan.num_oil16_blocks; counts7[2] = plan.num_oil8_blocks;
    counts7[3] = plan.num_oil4_blocks; counts7[4] = plan.num_oil2_blocks; counts7[5] = plan.num_spark_blocks;
    counts7[6] = plan.num_oil1_blocks;
}

// FormatRegistry::allocate_mix_blocks for a registry mix selected by name
// ("SPARK_MIX_Q0", "QUAD_SPARK_Q1", ...).  Returns the block count, -1 for an unknown name.
int64_t ref_mix_allocate(const char* mix_name, const float* data, int64_t n, int block_size, int64_t rows, int64_t cols,
                         uint8_t* fmts, int64_t* starts, int64_t* lens, int64_t cap, float* eff_bpw, uint8_t* tiers4, int* ntiers) {
    const oil::MixDescriptor* m = nullptr;
    for (const auto& x : oil::FormatRegistry::get_all_twi_mixes()) if (x.name == mix_name) m = &x;
    for (const auto& x : oil::FormatRegistry::get_all_four_mixes()) if (x.name == mix_name) m = &x;
    if (!m) return -1;
    if (eff_bpw) *eff_bpw = m->effective_bpw;
    if (ntiers) *ntiers = m->num_tiers;
    if (tiers4) {
        const oil::RegFormat t[4] = {m->tier1_fmt, m->tier2_fmt, m->tier3_fmt, m->tier4_fmt};
        for (int i = 0; i < 4; ++i) tiers4[i] = (uint8_t)oil::regformat_to_format(t[i]);
    }
    std::vector<int64_t> shape = {rows, cols};
    auto plan = oil::FormatRegistry::allocate_mix_blocks(*m, data, n, block_size, rows > 0 ? &shape : nullptr);
    const int64_t nb = (int64_t)plan.formats.size();
    for (int64_t b = 0; b < nb && b < cap; ++b) {
        fmts[b] = (uint8_t)plan.formats[(size_t)b];
        starts[b] = plan.block_starts[(size_t)b];
        lens[b] = plan.block_lens[(size_t)b];
    }
    return nb;
}

// registry tables, for checking the product's copies: kind 0 singles, 1 two-tier mixes, 2 four-tier mixes
int ref_registry_row(int kind, int i, char* name, int cap, float* bpw, uint8_t* tiers4, float* ratios4, int* ntiers) {
    if (kind == 0) {
        const auto& v = oil::FormatRegistry::get_all_singles();
        if (i >= (int)v.size()) return 0;
        std::snprintf(name, (size_t)cap, "%s", v[(size_t)i].name.c_str());
        *bpw = v[(size_t)i].bpw; *ntiers = 1;
        tiers4[0] = (uint8_t)oil::regformat_to_format(v[(size_t)i].id);
        return 1;
    }
    const auto& v = kind == 1 ? oil::FormatRegistry::get_all_twi_mixes() : oil::FormatRegistry::get_all_four_mixes();
    if (i >= (int)v.size()) return 0;
    const auto& m = v[(size_t)i];
    std::snprintf(name, (size_t)cap, "%s", m.name.c_str());
    *bpw = m.effective_bpw; *ntiers = m.num_tiers;
    const oil::RegFormat t[4] = {m.tier1_fmt, m.tier2_fmt, m.tier3_fmt, m.tier4_fmt};
    const float r[4] = {m.tier1_ratio, m.tier2_ratio, m.tier3_ratio, m.tier4_ratio};
    for (int k = 0; k < 4; ++k) { tiers4[k] = (uint8_t)oil::regformat_to_format(t[k]); ratios4[k] = r[k]; }
    return 1;
}

// OILWriter in the reference's own call order (tests/test_spark_mix.cpp:344-384): header, format
// table, tensor table, blocks.  Block b of the file encodes data[starts[b] .. +lens[b]) as fmts[b].
int ref_oil_write(const char* path, uint32_t version, uint32_t flags, const uint8_t* config, uint32_t config_size,
                  uint32_t ntensors, const char* const* names, const uint32_t* tensor_blocks, const float* data,
                  const uint8_t* fmts, const int64_t* starts, const int64_t* lens, uint32_t nblocks) {
    oil::OILWriter writer(path);
    oil::OILHeader hdr;
    std::memcpy(hdr.magic, "OIL1", 4);
    hdr.version = version; hdr.flags = flags; hdr.config_size = config_size;
    writer.write_header(hdr, config);
    std::vector<oil::FormatBlockEntry> ft;
    std::vector<oil::TensorEntry> te;
    std::vector<std::string> nm;
    std::vector<oil::BlockData> blocks;
    uint32_t id = 0;
    for (uint32_t t = 0; t < ntensors; ++t) {
        nm.push_back(names[t]);
        oil::TensorEntry e;
        e.name_len = (uint16_t)nm.back().size(); e.block_start = id; e.num_blocks = tensor_blocks[t];
        te.push_back(e);
        for (uint32_t b = 0; b < tensor_blocks[t]; ++b, ++id) {
            oil::BlockData blk;
            blk.format = (oil::Format)fmts[id];
            blk.num_weights = (uint32_t)lens[id];
            if (!oil::quantize_block_all(blk.format, data + starts[id], (int)lens[id], blk.indices, blk.codebook)) return -1;
            oil::FormatBlockEntry fe;
            fe.block_id = id; fe.format = fmts[id]; fe.cb_bytes = (uint32_t)blk.codebook.size();
            ft.push_back(fe);
            blocks.push_back(std::move(blk));
        }
    }
    if (id != nblocks) return -2;
    writer.write_format_table(ft);
    writer.write_tensor_table(te, nm);
    for (auto& b : blocks) writer.write_block(b);
    writer.close();
    return 0;
}

// OILReader::read_tensor; returns numel (or -1 when the file does not open / has no such tensor).
int64_t ref_oil_read_tensor(const char* path, const char* name, float* out, int64_t cap) {
    oil::OILReader r(path);
    if (!r.valid()) return -1;
    oil::Tensor t = r.read_tensor(name);
    const int64_t n = t.numel();
    if (n <= 0) return -1;
    if (out) std::memcpy(out, t.data<float>(), (size_t)std::min(n, cap) * 4);
    return n;
}

// OILReader metadata: block count, tensor count, and tensor_blocks() of one name.
int ref_oil_meta(const char* path, const char* name, uint32_t* nblocks, uint32_t* ntensors, uint32_t* start, uint32_t* count) {
    oil::OILReader r(path);
    if (!r.valid()) return -1;
    *nblocks = (uint32_t)r.num_blocks();
    *ntensors = (uint32_t)r.tensor_names().size();
    if (name && !r.tensor_blocks(name, *start, *count)) return -2;
    return 0;
}

// Oil1Engine / SparkEngine / OIL16Engine / OIL32Engine::quant_gemm (include/oil/oil_engines.h:103,123,167).
// b holds the engine's packed operand verbatim (floats, 2-bit codes, FP16 bits, floats).
void ref_engine_dense_gemm(int kind, const float* A, const void* b, size_t b_bytes, const float* scales, int64_t nscales,
                           int64_t block, float* C, int64_t M, int64_t N, int64_t K) {
    oil::Tensor a({M, K});
    std::memcpy(a.data<float>(), A, (size_t)(M * K) * 4);
    oil::Tensor c;
    if (kind == 16) {
        oil::Tensor bt({(int64_t)(b_bytes / 2)}, oil::DType::F16);
        std::memcpy(bt.data<uint16_t>(), b, b_bytes);
        oil::engines::OIL16Engine e;
        c = e.quant_gemm(a, bt, M, N, K);
    } else {
        oil::Tensor bt({(int64_t)((b_bytes + 3) / 4)});
        std::memcpy(bt.data<float>(), b, b_bytes);
        if (kind == 1) { oil::engines::Oil1Engine e; c = e.quant_gemm(a, bt, 1.0f, M, N, K); }
        else if (kind == 32) { oil::engines::OIL32Engine e; c = e.quant_gemm(a, bt, M, N, K); }
        else {
            oil::Tensor st({nscales});
            std::memcpy(st.data<float>(), scales, (size_t)nscales * 4);
            oil::engines::SparkEngine e(block);
            c = e.quant_gemm(a, bt, st, M, N, K);
        }
    }
    std::memcpy(C, c.data<float>(), (size_t)(M * N) * 4);
}

// dequant_tensor (scales null) / dequantize_per_block of the engines with their default codebooks.
void ref_engine_dequant(int bits, const uint8_t* idx, int64_t n, const float* scales, int64_t block, float* out) {
    if (!scales) {
        oil::Tensor t;
        if (bits == 8) { oil::engines::OIL8Engine e; t = e.dequant_tensor(idx, n); }
        else if (bits == 4) { oil::engines::OIL4Engine e; t = e.dequant_tensor(idx, n); }
        else { oil::engines::OIL2Engine e; t = e.dequant_tensor(idx, n); }
        std::memcpy(out, t.data<float>(), (size_t)n * 4);
    } else if (bits == 8) {
        oil::engines::OIL8Engine e; e.dequantize_per_block(idx, scales, n, block, out);
    } else {
        oil::engines::OIL4Engine e; e.dequantize_per_block(idx, scales, n, block, out);
    }
}

// include/oil/kernel.h:11-18: tl1_gemm (kind 1) / tl2_gemm (kind 2) over host arrays wrapped in tensors
void ref_tl_gemm(int kind, const uint8_t* w, size_t w_bytes, const float* a, float* out, int M, int N, int K) {
    oil::Tensor wt(oil::Shape{(int64_t)w_bytes}, oil::DType::U8), at(oil::Shape{(int64_t)N, (int64_t)K}), ot(oil::Shape{(int64_t)M, (int64_t)N});
    std::memcpy(wt.data<uint8_t>(), w, w_bytes);
    std::memcpy(at.data<float>(), a, sizeof(float) * (size_t)N * (size_t)K);
    if (kind == 1) oil::kernel::tl1_gemm(wt, at, ot, M, N, K);
    else oil::kernel::tl2_gemm(wt, at, ot, M, N, K);
    std::memcpy(out, ot.data<float>(), sizeof(float) * (size_t)M * (size_t)N);
}

// CodebookOIL4::half_to_float / float_to_half (include/oil/codebook.h:79-80)
float ref_kv_half_to_float(uint16_t h) { return oil::CodebookOIL4::half_to_float(h); }
uint16_t ref_kv_float_to_half(float f) { return oil::CodebookOIL4::float_to_half(f); }

// OIL4KVCache::quantize_block_oil4 / dequantize_block_oil4 (include/oil/kv_cache_oil4.h:52-57): one code per byte
void ref_kv_quantize_block(const float* src, int64_t n, uint16_t* cb16, uint8_t* codes) {
    oil::OIL4KVCache::quantize_block_oil4(src, codes, cb16, n);
}
void ref_kv_dequantize_block(const uint8_t* codes, const uint16_t* cb16, float* dst, int64_t n) {
    oil::OIL4KVCache::dequantize_block_oil4(codes, cb16, dst, n);
}

// One OIL4KVCache: n_appends calls of append(layer, k, v) with seq_lens[i] tokens each (k and v hold the tokens of
// all calls back to back, [token][heads * dim]), then get_range(layer, start, end).  Returns the number of tokens
// get_range gave back; size_bytes / context_len as the cache reports them.
int64_t ref_kv_run(int layers, int64_t max_seq, int64_t heads, int64_t dim, int64_t block, int layer,
                   const float* k, const float* v, const int64_t* seq_lens, int n_appends,
                   int64_t start, int64_t end, float* k_out, float* v_out, uint64_t* size_bytes, int* context_len) {
    oil::OIL4KVCache cache(layers, max_seq, heads, dim, block);
    const int64_t per_token = heads * dim;
    int64_t at = 0;
    for (int a = 0; a < n_appends; ++a) {
        const int64_t s = seq_lens[a];
        oil::Tensor kt(oil::Shape{1, heads, s, dim}), vt(oil::Shape{1, heads, s, dim});
        std::memcpy(kt.data<float>(), k + at * per_token, (size_t)(s * per_token) * 4);
        std::memcpy(vt.data<float>(), v + at * per_token, (size_t)(s * per_token) * 4);
        cache.append(layer, kt, vt);
        at += s;
    }
    if (size_bytes) *size_bytes = cache.size_bytes();
    if (context_len) *context_len = cache.context_len();
    auto kv = cache.get_range(layer, start, end);
    if (kv.first.numel() == 0) return 0;
    const int64_t len = kv.first.shape().dims[2];
    std::memcpy(k_out, kv.first.data<float>(), (size_t)(len * per_token) * 4);
    std::memcpy(v_out, kv.second.data<float>(), (size_t)(len * per_token) * 4);
    return len;
}

}  // extern "C"
