// api.hip -- C ABI of liboilhip: error text, device probe, weight upload, dispatch.
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <algorithm>
#include <map>
#include <tuple>
#include <queue>
#include <vector>

#include "common.h"
#include "run_decode.h"

namespace oilhip {

static thread_local std::string g_err;

void set_error(const std::string& msg) { g_err = msg; }
int fail(int code, const std::string& msg) {
    g_err = msg;
    return code;
}

// ---- decode tables: the reference's expressions evaluated once on the host ----
static std::mutex g_mu;
static const DecodeTables* g_tables[64] = {};
static int g_cus[64] = {};

int get_tables(const DecodeTables** out) {
    int dev = 0;
    OILHIP_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return fail(OILHIP_E_ARG, "device index out of range");
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_tables[dev]) {
        DecodeTables h;
        for (int q = 0; q < 256; ++q) {
            volatile float num = 16.0f * (float)q;          // block_codec.cpp:131: mul, div, add
            volatile float quo = num / 255.0f;
            h.lv8[q] = -8.0f + quo;
            volatile float t = (float)q / 255.0f;           // :326
            h.t255[q] = t;
            volatile float u = (float)q / 127.5f;           // :338
            h.t1275[q] = u - 1.0f;
            volatile float s = (float)(int8_t)(uint8_t)q / 127.0f;   // :690
            h.q127[q] = s;
        }
        DecodeTables* d = nullptr;
        OILHIP_HIP(hipMalloc(&d, sizeof(DecodeTables)));
        OILHIP_HIP(hipMemcpy(d, &h, sizeof(DecodeTables), hipMemcpyHostToDevice));
        g_tables[dev] = d;
    }
    *out = g_tables[dev];
    return OILHIP_OK;
}

int device_cu_count() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (!g_cus[dev]) {
        hipDeviceProp_t p;
        g_cus[dev] = (hipGetDeviceProperties(&p, dev) == hipSuccess && p.multiProcessorCount > 0)
                         ? p.multiProcessorCount : 256;
    }
    return g_cus[dev];
}

int ensure_max_lds(std::atomic<uint64_t>& done, const void* kernel, int bytes) {
    int dev = 0;
    OILHIP_HIP(hipGetDevice(&dev));
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return OILHIP_OK;
    OILHIP_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    done.fetch_or(bit, std::memory_order_release);
    return OILHIP_OK;
}

static std::mutex g_scratch_mu;
struct ScratchBuffers {
    void* first = nullptr;              // the buffer in use
    size_t second = 0;                  // its size
    std::vector<void*> outgrown;        // earlier, smaller buffers: kept because a captured graph may still point at them
};
static std::map<std::tuple<int, void*, int>, ScratchBuffers> g_scratch;

int stream_scratch(hipStream_t s, int slot, size_t bytes, void** out) {
    int dev = 0;
    OILHIP_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    auto& e = g_scratch[std::make_tuple(dev, (void*)s, slot)];
    if (e.second < bytes) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return fail(OILHIP_E_ARG, "this call needs " + std::to_string(bytes) + " bytes of device scratch on its stream and cannot "
                        "allocate them during stream capture: make the same call once on this stream outside capture first");
        }
        const size_t want = bytes > 2 * e.second ? bytes : 2 * e.second;
        void* p = nullptr;
        if (hipMalloc(&p, want) != hipSuccess) {
            (void)hipGetLastError();
            return fail(OILHIP_E_NOMEM, "hipMalloc of " + std::to_string(want) + " bytes of scratch failed");
        }
        if (hipMemset(p, 0, want) != hipSuccess) {
            (void)hipGetLastError();
            (void)hipFree(p);
            return fail(OILHIP_E_DEVICE, "hipMemset of the new scratch failed");
        }
        if (e.first) e.outgrown.push_back(e.first);   // the smaller buffer stays allocated until the stream's scratch is released
        e.first = p;
        e.second = want;
    }
    *out = e.first;
    return OILHIP_OK;
}

int check_matmul_shape(const oilhip_weights* w, const void* x, const void* y, int M) {
    if (!w || !x || !y) return fail(OILHIP_E_ARG, "null argument");
    if (M < 1) return fail(OILHIP_E_ARG, "M must be >= 1");
    if (!w->all_full || (w->cols % 256) != 0 || w->cols == 0 || w->rows == 0)
        return fail(OILHIP_E_ARG, "matmul needs cols a positive multiple of 256 and only full 256-weight blocks");
    if ((uint64_t)w->nblocks != w->rows * (w->cols / 256))
        return fail(OILHIP_E_ARG, "block count does not match rows * cols / 256");
    if (w->rows > 0xFFFFFFFFull || w->cols > 0xFFFFFFFFull)
        return fail(OILHIP_E_ARG, "rows/cols exceed 32 bits");
    return OILHIP_OK;
}

}  // namespace oilhip

using namespace oilhip;

extern "C" {

const char* oilhip_last_error(void) { return g_err.c_str(); }

int oilhip_probe(int* gfx, uint64_t* hbm_bytes, int* compute_units, char* name, size_t name_cap) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n < 1) return fail(OILHIP_E_NOGPU, "no HIP device visible");
    int dev = 0;
    OILHIP_HIP(hipGetDevice(&dev));
    hipDeviceProp_t p;
    OILHIP_HIP(hipGetDeviceProperties(&p, dev));
    int arch = 0;
    if (const char* g = std::strstr(p.gcnArchName, "gfx")) arch = (int)std::strtol(g + 3, nullptr, 10);
    if (gfx) *gfx = arch;
    if (hbm_bytes) *hbm_bytes = (uint64_t)p.totalGlobalMem;
    if (compute_units) *compute_units = p.multiProcessorCount;
    if (name && name_cap) {
        std::strncpy(name, p.name, name_cap - 1);
        name[name_cap - 1] = 0;
    }
    if (arch != 950) return fail(OILHIP_E_NOGPU, std::string("device is ") + p.gcnArchName + ", this library is built for gfx950 only");
    return OILHIP_OK;
}

// Mixed-format tensors of full blocks: rewrite `pay` as the window streams the segmented GEMV reads (layout in
// common.h, SegLayout) and point the descriptors at the blocks' new places.  Leaves everything as it is when the
// tensor does not fit the scheme.
static void pack_window_streams(std::vector<uint8_t>& pay, std::vector<DevBlock>& db, uint64_t rows, uint64_t cols,
                                SegLayout& g) {
    const uint64_t bpr = cols / 256, nblocks = db.size();
    if ((cols & 255) || bpr < 1 || bpr > 4096 || nblocks != rows * bpr || rows > 0x7FFFFFFFull) return;
    int slot_of[OILHIP_NUM_FORMATS];
    for (int& v : slot_of) v = -1;
    bool present[OILHIP_NUM_FORMATS] = {};
    for (const DevBlock& d : db) present[d.fmt] = true;
    uint32_t nf = 0;
    for (int f = 0; f < OILHIP_NUM_FORMATS; ++f)
        if (present[f]) {
            if (nf == (uint32_t)kSegMaxFormats) return;
            slot_of[f] = (int)nf;
            g.fmt[nf++] = (uint32_t)f;
        }
    bool seen[kSegMaxFormats] = {};
    for (const DevBlock& d : db) {                     // a format's full blocks must all have the same channel sizes
        const int s = slot_of[d.fmt];
        if (!seen[s]) {
            seen[s] = true;
            // the stream kernel decodes blocks of the size the quantizer writes; other channel sizes stay with the
            // kernels that follow the descriptors weight by weight
            if (d.cb_bytes != full_block_cb_bytes(d.fmt) || d.cb_bytes + d.idx_bytes != full_block_bytes(d.fmt)) return;
            g.cb_bytes[s] = d.cb_bytes;
            g.idx_bytes[s] = d.idx_bytes;
            g.stride[s] = ((uint32_t)d.cb_bytes + d.idx_bytes + 15u) & ~15u;
            if (g.stride[s] + 64u > kSegWindow) return;
        } else if (g.cb_bytes[s] != d.cb_bytes || g.idx_bytes[s] != d.idx_bytes) {
            return;
        }
    }
    // streams: at most two per SIMD, and as many as give every stream the same number of rows (or one less): streams of
    // five and six rows side by side would leave the fixed-size first windows a sixth empty
    const uint64_t max_streams = (uint64_t)device_cu_count() * 8, rows_each = (rows + max_streams - 1) / max_streams;
    const uint32_t ns = (uint32_t)((rows + rows_each - 1) / rows_each);
    // a block's tag is its row of the tile and its column block: one byte while a row has at most 64 blocks
    const uint32_t tagw = bpr <= 64 ? 1u : 2u, tag_shift = bpr <= 64 ? 6u : 12u;
    // `rec` counts the 8-byte units of the window's records: one per entry, and two (four row numbers) behind every
    // entry that closes a tile
    struct Entry { uint32_t slot, flags, nblk, data_off, tag_off, rows[kSegTileRows], nrows; };
    struct Window { std::vector<Entry> ent; std::vector<uint16_t> tags; std::vector<uint32_t> src; uint32_t data = 0, rec = 0; };
    auto bytes_of = [&](size_t nrec, size_t nb, uint32_t data) { return ((8 + 8 * nrec + tagw * nb + 15) & ~(size_t)15) + data; };
    // Rows go to streams by weight, heaviest first, each to the stream that is lightest so far: streams end up with
    // nearly the same number of bytes, so the first windows (fetched blind, all at the size of the fullest) carry
    // little slack and the wavefronts finish together.  A stream's rows need not be neighbours.
    std::vector<uint32_t> row_bytes(rows, 0);
    uint64_t widest = 0;
    for (uint64_t r = 0; r < rows; ++r)
        for (uint64_t c = 0; c < bpr; ++c) {
            const uint32_t st = g.stride[slot_of[db[r * bpr + c].fmt]];
            row_bytes[r] += st + tagw;
            widest = std::max<uint64_t>(widest, st);
        }
    std::vector<uint32_t> order(rows);
    for (uint32_t r = 0; r < rows; ++r) order[r] = r;
    std::stable_sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { return row_bytes[x] > row_bytes[y]; });
    std::vector<std::vector<uint32_t>> rows_of(ns);
    {
        using Load = std::pair<uint64_t, uint32_t>;                 // (bytes so far, stream)
        std::priority_queue<Load, std::vector<Load>, std::greater<Load>> light;
        for (uint32_t st = 0; st < ns; ++st) light.push({0, st});
        for (uint32_t r : order) {
            Load l = light.top();
            light.pop();
            rows_of[l.second].push_back(r);
            l.first += row_bytes[r];
            light.push(l);
        }
    }
    std::vector<std::vector<Window>> streams(ns);
    for (uint32_t st = 0; st < ns; ++st) {
        std::vector<Window>& ws = streams[st];
        ws.emplace_back();
        std::vector<uint32_t>& mine = rows_of[st];
        std::sort(mine.begin(), mine.end());
        for (size_t t0 = 0; t0 < mine.size(); t0 += kSegTileRows) {
            const uint32_t nr = (uint32_t)std::min<size_t>(kSegTileRows, mine.size() - t0);
            Entry* last = nullptr;
            for (uint32_t s = 0; s < nf; ++s) {
                bool open = false;                     // an entry of this tile and slot is open in the current window
                for (uint32_t j = 0; j < nr; ++j)
                    for (uint64_t c = 0; c < bpr; ++c) {
                        const uint32_t b = (uint32_t)((uint64_t)mine[t0 + j] * bpr + c);
                        if (slot_of[db[b].fmt] != (int)s) continue;
                        Window* w = &ws.back();
                        // room for the block, its tag, its entry if a new one opens, and the row record of a closing entry
                        if (bytes_of(w->rec + (open ? 0 : 1) + 2, w->tags.size() + 1, w->data + g.stride[s]) > kSegWindow) {
                            ws.emplace_back();
                            w = &ws.back();
                            open = false;
                        }
                        if (!open) {
                            Entry e{s, 0u, 0u, w->data, (uint32_t)w->tags.size(), {0, 0, 0, 0}, nr};
                            for (uint32_t q = 0; q < nr; ++q) e.rows[q] = mine[t0 + q];
                            w->ent.push_back(e);
                            ++w->rec;
                            open = true;
                        }
                        last = &w->ent.back();
                        ++last->nblk;
                        w->tags.push_back((uint16_t)((j << tag_shift) | c));
                        w->src.push_back(b);
                        w->data += g.stride[s];
                    }
            }
            last->flags |= 1u;                         // every tile has blocks: its last entry closes it
            ws.back().rec += 2;                        // ... and is followed by the tile's row numbers
        }
    }
    // first windows at a fixed stride (the fullest of them decides it), so that a wavefront finds its own from its
    // number alone; the windows after them packed one behind the other, each found through its predecessor's header
    auto used = [&](const Window& w) { return bytes_of(w.rec, w.tags.size(), w.data); };
    size_t first_used = 0;
    for (const auto& ws : streams) first_used = std::max(first_used, used(ws[0]));
    const uint64_t stride = (first_used + 15) & ~(size_t)15;
    uint64_t total = stride * ns;
    std::vector<std::vector<uint64_t>> at_of(ns);
    for (uint32_t st = 0; st < ns; ++st) {
        at_of[st].push_back(st * stride);
        for (size_t wi = 1; wi < streams[st].size(); ++wi) {
            at_of[st].push_back(total);
            total += (used(streams[st][wi]) + 15) & ~(size_t)15;
        }
    }
    if ((total >> 4) > 0xFFFFFFFFull) return;
    std::vector<uint8_t> out(total, 0);
    for (uint32_t st = 0; st < ns; ++st)
        for (size_t wi = 0; wi < streams[st].size(); ++wi) {
            const Window& w = streams[st][wi];
            uint8_t* base = out.data() + at_of[st][wi];
            const uint32_t tag_base = 8u + 8u * w.rec;
            const uint32_t data_base = (tag_base + tagw * (uint32_t)w.tags.size() + 15u) & ~15u;
            const bool more = wi + 1 < streams[st].size();
            const uint32_t hdr[2] = {w.rec | (more ? 1u << 12 : 0u) | (more ? (uint32_t)((used(streams[st][wi + 1]) + 15) >> 4) << 16 : 0u),
                                     more ? (uint32_t)(at_of[st][wi + 1] >> 4) : 0u};
            std::memcpy(base, hdr, 8);
            uint32_t at_rec = 8;
            for (const Entry& e : w.ent) {
                const uint32_t rec[2] = {e.slot | (g.fmt[e.slot] << 4) | (e.flags << 8) | (e.nrows << 9) | (e.nblk << 16),
                                         (data_base + e.data_off) | ((tag_base + tagw * e.tag_off) << 16)};
                std::memcpy(base + at_rec, rec, 8);
                at_rec += 8;
                if (e.flags & 1u) {
                    std::memcpy(base + at_rec, e.rows, 16);
                    at_rec += 16;
                }
            }
            if (tagw == 1) for (size_t i = 0; i < w.tags.size(); ++i) base[tag_base + i] = (uint8_t)w.tags[i];
            else std::memcpy(base + tag_base, w.tags.data(), 2 * w.tags.size());
            uint32_t at = data_base;
            for (uint32_t b : w.src) {
                DevBlock& d = db[b];
                std::memcpy(base + at, pay.data() + (size_t)d.off16 * 16, (size_t)d.cb_bytes + d.idx_bytes);
                d.off16 = (uint32_t)((at_of[st][wi] + at) >> 4);
                at += g.stride[slot_of[d.fmt]];
            }
        }
    g.tag_bytes = tagw;
    pay.swap(out);
    g.nf = nf;
    g.nstreams = ns;
    g.blind16 = (uint32_t)((first_used + 15) >> 4);
    g.stream_bytes = stride;
}

static int upload(std::vector<uint8_t>& pay, std::vector<DevBlock>& db, std::vector<uint64_t>& out_off,
                  uint64_t algo_bytes, uint64_t rows, uint64_t cols, oilhip_weights** out) {
    const uint32_t nblocks = (uint32_t)db.size();
    bool all_full = true, uniform = true, regular = nblocks > 0, nominal = true;
    uint64_t total_nw = 0;
    for (uint32_t b = 0; b < nblocks; ++b) {
        total_nw += db[b].nw;
        all_full &= db[b].nw == 256;
        nominal &= db[b].cb_bytes == full_block_cb_bytes(db[b].fmt) && (uint32_t)db[b].cb_bytes + db[b].idx_bytes == full_block_bytes(db[b].fmt);
        uniform &= db[b].fmt == db[0].fmt;
        if (b > 0) regular &= (db[b].off16 - db[b - 1].off16) == (db[1].off16 - db[0].off16) &&
                              db[b].idx_bytes == db[0].idx_bytes && db[b].cb_bytes == db[0].cb_bytes;
    }
    if (total_nw != rows * cols) return fail(OILHIP_E_ARG, "rows*cols does not equal the number of weights in the blocks");
    auto* w = new (std::nothrow) oilhip_weights();
    if (!w) return fail(OILHIP_E_NOMEM, "host allocation failed");
    auto bail = [&](hipError_t e, const char* what) {
        oilhip_weights_destroy(w);
        return fail(e == hipErrorOutOfMemory ? OILHIP_E_NOMEM : OILHIP_E_DEVICE, std::string(what) + ": " + hipGetErrorString(e));
    };
    hipError_t e;
    if ((e = hipGetDevice(&w->device)) != hipSuccess) return bail(e, "hipGetDevice");
    // window streams for every tensor of full blocks but the uniform OIL4 and OIL8 ones, which have kernels of their own
    // that read the blocks back to back
    const bool own_kernel = uniform && regular && nblocks && db[0].cb_bytes == 0 && db[0].off16 == 0 &&
                            ((db[0].fmt == OILHIP_OIL4 && db[0].idx_bytes == 128) || (db[0].fmt == OILHIP_OIL8 && db[0].idx_bytes == 256)) &&
                            (nblocks == 1 || (db[1].off16 - db[0].off16) * 16u == db[0].idx_bytes);
    if (all_full && nblocks && !own_kernel) pack_window_streams(pay, db, rows, cols, w->seg);
    if (w->seg.nstreams) regular = false;
    // 64 spare bytes so vector loads that straddle the end of the last block stay in bounds
    w->alloc_bytes = pay.size() + 64;
    if ((e = hipMalloc(&w->d_payload, w->alloc_bytes)) != hipSuccess) return bail(e, "hipMalloc(payload)");
    if ((e = hipMemset(w->d_payload, 0, w->alloc_bytes)) != hipSuccess) return bail(e, "hipMemset");
    if (!pay.empty() && (e = hipMemcpy(w->d_payload, pay.data(), pay.size(), hipMemcpyHostToDevice)) != hipSuccess)
        return bail(e, "hipMemcpy(payload)");
    if (nblocks) {
        if ((e = hipMalloc(&w->d_blocks, sizeof(DevBlock) * (size_t)nblocks)) != hipSuccess) return bail(e, "hipMalloc(blocks)");
        if ((e = hipMemcpy(w->d_blocks, db.data(), sizeof(DevBlock) * (size_t)nblocks, hipMemcpyHostToDevice)) != hipSuccess)
            return bail(e, "hipMemcpy(blocks)");
        if (!all_full) {
            if ((e = hipMalloc(&w->d_out_off, 8 * (size_t)nblocks)) != hipSuccess) return bail(e, "hipMalloc(out_off)");
            if ((e = hipMemcpy(w->d_out_off, out_off.data(), 8 * (size_t)nblocks, hipMemcpyHostToDevice)) != hipSuccess)
                return bail(e, "hipMemcpy(out_off)");
        }
    }
    w->payload_bytes = algo_bytes;
    w->rows = rows;
    w->cols = cols;
    w->nblocks = nblocks;
    w->uniform_fmt = (uniform && nblocks) ? db[0].fmt : -1;
    w->all_full = all_full && nblocks > 0;
    w->nominal = w->all_full && nominal;
    if (regular && uniform && nblocks)
        w->uniform_stride = nblocks > 1 ? (db[1].off16 - db[0].off16) * 16u
                                        : (uint32_t)((db[0].cb_bytes + db[0].idx_bytes + 15u) & ~15u);
    if (w->uniform_stride) {
        w->uniform_cb = db[0].cb_bytes;
        w->uniform_idx = db[0].idx_bytes;
        w->uniform_base = db[0].off16 * 16u;
    }
    *out = w;
    return OILHIP_OK;
}

int oilhip_weights_create(const uint8_t* payload, uint64_t payload_bytes, const oilhip_block_t* blocks,
                          uint32_t nblocks, uint64_t rows, uint64_t cols, oilhip_weights** out) {
    if (!out) return fail(OILHIP_E_ARG, "out is null");
    *out = nullptr;
    if ((!payload && payload_bytes) || (!blocks && nblocks)) return fail(OILHIP_E_ARG, "null payload/blocks");
    std::vector<uint8_t> pay;
    std::vector<DevBlock> db(nblocks);
    std::vector<uint64_t> off(nblocks);
    pay.reserve(payload_bytes + 16ull * nblocks);
    uint64_t nw_sum = 0, algo = 0;
    for (uint32_t b = 0; b < nblocks; ++b) {
        const oilhip_block_t& s = blocks[b];
        if (s.fmt >= OILHIP_NUM_FORMATS) return fail(OILHIP_E_ARG, "block " + std::to_string(b) + ": unknown format id");
        if (s.cb_off + s.cb_bytes > payload_bytes || s.idx_off + s.idx_bytes > payload_bytes)
            return fail(OILHIP_E_ARG, "block " + std::to_string(b) + ": payload range out of bounds");
        if (s.cb_bytes > 0xFFFFu) return fail(OILHIP_E_ARG, "block " + std::to_string(b) + ": codebook channel too large");
        if (s.nw == 0 || s.nw > (1u << 24)) return fail(OILHIP_E_ARG, "block " + std::to_string(b) + ": bad weight count");
        pay.resize((pay.size() + 15) & ~(size_t)15, 0);
        if ((pay.size() >> 4) > 0xFFFFFFFFull) return fail(OILHIP_E_ARG, "payload exceeds 64 GiB");
        db[b].off16 = (uint32_t)(pay.size() >> 4);
        db[b].idx_bytes = s.idx_bytes;
        db[b].nw = s.nw;
        db[b].cb_bytes = (uint16_t)s.cb_bytes;
        db[b].fmt = s.fmt;
        db[b].pad = 0;
        pay.insert(pay.end(), payload + s.cb_off, payload + s.cb_off + s.cb_bytes);
        pay.insert(pay.end(), payload + s.idx_off, payload + s.idx_off + s.idx_bytes);
        off[b] = nw_sum;
        nw_sum += s.nw;
        algo += (uint64_t)s.cb_bytes + s.idx_bytes;
    }
    return upload(pay, db, off, algo, rows, cols, out);
}

int oilhip_weights_create_from_records(const uint8_t* rec, uint64_t bytes, const uint8_t* fmts,
                                       uint32_t nblocks, uint64_t rows, uint64_t cols, oilhip_weights** out) {
    if (!out) return fail(OILHIP_E_ARG, "out is null");
    *out = nullptr;
    if (!rec || !fmts) return fail(OILHIP_E_ARG, "null records/fmts");
    std::vector<oilhip_block_t> blocks(nblocks);
    uint64_t at = 0;
    auto rd32 = [&](uint64_t o) { uint32_t v; std::memcpy(&v, rec + o, 4); return v; };
    for (uint32_t b = 0; b < nblocks; ++b) {
        if (at + 8 > bytes) return fail(OILHIP_E_ARG, "record " + std::to_string(b) + " truncated");
        const uint32_t nw = rd32(at), cbb = rd32(at + 4);
        if (at + 8 + cbb + 4 > bytes) return fail(OILHIP_E_ARG, "record " + std::to_string(b) + " truncated");
        const uint32_t ib = rd32(at + 8 + cbb);
        if (at + 12 + cbb + (uint64_t)ib > bytes) return fail(OILHIP_E_ARG, "record " + std::to_string(b) + " truncated");
        blocks[b] = oilhip_block_t{at + 8, at + 12 + cbb, cbb, ib, nw, fmts[b] <= 14 ? fmts[b] : (uint8_t)OILHIP_OIL32, {0, 0, 0}};
        at += 12ull + cbb + ib;
    }
    return oilhip_weights_create(rec, bytes, blocks.data(), nblocks, rows, cols, out);
}

int oilhip_weights_destroy(oilhip_weights* w) {
    if (!w) return OILHIP_OK;
    if (w->d_payload) (void)hipFree(w->d_payload);
    if (w->d_blocks) (void)hipFree(w->d_blocks);
    if (w->d_out_off) (void)hipFree(w->d_out_off);
    delete w;
    return OILHIP_OK;
}

// Several tensors of the same width and regular layout as one tensor of their rows, one after the other
// (device-to-device copy of the payloads; the parts stay valid).
int oilhip_weights_stack_rows(const oilhip_weights* const* parts, int n, oilhip_weights** out) {
    if (!parts || n <= 0 || !out) return fail(OILHIP_E_ARG, "stack_rows: bad arguments");
    *out = nullptr;
    const oilhip_weights* p0 = parts[0];
    uint64_t rows = 0, nblocks = 0, bytes = 0, algo = 0;
    bool regular = true;
    for (int i = 0; i < n; ++i) {
        const oilhip_weights* p = parts[i];
        if (!p || !p0 || p->cols != p0->cols || !p->all_full)
            return fail(OILHIP_E_ARG, "stack_rows: parts must share one width and hold full 256-weight blocks only");
        regular &= p->uniform_stride && p->uniform_fmt == p0->uniform_fmt && p->uniform_stride == p0->uniform_stride &&
                   p->uniform_cb == p0->uniform_cb && p->uniform_idx == p0->uniform_idx;
        rows += p->rows; nblocks += p->nblocks; bytes += (uint64_t)p->nblocks * p->uniform_stride; algo += p->payload_bytes;
    }
    if (!regular) {
        // parts that mix formats (or differ in format): fetch their blocks back and upload the concatenation, which
        // lays the rows out afresh (window streams for a mix)
        if (nblocks > 0xFFFFFFFFull) return fail(OILHIP_E_ARG, "stack_rows: too large");
        std::vector<uint8_t> pay;
        std::vector<DevBlock> db;
        std::vector<uint64_t> off;
        db.reserve((size_t)nblocks);
        for (int i = 0; i < n; ++i) {
            const oilhip_weights* p = parts[i];
            std::vector<uint8_t> hp((size_t)p->alloc_bytes);
            std::vector<DevBlock> hb(p->nblocks);
            OILHIP_HIP(hipMemcpy(hp.data(), p->d_payload, hp.size(), hipMemcpyDeviceToHost));
            OILHIP_HIP(hipMemcpy(hb.data(), p->d_blocks, sizeof(DevBlock) * hb.size(), hipMemcpyDeviceToHost));
            for (DevBlock d : hb) {
                const size_t nb = (size_t)d.cb_bytes + d.idx_bytes, at = pay.size();
                if ((at >> 4) > 0xFFFFFFFFull) return fail(OILHIP_E_ARG, "stack_rows: too large");
                pay.resize((at + nb + 15) & ~(size_t)15, 0);
                std::memcpy(pay.data() + at, hp.data() + (size_t)d.off16 * 16, nb);
                d.off16 = (uint32_t)(at >> 4);
                off.push_back((uint64_t)db.size() * 256u);
                db.push_back(d);
            }
        }
        return upload(pay, db, off, algo, rows, p0->cols, out);
    }
    if (nblocks > 0xFFFFFFFFull || bytes / 16 > 0xFFFFFFFFull) return fail(OILHIP_E_ARG, "stack_rows: too large");
    auto* w = new (std::nothrow) oilhip_weights();
    if (!w) return fail(OILHIP_E_NOMEM, "host allocation failed");
    auto bail = [&](hipError_t e, const char* what) {
        oilhip_weights_destroy(w);
        return fail(e == hipErrorOutOfMemory ? OILHIP_E_NOMEM : OILHIP_E_DEVICE, std::string(what) + ": " + hipGetErrorString(e));
    };
    hipError_t e;
    if ((e = hipGetDevice(&w->device)) != hipSuccess) return bail(e, "hipGetDevice");
    w->alloc_bytes = bytes + 64;
    if ((e = hipMalloc(&w->d_payload, w->alloc_bytes)) != hipSuccess) return bail(e, "hipMalloc(payload)");
    if ((e = hipMemset(w->d_payload + bytes, 0, 64)) != hipSuccess) return bail(e, "hipMemset");
    uint64_t off = 0;
    for (int i = 0; i < n; ++i) {
        const uint64_t nb = (uint64_t)parts[i]->nblocks * parts[i]->uniform_stride;
        if ((e = hipMemcpy(w->d_payload + off, parts[i]->d_payload + parts[i]->uniform_base, nb, hipMemcpyDeviceToDevice)) != hipSuccess)
            return bail(e, "hipMemcpy(payload)");
        off += nb;
    }
    std::vector<DevBlock> db((size_t)nblocks);
    for (uint64_t b = 0; b < nblocks; ++b)
        db[(size_t)b] = DevBlock{(uint32_t)(b * p0->uniform_stride / 16), p0->uniform_idx, 256u, (uint16_t)p0->uniform_cb, (uint8_t)p0->uniform_fmt, 0};
    if ((e = hipMalloc(&w->d_blocks, sizeof(DevBlock) * (size_t)nblocks)) != hipSuccess) return bail(e, "hipMalloc(blocks)");
    if ((e = hipMemcpy(w->d_blocks, db.data(), sizeof(DevBlock) * (size_t)nblocks, hipMemcpyHostToDevice)) != hipSuccess)
        return bail(e, "hipMemcpy(blocks)");
    w->payload_bytes = algo;
    w->rows = rows; w->cols = p0->cols; w->nblocks = (uint32_t)nblocks;
    w->uniform_fmt = p0->uniform_fmt; w->all_full = true; w->nominal = p0->nominal;
    w->uniform_stride = p0->uniform_stride; w->uniform_cb = p0->uniform_cb; w->uniform_idx = p0->uniform_idx; w->uniform_base = 0;
    *out = w;
    return OILHIP_OK;
}

int oilhip_weights_info(const oilhip_weights* w, uint64_t* rows, uint64_t* cols, uint32_t* nblocks,
                        uint64_t* payload_bytes, int* uniform_fmt) {
    if (!w) return fail(OILHIP_E_ARG, "null weights");
    if (rows) *rows = w->rows;
    if (cols) *cols = w->cols;
    if (nblocks) *nblocks = w->nblocks;
    if (payload_bytes) *payload_bytes = w->payload_bytes;
    if (uniform_fmt) *uniform_fmt = w->uniform_fmt;
    return OILHIP_OK;
}

int oilhip_weights_device_bytes(const oilhip_weights* w, uint64_t* stored_bytes, uint64_t* descriptor_bytes) {
    if (!w) return fail(OILHIP_E_ARG, "null weights");
    if (stored_bytes) *stored_bytes = w->alloc_bytes;
    if (descriptor_bytes) *descriptor_bytes = (uint64_t)w->nblocks * sizeof(DevBlock);
    return OILHIP_OK;
}

int oilhip_dequant_f32(const oilhip_weights* w, float* d_out, void* stream) {
    if (!w || !d_out) return fail(OILHIP_E_ARG, "null argument");
    return launch_dequant(*w, d_out, (hipStream_t)stream);
}

int oilhip_gemv_f32(const oilhip_weights* w, const float* d_x, float* d_y, int M, void* stream) {
    if (int rc = check_matmul_shape(w, d_x, d_y, M)) return rc;
    if (plain_oil4(*w)) {
        // one or two rows: the register-resident kernel; from three on the matrix-core kernel (16 rows per pass) is faster
        int rc = 1;                                                                          // 1: shape not covered
        if (M <= 2) rc = launch_gemv_oil4(*w, d_x, d_y, M, (hipStream_t)stream);
        if (rc == 1 && M >= 2)
            rc = launch_gemv_oil4_multi(*w, d_x, nullptr, d_y, M, (uint32_t)w->cols, (uint32_t)w->rows, (uint32_t)M,
                                        (hipStream_t)stream);
        if (rc == 1 && M > 2 && M <= 4) rc = launch_gemv_oil4(*w, d_x, d_y, M, (hipStream_t)stream);
        if (rc <= 0) return rc;
    }
    if (plain_oil8(*w)) {
        // the register-resident kernel takes up to four activation rows per launch
        int rc = 1;
        for (int m0 = 0; m0 < M; m0 += 4) {
            rc = launch_gemv_oil8(*w, d_x + (size_t)m0 * w->cols, d_y + (size_t)m0 * w->rows, M - m0 < 4 ? M - m0 : 4,
                                  (hipStream_t)stream);
            if (rc != 0) break;
        }
        if (rc <= 0) return rc;
    }
    if (w->seg.nstreams) {
        const int rc = launch_gemv_seg(*w, d_x, d_y, M, (hipStream_t)stream);
        if (rc <= 0) return rc;
    }
    const int rc = launch_gemv_runs(*w, d_x, d_y, M, (hipStream_t)stream);
    if (rc <= 0) return rc;
    return launch_gemv_generic(*w, d_x, d_y, M, (hipStream_t)stream);
}

// Test hook: the all-format kernel regardless of shape (the specialised kernels
// are checked against it as well as against the CPU oracle).
int oilhip_gemv_f32_general(const oilhip_weights* w, const float* d_x, float* d_y, int M, void* stream) {
    if (int rc = check_matmul_shape(w, d_x, d_y, M)) return rc;
    return launch_gemv_generic(*w, d_x, d_y, M, (hipStream_t)stream);
}

int oilhip_gemm_bf16(const oilhip_weights* w, const uint16_t* d_x, float* d_y, int M, void* stream) {
    if (int rc = check_matmul_shape(w, d_x, d_y, M)) return rc;
    if (plain_oil4(*w)) return launch_gemm_oil4_bf16(*w, d_x, d_y, M, (hipStream_t)stream);
    // any other tensor of full blocks: decoded to bf16 slab by slab, then the same kernel over a dense operand
    const int rc = launch_gemm_any_bf16(*w, d_x, d_y, M, (hipStream_t)stream);
    if (rc == 1) return fail(OILHIP_E_ARG, "bf16 prefill GEMM needs full blocks with the channel sizes the quantizer writes");
    return rc;
}

int oilhip_gemm_f32(const oilhip_weights* w, const float* d_x, float* d_y, int M, void* stream) {
    if (int rc = check_matmul_shape(w, d_x, d_y, M)) return rc;
    hipStream_t s = (hipStream_t)stream;
    // plain OIL4: the pre-pass of the prefill kernel rounds X on its way into fragment order
    if (plain_oil4(*w) && (reinterpret_cast<uintptr_t>(d_x) & 15u) == 0u) return launch_gemm_oil4_frag(*w, d_x, true, d_y, M, s);
    uint16_t* xb = nullptr;
    if (int rc = launch_x_to_bf16(d_x, (uint64_t)M * w->cols, &xb, s)) return rc;
    return oilhip_gemm_bf16(w, xb, d_y, M, stream);
}

int oilhip_release_stream_scratch(void* stream) {
    int dev = 0;
    OILHIP_HIP(hipGetDevice(&dev));
    OILHIP_HIP(hipStreamSynchronize((hipStream_t)stream));
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    for (auto it = g_scratch.begin(); it != g_scratch.end();) {
        if (std::get<0>(it->first) == dev && std::get<1>(it->first) == stream) {
            (void)hipFree(it->second.first);
            for (void* old : it->second.outgrown) (void)hipFree(old);
            it = g_scratch.erase(it);
        } else {
            ++it;
        }
    }
    return OILHIP_OK;
}

}  // extern "C"
