// common.h -- shared host-side declarations of liboilhip (not part of the C ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <string>

#include "../../include/oilhip.h"
#include "block_decode.h"

namespace oilhip {

// bytes of a full 256-weight block of each format (codebook channel + index channel) and of its codebook channel,
// as quantize_block_all writes them (src/block_codec.cpp:368-574)
__host__ __device__ constexpr uint32_t full_block_bytes(int f) {
    constexpr uint32_t n[15] = {16, 48, 64, 128, 256, 512, 1024, 32, 48, 80, 144, 272, 512, 64, 64};
    return f >= 0 && f < 15 ? n[f] : 0u;
}
__host__ __device__ constexpr uint32_t full_block_cb_bytes(int f) { return f == 0 ? 16u : 0u; }

// Thread-local text behind oilhip_last_error().
void set_error(const std::string& msg);
int fail(int code, const std::string& msg);

#define OILHIP_HIP(call)                                                                  \
    do {                                                                                  \
        hipError_t e_ = (call);                                                           \
        if (e_ != hipSuccess)                                                             \
            return ::oilhip::fail(OILHIP_E_DEVICE, std::string(#call) + ": " + hipGetErrorString(e_)); \
    } while (0)

// Per-device decode tables (device pointer), created on first use.
int get_tables(const DecodeTables** out);
int device_cu_count();
// shape rules shared by every matmul entry point: non-null pointers, M >= 1, full blocks, cols a multiple of 256
int check_matmul_shape(const oilhip_weights* w, const void* x, const void* y, int M);

// Raises a kernel's dynamic LDS limit once per device.  `done` is the call site's own flag word (one bit per device);
// concurrent first calls may both set the attribute, which is harmless.
int ensure_max_lds(std::atomic<uint64_t>& done, const void* kernel, int bytes);

// Device scratch of at least `bytes` that belongs to (current device, stream, slot): kernels queued on one stream run
// in order, so calls on different streams never share a buffer.  A buffer is never freed or moved while the process
// lives (a captured graph or a queued kernel may still point at it): a request that outgrows it gets a new, larger
// one and the old one stays allocated.  No allocation can happen while the stream is being captured, so the first
// call of a given size on a stream has to be made outside capture; otherwise the call fails with OILHIP_E_ARG.
// New buffers are zero-filled.
enum ScratchSlot { kScratchGemvPack = 0, kScratchGemmX = 1, kScratchTl = 2, kScratchGemmW = 3, kScratchGemmXb = 4 };
int stream_scratch(hipStream_t s, int slot, size_t bytes, void** out);

// Tensors whose rows mix formats are stored as `nstreams` streams of windows of at most 4 KB, one wavefront per stream
// (gemv_seg.hip).  The first window of stream s sits at byte s * stream_bytes of the payload buffer, the later ones
// behind all first windows, each found through its predecessor.  A stream covers a set of rows (chosen so that all
// streams weigh about the same) in tiles of at most kSegTileRows; inside a tile the blocks are ordered by format (in the
// order of `fmt`), inside a format by row and column.  Window: 2 dwords {8-byte units of records | 1 << 12 if another
// window follows | 16-byte pieces that window fills << 16, its byte offset / 16 in the buffer}; the records: per entry
// 2 dwords {slot | format << 4 | closes its tile << 8 | rows of the tile << 9 | blocks << 16, byte offset of the blocks |
// byte offset of their tags << 16}, and behind an entry that closes its tile 4 dwords with the tile's row numbers; the
// tags (per block: row of the tile and column block, in one byte (row << 6 | column) while a row has at most 64 blocks,
// else two (row << 12 | column)); the blocks, 16-byte aligned, whole.  `blind16` = 16-byte pieces the fullest first
// window fills.
constexpr int kSegMaxFormats = 15;
constexpr uint32_t kSegWindow = 4096;
constexpr int kSegTileRows = 4;
struct SegLayout {
    uint32_t nf = 0, nstreams = 0, blind16 = 0, tag_bytes = 2;
    uint64_t stream_bytes = 0;
    uint32_t fmt[kSegMaxFormats] = {}, cb_bytes[kSegMaxFormats] = {}, idx_bytes[kSegMaxFormats] = {}, stride[kSegMaxFormats] = {};
};

}  // namespace oilhip

// The handle behind oilhip_weights*.
struct oilhip_weights {
    int device = 0;
    uint8_t* d_payload = nullptr;           // block payloads, each 16-byte aligned
    oilhip::DevBlock* d_blocks = nullptr;   // one descriptor per block
    oilhip::SegLayout seg;                  // mixed-format tensors of full blocks: tile- and format-ordered storage
    uint64_t* d_out_off = nullptr;          // first output index per block (only when nw varies)
    uint64_t alloc_bytes = 0;               // size of d_payload
    uint64_t payload_bytes = 0;             // sum of cb_bytes + idx_bytes
    uint64_t rows = 0, cols = 0;
    uint32_t nblocks = 0;
    int uniform_fmt = -1;                   // single format id, or -1
    uint32_t uniform_stride = 0;            // bytes between consecutive blocks when regular, else 0
    uint32_t uniform_cb = 0, uniform_idx = 0;   // channel sizes of every block when regular
    uint32_t uniform_base = 0;              // byte offset of block 0 when regular
    bool all_full = false;                  // every block holds exactly 256 weights
    bool nominal = false;                   // ... and has the channel sizes the quantizer writes for its format
};

namespace oilhip {
// Uniform OIL4 / OIL8 tensors in the plain layout the specialised kernels read: every block's bytes in the index
// channel, blocks back to back from byte 0.  Anything else (a non-empty codebook channel, padding between blocks)
// goes through the kernels that follow the descriptors.
inline bool plain_oil4(const oilhip_weights& w) {
    return w.uniform_fmt == OILHIP_OIL4 && w.uniform_stride == 128 && w.uniform_cb == 0 && w.uniform_idx == 128 && w.uniform_base == 0;
}
inline bool plain_oil8(const oilhip_weights& w) {
    return w.uniform_fmt == OILHIP_OIL8 && w.uniform_stride == 256 && w.uniform_cb == 0 && w.uniform_idx == 256 && w.uniform_base == 0;
}

// kernels (each returns an OILHIP_* code and sets the error text)
int launch_dequant(const oilhip_weights& w, float* d_out, hipStream_t s);
int launch_dequant_bf16_blocks(const oilhip_weights& w, uint32_t b0, uint32_t nb, uint16_t* d_out, hipStream_t s);
bool dequant_bf16_blocks_covers(const oilhip_weights& w);   // whether launch_dequant_bf16_blocks takes this tensor's layout
int launch_gemv_generic(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s);
// fast paths return 1 when they do not cover the case (caller falls through to the general kernel)
int launch_gemv_oil4(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s);
// production gemv_oil4 form for one activation row: rows of K/2 code bytes, FP16 codebook of 16, one scale
int launch_gemv_flat4(const uint8_t* d_w, const uint16_t* d_cb16, float scale, const float* d_x, float* d_y, int rows, int K,
                      hipStream_t s);
int launch_gemv_oil8(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s);
// kernel::oil8_gemm form: rows of K index bytes, any 256-entry codebook; out[m*N + n] = scale * dot
int launch_gemv_flat8(const uint8_t* d_idx, const float* d_cb, const float* d_act, float* d_out, int M, int N, int K, float scale,
                      hipStream_t s);
// several activation rows at once (FP32 MFMA); x row tok[m] (or m) of an [xrows][ldx] matrix, y row stride ldy
int launch_gemv_oil4_multi(const oilhip_weights& w, const float* d_x, const int* d_tok, float* d_y, int M,
                           uint32_t ldx, uint32_t ldy, uint32_t xrows, hipStream_t s, const oilhip_weights* w2 = nullptr,
                           float* d_y2 = nullptr, uint32_t ldy2 = 0, const float* d_x2 = nullptr, uint32_t* d_pack = nullptr,
                           size_t pack_cap = 0);
void g_ordered_sums_set(int v);
// several batches of one tensor shape in one launch (gemv_oil4_multi.hip); kinds[b] = 0 / 1 / 2: batch b holds up to 8 / 16 / 32 rows
size_t gemv_oil4_multi_batches_bytes(int nb, uint64_t rows, uint64_t cols, bool two_tensors);   // two_tensors: every batch goes through wa[b] and wb[b]
int launch_gemv_oil4_multi_batches(int nb, const int* kinds, const oilhip_weights* const* wa, float* const* ya,
                                   const oilhip_weights* const* wb, float* const* yb, const int* M, const int* row0,
                                   const int* list, int nlist, const float* d_x, const float* d_x2, uint32_t ldx, uint32_t xrows,
                                   uint32_t ldy, void* d_ws, size_t ws_bytes, hipStream_t s, bool counters_clean = false,
                                   float* d_parts = nullptr, uint32_t parts_rows = 0);
uint32_t gemv_oil4_multi_parts(int kind, uint64_t cols);
bool gemv_oil4_multi_ordered();
// clears the slab counters at the start of a batch workspace; launches over it may then be told that they are clean
constexpr size_t kGemvBatchCounterBytes = 32u * 4096u;   // slab counters at the start of a batch workspace: a 4 KB page per job
int zero_gemv_oil4_multi_batch_counters(void* d_ws, hipStream_t s);
bool gemv_oil4_multi_batches_accumulate(int kind, uint64_t cols);
// widest row that kernel takes and the bytes of packed activations one pass of it needs (d_pack, or stream scratch)
constexpr uint32_t kGemvPackMaxCols = 32768;
constexpr size_t kGemvPackExpBytes = (size_t)(kGemvPackMaxCols >> 8) * 2u * 16u * 4u;    // one scale exponent per (token tile, block, column)
constexpr size_t kGemvPackBytes = (size_t)(kGemvPackMaxCols >> 8) * 128u * 128u * 2u + kGemvPackExpBytes;   // two token tiles, then the exponents
// rows that mix formats, stored tile by tile and format by format
int launch_gemv_seg(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s);
// every format, a lane per run of 32 weights
int launch_gemv_runs(const oilhip_weights& w, const float* d_x, float* d_y, int M, hipStream_t s);
int launch_gemm_oil4_bf16(const oilhip_weights& w, const uint16_t* d_x, float* d_y, int M, hipStream_t s);
int launch_gemm_any_bf16(const oilhip_weights& w, const uint16_t* d_x, float* d_y, int M, hipStream_t s);
// FP32 activations [M][K] rounded once to bf16 bit patterns (a scratch buffer of the stream)
int launch_x_to_bf16(const float* d_x, uint64_t n, uint16_t** out, hipStream_t s);
// plain uniform OIL4, more than 256 tokens: activations in fragment order straight from memory (gemm_oil4_frag.hip)
int launch_gemm_oil4_frag(const oilhip_weights& w, const void* d_x, bool x_is_f32, float* d_y, int M, hipStream_t s);
}  // namespace oilhip
