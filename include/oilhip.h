/*
 * oilhip.h -- C ABI of the MI355X (gfx950) OIL quantized-weight matmul library.
 *
 * Plain pointers and sizes only.  Every function returns 0 on success and a
 * negative OILHIP_E_* code on failure; oilhip_last_error() then describes the
 * failure for the calling thread.  Pointers named d_* are device (HBM)
 * pointers, all others are host pointers.  `stream` is a hipStream_t passed as
 * void* (NULL = the default stream); calls are asynchronous on that stream
 * unless stated otherwise.
 *
 * Each entry point names the reference interface it stands in for
 * (file:line relative to the reference tree).
 */
#ifndef OILHIP_H
#define OILHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OILHIP_OK            0
#define OILHIP_E_ARG        -1   /* bad argument / shape / unsupported combination */
#define OILHIP_E_DEVICE     -2   /* a HIP call failed                              */
#define OILHIP_E_NOGPU      -3   /* no gfx950 device visible                       */
#define OILHIP_E_NOMEM      -4

/* Wire formats, numbered as oil::Format (include/oil/types.h:19-35). */
enum {
    OILHIP_OIL1 = 0, OILHIP_SPARK_Q0 = 1, OILHIP_OIL2 = 2, OILHIP_OIL4 = 3, OILHIP_OIL8 = 4,
    OILHIP_OIL16 = 5, OILHIP_OIL32 = 6, OILHIP_OIL1_GRP = 7, OILHIP_SPARK_Q0_GRP = 8,
    OILHIP_OIL2_GRP = 9, OILHIP_OIL4_GRP = 10, OILHIP_OIL8_GRP = 11, OILHIP_OIL16_GRP = 12,
    OILHIP_SPARK_SPARSE = 13, OILHIP_SPARK_SPARSE_GRP = 14, OILHIP_NUM_FORMATS = 15
};

const char* oilhip_last_error(void);

/* Runtime probe of the device path: the counterpart of detect_cpu_isa()
 * (include/oil/kernel_production.h:19) and probe_hardware()
 * (include/oil/backend.h:98-139, src/backend.cpp:672-730).  Any out pointer
 * may be NULL.  gfx receives 950 on MI355X.  Synchronous. */
int oilhip_probe(int* gfx, uint64_t* hbm_bytes, int* compute_units, char* name, size_t name_cap);

/* ---------------------------------------------------------------- host codec
 * The reference quantizer runs on the CPU (it is the producer of .oil files,
 * not part of the accelerated path); these are its host-side counterparts.
 * oilhip_quantize_block  : quantize_block_all   (include/oil/block_codec.h:55-56)
 * oilhip_payload_bound   : upper bound of idx+cb bytes for n weights
 * oilhip_quantize_tensor : the per-256-block loop of FormatRegistry::quantize
 *                          (src/format_registry.cpp:158-197)                    */
typedef struct {
    uint64_t cb_off;      /* byte offset of the block's codebook channel in the payload */
    uint64_t idx_off;     /* byte offset of the block's index channel in the payload    */
    uint32_t cb_bytes;
    uint32_t idx_bytes;
    uint32_t nw;          /* weights in the block */
    uint8_t  fmt;         /* OILHIP_* format id   */
    uint8_t  reserved[3];
} oilhip_block_t;

size_t oilhip_payload_bound(int fmt, int n);
int oilhip_quantize_block(int fmt, const float* w, int n,
                          uint8_t* idx, size_t idx_cap, size_t* idx_len,
                          uint8_t* cb, size_t cb_cap, size_t* cb_len);
/* Block b covers w[b*256 ..) and is encoded as fmts[b]; payloads are appended
 * 16-byte aligned (codebook channel then index channel).  With payload == NULL
 * returns only the capacity bound in *total.  threads <= 0: all host cores. */
int oilhip_quantize_tensor(const uint8_t* fmts, uint32_t nblocks, const float* w, uint64_t numel,
                           uint8_t* payload, uint64_t cap, oilhip_block_t* blocks,
                           uint64_t* total, int threads);

/* --------------------------------------------------------------- format routing
 * Which wire format each 256-weight block gets (host side, like the reference).
 * oilhip_score_importance : FormatPlanner::score_importance (fisher = 0: mean |w|*|a| per block,
 *                           a = aux or 1) / score_importance_fisher (fisher = 1: aux = gradients)
 *                           (src/format_planner.cpp:12-61)
 * oilhip_plan_formats     : FormatPlanner::allocate (src/format_planner.cpp:133-315): fmts[b] for a
 *                           target bits-per-weight; scores may be NULL (blocks keep their order).
 *                           counts7 = blocks counted as {OIL32, OIL16, OIL8, OIL4, OIL2, SPARK, OIL1}
 *                           the way the reference's plan counts them (:236-249).
 * oilhip_mix_allocate     : FormatRegistry::allocate_mix_blocks (src/format_registry.cpp:477-599):
 *                           adaptive mix under a hard byte budget ceil(effective_bpw*n/8); tier_fmts are
 *                           the mix's member formats (SPARK_MIX_Q0 = {OIL8_GRP, OIL4_GRP, OIL2_GRP,
 *                           OIL1_GRP} at 1.925; QUAD_SPARK_Q1 = {OIL32, OIL8_GRP, OIL2_GRP, OIL1_GRP} at
 *                           2.075).  rows/cols: tensor shape or 0 (one block per row when cols <
 *                           block_size).  The per-candidate reconstruction errors are measured on the
 *                           GPU.  With fmts_out == NULL only *nblocks_out is set.  Synchronous. */
int oilhip_score_importance(const float* w, const float* aux, int64_t n, int block_size, int fisher,
                            float* scores, int64_t nblocks);
int oilhip_plan_formats(float target_bpw, const float* scores, int64_t nscores, int num_blocks,
                        uint8_t* fmts, float* achieved_bpw, int* uses_mix, int* counts7);
int oilhip_mix_allocate(const uint8_t* tier_fmts, int num_tiers, float effective_bpw, const float* data, int64_t n,
                        int block_size, int64_t rows, int64_t cols, uint8_t* fmts_out, int64_t* starts_out,
                        int64_t* lens_out, int64_t cap, int64_t* nblocks_out);

/* ------------------------------------------------------------- device weights
 * A quantized tensor resident in HBM: block payloads byte-identical to the
 * .oil file's, framing stripped into a descriptor table, uploaded once.
 * Stands in for OILReader::block_ptr/format_entry + Qwen35Engine::Th{start,
 * count,fmt,rows,cols} (src/oil_format.cpp:416-421, include/oil/oil_format.h:80-83,
 * include/oil/qwen35_engine.h:29).  rows*cols must equal the sum of nw; for the
 * matmul entry points cols must be a multiple of 256 and every block full.
 * Synchronous (returns after the upload). */
typedef struct oilhip_weights oilhip_weights;

int oilhip_weights_create(const uint8_t* payload, uint64_t payload_bytes,
                          const oilhip_block_t* blocks, uint32_t nblocks,
                          uint64_t rows, uint64_t cols, oilhip_weights** out);

/* Same, parsing on-disk block records [nw u32][cb_bytes u32][cb][idx_bytes u32][idx]
 * (src/oil_format.cpp:219-233) laid end to end, with the per-block format ids
 * from the file's format table (src/oil_format.cpp:329-350). */
int oilhip_weights_create_from_records(const uint8_t* records, uint64_t record_bytes,
                                       const uint8_t* fmts, uint32_t nblocks,
                                       uint64_t rows, uint64_t cols, oilhip_weights** out);

int oilhip_weights_destroy(oilhip_weights* w);

/* Facts about an uploaded tensor.  payload_bytes = sum of cb_bytes + idx_bytes
 * (the algorithmic weight bytes); uniform_fmt = the single format id or -1 for a
 * mixed tensor.  Any out pointer may be NULL. */
int oilhip_weights_info(const oilhip_weights* w, uint64_t* rows, uint64_t* cols,
                        uint32_t* nblocks, uint64_t* payload_bytes, int* uniform_fmt);

/* Device memory the tensor occupies: block bytes as stored (padding, and for every tensor of full blocks except uniform
 * OIL4 / OIL8 the window headers and block tags of its streams), and the 16-byte per-block descriptors.  The difference between stored_bytes
 * and payload_bytes is what a GEMV reads on top of the algorithmic bytes.  No counterpart in the reference, whose
 * tensors live in host memory (include/oil/qwen35_engine.h:29).  Either out pointer may be NULL. */
int oilhip_weights_device_bytes(const oilhip_weights* w, uint64_t* stored_bytes, uint64_t* descriptor_bytes);

/* ------------------------------------------------------------- .oil container
 * OILReader (include/oil/oil_format.h:66-108, src/oil_format.cpp:289-527) and OILWriter
 * (src/oil_format.cpp:189-283).  A file handle maps the file and indexes its block records once.
 * oilhip_file_open / _open_memory : OILReader ctor (memory: the bytes are copied); a bad magic or a file cut
 *                                   inside its tables is an error (the reference leaves valid() false)
 * oilhip_file_info                : header() fields, num_blocks(), tensor count
 * oilhip_file_config              : read_config()
 * oilhip_file_tensor / _find_tensor : tensor_names() / tensor_blocks(); num_weights = sum of the records' nw
 * oilhip_file_block               : read_block() / block_ptr() / format_entry(): pointers into the mapped file,
 *                                   valid until oilhip_file_close; format ids above 14 read as OIL32 (:405-408)
 * oilhip_file_upload_tensor       : a tensor's records straight into a device tensor (rows = cols = 0: 1 x numel)
 * oilhip_file_write               : OILWriter's header -> format table -> tensor table -> blocks sequence for
 *                                   tensors laid back to back (tensor i owns the next tensor_blocks[i] blocks) */
typedef struct oilhip_file oilhip_file;
int oilhip_file_open(const char* path, oilhip_file** out);
int oilhip_file_open_memory(const uint8_t* bytes, uint64_t n, oilhip_file** out);
int oilhip_file_close(oilhip_file* f);
int oilhip_file_info(const oilhip_file* f, uint32_t* version, uint32_t* flags, uint32_t* config_size,
                     uint32_t* num_blocks, uint32_t* num_tensors);
int oilhip_file_config(const oilhip_file* f, uint8_t* out, uint32_t cap);
int oilhip_file_tensor(const oilhip_file* f, uint32_t i, char* name, size_t name_cap, uint32_t* start,
                       uint32_t* count, uint64_t* num_weights);
int oilhip_file_find_tensor(const oilhip_file* f, const char* name, uint32_t* index);
int oilhip_file_block(const oilhip_file* f, uint32_t id, uint8_t* fmt, uint32_t* nw, const uint8_t** cb,
                      uint32_t* cb_bytes, const uint8_t** idx, uint32_t* idx_bytes);
int oilhip_file_upload_tensor(const oilhip_file* f, uint32_t tensor, uint64_t rows, uint64_t cols, oilhip_weights** out);
int oilhip_file_write(const char* path, uint32_t version, uint32_t flags, const uint8_t* config, uint32_t config_size,
                      uint32_t ntensors, const char* const* names, const uint32_t* tensor_blocks,
                      const uint8_t* payload, const oilhip_block_t* blocks, uint32_t nblocks);

/* dequantize_block_all over every block, back to back (include/oil/block_codec.h:60-63,
 * OILReader::read_tensor src/oil_format.cpp:464-477).  d_out holds rows*cols
 * floats.  Bit-exact with the reference decode. */
int oilhip_dequant_f32(const oilhip_weights* w, float* d_out, void* stream);

/* Qwen35Engine::gemm (src/adapters/tools/qwen35_engine.cpp:47-85):
 * d_y[b*rows + r] = sum_c W[r][c] * d_x[b*cols + c], FP32 in, FP32 out,
 * FP32 accumulation, 1 <= M (the reference caps a call at 512). */
int oilhip_gemv_f32(const oilhip_weights* w, const float* d_x, float* d_y, int M, void* stream);

/* The same product for uniform OIL4 tensors, for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc).  No counterpart in the reference.  It calls no
 * hipMalloc/hipFree: the scratch its multi-row kernel needs (packed activations and their exponents, 8 MB) is a fixed array in the
 * library's code object, one per GPU.  Limits: uniform OIL4 in the plain block layout, cols <= 32768; and, where
 * the rows are cut into three or more parts along K whose sums meet in the scratch (M >= 3 with cols > 8192, or
 * M > 16 with cols > 4096, ordered sums on), parts * tokens_per_pass * rows <= 1,043,456 floats (parts =
 * ceil(cols / 4096) for passes of up to 16 tokens, ceil(cols / 2048) for passes of 32; e.g. cols = 11008, M <= 16:
 * rows <= 21,738).  Anything else returns OILHIP_E_ARG.  All calls on one GPU share that array: calls that overlap on one GPU (two streams, two
 * threads) race on it and must be serialized by the caller. */
int oilhip_gemv_oil4_f32_noalloc(const oilhip_weights* w, const float* d_x, float* d_y, int M, void* stream);

/* Rows too wide for one workgroup pass of the multi-row OIL4 kernel (more than 16 blocks, 8 for batches beyond 16 rows)
 * are cut into parts whose partial sums have to meet.  ordered = 1 (the default): three or more parts are added in a
 * fixed order through a workspace, so a call returns the same bits every time, like the reference's sequential loop
 * (src/adapters/tools/qwen35_engine.cpp:71-78).  ordered = 0: float atomics, a few microseconds faster, last bits may
 * differ from run to run (within the 1e-5 bound).  Process-wide. */
int oilhip_set_ordered_sums(int ordered);


/* Prefill form of the same contraction: activations as bf16 bit patterns,
 * weights dequantized to bf16 (each value rounded once), MFMA with FP32 accumulation, FP32 out.
 * (The reference has no bf16 path; its FP32 prefill loop is
 * qwen35_engine.cpp:630-753 over the same gemm.)  Uniform OIL4 tensors are decoded tile by tile in LDS inside the
 * GEMM kernel.  Tensors of any other format, or that mix formats, are decoded to bf16 in slabs of weight rows (at
 * most 64 MB, a scratch buffer of the stream: the first call of a size on a stream allocates, so make it outside
 * graph capture) and multiplied by the same kernel reading a dense operand; they need full 256-weight blocks with
 * the channel sizes the quantizer writes (OILHIP_E_ARG otherwise). */
int oilhip_gemm_bf16(const oilhip_weights* w, const uint16_t* d_x_bf16, float* d_y, int M, void* stream);

/* The same prefill GEMM for the reference's own call: FP32 activations X[M][cols], as Qwen35Engine::prefill hands
 * them to gemm() in chunks of up to 512 tokens (src/adapters/tools/qwen35_engine.cpp:47-85,630-753).  X is rounded
 * once to bf16 on its way into the kernel's operand order (no extra pass for plain OIL4 and 16-byte aligned X;
 * otherwise one conversion launch into a scratch buffer of the stream).  The result is bit for bit what oilhip_gemm_bf16
 * returns for bf16(X): relative L2 <= 2e-3 against the FP32 contraction over the rounded activations, about 2.4e-3
 * against the one over the FP32 activations themselves (both operands' roundings, Gaussian data), where
 * oilhip_gemv_f32 keeps 1e-5: a caller chooses it per call. */
int oilhip_gemm_f32(const oilhip_weights* w, const float* d_x, float* d_y, int M, void* stream);

/* Frees the scratch buffers the library holds for `stream` on the current device (packed activations of the
 * multi-token GEMV, X' and decoded slabs of the prefill GEMM, the lookup kernels' codes; buffers that a larger request
 * has replaced included): before a stream is destroyed, or to trim after a large batch.  Synchronizes the stream
 * first, so the stream must still exist; no captured graph may still replay launches that were recorded on it.  (No counterpart in the reference, which owns no device memory.) */
int oilhip_release_stream_scratch(void* stream);

/* ---------------------------------------------------- flat-codebook kernels
 * oil::kernel::oil8_gemm (include/oil/kernel.h:24-26, src/kernel_oil8.cpp:71-79):
 *   out[m*N+n] = sum_k cb[idx[n*K+k]] * act[m*K+k]
 * oil::kernel::oil4_gemm (include/oil/kernel.h:30-32, src/kernel_oil4.cpp:120-128):
 *   out[m*N+n] = sum_k f16(cb[nib((m*N+n)*K+k)]) * act[n*K+k]                   */
int oilhip_flat_oil8_gemm(const uint8_t* d_idx, const float* d_cb256, const float* d_act,
                          float* d_out, int M, int N, int K, void* stream);
int oilhip_flat_oil4_gemm(const uint8_t* d_packed, const uint16_t* d_cb16, const float* d_act,
                          float* d_out, int M, int N, int K, void* stream);

/* oil::adapters::prod::gemv_{spark,oil4,oil8}_tiled / _batch
 * (include/oil/kernel_production.h:25-52; scalar bodies src/kernel_production.cpp:79-128):
 *   Y[n*M + m] = scale * sum_k dec(W[m][k]) * X[n*K + k],  n < batch            */
int oilhip_prod_gemv_spark(const uint8_t* d_w, float scale, const float* d_x, float* d_y,
                           int M, int K, int batch, void* stream);
int oilhip_prod_gemv_oil4(const uint8_t* d_w, const uint16_t* d_cb16, float scale, const float* d_x,
                          float* d_y, int M, int K, int batch, void* stream);
int oilhip_prod_gemv_oil8(const uint8_t* d_w, const float* d_cb256, float scale, const float* d_x,
                          float* d_y, int M, int K, int batch, void* stream);

/* oil::adapters::prod::KernelPerf + profile_gemv_{spark,oil4,oil8} (include/oil/kernel_production.h:68-82,
 * src/kernel_production.cpp:433-485): `repeats` launches of the tiled GEMV (batch 1) timed between two events on
 * `stream`, after one untimed launch.  kind 0 SPARK (d_cb unused), 4 OIL4 (d_cb = 16 FP16 entries), 8 OIL8 (d_cb =
 * 256 floats).  bytes_read / bytes_written / gflops use the reference's formulas; `cycles` is the time per launch in
 * shader clocks at the device's peak frequency, where the reference reads the CPU's timestamp counter.  Waits for
 * the stream; cannot be captured into a graph. */
typedef struct oilhip_kernel_perf {
    uint64_t cycles;
    uint64_t bytes_read;
    uint64_t bytes_written;
    double gflops;
} oilhip_kernel_perf_t;
int oilhip_profile_gemv(int kind, const uint8_t* d_w, const void* d_cb, float scale, const float* d_x, float* d_y,
                        int M, int K, int repeats, oilhip_kernel_perf_t* out, void* stream);

/* oil::engines::OIL{8,4,2}Engine::quant_gemm (include/oil/oil_engines.h:49,78,151;
 * src/oil_engines_oil8.cpp:197-216, oil4.cpp:238-261, oil2.cpp:210-229):
 *   C[m*N+n] = sum_k A[m*K+k] * cb[code(k*N+n)],  [K][N] packed codes, bits in {2,4,8} */
int oilhip_engine_quant_gemm(int bits, const float* d_a, const uint8_t* d_b_idx, const float* d_cb,
                             float* d_c, int64_t M, int64_t N, int64_t K, void* stream);

/* The engines whose B operand is not a codebook index, same [K][N] flat layout and loop order:
 *   kind 1  Oil1Engine::quant_gemm  (include/oil/oil_engines.h:123, src/oil_engines_oil1.cpp:61-82):
 *           d_b = one float per 32 flat positions
 *   kind 3  SparkEngine::quant_gemm (oil_engines.h:103, src/oil_engines_spark.cpp:154-186): d_b = 2-bit codes
 *           (2 -> +, 0 -> -, else 0), d_scales[flat / block] with block = the engine's block size
 *   kind 16 OIL16Engine::quant_gemm (oil_engines.h:167, src/oil_engines_fp.cpp:433-451): d_b = FP16 bits
 *   kind 32 OIL32Engine::quant_gemm (src/oil_engines_fp.cpp:531-547): d_b = FP32                        */
/* OIL{8,4,2}Engine::dequant_tensor (oil_engines.h:48,77,150; src/oil_engines_oil8.cpp:171-183, oil4.cpp:205-220,
 * oil2.cpp:184-193) when d_scales is NULL: n packed codes -> codebook values.  With d_scales:
 * OIL8Engine::dequantize_per_block (src/oil_engines_oil8.cpp:121-134, one scale per block) and
 * OIL4Engine::dequantize_per_block (src/oil_engines_oil4.cpp:136-150, {center, half_range} per block) over one
 * index byte per weight. */
int oilhip_engine_dequant(int bits, const uint8_t* d_idx, const float* d_cb, int64_t n, const float* d_scales,
                          int64_t block, float* d_out, void* stream);
int oilhip_engine_dense_gemm(int kind, const float* d_a, const void* d_b, const float* d_scales, int64_t block,
                             float* d_c, int64_t M, int64_t N, int64_t K, void* stream);

/* oil::kernel::tl1_gemm (kind 1) / tl2_gemm (kind 2) (include/oil/kernel.h:11-18, src/kernel_tl.cpp:32-90,124-184):
 * d_w holds one packed row of K two-bit ternary codes per (m, n) pair -- (K+3)/4 bytes for TL1, ((K+11)/12)*3 for
 * TL2 --, d_act is [N][K] FP32, quantized per row to int8 with scale 127 / max|a| as the reference does;
 * d_out[m*N+n] = (sum of products) / scale[n], TL1 with every pair sum clamped to int8 first.  Bit-identical to the
 * reference.  TL2 needs K % 3 == 0 (beyond that the reference reads past the activation row): OILHIP_E_ARG otherwise. */
int oilhip_tl_gemm(int kind, const uint8_t* d_w, const float* d_act, float* d_out, int M, int N, int K, void* stream);

/* backend::ComputeBackend's dense FP32 operations (include/oil/backend.h:49-80) on device pointers, with the meaning
 * of their CPU bodies in src/math.cpp (gemv :50-70, gemm :72-95, relu/gelu/silu :97-126, layer_norm :146-178,
 * rms_norm :180-203, softmax :205-247, add/mul/scale :249-283): what a gfx950 backend object behind
 * ComputeBackend::create runs.  Row-major, contiguous.
 *   gemm    : C[M][N] = alpha * A[M][K] . B[K][N] + beta * C      gemv : y[M] = alpha * A[M][N] . x + beta * y
 *   norm    : kind 0 layer_norm (mean/variance in double, gamma and beta), kind 1 rms_norm (gamma only, d_beta
 *             unused), over `rows` rows of n
 *   softmax : over `dim` entries that lie `inner` apart, for each of outer x inner lines
 *   map     : op 0 relu, 1 gelu (erf form), 2 silu, 3 a + b, 4 a * b, 5 s * a, 6 fill with s                  */
int oilhip_dense_gemm_f32(float alpha, const float* d_a, const float* d_b, float beta, float* d_c,
                          int64_t M, int64_t N, int64_t K, void* stream);
int oilhip_dense_gemv_f32(float alpha, const float* d_a, const float* d_x, float beta, float* d_y,
                          int64_t M, int64_t N, void* stream);
int oilhip_dense_norm_f32(int kind, const float* d_x, const float* d_gamma, const float* d_beta, float eps,
                          float* d_y, int64_t rows, int64_t n, void* stream);
int oilhip_dense_softmax_f32(const float* d_x, float* d_y, int64_t outer, int64_t dim, int64_t inner, void* stream);
int oilhip_dense_map_f32(int op, const float* d_a, const float* d_b, float s, float* d_y, int64_t n, void* stream);

/* ------------------------------------------------------------ decode-step pieces
 * oilhip_weights_stack_rows : several uploaded tensors of one width (full 256-weight blocks only) as one tensor of
 *                             their rows in order; the parts stay valid.  Parts of one format and regular layout
 *                             are copied on the device; parts that mix formats, or differ in format, are fetched
 *                             back and laid out afresh as one mixed tensor.  Lets the gate and up projections (or
 *                             q, k, v) run as one launch.  No reference counterpart: the reference walks each
 *                             tensor separately.
 * oilhip_rmsnorm_f32        : Qwen35Engine::rmsnorm (src/adapters/tools/qwen35_engine.cpp:39-44) over `rows` rows of
 *                             n floats: out = x * r * (1 + w), r = 1 / sqrt(mean(x^2) + 1e-6)
 * oilhip_gemv_rmsnorm_f32   : y[M][rows] = W . rmsnorm(x; normw), the rmsnorm + gemm pair in front of every projection
 *                             (:484-486 attention input, :611-614 MLP input).  With M = 1 and an OIL4 or window-stream
 *                             tensor the norm is formed while the GEMV stages x (one launch, d_xn unused and may be NULL);
 *                             otherwise d_xn[M][cols] receives the normalised rows and the GEMV reads them.
 * oilhip_mlp_step_f32       : Qwen35Engine::mlp_step (:611-621): y[M][D] = down(siluf(gate x) * up x), gate_up = the
 *                             gate and up projections stacked (2F x D, gate rows first), down = D x F.  A non-NULL
 *                             d_normw applies rmsnorm(x; d_normw) first, as the caller of mlp_step does.
 *                             d_scratch holds M * (3*F + D) floats.  With M = 1 and OIL4 or window-stream tensors the
 *                             norm rides on the first GEMV and the SwiGLU product on the second: two launches for the
 *                             whole step.
 * oilhip_embed_rows_f32     : the embedding lookup of Qwen35Engine::append_token (:756-760, decode_block :17-28):
 *                             rows d_ids[i] of a quantized [vocab][cols] tensor decoded to d_out[i][cols]; ids outside
 *                             the table give zero rows */
int oilhip_weights_stack_rows(const oilhip_weights* const* parts, int n, oilhip_weights** out);
int oilhip_rmsnorm_f32(const float* d_x, const float* d_w, int n, int rows, float* d_out, void* stream);
int oilhip_gemv_rmsnorm_f32(const oilhip_weights* w, const float* d_x, const float* d_normw, float* d_y, int M, float* d_xn,
                            void* stream);
int oilhip_mlp_step_f32(const oilhip_weights* gate_up, const oilhip_weights* down, const float* d_x, const float* d_normw,
                        float* d_y, int M, float* d_scratch, void* stream);
int oilhip_embed_rows_f32(const oilhip_weights* w, const int32_t* d_ids, int n, float* d_out, void* stream);

/* ------------------------------------------------------------ mixture of experts
 * oilhip_moe_route   : moe::softmax_with_topk (include/oil/moe_variants.h:693, src/moe_variants.cpp:97-134).
 *                      Host arrays: logits/probs [T][E], indices (int64) and weights [T][k]; weights are the
 *                      raw probabilities (no renormalisation), ties as std::partial_sort leaves them.
 * oilhip_moe_forward : moe::moe_dispatch_batched (moe_variants.h:701-706, src/moe_variants.cpp:767-827) with
 *                      ExpertFFN::forward (:77-91, SiLU): d_out[T][D] = sum over a token's experts of
 *                      w * down_e(silu(gate_e x) * up_e x), experts visited in ascending order, tokens of an
 *                      expert in ascending order.  gate[e], up[e]: F x D tensors, down[e]: D x F (Y = X W^T,
 *                      no bias, any wire format with full blocks; uniform OIL4 runs the fast kernel).
 *                      indices/weights are host arrays [T][K]; entries outside [0,E) are ignored, pairs with
 *                      weight <= 0 are counted in *dropped.  d_workspace: device memory of at least
 *                      oilhip_moe_workspace_bytes(T, K, D, F) bytes.  Returns after the token lists are on the
 *                      device; with z_loss != NULL it also waits for the result (sum of squared contributions).
 *                      Calls sharing a workspace must be ordered by the caller. */
int oilhip_moe_route(const float* logits, int64_t T, int64_t E, int64_t k, float* probs, int64_t* indices, float* weights);
size_t oilhip_moe_workspace_bytes(int64_t T, int64_t K, int64_t D, int64_t F);
int oilhip_moe_forward(const oilhip_weights* const* gate, const oilhip_weights* const* up,
                       const oilhip_weights* const* down, int E, const float* d_x, const int64_t* indices,
                       const float* weights, int64_t T, int64_t K, float* d_out, void* d_workspace,
                       size_t workspace_bytes, float* z_loss, int64_t* dropped, void* stream);

/* ------------------------------------------------------------ OIL4 KV cache
 * The device-resident oil::OIL4KVCache (include/oil/kv_cache_oil4.h:26-83, src/kv_cache_oil4.cpp): per layer the K and
 * V streams [token][heads * dim] as 4-bit codes (two per byte, low nibble first) with 16 FP16 centroids per block of
 * 32 / 64 / 128 consecutive values (any other block_size means 64, :25-26).  Codes and centroids are the
 * reference's bit for bit (inputs must be finite), also where heads * dim is odd and the reference's chunks share bytes.
 * oilhip_kv_create            : OIL4KVCache(num_layers, max_seq_len, num_heads, head_dim, block_size) / init (:13-43)
 * oilhip_kv_append            : append(layer, k, v) (:207-291); d_k, d_v: [seq_len][heads * dim] FP32 on the device.
 *                               Tokens beyond max_seq_len are dropped but still counted, layer >= num_layers is ignored,
 *                               as in the reference.  Chunks are quantized by the 16-level Lloyd-Max of :75-153.
 * oilhip_kv_get_range         : get_range(layer, start, end) (:293-362) -> d_k, d_v [len][heads * dim] FP32, *len = tokens
 *                               written (end is clipped to the tokens held; 0 where the reference returns empty tensors).
 *                               get_all is get_range(layer, 0, context).  Tokens that were dropped are never returned
 *                               (the reference reads past its arrays there).
 * oilhip_kv_info              : context_len() (layer 0), block_size(), size_bytes(), size_bytes_fp32_equivalent() (:364-392)
 * oilhip_kv_clear / _resize   : clear() (:394-402), resize(new_max_seq_len) (:404-416, every layer empty afterwards;
 *                               synchronises the device and reallocates)
 * oilhip_kv_state             : host copies of a layer's code and centroid arrays ((max_seq*heads*dim+1)/2 bytes and
 *                               16 uint16 per block each) for checks and checkpoints; any pointer may be NULL
 * oilhip_kv_quantize_blocks   : OIL4KVCache::quantize_block_oil4 (:165-168) over nblocks runs of n <= 128 values:
 *                               d_codes one code per byte [nblocks][n], d_cb16 [nblocks][16]
 * oilhip_kv_dequantize_blocks : OIL4KVCache::dequantize_block_oil4 (:170-174), any n, through
 *                               CodebookOIL4::half_to_float (src/codebook.cpp:36-64) */
typedef struct oilhip_kv oilhip_kv;
int oilhip_kv_create(int num_layers, int64_t max_seq_len, int64_t num_heads, int64_t head_dim, int64_t block_size,
                     oilhip_kv** out);
int oilhip_kv_destroy(oilhip_kv* c);
int oilhip_kv_append(oilhip_kv* c, int layer, const float* d_k, const float* d_v, int64_t seq_len, void* stream);
int oilhip_kv_get_range(const oilhip_kv* c, int layer, int64_t start, int64_t end, float* d_k, float* d_v, int64_t* len_out,
                        void* stream);
int oilhip_kv_info(const oilhip_kv* c, int* context_len, int64_t* block_size, uint64_t* size_bytes, uint64_t* fp32_bytes);
int oilhip_kv_clear(oilhip_kv* c, void* stream);
int oilhip_kv_resize(oilhip_kv* c, int64_t new_max_seq_len);
int oilhip_kv_state(const oilhip_kv* c, int layer, uint8_t* k_idx, uint8_t* v_idx, uint16_t* k_cb, uint16_t* v_cb);
int oilhip_kv_quantize_blocks(const float* d_src, int64_t n, int64_t nblocks, uint8_t* d_codes, uint16_t* d_cb16, void* stream);
int oilhip_kv_dequantize_blocks(const uint8_t* d_codes, const uint16_t* d_cb16, float* d_dst, int64_t n, int64_t nblocks,
                                void* stream);

#ifdef __cplusplus
}
#endif
#endif
