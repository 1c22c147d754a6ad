/*
 * f2cgt.h — C ABI of libf2cgt_hip.so: hand-written gfx950 (MI355X) kernels for the
 * fused feature-decompression + neighbour-aggregation path of F2CGT.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer to a dense row-major buffer unless stated;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); every call
 *     only enqueues work on that stream: no device-wide synchronisation, no host
 *     read-back, no allocation (outputs are caller-allocated);
 *   - return value 0 = success, < 0 = rejected arguments (F2CGT_E_*), > 0 = hipError_t
 *     of a failed launch; f2cgt_last_error() gives the message of the calling thread's
 *     last failure;
 *   - dtype arguments take the F2CGT_DT_* tags below;
 *   - CSC = indptr[num_rows + 1], indices[num_edges], both of `idx_dtype`
 *     (F2CGT_DT_I32 or F2CGT_DT_I64).  Source ids are clamped to [0, num_src_rows) and
 *     edge offsets to [0, num_edges], so malformed graphs give wrong sums, not faults.
 *
 * Each entry point names the reference interface (file:line under the reference
 * checkout) whose device work it replaces.
 */
#ifndef F2CGT_H_
#define F2CGT_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  F2CGT_DT_U8 = 0,
  F2CGT_DT_I8 = 1,
  F2CGT_DT_I16 = 2,
  F2CGT_DT_I32 = 3,
  F2CGT_DT_I64 = 4,
  F2CGT_DT_F16 = 5,
  F2CGT_DT_F32 = 6,
  F2CGT_DT_F64 = 7
};

enum {
  F2CGT_OK = 0,
  F2CGT_E_INVALID = -1,     /* bad size / null pointer / misaligned buffer */
  F2CGT_E_UNSUPPORTED = -2, /* dtype, target_bits or shape the kernels do not cover */
  F2CGT_E_DEVICE = -3       /* no usable gfx950 device */
};

enum { F2CGT_METRIC_L2 = 0, F2CGT_METRIC_COSINE = 1 };

/* Library version (major * 100 + minor). */
int f2cgt_version(void);

/* Message of the calling thread's most recent failure ("" if none). */
const char* f2cgt_last_error(void);

/* Number of compute units of the current device (the kernels size their grids by it). */
int f2cgt_num_cus(void);

/* How the row-block aggregation kernels (the SQ and affine-SQ fused operators) write their output
 * (no counterpart in the reference, whose kernels use plain stores, src/fusion_spmm.cu:173-236).
 *   F2CGT_STORE_AUTO    (default) outputs above 220 MB (above 140 MB when the output rows are whole
 *                       128-byte lines or the graph has six or more edges per row) are streamed past
 *                       the caches with non-temporal stores, smaller ones are written with plain stores
 *   F2CGT_STORE_STREAM  always streamed: the launch time no longer depends on what the caches hold
 *   F2CGT_STORE_CACHED  never streamed
 * Plain stores are fastest when the same output buffer is written again before the last-level cache
 * (256 MB) has been turned over, as in a loop over one buffer; a caller whose outputs are written
 * once and consumed later (a training step with other large kernels in between) is better off
 * streaming.  The fused VQ operator stores through the same path in every mode; in F2CGT_STORE_STREAM it
 * takes, at up to 16 edges per row, the form whose store instructions write whole lines (a few per cent
 * slower into a buffer that is still cached, 14 % faster into one that is not).
 * Results are identical in every mode.  Process-wide; returns the previous mode, or
 * F2CGT_E_INVALID for a value that is none of the three (the mode is then unchanged). */
#define F2CGT_STORE_AUTO 0
#define F2CGT_STORE_STREAM 1
#define F2CGT_STORE_CACHED 2
int f2cgt_set_store_mode(int mode);

/* Dry runs of the fused aggregation entry points (no counterpart in the reference; for tests and
 * tools that want to know what a shape dispatches to, with or without a GPU).  While switched on
 * for the calling thread, f2cgt_spmm_csr and the f2cgt_*_spmm_csr operators validate their
 * arguments and choose kernel and launch geometry exactly as usual, then return 0 without touching
 * the device or dereferencing any pointer (pointers only need the alignment of the real buffers;
 * the device is taken to have 256 compute units).  f2cgt_last_plan copies the last choice:
 * grid / block / lds_bytes of the launch, destination rows per workgroup (0 = not row-blocked),
 * and kernel-specific lane-group counts in aux[] (every one of them must be >= 1 for the kernel's
 * loops to advance).  f2cgt_set_plan_only returns the previous setting. */
typedef struct {
  char kernel[48];
  int64_t grid;
  int32_t block;
  int64_t lds_bytes;
  int32_t rows_per_block;
  int32_t aux[4];
} f2cgt_plan;
int f2cgt_set_plan_only(int on);
int f2cgt_last_plan(f2cgt_plan* out);

/* ---- bit packing ------------------------------------------------------------- */

/* Replaces packbits(), src/packbits.cu:44-64 (kernel :6-42).
 * unpack uint8 [rows, unpack_dim] -> pack uint8 [rows, ceil(unpack_dim / (8/bits))];
 * element i of a group goes to bits [bits*i, bits*(i+1)); target_bits in {1,2,4}. */
int f2cgt_packbits(const uint8_t* unpack, uint8_t* pack, int64_t rows, int64_t unpack_dim,
                   int target_bits, void* stream);

/* Replaces unpackbits(), src/packbits.cu:96-114 (kernel :66-94).
 * pack uint8 [rows, pack_dim] -> unpack uint8 [rows, unpack_dim]. */
int f2cgt_unpackbits(const uint8_t* pack, uint8_t* unpack, int64_t rows, int64_t pack_dim,
                     int64_t unpack_dim, int target_bits, void* stream);

/* ---- scalar quantisation (log domain, the reference's SQ) ---------------------- */

/* Replaces sq_compress(), src/sq_quantization.cu:65-83 (kernel :5-63).
 * src fp32 [rows, feat_dim] -> dst fp32 [rows, feat_dim] of integer-valued codes;
 * codebooks fp32 [num_codebooks, 5] = fmin,fmax,emin,emax,mean; column j uses
 * codebook j / column_slice; target_bits in {1,2,4,8,16}. */
int f2cgt_sq_compress(const float* src, float* dst, const float* codebooks, int64_t rows,
                      int64_t feat_dim, int64_t num_codebooks, int target_bits,
                      int64_t column_slice, void* stream);

/* One-pass form of the three calls every caller of sq_compress() makes next
 * (examples/process_compress.py:128-139: sq_compress -> cast -> packbits): writes the storage
 * tensor directly.  dst: uint8 [rows, ceil(feat_dim * bits / 8)] packed low bits first for
 * bits in {1,2,4}; int8 [rows, feat_dim] for 8; int16 [rows, feat_dim] for 16.  Bit for bit what
 * f2cgt_sq_compress + integer cast + f2cgt_packbits give. */
int f2cgt_sq_encode(const float* src, void* dst, const float* codebooks, int64_t rows,
                    int64_t feat_dim, int64_t num_codebooks, int target_bits, int64_t column_slice,
                    void* stream);

/* Replaces sq_decompress(), src/sq_quantization.cu:158-182 (kernel :85-156).
 * codes [rows, src_dim] of code_dtype (U8/I8 packed bytes for bits < 8, I8 for 8, I16 for 16)
 * -> out fp32 [rows, feat_dim].  Codebook per OUTPUT column.  8-bit codes are signed; U8 with
 * target_bits 8 is refused (F2CGT_E_UNSUPPORTED): the reference's dtype dispatch
 * (src/common.h:68-82) would read such a tensor as 0..255, which its encoder never writes. */
int f2cgt_sq_decompress(const void* codes, int code_dtype, float* out, const float* codebooks,
                        int64_t rows, int64_t src_dim, int64_t feat_dim,
                        int64_t num_codebooks, int target_bits, int64_t column_slice,
                        void* stream);

/* Per-column affine SQ decode (no counterpart in the reference; defined by the
 * benchmark configurations): out[r][c] = params[c] + code * params[feat_dim_stride + c]
 * with params fp32 [2, param_stride] (row 0 = min, row 1 = scale), unsigned codes,
 * sub-byte codes packed low bits first; target_bits in {1,2,4,8}. */
int f2cgt_sq_affine_decompress(const uint8_t* codes, float* out, const float* params,
                               int64_t param_stride, int64_t rows, int64_t src_dim,
                               int64_t feat_dim, int target_bits, void* stream);

/* ---- vector quantisation decode ---------------------------------------------- */

/* Replaces vq_decompress(), src/vq_quantization.cu:35-60 (kernel :5-33).
 * codes [rows, num_codebooks] (U8/I8/I16), codebooks [num_codebooks, K, width]
 * (F32 or F16) -> out fp32 [rows, feat_dim], feat_dim <= num_codebooks * width. */
int f2cgt_vq_decompress(const void* codes, int code_dtype, const void* codebooks, int cb_dtype,
                        float* out, int64_t rows, int64_t feat_dim, int64_t num_codebooks,
                        int64_t K, int64_t width, void* stream);

/* ---- CSC mean aggregation ---------------------------------------------------- */

/* Replaces SpMMCsr(), src/fusion_spmm.cu:45-70 (kernel :13-43).
 * feat [num_src_rows, feat_dim] of feat_dtype (F32/F16/F64) -> out same dtype
 * [num_rows, feat_dim]; out[r] = sum(feat[indices[e]]) / max(deg, 1). */
int f2cgt_spmm_csr(const void* feat, int feat_dtype, void* out, const void* indptr,
                   const void* indices, int idx_dtype, int64_t num_rows, int64_t num_edges,
                   int64_t num_src_rows, int64_t feat_dim, void* stream);

/* Replaces VqDecompressSpMMFusionCsr(), src/fusion_spmm.cu:107-141 (kernel :72-105,
 * decode src/cuda_utils.cuh:48-58).  fp32 codebooks; out fp32 [num_rows, feat_dim]. */
int f2cgt_vq_decompress_spmm_csr(const void* codes, int code_dtype, const float* codebooks,
                                 const void* indptr, const void* indices, int idx_dtype,
                                 float* out, int64_t num_rows, int64_t num_edges,
                                 int64_t num_src_rows, int64_t feat_dim,
                                 int64_t num_codebooks, int64_t K, int64_t width,
                                 void* stream);

/* Replaces SqDecompressSpMMFusionCsr(), src/fusion_spmm.cu:240-272 (kernel :143-238).
 * Codebook per PACKED BYTE (:180): byte j uses codebook j*(8/bits) / column_slice, which
 * equals the per-column choice of f2cgt_sq_decompress iff column_slice % (8/bits) == 0.
 * Code dtypes as for f2cgt_sq_decompress (8-bit codes must be I8). */
int f2cgt_sq_decompress_spmm_csr(const void* codes, int code_dtype, const float* codebooks,
                                 const void* indptr, const void* indices, int idx_dtype,
                                 float* out, int64_t num_rows, int64_t num_edges,
                                 int64_t num_src_rows, int64_t src_dim, int64_t feat_dim,
                                 int64_t num_codebooks, int target_bits, int64_t column_slice,
                                 void* stream);

/* Fused per-column affine SQ decode + mean aggregation (benchmark-defined extension;
 * argument order follows f2cgt_sq_decompress_spmm_csr). */
int f2cgt_sq_affine_decompress_spmm_csr(const uint8_t* codes, const float* params,
                                        int64_t param_stride, const void* indptr,
                                        const void* indices, int idx_dtype, float* out,
                                        int64_t num_rows, int64_t num_edges,
                                        int64_t num_src_rows, int64_t src_dim,
                                        int64_t feat_dim, int target_bits, void* stream);

/* Two-table fused decode + mean aggregation (benchmark-defined extension; the reference's
 * two-level mode, examples/compress.py:39-54,74-106, never mixes tables in one call).
 * row_map int32 [num_src_rows]: m >= 0 -> row m of the 8-bit affine SQ table
 * (sq_codes uint8 [num_sq_rows, feat_dim], sq_params fp32 [2, param_stride]);
 * m < 0 -> row -m-1 of the VQ table (vq_codes uint8 [num_vq_rows, num_codebooks],
 * vq_codebooks fp32 [num_codebooks, K, width]). */
int f2cgt_hybrid_decompress_spmm_csr(const int32_t* row_map, const uint8_t* sq_codes,
                                     const float* sq_params, int64_t param_stride,
                                     const uint8_t* vq_codes, const float* vq_codebooks,
                                     const void* indptr, const void* indices, int idx_dtype,
                                     float* out, int64_t num_rows, int64_t num_edges,
                                     int64_t num_src_rows, int64_t num_sq_rows,
                                     int64_t num_vq_rows, int64_t feat_dim,
                                     int64_t num_codebooks, int64_t K, int64_t width,
                                     void* stream);

/* ---- row fetch in front of the operators -------------------------------------- */

/* Replaces TensorCache.__getitem__, examples/tensor_cache.py:49-58: shmtensor.capi.uva_fetch
 * (slot_map NULL) and shmtensor.capi.cache_fetch (hot table + id -> slot map; the reference
 * keeps a GPU hash map, examples/tensor_cache.py:80-86, here a dense int32 array).
 * Tables hold opaque rows of row_bytes bytes each (code rows or plain feature rows).
 * out[i, :] = hot[slot_map[id], :] if slot_map && 0 <= slot_map[id] < num_hot_rows
 *            else table[id, :],   id = index[i] clamped to [0, num_rows).
 * `table` may be pinned host memory mapped into the device address space (its rows then
 * cross the host link); hot, slot_map [num_rows], index [num_index] and out
 * [num_index, row_bytes] are device buffers.  No alignment is required of any of them. */
int f2cgt_fetch_rows(const void* table, const void* hot, const int32_t* slot_map,
                     const void* index, int idx_dtype, void* out, int64_t num_index,
                     int64_t row_bytes, int64_t num_rows, int64_t num_hot_rows, void* stream);

/* ---- VQ encode ---------------------------------------------------------------- */

/* Replaces pairwise_distance(), src/kmeans.cu:102-118 (raft L2Unexpanded /
 * CosineExpanded).  x fp32 [m,k], y fp32 [n,k] -> dist fp32 [m,n]; metric L2 is the
 * squared distance sum((x-y)^2). */
int f2cgt_pairwise_distance(const float* x, const float* y, float* dist, int64_t m, int64_t n,
                            int64_t k, int metric, void* stream);

/* Replaces KMeans::predict(), src/kmeans.cu:77-98 (raft kmeans_predict) and the argmin
 * the callers run on pairwise_distance (examples/my_kmeans.py:116-125).
 * x fp32 [m,k], centers fp32 [n,k], n <= 65536.  Writes the index of the nearest centre
 * (first minimum) to labels_i64 [m] and/or labels_u8 [m] (either may be NULL; labels_u8
 * needs n <= 256).  The distance matrix is never materialised. */
int f2cgt_kmeans_predict(const float* x, const float* centers, int64_t* labels_i64,
                         uint8_t* labels_u8, int64_t m, int64_t n, int64_t k, int metric,
                         void* stream);

/* One Lloyd iteration's centre update, after f2cgt_kmeans_predict has produced the labels.
 * Replaces the update half of the reference's two training loops: compute_new_centers and the
 * centre-shift test of examples/my_kmeans.py:87-113,128-147 (plain mean whatever the metric, a centre
 * without members keeps its value) and the loop inside raft::cluster::kmeans::fit, src/kmeans.cu:61-75.
 * x fp32 [m,k]; labels int64 [m] or uint8 [m] (exactly one non-NULL; values clamped to [0,n));
 * centers fp32 [n,k], updated in place; shift fp32 [2] (device) receives sum_c |dc| and sum_c |dc|^2.
 * stop (device int32, may be NULL): when it is nonzero on entry the call does nothing, and the call
 * sets it when stop_rule says the centres are final (1: sum_c |dc|^2 < tol, raft's rule; 2:
 * (sum_c |dc|)^2 < tol, the rule of examples/my_kmeans.py:105; 0: never) -- a training loop can then
 * run without reading anything back per iteration.  workspace: device scratch for the partial sums,
 * at least f2cgt_kmeans_update_workspace_bytes(n, k) bytes, 16-byte aligned, contents irrelevant.
 * The sums are fp32 atomic adds: their last bits depend on the order the hardware takes them in. */
int64_t f2cgt_kmeans_update_workspace_bytes(int64_t n, int64_t k);
int f2cgt_kmeans_update(const float* x, const int64_t* labels_i64, const uint8_t* labels_u8, float* centers,
                        float* shift, int32_t* stop, int stop_rule, float tol, void* workspace,
                        int64_t workspace_bytes, int64_t m, int64_t n, int64_t k, void* stream);

/* f2cgt_kmeans_update without a workspace and without any allocation (no counterpart in the
 * reference: it is for callers that cannot allocate device memory -- code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  The partial sums live in a device array
 * inside the library (272 KB per device, kept until the process ends), so the problem is limited to
 * n * k <= 65536 sums and n <= 4096 centres; larger ones return F2CGT_E_UNSUPPORTED.  Same arguments,
 * results and stop-flag behaviour as f2cgt_kmeans_update.  Every call on a device uses that device's
 * one array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.
 * The first call on each device looks the array's address up (hipGetSymbolAddress, which may load
 * the code object): make that first call outside any stream capture; later calls only launch kernels. */
int f2cgt_kmeans_update_static(const float* x, const int64_t* labels_i64, const uint8_t* labels_u8,
                               float* centers, float* shift, int32_t* stop, int stop_rule, float tol,
                               int64_t m, int64_t n, int64_t k, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* F2CGT_H_ */
