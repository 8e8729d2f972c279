/*
 * ternary_spmm.h -- C ABI of libternary_spmm.so: ternary (-1/0/+1) sparse GEMM for
 * AMD MI355X (gfx950).
 *
 * The library replaces the four callables of the reference's pybind11 module
 * `ter_spmm` (ternaryLLM_GPU/csrc/ter_spmm_wrapper.cu:350-355) and the two device
 * kernels behind them (ternaryLLM_GPU/csrc/ter_spmm_kernel.cuh:24-78, :106-308).
 *
 * Conventions
 *   - plain pointers and sizes only; no torch / ATen / pybind types.
 *   - every function returns an int status: TL_OK (0) or a negative TL_ERR_* code;
 *     tl_last_error() returns a thread-local message for the last failure.
 *   - the library never allocates or frees device memory.  Device buffers
 *     (inputs, outputs, workspace) are the caller's; sizes come from the *_size /
 *     *_workspace calls.
 *   - host packers write into caller-provided arrays after a sizing call.
 *   - compute entry points enqueue on the hipStream_t passed as `void* stream`
 *     (NULL = the default stream) and return without synchronising.
 *   - all functions are re-entrant.  Process-wide state: the thread-local error text;
 *     the tuning knobs, read from the environment at the first launch (TL_* variables,
 *     see tl_reload_options); the compute-unit count of each device, asked once; and
 *     set-once flags that record that a kernel's LDS limit has been raised.
 */
#ifndef TERNARY_SPMM_H
#define TERNARY_SPMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes ------------------------------------------------------ */
#define TL_OK 0
#define TL_ERR_ARG (-1)         /* null pointer, negative size, bad flag          */
#define TL_ERR_SHAPE (-2)       /* sizes inconsistent with each other             */
#define TL_ERR_DTYPE (-3)       /* unknown dtype code                             */
#define TL_ERR_ALIGN (-4)       /* pointer or leading dimension not aligned       */
#define TL_ERR_UNSUPPORTED (-5) /* valid request this build cannot serve          */
#define TL_ERR_LAUNCH (-6)      /* HIP reported an error at launch                */
#define TL_ERR_VALUE (-7)       /* data error: non-ternary weight, count mismatch */
#define TL_ERR_SIZE (-8)        /* caller buffer too small                        */
#define TL_ERR_FORMAT (-9)      /* packed blob failed validation                  */

/* ---- dtype / layout / flag codes --------------------------------------- */
#define TL_F32 0
#define TL_F16 1

#define TL_X_ROW_MAJOR 0 /* X is [M][ldx], K contiguous (what the nn.Module callers pass)      */
#define TL_X_K_MAJOR 1   /* X is [K][ldx], M contiguous (what the reference kernel itself reads, */
                         /* ter_spmm_kernel.cuh:173)                                            */

#define TL_PRODUCER_NONE 0        /* x = in                                                    */
#define TL_PRODUCER_SILU_GATE 1   /* tl_spmv_fused: x = silu(in[:K]) * in[K:]                  */
#define TL_PRODUCER_ADD_RMSNORM 2 /* tl_spmv_fused: x = RMSNorm(in + in2) * norm_weight        */
#define TL_PRODUCER_RMSNORM 3     /* tl_spmv_fused: x = RMSNorm(in) * norm_weight, factor applied to the sums */
#define TL_PRODUCER_RMSNORM_SUMS 4 /* tl_spmv_fused: TL_PRODUCER_RMSNORM on what tl_spmv_add_norm left behind */

#define TL_ACT_NONE 0
#define TL_ACT_SILU_GATE 1 /* out = silu(gate) * up, for tl_mlp_gate_up */

const char* tl_last_error(void);
int tl_version(void);

/* The launchers' tuning knobs (environment variables TL_SMALL_LDS, TL_TILE_GROUP, TL_QUAD_SHARE, TL_LW,
 * TL_SPMV_SHARE, TL_SPMV_WIDE, TL_SPMV_TILES, TL_SMALL_MT, TL_SPMV_DIRECT, TL_BLOCK_SET, TL_ROWS_SPLIT,
 * TL_OCTET, TL_QUAD_WIDE, TL_RES16; unset = the launcher's own choice) are read once per process.  This
 * reads them again -- for tests and tuning runs that change them between calls. */
int tl_reload_options(void);

/* ======================================================================== */
/* Host packers: bit-exact replacements of the reference's converters.      */
/* `w` is a host, row-major int32 [inners][columns] matrix with values in   */
/* {-1, 0, +1}; argument order follows the reference (columns BEFORE        */
/* inners, cnt_pos BEFORE cnt_neg, outputs negative stream first).          */
/* ======================================================================== */

/* Counts the +1 and -1 entries (the reference caller does this in Python,
 * TernaryLinear.py:104-105).  Fails with TL_ERR_VALUE on any other value. */
int tl_count_nnz(const int32_t* w, int columns, int inners, int64_t* cnt_pos, int64_t* cnt_neg);

/* Replaces convert_to_ter_csc (ter_spmm_wrapper.cu:39-78).
 * neg_row[cnt_neg], neg_off[columns+1], pos_row[cnt_pos], pos_off[columns+1]. */
int tl_convert_to_ter_csc(const int32_t* w, int columns, int inners, int cnt_pos, int cnt_neg,
                          int32_t* neg_row, int32_t* neg_off, int32_t* pos_row, int32_t* pos_off);

/* Replaces convert_to_ter_tiled_csc (ter_spmm_wrapper.cu:92-152).
 * Offsets hold columns * ceil(inners / tile_k) * 2 entries:
 * off[(y*T + t)*2 + {0,1}] = [start, end) of tile t of column y; row indices are
 * tile-local.  Rows past `inners` in a ragged last tile count as zero (the
 * reference reads out of bounds there). */
int tl_convert_to_ter_tiled_csc(const int32_t* w, int columns, int inners, int cnt_pos, int cnt_neg,
                                int tile_k, int32_t* neg_row, int32_t* neg_off_tiled,
                                int32_t* pos_row, int32_t* pos_off_tiled);

/* Sizing call for tl_convert_to_ter_tiled_mcsc: number of entries of the merged
 * index array (cnt_pos + cnt_neg, or the padded total, ter_spmm_wrapper.cu:198-230). */
int tl_tiled_mcsc_size(const int32_t* w, int columns, int inners, int cnt_pos, int cnt_neg,
                       int tile_k, int padding, int padding_size, int64_t* n_index);

/* Replaces convert_to_ter_tiled_mcsc + inter_tile_swizzle
 * (ter_spmm_wrapper.cu:156-315, :9-27), including the truncation of the pair and
 * remainder counts to multiples of 4 (:277-291) and the overwrite order.
 * merged_row[n_index], merged_off[columns*T*4], col_tile_idx[columns*T]. */
int tl_convert_to_ter_tiled_mcsc(const int32_t* w, int columns, int inners, int cnt_pos, int cnt_neg,
                                 int tile_k, int padding, int padding_size,
                                 int32_t* merged_row, int64_t n_index,
                                 int32_t* merged_off, int32_t* col_tile_idx);

/* Decodes merged arrays back to the ternary matrix they encode, i.e. the matrix
 * the reference kernels' loops (ter_spmm_kernel.cuh:197-300) would multiply by.
 * index_width is 2 (int16, what TernaryLinear stores, TernaryLinear.py:110) or 4.
 * w_out is int32 [inners][columns].  TL_ERR_VALUE when an entry of the decoded
 * matrix falls outside {-1, 0, +1} (possible only with padded arrays). */
int tl_tiled_mcsc_to_dense(const void* merged_row, int index_width, int64_t n_index,
                           const int32_t* merged_off, int columns, int inners, int tile_k,
                           int32_t* w_out);

/* ======================================================================== */
/* Device format ("wave-tiled CSC"): one relocatable blob, built on the     */
/* host from tiled CSC, copied to the GPU by the caller.                    */
/*   - K is cut into tiles of `tile_rows` <= 255 rows; indices are 8-bit    */
/*     tile-local, value 255 is a padding sentinel that addresses a zero.   */
/*   - columns are grouped in blocks of 16.  The unit of the stream is the  */
/*     chunk of one (block, tile): 16 descriptor dwords, then the runs of   */
/*     the block's 16 columns for that tile.  Per column the +1 rows and    */
/*     the -1 rows are two separate runs, each padded to a multiple of 4    */
/*     bytes (the -1 run follows the +1 run).  A chunk is padded to a       */
/*     multiple of 16 bytes.                                                */
/*   - descriptor: +1 count (bits 0-7), -1 count (bits 8-15), dword offset  */
/*     of the column's runs from the start of the chunk (bits 16-31).       */
/*   - the rows of a run may come in any order; a row may repeat (it is     */
/*     then added that many times) and may sit in both runs (it cancels):   */
/*     a blob built from dense ternary weights holds every row once, one    */
/*     built from the reference's merged arrays holds what they encode.     */
/*     The builder orders the rows of a run so that the LDS reads of the    */
/*     single-row kernel and of the 16-row kernel spread over the banks.    */
/*   - the stream is block-major: all tiles of block 0, then block 1, ...;  */
/*     chunkstart[block * T + tile] is the dword where a chunk begins       */
/*     (one extra entry marks the end).                                     */
/* The blob starts with a tl_layout_header (256 bytes).                     */
/* ======================================================================== */

#define TL_LAYOUT_MAGIC 0x35474C54u /* "TLG5" */
#define TL_LAYOUT_VERSION 5
#define TL_BLOCK_COLUMNS 16

typedef struct tl_layout_header {
    uint32_t magic;
    uint32_t version;
    uint32_t inners;      /* K */
    uint32_t columns;     /* N */
    uint32_t tile_rows;   /* rows per device tile, <= 255 */
    uint32_t n_tiles;     /* T = ceil(K / tile_rows) */
    uint32_t n_blocks;    /* NB = ceil(N / 16) */
    uint32_t max_chunk_dwords; /* largest chunk, descriptors included */
    uint64_t nnz_pos;
    uint64_t nnz_neg;
    uint64_t off_chunkstart; /* byte offset of uint32 chunkstart[NB*T + 1] (dword units into the stream) */
    uint64_t off_stream;     /* byte offset of the stream (descriptors + index bytes)                     */
    uint64_t stream_bytes;   /* bytes of the stream (multiple of 16)                                      */
    uint64_t total_bytes;    /* bytes of the blob that are in use, multiple of 256                        */
    uint32_t max_run_dwords; /* largest (+1 run dwords + -1 run dwords) of any (column, tile)             */
    uint32_t mean_run_dwords_x16; /* mean of the same, times 16, rounded up                               */
    uint64_t checksum;       /* FNV-1a (64-bit, one step per dword) over the chunk table, then the stream */
    uint32_t reserved[40];   /* zero */
} tl_layout_header;

/* Bytes of the blob that tl_layout_build will write for these tiled-CSC arrays
 * (as produced by tl_convert_to_ter_tiled_csc with tile height tile_k).
 * tile_rows = 0 picks the default (the largest balanced height <= 255). */
int tl_layout_size(const int32_t* neg_off_tiled, const int32_t* pos_off_tiled,
                   int columns, int inners, int tile_k, int tile_rows, int64_t* blob_bytes);

/* Builds the blob into host memory `blob` (blob_bytes as returned above).  The pass that orders the rows of each
 * tile runs on worker threads (environment variable TL_PACK_THREADS, read at every call; default: the hardware
 * threads, 8 at most, divided among the calls in that pass at the moment); the blob does not depend on their number. */
int tl_layout_build(const int32_t* neg_row, const int32_t* neg_off_tiled,
                    const int32_t* pos_row, const int32_t* pos_off_tiled,
                    int columns, int inners, int tile_k, int tile_rows,
                    void* blob, int64_t blob_bytes);

/* Convenience: dense int32 [inners][columns] -> blob (runs the tiled-CSC packer
 * internally).  Call with blob == NULL to get blob_bytes only. */
int tl_layout_from_dense(const int32_t* w, int columns, int inners, int tile_rows,
                         void* blob, int64_t* blob_bytes);

/* Builds the blob straight from the reference's merged tiled-CSC arrays
 * (convert_to_ter_tiled_mcsc, ter_spmm_wrapper.cu:156-315; index_width 2 = int16 as
 * TernaryLinear stores them, TernaryLinear.py:110, or 4), so that the product through
 * it is what the reference kernels' walk of those arrays adds up
 * (ter_spmm_kernel.cuh:197-300): per tile the pairs (+x[p] - x[n]) over
 * [off0, off1), then sign * x[c] over [off1, off2).  A row that the arrays name
 * several times (possible with padded arrays) is added that many times.
 * `uniformed` != 0 leaves the [off1, off2) part out, as the reference's kernels do
 * when that flag is set (ter_spmm_kernel.cuh:59,249).
 * Call with blob == NULL to get blob_bytes only. */
int tl_layout_from_mcsc(const void* merged_row, int index_width, int64_t n_index,
                        const int32_t* merged_off, int columns, int inners, int tile_k,
                        int uniformed, int tile_rows, void* blob, int64_t* blob_bytes);

/* Validates a host copy of a blob (header, bounds, monotone offsets, row range, sentinel use, checksum). */
int tl_layout_validate(const void* blob, int64_t blob_bytes);

/* Decodes a host blob back to dense int32 [inners][columns] (round-trip check): an entry is the
 * number of times its row sits in the column's +1 run minus the times it sits in the -1 run. */
int tl_layout_to_dense(const void* blob, int64_t blob_bytes, int32_t* w_out);

/* ======================================================================== */
/* Compute.                                                                 */
/* ======================================================================== */

/* Workspace bytes tl_spmm needs for M rows of x_dtype in x_layout (0 when none).
 * `header` is a host copy of the blob's first 256 bytes.  The workspace carries no
 * state between calls; two calls that may run concurrently need different ones. */
int tl_spmm_workspace(const tl_layout_header* header, int64_t M, int x_dtype, int x_layout,
                      int64_t* workspace_bytes);

/* Y[M][N] = (X[M][K] * W) * scale  -- replaces ter_spmm (ter_spmm_wrapper.cu:318-348)
 * and both kernels behind it (ter_spmm_kernel.cuh:24-78 for M = 1, :106-308 for M > 1).
 *   header      host copy of the blob header
 *   blob_dev    device pointer to the whole blob (256-byte aligned)
 *   X           device, x_dtype, layout x_layout, leading dimension ldx (elements)
 *   Y           device, y_dtype, row-major [M][ldy]
 *   scale       device per-output-column factor of scale_dtype, or NULL (the
 *               reference has none; its result equals scale == NULL)
 *   workspace   device scratch of at least tl_spmm_workspace() bytes (may be NULL when 0)
 * Accumulation is always fp32. */
int tl_spmm(const tl_layout_header* header, const void* blob_dev,
            const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
            void* Y, int y_dtype, int64_t ldy,
            const void* scale, int scale_dtype,
            void* workspace, int64_t workspace_bytes, void* stream);

/* tl_spmm for callers that cannot allocate or pass a workspace: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * arguments and result as tl_spmm, minus the workspace: what tl_spmm stages there (the K-major image of the
 * activations) goes into a 32 MiB array inside the library's device code, one copy per GPU, held until
 * the process ends.  The call allocates and frees nothing.  TL_ERR_SIZE when the image would not fit
 * (e.g. 1024 x 11008 fp16 fits, 1024 x 11008 fp32 does not).  The kernels write every byte of the array
 * before they read it, so nothing is cleared between calls; all calls on one GPU share the array, so
 * calls that may overlap on one GPU (different streams) race -- keep them on one stream or use tl_spmm.
 * The first call on a device looks the array's address up; make it outside graph capture. */
int tl_spmm_noalloc(const tl_layout_header* header, const void* blob_dev,
                    const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                    void* Y, int y_dtype, int64_t ldy,
                    const void* scale, int scale_dtype, void* stream);

/* H[M][N] = act(X*Wg * sg, X*Wu * su): the gate and up projections of the
 * reference's LlamaTernaryMLP (TernaryLLM/TernaryMLP.py:33-35) in one pass over X
 * with the SiLU-gate product fused into the epilogue (the reference runs two
 * ter_spmm calls and two elementwise kernels).  Both blobs must share K, N and
 * tile_rows.  Arguments as for tl_spmm. */
int tl_mlp_gate_up(const tl_layout_header* gate_header, const void* gate_blob_dev,
                   const tl_layout_header* up_header, const void* up_blob_dev,
                   const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                   void* H, int h_dtype, int64_t ldh,
                   const void* gate_scale, const void* up_scale, int scale_dtype,
                   int activation,
                   void* workspace, int64_t workspace_bytes, void* stream);

/* Times `iters` back-to-back tl_spmm launches on `stream` with HIP events recorded
 * on that same stream and returns the mean milliseconds per launch.  Used by the
 * benchmark so that the figure covers exactly the kernels tl_spmm enqueues. */
int tl_spmm_time(const tl_layout_header* header, const void* blob_dev,
                 const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                 void* Y, int y_dtype, int64_t ldy,
                 const void* scale, int scale_dtype,
                 void* workspace, int64_t workspace_bytes, void* stream,
                 int iters, float* mean_ms);

/* Measurement helper with no counterpart in the reference: one launch that only READS `bytes` bytes
 * (a multiple of 16, 16-byte aligned) of device memory, every lane 16 bytes at a time, and leaves one
 * folded dword per workgroup in out[0 .. tl_read_probe_workgroups() - 1].  The benchmark runs it under
 * the same HIP-graph replay as the single-row products: the box's own floor for a launch that must
 * stream a weight of that size once. */
int tl_read_probe_workgroups(void);
int tl_stream_read_probe(const void* src, int64_t bytes, void* out, void* stream);

/* ======================================================================== */
/* Around the products of a single-token decode step.                       */
/* ======================================================================== */

/* Rotary embedding of q and k fused with the KV-cache update -- stands where the
 * reference's attention calls apply_rotary_pos_emb and Cache.update of the
 * transformers package (TernaryLLM/TernaryAttn.py:93-98).
 *   qkv        device [batch][3][heads][head_dim]: q, k, v of one token per batch row
 *   cos_table, sin_table  device [max_seq][head_dim], rotate-half form (both halves of a row alike)
 *   pos_dev    device pointer to one int64: the token's position = the cache row written
 *   q_out      device [batch][heads][head_dim]
 *   k_cache, v_cache      device [batch][heads][max_seq][head_dim]
 * A position outside [0, max_seq) writes nothing. */
int tl_rope_cache_update(const void* qkv, int dtype, int64_t batch, int heads, int head_dim,
                         const void* cos_table, const void* sin_table, const int64_t* pos_dev,
                         void* q_out, void* k_cache, void* v_cache, int64_t max_seq, void* stream);

/* Softmax attention of one query per (batch row, head) over cache rows [0, *pos_dev] --
 * the reference's eager matmul / softmax / matmul for q_len == 1
 * (TernaryLLM/TernaryAttn.py:100-113), scores and softmax in fp32.
 *   q          device [batch][heads][head_dim]
 *   out        device [batch][heads * head_dim]
 * head_dim 64, 128 or 256; one pass over the cache (running maximum and sums), any max_seq.
 * out_kmajor_ld: 0, or the leading dimension (>= batch) of a K-major output [heads * head_dim][ld] --
 * the layout tl_spmm multiplies 5 to 48 rows from without a re-layout pass (here and in the two
 * functions below). */
int tl_decode_attention(const void* q, const void* k_cache, const void* v_cache, int dtype,
                        int64_t batch, int heads, int head_dim, int64_t max_seq,
                        const int64_t* pos_dev, void* out, int64_t out_kmajor_ld, void* stream);

/* tl_decode_attention with the cache rows of every (batch row, head) shared out among `splits` workgroups
 * (1 to 8), for steps with fewer (batch row, head) pairs than the GPU has compute units: one compute unit
 * streams a head's cache rows at a fraction of what the chip can.  Each workgroup leaves a piece in
 * `workspace`: fp32 [batch * heads][splits][head_dim + 4] -- head_dim unnormalised sums, then the piece's
 * maximum and its sum of exponentials (16-byte aligned; TL_ERR_SIZE when the workspace is smaller) -- and a
 * second small launch folds the pieces into `out`.  With out == NULL that launch is left out and the pieces
 * are the result (any splits >= 1): tl_spmv_attn_combine folds them inside the output projection.
 * splits == 1 with an `out` is tl_decode_attention (the workspace is not touched).  Same reference lines. */
int tl_decode_attention_split(const void* q, const void* k_cache, const void* v_cache, int dtype,
                              int64_t batch, int heads, int head_dim, int64_t max_seq,
                              const int64_t* pos_dev, void* out, int64_t out_kmajor_ld,
                              int splits, void* workspace, int64_t workspace_bytes, void* stream);

/* tl_rope_cache_update and tl_decode_attention_split as ONE launch: the attention kernel rotates q on the way
 * in, lets the token's rotated key and its value stand in for cache row *pos_dev (which the cache does not
 * hold yet), and the workgroup whose rows include that row writes them into the caches for the steps to come
 * (TernaryLLM/TernaryAttn.py:93-113).  qkv, cos_table, sin_table as in tl_rope_cache_update; the rest as in
 * tl_decode_attention_split (workspace may be NULL when splits == 1 and out is given).  Values are rounded to
 * `dtype` where the two separate calls store them: out, the pieces and the caches equal theirs bit for bit.
 * A position outside [0, max_seq) writes nothing; the attention then covers the rows the cache has. */
int tl_decode_attention_rope(const void* qkv, const void* cos_table, const void* sin_table,
                             void* k_cache, void* v_cache, int dtype,
                             int64_t batch, int heads, int head_dim, int64_t max_seq,
                             const int64_t* pos_dev, void* out, int64_t out_kmajor_ld,
                             int splits, void* workspace, int64_t workspace_bytes, void* stream);

/* tl_decode_attention_split (q given, qkv NULL) or tl_decode_attention_rope (qkv with its tables given, q NULL) for
 * 2 to 8 splits without the second launch: each workgroup of a (batch row, head) counts itself in once its piece is
 * in `workspace`, and the one that finds the others counted folds the pieces into `out` -- no workgroup waits for
 * another.  arrivals: batch * heads 32-bit counters in device memory, zero before the first call; every call leaves
 * them zero.  Calls that share `arrivals` or `workspace` must not overlap (work on one stream does not).  The
 * result equals the two-launch form's bit for bit (same pieces, same fold).  Same reference lines. */
int tl_decode_attention_fold(const void* q, const void* qkv, const void* cos_table, const void* sin_table,
                             void* k_cache, void* v_cache, int dtype,
                             int64_t batch, int heads, int head_dim, int64_t max_seq,
                             const int64_t* pos_dev, void* out, int64_t out_kmajor_ld,
                             int splits, void* workspace, int64_t workspace_bytes, uint32_t* arrivals, void* stream);

/* Y[N] = (x * W) * scale for ONE activation row x that the call produces itself, so that a decode step
 * needs neither a launch nor a trip through memory for the producer (the reference leaves these steps to
 * separate torch operators, TernaryLLM/TernaryMLP.py:34 and the Hugging Face decoder layer it patches):
 *   TL_PRODUCER_SILU_GATE    x[k] = silu(in[k]) * in[K + k], `in` a side-by-side gate | up row of 2K values
 *                            (tl_silu_mul followed by tl_spmm); in2, norm_weight, sum_out must be NULL
 *   TL_PRODUCER_ADD_RMSNORM  s = in + in2 (in2 may be NULL), x = s * rsqrt(mean(s^2) + eps) * norm_weight;
 *                            s is also written to sum_out when that is not NULL (tl_add_rmsnorm followed
 *                            by tl_spmm).  sum_out must not alias in or in2.
 *   TL_PRODUCER_RMSNORM      x = in * rsqrt(mean(in^2) + eps) * norm_weight, with the factor, one number for the
 *                            row, applied to the column sums instead of the row: the row that is multiplied is
 *                            in * norm_weight rounded to x_dtype, and no part of the kernel waits for the mean.
 *                            Equal to TL_PRODUCER_ADD_RMSNORM with in2 == NULL up to that rounding; in2 and
 *                            sum_out must be NULL.  (The residual add belongs to the product BEFORE the norm
 *                            then: tl_spmv_add, tl_spmv_attn_combine_add.)
 *   TL_PRODUCER_RMSNORM_SUMS the same product, for a row that the product before it prepared (tl_spmv_add_norm):
 *                            in = its image (row * norm_weight, x_dtype), in2 = its sums of squares, float32, one per
 *                            16 values of the row (ceil(K / 16) numbers); norm_weight and sum_out must be NULL.  The
 *                            kernel is then the plain single-row product with one factor at the end.
 *                            TL_ERR_UNSUPPORTED where a column block's tiles do not fit the LDS of that kernel.
 * in, in2, norm_weight, sum_out are of x_dtype, K values each (2K for the gate | up row), 16-byte aligned.
 * Roundings are those of the separate kernels.  TL_ERR_UNSUPPORTED when K or the blob's tile height is not
 * a whole number of 16-byte pieces (use the separate kernels then). */
int tl_spmv_fused(const tl_layout_header* header, const void* blob_dev, int producer,
                  const void* in, const void* in2, const void* norm_weight, float eps, void* sum_out, int x_dtype,
                  void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream);

/* Y[N] = residual[N] + (x * W) * scale for one contiguous, 16-byte aligned row x: the residual add of a decoder
 * layer (the Hugging Face decoder layer the reference patches, TernaryLLM/TernaryLlama.py:69-75) in the epilogue of
 * the product in front of it, rounded as a separate add of the stored product would round (the product to y_dtype,
 * then the sum).  residual: N values of y_dtype; Y may be the residual row itself.  TL_ERR_UNSUPPORTED where the
 * single-row kernels do not apply (K or the tile height not whole 16-byte pieces). */
int tl_spmv_add(const tl_layout_header* header, const void* blob_dev, const void* x, int x_dtype, const void* residual,
                void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream);

/* tl_spmv_add for a row that goes on into an RMSNorm and a product (the post-attention norm and gate | up after the
 * output projection, the next layer's input norm and q | k | v after the down projection, the final norm and the head:
 * TernaryLLM/TernaryLlama.py:69-75 and the Hugging Face decoder layer behind it).  Beside Y the epilogue leaves
 * image_out[n] = Y[n] * next_norm_weight[n] (y_dtype, N values) and squares_out[b] = sum of Y[n]^2 over column block b
 * (float32, ceil(N / 16) numbers): what tl_spmv_fused with TL_PRODUCER_RMSNORM_SUMS starts from, so that the product
 * after the norm neither multiplies the row nor sums its squares.  next_norm_weight: N values of y_dtype.  All three
 * 16-byte aligned; image_out a row of its own.  TL_ERR_UNSUPPORTED where the single-row kernel with this epilogue
 * does not take the weight (call tl_spmv_add and TL_PRODUCER_RMSNORM then). */
int tl_spmv_add_norm(const tl_layout_header* header, const void* blob_dev, const void* x, int x_dtype, const void* residual,
                     void* Y, int y_dtype, const void* scale, int scale_dtype, const void* next_norm_weight,
                     void* image_out, float* squares_out, void* stream);

/* A decoder layer at 9 to 16 fp16 rows without kernels of its own for the residual add and the RMSNorm (the Hugging
 * Face decoder layer the reference patches, TernaryLLM/TernaryLlama.py:69-75): the products on either side do them.
 * The product that ENDS a block (o, down) adds the residual rows and leaves, beside the new residual rows Y, what the
 * next norm needs: the K-major image of Y[m][n] * next_norm_weight[n] (the activations of the product that follows)
 * and, per block of 16 columns, the sum of Y[m][n]^2 over the block.  The product that STARTS a block (q|k|v,
 * gate|up, head) multiplies that image and applies rsqrt(mean square + eps) of each row to its sums -- the
 * normalisation factor is one number per row, so it can wait until the end (the image is then rounded as
 * Y * weight, not Y * factor * weight). */
typedef struct tl_chain {
    const void* residual;         /* NULL, or [M][residual_ld] of y_dtype: Y = residual + product (may be Y itself) */
    int64_t residual_ld;
    const void* next_norm_weight; /* NULL, or [N] of y_dtype; with it: */
    void* image_out;              /*   K-major [N][image_ld] of y_dtype, M <= image_ld <= 16, rows M..image_ld-1 zeroed */
    int64_t image_ld;
    float* squares_out;           /*   [ceil(N / 16)][16], 16-byte aligned (as squares_in) */
    const float* squares_in;      /* NULL, or [squares_blocks][16] as a chained product left them: the rows of X are */
    int32_t squares_blocks;       /*   those of an image_out, and the sums are scaled by rsqrt(sum / K + eps) per row */
    float eps;
} tl_chain;

/* tl_spmm (y_layout < 0) or tl_spmm_gated (y_layout = TL_X_ROW_MAJOR / TL_X_K_MAJOR) with the chain steps above.
 * TL_ERR_UNSUPPORTED unless 9 <= M <= 16 and x, y are fp16; the residual / image epilogue only in the kernel for
 * N < 64 * compute units (wider outputs: the separate tl_add_rmsnorm). */
int tl_spmm_chain(const tl_layout_header* header, const void* blob_dev,
                  const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                  void* Y, int y_dtype, int64_t ldy, int y_layout,
                  const void* scale, int scale_dtype, const tl_chain* chain,
                  void* workspace, int64_t workspace_bytes, void* stream);

/* tl_spmv_fused with the epilogue of tl_spmm_gated: the weight's columns are (gate, up) pairs and Y holds the N / 2
 * values silu(y[2j]) * y[2j + 1].  Same arguments otherwise. */
int tl_spmv_fused_gated(const tl_layout_header* header, const void* blob_dev, int producer,
                        const void* in, const void* in2, const void* norm_weight, float eps, void* sum_out, int x_dtype,
                        void* Y, int y_dtype, const void* scale, int scale_dtype, void* stream);

/* Y[N] = (x * W) * scale for the single row x = the attention output that the pieces of
 * tl_decode_attention_split (out == NULL) add up to, batch 1: the output projection of a decode step
 * (o_proj over the eager softmax(QK^T)V, TernaryLLM/TernaryAttn.py:100-116) without a launch for the fold.
 *   pieces    device fp32 [K / head_dim][splits][head_dim + 4], 16-byte aligned
 *   x_dtype   the type x is rounded to before the product (the type a separate fold would write)
 * Needs a blob whose tile height and K are whole 16-byte pieces of x_dtype (else TL_ERR_UNSUPPORTED) and
 * head_dim a multiple of 16 bytes of it that divides K. */
int tl_spmv_attn_combine(const tl_layout_header* header, const void* blob_dev, const void* pieces,
                         int splits, int head_dim, int x_dtype, void* Y, int y_dtype,
                         const void* scale, int scale_dtype, void* stream);

/* tl_spmv_attn_combine with the residual add of tl_spmv_add in its epilogue. */
int tl_spmv_attn_combine_add(const tl_layout_header* header, const void* blob_dev, const void* pieces,
                             int splits, int head_dim, int x_dtype, const void* residual, void* Y, int y_dtype,
                             const void* scale, int scale_dtype, void* stream);

/* tl_spmv_attn_combine_add that also leaves what tl_spmv_add_norm leaves for the RMSNorm and product behind it:
 * image_out[N] = Y * next_norm_weight and squares_out[ceil(N / 16)], the sums of Y^2 over runs of 16 values.  Served
 * by the kernel that folds the pieces of each wave's own tiles; TL_ERR_UNSUPPORTED where the weight's blocks do not
 * fit it (more than two tiles per wave, or more heads x splits under one tile than its table holds). */
int tl_spmv_attn_combine_add_norm(const tl_layout_header* header, const void* blob_dev, const void* pieces,
                                  int splits, int head_dim, int x_dtype, const void* residual, void* Y, int y_dtype,
                                  const void* scale, int scale_dtype, const void* next_norm_weight,
                                  void* image_out, float* squares_out, void* stream);

/* The end of a greedy decode step in one launch: token[b] = argmax of logits[b][0 .. vocab) (the first of equal
 * values; a NaN counts as larger than any number -- torch.argmax's rule), then, when pos_dev is not NULL,
 * *pos_dev = min(*pos_dev + 1, max_pos) and, when mask is not NULL too, mask[*pos_dev] = 1 (one byte per cache slot).
 * It stands for the argmax, copy, add, clamp and index_fill launches with which the reference's generation loop
 * (Hugging Face generate() behind TernaryLLM/TernaryLlama.py) ends a step.  logits: [batch][vocab] of `dtype`,
 * contiguous; token: int64 [batch]. */
int tl_greedy_advance(const void* logits, int dtype, int64_t batch, int vocab, int64_t* token, int64_t* pos_dev,
                      int64_t max_pos, void* mask, void* stream);

/* x_out = x + y, h_out = RMSNorm(x_out) * weight, row by row ([rows][width], one dtype): the residual
 * add of a decoder layer fused with the normalisation that follows (the reference leaves both to the
 * Hugging Face Llama it patches, TernaryLLM/TernaryLlama.py:69-75).  y may be NULL: plain RMSNorm of x,
 * x_out then optional.  h_kmajor_ld: 0, or the leading dimension (>= rows) of a K-major h_out [width][ld]. */
int tl_add_rmsnorm(const void* x, const void* y, const void* weight, int dtype, int64_t rows, int width,
                   float eps, void* x_out, void* h_out, int64_t h_kmajor_ld, void* stream);

/* out[rows][width] = silu(gate_up[:, :width]) * gate_up[:, width:] for gate_up [rows][2 * width]: the
 * gate of LlamaTernaryMLP (TernaryLLM/TernaryMLP.py:33-35) on a side-by-side gate | up product.
 * out_kmajor_ld: 0, or the leading dimension (>= rows) of a K-major out [width][ld]. */
int tl_silu_mul(const void* gate_up, int dtype, int64_t rows, int width, void* out, int64_t out_kmajor_ld, void* stream);

/* tl_silu_mul for a gate | up product whose columns are PAIRS -- column 2j the gate and column 2j + 1 the up
 * projection of output j (a weight packed that way lets a product's kernel finish both halves of a pair in one
 * workgroup, see tl_spmm_gated): out[r][j] = silu(gate_up[r][2j]) * gate_up[r][2j + 1].  Same reference lines. */
int tl_silu_mul_pairs(const void* gate_up, int dtype, int64_t rows, int width, void* out, int64_t out_kmajor_ld, void* stream);

/* tl_spmm with the SiLU gate of LlamaTernaryMLP (TernaryLLM/TernaryMLP.py:33-35) in the epilogue, for a weight
 * whose columns are (gate, up) pairs as above: Y[m][j] = silu(y[m][2j]) * y[m][2j + 1] with y = (X * W) * scale,
 * N / 2 outputs per row -- what tl_spmm followed by tl_silu_mul_pairs computes, bit for bit (y and the SiLU are
 * rounded to y_dtype where those would store them), without the launch and the trip through memory.
 *   y_layout   TL_X_ROW_MAJOR: Y [M][ldy], ldy >= N / 2;  TL_X_K_MAJOR: Y [N / 2][ldy], ldy >= M, rows M..ldy-1
 *              zeroed -- the image tl_spmm multiplies 5 to 48 rows from (9 to 16 rows only)
 * The kernels with this epilogue are those of M = 1 (a contiguous aligned row), of fp16 rows in groups of 16
 * (9 to 48 rows) with N >= 64 * compute units, and of more than 48 rows (row-major Y); any other call returns
 * TL_ERR_UNSUPPORTED and the two separate calls do the work.  (For separate gate and up weights and more than
 * 48 rows there is tl_mlp_gate_up; the paired weight is the faster of the two, one launch over twice the
 * columns.) */
int tl_spmm_gated(const tl_layout_header* header, const void* blob_dev,
                  const void* X, int x_dtype, int x_layout, int64_t ldx, int64_t M,
                  void* Y, int y_dtype, int64_t ldy, int y_layout,
                  const void* scale, int scale_dtype,
                  void* workspace, int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TERNARY_SPMM_H */
