/*
 * tq_hip.h -- C ABI of libtq_hip.so, the MI355X (gfx950) TurboQuant KV-cache kernels.
 *
 * The reference project is pure Python and has no FFI of its own; each entry
 * point below names the reference function (file:line, relative to the
 * reference checkout) whose arithmetic it replaces.  The host side that mirrors
 * the reference's Python API binds these symbols with ctypes.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the comment says "host";
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - `dtype` tags the element type of floating inputs: TQ_F32 / TQ_F16 / TQ_BF16;
 *   - the caller allocates every output and the decode workspace; no entry
 *     point allocates device memory, frees or synchronises;
 *   - calls on different streams may overlap (tq_decode_attn_paged_noalloc excepted, see there).  State the
 *     library keeps, all of it listed here:
 *       per host thread and device - a side stream with two events that tq_append_kv_paged and its siblings
 *         create on first use for large appends, and the pair of events armed by tq_time_next_*_kernel;
 *       per process - the launch attributes set on a kernel's first use, the compute-unit count of the first
 *         device used (the cards of one machine are taken to be alike), and the knobs of tq_set_option, which
 *         select grid shapes and the carving of the workspace: they must not change between the `stages`
 *         calls of one step, nor while another thread is inside a decode or append call;
 *       per device - the static scratch array of tq_decode_attn_paged_noalloc (TQ_NOALLOC_SCRATCH_BYTES),
 *         shared by every caller of that entry point on the device;
 *   - block tables are device data the host cannot inspect, so the kernels bound them:
 *     a logical page beyond the table row, or a table entry outside [0, num_pages), is
 *     never written through (append) and contributes no token (decode); see each entry;
 *   - return value: 0 on success, a negative TQ_E* code for a rejected argument
 *     (nothing was launched), or a positive hipError_t from the launch.
 */
#ifndef TQ_HIP_H
#define TQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TQ_ABI_VERSION 2

enum { TQ_F32 = 0, TQ_F16 = 1, TQ_BF16 = 2 };

enum {
  TQ_OK = 0,
  TQ_EINVAL = -1,       /* a size, stride or enum is out of range                */
  TQ_EUNSUPPORTED = -2, /* a legal request this build has no kernel for          */
  TQ_ENULL = -3,        /* a required pointer is NULL                            */
  TQ_ETOOBIG = -4       /* the call needs more scratch than the library's static area holds */
};

#define TQ_PAGE_TOKENS 16
#define TQ_MAX_TERMS 15

/* Per-layer constants of the key quantiser (reference quantizer.py:101-127,186-212).
 * All arrays live in device memory and are owned by the caller. */
typedef struct tq_layer {
  int32_t d;               /* head_dim; multiple of 64, 64..768                             */
  int32_t mse_bits;        /* bits of the Lloyd-Max stage = key_bits - 1, 1..4              */
  const float *Pi;         /* d*d row-major rotation (rotation.py:17-40)                    */
  const float *PiT;        /* its transpose, row-major                                      */
  const float *S;          /* d*d row-major Gaussian sketch (rotation.py:43-56)             */
  const float *ST;         /* its transpose, row-major                                      */
  const float *centroids;  /* 2^mse_bits                                                    */
  const float *thresholds; /* 2^mse_bits - 1 interior boundaries (quantizer.py:127)         */
  float qjl_scale;         /* sqrt(pi/2)/d (quantizer.py:212)                               */
  /* Optional operands of the matrix-core quantise / de-quantise kernels: Pi, its transpose, S and its transpose, each
   * written as the exact sum of three bf16 matrices (term t rounds what terms < t left),
   * raw bf16 bit patterns, 3*d*d each, stored in the order the kernel loads its MFMA
   * operands: element (row, col) of term t sits at
   *   ((((t*(d/16) + row/16)*(d/32) + col/32)*4 + (col%32)/8)*16 + row%16)*8 + col%8.
   * ST_split (the transpose of S) serves the de-quantiser.  NULL selects the vector-ALU
   * kernels.  At the head sizes of the wide-head decode kernel (320 ... 704 in steps of 64)
   * Pi_split and S_split alone serve the decode step's query rotation (bf16 / fp16 queries); the
   * transposes may stay NULL there.                                                    */
  const uint16_t *Pi_split, *PiT_split, *S_split, *ST_split;
  /* Optional constants of the fused query-preparation kernel of the decode path:
   * Pi_colsum[i] = sum_j Pi[j][i], S_colsum[i] = sum_j S[j][i] (d floats each) and the
   * largest row norm of S.  NULL selects the two-kernel preparation.                    */
  const float *Pi_colsum, *S_colsum;
  float S_rownorm_max;
  /* Optional operands of the centroid contraction x_hat = c[idx] Pi (quantizer.py:160) of the matrix-core
   * key quantiser, head_dim 128, codebooks whose Walsh expansion has only single-bit terms (the symmetric
   * 1- and 2-bit Lloyd-Max codebooks).  The index bit planes are the fp4 operand of the block-scaled
   * 16x16x128 MFMA; Pi^T is its fp6 operand, five fp6 (e2m3) digits per value:
   *   PiT_fp6       uint32 [d/16 row tiles][d/128][5 terms][64 lanes][6]: lane (row % 16, block b) holds the
   *                 32 six-bit codes of (row, contraction indices 32 b ..), index s at bits 6 s .. 6 s + 5;
   *                 contraction index 32 w + 8 (c % 4) + c / 4 is coordinate c of plane word w, and the value is
   *                 Pi^T[row][coordinate] divided by 0.5, 1, 2, 0.5 for c % 4 = 0..3 (the fp4 values of a set
   *                 bit at that position): v = 2^E sum_t digit_t 2^(-2 - 5 t), 2^E >= the block's largest |v|;
   *   PiT_fp6_scale uint32 [d/16][d/128][64 lanes][2]: E8M0 codes 127 + E - 2 - 5 t, terms 0..3 in the bytes of
   *                 the first word, term 4 in the lowest byte of the second.
   * Needs Pi_colsum.  NULL selects the bf16 term products for this contraction too.  (turboquant_amd._ffi
   * .split_fp6x5 builds both.)                                                                            */
  const uint32_t *PiT_fp6, *PiT_fp6_scale;
  /* Walsh expansion of the codebook over the index bits, used by the decode
   * kernel: centroids[idx] = term_const + sum_t term_coef[t] * parity(idx & term_mask[t]).
   * Filled by tq_layer_fill_terms from the host copy of the centroids.          */
  int32_t n_terms;
  int32_t term_mask[TQ_MAX_TERMS];
  float term_coef[TQ_MAX_TERMS];
  float term_const;
} tq_layer;

/* Geometry of one page = TQ_PAGE_TOKENS tokens of one KV head (new design; the
 * reference keeps python lists of chunk tensors, store.py:59-63).  Offsets are
 * in bytes from the start of the page; every section starts 16-byte aligned.
 *   keys   : key_bits = mse_bits+1 bit-planes (index bits high..low, then the QJL
 *            sign).  Word j of plane p of token n holds coordinates 32j..32j+31
 *            (bit i = coordinate 32j+i).  With key_lane_major != 0 (d a multiple
 *            of 128, or 64) the words are stored as [j%4][n][j/4][p], so that the
 *            words one wavefront lane (token n, coordinate quarter j%4) consumes
 *            are contiguous, 128 coordinates after 128 (d = 64: [j][n][p]);
 *            otherwise as [p][j][n].
 *   meta   : per token {float norm, float rnorm}: the key norm (a value of the
 *            input dtype, widened losslessly) and ||r||.
 *   vdata  : per channel c a little-endian field of 16*value_bits bits, token n's
 *            code at bit value_bits*n; fields ordered [c%16][c/16].
 *   vscale / vzero : [d/group][16 tokens] in the input dtype.                  */
typedef struct tq_page_layout {
  int32_t d, mse_bits, value_bits, group_size, dtype, key_lane_major;
  int32_t off_keys, off_meta, off_vdata, off_vscale, off_vzero;
  int32_t page_bytes;      /* stride between (page, head) records, multiple of 128 */
} tq_page_layout;

int tq_version(void);

/* Host helper: fills the term_* fields of `layer` from a HOST array of its
 * 2^mse_bits centroids; coefficients below 1e-9 of the largest are dropped. */
int tq_layer_fill_terms(tq_layer *layer /*host*/, const float *centroids_host);

/* Host helper: computes the page geometry for inputs of `dtype`;
 * value_bits 2, 4 or 8, d a multiple of 64 and of group_size (>= 16).                  */
int tq_page_layout_init(tq_page_layout *out /*host*/, int d, int mse_bits, int value_bits,
                        int group_size, int dtype);

/* ---- parity entry points on the reference's own tensor layouts ------------------ */

/* idx = #{t : !(y <= thresholds[t])}, packed little-end-first into bytes, 1/2/4/4
 * bits per index for mse_bits 1/2/3/4 (quantizer.py:144 + _pack_indices :38-69).
 * y is (n_vec, d) fp32 contiguous; idx_out is (n_vec, ceil(d/per_byte)).          */
int tq_bucketize_pack(const float *y, int64_t n_vec, int d, const float *thresholds, int mse_bits,
                      uint8_t *idx_out, void *stream);

/* bit j of byte k = (p[8k+j] > 0) (quantizer.py:214-222). p is (n_vec, d) fp32.    */
int tq_sign_pack(const float *p, int64_t n_vec, int d, uint8_t *sign_out, void *stream);

/* TurboQuantProd.quantize (quantizer.py:231-257 with :129-165 inlined).
 * x is (n_vec, d) with `row_stride` elements between vectors.  norm_out has the
 * input dtype, rnorm_out is fp32.  y_dbg / p_dbg (nullable, (n_vec,d) fp32)
 * receive the rotated unit vector and the projected residual.  With
 * mse_only != 0 only the first stage runs (TurboQuantMSE.quantize :129-149) and
 * sign_out / rnorm_out may be NULL.                                               */
int tq_quantize_keys(const void *x, int dtype, int64_t n_vec, int64_t row_stride, const tq_layer *layer,
                     uint8_t *idx_out, uint8_t *sign_out, void *norm_out, float *rnorm_out,
                     float *y_dbg, float *p_dbg, int mse_only, void *stream);

/* quantize_values (kv_cache.py:45-98): per-group min/max affine codes, computed
 * with the per-operation rounding of the input dtype.  bits 2, 4 or 8.
 * data_out (n_vec, d*bits/8), scale_out / zero_out (n_vec, d/group) input dtype.  */
int tq_quantize_values(const void *v, int dtype, int64_t n_vec, int64_t row_stride, int d, int group_size,
                       int bits, uint8_t *data_out, void *scale_out, void *zero_out, void *stream);

/* TurboQuantMSE.dequantize / TurboQuantProd.dequantize (quantizer.py:151-165,
 * 259-272) -> out (n_vec, d) fp32.  norm_dtype tags `norms`.  signs / rnorms may
 * be NULL for the MSE-only form.                                                  */
int tq_dequant_keys(const uint8_t *idx, const uint8_t *signs, const void *norms, int norm_dtype,
                    const float *rnorms, int64_t n_vec, const tq_layer *layer, float *out, void *stream);

/* dequantize_values (kv_cache.py:101-116) -> out (n_vec, d) fp32.                  */
int tq_dequant_values(const uint8_t *data, const void *scales, const void *zeros, int dtype, int64_t n_vec,
                      int d, int group_size, int bits, float *out, void *stream);

/* TurboQuantProd.attention_score (quantizer.py:274-302) in the rotated-query
 * form of triton_kernels.py:49-53,138: for each of `batch` independent
 * problems, scores[b, i, k] = norm_k * <q_i Pi^T, c[idx_k]> + qjl_scale * rnorm_k *
 * <q_i S^T, sigma_k>.  q (batch, n_q, d) `dtype`; key arrays (batch, n_k, ...);
 * scores (batch, n_q, n_k) fp32; no 1/sqrt(d).  work is a caller buffer of
 * 2*batch*n_q*d floats for the rotated and sketched queries.                      */
int tq_score(const void *q, int dtype, int64_t batch, int64_t n_q, const uint8_t *idx, const uint8_t *signs,
             const void *norms, int norm_dtype, const float *rnorms, int64_t n_k, const tq_layer *layer,
             float *scores, float *work, void *stream);

/* q_rot = q Pi^T and q_sk = q S^T in fp32 for `rows` vectors of `dtype`
 * (triton_kernels.py:527-528); the prologue of tq_score and of the decode kernel. */
int tq_rotate_query(const void *q, int dtype, int64_t rows, const tq_layer *layer, float *q_rot, float *q_sk,
                    void *stream);

/* ---- paged store ---------------------------------------------------------------- */

/* Quantise T new tokens of each of B sequences and write them into pages
 * (fused a8 + a11 of the reference, store.py:73-90, for a batch of sequences).
 * k, v: element (b, t, h, :) at  base + b*stride_b + t*stride_t + h*stride_h  (in
 * elements), innermost dimension contiguous.  Token t of sequence b goes to
 * logical position start_pos[b] + t, i.e. page block_table[b*max_pages + pos/16],
 * slot pos%16.  start_pos may be NULL (all zero).  pool is (num_pages, H, page_bytes).
 * Tokens whose logical page lies beyond the table row (pos/16 >= max_pages) or whose table entry is not
 * in [0, num_pages) are dropped: nothing outside the pool is written.  Without start_pos the run length is
 * known on the host and T > 16*max_pages is TQ_EINVAL.
 * Large appends run their value kernel on a side stream of the calling thread (created on
 * first use, default priority) that is forked from and joined back into `stream` with
 * events: the call is ordered on `stream` like any other and stays capturable.           */
int tq_append_kv_paged(const void *k, const void *v, int dtype, int B, int T, int H, int64_t stride_b,
                       int64_t stride_t, int64_t stride_h, const int32_t *start_pos, const int32_t *block_table,
                       int max_pages, const tq_layer *layer, const tq_page_layout *layout, uint8_t *pool,
                       int64_t num_pages, void *stream);

/* Ragged batch of runs (the batch counterpart of CompressedKVStore.append_chunk, store.py:73-90, for an
 * engine step that carries several sequences): k / v are (rows, H, d) `dtype` with element strides
 * stride_t / stride_h, the run of sequence b is rows row0[b] .. row0[b] + run_len[b] - 1 (run_len[b] <=
 * T_max, 0 = nothing) and lands at token positions start_pos[b] .. of the pages block_table[b*max_pages + i].
 * All three arrays are device int32 (B,): row0 = query_start_loc[:-1], run_len = its differences,
 * start_pos = seq_lens - run_len for an engine's step metadata.  Pages as tq_append_kv_paged writes them. */
int tq_append_kv_ragged(const void *k, const void *v, int dtype, int B, int T_max, int H, int64_t stride_t,
                        int64_t stride_h, const int32_t *row0, const int32_t *run_len, const int32_t *start_pos,
                        const int32_t *block_table, int max_pages, const tq_layer *layer,
                        const tq_page_layout *layout, uint8_t *pool, int64_t num_pages, void *stream);

/* The same for tokens that already sit in a paged exact KV cache (gather + quantise in one pass;
 * capture.py:187-217 ingest_prefill_from_paged_cache gathers the blocks with torch indexing first).
 * k_cache, v_cache: blocks of 16 tokens, element (block, slot, h, :) at
 * base + block*stride_blk + slot*stride_t + h*stride_h.  Sequence b's token at absolute position p
 * is slot p%16 of block src_table[b*src_stride + p/16]; positions start_pos[b] .. start_pos[b] +
 * min(run_len[b], T) - 1 are quantised (start_pos NULL = 0, run_len NULL = T for every sequence) and
 * written to page block_table[b*max_pages + p/16], slot p%16, as by tq_append_kv_paged.             */
int tq_append_kv_from_blocks(const void *k_cache, const void *v_cache, int dtype, int B, int T, int H,
                             int64_t stride_blk, int64_t stride_t, int64_t stride_h, const int32_t *src_table,
                             int src_stride, const int32_t *start_pos, const int32_t *run_len,
                             const int32_t *block_table, int max_pages, const tq_layer *layer,
                             const tq_page_layout *layout, uint8_t *pool, int64_t num_pages, void *stream);

/* Gather a sequence's pages back into the reference's flat tensors
 * (store.py:92-114 get_flat_cache): idx (H, n_tok, d*eff/8), signs (H, n_tok, d/8),
 * norms (H, n_tok) input dtype, rnorms fp32, v_data (H, n_tok, d*vb/8),
 * v_scales / v_zeros (H, n_tok, d/group).  block_table is this sequence's row
 * (at least ceil(n_tok/16) entries); an entry outside [0, num_pages) is read as page 0. */
int tq_pool_export(const uint8_t *pool, int64_t num_pages, int H, const int32_t *block_table, int n_tok,
                   const tq_page_layout *layout, uint8_t *idx, uint8_t *signs, void *norms, float *rnorms,
                   uint8_t *v_data, void *v_scales, void *v_zeros, void *stream);

/* No counterpart in the reference: which page kernel a decode step over this layer and page layout runs (with at
 * most 8 query heads per group of a KV head; the current options applied): 0 the general vector-ALU kernel,
 * 1 the matrix-core kernel of head_dim 64 / 128 / 256 (a block of 64 tokens per wavefront), 2 the matrix-core
 * kernel of the head sizes 320 .. 704 (a block of 32 tokens per workgroup).  Negative: an error code.           */
int tq_decode_page_kernel(const tq_layer *layer /*host*/, const tq_page_layout *layout /*host*/);

/* Bytes of workspace tq_decode_attn_paged needs for these sizes.                   */
size_t tq_decode_workspace_bytes(int B, int Hq, int d, int n_split);

/* Fused decode attention over the paged compressed history plus an optional
 * exact tail (compute_hybrid_attention, score.py:29-173; kernel semantics of
 * triton_kernels.py:209-356 with GQA sharing, paging and split-K added).
 * q (B, Hq, d) `dtype` contiguous (it need not be the pages' dtype); query head h
 * reads KV head h / (Hq/Hkv); Hq / Hkv is any whole number up to 128 (the reference's
 * _matmul_attend, score.py:138-173, takes any ratio): the page kernels serve a KV head's
 * heads in groups of at most 8 (matrix cores) or 16 (general kernel).
 * seq_lens[b] compressed tokens of sequence b sit in block_table[b*bt_stride + i]:
 * bt_stride > 0 is a row of that many entries per sequence; bt_stride < 0 one row of -bt_stride entries
 * shared by all sequences; 0 one shared row of unchecked length.  A length beyond the row is cut to
 * 16 entries per row entry, and the tokens of a page whose entry is not in [0, num_pages) get no weight.  recent_k / recent_v (nullable)
 * hold exact tokens (b, r, h, :) `dtype`, element strides rs_b, rs_r, rs_h, with
 * recent_len[b] valid rows (NULL = recent_rows for all).  out (B, Hq, d) `dtype`:
 * softmax(sm_scale * [scores_hist ; q k_recent^T]) [v_hist ; v_recent]; all-empty
 * rows give zeros.                                                                */
int tq_decode_attn_paged(const void *q, int dtype, int B, int Hq, int Hkv, const uint8_t *pool,
                         int64_t num_pages, const int32_t *block_table, int bt_stride, const int32_t *seq_lens,
                         float sm_scale, const tq_layer *layer, const tq_page_layout *layout,
                         const void *recent_k, const void *recent_v, int recent_rows, int64_t rs_b,
                         int64_t rs_r, int64_t rs_h, const int32_t *recent_len, void *out, void *workspace,
                         int n_split, void *stream);

/* The same call restricted to some of its three stages, for timing them apart:
 * bit 0 query rotation / sketch, bit 1 the page-streaming kernel (and the exact
 * tail), bit 2 the merge.  stages = 7 is tq_decode_attn_paged.  A later stage
 * expects the workspace an earlier call left behind.                            */
int tq_decode_attn_paged_stages(const void *q, int dtype, int B, int Hq, int Hkv, const uint8_t *pool,
                                int64_t num_pages, const int32_t *block_table, int bt_stride,
                                const int32_t *seq_lens, float sm_scale, const tq_layer *layer,
                                const tq_page_layout *layout, const void *recent_k, const void *recent_v,
                                int recent_rows, int64_t rs_b, int64_t rs_r, int64_t rs_h,
                                const int32_t *recent_len, void *out, void *workspace, int n_split, int stages,
                                void *stream);

/* Hybrid decode step straight from the engine's paged exact cache (the reference keeps the exact recent
 * tokens in a ring of its own, capture.py:75-131, and concatenates them in score.py:99-111; here they are
 * read in place).  seq_lens[b] counts ALL tokens of sequence b.  The newest min(seq_lens[b], ring_rows) of
 * them are attended to exactly, from k_cache / v_cache: blocks of 16 tokens, token p of sequence b in slot
 * p % 16 of block block_table[b*bt_stride + p/16], element strides cs_blk (block), cs_t (token), cs_h (KV
 * head), channels contiguous, `dtype`; 16-bit caches need even strides and 4-byte aligned bases
 * (TQ_EUNSUPPORTED otherwise).  The tokens before them come from the compressed pages of the same block
 * numbers.  Result as tq_decode_attn_paged with recent_k / recent_v = those rows and seq_lens reduced by
 * their count, bit for bit.  ring_rows <= 1024.                                                         */
int tq_decode_attn_paged_ring(const void *q, int dtype, int B, int Hq, int Hkv, const uint8_t *pool,
                              int64_t num_pages, const int32_t *block_table, int bt_stride, const int32_t *seq_lens,
                              float sm_scale, const tq_layer *layer, const tq_page_layout *layout,
                              const void *k_cache, const void *v_cache, int64_t cs_blk, int64_t cs_t, int64_t cs_h,
                              int ring_rows, void *out, void *workspace, int n_split, void *stream);

/* tq_decode_attn_paged for callers that cannot allocate or pass a workspace (code under HIP graph capture
 * that owns no buffers, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments and result, bit for bit, as tq_decode_attn_paged with the same n_split, minus the
 * workspace: partials, rotated queries and query operands live in a file-scope device array of
 * TQ_NOALLOC_SCRATCH_BYTES inside the library (one copy per GPU, held until the process ends; its address is
 * looked up with hipGetSymbolAddress by tq_noalloc_init, or by the first call on a device).  The call
 * allocates nothing and frees nothing.  A call that needs more than the array holds returns TQ_ETOOBIG and
 * launches nothing; tq_decode_noalloc_bytes gives the exact requirement of a shape.  All calls on one GPU share
 * the array: calls that overlap on one GPU (different streams or threads) race; serialise them or use the
 * workspace form.  The device that is current must be the stream's device.  Under stream capture, call
 * tq_noalloc_init (or make one un-captured call) on the device first: the symbol lookup is not a stream
 * operation and should not happen while a capture is open.                                              */
#define TQ_NOALLOC_SCRATCH_BYTES (16u << 20)
int tq_decode_attn_paged_noalloc(const void *q, int dtype, int B, int Hq, int Hkv, const uint8_t *pool,
                                 int64_t num_pages, const int32_t *block_table, int bt_stride, const int32_t *seq_lens,
                                 float sm_scale, const tq_layer *layer, const tq_page_layout *layout,
                                 const void *recent_k, const void *recent_v, int recent_rows, int64_t rs_b,
                                 int64_t rs_r, int64_t rs_h, const int32_t *recent_len, void *out, int n_split,
                                 void *stream);

/* Bytes of the static scratch array a tq_decode_attn_paged_noalloc call of this shape uses (no counterpart in
 * the reference); the call returns TQ_ETOOBIG exactly when this exceeds TQ_NOALLOC_SCRATCH_BYTES.  `layer` is
 * read on the host (head_dim, index bits, codebook terms).  0 for a NULL layer or sizes that are not positive. */
size_t tq_decode_noalloc_bytes(int B, int Hq, int Hkv, int n_split, const tq_layer *layer);

/* Resolves the address of the current device's scratch array (hipGetSymbolAddress, once per device), so that
 * the first tq_decode_attn_paged_noalloc call on that device does nothing but launch.  Idempotent.         */
int tq_noalloc_init(void);

/* Log-sum-exp merge of n_parts partial results per (b, query head):
 * parts (B*Hq, n_parts, d+2) fp32 = [running max, sum of exp, un-normalised acc];
 * out (B*Hq, d) `dtype`.  The same operator a context-parallel shard exchange
 * would use.                                                                      */
int tq_decode_merge(const float *parts, int64_t rows, int n_parts, int d, int dtype, void *out, void *stream);

/* Measurement aid (no counterpart in the reference).  Arms the calling thread: the next
 * page-streaming kernel that tq_decode_attn_paged[_stages] launches from this thread (matrix-core or
 * general) is launched with `start_event` / `stop_event` (hipEvent_t, created with timing enabled)
 * attached to its own dispatch, so that hipEventElapsedTime(start, stop) is that kernel's execution
 * time alone - what a profiler's kernel trace reports - and not the interval between two markers in the
 * stream, which also contains the dispatch gap.  Pass NULLs to disarm.                             */
void tq_time_next_page_kernel(void *start_event, void *stop_event);

/* The same for the next matrix-core key-quantise kernel that tq_append_kv_paged and its siblings launch from
 * this thread (head_dim 128 / 256, 16-byte aligned inputs): its execution time alone, without the value
 * kernel that runs beside it.                                                                        */
void tq_time_next_key_kernel(void *start_event, void *stop_event);

/* Tuning and test knobs (no counterpart in the reference); process-wide, take effect at the next call.
 *   "prefetch_trips"   -1..64: the preparation launch of a step on the matrix-core path carries extra workgroups
 *                      that read the pages every page-kernel workgroup asks for first (this many trips of each of
 *                      its block walkers, at most 96 KB per workgroup) into the caches ahead of it; 0: none;
 *                      -1 (default): one trip at head_dim 256, none at the other head sizes (where the read-ahead
 *                      moves as much time into the preparation launch as it saves).  Same result bit for bit.
 *   "prep_mfma"        1 (default): bf16 queries at head_dim 128, and at head_dim 256 from 64 (row tile, plane word)
 *                      workgroups on, are rotated, sketched and packed on the matrix cores (three-term bf16 products
 *                      with Pi_split / S_split: fp32-accurate, summed in another order than the vector-ALU kernel,
 *                      so outputs agree to rounding, not bit for bit); 2: wherever the kernel applies; 0: never.
 *                      At the head sizes of the wide-head kernel, 1 or 2: bf16 and fp16 queries are rotated and packed
 *                      on the matrix cores when the layer has Pi_split and S_split.
 *   "merge_in_kernel"  1 (default): a compressed-only decode step on the matrix-core kernel with at most 8 context
 *                      splits has its splits merged by the last workgroup of the page kernel (two launches per
 *                      step); 0: always the separate merge kernel.
 *   "page_pairs"       1 (default): head_dim 64 with at most 4 query heads per KV head scores two pages per
 *                      matrix instruction (block-diagonal query operand); 0: one page per instruction, half
 *                      of the contraction idle (the kernel of more than 4 heads per KV head).
 *   "narrow_rows"      1 (default): head_dim 128 / 256 with at most 4 query heads per KV head puts the four fp6
 *                      terms of a head into one score operand (one matrix instruction per plane word); 0: two.
 *   "wide_workgroups"  1 (default): at head_dim 64 / 128, with an even split count and at most 16 blocks of 64 tokens
 *                      per wavefront (judged by the width of the block table), a step runs workgroups of 8
 *                      wavefronts on half the split count it was given; 0: always 4 wavefronts per workgroup.
 *   "wide_heads"       1 (default): head sizes 320 .. 704 (16-bit pages, value groups of 32) run the matrix-core page kernel
 *                      that works on a block of 32 tokens per workgroup, 512 and 576 in instantiations with constant page
 *                      geometry; 2: every such head size on the instantiation that takes the geometry at run time (same
 *                      result bit for bit); 0: the general vector-ALU kernel (results agree to rounding).
 *   "wide_prepack"     1 (default): at the head sizes of that kernel the rotation launch of a decode step packs the kernel's
 *                      query operands once per group of heads; 0: every page-kernel workgroup packs its own (results agree to
 *                      rounding: the operands are normalised by other bounds).
 *   "append_small"     -1 (default), 0, or a tile count: an append to pages of at most this many 16-vector tiles (-1: two
 *                      per compute unit) gives every tile a workgroup that computes that tile only - the page write of
 *                      a decode step, a token per sequence; 0: always workgroups over groups of tiles.  Same bytes.
 *   "prep_words"       -1 (default), 0 or 1: the matrix-core query preparation runs a workgroup per (tile of up to 16 query
 *                      rows, 32-coordinate plane word) (0) or a workgroup per tile whose four wavefronts take a word each
 *                      (1: a quarter or an eighth of the workgroups); -1: the second at head_dim 128 when the first would not
 *                      fit the card at once.  Same operands bit for bit.
 *   "sequence_walkers" -1 (default), 4, 2 or 1: at head_dim 64 / 128 a step with a single context split lets 4, 2 or 1
 *                      wavefronts of a workgroup walk a (sequence, group of query heads), so a workgroup serves 1, 2 or
 *                      4 of those pairs (fewer workgroups, more trips after each prologue, fewer walkers to merge);
 *                      -1: the largest of the three with which all wavefronts of the launch are resident at once
 *                      (8 per compute unit), one if there are more pairs than that.
 *   "split_skew"       0..8, default 1: at head_dim 256, when a launch of 4-wavefront workgroups fills (nearly) every
 *                      compute unit twice and the split count is even, the workgroups of the first half of the grid
 *                      (dispatched first, served first by their SIMDs) take the even splits and this many sixteenths
 *                      of a split's trips over from the odd splits of the second half; 0: equal shares.
 *   "tail_chunks"      1 (default): a hybrid step with more than 8 context splits and few (sequence, KV head)
 *                      pairs lets 2 or 4 workgroups share the exact tokens of a group of query heads, each with
 *                      a partial of its own for the merge kernel; 0: one workgroup and one partial.
 *   "merge_row_groups" 1 (default): the merge kernel gives a row of partials to 2 or 4 workgroups (a share of the
 *                      channels each) when there are fewer rows than compute units; 0: one workgroup per row.
 *   "fp6_centroids"    1 (default): the key quantiser takes the fp6 x fp4 centroid contraction when the layer
 *                      carries PiT_fp6; 0: always the bf16 term products (for A/B runs).
 *   "append_parts"     measurement only: 3 (default) = the append entry points quantise keys and values,
 *                      1 = keys only, 2 = values only (the other half of every page is left as it was), so
 *                      that either kernel can be timed without the other running beside it.
 * Returns TQ_EINVAL for an unknown name or a value out of range.                                        */
int tq_set_option(const char *name, int64_t value);

/* Measurement aid (no counterpart in the reference).  Reads `bytes` (a multiple of 16) from `src`
 * (16-byte aligned) with `workgroups_per_cu` workgroups of 256 lanes per compute unit, each lane keeping
 * `loads_in_flight` (1, 4 or 8) 16-byte loads outstanding, and writes nothing (`sink`, 4 bytes, may be
 * NULL).  Timed over a buffer larger than the caches it gives the read bandwidth the card really
 * delivers, against which the page-streaming kernels are reported beside the vendor's peak.          */
int tq_stream_read(const void *src, size_t bytes, int workgroups_per_cu, int loads_in_flight,
                   uint32_t *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TQ_HIP_H */
