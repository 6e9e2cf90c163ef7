/* C ABI of libxattn_hip.so: the gfx950 (MI355X) kernels behind the XAttention
 * prefill operator.
 *
 * Conventions shared by every entry point
 *  - all pointers are DEVICE pointers unless a parameter says "host";
 *  - q/k/v/out are bf16, laid out [head][token][128] with the feature dimension
 *    contiguous; head and token strides are given in ELEMENTS and must be
 *    multiples of 8 (16-byte rows), base pointers 16-byte aligned;
 *  - batch is 1 (the reference asserts it, xattn/src/Xattention.py:357);
 *  - K/V may carry fewer heads than Q: query head h reads KV head
 *    h / (num_heads / num_kv_heads);
 *  - `stream` is a hipStream_t passed as void*; work is enqueued on it and the
 *    call returns without synchronising; nothing is allocated inside;
 *  - the return value is XATTN_OK or a negative XATTN_ERR_* code; arguments are
 *    validated on the host before anything is launched, nothing is thrown.
 *
 * Paths cited as xattn/... are files of mit-han-lab/x-attention.
 */
#ifndef XATTN_HIP_H
#define XATTN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  XATTN_OK = 0,
  XATTN_ERR_NULL = -1,      /* a required pointer is null                       */
  XATTN_ERR_HEAD_DIM = -2,  /* head_dim != 128                                  */
  XATTN_ERR_HEADS = -3,     /* num_heads not a positive multiple of kv heads    */
  XATTN_ERR_SHAPE = -4,     /* lengths / block counts / pitches out of range    */
  XATTN_ERR_ALIGN = -5,     /* pointer or stride not 16-byte aligned            */
  XATTN_ERR_STRIDE = -6,    /* antidiagonal stride not one of 4, 8, 16          */
  XATTN_ERR_WORKSPACE = -7, /* workspace too small                              */
  XATTN_ERR_LAUNCH = -8     /* the HIP runtime refused the launch               */
};

/* Library ABI version (bumped when a signature changes). */
int xattn_abi_version(void);

/* Text for an XATTN_ERR_* code (static storage, never null). */
const char* xattn_error_string(int code);

/* ---------------------------------------------------------------------------
 * Antidiagonal estimator.  Replaces, fused and without materialising the
 * strided score matrix, the pair
 *   flat_group_gemm_fuse_reshape   xattn/src/kernels.py:325-363 (kernel 197-235)
 *   softmax_fuse_block_sum         xattn/src/kernels.py:238-289 (kernels 5-156)
 * as driven by the chunk loop of xattn_estimate, xattn/src/Xattention.py:138-172
 * (torch branch 174-252).
 *
 * Q and K are treated as zero-padded to multiples of chunk_size
 * (Xattention.py:33-51).  With n_rq = q_len_padded/stride reshaped query rows
 * and n_rk = k_len_padded/stride reshaped keys,
 *   score[m][n] = sum_i Q[m*stride + stride-1-i] . K[n*stride + i]
 * is scaled by `scale` (= 1/sqrt(128)/stride/norm), soft-maxed over the
 * visible n of each row, and summed into (block_size/stride)^2 tiles:
 *   block_sums[h][i][j], i < q_len_padded/block_size, j < k_len_padded/block_size.
 * causal != 0: reshaped key n is visible to row m iff
 *   k_lo(m) <= n <= m + (n_rk - n_rq)            (inclusive, Xattention.py:204-214)
 * with k_lo = 0 when own_chunk_only == 0 (the reference's Triton branch) or the
 * first reshaped key of the row's own chunk when own_chunk_only != 0 (what the
 * reference's torch branch computes when k_len is a multiple of chunk_size,
 * Xattention.py:201).  causal == 0: every n is visible, zero-padded keys
 * included.  Rows m >= n_rq - (q_len_padded - q_len)/stride are all-zero
 * (Xattention.py:237-238; see zero_rows_from).  Zero-padded keys are never
 * hidden: the reference's -inf over them (Xattention.py:201) is overwritten by
 * the triangle of the only chunk whose rows reach them (:203-214).
 * Only query chunks [chunk_begin, chunk_end) are processed (rows of block_sums
 * outside them are left untouched), so a caller may pipeline chunks on streams.
 * `scores_out`, when non-null, receives the un-scaled scores of those chunks as
 * fp32 [num_heads][n_rq][n_rk] (entries of tiles with no visible pair are left
 * untouched) - the flat_group_gemm_fuse_reshape seam, for tests.
 * `slab_pairs` (HOST pointer, 2 * num_slab_pairs ints, at most 64 pairs; NULL /
 * 0 for the default) generalises the reshape to the reference's other
 * select_mode settings (torch branch only, Xattention.py:72-135): the score is
 *   sum over pairs (a, b) of Q[m*stride + a] . K[n*stride + b],
 * the default being the pairs (stride-1-i, i).  "slash" is (i, i); "random"
 * (perm[i], i); "double" adds (stride-1-i, (i+1) % stride); "triple" weights
 * (stride-1-i, i) twice and adds (stride-1-i, (i+1) % stride) and
 * (stride-1-i, (i-1) % stride) (the reference adds the rolled key slabs in the
 * input precision before the product, this sum is taken in fp32).
 * softmax == 0 writes block sums of exp(scaled score) over the visible keys
 * instead of softmax probabilities (Xattention.py:231-234).
 * kdb > 1 subsamples the reshaped query rows (torch branch only,
 * Xattention.py:88-93, 174-181, 217-222, 245): query row j takes the tokens of
 * reshaped row j*kdb, sees (when causal) the keys of reshaped row j*kdb+kdb-1,
 * and a query block sums block_size/stride/kdb rows; kdb must divide
 * block_size/stride and needs the default reshape (num_slab_pairs == 0).
 * zero_rows_from: query rows (after subsampling) at or beyond this index give
 * all-zero block sums; negative = n_rq/kdb - (q_len_padded - q_len)/stride/kdb,
 * the torch branch's padded tail.  The reference's Triton branch zeroes rows by
 * their position on the key axis instead (xattn/src/kernels.py:70 with the
 * real_q_len of Xattention.py:169): n_rq - (k_len_padded - k_len)/stride; padded
 * query rows that rule leaves alone carry the uniform softmax of a zero query.
 * window_row0 / window_rows: block_sums may hold only the q-block rows
 * [window_row0, window_row0 + window_rows) of every head, laid out
 * [num_heads][window_rows][k_len_padded/block_size] (row i of the result at row
 * i - window_row0); the chunks of the call must lie inside the window.
 * window_rows <= 0 means the whole padded result.  A caller that works through
 * a long sequence in groups of query chunks needs buffers for one group only.
 * `workspace` must hold xattn_estimate_workspace_bytes(...) bytes, where
 * chunks_per_call is the largest chunk_end - chunk_begin used (<= 0: all chunks);
 * the function returns 0 for arguments the estimator rejects.
 */
size_t xattn_estimate_workspace_bytes(int num_heads, int q_len, int k_len, int stride, int block_size,
                                      int chunk_size, int chunks_per_call);

int xattn_estimate_block_sums(const void* q, const void* k, float* block_sums, void* workspace,
                              size_t workspace_bytes, float* scores_out, int num_heads,
                              int num_kv_heads, int q_len, int k_len, int head_dim, int64_t q_stride_h,
                              int64_t q_stride_n, int64_t k_stride_h, int64_t k_stride_n, int stride,
                              int block_size, int chunk_size, int chunk_begin, int chunk_end, int causal,
                              int own_chunk_only, float scale, const int32_t* slab_pairs,
                              int num_slab_pairs, int softmax, int kdb, int zero_rows_from, int window_row0,
                              int window_rows, void* stream);

/* ---------------------------------------------------------------------------
 * Threshold block selection.  Replaces find_blocks_chunked,
 * xattn/src/utils.py:44-191 (prefill branch), together with the mask
 * post-processing of xattn_estimate, xattn/src/Xattention.py:275-297.
 *
 * For q-block rows [row_begin, row_end) of every head: in fp64, required =
 * tau[h] * sum(row).  causal != 0: column 0 and the diagonal column
 * row + diag_offset are always kept; the remaining columns are visited by
 * descending block sum and kept while (forced mass + mass of those visited
 * before) < required; columns beyond the diagonal are cleared (block sums there
 * are taken as zero, which is what the estimator writes).  Rows are grouped
 * into query chunks of blocks_per_chunk rows; in a chunk whose first diagonal is
 * column 0 (diag_offset == 0 and row < blocks_per_chunk) the reference's eye()
 * assignment overwrites the forced sink (utils.py:100-106) while its prefix
 * still reserves two slots (utils.py:115-124): there only the diagonal is
 * forced, the largest other block is always kept and each later one is judged
 * against the mass gathered before its predecessor; column 0 ends up kept
 * through the scatter of unselected ranks (utils.py:142).  causal == 0:
 * all columns are visited by descending block sum and kept while the mass
 * visited before is < required; if any column is left out, column 0 is kept
 * (utils.py:164).  keep_sink sets q-block row 0 entirely (Xattention.py:286-287);
 * keep_recent sets the diagonal (288-297).  Ties in block sum are broken by
 * ascending column.
 * Outputs: mask [H][nq_blocks][nk_blocks] bytes (0/1);
 *          col_idx [H][nq_blocks][idx_pitch] ascending kept columns that are
 *          < list_cols and, when causal, hold a key visible to the row's last
 *          query token given kv_off_tokens = k_len - q_len;  col_cnt [H][nq_blocks].
 * col_idx/col_cnt may both be null; so may mask when the lists are asked for
 * (the operator itself only needs the lists).  nk_blocks <= 16384.
 * window_row0 / window_rows: block_sums, mask, col_idx and col_cnt hold the
 * q-block rows [window_row0, window_row0 + window_rows) of every head (row i at
 * row i - window_row0; per-head pitch window_rows rows); [row_begin, row_end)
 * must lie inside.  window_rows <= 0 means all nq_blocks rows.
 */
int xattn_select_blocks(const float* block_sums, const double* tau_per_head, uint8_t* mask,
                        int32_t* col_idx, int32_t* col_cnt, int64_t idx_pitch, int num_heads,
                        int nq_blocks, int nk_blocks, int row_begin, int row_end, int diag_offset,
                        int causal, int keep_sink, int keep_recent, int list_cols, int q_len,
                        int kv_off_tokens, int blocks_per_chunk, int window_row0, int window_rows,
                        void* stream);

/* ---------------------------------------------------------------------------
 * Estimate and selection in one call, for callers that want the column lists
 * (or the mask) and not the block sums - what the operator does at
 * xattn/src/Xattention.py:358-385, which never looks at attn_sums.  Same
 * arithmetic and results as xattn_estimate_block_sums followed by
 * xattn_select_blocks over the q-block rows of chunks [chunk_begin, chunk_end)
 * (replaces xattn/src/kernels.py:68-90 + xattn/src/utils.py:87-146 for that
 * use): the normalisation pass leaves each q-block row's block sums in LDS and
 * one wavefront selects from them there, so the sums make no round trip through
 * memory.  Arguments are those of the two entry points (the selection's geometry
 * - diagonal offset, list_cols, kv_off_tokens, blocks_per_chunk - follows from
 * the lengths); `block_sums` may be null, or receive the sums as well.  The
 * default reshape's row subsampling (kdb) is not available here, and padded key
 * lengths beyond 8192 blocks are refused with XATTN_ERR_SHAPE (use the two
 * entry points).  mask, col_idx/col_cnt, window_row0/window_rows as for
 * xattn_select_blocks.  `stages`: 3 runs both passes; 1 only the MFMA pass
 * (partial sums into the workspace), 2 only the normalise-and-select pass over a
 * workspace a stages = 1 call with the same arguments filled - for callers that
 * want an event or another stream between the two.
 */
int xattn_estimate_select(const void* q, const void* k, float* block_sums, void* workspace,
                          size_t workspace_bytes, int num_heads, int num_kv_heads, int q_len, int k_len,
                          int head_dim, int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_h,
                          int64_t k_stride_n, int stride, int block_size, int chunk_size, int chunk_begin,
                          int chunk_end, int causal, int own_chunk_only, float scale,
                          const int32_t* slab_pairs, int num_slab_pairs, int softmax, int zero_rows_from,
                          int window_row0, int window_rows, const double* tau_per_head, uint8_t* mask,
                          int32_t* col_idx, int32_t* col_cnt, int64_t idx_pitch, int keep_sink,
                          int keep_recent, int stages, void* stream);

/* ---------------------------------------------------------------------------
 * Block-sparse FlashAttention forward.  Replaces the call
 *   block_sparse_attn_func(q, k, v, cu_q, cu_k, head_mask_type, None, mask,
 *                          q_len, k_len, p_dropout=0, deterministic=True,
 *                          is_causal=causal)      xattn/src/Xattention.py:377-391
 * for one sequence (cu_seqlens = [0, len]) and per-head masks.  Query block
 * qb (128 tokens) of head h visits the col_cnt[h][qb] key blocks listed in
 * col_idx[h][qb - idx_row0][*] (arrays of idx_rows rows per head holding the
 * q-blocks [idx_row0, idx_row0 + idx_rows), each row idx_pitch entries long, as
 * xattn_select_blocks writes them; the q-blocks of the launch must lie inside);
 * inside a block, when causal, key c is visible to query t
 * iff c <= t + (k_len - q_len).  A query row with no visible key yields zeros.
 * col_idx == col_cnt == null visits every visible block: dense FlashAttention,
 * the baseline the speedup is quoted against.  Only query blocks
 * [q_block_begin, q_block_end) are computed (q_block_end < 0: up to the last),
 * so query chunks can be launched as their block lists become available.
 * Token strides of q, k, v and out: 128 .. 2^22 elements (all four are moved
 * as 128-row tiles whose byte offsets are held in 32 bits).
 */
int xattn_block_sparse_fwd(const void* q, const void* k, const void* v, void* out,
                           const int32_t* col_idx, const int32_t* col_cnt, int64_t idx_pitch,
                           int idx_rows, int idx_row0, int num_heads, int num_kv_heads, int q_len,
                           int k_len, int head_dim,
                           int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_h,
                           int64_t k_stride_n, int64_t v_stride_h, int64_t v_stride_n,
                           int64_t o_stride_h, int64_t o_stride_n, int q_block_begin, int q_block_end,
                           int causal, float softmax_scale, void* stream);

/* ---------------------------------------------------------------------------
 * Single-token decode attention over a KV cache.  Replaces the call to the
 * third-party flashinfer.single_decode_with_kv_cache(q, k, v, kv_layout="HND")
 * in the reference's Llama attention forward, xattn/src/load_llama.py:191-196:
 *   out[h] = softmax(q[h] . K[h/g]^T * softmax_scale) V[h/g],  g = H / H_kv <= 32.
 * q and out are [H][128] (head stride in elements), k and v [H_kv][k_len][128]
 * with head and token strides in elements (token stride 128..2^22, so both the
 * "HND" and the "NHD" cache layouts are views).  `workspace` holds the per-range
 * partial results: at least xattn_decode_workspace_bytes() bytes, 16-byte
 * aligned, contents undefined on entry and on return.
 */
size_t xattn_decode_workspace_bytes(int num_heads, int num_kv_heads, int k_len);

int xattn_decode_fwd(const void* q, const void* k, const void* v, void* out, void* workspace,
                     size_t workspace_bytes, int num_heads, int num_kv_heads, int k_len, int head_dim,
                     int64_t q_stride_h, int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_h,
                     int64_t v_stride_n, int64_t o_stride_h, float softmax_scale, void* stream);

/* Allocation-free form of xattn_decode_fwd.  It has no counterpart in the
 * reference: it exists for callers that cannot allocate device memory around
 * the call - code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  Same arguments and result as xattn_decode_fwd minus the
 * workspace: the per-range partial results live in a device array of
 * XATTN_DECODE_STATIC_SCRATCH_BYTES that is part of the library (each GPU the
 * library runs on holds its own copy until the process ends; its address on
 * the current device is looked up on the first call there, so the device the
 * stream belongs to must be current).  Problems whose
 * xattn_decode_workspace_bytes() exceeds that size (more than 256 * 32
 * (key range, query head) pairs: only with more than 256 KV heads) are refused
 * with XATTN_ERR_WORKSPACE.  The function calls no hipMalloc / hipFree.  All
 * calls on one GPU share the array: calls that may overlap on one GPU (two
 * streams, two threads) race on it and must be ordered by the caller; nothing
 * needs clearing between calls (every partial a launch reads it has written).
 */
#define XATTN_DECODE_STATIC_SCRATCH_BYTES (256 * 32 * 132 * 4)

int xattn_decode_fwd_static(const void* q, const void* k, const void* v, void* out, int num_heads,
                            int num_kv_heads, int k_len, int head_dim, int64_t q_stride_h,
                            int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_h, int64_t v_stride_n,
                            int64_t o_stride_h, float softmax_scale, void* stream);

/* ---------------------------------------------------------------------------
 * Stand-alone softmax + block sums over a score matrix in memory: the seam
 * softmax_fuse_block_sum, xattn/src/kernels.py:238-289 (kernels :5-156), for
 * callers that hold the strided scores themselves (the fused estimator above
 * does not use it).  `scores` is bf16 [num_heads][n_rq][n_rk] with head / row
 * strides in elements (multiples of 8, rows contiguous); row i sits at key
 * position chunk_start + i.  p = exp2(score * scale - rowmax) / rowsum over the
 * visible keys (causal != 0: keys <= chunk_start + i; else all n_rk), rows at
 * positions >= real_q_len give zeros; block_sums is fp32
 * [num_heads][n_rq / rbs][n_rk / rbs], rbs = reshaped_block_size in {8, 16, 32}.
 */
int xattn_softmax_block_sums(const void* scores, float* block_sums, int num_heads, int n_rq, int n_rk,
                             int64_t stride_h, int64_t stride_row, int reshaped_block_size, int chunk_start,
                             int real_q_len, float scale, int causal, void* stream);

/* ---------------------------------------------------------------------------
 * Threshold profiler, xattn/threshold/profile_threshold/profile_threshold.py.
 *
 * xattn_block_mass replaces chunk_prefill_to_attn_sum (:15-57): the true
 * softmax(q k^T * softmax_scale) probabilities (token-causal when `causal`,
 * bottom-right aligned when k_len > q_len; the reference always masks
 * causally and asserts equal block counts) summed over each 128 x 128 block,
 *   mass[h][i][j] = sum over rows of q-block i, keys of k-block j,
 * fp32 [H][ceil(q_len/128)][ceil(k_len/128)], every entry written (zeros for
 * blocks no row of the q-block sees).  Rows past q_len carry no mass, so a
 * full q-block row of `mass` sums to 128.  Nothing is materialised.
 *
 * xattn_threshold_rows does the per-row part of xattn_prefill_profile
 * (:84-93): for (head, q-block row) it takes blocks by decreasing mass until
 * `coverage` (0.9 in the reference) of the row's mass is reached, including the
 * block that crosses, finds the smallest estimate_sums value among them and
 * writes rows_out[h][i] = { sum of the row's estimate_sums at or above that
 * value, sum of the row's estimate_sums }.  The profiled threshold of head h is
 * sum_i rows_out[h][i][0] / (sum_i rows_out[h][i][1] + 1e-8) (:93); the caller
 * adds the rows up.  estimate_sums is read as [h * est_head_pitch +
 * i * est_row_pitch + j] (elements), so the padded output of
 * xattn_estimate_block_sums can be passed as it is.  nk_blocks <= 16384.
 */
int xattn_block_mass(const void* q, const void* k, float* mass, int num_heads, int num_kv_heads,
                     int q_len, int k_len, int head_dim, int64_t q_stride_h, int64_t q_stride_n,
                     int64_t k_stride_h, int64_t k_stride_n, int causal, float softmax_scale, void* stream);

int xattn_threshold_rows(const float* block_mass, const float* estimate_sums, float* rows_out,
                         int num_heads, int nq_blocks, int nk_blocks, int64_t est_head_pitch,
                         int64_t est_row_pitch, float coverage, void* stream);

/* ---------------------------------------------------------------------------
 * Measurement aid, no counterpart in the reference: copies `bytes` (a multiple
 * of 16) from src to dst with a plain kernel, i.e. reads `bytes` and writes
 * `bytes` of HBM.  Profiling runs use it to scale hardware byte counters.
 */
int xattn_calibration_copy(void* dst, const void* src, size_t bytes, void* stream);

/* Measurement aid, no counterpart in the reference: 512 workgroups (two
 * wavefronts per SIMD on 256 CUs) issue nothing but bf16 32x32x16 MFMAs,
 * 16 * iters per wavefront, on register operands taken once from
 * `operand_bits` (device, 64 KiB: 4096 fragments of 8 bf16).  The number of
 * floating-point operations of the launch is written to *flops_out (host, may
 * be null); the caller times the launch.  Equal bits everywhere measure the
 * data-independent rate, random bits the rate the part sustains at the
 * switching activity of real inputs.  With valu_mix != 0 every MFMA is
 * accompanied by one v_exp_f32 and three v_fma_f32 on unrelated registers (the
 * vector-ALU load per MFMA of the attention tile loop, with no dependences and
 * no memory traffic): the rate then is what the SIMD's instruction issue
 * leaves of the MFMA stream under that mix.  `sink` is one float of device
 * memory that is practically never written.
 */
int xattn_mfma_rate_probe(const void* operand_bits, int iters, int valu_mix, float* sink, double* flops_out,
                          void* stream);

#ifdef __cplusplus
}
#endif
#endif /* XATTN_HIP_H */
