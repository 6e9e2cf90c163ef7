// Threshold block selection for gfx950: one wavefront per (head, q-block row).
//
// Replaces find_blocks_chunked (xattn/src/utils.py:44-191, prefill branch) and
// the mask post-processing of xattn_estimate (xattn/src/Xattention.py:275-297).
// The reference runs ~15 eager torch ops over an fp64 copy of the block sums
// (two full sorts, a cumsum, an advanced-index scatter) and synchronises the
// device once per chunk; here a row's candidates (only the columns up to the
// diagonal when causal - the problem size follows the row) are first tried by
// extraction: the wavefront pulls out the largest remaining block, adds its
// mass, and stops as soon as the threshold is reached - on sparse rows that is a
// handful of wavefront reductions.  Rows that need more than kMaxExtract blocks
// fall back to a bitonic sort of the candidates in LDS followed by an fp64
// wavefront prefix scan.  Both visit blocks in the same order (descending sum,
// ascending column among equals) and apply the same rule.  The kernel emits the
// final mask row plus the compacted, ascending column list the attention kernel
// walks.
//
// The causal rule, as the reference's tensors define it (utils.py:107-141): the
// row is ranked by a key that is the block sum for ordinary blocks and
// 100000 * (1 + sum) for the forced ones; rank r is kept while M(r) < tau *
// total, with M(0) = M(1) = 0 and M(r) = forced_sum + the r - 2 largest
// ordinary sums.  With softmax block sums (at most block_size / stride per
// block) the forced blocks always rank first, so the i-th largest ordinary
// block sits at rank i + 2 (i + 1 in the first query chunk, where only the
// diagonal is forced) - but un-normalised sums (softmax = 0) can exceed a
// forced key, and such a block then moves up one or two ranks.  rank_mass()
// implements exactly that: the i-th ordinary block with `ahead` forced keys
// before it is judged against M(i + ahead).
#include "select_row.h"
#include "xattn_hip.h"

namespace xattn {

__global__ __launch_bounds__(64) void select_blocks_kernel(SelParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  uint64_t* keys = reinterpret_cast<uint64_t*>(smem);
  uint8_t* flags = reinterpret_cast<uint8_t*>(smem + (size_t)p.npow2 * 8);
  const int rows = p.row_end - p.row_begin;
  const int head = blockIdx.x / rows;
  const int row = p.row_begin + blockIdx.x % rows;
  const int64_t slot = (int64_t)head * p.win_rows + (row - p.win_row0);
  select_row(p, p.sums + slot * p.nkb, head, row, keys, flags, threadIdx.x);
}

}  // namespace xattn

using namespace xattn;

extern "C" int xattn_select_blocks(const float* block_sums, const double* tau_per_head, uint8_t* mask,
                                   int32_t* col_idx, int32_t* col_cnt, int64_t idx_pitch, int num_heads,
                                   int nq_blocks, int nk_blocks, int row_begin, int row_end,
                                   int diag_offset, int causal, int keep_sink, int keep_recent,
                                   int list_cols, int q_len, int kv_off_tokens, int blocks_per_chunk,
                                   int window_row0, int window_rows, void* stream) {
  if (!block_sums || !tau_per_head) return XATTN_ERR_NULL;
  if ((col_idx == nullptr) != (col_cnt == nullptr)) return XATTN_ERR_NULL;
  if (!mask && !col_idx) return XATTN_ERR_NULL;     // nothing to write
  if (num_heads <= 0 || nq_blocks <= 0 || nk_blocks <= 0 || nk_blocks > 16384) return XATTN_ERR_SHAPE;
  if (row_begin < 0 || row_end > nq_blocks || row_begin >= row_end) return XATTN_ERR_SHAPE;
  if (col_idx && idx_pitch < 1) return XATTN_ERR_SHAPE;
  if (diag_offset < 0 || blocks_per_chunk < 1) return XATTN_ERR_SHAPE;
  SelParams p;
  p.sums = block_sums; p.tau = tau_per_head; p.mask = mask; p.col_idx = col_idx; p.col_cnt = col_cnt;
  p.idx_pitch = idx_pitch; p.H = num_heads; p.nqb = nq_blocks; p.nkb = nk_blocks;
  p.row_begin = row_begin; p.row_end = row_end; p.diag_offset = diag_offset;
  p.causal = causal ? 1 : 0; p.keep_sink = keep_sink ? 1 : 0; p.keep_recent = keep_recent ? 1 : 0;
  p.list_cols = list_cols; p.q_len = q_len; p.kv_off = kv_off_tokens;
  p.blocks_per_chunk = blocks_per_chunk;
  if (window_rows <= 0) { window_row0 = 0; window_rows = nq_blocks; }
  if (window_row0 < 0 || row_begin < window_row0 || row_end > window_row0 + window_rows) return XATTN_ERR_SHAPE;
  p.win_row0 = window_row0; p.win_rows = window_rows;
  int np2 = 64;
  while (np2 < nk_blocks) np2 <<= 1;
  p.npow2 = np2;
  const size_t lds = (size_t)np2 * 8 + (((size_t)nk_blocks + 15) & ~(size_t)15);
  const int64_t grid = (int64_t)num_heads * (row_end - row_begin);
  if (grid > 0x7fffffff) return XATTN_ERR_SHAPE;
  if (lds > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&select_blocks_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return XATTN_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(select_blocks_kernel, dim3((unsigned)grid), dim3(64), lds,
                     static_cast<hipStream_t>(stream), p);
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}
