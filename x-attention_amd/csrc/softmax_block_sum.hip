// Softmax + block sums over a score matrix that already sits in memory.
//
// Stand-alone counterpart of the reference's second estimator kernel,
// softmax_fuse_block_sum (xattn/src/kernels.py:238-289, kernels :5-156), for
// callers that hold the strided scores themselves.  The fused estimator never
// writes the scores and does not use this kernel.
//
// One workgroup per (head, query block of rbs rows).  Phase A: each wavefront
// takes every fourth row and computes its maximum and sum over the visible keys
// (exp2 domain, `scale` carries log2 e like the reference's).  Phase B: lanes own
// 8 consecutive keys; for each 512-key strip a wavefront adds the normalised
// probabilities of its rows, lanes of one key block meet by shuffles and the four
// wavefronts in LDS - a fixed order, so results repeat bit for bit.  The matrix
// is read twice (the second time mostly from L2): the kernel is HBM-bound.
#include "xattn_common.h"
#include "xattn_hip.h"

namespace xattn {

struct SbsParams {
  const __bf16* x;      // [H][n_rq][n_rk], row stride x_sr, head stride x_sh (elements)
  float* out;           // [H][n_rq / rbs][n_rk / rbs]
  int64_t x_sh, x_sr;
  int H, n_rq, n_rk, rbs;
  int chunk_start;      // position of row 0 on the key axis
  int real_q_len;       // rows at positions >= real_q_len are padding: zeros
  int causal;
  float scale;          // multiplies the raw score; includes log2(e)
};

__global__ __launch_bounds__(256) void softmax_block_sum_kernel(SbsParams p) {
  __shared__ float rowM[32], rowInv[32];
  __shared__ float part[4][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int qb = blockIdx.x, head = blockIdx.y;
  const __bf16* xb = p.x + (int64_t)head * p.x_sh + (int64_t)qb * p.rbs * p.x_sr;
  float* out = p.out + ((int64_t)head * (p.n_rq / p.rbs) + qb) * (p.n_rk / p.rbs);

  // ---- phase A: row statistics
  for (int r = wave; r < p.rbs; r += 4) {
    const int pos = p.chunk_start + qb * p.rbs + r;
    const int last = p.causal ? (pos < p.n_rk - 1 ? pos : p.n_rk - 1) : p.n_rk - 1;   // last visible key
    const __bf16* row = xb + (int64_t)r * p.x_sr;
    float m = -INFINITY, l = 0.f;
    for (int c0 = lane * 8; c0 <= last; c0 += 512) {
      const bf16x8 v = *reinterpret_cast<const bf16x8*>(row + c0);
      float s[8], mx = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        s[e] = (c0 + e <= last) ? (float)v[e] * p.scale : -INFINITY;
        mx = fmaxf(mx, s[e]);
      }
      const float mn = fmaxf(m, mx);
      float add = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) add += fast_exp2(s[e] - mn);
      l = l * fast_exp2(m - mn) + add;     // mn is finite here: column c0 itself is visible
      m = mn;
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
      const float om = __shfl_xor(m, d, 64), ol = __shfl_xor(l, d, 64);
      const float mn = fmaxf(m, om);
      const float safe = (mn == -INFINITY) ? 0.f : mn;
      l = l * fast_exp2(m - safe) + ol * fast_exp2(om - safe);
      m = mn;
    }
    if (lane == 0) {
      const bool real = pos < p.real_q_len && l > 0.f;
      rowM[r] = (m == -INFINITY) ? 0.f : m;
      rowInv[r] = real ? 1.f / l : 0.f;
    }
  }
  __syncthreads();

  // ---- phase B: block sums, 512 keys (64 lanes x 8) per strip
  const int lanes_per_block = p.rbs / 8;            // 1, 2 or 4
  const int blocks_per_strip = 512 / p.rbs;
  for (int c0 = 0; c0 < p.n_rk; c0 += 512) {
    const int c = c0 + lane * 8;
    float acc = 0.f;
    if (c < p.n_rk) {
      for (int r = wave; r < p.rbs; r += 4) {
        const int pos = p.chunk_start + qb * p.rbs + r;
        const int last = p.causal ? pos : p.n_rk - 1;
        if (c > last) continue;
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(xb + (int64_t)r * p.x_sr + c);
        const float m = rowM[r], inv = rowInv[r];
        float s = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) s += (c + e <= last) ? fast_exp2((float)v[e] * p.scale - m) : 0.f;
        acc += s * inv;
      }
    }
    for (int d = 1; d < lanes_per_block; d <<= 1) acc += __shfl_xor(acc, d, 64);
    part[wave][lane] = acc;
    __syncthreads();
    if (tid < blocks_per_strip) {
      const int src = tid * lanes_per_block;
      const int kb = c0 / p.rbs + tid;
      if (kb < p.n_rk / p.rbs) out[kb] = (part[0][src] + part[1][src]) + (part[2][src] + part[3][src]);
    }
    __syncthreads();
  }
}

}  // namespace xattn

using namespace xattn;

extern "C" int xattn_softmax_block_sums(const void* scores, float* block_sums, int num_heads, int n_rq, int n_rk,
                                        int64_t stride_h, int64_t stride_row, int reshaped_block_size,
                                        int chunk_start, int real_q_len, float scale, int causal, void* stream) {
  if (!scores || !block_sums) return XATTN_ERR_NULL;
  if (num_heads <= 0 || num_heads > 65535 || n_rq <= 0 || n_rk <= 0) return XATTN_ERR_SHAPE;
  if (reshaped_block_size != 8 && reshaped_block_size != 16 && reshaped_block_size != 32) return XATTN_ERR_STRIDE;
  if (n_rq % reshaped_block_size || n_rk % reshaped_block_size) return XATTN_ERR_SHAPE;
  if (stride_row % 8 || stride_h % 8 || stride_row < n_rk || (reinterpret_cast<uintptr_t>(scores) & 15))
    return XATTN_ERR_ALIGN;
  if (chunk_start < 0) return XATTN_ERR_SHAPE;
  SbsParams p;
  p.x = static_cast<const __bf16*>(scores);
  p.out = block_sums;
  p.x_sh = stride_h; p.x_sr = stride_row;
  p.H = num_heads; p.n_rq = n_rq; p.n_rk = n_rk; p.rbs = reshaped_block_size;
  p.chunk_start = chunk_start; p.real_q_len = real_q_len; p.causal = causal ? 1 : 0; p.scale = scale;
  hipLaunchKernelGGL(softmax_block_sum_kernel, dim3((unsigned)(n_rq / reshaped_block_size), (unsigned)num_heads),
                     dim3(256), 0, static_cast<hipStream_t>(stream), p);
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}
