// Kernels of the threshold profiler for gfx950.
//
// The reference profiles per-head thresholds offline
// (xattn/threshold/profile_threshold/profile_threshold.py): for every layer it
// (1) materialises the true attention probabilities q-block by q-block in torch
//     and sums them per 128x128 block (chunk_prefill_to_attn_sum, :15-57),
// (2) finds per q-block row the fewest blocks holding 90 % of that mass and the
//     smallest antidiagonal estimate among them, and reports per head which
//     share of the total estimate lies in blocks at or above that value
//     (xattn_prefill_profile, :84-96).
//
// block_mass_kernel does (1) without materialising anything: two sweeps of
// K Q^T per q-block (the first for the row maxima and sums, the second for the
// normalised probabilities, added up over the block's 128 rows), tiles moved
// exactly as in the attention kernel.  threshold_rows_kernel does the per-row
// part of (2); the sum over a head's rows is left to the caller.
#include "attn_tiles.h"
#include "xattn_hip.h"

namespace xattn {

struct MassParams {
  const __bf16* q;
  const __bf16* k;
  float* mass;              // [H][nqb][nkb]
  int64_t q_sh, q_sn, k_sh, k_sn;
  int H, Hkv, Lq, Lk, nqb, nkb;
  int causal, kv_off;
  float scale_log2;
};

__global__ __launch_bounds__(256, 2) void block_mass_kernel(MassParams p) {
  __shared__ __attribute__((aligned(1024))) char Kbuf[2][kTileBytes];
  __shared__ float red[2][4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, hh = lane >> 5;

  int head, qb;
  if (!map_workgroup(blockIdx.x, p.H, p.Hkv, 0, p.nqb, &head, &qb)) return;
  const int kvh = head / (p.H / p.Hkv);
  const __bf16* qbase = p.q + (int64_t)head * p.q_sh;
  const __bf16* kbase = p.k + (int64_t)kvh * p.k_sh;
  float* out = p.mass + ((int64_t)head * p.nqb + qb) * p.nkb;

  const int q_row = qb * kBlk + wave * 32 + r;
  const int q_pos = q_row + p.kv_off;
  const bool row_ok = q_row < p.Lq;
  int visible;
  {
    const int q_last = (qb * kBlk + kBlk - 1 < p.Lq ? qb * kBlk + kBlk - 1 : p.Lq - 1) + p.kv_off;
    visible = p.causal ? (q_last < 0 ? 0 : q_last / kBlk + 1) : p.nkb;
    visible = visible < p.nkb ? visible : p.nkb;
  }
  for (int kb = visible + tid; kb < p.nkb; kb += 256) out[kb] = 0.f;
  if (visible == 0) return;

  bf16x8 qreg[8];
  {
    const int row = row_ok ? q_row : p.Lq - 1;
    const __bf16* src = qbase + (int64_t)row * p.q_sn + hh * 8;
#pragma unroll
    for (int s = 0; s < 8; ++s) qreg[s] = *reinterpret_cast<const bf16x8*>(src + s * 16);
  }
  int voffK[8];
  tile_offsets(p.k_sn, lane, wave, voffK);
  int kaddr[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) kaddr[s] = r * 256 + (((2 * s + hh) ^ swz(r)) << 4);

  float m_run = -INFINITY, l_run = 0.f;   // sweep 1: running row maximum (exp2 domain) and this lane's share of the sum
  float inv_l = 0.f;                      // sweep 2: 1 / row sum

  // step jj visits key block jj % visible; steps [0, visible) are sweep 1,
  // [visible, 2*visible) sweep 2; the copy of the next step's block overlaps
  // the current step's arithmetic (two tile buffers, one barrier per step)
  const int steps = 2 * visible;
  copy_tile(kbase, p.k_sn, p.Lk, 0, voffK, Kbuf[0], wave);
  for (int jj = 0; jj < steps; ++jj) {
    const int kb = jj < visible ? jj : jj - visible;
    const char* Ks = Kbuf[jj & 1];
    wait_vm0();
    __syncthreads();   // block kb landed; everyone is done with the other buffer and with red[jj & 1]
    if (jj + 1 < steps) {
      const int nb = jj + 1 < visible ? jj + 1 : jj + 1 - visible;
      copy_tile(kbase, p.k_sn, p.Lk, nb, voffK, Kbuf[(jj + 1) & 1], wave);
    }
    if (jj > visible && tid == 0) {
      const float* rr = red[(jj - 1) & 1];
      out[kb - 1] = (rr[0] + rr[1]) + (rr[2] + rr[3]);
    }

    f32x16 sacc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) sacc[i][v] = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      bf16x8 kf[4];
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) kf[nt] = *reinterpret_cast<const bf16x8*>(Ks + kaddr[s] + nt * 8192);
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) sacc[nt] = mfma32(kf[nt], qreg[s], sacc[nt]);
    }
    const bool need_mask = (kb * kBlk + kBlk > p.Lk) || (p.causal && kb * kBlk + kBlk - 1 > qb * kBlk + p.kv_off);
    if (need_mask) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int kpos = kb * kBlk + nt * 32 + (v >> 2) * 8 + hh * 4 + (v & 3);
          const bool dead = kpos >= p.Lk || (p.causal && kpos > q_pos);
          sacc[nt][v] = dead ? -INFINITY : sacc[nt][v];
        }
    }
    if (jj < visible) {
      float mx = -INFINITY;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[nt][v]);
      mx = half_max(mx) * p.scale_log2;
      const float m_new = fmaxf(m_run, mx);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      float psum = 0.f;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) psum += fast_exp2(__builtin_fmaf(sacc[nt][v], p.scale_log2, -m_safe));
      l_run = l_run * ((m_run == -INFINITY) ? 0.f : fast_exp2(m_run - m_safe)) + psum;
      m_run = m_new;
      if (jj == visible - 1) {
        const float l_tot = half_sum(l_run);
        inv_l = (row_ok && l_tot > 0.f) ? 1.f / l_tot : 0.f;   // padded rows carry no mass
      }
    } else {
      const float m_safe = (m_run == -INFINITY) ? 0.f : m_run;
      float psum = 0.f;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) psum += fast_exp2(__builtin_fmaf(sacc[nt][v], p.scale_log2, -m_safe));
      psum *= inv_l;
#pragma unroll
      for (int d = 32; d > 0; d >>= 1) psum += __shfl_xor(psum, d, 64);
      if (lane == 0) red[jj & 1][wave] = psum;
    }
  }
  __syncthreads();
  if (tid == 0) {
    const float* rr = red[(steps - 1) & 1];
    out[visible - 1] = (rr[0] + rr[1]) + (rr[2] + rr[3]);
  }
}

struct RowParams {
  const float* mass;     // [H][nqb][nkb]
  const float* est;      // estimate sums, head pitch est_ph, row pitch est_pr (elements)
  float* rows;           // [H][nqb][2]: sum of estimate at or above the row's cut, sum of estimate
  int64_t est_ph, est_pr;
  int H, nqb, nkb;
  float coverage;
};

// One wavefront per (head, q-block row).  Blocks are taken in order of
// decreasing true mass (lowest column first among equals) until the running
// mass reaches coverage * total - the block that crosses is taken too, i.e.
// need_len = #(cumsum < coverage * total) + 1 of the reference; the smallest
// estimate among the taken blocks is the row's cut.
__global__ __launch_bounds__(64) void threshold_rows_kernel(RowParams p) {
  extern __shared__ float row_lds[];
  float* a = row_lds;
  float* x = row_lds + p.nkb;
  const int lane = threadIdx.x;
  const int row = blockIdx.x % p.nqb, head = blockIdx.x / p.nqb;
  const float* am = p.mass + ((int64_t)head * p.nqb + row) * p.nkb;
  const float* xe = p.est + (int64_t)head * p.est_ph + (int64_t)row * p.est_pr;

  double tot = 0.0;
  float xall = 0.f;
  for (int j = lane; j < p.nkb; j += 64) {
    const float av = am[j], xv = xe[j];
    a[j] = av;
    x[j] = xv;
    tot += av;
    xall += xv;
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) {
    tot += __shfl_xor(tot, d, 64);
    xall += __shfl_xor(xall, d, 64);
  }
  __syncthreads();
  const double need = (double)p.coverage * tot;
  double cum = 0.0;
  float cut = INFINITY;
  for (int taken = 0; taken < p.nkb; ++taken) {
    float best = -1.f;
    int bidx = 0x7fffffff;
    for (int j = lane; j < p.nkb; j += 64) {
      const float av = a[j];
      if (av > best) {   // strided ascending scan: the first maximum a lane meets is its lowest column
        best = av;
        bidx = j;
      }
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
      const float ob = __shfl_xor(best, d, 64);
      const int oi = __shfl_xor(bidx, d, 64);
      if (ob > best || (ob == best && oi < bidx)) {
        best = ob;
        bidx = oi;
      }
    }
    // (a block without mass is only ever taken as a row's first: it cannot move the running mass)
    if (best < 0.f || (taken > 0 && best == 0.f)) break;
    cut = fminf(cut, x[bidx]);
    if (lane == 0) a[bidx] = -1.f;
    __syncthreads();
    cum += best;
    if (!(cum < need)) break;
  }
  float xge = 0.f;
  for (int j = lane; j < p.nkb; j += 64) xge += x[j] >= cut ? x[j] : 0.f;
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) xge += __shfl_xor(xge, d, 64);
  if (lane == 0) {
    float* o = p.rows + ((int64_t)head * p.nqb + row) * 2;
    o[0] = xge;
    o[1] = xall;
  }
}

}  // namespace xattn

using namespace xattn;

extern "C" int xattn_block_mass(const void* q, const void* k, float* mass, int num_heads, int num_kv_heads,
                                int q_len, int k_len, int head_dim, int64_t q_stride_h, int64_t q_stride_n,
                                int64_t k_stride_h, int64_t k_stride_n, int causal, float softmax_scale,
                                void* stream) {
  if (!q || !k || !mass) return XATTN_ERR_NULL;
  if (head_dim != kHeadDim) return XATTN_ERR_HEAD_DIM;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads) return XATTN_ERR_HEADS;
  if (q_len <= 0 || k_len <= 0 || k_len < q_len) return XATTN_ERR_SHAPE;
  const int64_t strides[] = {q_stride_h, q_stride_n, k_stride_h, k_stride_n};
  for (int64_t s : strides)
    if (s % 8) return XATTN_ERR_ALIGN;
  if ((reinterpret_cast<uintptr_t>(q) & 15) || (reinterpret_cast<uintptr_t>(k) & 15)) return XATTN_ERR_ALIGN;
  if (!tile_stride_ok(k_stride_n) || q_stride_n < kHeadDim) return XATTN_ERR_SHAPE;
  if (!scale_ok(softmax_scale)) return XATTN_ERR_SHAPE;
  MassParams p;
  p.q = static_cast<const __bf16*>(q);
  p.k = static_cast<const __bf16*>(k);
  p.mass = mass;
  p.q_sh = q_stride_h; p.q_sn = q_stride_n; p.k_sh = k_stride_h; p.k_sn = k_stride_n;
  p.H = num_heads; p.Hkv = num_kv_heads; p.Lq = q_len; p.Lk = k_len;
  p.nqb = (q_len + kBlk - 1) / kBlk;
  p.nkb = (k_len + kBlk - 1) / kBlk;
  p.causal = causal ? 1 : 0;
  p.kv_off = k_len - q_len;
  p.scale_log2 = softmax_scale * kLog2e;
  const int64_t grid = grid_for(p.H, p.Hkv, p.nqb);
  if (grid > 0x7fffffff) return XATTN_ERR_SHAPE;
  hipLaunchKernelGGL(block_mass_kernel, dim3((unsigned)grid), dim3(256), 0, static_cast<hipStream_t>(stream), p);
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}

extern "C" int xattn_threshold_rows(const float* block_mass, const float* estimate_sums, float* rows_out,
                                    int num_heads, int nq_blocks, int nk_blocks, int64_t est_head_pitch,
                                    int64_t est_row_pitch, float coverage, void* stream) {
  if (!block_mass || !estimate_sums || !rows_out) return XATTN_ERR_NULL;
  if (num_heads <= 0 || nq_blocks <= 0 || nk_blocks <= 0 || nk_blocks > 16384) return XATTN_ERR_SHAPE;
  if (est_row_pitch < nk_blocks || est_head_pitch < est_row_pitch * nq_blocks) return XATTN_ERR_SHAPE;
  if (!(coverage >= 0.f && coverage <= 1.f)) return XATTN_ERR_SHAPE;
  const int64_t grid = (int64_t)num_heads * nq_blocks;
  if (grid > 0x7fffffff) return XATTN_ERR_SHAPE;
  RowParams p;
  p.mass = block_mass; p.est = estimate_sums; p.rows = rows_out;
  p.est_ph = est_head_pitch; p.est_pr = est_row_pitch;
  p.H = num_heads; p.nqb = nq_blocks; p.nkb = nk_blocks;
  p.coverage = coverage;
  const size_t lds = (size_t)nk_blocks * 2 * sizeof(float);
  if (lds > 65536) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(threshold_rows_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return XATTN_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(threshold_rows_kernel, dim3((unsigned)grid), dim3(64), lds, static_cast<hipStream_t>(stream), p);
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}
