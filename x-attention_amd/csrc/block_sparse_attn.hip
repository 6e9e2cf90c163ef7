// Block-sparse FlashAttention forward for gfx950 (bf16 MFMA, fp32 softmax).
//
// Replaces the reference's call to the third-party CUDA kernel
// block_sparse_attn_func (xattn/src/Xattention.py:377-391): for every query
// block of 128 tokens only the key/value blocks named by a per-(head, q-block)
// column list are visited, with token-level causal masking (bottom-right
// aligned when k_len > q_len) and grouped-query attention by KV-head sharing.
// With no column list the same kernel visits every visible block, which is the
// dense FlashAttention baseline the speedup is quoted against.
//
// Work decomposition: one workgroup (4 wavefronts) per (head, q-block); each
// wavefront owns 32 query rows.  Scores are produced transposed,
// S^T = K Q^T, so that one lane owns one query row (softmax statistics need a
// single cross-lane exchange) and the fp32 accumulator registers of S^T are,
// unchanged, the B operand of O^T += V^T P^T.  K is staged row-major and V
// transposed (with the accumulator's row permutation folded in) through LDS;
// the next tile's global loads are in flight while the current one is
// multiplied.  Two workgroups fit per CU (68 KiB LDS each) so one's softmax
// overlaps the other's MFMA.
#include "xattn_common.h"
#include "xattn_hip.h"

namespace xattn {

constexpr int kBlk = 128;          // block_size of the operator
constexpr int kLdsRow = 136;       // bf16 per LDS row: 128 + 8 pad (272 B) -> conflict-free b128 reads

struct AttnParams {
  const __bf16* q;
  const __bf16* k;
  const __bf16* v;
  __bf16* o;
  int64_t q_sh, q_sn, k_sh, k_sn, v_sh, v_sn, o_sh, o_sn;  // element strides (head, token)
  const int32_t* col_idx;   // [H, nqb, idx_pitch] ascending k-block ids, or null = all visible
  const int32_t* col_cnt;   // [H, nqb]
  int64_t idx_pitch;
  int idx_rows;             // q-block rows per head in col_idx / col_cnt (>= nqb)
  int H, Hkv, Lq, Lk, nqb, nkb;
  int causal, kv_off;       // kv_off = Lk - Lq
  float scale_log2;         // softmax_scale * log2(e)
};

__device__ __forceinline__ int clamp_block(int kb, int nkb) { return kb < 0 ? 0 : (kb < nkb ? kb : nkb - 1); }

__device__ __forceinline__ void load_k_tile(const AttnParams& p, const __bf16* kbase, int kb, int tid,
                                            u32x4 (&st)[8]) {
  const int chunk = tid & 15, row0 = tid >> 4;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    int n = kb * kBlk + i * 16 + row0;
    n = n < p.Lk ? n : p.Lk - 1;   // rows past the end are masked in the softmax
    st[i] = *reinterpret_cast<const u32x4*>(kbase + (int64_t)n * p.k_sn + chunk * 8);
  }
}

__device__ __forceinline__ void store_k_tile(__bf16* Ks, int tid, const u32x4 (&st)[8]) {
  const int chunk = tid & 15, row0 = tid >> 4;
#pragma unroll
  for (int i = 0; i < 8; ++i)
    *reinterpret_cast<u32x4*>(Ks + (i * 16 + row0) * kLdsRow + chunk * 8) = st[i];
}

// thread -> (4 consecutive key rows) x (8 consecutive features), twice
__device__ __forceinline__ void load_v_tile(const AttnParams& p, const __bf16* vbase, int kb, int tid,
                                            u32x4 (&st)[8]) {
  const int lane = tid & 63, wave = tid >> 6;
  const int ng = lane & 15, dc = (lane >> 4) + 4 * wave;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int n = kb * kBlk + hf * 64 + ng * 4 + i;
      bool ok = n < p.Lk;
      n = ok ? n : p.Lk - 1;
      u32x4 x = *reinterpret_cast<const u32x4*>(vbase + (int64_t)n * p.v_sn + dc * 8);
      const u32x4 z = {0u, 0u, 0u, 0u};
      st[hf * 4 + i] = ok ? x : z;   // rows past the sequence end must be exact zeros
    }
}

// Writes V^T: LDS row = feature, column = key position permuted so that the 8
// keys one MFMA lane needs (n = 16s + 8a + 4h + t -> 16s + 8h + 4a + t) are
// contiguous.
__device__ __forceinline__ void store_v_tile_t(__bf16* Vt, int tid, const u32x4 (&st)[8]) {
  const int lane = tid & 63, wave = tid >> 6;
  const int ng = lane & 15, dc = (lane >> 4) + 4 * wave;
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    const int n0 = hf * 64 + ng * 4;
    const int pos = (n0 & ~15) + ((n0 >> 2) & 1) * 8 + ((n0 >> 3) & 1) * 4;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t a = st[hf * 4 + 0][j >> 1], b = st[hf * 4 + 1][j >> 1];
      uint32_t c = st[hf * 4 + 2][j >> 1], d = st[hf * 4 + 3][j >> 1];
      u32x2 w;
      if (j & 1) {
        w[0] = (a >> 16) | (b & 0xffff0000u);
        w[1] = (c >> 16) | (d & 0xffff0000u);
      } else {
        w[0] = (a & 0xffffu) | (b << 16);
        w[1] = (c & 0xffffu) | (d << 16);
      }
      *reinterpret_cast<u32x2*>(Vt + (dc * 8 + j) * kLdsRow + pos) = w;
    }
  }
}

// kHasList = false is the dense baseline (its own symbol, so profiles tell the two apart)
template <bool kHasList>
__global__ __launch_bounds__(256, 2) void block_sparse_fwd_kernel(AttnParams p) {
  __shared__ __attribute__((aligned(16))) __bf16 Ks[kBlk * kLdsRow];
  __shared__ __attribute__((aligned(16))) __bf16 Vt[kBlk * kLdsRow];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, hh = lane >> 5;

  // Workgroup ids are dealt round-robin to the 8 XCDs.  Eight consecutive ids
  // take eight consecutive q-blocks of ONE head, so every head's rows - whose
  // list lengths vary smoothly with the row but by orders of magnitude between
  // heads - are spread evenly over the XCDs; the next eight ids take the next
  // head, so the query heads of a KV group with the same q-block run side by
  // side on one XCD and share its L2 for K/V.  Rows go out last (longest, when
  // causal) first.
  int head, qb;
  {
    const int id = blockIdx.x;
    const int x = id & 7, s = id >> 3;
    head = s % p.H;
    const int from_end = (s / p.H) * 8 + x;
    if (from_end >= p.nqb) return;
    qb = p.nqb - 1 - from_end;
  }
  const int kvh = head / (p.H / p.Hkv);
  const __bf16* qbase = p.q + (int64_t)head * p.q_sh;
  const __bf16* kbase = p.k + (int64_t)kvh * p.k_sh;
  const __bf16* vbase = p.v + (int64_t)kvh * p.v_sh;

  const int q_row = qb * kBlk + wave * 32 + r;          // this lane's query token
  const int q_pos = q_row + p.kv_off;                   // its position on the key axis
  int n_blocks;
  const int32_t* list = nullptr;
  {
    const int q_last = (qb * kBlk + kBlk - 1 < p.Lq ? qb * kBlk + kBlk - 1 : p.Lq - 1) + p.kv_off;
    int visible = p.causal ? (q_last < 0 ? 0 : q_last / kBlk + 1) : p.nkb;
    visible = visible < p.nkb ? visible : p.nkb;
    if (kHasList) {
      list = p.col_idx + ((int64_t)head * p.idx_rows + qb) * p.idx_pitch;
      n_blocks = p.col_cnt[head * p.idx_rows + qb];
      n_blocks = n_blocks < 0 ? 0 : (n_blocks > p.idx_pitch ? (int)p.idx_pitch : n_blocks);
    } else {
      n_blocks = visible;
    }
  }

  // Q^T fragments stay in registers for the whole sweep.
  bf16x8 qreg[8];
  {
    const int row = q_row < p.Lq ? q_row : p.Lq - 1;
    const __bf16* src = qbase + (int64_t)row * p.q_sn + hh * 8;
#pragma unroll
    for (int s = 0; s < 8; ++s) qreg[s] = *reinterpret_cast<const bf16x8*>(src + s * 16);
  }

  f32x16 oacc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[i][v] = 0.f;
  float m_run = -INFINITY;   // running row maximum, already multiplied by scale_log2
  float l_run = 0.f;         // this lane's share of the running row sum

  u32x4 stage[8];
  int kb = 0;
  if (n_blocks > 0) {
    kb = kHasList ? clamp_block(list[0], p.nkb) : 0;
    load_k_tile(p, kbase, kb, tid, stage);
    store_k_tile(Ks, tid, stage);
    load_v_tile(p, vbase, kb, tid, stage);
  }

  for (int j = 0; j < n_blocks; ++j) {
    const int kb_next = (j + 1 < n_blocks) ? (kHasList ? clamp_block(list[j + 1], p.nkb) : j + 1) : -1;
    __syncthreads();                       // K_j visible in Ks; everyone is done with V_{j-1}
    store_v_tile_t(Vt, tid, stage);
    if (kb_next >= 0) load_k_tile(p, kbase, kb_next, tid, stage);

    // ---- S^T = K_j Q^T : lane owns query row r, key rows 8g + 4hh + t of each 32-row tile
    f32x16 sacc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) sacc[i][v] = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        bf16x8 a = *reinterpret_cast<const bf16x8*>(Ks + (nt * 32 + r) * kLdsRow + s * 16 + hh * 8);
        sacc[nt] = mfma32(a, qreg[s], sacc[nt]);
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

    // ---- online softmax in the exp2 domain
    float mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[nt][v]);
    mx = fmaxf(mx, swap_half(mx));
    const float m_new = fmaxf(m_run, mx * p.scale_log2);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);
    m_run = m_new;
    float psum = 0.f;
    bf16x8 pfrag[8];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float e = fast_exp2(__builtin_fmaf(sacc[nt][v], p.scale_log2, -m_safe));
        psum += e;
        pfrag[nt * 2 + (v >> 3)][v & 7] = (__bf16)e;
      }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[dt][v] *= alpha;

    __syncthreads();                       // V_j^T visible in Vt; everyone is done with K_j
    if (kb_next >= 0) {
      store_k_tile(Ks, tid, stage);
      load_v_tile(p, vbase, kb_next, tid, stage);
    }

    // ---- O^T += V_j^T P^T
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        bf16x8 a = *reinterpret_cast<const bf16x8*>(Vt + (dt * 32 + r) * kLdsRow + ks * 16 + hh * 8);
        oacc[dt] = mfma32(a, pfrag[ks], oacc[dt]);
      }
    kb = kb_next;
  }

  const float l_tot = l_run + swap_half(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (q_row < p.Lq) {
    __bf16* dst = p.o + (int64_t)head * p.o_sh + (int64_t)q_row * p.o_sn + hh * 4;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = pack_bf16(oacc[dt][g * 4 + 0] * inv, oacc[dt][g * 4 + 1] * inv);
        w[1] = pack_bf16(oacc[dt][g * 4 + 2] * inv, oacc[dt][g * 4 + 3] * inv);
        *reinterpret_cast<u32x2*>(dst + dt * 32 + g * 8) = w;
      }
  }
}

}  // namespace xattn

using namespace xattn;

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

extern "C" int xattn_block_sparse_fwd(const void* q, const void* k, const void* v, void* out,
                                      const int32_t* col_idx, const int32_t* col_cnt, int64_t idx_pitch,
                                      int idx_rows, int num_heads, int num_kv_heads, int q_len, int k_len, int head_dim,
                                      int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_h,
                                      int64_t k_stride_n, int64_t v_stride_h, int64_t v_stride_n,
                                      int64_t o_stride_h, int64_t o_stride_n, int causal, float softmax_scale,
                                      void* stream) {
  if (!q || !k || !v || !out) return XATTN_ERR_NULL;
  if (head_dim != kHeadDim) return XATTN_ERR_HEAD_DIM;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads) return XATTN_ERR_HEADS;
  if (q_len <= 0 || k_len <= 0) return XATTN_ERR_SHAPE;
  if ((col_idx == nullptr) != (col_cnt == nullptr)) return XATTN_ERR_NULL;
  const int64_t strides[] = {q_stride_h, q_stride_n, k_stride_h, k_stride_n,
                             v_stride_h, v_stride_n, o_stride_h, o_stride_n};
  for (int64_t s : strides)
    if (s % 8) return XATTN_ERR_ALIGN;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return XATTN_ERR_ALIGN;

  AttnParams p;
  p.q = static_cast<const __bf16*>(q);
  p.k = static_cast<const __bf16*>(k);
  p.v = static_cast<const __bf16*>(v);
  p.o = static_cast<__bf16*>(out);
  p.q_sh = q_stride_h; p.q_sn = q_stride_n; p.k_sh = k_stride_h; p.k_sn = k_stride_n;
  p.v_sh = v_stride_h; p.v_sn = v_stride_n; p.o_sh = o_stride_h; p.o_sn = o_stride_n;
  p.col_idx = col_idx; p.col_cnt = col_cnt; p.idx_pitch = idx_pitch;
  p.H = num_heads; p.Hkv = num_kv_heads; p.Lq = q_len; p.Lk = k_len;
  p.nqb = (q_len + kBlk - 1) / kBlk;
  p.nkb = (k_len + kBlk - 1) / kBlk;
  p.causal = causal ? 1 : 0;
  p.kv_off = k_len - q_len;
  p.scale_log2 = softmax_scale * kLog2e;
  if (col_idx && (idx_pitch < 1 || idx_rows < p.nqb)) return XATTN_ERR_SHAPE;
  p.idx_rows = idx_rows;

  const int64_t grid = (int64_t)p.H * ((p.nqb + 7) / 8) * 8;
  if (grid > 0x7fffffff) return XATTN_ERR_SHAPE;
  if (col_idx)
    hipLaunchKernelGGL(block_sparse_fwd_kernel<true>, dim3((unsigned)grid), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
  else
    hipLaunchKernelGGL(block_sparse_fwd_kernel<false>, dim3((unsigned)grid), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}
