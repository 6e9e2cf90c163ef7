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
// unchanged, the B operand of O^T += V^T P^T.  K and V tiles (128 keys x 128
// features, row-major, XOR-swizzled 16-byte chunks) are copied global -> LDS by
// buffer loads that write LDS directly; keys past the sequence end fall outside
// the buffer resource and arrive as zeros.  K fragments are read with
// ds_read_b128, V^T fragments with the transposing ds_read_b64_tr_b16, both
// issued one k-step ahead of the MFMAs that consume them.  The copy of the next
// K tile overlaps softmax and P.V, the copy of the next V tile overlaps Q.K^T
// (both issued from assembly, see copy_tile_async: the compiler would make the
// transposing reads wait for every copy it knows of).
// Two workgroups fit per CU (64 KiB LDS each) so one's softmax overlaps the
// other's MFMA.  The query block enters and the output block leaves through
// the same LDS tiles as full 256-byte rows (the q-block is copied like a K
// tile before V_0 is requested; the output is staged in the K tile after the
// sweep): row-per-lane accesses to global memory would be hundreds of partial
// line requests per wavefront, and a workgroup keeps its registers and LDS
// until the last of its stores is acknowledged.
#include "attn_tiles.h"
#include "xattn_hip.h"

namespace xattn {

struct AttnParams {
  const __bf16* q;
  const __bf16* k;
  const __bf16* v;
  __bf16* o;
  int64_t q_sh, q_sn, k_sh, k_sn, v_sh, v_sn, o_sh, o_sn;  // element strides (head, token)
  const int32_t* col_idx;   // [H, idx_rows, idx_pitch] ascending k-block ids, or null = all visible
  const int32_t* col_cnt;   // [H, idx_rows]
  int64_t idx_pitch;
  int idx_rows;             // q-block rows per head in col_idx / col_cnt
  int idx_row0;             // q-block held by their row 0
  int H, Hkv, Lq, Lk, nqb, nkb;
  int qb_begin, qb_end;     // q-blocks handled by this launch
  int causal, kv_off;       // kv_off = Lk - Lq
  float scale_log2;         // softmax_scale * log2(e)
  DispatchShape shape;      // dispatch_shape(H, Hkv), computed on the host
};

__device__ __forceinline__ int clamp_block(int kb, int nkb) { return kb < 0 ? 0 : (kb < nkb ? kb : nkb - 1); }

// Per-lane addressing that does not depend on the (head, q-block) being worked on.
struct LaneAddr {
  int voffK[8], voffV[8];   // tile copy: byte offsets of the lane's rows
  int kaddr[8];             // K fragment (k-step s, key tile nt): row nt*32 + r, logical chunk 2s + hh
  int vaddr[4][2];          // V^T fragment (k-step ks, half a, feature tile dt)
};

__device__ __forceinline__ void lane_addressing(const AttnParams& p, int lane, int wave, LaneAddr& a) {
  const int r = lane & 31, hh = lane >> 5;
  tile_offsets(p.k_sn, lane, wave, a.voffK);
  tile_offsets(p.v_sn, lane, wave, a.voffV);
#pragma unroll
  for (int s = 0; s < 8; ++s) a.kaddr[s] = r * 256 + (((2 * s + hh) ^ swz(r)) << 4);
  // the transposing read hands lane l the feature dt*32 + (l % 32) of keys
  // 16ks + 8a + 4hh + {0..3}; as a source lane it points at key e = (l%16)/4 of
  // that quad, features dt*32 + 16*((l/16)%2) + 4*(l%4) .. +3.
  const int e = (lane & 15) >> 2, j = lane & 3, g2 = (lane >> 4) & 1;
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      const int row = 8 * h2 + 4 * hh + e;                       // + 16*ks
      const int c = dt * 4 + 2 * g2 + (j >> 1);
      a.vaddr[dt][h2] = row * 256 + ((c ^ swz(row)) << 4) + (j & 1) * 8;
    }
}

// S^T = K_j Q^T : lane owns query row r, key rows 8g + 4hh + t of each 32-row tile
__device__ __forceinline__ void qk_tile(const char* Ks, const int (&kaddr)[8], const bf16x8 (&qreg)[8], f32x16 (&sacc)[4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) sacc[i][v] = 0.f;
  bf16x8 kf[2][4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) kf[0][nt] = *reinterpret_cast<const bf16x8*>(Ks + kaddr[0] + nt * 8192);
  __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    if (s < 7) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
        kf[(s + 1) & 1][nt] = *reinterpret_cast<const bf16x8*>(Ks + kaddr[s + 1] + nt * 8192);
    }
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) sacc[nt] = mfma32(kf[s & 1][nt], qreg[s], sacc[nt]);
    if (s < 7) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
    } else {
      __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
    }
  }
}

// Online softmax in the exp2 domain on the scores of one tile; leaves the bf16
// probabilities in pfrag (already in the B-operand layout of O^T += V^T P^T).
// The reference maximum m_run is only moved when a row's maximum outgrows it
// by more than 2^8 (or on the row's first visible key): exp2 arguments then
// stay <= 8, which fp32 sums and bf16 probabilities hold without loss, and
// the rescaling of l and of the 64 output accumulators is skipped for the
// wavefront whenever no row needs it.  O / l does not depend on the choice.
__device__ __forceinline__ void softmax_tile(f32x16 (&sacc)[4], f32x16 (&oacc)[4], float& m_run, float& l_run,
                                             float scale_log2, bf16x8 (&pfrag)[8]) {
  float mx = -INFINITY;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[nt][v]);
  mx = half_max(mx) * scale_log2;
  const bool move = mx > m_run + 8.f || (m_run == -INFINITY && mx > -INFINITY);
  if (__any(move)) {
    const float m_new = move ? mx : m_run;
    const float alpha = (m_new == -INFINITY) ? 1.f : fast_exp2(m_run - m_new);
    m_run = m_new;
    l_run *= alpha;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[dt][v] *= alpha;
  }
  const float m_safe = (m_run == -INFINITY) ? 0.f : m_run;
  float psum = 0.f;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float e = fast_exp2(__builtin_fmaf(sacc[nt][v], scale_log2, -m_safe));
      psum += e;
      pfrag[nt * 2 + (v >> 3)][v & 7] = (__bf16)e;
    }
  l_run += psum;
}

// O^T += V_j^T P^T
__device__ __forceinline__ void pv_tile(const char* Vs, const int (&vaddr)[4][2], const bf16x8 (&pfrag)[8], f32x16 (&oacc)[4]) {
  i16x4 vf[2][4][2];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int a = 0; a < 2; ++a)
      vf[0][dt][a] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) i16x4*)(Vs + vaddr[dt][a]));
  __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    if (ks < 7) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int a = 0; a < 2; ++a)
          vf[(ks + 1) & 1][dt][a] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) i16x4*)(Vs + vaddr[dt][a] + (ks + 1) * 4096));
    }
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      typedef __attribute__((__vector_size__(8 * sizeof(short)))) short i16x8;
      i16x8 av;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        av[u] = vf[ks & 1][dt][0][u];
        av[4 + u] = vf[ks & 1][dt][1][u];
      }
      oacc[dt] = mfma32(__builtin_bit_cast(bf16x8, av), pfrag[ks], oacc[dt]);
    }
    if (ks < 7) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
    } else {
      __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
    }
  }
}

// token-level masking of one tile's scores: keys past the sequence end, and (causal) keys after the query.
// The lane's last visible key is taken relative to its first key of the tile once, so that each score costs one
// compare against a constant and one select.
__device__ __forceinline__ void mask_tile(f32x16 (&sacc)[4], int kb, int hh, int q_pos, int Lk, int causal) {
  int last = Lk - 1;
  if (causal) last = last < q_pos ? last : q_pos;
  const int lim = last - kb * kBlk - hh * 4;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int c = nt * 32 + (v >> 2) * 8 + (v & 3);     // key offset inside the tile, without the lane's hh * 4
      sacc[nt][v] = c > lim ? -INFINITY : sacc[nt][v];
    }
}

// Normalises this wavefront's 32 output rows and stores them through LDS.  Lane (r, hh) holds half of row r in
// 8-byte pieces; written straight to memory those are 512 sixteen-byte requests per wavefront, and a
// workgroup's registers and LDS stay allocated until its last store is acknowledged - on lists of a few blocks
// that wait was a quarter of a workgroup's life.  Staged through the wavefront's own 8 KiB of the K tile
// (free once the sweep is over), 16 lanes write one 256-byte row: 64 full-line requests.
__device__ __forceinline__ void store_out(const AttnParams& p, int head, int qb, int wave, int lane, int r, int hh,
                                          const f32x16 (&oacc)[4], float l_run, char* stage) {
  const float l_tot = half_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      u32x2 w;
      w[0] = pack_bf16(oacc[dt][g * 4 + 0] * inv, oacc[dt][g * 4 + 1] * inv);
      w[1] = pack_bf16(oacc[dt][g * 4 + 2] * inv, oacc[dt][g * 4 + 3] * inv);
      const int c = dt * 4 + g;                          // 16-byte chunk of the row; XOR-swizzled against bank conflicts
      *reinterpret_cast<u32x2*>(stage + r * 256 + ((c ^ (r & 15)) << 4) + hh * 8) = w;
    }
  // written and read by the same wavefront: the LDS keeps a wavefront's accesses in order, no barrier.
  // The rows leave through a buffer resource that ends with the sequence (rows past it are dropped), rebased to
  // the q-block so that a lane's offset is one 32-bit product plus a multiple of four rows.
  const int rows_left = p.Lq - qb * kBlk;
  const int rows = rows_left < kBlk ? rows_left : kBlk;
  const __amdgpu_buffer_rsrc_t ores = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(p.o + (int64_t)head * p.o_sh + (int64_t)qb * kBlk * p.o_sn), 0, (int)((int64_t)rows * p.o_sn * 2), 0x00020000);
  const int c = lane & 15;
  const uint32_t row_bytes = (uint32_t)p.o_sn * 2u;
  const uint32_t voff0 = (uint32_t)(wave * 32 + (lane >> 4)) * row_bytes + (uint32_t)c * 16u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = i * 4 + (lane >> 4);
    const u32x4 w = *reinterpret_cast<const u32x4*>(stage + row * 256 + ((c ^ (row & 15)) << 4));
    __builtin_amdgcn_raw_buffer_store_b128(w, ores, (int)(voff0 + (uint32_t)(i * 4) * row_bytes), 0, 0);
  }
}

typedef const __attribute__((address_space(4))) int32_t* const_i32_ptr;

// kHasList = false is the dense baseline (its own symbol, so profiles tell the two apart)
template <bool kHasList>
__global__ __launch_bounds__(256, 2) void block_sparse_fwd_kernel(AttnParams p) {
  __shared__ __attribute__((aligned(1024))) char Ks[kTileBytes];
  __shared__ __attribute__((aligned(1024))) char Vs[kTileBytes];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, hh = lane >> 5;

  int head, qb, kvh;
  if (!map_workgroup(blockIdx.x, p.shape, p.qb_begin, p.qb_end, &head, &qb, &kvh)) return;
  const __bf16* qbase = p.q + (int64_t)head * p.q_sh;
  const __bf16* kbase = p.k + (int64_t)kvh * p.k_sh;
  const __bf16* vbase = p.v + (int64_t)kvh * p.v_sh;

  const int q_row = qb * kBlk + wave * 32 + r;          // this lane's query token
  const int q_pos = q_row + p.kv_off;                   // its position on the key axis
  int n_blocks, first = 0;
  // the column list is read through the scalar cache (uniform, read-only), so that
  // fetching the next block id never waits on the tile copies in flight
  const_i32_ptr list = nullptr;
  {
    const int q_last = (qb * kBlk + kBlk - 1 < p.Lq ? qb * kBlk + kBlk - 1 : p.Lq - 1) + p.kv_off;
    int visible = p.causal ? (q_last < 0 ? 0 : q_last / kBlk + 1) : p.nkb;
    visible = visible < p.nkb ? visible : p.nkb;
    if (kHasList) {
      const int64_t slot = (int64_t)head * p.idx_rows + (qb - p.idx_row0);
      list = (const_i32_ptr)(uintptr_t)(p.col_idx + slot * p.idx_pitch);
      n_blocks = ((const_i32_ptr)(uintptr_t)p.col_cnt)[slot];
      first = list[0];                     // idx_pitch >= 1: readable whatever the count
      n_blocks = n_blocks < 0 ? 0 : (n_blocks > p.idx_pitch ? (int)p.idx_pitch : n_blocks);
    } else {
      n_blocks = visible;
    }
  }

  bf16x8 qreg[8];   // Q^T fragments stay in registers for the whole sweep
  LaneAddr la;
  lane_addressing(p, lane, wave, la);

  f32x16 oacc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[i][v] = 0.f;
  float m_run = -INFINITY;   // running row maximum, already multiplied by scale_log2
  float l_run = 0.f;         // this lane's share of the running row sum

  int kb = 0;
  {
    // The q-block is a tile like any other: copied row-wise (full lines) into the V tile, where each wavefront's
    // eighth-of-a-tile copies are its own 32 query rows, and read back as fragments before V_0 is requested.
    int voffQ[8];
    tile_offsets(p.q_sn, lane, wave, voffQ);
    copy_tile(qbase, p.q_sn, p.Lq, qb, voffQ, Vs, wave);
    if (n_blocks > 0) {
      kb = kHasList ? clamp_block(first, p.nkb) : 0;
      copy_tile(kbase, p.k_sn, p.Lk, kb, la.voffK, Ks, wave);
    }
    wait_vm0();
#pragma unroll
    for (int s = 0; s < 8; ++s) qreg[s] = *reinterpret_cast<const bf16x8*>(Vs + wave * 8192 + la.kaddr[s]);
    __builtin_amdgcn_s_waitcnt(0xC07F);      // the fragments are in registers before V_0 may overwrite them
    asm volatile("" ::: "memory");
    if (n_blocks > 0) copy_tile_async(vbase, p.v_sn, p.Lk, kb, la.voffV, Vs, wave);
  }
  // K_0 landed before the fragments were read (every wavefront waited for its share); V_0 stays in flight during
  // the first Q.K^T and is waited for with the tile's own barrier
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  for (int j = 0; j < n_blocks; ++j) {
    const int kb_next = (j + 1 < n_blocks) ? (kHasList ? clamp_block(list[j + 1], p.nkb) : j + 1) : -1;
    f32x16 sacc[4];
    qk_tile(Ks, la.kaddr, qreg, sacc);
    wait_vm0();
    __syncthreads();                       // everyone is done with K_j; V_j landed and visible
    if (kb_next >= 0) copy_tile_async(kbase, p.k_sn, p.Lk, kb_next, la.voffK, Ks, wave);

    const bool need_mask = (kb * kBlk + kBlk > p.Lk) || (p.causal && kb * kBlk + kBlk - 1 > qb * kBlk + p.kv_off);
    if (need_mask) mask_tile(sacc, kb, hh, q_pos, p.Lk, p.causal);
    bf16x8 pfrag[8];
    softmax_tile(sacc, oacc, m_run, l_run, p.scale_log2, pfrag);
    pv_tile(Vs, la.vaddr, pfrag, oacc);
    wait_vm0();
    __syncthreads();                       // everyone is done with V_j; K_{j+1} landed and visible
    if (kb_next >= 0) copy_tile_async(vbase, p.v_sn, p.Lk, kb_next, la.voffV, Vs, wave);
    kb = kb_next;
  }
  // the last barrier of the sweep (or the one before it, for an empty list) left both tiles unused
  store_out(p, head, qb, wave, lane, r, hh, oacc, l_run, Ks + wave * 8192);
}

}  // namespace xattn

using namespace xattn;

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

extern "C" int xattn_block_sparse_fwd(const void* q, const void* k, const void* v, void* out,
                                      const int32_t* col_idx, const int32_t* col_cnt, int64_t idx_pitch,
                                      int idx_rows, int idx_row0, int num_heads, int num_kv_heads, int q_len, int k_len,
                                      int head_dim,
                                      int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_h,
                                      int64_t k_stride_n, int64_t v_stride_h, int64_t v_stride_n,
                                      int64_t o_stride_h, int64_t o_stride_n, int q_block_begin, int q_block_end,
                                      int causal, float softmax_scale, void* stream) {
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
  if (!tile_stride_ok(k_stride_n) || !tile_stride_ok(v_stride_n) || !tile_stride_ok(q_stride_n) || !tile_stride_ok(o_stride_n))
    return XATTN_ERR_SHAPE;
  if (!scale_ok(softmax_scale)) return XATTN_ERR_SHAPE;

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
  if (q_block_end < 0) q_block_end = p.nqb;
  if (q_block_begin < 0 || q_block_begin >= q_block_end || q_block_end > p.nqb) return XATTN_ERR_SHAPE;
  // the lists may hold a window of q-block rows only; the q-blocks of this launch must lie inside it
  if (col_idx && (idx_pitch < 1 || idx_row0 < 0 || q_block_begin < idx_row0 || q_block_end > idx_row0 + idx_rows))
    return XATTN_ERR_SHAPE;
  p.idx_rows = idx_rows;
  p.idx_row0 = idx_row0;
  p.qb_begin = q_block_begin;
  p.qb_end = q_block_end;
  p.shape = dispatch_shape(p.H, p.Hkv);
  const int64_t grid = grid_for(p.H, p.Hkv, q_block_end - q_block_begin);
  if (grid > 0x7fffffff) return XATTN_ERR_SHAPE;
  if (col_idx)
    hipLaunchKernelGGL(block_sparse_fwd_kernel<true>, dim3((unsigned)grid), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
  else
    hipLaunchKernelGGL(block_sparse_fwd_kernel<false>, dim3((unsigned)grid), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p);
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}
