// Antidiagonal block-score estimator for gfx950.
//
// Fuses what the reference does with two Triton kernels and an HBM round trip
// of the strided score matrix (flat_group_gemm_fuse_reshape,
// xattn/src/kernels.py:197-235, then softmax_fuse_block_sum, :5-156; driven by
// xattn/src/Xattention.py:138-172):
//
//  kernel 1 (estimate_gemm_kernel): a bf16 MFMA GEMM over the reshaped
//    operands, gathered on the fly - reshaped key n at depth slab i is token
//    n*S+i, reshaped query m is token m*S+S-1-i - with a 256x256 tile per
//    workgroup of eight wavefronts, 128 keys x 64 query rows each.  Scores are produced transposed
//    (keys along accumulator rows) so one lane owns one query row.  In the
//    epilogue each wavefront scales, masks, takes the row maximum over ITS 128
//    keys, exponentiates against that local maximum and adds up groups of
//    block_size/S keys.  It writes, per (query row, 128-key tile), the local
//    maximum and sum, and per (query row, key block) the partial sum - 1/S of
//    the score matrix, in fp32 - never the scores themselves.  One workgroup
//    per CU works through its share of the tiles with the slab pipeline
//    (global -> registers -> LDS, two k-steps deep) running on across tile
//    boundaries.
//  kernel 2 (estimate_normalize_kernel): per query row, combines the tile
//    maxima/sums into the row's softmax statistics, rescales the partial sums
//    and adds the block_size/S rows of each query block.
#include <mutex>

#include "select_row.h"
#include "xattn_hip.h"

namespace xattn {

constexpr int kTile = 256;       // workgroup tile edge (reshaped rows / keys)
constexpr int kSub = 128;        // keys per wavefront tile (and per softmax tile)
constexpr int kRowsW = 64;       // reshaped query rows per wavefront tile
constexpr int kWaves = 8;        // wavefronts per workgroup: 2 key halves x 4 query quarters
constexpr int kDepth = 64;       // bf16 per k-step (one 128-byte line per row)
constexpr int kStageBytes = 2 * kTile * kDepth * 2;  // K' + Q' slabs of one stage

struct EstParams {
  const __bf16* q;
  const __bf16* k;
  int64_t q_sh, q_sn, k_sh, k_sn;
  float* P;        // [H][nkb][rows]  partial block sums relative to the tile maximum
  float* Mt;       // [H][nT][rows]   tile maximum (exp2 domain)
  float* Lt;       // [H][nT][rows]   tile sum
  float* scores;   // optional [H][n_rq][n_rk] raw scores
  float* sums;     // output block sums: [H][win_rows][nkb], q-block row i stored at row i - win_row0
  int win_row0, win_rows;
  int H, Hkv, Lq, Lk, S, rbs;
  int n_rq, n_rk, nkb, nqb, nT;
  int rcs;                  // reshaped keys per chunk
  int kdb;                  // query-row subsampling: query row m stands for reshaped row m * kdb
  int rcs_q, rbs_q;         // query rows per chunk / per query block (rcs / kdb, rbs / kdb)
  int row_begin, row_end;   // query rows handled by this call
  int rows;                 // row_end - row_begin (pitch of P / Mt / Lt)
  int off;                  // position of reshaped row 0 on the key axis: n_rk - n_rq * kdb
  int real_rows;            // query rows >= real_rows give all-zero block sums
  int causal, own_chunk_only;
  int no_softmax;           // block sums of exp(scaled score) instead of softmax probabilities
  float scale_log2;
  // Depth slabs of the reshaped GEMM.  Slab j multiplies query token
  // m*S + (pairs[j] >> 4) with key token n*S + (pairs[j] & 15); n_pairs = 0 means
  // the S pairs (S-1-i, i) of the antidiagonal reshape, in closed form.
  int n_pairs;
  uint8_t pairs[64];
  int nMT, nNT;             // tile rows over [row_begin, row_end) / tile columns over n_rk
  int tiles_per_head;       // tiles with a visible pair, per head
  int64_t total_tiles;      // tiles_per_head * H
};

// first / last visible reshaped key of reshaped query row m
// (with kdb > 1 the row's causal limit is that of the LAST reshaped row of its
// group, xattn/src/Xattention.py:217-222, while its tokens are those of the first, :88-93)
__host__ __device__ inline int row_lo(const EstParams& p, int m) {
  return (p.causal && p.own_chunk_only) ? (m / p.rcs_q) * p.rcs + p.off : 0;
}
__host__ __device__ inline int row_hi(const EstParams& p, int m) {
  return p.causal ? m * p.kdb + p.kdb - 1 + p.off : p.n_rk - 1;
}

// A k-step slab is 256 rows x 64 bf16 (one 128-byte line per row) per operand.
// It travels global -> registers -> LDS: each wavefront instruction loads
// 64 x 16 bytes = 8 rows (full lines) and later writes them as one contiguous
// KiB.  Loads are issued two k-steps ahead of their use and written to LDS one
// step ahead, so a load has a whole step to arrive and no barrier waits for
// memory.  (Buffer loads that write LDS directly save the registers, but had
// to be issued at most one step ahead - the stage they fill must be free -
// and the kernel then ran 4-8 % slower.)  Tokens past the real length fall
// outside the buffer resource and arrive as zeros - the zero padding of
// xattn/src/Xattention.py:33-51.
//
// LDS slab layout: row r at byte r*128; its 16-byte chunk c sits at position
// c ^ ((r >> 1) & 7), so the 16 lanes of one ds_read_b128 pass - the same
// logical chunk of 16 consecutive rows - touch each of the 64 banks once.  The
// swizzle is applied on the global side of the copy (the lane that fills
// position c fetches chunk c ^ ((r >> 1) & 7)).

// Per-lane byte offsets (relative to the tile's first token) of the 8 rows a
// lane copies per slab, for token 0 of each reshaped row's group and feature 0;
// the k-step adds a uniform term.  The host checks that a tile spans < 2^31 bytes.
__device__ __forceinline__ void slab_offsets(int64_t sn_bytes, int S, int lane, int wave, int (&voff)[4]) {
  const int c = lane & 7, rl = lane >> 3;
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int r = it * 64 + wave * 8 + rl;
    voff[it] = (int)((int64_t)r * S * sn_bytes) + ((c ^ ((r >> 1) & 7)) << 4);
  }
}

__device__ __forceinline__ bf16x8 read_frag(const char* slab, int row, int chunk) {
  return *reinterpret_cast<const bf16x8*>(slab + row * 128 + ((chunk ^ ((row >> 1) & 7)) << 4));
}


// Tile assignment.  Only tiles holding a visible (row, key) pair are
// enumerated: per KV group, by query tile row, then key tile, then query head
// of the group.  Tile ids are dealt round-robin to the 8 XCDs (workgroup b
// runs on XCD b % 8 and takes ids b, b + grid, ... with the grid a multiple of
// 8), so runs of 32 consecutive tiles are given to one XCD: the 32 tiles an XCD
// works on at a time are then 8 key tiles x the heads of one group for one
// query tile row, which share their K' slabs across heads and their Q' slabs
// across key tiles in that XCD's L2, and every XCD gets the same number of tiles.
// Returns false when id is past the last tile.
//
// A workgroup visits its tiles in increasing order, so the search for a tile's query-tile row resumes from the
// row of the previous tile (TileCursor) instead of walking all rows again: between two tiles of a workgroup the
// matrix pipes have nothing to do, and a walk over 32 rows with their visibility limits was 6 % of a tile's time.
struct TileCursor {
  int g = -1;          // KV group of the previous tile
  int mt_row = 0;      // its query-tile row
  int row_base = 0;    // (row, key tile) pairs of the group before that row
};

__device__ __forceinline__ bool decode_tile(const EstParams& p, int64_t id, TileCursor& c, int* head, int* m0, int* n0) {
  const int64_t lin64 = ((id >> 8) * 8 + (id & 7)) * 32 + ((id >> 3) & 31);
  if (lin64 >= p.total_tiles) return false;
  const uint32_t lin = (uint32_t)lin64;                  // the host refuses launches of 2^31 tiles or more
  const uint32_t G = (uint32_t)(p.H / p.Hkv);
  const uint32_t per_group = (uint32_t)p.tiles_per_head * G;
  const uint32_t g = lin / per_group;
  const uint32_t rem = lin - g * per_group;
  *head = (int)(g * G + rem % G);
  const int tt = (int)(rem / G);                          // the tile among the group's (row, key tile) pairs
  if ((int)g != c.g) {
    c.g = (int)g;
    c.mt_row = 0;
    c.row_base = 0;
  }
  int nt_first = 0;
  for (;;) {
    const int mfirst = p.row_begin + c.mt_row * kTile;
    const int mlast = (mfirst + kTile - 1 < p.row_end ? mfirst + kTile - 1 : p.row_end - 1);
    int hi = row_hi(p, mlast) / kTile;
    hi = hi < p.nNT - 1 ? hi : p.nNT - 1;
    nt_first = row_lo(p, mfirst) / kTile;
    const int cnt = hi - nt_first + 1;
    if (tt < c.row_base + cnt || c.mt_row + 1 >= p.nMT) break;
    c.row_base += cnt;
    ++c.mt_row;
  }
  *m0 = p.row_begin + c.mt_row * kTile;
  *n0 = (nt_first + (tt - c.row_base)) * kTile;
  return true;
}

// kDump: also write the raw scores (test / seam builds only; kept out of the production instantiation)
// kTable: the depth slabs come from p.pairs (the non-default select modes); the default keeps its closed form
template <int RBS, bool kDump, bool kTable>
__global__ __launch_bounds__(512) void estimate_gemm_kernel(EstParams p) {
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, hh = lane >> 5;
  const int wm = wave & 3, wn = wave >> 2;   // query quarter, key half
  // A workgroup works through tiles id, id + grid, ...: one workgroup fits a CU, so nothing else could hide
  // the wait for a tile's first slabs.  The slab pipeline therefore runs on across the tile boundary: the load
  // slots of a tile's last two k-steps fetch the first slabs of the NEXT tile, and the last sub-step reads its
  // first fragments, so after the epilogue (which needs no LDS) the next tile starts at full speed.
  int64_t id = blockIdx.x;
  int head, m0, n0;
  TileCursor cursor;
  if (!decode_tile(p, id, cursor, &head, &m0, &n0)) return;

  const int64_t q_snb = p.q_sn * 2, k_snb = p.k_sn * 2;
  const int64_t span = (int64_t)kTile * p.S;
  // Buffer resources are rebased to the tile's first token and end at the real
  // sequence end (or the tile's end), so lane offsets stay small whatever the
  // token stride, and tokens past the real length read as zeros.
  auto q_resource = [&](int h, int m) {
    const int64_t tok0 = (int64_t)m * p.S * p.kdb, left = p.Lq - tok0;
    const int64_t rows = left < 0 ? 0 : (left < span * p.kdb ? left : span * p.kdb);
    return __builtin_amdgcn_make_buffer_rsrc((void*)(p.q + (int64_t)h * p.q_sh + (rows > 0 ? tok0 * p.q_sn : 0)), 0,
                                             (int)(rows * q_snb), 0x00020000);
  };
  auto k_resource = [&](int h, int n) {
    const int64_t tok0 = (int64_t)n * p.S, left = p.Lk - tok0;
    const int64_t rows = left < 0 ? 0 : (left < span ? left : span);
    return __builtin_amdgcn_make_buffer_rsrc((void*)(p.k + (int64_t)(h / (p.H / p.Hkv)) * p.k_sh + (rows > 0 ? tok0 * p.k_sn : 0)),
                                             0, (int)(rows * k_snb), 0x00020000);
  };
  __amdgpu_buffer_rsrc_t qres = q_resource(head, m0), kres = k_resource(head, n0);
  __amdgpu_buffer_rsrc_t qres_next = qres, kres_next = kres;

  // k-step t covers token i = t / 2 of every reshaped row's group, features
  // 64*(t % 2) .. +63, and is read from LDS stage t % 2.
  //
  // Software pipeline.  A step is four sub-steps of 8 MFMAs per wavefront; the 6
  // fragment reads of the next sub-step and up to 3 of the 8 slab pieces (an LDS
  // write of the next step's piece, then the load of the piece two steps on
  // into the same registers) are issued between them, in chunks the scheduler
  // may not mix (one piece, two reads, two MFMAs), so that neither pieces nor
  // reads bunch up in front of the MFMAs.  Two wavefronts share a SIMD: while
  // one waits at the barrier or on a fragment the other keeps the matrix pipe
  // fed.  The workgroup barrier sits before the LAST sub-step's MFMAs: at that
  // point every fragment of the current stage has been read and every piece of
  // the next stage written, so the sub-step can prefetch the next stage's first
  // fragments while its MFMAs run.
  const int steps = (kTable ? p.n_pairs : p.S) * 2;
  int voffK[4], voffQ[4];
  slab_offsets(k_snb, p.S, lane, wave, voffK);
  slab_offsets(q_snb, p.S * p.kdb, lane, wave, voffQ);
  auto step_off_k = [&](int t) {
    const int i = kTable ? (p.pairs[t >> 1] & 15) : (t >> 1);
    return i * (int)k_snb + (t & 1) * kDepth * 2;
  };
  auto step_off_q = [&](int t) {
    const int i = kTable ? (p.pairs[t >> 1] >> 4) : (p.S - 1 - (t >> 1));
    return i * (int)q_snb + (t & 1) * kDepth * 2;
  };
  // Piece j (0..7) of k-step t: slab rows it = j / 2 of K' (j even) or Q' (j odd), 8 rows per wavefront.  It is
  // loaded into R[j] during step t - 2 and written to LDS stage t % 2 during step t - 1.  Steps `steps` and
  // `steps + 1` are steps 0 and 1 of the next tile (of this tile again when it is the workgroup's last: a harmless
  // repeat nobody reads).
  u32x4 R[8];
  auto load_j = [&](int j, int t) __attribute__((always_inline)) {
    const bool ahead = t >= steps;
    const int tc = ahead ? t - steps : t;
    if (j & 1)
      R[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(
          ahead ? qres_next : qres, (int)((unsigned)voffQ[j >> 1] + (unsigned)step_off_q(tc)), 0, 0));
    else
      R[j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(
          ahead ? kres_next : kres, (int)((unsigned)voffK[j >> 1] + (unsigned)step_off_k(tc)), 0, 0));
  };
  const int lane_dst = wave * 8 * 128 + lane * 16;
  auto write_j = [&](int j, char* stage) __attribute__((always_inline)) {
    *reinterpret_cast<u32x4*>(stage + (j & 1) * kTile * 128 + (j >> 1) * 64 * 128 + lane_dst) = R[j];
  };
  // Workgroup barrier that waits for this wavefront's LDS accesses only: the loads in flight into R must not be
  // drained here (a __syncthreads() would wait for them).
  auto lds_barrier = [&]() __attribute__((always_inline)) {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  };
  // the workgroup's first tile: step 0 into stage 0, step 1 into the registers, then its first fragments
#pragma unroll
  for (int j = 0; j < 8; ++j) load_j(j, 0);
#pragma unroll
  for (int j = 0; j < 8; ++j) write_j(j, lds);
#pragma unroll
  for (int j = 0; j < 8; ++j) load_j(j, 1);
  lds_barrier();
  bf16x8 fa[2][4], fb[2][2];
#pragma unroll
  for (int x = 0; x < 4; ++x) fa[0][x] = read_frag(lds, wn * kSub + x * 32 + r, hh);
#pragma unroll
  for (int x = 0; x < 2; ++x) fb[0][x] = read_frag(lds + kTile * 128, wm * kRowsW + x * 32 + r, hh);

  for (;;) {
  const int64_t id_next = id + gridDim.x;
  int head_next, m0_next, n0_next;
  const bool more = decode_tile(p, id_next, cursor, &head_next, &m0_next, &n0_next);
  if (more) {
    qres_next = q_resource(head_next, m0_next);
    kres_next = k_resource(head_next, n0_next);
  }
  f32x16 acc[4][2];   // [key tile nt][query tile mt]
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  for (int t = 0; t < steps; ++t) {
    char* cur = lds + (t & 1) * kStageBytes;
    char* nxt = lds + ((t + 1) & 1) * kStageBytes;
#pragma unroll
    for (int ss = 0; ss < 4; ++ss) {
      if (ss == 3) {
        // every piece of step t+1 has been written to the other stage; every wavefront has read its last
        // fragment of step t (the reads were issued during sub-step 2)
        __builtin_amdgcn_sched_barrier(0);
        lds_barrier();
      }
      const char* fragK = ss < 3 ? cur : nxt;             // where the next sub-step's fragments live
      const char* fragQ = fragK + kTile * 128;
      const int nss = (ss + 1) & 3;                        // its sub-step index within that stage
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        __builtin_amdgcn_sched_barrier(0);
        {
          // pieces 0..2 | 3..5 | 6..7 of step t+1 go to the other stage; their registers then take step t+2
          const int j = ss * 3 + c;
          if (ss < 3 && c < 3 && j < 8) {
            write_j(j, nxt);
            load_j(j, t + 2);
          }
        }
        if (c < 2) {
          fa[(ss + 1) & 1][2 * c] = read_frag(fragK, wn * kSub + (2 * c) * 32 + r, nss * 2 + hh);
          fa[(ss + 1) & 1][2 * c + 1] = read_frag(fragK, wn * kSub + (2 * c + 1) * 32 + r, nss * 2 + hh);
        } else if (c == 2) {
          fb[(ss + 1) & 1][0] = read_frag(fragQ, wm * kRowsW + r, nss * 2 + hh);
          fb[(ss + 1) & 1][1] = read_frag(fragQ, wm * kRowsW + 32 + r, nss * 2 + hh);
        }
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) acc[c][mt] = mfma32(fa[ss & 1][c], fb[ss & 1][mt], acc[c][mt]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // fa[0] / fb[0] now hold the first fragments of the next tile, whose step 0 sits in stage 0 and whose step 1
  // is on its way into stage 1

  // ---- epilogue: this wavefront's 128 keys x 64 query rows
  const int nbase = n0 + wn * kSub;       // first key of the wavefront tile
  const int T = nbase / kSub;
  if (nbase < p.n_rk) {
  float* Pst = p.P + (int64_t)head * p.nkb * p.rows;
  float* Mst = p.Mt + ((int64_t)head * p.nT + T) * p.rows;
  float* Lst = p.Lt + ((int64_t)head * p.nT + T) * p.rows;
  // every key of this wavefront tile visible to every one of its query rows?
  // (true away from the diagonal and the sequence end: no per-element masking)
  const int mw0 = m0 + wm * kRowsW;
  const bool all_visible = nbase + kSub <= p.n_rk && nbase + kSub - 1 <= row_hi(p, mw0) &&
                           nbase >= row_lo(p, mw0 + kRowsW - 1);
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
    const int m = m0 + wm * kRowsW + mt * 32 + r;
    const bool row_ok = m < p.row_end;
    const int lo = row_lo(p, m), hi = row_hi(p, m);
    if (kDump && row_ok) {
      float* dst = p.scores + ((int64_t)head * p.n_rq + m) * p.n_rk;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int n = nbase + nt * 32 + (v >> 2) * 8 + hh * 4 + (v & 3);
          if (n < p.n_rk) dst[n] = acc[nt][mt][v];
        }
    }
    // Tiles on the diagonal or at the sequence end first overwrite the scores of invisible keys with -inf: they
    // then drop out of the maximum and exponentiate to zero, and the two passes below need neither a test per
    // score nor a second copy.
    if (!all_visible) {
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int n = nbase + nt * 32 + (v >> 2) * 8 + hh * 4 + (v & 3);
          const bool vis = n >= lo && n <= hi && n < p.n_rk;
          acc[nt][mt][v] = vis ? acc[nt][mt][v] : -INFINITY;
        }
    }
    // pass 1: row maximum over this tile's visible keys (exp2 domain)
    float mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int v = 0; v < 16; ++v) mx = fmaxf(mx, acc[nt][mt][v]);
    mx *= p.scale_log2;   // scale > 0
    mx = half_max(mx);
    const float safe = (mx == -INFINITY) ? 0.f : mx;
    float tot = 0.f;
    const int mrel = m - p.row_begin;
    constexpr int G = RBS / 8;   // 8-key groups (one per accumulator quad pair) per key block
    // what the stores below share: the first key block of this wavefront tile and how many of its key blocks
    // exist (uniform), the row of P they start from (uniform) and each half-wave's predicate
    const int kb_first = (int)((uint32_t)nbase / (uint32_t)RBS);
    const int kb_left = p.nkb - kb_first;
    float* const prow = Pst + (int64_t)kb_first * p.rows + mrel;
    const int64_t rows64 = p.rows;
    const bool st0 = row_ok && hh == 0, st1 = row_ok && hh == 1;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      float s[4];       // this lane's share of the sums over keys nbase + nt*32 + 8g .. +7 (the other half-wave has the rest)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        s[g] = 0.f;
#pragma unroll
        for (int t2 = 0; t2 < 4; ++t2) {
          const int v = g * 4 + t2;
          s[g] += fast_exp2(__builtin_fmaf(acc[nt][mt][v], p.scale_log2, -safe));
        }
      }
      // Key blocks go out in pairs: one swap leaves the first block's sum in the lower half-wave and the second
      // block's in the upper one, which are the lanes that store them.  tot adds up what a lane stores; the two
      // half-waves are combined once at the end.
      if (G == 1) {
#pragma unroll
        for (int q2 = 0; q2 < 2; ++q2) {
          const float both = half_sum_pair(s[2 * q2], s[2 * q2 + 1]);
          tot += both;
          const int k = nt * 4 + 2 * q2;
          if (k < kb_left && st0) prow[k * rows64] = both;
          if (k + 1 < kb_left && st1) prow[(k + 1) * rows64] = both;
        }
      } else if (G == 2) {
        const float both = half_sum_pair(s[0] + s[1], s[2] + s[3]);
        tot += both;
        const int k = nt * 2;
        if (k < kb_left && st0) prow[k * rows64] = both;
        if (k + 1 < kb_left && st1) prow[(k + 1) * rows64] = both;
      } else {
        const float all = half_sum(s[0] + s[1] + s[2] + s[3]);
        tot += hh == 0 ? all : 0.f;
        if (nt < kb_left && st0) prow[nt * rows64] = all;
      }
    }
    tot = half_sum(tot);
    if (row_ok && hh == 0) {
      Mst[mrel] = mx;
      Lst[mrel] = tot;
    }
    // keep the query-tile passes apart: interleaving them only lengthens live ranges
    __builtin_amdgcn_sched_barrier(0);
  }
  }   // epilogue

  if (!more) break;
  id = id_next;
  head = head_next;
  m0 = m0_next;
  n0 = n0_next;
  qres = qres_next;
  kres = kres_next;
  }   // tiles of this workgroup
}

// The arithmetic of the normalisation, shared by the stand-alone pass and the fused normalise-and-select kernel
// so that both give the same bits (fixed operation order, no contraction into fused multiply-adds).
#pragma clang fp contract(off)
// folds tile T's maximum / sum into a running (M, L)
__device__ __forceinline__ void stat_step(float& M, float& L, float mt, float lt) {
  const float Mn = fmaxf(M, mt);
  const float safe = (Mn == -INFINITY) ? 0.f : Mn;
  L = L * fast_exp2(M - safe) + lt * fast_exp2(mt - safe);
  M = Mn;
}
// combines the four partial (M, L) of a row (tiles T = first + w, + 4, ... for w = 0..3) into the row's
// maximum (0 when the row sees nothing, or without softmax) and 1 / sum (0 for rows that give zeros)
__device__ __forceinline__ void stat_combine(const float (&Mw)[4], const float (&Lw)[4], bool real_row, int no_softmax,
                                             float* rowM, float* rowInv) {
  const float Mr = fmaxf(fmaxf(Mw[0], Mw[1]), fmaxf(Mw[2], Mw[3]));
  const float safe = (Mr == -INFINITY) ? 0.f : Mr;
  float Lr = 0.f;
#pragma unroll
  for (int w = 0; w < 4; ++w) Lr += Lw[w] * fast_exp2(Mw[w] - safe);
  const bool real = real_row && Lr > 0.f;
  // without softmax the partial sums are referred to 2^0 and left unnormalised
  *rowM = no_softmax ? 0.f : safe;
  *rowInv = real ? (no_softmax ? 1.f : 1.f / Lr) : 0.f;
}
// normalised partial sums of four consecutive rows, added up
__device__ __forceinline__ float group_sum4(const f32x4& pv, const f32x4& mt, const f32x4& rM, const f32x4& rI) {
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) acc += (rI[i] != 0.f) ? pv[i] * (fast_exp2(mt[i] - rM[i]) * rI[i]) : 0.f;
  return acc;
}
#pragma clang fp contract(fast)

// One workgroup = 64 consecutive reshaped query rows of one head.
// Pass 1 (lane <-> row, wavefronts split the 128-key tiles) combines the tile
// maxima / sums into each row's softmax statistics.  Pass 2 rescales the partial
// block sums and adds the RBS rows of each query block: a lane then owns 4
// consecutive rows (one 16-byte load per key block), 16 lanes cover the 64 rows
// and the four lane groups of a wavefront take four key blocks at a time.
template <int RBS>
__global__ __launch_bounds__(256) void estimate_normalize_kernel(EstParams p) {
  __shared__ float redM[4][64];
  __shared__ float redL[4][64];
  __shared__ __attribute__((aligned(16))) float rowM[64];     // row maximum (0 when the row sees nothing)
  __shared__ __attribute__((aligned(16))) float rowInv[64];   // 1 / row sum, 0 for padded rows
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int head = blockIdx.y;
  const int strip0 = p.row_begin + blockIdx.x * 64;
  const float* Pst = p.P + (int64_t)head * p.nkb * p.rows;
  const float* Mst = p.Mt + (int64_t)head * p.nT * p.rows;
  const float* Lst = p.Lt + (int64_t)head * p.nT * p.rows;

  {
    const int m = strip0 + lane;
    const bool row_ok = m < p.row_end;
    const int mc = row_ok ? m : p.row_end - 1;
    const int mrel = mc - p.row_begin;
    const int lo = row_lo(p, mc);
    int hi = row_hi(p, mc);
    hi = hi < p.n_rk - 1 ? hi : p.n_rk - 1;
    float M = -INFINITY, L = 0.f;
    for (int T = lo / kSub + wave; T <= hi / kSub; T += 4)
      stat_step(M, L, Mst[(int64_t)T * p.rows + mrel], Lst[(int64_t)T * p.rows + mrel]);
    redM[wave][lane] = M;
    redL[wave][lane] = L;
    __syncthreads();
    if (wave == 0) {
      const float Mw[4] = {redM[0][lane], redM[1][lane], redM[2][lane], redM[3][lane]};
      const float Lw[4] = {redL[0][lane], redL[1][lane], redL[2][lane], redL[3][lane]};
      stat_combine(Mw, Lw, row_ok && mc < p.real_rows, p.no_softmax, &rowM[lane], &rowInv[lane]);
    }
    __syncthreads();
  }

  const int l16 = lane & 15, kgrp = lane >> 4;
  const int m4 = strip0 + l16 * 4;                 // first of this lane's 4 rows
  const bool rows_ok = m4 < p.row_end;             // row ranges are multiples of 8: all 4 or none
  const int mc4 = rows_ok ? m4 : p.row_begin;
  const int mrel4 = mc4 - p.row_begin;
  const f32x4 rM = *reinterpret_cast<const f32x4*>(rowM + l16 * 4);
  const f32x4 rI = *reinterpret_cast<const f32x4*>(rowInv + l16 * 4);
  // the RBS rows of a query block share their first / last visible key block
  const int kb_lo = row_lo(p, mc4) / RBS;
  int hi4 = row_hi(p, mc4);
  hi4 = hi4 < p.n_rk - 1 ? hi4 : p.n_rk - 1;
  const int kb_hi = hi4 / RBS;
  float* out = p.sums + ((int64_t)head * p.win_rows + (mc4 / RBS - p.win_row0)) * p.nkb;
  constexpr int kLanesPerBlock = RBS / 4;          // lanes whose 4-row sums make up one query block
  // Four trips' worth of loads are issued before any of them is used, so that each wavefront keeps four
  // 16-byte loads in flight instead of one (the pass is bound by memory latency times loads in flight).
  // A 128-key tile holds 128 / RBS <= 16 key blocks and consecutive trips are 16 key blocks apart, so every
  // trip lies in another tile: its weights are computed per trip (one load of four tile maxima, four exp2).
  constexpr int kUnroll = 4;
  for (int kb0 = wave * 4; kb0 < p.nkb; kb0 += 16 * kUnroll) {
    f32x4 pv[kUnroll], mt[kUnroll];
    bool live[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int kb = kb0 + 16 * u + kgrp;
      live[u] = rows_ok && kb < p.nkb && kb >= kb_lo && kb <= kb_hi;
      if (live[u]) {
        const int T = (kb * RBS) / kSub;
        mt[u] = *reinterpret_cast<const f32x4*>(Mst + (int64_t)T * p.rows + mrel4);
        pv[u] = *reinterpret_cast<const f32x4*>(Pst + (int64_t)kb * p.rows + mrel4);
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int kb = kb0 + 16 * u + kgrp;
      float acc = live[u] ? group_sum4(pv[u], mt[u], rM, rI) : 0.f;
#pragma unroll
      for (int d = 1; d < kLanesPerBlock; d <<= 1) acc += __shfl_xor(acc, d, 64);
      if (rows_ok && kb < p.nkb && (l16 % kLanesPerBlock) == 0) out[kb] = acc;
    }
  }
}

// Normalisation and selection in one pass, for callers that want the column lists (or the mask) and not the
// block sums: a workgroup of QB wavefronts takes QB consecutive q-block rows of one head (QB * RBS reshaped
// query rows), computes their softmax statistics and normalised block sums exactly as the kernel above does -
// same loads, same operation order - but leaves the sums in LDS, where wavefront i then runs the selection of
// row i (select_row.h).  The block sums never travel to memory and back.
template <int RBS>
__global__ __launch_bounds__(256) void estimate_select_kernel(EstParams p, SelParams sp, int qb_per_wg) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rows_wg = qb_per_wg * RBS;                   // reshaped rows of the workgroup (<= 128)
  const int nkb_pad = (p.nkb + 15) & ~15;
  // LDS: statistics, then per wavefront its sort keys (with the row's block sums) and flags
  float* redM = reinterpret_cast<float*>(smem);          // [4][rows_wg]
  float* redL = redM + 4 * rows_wg;                      // [4][rows_wg]
  float* rowM = redL + 4 * rows_wg;                      // [rows_wg]
  float* rowInv = rowM + rows_wg;                        // [rows_wg]
  char* per_wave = smem + 10 * rows_wg * sizeof(float);
  // per wavefront: sort keys, flags; the row's block sums share the tail of the key array (select_row.h)
  const size_t wave_bytes = (size_t)sp.npow2 * 8 + nkb_pad;
  const size_t xs_off = (size_t)sp.npow2 * 8 - (size_t)nkb_pad * 4;

  const int qrows = (p.row_end - p.row_begin) / RBS;     // q-block rows of this call
  const int groups = (qrows + qb_per_wg - 1) / qb_per_wg;
  const int head = blockIdx.x / groups;
  const int grp = blockIdx.x % groups;
  const int strip0 = p.row_begin + grp * rows_wg;        // first reshaped row of the workgroup
  const float* Pst = p.P + (int64_t)head * p.nkb * p.rows;
  const float* Mst = p.Mt + (int64_t)head * p.nT * p.rows;
  const float* Lst = p.Lt + (int64_t)head * p.nT * p.rows;

  // pass 1: thread (row, w) folds tiles first + w, + 4, ... of its row
  for (int idx = tid; idx < rows_wg * 4; idx += blockDim.x) {
    const int lrow = idx % rows_wg, w = idx / rows_wg;
    const int m = strip0 + lrow;
    const int mc = m < p.row_end ? m : p.row_end - 1;
    const int mrel = mc - p.row_begin;
    const int lo = row_lo(p, mc);
    int hi = row_hi(p, mc);
    hi = hi < p.n_rk - 1 ? hi : p.n_rk - 1;
    float M = -INFINITY, L = 0.f;
    // eight tiles' statistics are requested before the first is folded in (the folding is a dependent chain)
    for (int T0 = lo / kSub + w; T0 <= hi / kSub; T0 += 32) {
      float mt[8], lt[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int T = T0 + 4 * u;
        if (T <= hi / kSub) {
          mt[u] = Mst[(int64_t)T * p.rows + mrel];
          lt[u] = Lst[(int64_t)T * p.rows + mrel];
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (T0 + 4 * u <= hi / kSub) stat_step(M, L, mt[u], lt[u]);
    }
    redM[w * rows_wg + lrow] = M;
    redL[w * rows_wg + lrow] = L;
  }
  __syncthreads();
  for (int lrow = tid; lrow < rows_wg; lrow += blockDim.x) {
    const int m = strip0 + lrow;
    const bool row_ok = m < p.row_end;
    const float Mw[4] = {redM[lrow], redM[rows_wg + lrow], redM[2 * rows_wg + lrow], redM[3 * rows_wg + lrow]};
    const float Lw[4] = {redL[lrow], redL[rows_wg + lrow], redL[2 * rows_wg + lrow], redL[3 * rows_wg + lrow]};
    stat_combine(Mw, Lw, row_ok && m < p.real_rows, p.no_softmax, &rowM[lrow], &rowInv[lrow]);
  }
  __syncthreads();

  // pass 2: a thread owns 4 consecutive rows; lpk threads cover the workgroup's rows, the rest of the
  // thread index runs over key blocks
  {
    constexpr int kLanesPerBlock = RBS / 4;
    const int lpk = rows_wg / 4;
    const int l = tid % lpk, kgrp = tid / lpk, kb_step = blockDim.x / lpk;
    const int m4 = strip0 + l * 4;
    const bool rows_ok = m4 < p.row_end;
    const int mc4 = rows_ok ? m4 : p.row_begin;
    const int mrel4 = mc4 - p.row_begin;
    const f32x4 rM = *reinterpret_cast<const f32x4*>(rowM + l * 4);
    const f32x4 rI = *reinterpret_cast<const f32x4*>(rowInv + l * 4);
    const int kb_lo = row_lo(p, mc4) / RBS;
    int hi4 = row_hi(p, mc4);
    hi4 = hi4 < p.n_rk - 1 ? hi4 : p.n_rk - 1;
    const int kb_hi = hi4 / RBS;
    float* xs = reinterpret_cast<float*>(per_wave + (size_t)(l / kLanesPerBlock) * wave_bytes + xs_off);
    float* gout = p.sums ? p.sums + ((int64_t)head * p.win_rows + (mc4 / RBS - p.win_row0)) * p.nkb : nullptr;
    constexpr int kUnroll = 8;
    for (int kb0 = kgrp; kb0 < p.nkb; kb0 += kb_step * kUnroll) {
      f32x4 pv[kUnroll], mt[kUnroll];
      bool live[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int kb = kb0 + kb_step * u;
        live[u] = rows_ok && kb < p.nkb && kb >= kb_lo && kb <= kb_hi;
        if (live[u]) {
          const int T = (kb * RBS) / kSub;
          mt[u] = *reinterpret_cast<const f32x4*>(Mst + (int64_t)T * p.rows + mrel4);
          pv[u] = *reinterpret_cast<const f32x4*>(Pst + (int64_t)kb * p.rows + mrel4);
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int kb = kb0 + kb_step * u;
        float acc = live[u] ? group_sum4(pv[u], mt[u], rM, rI) : 0.f;
#pragma unroll
        for (int d = 1; d < kLanesPerBlock; d <<= 1) acc += __shfl_xor(acc, d, 64);
        if (kb < p.nkb && (l % kLanesPerBlock) == 0) {
          xs[kb] = acc;
          if (gout && rows_ok) gout[kb] = acc;
        }
      }
    }
  }
  __syncthreads();

  // selection: wavefront i takes q-block row i of the group
  if (wave < qb_per_wg) {
    const int row = strip0 / RBS + wave;                 // q-block row (row_begin is a multiple of RBS)
    if (row < p.row_end / RBS) {
      char* mine = per_wave + (size_t)wave * wave_bytes;
      select_row(sp, reinterpret_cast<const float*>(mine + xs_off), head, row, reinterpret_cast<uint64_t*>(mine),
                 reinterpret_cast<uint8_t*>(mine + (size_t)sp.npow2 * 8), lane);
    }
  }
}

// The same normalisation for subsampled query rows (kdb > 1): a query block then
// has rbs / kdb rows (possibly fewer than four), which the vectorised kernel
// above does not handle.  One workgroup per (query block, head): thread
// (row = tid % 32, part = tid / 32) folds every 8th key tile into the row's
// statistics, then each thread owns key blocks tid, tid + 256, ...
__global__ __launch_bounds__(256) void estimate_normalize_rows_kernel(EstParams p) {
  __shared__ float redM[8][32];
  __shared__ float redL[8][32];
  __shared__ float rowM[32];
  __shared__ float rowInv[32];
  const int tid = threadIdx.x, row = tid & 31, part = tid >> 5;
  const int head = blockIdx.y;
  const int m0 = p.row_begin + blockIdx.x * p.rbs_q;     // first query row of the block
  const float* Pst = p.P + (int64_t)head * p.nkb * p.rows;
  const float* Mst = p.Mt + (int64_t)head * p.nT * p.rows;
  const float* Lst = p.Lt + (int64_t)head * p.nT * p.rows;
  const bool row_ok = row < p.rbs_q && m0 + row < p.row_end;
  const int m = row_ok ? m0 + row : m0;
  const int mrel = m - p.row_begin;
  const int lo = row_lo(p, m);
  int hi = row_hi(p, m);
  hi = hi < p.n_rk - 1 ? hi : p.n_rk - 1;
  float M = -INFINITY, L = 0.f;
  for (int T = lo / kSub + part; T <= hi / kSub; T += 8) {
    const float mt = Mst[(int64_t)T * p.rows + mrel];
    const float lt = Lst[(int64_t)T * p.rows + mrel];
    const float Mn = fmaxf(M, mt);
    const float safe = (Mn == -INFINITY) ? 0.f : Mn;
    L = L * fast_exp2(M - safe) + lt * fast_exp2(mt - safe);
    M = Mn;
  }
  redM[part][row] = M;
  redL[part][row] = L;
  __syncthreads();
  if (part == 0) {
    float Mr = -INFINITY;
    for (int w = 0; w < 8; ++w) Mr = fmaxf(Mr, redM[w][row]);
    const float safe = (Mr == -INFINITY) ? 0.f : Mr;
    float Lr = 0.f;
    for (int w = 0; w < 8; ++w) Lr += redL[w][row] * fast_exp2(redM[w][row] - safe);
    const bool real = row_ok && m < p.real_rows && Lr > 0.f;
    rowM[row] = p.no_softmax ? 0.f : safe;
    rowInv[row] = real ? (p.no_softmax ? 1.f : 1.f / Lr) : 0.f;
  }
  __syncthreads();
  float* out = p.sums + ((int64_t)head * p.win_rows + (m0 / p.rbs_q - p.win_row0)) * p.nkb;
  for (int kb = tid; kb < p.nkb; kb += 256) {
    const int T = (kb * p.rbs) / kSub;
    float acc = 0.f;
    for (int r = 0; r < p.rbs_q; ++r) {
      const int mr = m0 + r;
      if (mr >= p.row_end || rowInv[r] == 0.f) continue;
      int h2 = row_hi(p, mr);
      h2 = h2 < p.n_rk - 1 ? h2 : p.n_rk - 1;
      if (kb < row_lo(p, mr) / p.rbs || kb > h2 / p.rbs) continue;
      const int rel = mr - p.row_begin;
      acc += Pst[(int64_t)kb * p.rows + rel] * fast_exp2(Mst[(int64_t)T * p.rows + rel] - rowM[r]) * rowInv[r];
    }
    out[kb] = acc;
  }
}

}  // namespace xattn

using namespace xattn;

namespace {
template <int RBS>
hipError_t launch_gemm(const EstParams& p, dim3 grid, size_t lds, hipStream_t s) {
  auto kernel = p.n_pairs ? (p.scores ? &estimate_gemm_kernel<RBS, true, true> : &estimate_gemm_kernel<RBS, false, true>)
                          : (p.scores ? &estimate_gemm_kernel<RBS, true, false> : &estimate_gemm_kernel<RBS, false, false>);
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kernel, grid, dim3(kWaves * 64), lds, s, p);
  return hipSuccess;
}

// CUs of the current device, rounded down to a multiple of 8 (tile ids are dealt to the 8 XCDs in turn)
int resident_workgroups() {
  static std::mutex mu;
  static int per_device[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  std::lock_guard<std::mutex> lock(mu);
  if (per_device[dev] == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    per_device[dev] = cus >= 8 ? cus / 8 * 8 : 8;
  }
  return per_device[dev];
}

struct Geometry {
  int q_pad, k_pad, n_rq, n_rk, nqb, nkb, nT, rcs, q_chunks;   // n_rq: reshaped query rows before subsampling
};

bool geometry(int q_len, int k_len, int stride, int block_size, int chunk_size, Geometry* g) {
  if (q_len <= 0 || k_len <= 0 || chunk_size <= 0) return false;
  if (chunk_size % block_size) return false;
  const int64_t qp = ((int64_t)q_len + chunk_size - 1) / chunk_size * chunk_size;
  const int64_t kp = ((int64_t)k_len + chunk_size - 1) / chunk_size * chunk_size;
  if (kp > (int64_t)1 << 30 || kp < qp) return false;
  g->q_pad = (int)(qp - q_len);
  g->k_pad = (int)(kp - k_len);
  g->n_rq = (int)(qp / stride);
  g->n_rk = (int)(kp / stride);
  g->nqb = (int)(qp / block_size);
  g->nkb = (int)(kp / block_size);
  g->nT = (g->n_rk + kSub - 1) / kSub;
  g->rcs = chunk_size / stride;
  g->q_chunks = (int)(qp / chunk_size);
  return true;
}

size_t workspace_bytes(int H, const Geometry& g, int rows) {
  return (size_t)H * rows * ((size_t)g.nkb + 2 * (size_t)g.nT) * sizeof(float);
}
}  // namespace

extern "C" size_t xattn_estimate_workspace_bytes(int num_heads, int q_len, int k_len, int stride,
                                                 int block_size, int chunk_size, int chunks_per_call) {
  Geometry g;
  if (num_heads <= 0 || block_size != 128 || (stride != 4 && stride != 8 && stride != 16)) return 0;
  if (!geometry(q_len, k_len, stride, block_size, chunk_size, &g)) return 0;
  int c = (chunks_per_call <= 0 || chunks_per_call > g.q_chunks) ? g.q_chunks : chunks_per_call;
  return workspace_bytes(num_heads, g, c * g.rcs);   // (an upper bound when query rows are subsampled)
}

namespace {
// what the fused normalise-and-select pass needs beside the estimator's own arguments
struct SelectArgs {
  const double* tau;
  uint8_t* mask;
  int32_t* col_idx;
  int32_t* col_cnt;
  int64_t idx_pitch;
  int keep_sink, keep_recent;
  int stages;               // bit 0: run the GEMM pass, bit 1: run the normalise-and-select pass
};

int estimate_impl(const void* q, const void* k, float* block_sums, void* workspace, size_t workspace_size,
                  float* scores_out, int num_heads, int num_kv_heads, int q_len, int k_len, int head_dim,
                  int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_h, int64_t k_stride_n, int stride,
                  int block_size, int chunk_size, int chunk_begin, int chunk_end, int causal, int own_chunk_only,
                  float scale, const int32_t* slab_pairs, int num_slab_pairs, int softmax, int kdb,
                  int zero_rows_from, int window_row0, int window_rows, void* stream, const SelectArgs* sel) {
  if (!q || !k || !workspace) return XATTN_ERR_NULL;
  if (!block_sums && !sel) return XATTN_ERR_NULL;
  if (sel) {
    if (!sel->tau) return XATTN_ERR_NULL;
    if ((sel->col_idx == nullptr) != (sel->col_cnt == nullptr)) return XATTN_ERR_NULL;
    if (!sel->mask && !sel->col_idx) return XATTN_ERR_NULL;     // nothing to write
    if (sel->col_idx && sel->idx_pitch < 1) return XATTN_ERR_SHAPE;
    if (kdb != 1) return XATTN_ERR_SHAPE;                        // the fused pass needs whole query blocks of rows
    if (!(sel->stages & 3) || (sel->stages & ~3)) return XATTN_ERR_SHAPE;
  }
  if (head_dim != kHeadDim) return XATTN_ERR_HEAD_DIM;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads) return XATTN_ERR_HEADS;
  if (block_size != 128 || (stride != 4 && stride != 8 && stride != 16)) return XATTN_ERR_STRIDE;
  Geometry g;
  if (!geometry(q_len, k_len, stride, block_size, chunk_size, &g)) return XATTN_ERR_SHAPE;
  if (chunk_begin < 0 || chunk_end > g.q_chunks || chunk_begin >= chunk_end) return XATTN_ERR_SHAPE;
  // query-row subsampling must divide the rows of a chunk and of a query block; only the
  // antidiagonal reshape has it (xattn/src/Xattention.py:88-93)
  if (kdb < 1 || (block_size / stride) % kdb || g.rcs % kdb || (kdb > 1 && num_slab_pairs != 0)) return XATTN_ERR_SHAPE;
  if (!(scale > 0.f) || !(scale < 1e30f)) return XATTN_ERR_SHAPE;
  if (q_stride_h % 8 || q_stride_n % 8 || k_stride_h % 8 || k_stride_n % 8) return XATTN_ERR_ALIGN;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k)) & 15) return XATTN_ERR_ALIGN;

  EstParams p;
  p.q = static_cast<const __bf16*>(q);
  p.k = static_cast<const __bf16*>(k);
  p.q_sh = q_stride_h; p.q_sn = q_stride_n; p.k_sh = k_stride_h; p.k_sn = k_stride_n;
  if (q_stride_n < kHeadDim || k_stride_n < kHeadDim) return XATTN_ERR_ALIGN;
  // one 256-row tile (256 * stride tokens) must span less than 2^31 bytes
  if ((int64_t)(kTile + 1) * stride * kdb * q_stride_n * 2 >= 0x7fffffff ||
      (int64_t)(kTile + 1) * stride * k_stride_n * 2 >= 0x7fffffff)
    return XATTN_ERR_SHAPE;
  p.H = num_heads; p.Hkv = num_kv_heads; p.Lq = q_len; p.Lk = k_len; p.S = stride;
  p.rbs = block_size / stride;
  p.n_rq = g.n_rq / kdb; p.n_rk = g.n_rk; p.nkb = g.nkb; p.nqb = g.nqb; p.nT = g.nT; p.rcs = g.rcs;
  p.kdb = kdb; p.rcs_q = g.rcs / kdb; p.rbs_q = p.rbs / kdb;
  p.row_begin = chunk_begin * p.rcs_q;
  p.row_end = chunk_end * p.rcs_q;
  p.rows = p.row_end - p.row_begin;
  p.off = g.n_rk - g.n_rq;
  // default: the torch branch's rule for kdb = 1 (the padded tail, xattn/src/Xattention.py:237-238)
  p.real_rows = zero_rows_from >= 0 ? zero_rows_from : p.n_rq - g.q_pad / stride / kdb;
  p.causal = causal ? 1 : 0;
  p.own_chunk_only = own_chunk_only ? 1 : 0;
  p.scale_log2 = scale * kLog2e;
  p.no_softmax = softmax ? 0 : 1;
  p.n_pairs = 0;
  if (num_slab_pairs < 0 || num_slab_pairs > 64 || (num_slab_pairs > 0 && !slab_pairs)) return XATTN_ERR_SHAPE;
  for (int j = 0; j < num_slab_pairs; ++j) {
    const int qo = slab_pairs[2 * j], ko = slab_pairs[2 * j + 1];
    if (qo < 0 || qo >= stride || ko < 0 || ko >= stride) return XATTN_ERR_SHAPE;
    p.pairs[j] = (uint8_t)((qo << 4) | ko);
  }
  p.n_pairs = num_slab_pairs;
  p.scores = scores_out;
  p.sums = block_sums;
  // block_sums may hold a window of q-block rows only; the chunks of this call must lie inside it
  {
    const int bpc = chunk_size / block_size;
    if (window_rows <= 0) { window_row0 = 0; window_rows = g.nqb; }
    if (window_row0 < 0 || chunk_begin * bpc < window_row0 || chunk_end * bpc > window_row0 + window_rows)
      return XATTN_ERR_SHAPE;
    p.win_row0 = window_row0;
    p.win_rows = window_rows;
  }
  if (workspace_size < workspace_bytes(num_heads, g, p.rows)) return XATTN_ERR_WORKSPACE;
  float* ws = static_cast<float*>(workspace);
  p.P = ws;
  p.Mt = ws + (size_t)num_heads * g.nkb * p.rows;
  p.Lt = p.Mt + (size_t)num_heads * g.nT * p.rows;

  hipStream_t s = static_cast<hipStream_t>(stream);
  p.nMT = (p.rows + kTile - 1) / kTile;
  p.nNT = (g.n_rk + kTile - 1) / kTile;
  p.tiles_per_head = 0;
  for (int r = 0; r < p.nMT; ++r) {   // same visibility rule as the kernel's row_lo / row_hi
    const int mfirst = p.row_begin + r * kTile;
    const int mlast = (mfirst + kTile - 1 < p.row_end ? mfirst + kTile - 1 : p.row_end - 1);
    int hi = row_hi(p, mlast) / kTile;
    hi = hi < p.nNT - 1 ? hi : p.nNT - 1;
    const int lo = row_lo(p, mfirst) / kTile;
    p.tiles_per_head += hi - lo + 1;
  }
  p.total_tiles = (int64_t)p.tiles_per_head * num_heads;
  const int64_t ids = (p.total_tiles + 255) / 256 * 256;
  if (ids > 0x7fffffff) return XATTN_ERR_SHAPE;
  // one workgroup per CU (its LDS stages fill a CU), each working through tile ids b, b + grid, ...
  const int resident = resident_workgroups();
  if (resident <= 0) return XATTN_ERR_LAUNCH;
  const dim3 grid1((unsigned)(ids < resident ? ids : resident));
  const dim3 grid2((p.rows + 63) / 64, num_heads);
  if (grid2.y > 65535) return XATTN_ERR_SHAPE;
  const size_t lds = 2 * (size_t)kStageBytes;
  // the fused normalise-and-select pass: QB q-block rows (one wavefront each) per workgroup, as many as keep a
  // workgroup's LDS (statistics + per wavefront: the row's sums, sort keys, flags) within 64 KiB
  SelParams sp;
  int qb_per_wg = 0;
  size_t lds_sel = 0;
  dim3 grid_sel(1);
  if (sel) {
    if (g.nkb > 8192) return XATTN_ERR_SHAPE;      // (longer rows: block sums through memory, xattn_select_blocks)
    const int bpc = chunk_size / block_size;
    sp.sums = nullptr; sp.tau = sel->tau; sp.mask = sel->mask; sp.col_idx = sel->col_idx; sp.col_cnt = sel->col_cnt;
    sp.idx_pitch = sel->idx_pitch; sp.H = num_heads; sp.nqb = g.nqb; sp.nkb = g.nkb;
    sp.row_begin = chunk_begin * bpc; sp.row_end = chunk_end * bpc; sp.diag_offset = g.nkb - g.nqb;
    sp.win_row0 = p.win_row0; sp.win_rows = p.win_rows;
    sp.causal = p.causal; sp.keep_sink = sel->keep_sink ? 1 : 0; sp.keep_recent = sel->keep_recent ? 1 : 0;
    sp.list_cols = (k_len + block_size - 1) / block_size; sp.q_len = q_len; sp.kv_off = k_len - q_len;
    sp.blocks_per_chunk = bpc;
    int np2 = 64;
    while (np2 < g.nkb) np2 <<= 1;
    sp.npow2 = np2;
    const size_t nkb_pad = ((size_t)g.nkb + 15) & ~(size_t)15;
    const size_t wave_bytes = (size_t)np2 * 8 + nkb_pad;
    qb_per_wg = 4;
    while (qb_per_wg > 1 && (qb_per_wg * (wave_bytes + 10 * p.rbs * sizeof(float)) > 64 * 1024 || qb_per_wg * p.rbs > 128))
      qb_per_wg >>= 1;
    lds_sel = qb_per_wg * (wave_bytes + 10 * p.rbs * sizeof(float));
    const int qrows = p.rows / p.rbs;
    const int64_t wgs = (int64_t)num_heads * ((qrows + qb_per_wg - 1) / qb_per_wg);
    if (wgs > 0x7fffffff) return XATTN_ERR_SHAPE;
    grid_sel = dim3((unsigned)wgs);
  }
  auto launch_rest = [&](auto normalize, auto fused) -> hipError_t {
    if (!sel) {
      if (kdb == 1) hipLaunchKernelGGL(normalize, grid2, dim3(256), 0, s, p);
      return hipSuccess;
    }
    hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(fused), hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)lds_sel);
    if (e2 != hipSuccess) return e2;
    hipLaunchKernelGGL(fused, grid_sel, dim3(64 * qb_per_wg), lds_sel, s, p, sp, qb_per_wg);
    return hipSuccess;
  };
  const bool run_gemm = !sel || (sel->stages & 1), run_rest = !sel || (sel->stages & 2);
  hipError_t e = hipSuccess;
  switch (p.rbs) {
    case 8:
      if (run_gemm) e = launch_gemm<8>(p, grid1, lds, s);
      if (e == hipSuccess && run_rest) e = launch_rest(&estimate_normalize_kernel<8>, &estimate_select_kernel<8>);
      break;
    case 16:
      if (run_gemm) e = launch_gemm<16>(p, grid1, lds, s);
      if (e == hipSuccess && run_rest) e = launch_rest(&estimate_normalize_kernel<16>, &estimate_select_kernel<16>);
      break;
    default:
      if (run_gemm) e = launch_gemm<32>(p, grid1, lds, s);
      if (e == hipSuccess && run_rest) e = launch_rest(&estimate_normalize_kernel<32>, &estimate_select_kernel<32>);
      break;
  }
  if (e != hipSuccess) return XATTN_ERR_LAUNCH;
  if (kdb != 1) {
    const dim3 grid3(p.rows / p.rbs_q, num_heads);
    hipLaunchKernelGGL(estimate_normalize_rows_kernel, grid3, dim3(256), 0, s, p);
  }
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}
}  // namespace

extern "C" int xattn_estimate_block_sums(const void* q, const void* k, float* block_sums, void* workspace,
                                         size_t workspace_size, float* scores_out, int num_heads,
                                         int num_kv_heads, int q_len, int k_len, int head_dim,
                                         int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_h,
                                         int64_t k_stride_n, int stride, int block_size, int chunk_size,
                                         int chunk_begin, int chunk_end, int causal, int own_chunk_only,
                                         float scale, const int32_t* slab_pairs, int num_slab_pairs,
                                         int softmax, int kdb, int zero_rows_from, int window_row0,
                                         int window_rows, void* stream) {
  if (!block_sums) return XATTN_ERR_NULL;
  return estimate_impl(q, k, block_sums, workspace, workspace_size, scores_out, num_heads, num_kv_heads, q_len, k_len,
                       head_dim, q_stride_h, q_stride_n, k_stride_h, k_stride_n, stride, block_size, chunk_size,
                       chunk_begin, chunk_end, causal, own_chunk_only, scale, slab_pairs, num_slab_pairs, softmax, kdb,
                       zero_rows_from, window_row0, window_rows, stream, nullptr);
}

extern "C" int xattn_estimate_select(const void* q, const void* k, float* block_sums, void* workspace,
                                     size_t workspace_size, int num_heads, int num_kv_heads, int q_len, int k_len,
                                     int head_dim, int64_t q_stride_h, int64_t q_stride_n, int64_t k_stride_h,
                                     int64_t k_stride_n, int stride, int block_size, int chunk_size, int chunk_begin,
                                     int chunk_end, int causal, int own_chunk_only, float scale,
                                     const int32_t* slab_pairs, int num_slab_pairs, int softmax, int zero_rows_from,
                                     int window_row0, int window_rows, const double* tau_per_head, uint8_t* mask,
                                     int32_t* col_idx, int32_t* col_cnt, int64_t idx_pitch, int keep_sink,
                                     int keep_recent, int stages, void* stream) {
  const SelectArgs sel = {tau_per_head, mask, col_idx, col_cnt, idx_pitch, keep_sink, keep_recent, stages};
  return estimate_impl(q, k, block_sums, workspace, workspace_size, nullptr, num_heads, num_kv_heads, q_len, k_len,
                       head_dim, q_stride_h, q_stride_n, k_stride_h, k_stride_n, stride, block_size, chunk_size,
                       chunk_begin, chunk_end, causal, own_chunk_only, scale, slab_pairs, num_slab_pairs, softmax, 1,
                       zero_rows_from, window_row0, window_rows, stream, &sel);
}
