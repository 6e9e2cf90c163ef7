// Threshold block selection of one q-block row by one wavefront: shared by the stand-alone selection kernel
// (block sums from memory) and the estimator's fused normalise-and-select kernel (block sums from LDS).
#pragma once
#include "xattn_common.h"

namespace xattn {

struct SelParams {
  const float* sums;
  const double* tau;
  uint8_t* mask;
  int32_t* col_idx;
  int32_t* col_cnt;
  int64_t idx_pitch;
  int H, nqb, nkb, row_begin, row_end, diag_offset;
  int win_row0, win_rows;   // the arrays hold q-block rows [win_row0, win_row0 + win_rows) of every head
  int causal, keep_sink, keep_recent, list_cols, q_len, kv_off;
  int blocks_per_chunk;
  int npow2;   // LDS key capacity (power of two >= nkb)
};

constexpr int kSlots = 16;        // candidates per lane held in registers (rows up to 1024 candidates)
constexpr int kMaxExtract = 32;   // blocks pulled out one by one before falling back to the sort

// value encoded in a sort key (0 for forced blocks and padding)
__device__ __forceinline__ double key_value(uint64_t key) {
  const uint32_t hi = (uint32_t)(key >> 32);
  return hi ? (double)__uint_as_float(hi - 1u) : 0.0;
}

__device__ __forceinline__ double wave_sum(double x) {
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) x += __shfl_xor(x, d, 64);
  return x;
}

// M(i + ahead) from the masses before the i-th ordinary block (b0), before its predecessor (b1) and before
// the one ahead of that (b2); ranks 0 and 1 carry no mass
__device__ __forceinline__ double rank_mass(int i, int ahead, double b0, double b1, double b2) {
  const int back = 2 - ahead;          // 0, 1 or 2 ordinary blocks fewer than all those ahead of it
  if (i < back) return 0.0;
  return back == 0 ? b0 : (back == 1 ? b1 : b2);
}

// Selection for q-block row `row` of `head` by ONE wavefront (lane = its lane number).  x: the row's nkb block
// sums (global or LDS); keys (npow2 entries) and flags (nkb bytes): LDS scratch of this wavefront.  All LDS
// traffic is the wavefront's own, which the LDS keeps in program order: the points where the lanes exchange
// data through it need no workgroup barrier.  x may occupy the LAST 4 * nkb bytes of the key array (rounded up
// to 64 bytes): key c then lands on sums 2c - (2 npow2 - nkb) and the one after, both below c, i.e. sums that
// the loops which fill the keys (ascending c, a whole wavefront's reads before its writes) have read already.
__device__ __forceinline__ void select_row(const SelParams& p, const float* x, int head, int row, uint64_t* keys,
                                           uint8_t* flags, int lane) {
  const int64_t slot = (int64_t)head * p.win_rows + (row - p.win_row0);   // this row's place in the arrays
  const int diag = row + p.diag_offset;
  // Column index of the first diagonal of the row's query chunk.  When it is 0
  // the reference's eye() assignment overwrites the forced sink column
  // (utils.py:100-106), leaving the diagonal as the only forced block while
  // the [0, forced_sum, ...] prefix (utils.py:115-124) still reserves two
  // slots: the largest other block is then always kept and every later one is
  // judged against the mass gathered before its predecessor.
  const int chunk_first = p.diag_offset + (row / p.blocks_per_chunk) * p.blocks_per_chunk;
  const bool one_forced = p.causal && chunk_first == 0;

  // candidates: columns [0, ncand); when causal nothing beyond the diagonal can be kept
  int ncand = p.nkb;
  if (p.causal) ncand = diag + 1 < p.nkb ? diag + 1 : p.nkb;
  if (ncand < 0) ncand = 0;
  int np2 = 64;
  while (np2 < ncand) np2 <<= 1;

  // (the forced blocks' sums are read before any sort key is written: x may share its memory with the tail of
  // the key array, see below)
  double forced_sum = 0.0;
  // sort keys of the forced blocks (utils.py:126-130); key_hi >= key_lo, equal when only one block is forced
  double key_lo = 0.0, key_hi = 0.0;
  if (p.causal && ncand > 0) {
    if (!one_forced || diag == 0) forced_sum = (double)x[0];
    if (diag != 0 && diag < p.nkb) forced_sum += (double)x[diag];
    const double kd = 100000.0 * (1.0 + (double)x[diag < p.nkb ? diag : 0]);
    const double k0 = one_forced ? kd : 100000.0 * (1.0 + (double)x[0]);
    key_lo = kd < k0 ? kd : k0;
    key_hi = kd < k0 ? k0 : kd;
  }
  double total = 0.0;
  uint32_t vals[kSlots];      // this lane's candidates: slot u holds column u*64 + lane (0 = none)
  int n_others = 0;
#pragma unroll
  for (int u = 0; u < kSlots; ++u) vals[u] = 0;
  // value bits of candidate c (0 for forced blocks and columns past the candidates); adds it to `total` on request
  auto load_one = [&](int c, bool count) -> uint32_t {
    uint32_t bits = 0;
    if (c < ncand) {
      const float v = x[c];
      if (count) total += (double)v;
      const bool forced = p.causal && (c == diag || (c == 0 && !one_forced));
      // block sums are >= 0, so their bit pattern orders like the value (+1
      // keeps every candidate ahead of the forced blocks, which sort last)
      bits = forced ? 0u : __float_as_uint(v > 0.f ? v : 0.f) + 1u;
    }
    return bits;
  };
  // sort key: low word = ~column makes equal sums come out by ascending column; padding (c >= ncand) sorts
  // last and carries an out-of-range column
  auto sort_key = [&](int c, uint32_t bits) -> uint64_t {
    return c < ncand ? (((uint64_t)bits << 32) | (uint32_t)(~(uint32_t)c)) : 0ull;
  };
  const bool small = np2 <= kSlots * 64;
  if (small) {      // candidates stay in registers; the sort keys are only written if the extraction gives up
#pragma unroll
    for (int u = 0; u < kSlots; ++u)
      if (u * 64 < np2) {
        vals[u] = load_one(u * 64 + lane, true);
        n_others += vals[u] != 0;
      }
  } else {
    for (int c = lane; c < np2; c += 64) keys[c] = sort_key(c, load_one(c, true));
  }
  for (int c = lane; c < p.nkb; c += 64) flags[c] = 0;
  total = wave_sum(total);
  const double required = total * p.tau[head];
  const int n_forced = one_forced ? 1 : 2;
  // forced keys ranked ahead of an ordinary block of sum v (all of them unless v is beyond 100000)
  auto forced_ahead = [&](double v) -> int {
    if (!(v > key_lo)) return n_forced;
    return one_forced ? 0 : (v > key_hi ? 0 : 1);
  };
  __builtin_amdgcn_wave_barrier();

  int dropped = 0;
  bool finished = false;
  // no block sum can exceed a forced key unless the row's total does: otherwise the forced blocks rank first
  // and a decision does not need the block's own value
  const bool may_outrank = p.causal && total > key_lo;
  if (small) {
    // ---- extraction: keep pulling out the largest remaining block while the rule says "keep"
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) n_others += __shfl_xor(n_others, d, 64);
    double before = forced_sum, prev_before = 0.0, prev2_before = 0.0;
    for (int it = 0; it < kMaxExtract; ++it) {
      if (n_others == 0) {
        finished = true;
        break;
      }
      if (!may_outrank) {
        const double mass = p.causal ? rank_mass(it, n_forced, before, prev_before, prev2_before) : before;
        if (!(mass < required)) {
          finished = true;
          dropped = 1;
          break;
        }
      }
      uint32_t best = 0;
#pragma unroll
      for (int u = 0; u < kSlots; ++u) best = vals[u] > best ? vals[u] : best;
#pragma unroll
      for (int d = 32; d > 0; d >>= 1) {
        const uint32_t o = __shfl_xor(best, d, 64);
        best = o > best ? o : best;
      }
      const double best_val = (double)__uint_as_float(best - 1u);
      if (may_outrank) {
        const double mass = rank_mass(it, forced_ahead(best_val), before, prev_before, prev2_before);
        if (!(mass < required)) {
          finished = true;
          dropped = 1;
          break;
        }
      }
      uint32_t col = 0xffffffffu;     // lowest column holding the maximum
#pragma unroll
      for (int u = kSlots - 1; u >= 0; --u) col = vals[u] == best ? (uint32_t)(u * 64 + lane) : col;
#pragma unroll
      for (int d = 32; d > 0; d >>= 1) {
        const uint32_t o = __shfl_xor(col, d, 64);
        col = o < col ? o : col;
      }
#pragma unroll
      for (int u = 0; u < kSlots; ++u) vals[u] = (uint32_t)(u * 64 + lane) == col ? 0u : vals[u];
      if (lane == 0) flags[col] = 1;
      prev2_before = prev_before;
      prev_before = before;
      before += best_val;
      --n_others;
    }
  }

  if (!finished) {
  if (small) {
    for (int c = lane; c < np2; c += 64) keys[c] = sort_key(c, load_one(c, false));
    __builtin_amdgcn_wave_barrier();
  }
  // ---- bitonic sort, descending
  for (int k = 2; k <= np2; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = lane; t < (np2 >> 1); t += 64) {
        const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
        const int l = i | j;
        const uint64_t a = keys[i], b = keys[l];
        const bool up = (i & k) == 0;        // this pair's run is descending
        if ((a < b) == up) {
          keys[i] = b;
          keys[l] = a;
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }

  // fp64 exclusive prefix over the sorted values; rank kept while mass before it < required
  const int per = np2 >> 6;
  double local = 0.0;
  for (int u = 0; u < per; ++u) local += key_value(keys[lane * per + u]);
  double incl = local;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const double o = __shfl_up(incl, d, 64);
    if (lane >= d) incl += o;
  }
  double before = forced_sum + (incl - local);
  for (int u = 0; u < per; ++u) {
    const int rank = lane * per + u;
    const uint64_t key = keys[rank];
    const uint32_t col = ~(uint32_t)key;
    if (col < (uint32_t)ncand && (key >> 32) != 0) {
      double mass = before;
      if (may_outrank) {
        const double b1 = rank > 0 ? before - key_value(keys[rank - 1]) : 0.0;
        const double b2 = rank > 1 ? b1 - key_value(keys[rank - 2]) : 0.0;
        mass = rank_mass(rank, forced_ahead(key_value(key)), before, b1, b2);
      } else if (one_forced) {
        mass = rank == 0 ? 0.0 : before - key_value(keys[rank - 1]);
      }
      if (mass < required) flags[col] = 1;
      else dropped = 1;
    }
    before += key_value(key);
  }
  }   // sort path
  const bool any_dropped = __any(dropped);
  __builtin_amdgcn_wave_barrier();
  if (lane == 0) {
    if (p.causal) {
      if (p.nkb > 0) flags[0] = 1;
      if (diag >= 0 && diag < p.nkb) flags[diag] = 1;
    } else if (any_dropped) {
      flags[0] = 1;     // unselected ranks scatter to column 0 (utils.py:164)
    }
    if (p.keep_recent && diag >= 0 && diag < p.nkb) flags[diag] = 1;
  }
  __builtin_amdgcn_wave_barrier();
  if (p.keep_sink && row == 0)
    for (int c = lane; c < p.nkb; c += 64) flags[c] = 1;
  __builtin_amdgcn_wave_barrier();

  if (p.mask) {
    uint8_t* mrow = p.mask + slot * p.nkb;
    for (int c = lane; c < p.nkb; c += 64) mrow[c] = flags[c];
  }

  if (p.col_idx) {
    int32_t* list = p.col_idx + slot * p.idx_pitch;
    const int q_last = (row * 128 + 127 < p.q_len ? row * 128 + 127 : p.q_len - 1) + p.kv_off;
    int count = 0;
    for (int c0 = 0; c0 < p.nkb; c0 += 64) {
      const int c = c0 + lane;
      bool keep = c < p.nkb && flags[c] && c < p.list_cols;
      if (p.causal) keep = keep && (c * 128 <= q_last);
      const uint64_t ballot = __ballot(keep);
      const int pos = count + __popcll(ballot & ((1ull << lane) - 1ull));
      if (keep && pos < p.idx_pitch) list[pos] = c;
      count += __popcll(ballot);
    }
    if (lane == 0) p.col_cnt[slot] = count < p.idx_pitch ? count : (int)p.idx_pitch;
  }
}

}  // namespace xattn
