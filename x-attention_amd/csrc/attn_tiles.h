// K/V tile movement and workgroup dispatch shared by the attention-shaped
// kernels (block-sparse forward, block-mass profiler).
#pragma once
#include "xattn_common.h"

namespace xattn {

constexpr int kBlk = 128;          // block_size of the operator
constexpr int kTileBytes = kBlk * 256;   // one K or V tile in LDS
constexpr int kUnit = 64;                // workgroups resident on one XCD (32 CUs x 2)

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short i16x4;

// LDS tile layout: row n at byte n*256, its 16-byte chunk c stored at chunk
// c ^ swz(n).  swz takes all 16 values over 16 consecutive rows (row-per-lane
// b128 reads of one logical chunk are conflict-free) and moves rows n..n+3 into
// different 64-byte groups (the 4-row x 32-byte gathers of the transposing read
// are conflict-free too).
__device__ __forceinline__ int swz(int n) { return ((n & 3) << 2) | ((n >> 2) & 3); }

// Copies key block kb of one head (row stride sn elements) into an LDS tile.
// Wavefront w issues 8 instructions of 1 KiB (4 rows) each; voff[i] is the
// lane's byte offset inside the block for instruction i.
__device__ __forceinline__ void copy_tile(const __bf16* base, int64_t sn, int len, int kb, const int (&voff)[8],
                                          char* tile, int wave) {
  const int rows_left = len - kb * kBlk;
  const int rows = rows_left < kBlk ? rows_left : kBlk;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(base + (int64_t)kb * kBlk * sn), 0, (int)((int64_t)rows * sn * 2), 0x00020000);
#pragma unroll
  for (int i = 0; i < 8; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)(tile + (wave * 8 + i) * 1024), 16, voff[i], 0, 0, 0);
}

__device__ __forceinline__ void tile_offsets(int64_t sn, int lane, int wave, int (&voff)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = 4 * (wave * 8 + i) + (lane >> 4);
    const int c = (lane & 15) ^ swz(row);
    voff[i] = (int)(row * sn * 2) + (c << 4);
  }
}


// Workgroup ids are dealt round-robin to the 8 XCDs, and an XCD (32 CUs, two
// workgroups each, one L2) starts its workgroups in id order.  The 64 ids that
// land on one XCD one after the other form a unit: the query heads of ONE KV
// head times a run of adjacent q-blocks, so everything resident on the XCD
// streams the same K/V through its L2 at about the same place.  Units are
// dealt to XCDs in turn; the KV head of a unit rotates with the q-block run,
// so every XCD sees every head equally often (heads differ by orders of
// magnitude in list length).  Runs go out last (longest, when causal) first.
// Returns false for ids that carry no work.
__device__ __forceinline__ bool map_workgroup(int id, int H, int Hkv, int unit_rows, int qb_begin, int qb_end,
                                              int* head, int* qb) {
  const int group = H / Hkv;
  const int x = id & 7, s = id >> 3;
  const int unit = (s / kUnit) * 8 + x, w = s % kUnit;
  const int run = unit / Hkv;
  const int kvh = (unit % Hkv + run) % Hkv;
  const int from_end = run * unit_rows + w / group;
  if (w >= group * unit_rows || from_end >= qb_end - qb_begin) return false;
  *qb = qb_end - 1 - from_end;
  *head = kvh * group + w % group;
  return true;
}

// q-blocks per unit and grid size of a launch over [qb_begin, qb_end)
inline int unit_rows_for(int H, int Hkv) {
  const int group = H / Hkv;
  return group >= kUnit ? 1 : kUnit / group;
}
inline int64_t grid_for(int H, int Hkv, int n_qblocks) {
  const int ur = unit_rows_for(H, Hkv);
  const int64_t runs = (n_qblocks + ur - 1) / ur;
  return ((runs * Hkv + 7) / 8 * 8) * kUnit;
}

}  // namespace xattn
