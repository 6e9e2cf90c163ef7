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

// The same copy issued from one assembly block, M0 (the LDS destination) included.  The compiler makes the
// transposing LDS reads wait for every buffer load into LDS it knows of (the two might alias), which exposes
// the whole copy latency at the next fragment read; loads issued this way are not counted by the compiler, so
// the caller waits for them itself (wait_vm0) before the barrier that publishes the tile.  Loads return in
// order, so the compiler's own vmcnt waits for its own loads stay sufficient.
__device__ __forceinline__ void copy_tile_async(const __bf16* base, int64_t sn, int len, int kb, const int (&voff)[8],
                                                char* tile, int wave) {
  const int rows_left = len - kb * kBlk;
  const int rows = rows_left < kBlk ? rows_left : kBlk;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(base + (int64_t)kb * kBlk * sn), 0, (int)((int64_t)rows * sn * 2), 0x00020000);
  const uint32_t dst = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)(tile + wave * 8 * 1024));
  asm volatile(
      "s_mov_b32 m0, %[dst]\n\ts_nop 0\n\t"
      "buffer_load_dwordx4 %[v0], %[rs], 0 offen lds\n\ts_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "buffer_load_dwordx4 %[v1], %[rs], 0 offen lds\n\ts_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "buffer_load_dwordx4 %[v2], %[rs], 0 offen lds\n\ts_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "buffer_load_dwordx4 %[v3], %[rs], 0 offen lds\n\ts_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "buffer_load_dwordx4 %[v4], %[rs], 0 offen lds\n\ts_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "buffer_load_dwordx4 %[v5], %[rs], 0 offen lds\n\ts_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "buffer_load_dwordx4 %[v6], %[rs], 0 offen lds\n\ts_add_u32 m0, m0, 0x400\n\ts_nop 0\n\t"
      "buffer_load_dwordx4 %[v7], %[rs], 0 offen lds"
      :
      : [dst] "s"(dst), [rs] "s"(rsrc), [v0] "v"(voff[0]), [v1] "v"(voff[1]), [v2] "v"(voff[2]), [v3] "v"(voff[3]),
        [v4] "v"(voff[4]), [v5] "v"(voff[5]), [v6] "v"(voff[6]), [v7] "v"(voff[7])
      : "memory", "m0", "scc");
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
// streams the same K/V through its L2 at about the same place.  A KV head with
// more than 64 query heads is dealt as several head sets of equal size (each a
// dispatch group of its own).  Units are dealt to XCDs in turn; the dispatch
// group of a unit rotates with the q-block run, so every XCD sees every head
// equally often (heads differ by orders of magnitude in list length).  Runs go
// out last (longest, when causal) first.
struct DispatchShape {
  int group;       // query heads per KV head
  int sets;        // head sets per KV head (1 unless group > kUnit)
  int set_heads;   // query heads per set (<= kUnit)
  int n_groups;    // dispatch groups: Hkv * sets
  int unit_rows;   // q-blocks per unit
};
__host__ __device__ inline DispatchShape dispatch_shape(int H, int Hkv) {
  DispatchShape d;
  d.group = H / Hkv;
  d.sets = (d.group + kUnit - 1) / kUnit;
  d.set_heads = (d.group + d.sets - 1) / d.sets;
  d.n_groups = Hkv * d.sets;
  d.unit_rows = kUnit / d.set_heads;
  return d;
}

// Returns false for ids that carry no work.  The shape is computed once on the host (dispatch_shape) and the
// arithmetic is unsigned: this runs at the start of every workgroup, where its divisions are a measurable part
// of what a short unit costs.
__host__ __device__ inline bool map_workgroup(int id, const DispatchShape& d, int qb_begin, int qb_end, int* head,
                                              int* qb, int* kv_head) {
  if (id < 0) return false;
  const uint32_t x = (uint32_t)id & 7u, s = (uint32_t)id >> 3;
  const uint32_t unit = (s / kUnit) * 8u + x, w = s % kUnit;
  const uint32_t ng = (uint32_t)d.n_groups, sh = (uint32_t)d.set_heads;
  const uint32_t run = unit / ng;
  const uint32_t dg = (unit + run) % ng;      // the unit's group, rotated by its run
  const uint32_t w_row = w / sh, w_head = w - w_row * sh;
  const uint32_t from_end = run * (uint32_t)d.unit_rows + w_row;
  uint32_t set = 0, kvh = dg;
  if (d.sets != 1) {
    kvh = dg / (uint32_t)d.sets;
    set = dg - kvh * (uint32_t)d.sets;
  }
  const uint32_t in_group = set * sh + w_head;             // head index inside its KV group
  if (w >= sh * (uint32_t)d.unit_rows || from_end >= (uint32_t)(qb_end - qb_begin) || in_group >= (uint32_t)d.group)
    return false;
  *qb = qb_end - 1 - (int)from_end;
  *head = (int)(kvh * (uint32_t)d.group + in_group);
  *kv_head = (int)kvh;
  return true;
}
__host__ __device__ inline bool map_workgroup(int id, int H, int Hkv, int qb_begin, int qb_end, int* head, int* qb) {
  int kv_head;
  return map_workgroup(id, dispatch_shape(H, Hkv), qb_begin, qb_end, head, qb, &kv_head);
}

// grid size of a launch over n_qblocks q-blocks
inline int64_t grid_for(int H, int Hkv, int n_qblocks) {
  const DispatchShape d = dispatch_shape(H, Hkv);
  const int64_t runs = (n_qblocks + d.unit_rows - 1) / d.unit_rows;
  return ((runs * d.n_groups + 7) / 8 * 8) * kUnit;
}

// Token strides of K and V the tile copies can address (byte offsets inside a
// 128-row tile are held in 32 bits), and a usable softmax scale.
inline bool tile_stride_ok(int64_t sn) { return sn >= kHeadDim && sn <= ((int64_t)1 << 22); }
inline bool scale_ok(float s) { return s > 0.f && s < 1e30f; }

}  // namespace xattn
