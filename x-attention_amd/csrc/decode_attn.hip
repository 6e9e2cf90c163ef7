// Single-token decode attention over a KV cache for gfx950.
//
// Replaces the reference's call to the third-party
// flashinfer.single_decode_with_kv_cache(q[H,d], k[Hkv,L,d], v[Hkv,L,d],
// kv_layout="HND") in its Llama attention forward
// (xattn/src/load_llama.py:191-196): out[h] = softmax(q[h] K[h/g]^T / sqrt(d)) V[h/g].
//
// The step reads every key and value once and does four flops per byte, so it
// is bound by HBM bandwidth; the design keeps as many bytes in flight per CU as
// LDS can hold.  One workgroup of four wavefronts per CU owns all 160 KiB of
// LDS; every wavefront streams its own contiguous range of 32-key tiles through
// a private ring of five 8 KiB slots (K_i, V_i, K_i+1, V_i+1, K_i+2) filled by
// buffer loads that write LDS directly, so four tiles per wavefront are always
// in flight and no workgroup barrier is needed.  A KV head's query heads (the
// GQA group, at most 32) are the columns of one MFMA tile: S^T = K Q^T gives
// each lane one query head, the softmax is the same lane-owns-a-row form as in
// the prefill kernel and its accumulators feed O^T += V^T P^T unchanged.  The
// four wavefronts combine (max, sum, unnormalised output) of their key ranges in
// LDS and write one partial result per workgroup; a second small kernel merges
// the workgroups of a head.
#include <mutex>

#include "xattn_common.h"
#include "xattn_hip.h"

namespace xattn {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short i16x4;
typedef __attribute__((__vector_size__(8 * sizeof(short)))) short i16x8;

constexpr int kDecKeys = 32;                  // keys per tile
constexpr int kDecTileBytes = kDecKeys * 256;
constexpr int kDecSlots = 5;
constexpr int kDecWaves = 4;
constexpr int kDecLds = kDecWaves * kDecSlots * kDecTileBytes;   // 160 KiB
constexpr int kPartStride = 132;              // floats per (range, query head): 128 outputs, max, sum, 2 pad
constexpr int kDecCUs = 256;

struct DecodeParams {
  const __bf16* q;
  const __bf16* k;
  const __bf16* v;
  __bf16* o;
  float* part;
  int64_t q_sh, k_sh, k_sn, v_sh, v_sn, o_sh;   // element strides
  int H, Hkv, group, Lk;
  int n_tiles, tiles_per_wave, ranges_per_head;   // ranges_per_head is a multiple of kDecWaves
  float scale_log2;
};

__device__ __forceinline__ int dec_swz(int n) { return ((n & 3) << 2) | ((n >> 2) & 3); }

// waits until at most 32 of this wavefront's buffer loads are outstanding
// (loads complete in order, so everything older than the newest four tiles has
// landed in LDS); other counters untouched
__device__ __forceinline__ void wait_vm32() {
  __builtin_amdgcn_s_waitcnt(0x8F70);
  asm volatile("" ::: "memory");
}
__device__ __forceinline__ void wait_lgkm0() {
  __builtin_amdgcn_s_waitcnt(0xC07F);
  asm volatile("" ::: "memory");
}

// One 32-key tile, global -> this wavefront's LDS slot.  Tiles outside
// [0, n_tiles) are issued with an empty buffer resource: they move no data but
// keep the count of outstanding loads the same on every iteration.
__device__ __forceinline__ void dec_copy(const __bf16* base, int64_t sn, int len, int tile, int n_tiles,
                                         const int (&voff)[8], char* slot) {
  const bool live = tile < n_tiles;
  const int t = live ? tile : 0;
  const int rows_left = len - t * kDecKeys;
  const int rows = live ? (rows_left < kDecKeys ? rows_left : kDecKeys) : 0;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(base + (int64_t)t * kDecKeys * sn), 0, (int)((int64_t)rows * sn * 2), 0x00020000);
#pragma unroll
  for (int i = 0; i < 8; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)(slot + i * 1024), 16, voff[i], 0, 0, 0);
}

__global__ __launch_bounds__(256, 1) void decode_partial_kernel(DecodeParams p) {
  extern __shared__ __attribute__((aligned(1024))) char ring_all[];

  const int tid = threadIdx.x, lane = tid & 63;
  // the wavefront number in a scalar register: tile ranges, buffer resources and
  // LDS slots derived from it are then uniform values for the compiler too
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31, hh = lane >> 5;
  const int wgs_per_head = p.ranges_per_head / kDecWaves;
  const int kvh = blockIdx.x / wgs_per_head;
  const int range = (blockIdx.x % wgs_per_head) * kDecWaves + wave;
  const int t0 = range * p.tiles_per_wave;
  int t1 = t0 + p.tiles_per_wave;
  t1 = t1 < p.n_tiles ? t1 : p.n_tiles;
  const int n = t1 > t0 ? t1 - t0 : 0;

  char* ring = ring_all + wave * (kDecSlots * kDecTileBytes);
  // the same place as an LDS byte address
  const uint32_t ring_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)ring_all +
                            (uint32_t)(wave * (kDecSlots * kDecTileBytes));
  const __bf16* kbase = p.k + (int64_t)kvh * p.k_sh;
  const __bf16* vbase = p.v + (int64_t)kvh * p.v_sh;

  // Q^T fragments: lane r holds query head kvh*group + r (zeros beyond the group)
  bf16x8 qreg[8];
  {
    const bool live = r < p.group;
    const __bf16* src = p.q + (int64_t)(kvh * p.group + (live ? r : 0)) * p.q_sh + hh * 8;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      bf16x8 x = *reinterpret_cast<const bf16x8*>(src + s * 16);
#pragma unroll
      for (int e = 0; e < 8; ++e) qreg[s][e] = live ? x[e] : (__bf16)0.f;
    }
  }

  int voffK[8], voffV[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = 4 * i + (lane >> 4);
    const int c = (lane & 15) ^ dec_swz(row);
    voffK[i] = (int)(row * p.k_sn * 2) + (c << 4);
    voffV[i] = (int)(row * p.v_sn * 2) + (c << 4);
  }
  int kaddr[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) kaddr[s] = r * 256 + (((2 * s + hh) ^ dec_swz(r)) << 4);
  int vaddr[4][2];
  {
    const int e = (lane & 15) >> 2, j = lane & 3, g2 = (lane >> 4) & 1;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const int row = 8 * a + 4 * hh + e;                       // + 16*ks
        const int c = dt * 4 + 2 * g2 + (j >> 1);
        vaddr[dt][a] = row * 256 + ((c ^ dec_swz(row)) << 4) + (j & 1) * 8;
      }
  }

  f32x16 oacc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[i][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // load number j of the sequence K_0 V_0 K_1 V_1 ... goes to slot j % 5
  const int t_end = t0 + n;
  dec_copy(kbase, p.k_sn, p.Lk, t0, t_end, voffK, ring + 0 * kDecTileBytes);
  dec_copy(vbase, p.v_sn, p.Lk, t0, t_end, voffV, ring + 1 * kDecTileBytes);
  dec_copy(kbase, p.k_sn, p.Lk, t0 + 1, t_end, voffK, ring + 2 * kDecTileBytes);
  dec_copy(vbase, p.v_sn, p.Lk, t0 + 1, t_end, voffV, ring + 3 * kDecTileBytes);

  int slot = 0;   // slot of K_i
  for (int i = 0; i < n; ++i) {
    const int tile = t0 + i;
    char* Kt = ring + slot * kDecTileBytes;
    const int sv = slot + 1 >= kDecSlots ? slot + 1 - kDecSlots : slot + 1;
    const int s4 = slot + 4 >= kDecSlots ? slot + 4 - kDecSlots : slot + 4;   // freed by V_{i-1}

    wait_lgkm0();   // this wavefront's reads of the slot about to be refilled have returned
    dec_copy(kbase, p.k_sn, p.Lk, tile + 2, t_end, voffK, ring + s4 * kDecTileBytes);
    wait_vm32();    // K_i landed

    f32x16 sacc;
#pragma unroll
    for (int v = 0; v < 16; ++v) sacc[v] = 0.f;
    {
      bf16x8 kf[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) kf[s] = *reinterpret_cast<const bf16x8*>(Kt + kaddr[s]);
#pragma unroll
      for (int s = 0; s < 8; ++s) sacc = mfma32(kf[s], qreg[s], sacc);
    }
    if (tile * kDecKeys + kDecKeys > p.Lk) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int kpos = tile * kDecKeys + (v >> 2) * 8 + hh * 4 + (v & 3);
        sacc[v] = kpos >= p.Lk ? -INFINITY : sacc[v];
      }
    }
    // K_i is in registers (the MFMAs above consumed every fragment): its slot takes V_{i+2}
    wait_lgkm0();
    dec_copy(vbase, p.v_sn, p.Lk, tile + 2, t_end, voffV, Kt);

    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < 16; ++v) mx = fmaxf(mx, sacc[v]);
    mx = half_max(mx) * p.scale_log2;
    const float m_new = fmaxf(m_run, mx);          // finite: every tile holds at least one real key
    const float alpha = fast_exp2(m_run - m_new);  // 0 on the first tile
    m_run = m_new;
    l_run *= alpha;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int v = 0; v < 16; ++v) oacc[dt][v] *= alpha;
    float psum = 0.f;
    bf16x8 pfrag[2];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float e = fast_exp2(__builtin_fmaf(sacc[v], p.scale_log2, -m_run));
      psum += e;
      pfrag[v >> 3][v & 7] = (__bf16)e;
    }
    l_run += psum;

    wait_vm32();    // V_i landed
    {
      // The sixteen transposing reads of V_i are issued from one asm statement:
      // an LDS read the compiler can see would make it wait for EVERY buffer
      // load in flight (it cannot tell the ring's slots apart), which would
      // empty the ring on each iteration.
      i16x4 t[4][2][2];   // [feature tile][half a][k-step]
      const uint32_t vt = ring_lds + (uint32_t)(sv * kDecTileBytes);
      uint32_t a[4][2];
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) a[dt][h2] = vt + (uint32_t)vaddr[dt][h2];
      asm volatile(
          "ds_read_b64_tr_b16 %0, %16\n\t"
          "ds_read_b64_tr_b16 %1, %16 offset:4096\n\t"
          "ds_read_b64_tr_b16 %2, %17\n\t"
          "ds_read_b64_tr_b16 %3, %17 offset:4096\n\t"
          "ds_read_b64_tr_b16 %4, %18\n\t"
          "ds_read_b64_tr_b16 %5, %18 offset:4096\n\t"
          "ds_read_b64_tr_b16 %6, %19\n\t"
          "ds_read_b64_tr_b16 %7, %19 offset:4096\n\t"
          "ds_read_b64_tr_b16 %8, %20\n\t"
          "ds_read_b64_tr_b16 %9, %20 offset:4096\n\t"
          "ds_read_b64_tr_b16 %10, %21\n\t"
          "ds_read_b64_tr_b16 %11, %21 offset:4096\n\t"
          "ds_read_b64_tr_b16 %12, %22\n\t"
          "ds_read_b64_tr_b16 %13, %22 offset:4096\n\t"
          "ds_read_b64_tr_b16 %14, %23\n\t"
          "ds_read_b64_tr_b16 %15, %23 offset:4096\n\t"
          "s_waitcnt lgkmcnt(0)"
          : "=&v"(t[0][0][0]), "=&v"(t[0][0][1]), "=&v"(t[0][1][0]), "=&v"(t[0][1][1]),
            "=&v"(t[1][0][0]), "=&v"(t[1][0][1]), "=&v"(t[1][1][0]), "=&v"(t[1][1][1]),
            "=&v"(t[2][0][0]), "=&v"(t[2][0][1]), "=&v"(t[2][1][0]), "=&v"(t[2][1][1]),
            "=&v"(t[3][0][0]), "=&v"(t[3][0][1]), "=&v"(t[3][1][0]), "=&v"(t[3][1][1])
          : "v"(a[0][0]), "v"(a[0][1]), "v"(a[1][0]), "v"(a[1][1]),
            "v"(a[2][0]), "v"(a[2][1]), "v"(a[3][0]), "v"(a[3][1])
          : "memory");
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
          i16x8 av;
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            av[u] = t[dt][0][ks][u];
            av[4 + u] = t[dt][1][ks][u];
          }
          oacc[dt] = mfma32(__builtin_bit_cast(bf16x8, av), pfrag[ks], oacc[dt]);
        }
    }
    slot = slot + 2 >= kDecSlots ? slot + 2 - kDecSlots : slot + 2;
  }
  wait_vm0();   // nothing is still writing this wavefront's LDS

  // The four wavefronts' results meet in LDS (each uses the start of its own,
  // now idle, ring) and leave as one partial result per workgroup.
  const float l_tot = half_sum(l_run);
  float* mine = reinterpret_cast<float*>(ring);
  if (r < p.group) {
    float* dst = mine + r * kPartStride;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 w;
#pragma unroll
        for (int u = 0; u < 4; ++u) w[u] = oacc[dt][g * 4 + u];
        *reinterpret_cast<f32x4*>(dst + dt * 32 + g * 8 + hh * 4) = w;
      }
    if (hh == 0) {
      dst[128] = m_run;    // -inf for an empty range
      dst[129] = l_tot;    // 0 for an empty range
    }
  }
  __syncthreads();
  {
    constexpr int kWaveFloats = kDecSlots * kDecTileBytes / 4;
    const float* all = reinterpret_cast<const float*>(ring_all);
    float* out = p.part + (int64_t)blockIdx.x * p.group * kPartStride;
    for (int e = tid; e < p.group * 128; e += 256) {
      const int g = e >> 7, d = e & 127;
      float mw[kDecWaves], m = -INFINITY;
#pragma unroll
      for (int w = 0; w < kDecWaves; ++w) {
        mw[w] = all[w * kWaveFloats + g * kPartStride + 128];
        m = fmaxf(m, mw[w]);
      }
      float acc = 0.f, l = 0.f;
#pragma unroll
      for (int w = 0; w < kDecWaves; ++w) {
        const float wt = mw[w] == -INFINITY ? 0.f : fast_exp2(mw[w] - m);
        acc += wt * all[w * kWaveFloats + g * kPartStride + d];
        l += wt * all[w * kWaveFloats + g * kPartStride + 129];
      }
      out[g * kPartStride + d] = acc;
      if (d == 0) {
        out[g * kPartStride + 128] = m;
        out[g * kPartStride + 129] = l;
      }
    }
  }
}

// out[h][d] = sum_s w_s O_s[d] / sum_s w_s l_s,  w_s = 2^(m_s - max m), over the
// head's workgroups s.  Thread t takes features 4*(t%32).. of every eighth
// partial result, keeping a running maximum; the eight lanes-of-ranges then meet
// in LDS.
__global__ __launch_bounds__(256) void decode_merge_kernel(DecodeParams p) {
  __shared__ __attribute__((aligned(16))) float accs[8][128];
  __shared__ float ms[8], ls[8];
  const int head = blockIdx.x, tid = threadIdx.x;
  const int kvh = head / p.group, g = head % p.group;
  const int wgs = p.ranges_per_head / kDecWaves;
  const float* base = p.part + ((int64_t)kvh * wgs * p.group + g) * kPartStride;
  const int64_t step = (int64_t)p.group * kPartStride;
  const int slot = tid >> 5, dg = tid & 31;

  float m = -INFINITY, l = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int s = slot; s < wgs; s += 8) {
    const float* ps = base + s * step;
    const f32x4 o = *reinterpret_cast<const f32x4*>(ps + dg * 4);
    const float m_s = ps[128], l_s = ps[129];
    if (m_s == -INFINITY) continue;
    const float m_new = fmaxf(m, m_s);
    const float a = fast_exp2(m - m_new), b = fast_exp2(m_s - m_new);
    m = m_new;
    l = l * a + l_s * b;
#pragma unroll
    for (int u = 0; u < 4; ++u) acc[u] = acc[u] * a + o[u] * b;
  }
  *reinterpret_cast<f32x4*>(&accs[slot][dg * 4]) = acc;
  if (dg == 0) {
    ms[slot] = m;
    ls[slot] = l;
  }
  __syncthreads();
  if (tid < 128) {
    float mt = -INFINITY;
#pragma unroll
    for (int s = 0; s < 8; ++s) mt = fmaxf(mt, ms[s]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const float w = ms[s] == -INFINITY ? 0.f : fast_exp2(ms[s] - mt);
      num += w * accs[s][tid];
      den += w * ls[s];
    }
    p.o[(int64_t)head * p.o_sh + tid] = (__bf16)(den > 0.f ? num / den : 0.f);
  }
}

struct DecodeGeometry {
  int n_tiles, tiles_per_wave, ranges_per_head;
};

// One workgroup per CU at most: a KV head gets 256 / H_kv workgroups (at least
// one), i.e. four times as many key ranges, unless it has fewer tiles than that.
static DecodeGeometry decode_geometry(int num_kv_heads, int k_len) {
  DecodeGeometry g;
  g.n_tiles = (k_len + kDecKeys - 1) / kDecKeys;
  int wgs = kDecCUs / num_kv_heads;
  if (wgs < 1) wgs = 1;
  g.tiles_per_wave = (g.n_tiles + wgs * kDecWaves - 1) / (wgs * kDecWaves);
  const int ranges = (g.n_tiles + g.tiles_per_wave - 1) / g.tiles_per_wave;
  g.ranges_per_head = (ranges + kDecWaves - 1) / kDecWaves * kDecWaves;
  return g;
}

}  // namespace xattn

using namespace xattn;

extern "C" size_t xattn_decode_workspace_bytes(int num_heads, int num_kv_heads, int k_len) {
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads || k_len <= 0) return 0;
  const DecodeGeometry g = decode_geometry(num_kv_heads, k_len);
  return (size_t)(g.ranges_per_head / kDecWaves) * num_heads * kPartStride * sizeof(float);
}

namespace {
// Validates, fills the launch parameters and enqueues both kernels; `part` holds
// part_bytes bytes of per-range partial results.
int decode_launch(const void* q, const void* k, const void* v, void* out, void* part, size_t part_bytes,
                  int num_heads, int num_kv_heads, int k_len, int head_dim, int64_t q_stride_h,
                  int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_h, int64_t v_stride_n,
                  int64_t o_stride_h, float softmax_scale, void* stream) {
  if (!q || !k || !v || !out || !part) return XATTN_ERR_NULL;
  if (head_dim != kHeadDim) return XATTN_ERR_HEAD_DIM;
  if (num_heads <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads) return XATTN_ERR_HEADS;
  if (num_heads / num_kv_heads > 32) return XATTN_ERR_HEADS;
  if (k_len <= 0) return XATTN_ERR_SHAPE;
  const int64_t strides[] = {q_stride_h, k_stride_h, k_stride_n, v_stride_h, v_stride_n};
  for (int64_t s : strides)
    if (s % 8) return XATTN_ERR_ALIGN;
  auto a16 = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; };
  if (!a16(q) || !a16(k) || !a16(v) || !a16(part)) return XATTN_ERR_ALIGN;
  // a tile's byte offsets are held in 32 bits
  if (k_stride_n > (1 << 22) || v_stride_n > (1 << 22) || k_stride_n < kHeadDim || v_stride_n < kHeadDim)
    return XATTN_ERR_SHAPE;
  if (part_bytes < xattn_decode_workspace_bytes(num_heads, num_kv_heads, k_len)) return XATTN_ERR_WORKSPACE;

  const DecodeGeometry g = decode_geometry(num_kv_heads, k_len);
  DecodeParams p;
  p.q = static_cast<const __bf16*>(q);
  p.k = static_cast<const __bf16*>(k);
  p.v = static_cast<const __bf16*>(v);
  p.o = static_cast<__bf16*>(out);
  p.part = static_cast<float*>(part);
  p.q_sh = q_stride_h; p.k_sh = k_stride_h; p.k_sn = k_stride_n;
  p.v_sh = v_stride_h; p.v_sn = v_stride_n; p.o_sh = o_stride_h;
  p.H = num_heads; p.Hkv = num_kv_heads; p.group = num_heads / num_kv_heads; p.Lk = k_len;
  p.n_tiles = g.n_tiles; p.tiles_per_wave = g.tiles_per_wave; p.ranges_per_head = g.ranges_per_head;
  p.scale_log2 = softmax_scale * kLog2e;

  hipStream_t s = static_cast<hipStream_t>(stream);
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(decode_partial_kernel),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kDecLds) != hipSuccess)
    return XATTN_ERR_LAUNCH;
  const unsigned grid = (unsigned)(num_kv_heads * (g.ranges_per_head / kDecWaves));
  hipLaunchKernelGGL(decode_partial_kernel, dim3(grid), dim3(256), kDecLds, s, p);
  hipLaunchKernelGGL(decode_merge_kernel, dim3((unsigned)num_heads), dim3(256), 0, s, p);
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}
}  // namespace

extern "C" int xattn_decode_fwd(const void* q, const void* k, const void* v, void* out, void* workspace,
                                size_t workspace_bytes, int num_heads, int num_kv_heads, int k_len, int head_dim,
                                int64_t q_stride_h, int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_h,
                                int64_t v_stride_n, int64_t o_stride_h, float softmax_scale, void* stream) {
  return decode_launch(q, k, v, out, workspace, workspace_bytes, num_heads, num_kv_heads, k_len, head_dim, q_stride_h,
                       k_stride_h, k_stride_n, v_stride_h, v_stride_n, o_stride_h, softmax_scale, stream);
}

// ---------------------------------------------------------------------------
// The same decode step for callers that may not allocate: the partial results
// live in a device array that is part of this library's code object.  Every GPU
// the library runs on holds its own copy of the array at its own address; the
// address is looked up once per device and kept.  In host code the array's name
// is only a handle for that lookup, never a pointer a kernel could use.
namespace {
// (256 / H_kv workgroups per KV head) x H query heads is at most 256 * 32
// (range, head) pairs while H_kv <= 256 and H <= 32 H_kv.
constexpr size_t kDecScratchBytes = (size_t)kDecCUs * 32 * kPartStride * sizeof(float);   // 4.125 MiB
static_assert(kDecScratchBytes == XATTN_DECODE_STATIC_SCRATCH_BYTES, "header and kernel disagree on the scratch size");
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kDecScratchBytes];
namespace {
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up on first use).
int scratch_of_current_device(void** ptr_out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return XATTN_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return XATTN_ERR_LAUNCH;
    g_scratch_ptr[dev] = ptr;
  }
  *ptr_out = g_scratch_ptr[dev];
  return XATTN_OK;
}
}  // namespace

extern "C" int xattn_decode_fwd_static(const void* q, const void* k, const void* v, void* out, int num_heads,
                                       int num_kv_heads, int k_len, int head_dim, int64_t q_stride_h,
                                       int64_t k_stride_h, int64_t k_stride_n, int64_t v_stride_h,
                                       int64_t v_stride_n, int64_t o_stride_h, float softmax_scale, void* stream) {
  const size_t need = xattn_decode_workspace_bytes(num_heads, num_kv_heads, k_len);
  if (need == 0) {
    if (num_heads <= 0 || num_kv_heads <= 0 || (num_kv_heads > 0 && num_heads % num_kv_heads)) return XATTN_ERR_HEADS;
    return XATTN_ERR_SHAPE;
  }
  if (need > kDecScratchBytes) return XATTN_ERR_WORKSPACE;   // more (range, head) pairs than the array holds
  void* ptr = nullptr;
  const int rc = scratch_of_current_device(&ptr);
  if (rc != XATTN_OK) return rc;
  return decode_launch(q, k, v, out, ptr, kDecScratchBytes, num_heads, num_kv_heads, k_len, head_dim, q_stride_h,
                       k_stride_h, k_stride_n, v_stride_h, v_stride_n, o_stride_h, softmax_scale, stream);
}
