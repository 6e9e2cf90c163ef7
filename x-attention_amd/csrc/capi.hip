// Library-level entry points of libxattn_hip.so.
#include <hip/hip_runtime.h>

#include "xattn_hip.h"

namespace xattn {
// Plain grid-stride copy, 16 bytes per lane per trip: a kernel of exactly known
// HBM traffic (reads `bytes`, writes `bytes`) used to scale byte counters.
__global__ __launch_bounds__(256) void calibration_copy_kernel(const uint4* __restrict__ src,
                                                               uint4* __restrict__ dst, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
    dst[i] = src[i];
}

// Nothing but bf16 32x32x16 MFMAs on register operands: what the matrix pipes
// sustain with no memory, LDS or VALU work beside them.  The operands are 16
// fragments per lane read once from `bits` (4 KiB-entries table of 16-byte
// fragments): all-equal bits give the data-independent rate, random bits the
// rate at the switching activity of real inputs - the clock the part holds
// differs between the two.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 probe_bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float probe_f32x16;
// kMix: beside every MFMA the wavefront also issues one v_exp_f32 and three
// v_fma_f32 on registers no MFMA touches and with no dependence on it - the
// per-MFMA vector-ALU load of the attention tile loop (64 MFMAs, 65
// exponentials and about 190 other VALU instructions per tile and wavefront)
// with every wait taken away.  Its rate is what the SIMD's issue logic leaves
// of the MFMA stream under that mix, an upper bound for an attention kernel.
template <bool kMix>
__global__ __launch_bounds__(256) void mfma_rate_probe_kernel(const probe_bf16x8* __restrict__ bits, int iters,
                                                              float* sink) {
  probe_bf16x8 a[8], b[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a[e] = bits[(threadIdx.x * 16 + e) & 4095];
    b[e] = bits[(threadIdx.x * 16 + 8 + e) & 4095];
  }
  probe_f32x16 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  float ex[8], fm[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    ex[e] = (float)a[e][0] * 0.01f;
    fm[e] = (float)b[e][0];
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u * 4 + i) & 7], b[(u + i) & 7], acc[i], 0, 0, 0);
        if (kMix) {
          const int j = (u * 4 + i) & 7;
          ex[j] = __builtin_fmaf(__builtin_amdgcn_exp2f(ex[j]), 0.5f, 0.01f);
          fm[j] = __builtin_fmaf(fm[j], 0.999f, 0.5f);
          fm[(j + 4) & 7] = __builtin_fmaf(fm[(j + 4) & 7], 0.998f, 0.25f);
        }
      }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[i][v];
  if (kMix) {
#pragma unroll
    for (int e = 0; e < 8; ++e) s += ex[e] + fm[e];
  }
  if (s == 12345.678f) sink[0] = s;   // keeps the results live; practically never taken
}
}  // namespace xattn

extern "C" int xattn_abi_version(void) { return 7; }

extern "C" const char* xattn_error_string(int code) {
  switch (code) {
    case XATTN_OK: return "ok";
    case XATTN_ERR_NULL: return "a required pointer is null";
    case XATTN_ERR_HEAD_DIM: return "head_dim must be 128";
    case XATTN_ERR_HEADS: return "num_heads must be a positive multiple of num_kv_heads";
    case XATTN_ERR_SHAPE: return "length, block count or pitch out of range";
    case XATTN_ERR_ALIGN: return "pointers must be 16-byte aligned and strides multiples of 8 elements";
    case XATTN_ERR_STRIDE: return "antidiagonal stride must be 4, 8 or 16 and block_size 128";
    case XATTN_ERR_WORKSPACE: return "workspace too small";
    case XATTN_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown error code";
  }
}

extern "C" int xattn_calibration_copy(void* dst, const void* src, size_t bytes, void* stream) {
  if (!dst || !src) return XATTN_ERR_NULL;
  if (bytes == 0 || bytes % 16) return XATTN_ERR_SHAPE;
  if ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15) return XATTN_ERR_ALIGN;
  hipLaunchKernelGGL(xattn::calibration_copy_kernel, dim3(256 * 32), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4*>(src),
                     static_cast<uint4*>(dst), bytes / 16);
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}

extern "C" int xattn_mfma_rate_probe(const void* operand_bits, int iters, int valu_mix, float* sink,
                                     double* flops_out, void* stream) {
  if (!operand_bits || !sink) return XATTN_ERR_NULL;
  if (iters <= 0 || iters > (1 << 22)) return XATTN_ERR_SHAPE;
  if (reinterpret_cast<uintptr_t>(operand_bits) & 15) return XATTN_ERR_ALIGN;
  const int grid = 256 * 2;   // two workgroups of four wavefronts per CU: two wavefronts per SIMD
  if (flops_out) *flops_out = (double)grid * 4.0 * iters * 16.0 * 32768.0;
  if (valu_mix)
    hipLaunchKernelGGL(xattn::mfma_rate_probe_kernel<true>, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const xattn::probe_bf16x8*>(operand_bits), iters, sink);
  else
    hipLaunchKernelGGL(xattn::mfma_rate_probe_kernel<false>, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const xattn::probe_bf16x8*>(operand_bits), iters, sink);
  return hipGetLastError() == hipSuccess ? XATTN_OK : XATTN_ERR_LAUNCH;
}
