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
}  // namespace xattn

extern "C" int xattn_abi_version(void) { return 2; }

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
