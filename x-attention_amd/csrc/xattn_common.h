// Shared device helpers for the gfx950 XAttention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace xattn {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;

constexpr int kWave = 64;
constexpr int kHeadDim = 128;
constexpr float kLog2e = 1.4426950408889634f;

// D[32x32] += A[32x16] * B[16x32], bf16 in, fp32 accumulate.
// Lane l (r = l % 32, h = l / 32) supplies A[r][8h..8h+7] and B[8h..8h+7][r];
// it receives D[8*(v/4) + 4h + v%4][r] in element v of the accumulator.
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
  bf16x2 p;
  p[0] = (__bf16)lo;
  p[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, p);
}

// waits until every outstanding global/buffer load of this wavefront (including
// loads that write LDS directly) has completed; LDS and scalar counters untouched
__device__ __forceinline__ void wait_vm0() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// value held by the lane 32 positions away (the other half-wave)
__device__ __forceinline__ float swap_half(float x) { return __shfl_xor(x, 32, 64); }

// x combined with the value of the lane 32 positions away, in every lane.  One
// v_permlane32_swap exchanges the upper half of its first operand with the lower
// half of its second: fed two copies of x it leaves (lower half, lower half) in
// the first and (upper half, upper half) in the second - both partners in every
// lane, without a trip through the LDS crossbar.  Written as inline assembly
// (the compiler's builtin hands back the first result twice); the s_nop pairs
// cover the wait states the instruction needs after a VALU write of its
// operands and before a VALU read of its results.
__device__ __forceinline__ void half_pair(float x, float& lo, float& hi) {
  lo = x;
  hi = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
}
// Two values combined across the half-waves at once: the lower half-wave ends up with a of the lane plus a of its
// partner, the upper half-wave with b plus b of its partner - one swap where two half_sum() calls need two.
__device__ __forceinline__ float half_sum_pair(float a, float b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}
__device__ __forceinline__ float half_sum(float x) {
  float lo, hi;
  half_pair(x, lo, hi);
  return lo + hi;
}
__device__ __forceinline__ float half_max(float x) {
  float lo, hi;
  half_pair(x, lo, hi);
  return fmaxf(lo, hi);
}

}  // namespace xattn
