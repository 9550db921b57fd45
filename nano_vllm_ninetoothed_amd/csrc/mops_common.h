// Shared helpers for the gfx950 kernels: vector types, bf16 <-> fp32, wave64 reductions, launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/mops_hip.h"

namespace mops {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

__device__ __forceinline__ float bf16lo_to_f32(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// Round-to-nearest-even fp32 -> bf16 (v_cvt_pk_bf16_f32 on gfx950), returned as raw bits.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  __bf16 b = (__bf16)f;
  return (uint32_t)__builtin_bit_cast(unsigned short, b);
}
// Two fp32 -> one dword of two bf16 (lo in bits 0..15), one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  const f32x2_t f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}
__device__ __forceinline__ float round_to_bf16(float f) { return (float)(__bf16)f; }

__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void store16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }
// Streaming variants: data touched once should not displace reusable lines.
__device__ __forceinline__ u32x4 load16_stream(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void store16_stream(void* p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// The value of the lane ROT places further on inside its row of 16 lanes (wrapping): a DPP operand, no trip through the
// LDS crossbar.
template <int ROT>
__device__ __forceinline__ float row_rotate(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 | ROT, 0xf, 0xf, false));   // row_ror:ROT
}
// Sum over groups of WIDTH consecutive lanes (WIDTH a power of two <= 64); every lane gets the total.  The steps of a
// butterfly (partner = lane ^ off); for off < 16 the partner's value is taken from the lane `off` places around the row
// instead, which holds the same number: the first such step pairs lanes 8 apart either way, and after each step the
// partial sums repeat with the period of the next one, so every lane adds the same two numbers as in the butterfly.
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
  if (WIDTH < 16) {   // groups smaller than a row: a rotation would reach into the neighbouring group
#pragma unroll
    for (int off = WIDTH / 2; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
  }
#pragma unroll
  for (int off = WIDTH / 2; off >= 16; off >>= 1) v += __shfl_xor(v, off, kWave);
  v += row_rotate<8>(v);
  v += row_rotate<4>(v);
  v += row_rotate<2>(v);
  v += row_rotate<1>(v);
  return v;
}
template <int WIDTH>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int off = WIDTH / 2; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Records the launch error (if any) for mops_hip_last_hip_error and maps it to a status.
int finish_launch();
// Records a failed HIP runtime call the same way; returns MOPS_HIP_ELAUNCH.
int record_hip_error(hipError_t e);

}  // namespace mops
