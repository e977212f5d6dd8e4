// Shared definitions for the gfx950 kernels: element types, error codes, small device helpers.
// Every entry point is extern "C", takes raw device pointers and a hipStream_t, launches
// asynchronously on that stream and returns 0, or a negative code without launching anything.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#define CW_OK 0
#define CW_ERR_ARG -1      // a size or pointer the kernel does not take
#define CW_ERR_DTYPE -2    // unknown element type code
#define CW_ERR_LAUNCH -3   // the HIP runtime refused the launch
#define CW_ERR_SIZE -4     // beyond a stated maximum

#define CW_F32 0
#define CW_BF16 1

#define CW_EXPORT extern "C" __attribute__((visibility("default")))

typedef __hip_bfloat16 bf16_t;

__device__ __forceinline__ float cw_to_float(float x) { return x; }
__device__ __forceinline__ float cw_to_float(bf16_t x) { return __bfloat162float(x); }

template <typename T> __device__ __forceinline__ T cw_from_float(float x);
template <> __device__ __forceinline__ float cw_from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t cw_from_float<bf16_t>(float x) { return __float2bfloat16(x); }

// bfloat16 bits <-> float without going through the class type (for packed 16-byte loads)
__device__ __forceinline__ float cw_bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
__device__ __forceinline__ uint16_t cw_float_to_bf16_bits(float f) {
  // round to nearest even; NaN stays NaN
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// Maximum / sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 of a wave, on the vector unit: the
// swaps of 16-lane rows and of the wave's halves (v_permlane16_swap, v_permlane32_swap) hand every
// lane both values of its pair, so all four lanes end with the same result, summed as
// (l + l^16) + (l^32 + l^48). (A shuffle goes through the LDS unit and waits behind its queue.)
typedef __attribute__((ext_vector_type(2))) unsigned int cw_u32x2_t;
__device__ __forceinline__ float cw_quad_max(float v) {
  const cw_u32x2_t a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const cw_u32x2_t b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float cw_quad_sum(float v) {
  const cw_u32x2_t a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const cw_u32x2_t b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

__device__ __forceinline__ float cw_wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float cw_wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// A workgroup barrier for data that waves hand each other through LDS: LDS writes made before it
// are visible after it. __syncthreads() also orders global memory, and for that it waits until
// every global store the wave has issued is done; the counter it waits on counts loads as well, in
// order, so a wave that has prefetched its next tile and then stored a result waits at the barrier
// for the prefetch too, and the loop loses the overlap it was built for. Kernels whose global
// stores nobody in the workgroup reads back use this barrier in such loops.
__device__ __forceinline__ void cw_lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

static inline int cw_launch_status() {
  return hipGetLastError() == hipSuccess ? CW_OK : CW_ERR_LAUNCH;
}
