// Shared device helpers for the gfx950 kernels: element types, conversions,
// wavefront (64 lanes) and workgroup reductions, and the host-side error slot.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define RA_WAVE 64

// element-type tags of the C interface
enum { RA_F32 = 0, RA_BF16 = 1 };

// XCDs of the chip: workgroups are dealt round them in the order of their numbers, each XCD has an L2 of its own
#define RA_XCDS 8

typedef __bf16 bf16_t;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
// round to nearest even; the hardware conversion of gfx950
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = RA_WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, RA_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = RA_WAVE / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, RA_WAVE));
  return v;
}

// Sum over a workgroup of up to 1024 threads; every thread gets the result.
// `red` is LDS for 17 floats. All threads of the workgroup must call it.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int nwave = (blockDim.x + RA_WAVE - 1) / RA_WAVE;
  v = wave_sum(v);
  __syncthreads();               // red may still be read from an earlier call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwave; ++i) t += red[i];   // fixed order: deterministic
  return t;
}

// ---- cache layout -----------------------------------------------------------
// A block of the cache holds block_size (a multiple of 16) slots of one KV head
// as block_size/16 tiles of 16 slots x d elements, 16*d elements each, laid out
// in the order the MFMA operands want them, so that a wave's load of a tile is
// one contiguous run and LDS copies of it have no bank conflicts:
//   K tile: [d/8][16 slots][8]      element (slot, e) at ((e/8)*16 + slot)*8 + e%8
//   V tile: [d/16][4][16][4]        element (slot, e) at (((e/16)*4 + slot/4)*16 + e%16)*4 + slot%4
// `off` is the slot inside the block; d is a multiple of 16.
__host__ __device__ __forceinline__ size_t cache_k_index(int off, int e, int d) {
  return (size_t)(off >> 4) * 16 * d + (size_t)(((e >> 3) * 16 + (off & 15)) * 8 + (e & 7));
}
__host__ __device__ __forceinline__ size_t cache_v_index(int off, int e, int d) {
  const int s = off & 15;
  return (size_t)(off >> 4) * 16 * d + (size_t)((((e >> 4) * 4 + (s >> 2)) * 16 + (e & 15)) * 4 + (s & 3));
}

// ---- host side -------------------------------------------------------------
// One message slot per thread; ra_last_error() hands it to the caller.
extern thread_local char ra_error_text[512];
int ra_fail(const char* fmt, ...);

// Compute units of the current device (cached per device; 256 if the device cannot be asked).
int ra_cu_count(void);

#define RA_CHECK(cond, ...)                    \
  do {                                         \
    if (!(cond)) return ra_fail(__VA_ARGS__);  \
  } while (0)

#define RA_LAUNCH_CHECK(name)                                                   \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess) return ra_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); \
  } while (0)
