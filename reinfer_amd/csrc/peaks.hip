// What the machine gives at best, to price the engine's kernels against beside the published peaks:
// a read of a large buffer that does nothing else, and a loop of matrix-core products on registers.
// Neither is on the product path; bench.py calls them once.
#include "common.h"
#include "reinfer_hip.h"

// A workgroup reads 32 KB that lie together at a time (every thread eight loads of 16 bytes, all in
// flight at once) and moves on by the grid's width; what it read is folded into one word so that no load
// can be dropped, and written only if it is a value that random data does not give.
__global__ void __launch_bounds__(256)
stream_read_kernel(const uint4* __restrict__ src, size_t n16, unsigned* __restrict__ sink) {
  constexpr size_t RUN = 8 * 256;                       // 16-byte pieces a workgroup reads a round
  unsigned acc = 0;
  size_t base = (size_t)blockIdx.x * RUN;
  for (; base + RUN <= n16; base += (size_t)gridDim.x * RUN) {
    uint4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[base + u * 256 + threadIdx.x];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (size_t i = base + threadIdx.x; i < n16 && i < base + RUN; i += 256) {      // the last, partial run
    const uint4 v = src[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9E3779B9u) sink[0] = acc;
}

// Four independent 32x32x16 bfloat16 products an iteration on operands that stay in registers.
__global__ void __launch_bounds__(256)
mfma_loop32_kernel(int iters, float* __restrict__ sink) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  bf16x8_t a, b;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = (bf16_t)(0.001f * (float)((lane + j) & 7));
    b[j] = (bf16_t)(0.002f * (float)((lane * 3 + j) & 7));
  }
  f32x16_t acc[4];                    // different from each other, or the compiler makes one of them
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[k][i] = (float)(k * 16 + i + lane);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int k = 0; k < 4; ++k) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[k], 0, 0, 0);
  }
  float t = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) t += acc[k][i];
  if (t == -1.f) sink[0] = t;
}

// Eight independent 16x16x32 bfloat16 products an iteration on operands that stay in registers.
__global__ void __launch_bounds__(256)
mfma_loop_kernel(int iters, float* __restrict__ sink) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  bf16x8_t a, b;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = (bf16_t)(0.001f * (float)((lane + j) & 7));
    b[j] = (bf16_t)(0.002f * (float)((lane * 3 + j) & 7));
  }
  f32x4_t acc[8];                     // different from each other, or the compiler makes one of them
#pragma unroll
  for (int k = 0; k < 8; ++k) acc[k] = (f32x4_t){(float)(k + lane), (float)(k + 8), (float)(k + 16), (float)(k + 24)};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[k], 0, 0, 0);
  }
  float t = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) t += acc[k][0] + acc[k][1] + acc[k][2] + acc[k][3];
  if (t == -1.f) sink[0] = t;          // sums of non-negative numbers: never
}

// Reads `bytes` (a multiple of 16, 16-byte aligned) once. `sink` is 4 bytes of device memory.
extern "C" int ra_stream_read(const void* src, long bytes, void* sink, hipStream_t stream) {
  RA_CHECK(src && sink && bytes >= 16 && bytes % 16 == 0 && ((uintptr_t)src % 16) == 0,
           "stream_read: a 16-byte aligned buffer of a multiple of 16 bytes, got %ld", bytes);
  const int cus = ra_cu_count();
  RA_CHECK(cus > 0, "stream_read: no compute units reported");
  stream_read_kernel<<<cus * 8, 256, 0, stream>>>((const uint4*)src, (size_t)bytes / 16, (unsigned*)sink);
  RA_LAUNCH_CHECK("stream_read");
  return 0;
}

// Runs `iters` iterations (eight 16x16x32 products, or four 32x32x16 ones; measured on MI355X both
// shapes give 2.1 to 2.45 PFLOP/s, depending on how warm the chip is) in `waves_per_cu` waves on every
// CU; *flops is what all of them did.
extern "C" int ra_mfma_loop(int shape, int iters, int waves_per_cu, void* sink, double* flops, hipStream_t stream) {
  RA_CHECK(shape == 16 || shape == 32, "mfma_loop: shape %d; 16 (16x16x32) or 32 (32x32x16)", shape);
  const bool big = shape == 32;
  RA_CHECK(iters > 0 && waves_per_cu >= 4 && waves_per_cu % 4 == 0 && waves_per_cu <= 32 && sink && flops,
           "mfma_loop: iterations (%d) and waves a CU (%d: a multiple of 4 up to 32)", iters, waves_per_cu);
  const int cus = ra_cu_count();
  RA_CHECK(cus > 0, "mfma_loop: no compute units reported");
  const int blocks = cus * (waves_per_cu / 4);
  if (big) mfma_loop32_kernel<<<blocks, 256, 0, stream>>>(iters, (float*)sink);
  else mfma_loop_kernel<<<blocks, 256, 0, stream>>>(iters, (float*)sink);
  RA_LAUNCH_CHECK("mfma_loop");
  *flops = (double)blocks * 4.0 * (double)iters * (big ? 4.0 * (2.0 * 32 * 32 * 16) : 8.0 * (2.0 * 16 * 16 * 32));
  return 0;
}
