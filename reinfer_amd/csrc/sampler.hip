// On-GPU sampling over [rows, vocab] float logits, many workgroups per row.
//   temperature <= 0: the first maximum (lowest id among equal maxima;
//     crates/cuda/src/engine.rs:6512-6520)
//   temperature  > 0: Gumbel-max, argmax_v( logit_v / T + g_v ),
//     g_v = -ln(-ln u_v), u_v = top 24 bits of mix(base ^ mix(v)) / 2^24
//     (crates/cuda/kernels/sampler_kernel.cu:61-77, 364-397), with
//     base = splitmix64(seed ^ position * golden): a pure function of the
//     request's seed, the position and the token id
//     (crates/scheduler/src/rng.rs:52-58), so a token does not depend on
//     what else is in the batch.
// Non-finite logits never win; a row without a finite logit yields -1.
// The reference's sampler is one 256-thread workgroup
// (sampler_kernel.cu:157); here stage 1 scans slices of the row in parallel
// and stage 2 merges the slice winners in a fixed order.
#include "common.h"
#include "reinfer_hip.h"

#define SAMPLE_THREADS 256
#define SAMPLE_SLICE 2048

__device__ __forceinline__ unsigned long long mix64(unsigned long long z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
__device__ __forceinline__ unsigned long long splitmix64(unsigned long long x) {
  return mix64(x + 0x9E3779B97F4A7C15ull);
}

struct Best {
  float val;
  int idx;
};
__device__ __forceinline__ Best better(Best a, Best b) {
  if (b.idx < 0) return a;
  if (a.idx < 0) return b;
  if (b.val > a.val || (b.val == a.val && b.idx < a.idx)) return b;
  return a;
}

__device__ __forceinline__ Best block_best(Best b, Best* red) {
#pragma unroll
  for (int m = RA_WAVE / 2; m > 0; m >>= 1) {
    Best o;
    o.val = __shfl_xor(b.val, m, RA_WAVE);
    o.idx = __shfl_xor(b.idx, m, RA_WAVE);
    b = better(b, o);
  }
  const int lane = threadIdx.x & (RA_WAVE - 1), wave = threadIdx.x / RA_WAVE;
  if (lane == 0) red[wave] = b;
  __syncthreads();
  Best r = red[0];
  for (int i = 1; i < SAMPLE_THREADS / RA_WAVE; ++i) r = better(r, red[i]);
  return r;
}

__global__ void sample_stage1(const float* __restrict__ logits, int vocab, int row_stride,
                              const float* __restrict__ temperature,
                              const long long* __restrict__ seeds, const int* __restrict__ positions,
                              float* __restrict__ part_val, int* __restrict__ part_idx, int n_slices) {
  __shared__ Best red[SAMPLE_THREADS / RA_WAVE];
  const int row = blockIdx.y, slice = blockIdx.x;
  const float* lg = logits + (size_t)row * row_stride;
  const float T = temperature[row];
  const unsigned long long base =
      splitmix64((unsigned long long)seeds[row] ^ ((unsigned long long)positions[row] * 0x9E3779B97F4A7C15ull));
  Best b;
  b.val = -INFINITY;
  b.idx = -1;
  const int end = min(vocab, (slice + 1) * SAMPLE_SLICE);
  for (int v = slice * SAMPLE_SLICE + threadIdx.x; v < end; v += SAMPLE_THREADS) {
    float x = lg[v];
    if (!isfinite(x)) continue;
    if (T > 0.f) {
      const float u = (float)(mix64(base ^ mix64((unsigned long long)v)) >> 40) * (1.0f / 16777216.0f);
      if (u <= 0.f) continue;            // -ln(-ln 0) = -inf: never wins
      x = x / T - logf(-logf(u));
    }
    Best c;
    c.val = x;
    c.idx = v;
    b = better(b, c);
  }
  b = block_best(b, red);
  if (threadIdx.x == 0) {
    part_val[(size_t)row * n_slices + slice] = b.val;
    part_idx[(size_t)row * n_slices + slice] = b.idx;
  }
}

__global__ void sample_stage2(const float* __restrict__ part_val, const int* __restrict__ part_idx,
                              int n_slices, int* __restrict__ tokens) {
  __shared__ Best red[SAMPLE_THREADS / RA_WAVE];
  const int row = blockIdx.x;
  Best b;
  b.val = -INFINITY;
  b.idx = -1;
  for (int s = threadIdx.x; s < n_slices; s += SAMPLE_THREADS) {
    Best c;
    c.val = part_val[(size_t)row * n_slices + s];
    c.idx = part_idx[(size_t)row * n_slices + s];
    b = better(b, c);
  }
  b = block_best(b, red);
  if (threadIdx.x == 0) tokens[row] = b.idx;
}

extern "C" int ra_sample_slices(int vocab) { return (vocab + SAMPLE_SLICE - 1) / SAMPLE_SLICE; }

extern "C" int ra_sample(const float* logits, int n_rows, int vocab, int row_stride,
                         const float* temperature, const long long* seeds, const int* positions,
                         float* scratch_val, int* scratch_idx, int* tokens, hipStream_t stream) {
  RA_CHECK(n_rows > 0 && vocab > 0, "sample: empty input (%d rows, vocabulary %d)", n_rows, vocab);
  RA_CHECK(row_stride >= vocab, "sample: row stride %d below the vocabulary %d", row_stride, vocab);
  RA_CHECK(n_rows <= 65535, "sample: %d rows in one launch (max 65535)", n_rows);
  const int n_slices = ra_sample_slices(vocab);
  dim3 grid(n_slices, n_rows);
  sample_stage1<<<grid, SAMPLE_THREADS, 0, stream>>>(logits, vocab, row_stride, temperature, seeds,
                                                     positions, scratch_val, scratch_idx, n_slices);
  RA_LAUNCH_CHECK("sample stage 1");
  sample_stage2<<<n_rows, SAMPLE_THREADS, 0, stream>>>(scratch_val, scratch_idx, n_slices, tokens);
  RA_LAUNCH_CHECK("sample stage 2");
  return 0;
}
