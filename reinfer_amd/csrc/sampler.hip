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
#include <mutex>
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

// ---------------------------------------------------------------------------
// The same two stages for callers that cannot allocate: the slice winners go
// to a file-scope array of device memory instead of buffers the caller brings.
// Each GPU holds its own copy of the array, at its own address, until the
// process ends (SAMPLE_STATIC_PAIRS * 8 bytes = 512 KiB). In host code the
// array's name is only a handle for hipGetSymbolAddress: the address it
// yields, looked up once per device with that device current, is what the
// kernels get. Stage 1 writes every pair that stage 2 reads, so nothing has to
// be cleared between calls; what an earlier call left beyond that is never read.
// ---------------------------------------------------------------------------
#define SAMPLE_STATIC_PAIRS 65536            // (row, slice) pairs a call may need
#define SAMPLE_STATIC_DEVICES 64

static __device__ __align__(256) unsigned char scratch[SAMPLE_STATIC_PAIRS * (sizeof(float) + sizeof(int))];

static void* scratch_of_device[SAMPLE_STATIC_DEVICES];     // device address of `scratch`, per GPU
static std::mutex scratch_lock;

static int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  RA_CHECK(e == hipSuccess, "sample_static: no current device: %s", hipGetErrorString(e));
  RA_CHECK(dev >= 0 && dev < SAMPLE_STATIC_DEVICES, "sample_static: device %d (at most %d are known)", dev,
           SAMPLE_STATIC_DEVICES);
  std::lock_guard<std::mutex> hold(scratch_lock);
  if (scratch_of_device[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    RA_CHECK(e == hipSuccess && p != nullptr, "sample_static: the scratch array has no address on device %d: %s", dev,
             hipGetErrorString(e));
    scratch_of_device[dev] = p;
  }
  *out = scratch_of_device[dev];
  return 0;
}

extern "C" long ra_sample_static_max_pairs(void) { return SAMPLE_STATIC_PAIRS; }

// Looks the array's address up for the current device, so that no later call has to: a caller that will
// run ra_sample_static under stream capture calls this once per device beforehand (a first call inside a
// capture would make the lookup inside it).
extern "C" int ra_sample_static_prepare(void) {
  void* base = nullptr;
  return static_scratch(&base);
}

extern "C" int ra_sample_static(const float* logits, int n_rows, int vocab, int row_stride,
                                const float* temperature, const long long* seeds, const int* positions,
                                int* tokens, hipStream_t stream) {
  RA_CHECK(n_rows > 0 && vocab > 0, "sample_static: empty input (%d rows, vocabulary %d)", n_rows, vocab);
  RA_CHECK(row_stride >= vocab, "sample_static: row stride %d below the vocabulary %d", row_stride, vocab);
  RA_CHECK(n_rows <= 65535, "sample_static: %d rows in one launch (max 65535)", n_rows);
  const int n_slices = ra_sample_slices(vocab);
  RA_CHECK((long)n_rows * n_slices <= SAMPLE_STATIC_PAIRS,
           "sample_static: %d rows of %d slices need %ld pairs of scratch, the array holds %d "
           "(use ra_sample with buffers of your own)",
           n_rows, n_slices, (long)n_rows * n_slices, SAMPLE_STATIC_PAIRS);
  void* base = nullptr;
  if (static_scratch(&base) != 0) return 1;
  float* part_val = (float*)base;
  int* part_idx = (int*)((unsigned char*)base + SAMPLE_STATIC_PAIRS * sizeof(float));
  dim3 grid(n_slices, n_rows);
  sample_stage1<<<grid, SAMPLE_THREADS, 0, stream>>>(logits, vocab, row_stride, temperature, seeds,
                                                     positions, part_val, part_idx, n_slices);
  RA_LAUNCH_CHECK("sample_static stage 1");
  sample_stage2<<<n_rows, SAMPLE_THREADS, 0, stream>>>(part_val, part_idx, n_slices, tokens);
  RA_LAUNCH_CHECK("sample_static stage 2");
  return 0;
}

// ---------------------------------------------------------------------------
// Filters and penalties, applied to a row of logits in place before ra_sample:
//   frequency/presence: logit -= count * freq + pres for tokens among the last
//     n of the request; repetition: logit > 0 divided, else multiplied by the
//     penalty (crates/cuda/kernels/sampler_kernel.cu:207-221);
//   then, on p = softmax(logit / T) and only if T > 0 (at T <= 0 the maximum
//     survives every filter, sampler_kernel.cu:236-252):
//   min_p: keep p >= min_p * max p; top_k: the k largest (value, then lower id);
//   top_p: keep p >= theta, theta the largest value with
//     sum_{kept, p >= theta} p >= top_p * (mass kept so far)
//   (order and boundary rules: sampler_kernel.cu:20-43, 287-372). Removed
//   tokens get -inf; ra_sample then applies the temperature and draws.
// One workgroup per row; counts and sums are reduced in a fixed order.
// ---------------------------------------------------------------------------
#define FILTER_THREADS 1024

__device__ __forceinline__ unsigned sortable(float v) {      // ascending order of floats as unsigned
  const unsigned b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

template <typename T>
__device__ __forceinline__ T filter_block_sum(T v, T* red) {
#pragma unroll
  for (int m = RA_WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, RA_WAVE);
  const int lane = threadIdx.x & (RA_WAVE - 1), wave = threadIdx.x / RA_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  T t = 0;
  for (int i = 0; i < FILTER_THREADS / RA_WAVE; ++i) t += red[i];
  return t;
}
__device__ __forceinline__ float filter_block_max(float v, float* red) {
  v = wave_max(v);
  const int lane = threadIdx.x & (RA_WAVE - 1), wave = threadIdx.x / RA_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = -INFINITY;
  for (int i = 0; i < FILTER_THREADS / RA_WAVE; ++i) t = fmaxf(t, red[i]);
  return t;
}

struct FilterRow {           // one per row, in device memory
  float temperature, top_p, min_p, repeat_penalty, frequency_penalty, presence_penalty;
  int top_k, window_off, window_len;
  int bias_off, bias_len;      // logit bias: bias_len pairs (token id, float bits) at window[bias_off]
  int pad;
};

__global__ void __launch_bounds__(FILTER_THREADS)
filter_logits_kernel(float* __restrict__ logits, int vocab, int row_stride, const FilterRow* __restrict__ rows,
                     const int* __restrict__ window) {
  __shared__ float redf[FILTER_THREADS / RA_WAVE];
  __shared__ unsigned long long redu[FILTER_THREADS / RA_WAVE];
  const FilterRow fr = rows[blockIdx.x];
  float* lg = logits + (size_t)blockIdx.x * row_stride;
  const int tid = threadIdx.x;

  // additive bias per token id, before everything else (crates/cuda/kernels/sampler_kernel.cu:189-203);
  // the caller lists every id once
  if (fr.bias_len > 0) {
    const int* bp = window + fr.bias_off;
    for (int b = tid; b < fr.bias_len; b += FILTER_THREADS) {
      const int tok = bp[2 * b];
      if (tok < 0 || tok >= vocab) continue;
      const float l = lg[tok];
      if (isfinite(l)) lg[tok] = l + __int_as_float(bp[2 * b + 1]);
    }
    __syncthreads();
  }
  // penalties: the first occurrence of a token in the window carries its count
  const bool pen = fr.repeat_penalty > 1.f || fr.frequency_penalty > 0.f || fr.presence_penalty > 0.f;
  if (pen && fr.window_len > 0) {
    const int* win = window + fr.window_off;
    for (int w = tid; w < fr.window_len; w += FILTER_THREADS) {
      const int tok = win[w];
      if (tok < 0 || tok >= vocab) continue;
      bool first = true;
      int cnt = 0;
      for (int x = 0; x < fr.window_len; ++x) {
        if (win[x] == tok) {
          if (x < w) { first = false; break; }
          ++cnt;
        }
      }
      if (!first) continue;
      float l = lg[tok];
      if (!isfinite(l)) continue;
      l -= fr.frequency_penalty * (float)cnt + fr.presence_penalty;
      if (fr.repeat_penalty > 1.f) l = l > 0.f ? l / fr.repeat_penalty : l * fr.repeat_penalty;
      lg[tok] = l;
    }
    __syncthreads();
  }
  const float T = fr.temperature;
  const bool use_k = fr.top_k > 0 && fr.top_k < vocab;
  const bool use_p = fr.top_p > 0.f && fr.top_p < 1.f;
  const bool use_m = fr.min_p > 0.f;
  if (!(T > 0.f) || !(use_k || use_p || use_m)) return;

  // x = logit / T; e = exp(x - max x) = p / max p
  float mx = -INFINITY;
  for (int v = tid; v < vocab; v += FILTER_THREADS) {
    const float l = lg[v];
    if (isfinite(l)) mx = fmaxf(mx, l / T);
  }
  mx = filter_block_max(mx, redf);
  if (mx == -INFINITY) return;               // no finite logit: ra_sample reports it
  // what is kept so far is described by two thresholds: e >= e_min and key >= key_min
  float e_min = use_m ? fr.min_p : 0.f;      // min_p: p >= min_p * max p  <=>  e >= min_p
  unsigned long long key_min = 0ull;
  auto key_of = [&](int v, float x) { return ((unsigned long long)sortable(x) << 32) | (unsigned)(~v); };
  if (use_k) {
    // the k-th largest (value, lower id first) pair by bisection on the 64-bit key
    unsigned long long lo = 0ull, hi = ~0ull;           // count(key >= lo) >= k > count(key >= hi)
    for (int round = 0; round < 64 && hi - lo > 1ull; ++round) {
      const unsigned long long mid = lo + (hi - lo) / 2ull;
      unsigned long long c = 0ull;
      for (int v = tid; v < vocab; v += FILTER_THREADS) {
        const float l = lg[v];
        if (isfinite(l) && key_of(v, l / T) >= mid) ++c;
      }
      c = filter_block_sum<unsigned long long>(c, redu);
      if (c >= (unsigned long long)fr.top_k) lo = mid; else hi = mid;
    }
    key_min = lo;
  }
  float theta = 0.f;                          // top_p boundary on e
  if (use_p) {
    float zs = 0.f;
    for (int v = tid; v < vocab; v += FILTER_THREADS) {
      const float l = lg[v];
      if (!isfinite(l)) continue;
      const float x = l / T, e = __expf(x - mx);
      if (e >= e_min && key_of(v, x) >= key_min) zs += e;
    }
    zs = filter_block_sum<float>(zs, redf);
    const float need = fr.top_p * zs;
    float flo = 0.f, fhi = 1.f;               // mass(e >= flo) >= need; e <= 1 always
    for (int round = 0; round < 30; ++round) {
      const float mid = 0.5f * (flo + fhi);
      float mass = 0.f;
      for (int v = tid; v < vocab; v += FILTER_THREADS) {
        const float l = lg[v];
        if (!isfinite(l)) continue;
        const float x = l / T, e = __expf(x - mx);
        if (e >= mid && e >= e_min && key_of(v, x) >= key_min) mass += e;
      }
      mass = filter_block_sum<float>(mass, redf);
      if (mass >= need) flo = mid; else fhi = mid;
    }
    theta = flo;
  }
  for (int v = tid; v < vocab; v += FILTER_THREADS) {
    const float l = lg[v];
    if (!isfinite(l)) continue;
    const float x = l / T, e = __expf(x - mx);
    if (!(e >= e_min && e >= theta && key_of(v, x) >= key_min)) lg[v] = -INFINITY;
  }
}

extern "C" int ra_filter_logits(float* logits, int n_rows, int vocab, int row_stride, const void* rows,
                                const int* window, hipStream_t stream) {
  RA_CHECK(n_rows > 0 && vocab > 0, "filter_logits: empty input (%d rows, vocabulary %d)", n_rows, vocab);
  RA_CHECK(row_stride >= vocab, "filter_logits: row stride %d below the vocabulary %d", row_stride, vocab);
  RA_CHECK(n_rows <= 65535, "filter_logits: %d rows in one launch (max 65535)", n_rows);
  RA_CHECK(rows != nullptr, "filter_logits: no row parameters");
  filter_logits_kernel<<<n_rows, FILTER_THREADS, 0, stream>>>(logits, vocab, row_stride, (const FilterRow*)rows, window);
  RA_LAUNCH_CHECK("filter_logits");
  return 0;
}
