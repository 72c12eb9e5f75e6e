// Flash-decode attention over the paged cache, bfloat16: one query token per
// (request, position), the query heads of one KV head handled together so that
// every key and value is read once for the whole group, the keys split over
// several workgroups (split-KV) and merged by a second small kernel.
//
// A workgroup of 256 threads takes (split, KV head, token). A key's row of d
// elements is spread over d/8 adjacent lanes, 16 bytes a lane, so a wavefront
// reads whole rows, consecutive keys of a block back to back. Each group of
// lanes keeps its own running maximum, sum and weighted values (online
// softmax, float), so the key loop has no workgroup barrier; the groups are
// merged once at the end (shuffles inside a wavefront, LDS across wavefronts).
// Dot products use v_dot2_f32_bf16 (float accumulate).
//
// The reference's flash decode keeps the whole score row in shared memory,
// which caps the context at (d + max_kv) * 4 <= 48 KB (crates/cuda/src/decode.rs:49-52;
// crates/cuda/kernels/decode_flash_kernels.cu:212-350), and takes one CTA per
// query head; the online form here has no such cap and shares K/V in a group.
#include "common.h"
#include "reinfer_hip.h"

#define FD_THREADS 256
#define FD_U 4

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// DLP: lanes per key row (a power of two >= d/8); G: query heads per KV head
template <int DLP, int G>
__global__ void __launch_bounds__(FD_THREADS)
flash_decode_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                    const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
                    const int* __restrict__ block_tables, int max_blocks,
                    const int* __restrict__ token_list, const int* __restrict__ seq_of_token,
                    const int* __restrict__ positions, int block_size, int Hkv, int d,
                    float scale_log2, int window, int n_splits, float* __restrict__ part_o,
                    float* __restrict__ part_ml) {
  constexpr int NSUB = FD_THREADS / DLP;          // key rows a workgroup reads per load
  constexpr int SUB_PER_WAVE = RA_WAVE / DLP;
  __shared__ float lds_o[FD_THREADS / RA_WAVE][G][DLP * 8];
  __shared__ float lds_ml[FD_THREADS / RA_WAVE][G][2];

  const int split = blockIdx.x, kvh = blockIdx.y, li = blockIdx.z;
  const int t = token_list ? token_list[li] : li;
  const int seq = seq_of_token[t];
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int n_keys = p + 1 - lo;
  int chunk = (n_keys + n_splits - 1) / n_splits;
  chunk = (chunk + NSUB * FD_U - 1) / (NSUB * FD_U) * (NSUB * FD_U);
  const int start = lo + split * chunk;
  const int end = min(p + 1, start + chunk);

  const int tid = threadIdx.x;
  const int dc = tid % DLP, sub = tid / DLP;
  const int DL = d / 8;
  const bool active = dc < DL;
  const int Hq = Hkv * G;
  const int* table = block_tables + (size_t)seq * max_blocks;

  // this lane's 8 elements of each query head of the group, as bfloat16 pairs
  bf16x2_t qp[G][4];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    bf16x8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (active) v = *(const bf16x8_t*)(q + (size_t)t * q_stride + (size_t)(kvh * G + h) * d + dc * 8);
#pragma unroll
    for (int j = 0; j < 4; ++j) qp[h][j] = (bf16x2_t){v[2 * j], v[2 * j + 1]};
  }
  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[h][j] = 0.f;
  }

  for (int base = start; base < end; base += NSUB * FD_U) {
    bf16x8_t kx[FD_U], vx[FD_U];
    bool ok[FD_U];
#pragma unroll
    for (int u = 0; u < FD_U; ++u) {
      const int key = base + u * NSUB + sub;
      ok[u] = key < end;
      kx[u] = (bf16x8_t){0, 0, 0, 0, 0, 0, 0, 0};
      vx[u] = kx[u];
      if (ok[u] && active) {
        const int blk = table[key / block_size];
        const size_t off = (((size_t)blk * Hkv + kvh) * block_size + key % block_size) * d + dc * 8;
        kx[u] = *(const bf16x8_t*)(kcache + off);
        vx[u] = *(const bf16x8_t*)(vcache + off);
      }
    }
    float s[FD_U][G];
#pragma unroll
    for (int u = 0; u < FD_U; ++u) {
#pragma unroll
      for (int h = 0; h < G; ++h) {
        float dot = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          dot = __builtin_amdgcn_fdot2_f32_bf16((bf16x2_t){kx[u][2 * j], kx[u][2 * j + 1]}, qp[h][j], dot, false);
#pragma unroll
        for (int o = DLP / 2; o > 0; o >>= 1) dot += __shfl_xor(dot, o, RA_WAVE);
        s[u][h] = ok[u] ? dot * scale_log2 : -INFINITY;
      }
    }
    float vf[FD_U][8];
#pragma unroll
    for (int u = 0; u < FD_U; ++u)
#pragma unroll
      for (int j = 0; j < 8; ++j) vf[u][j] = (float)vx[u][j];
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float mn = m[h];
#pragma unroll
      for (int u = 0; u < FD_U; ++u) mn = fmaxf(mn, s[u][h]);
      if (mn == -INFINITY) continue;           // nothing seen yet and nothing here
      const float corr = fast_exp2(m[h] - mn);  // m = -inf gives 0
      float pr[FD_U], psum = 0.f;
#pragma unroll
      for (int u = 0; u < FD_U; ++u) {
        pr[u] = fast_exp2(s[u][h] - mn);        // masked keys: exp2(-inf) = 0
        psum += pr[u];
      }
      l[h] = l[h] * corr + psum;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float a = acc[h][j] * corr;
#pragma unroll
        for (int u = 0; u < FD_U; ++u) a = fmaf(pr[u], vf[u][j], a);
        acc[h][j] = a;
      }
      m[h] = mn;
    }
  }

  // merge the lane groups of a wavefront (same d chunk, different keys)
#pragma unroll
  for (int o = DLP; o < RA_WAVE; o <<= 1) {
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const float mo = __shfl_xor(m[h], o, RA_WAVE);
      const float mn = fmaxf(m[h], mo);
      const float c = (mn == -INFINITY) ? 0.f : fast_exp2(m[h] - mn);
      const float ls = l[h] * c;
      l[h] = ls + __shfl_xor(ls, o, RA_WAVE);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float a = acc[h][j] * c;
        acc[h][j] = a + __shfl_xor(a, o, RA_WAVE);
      }
      m[h] = mn;
    }
  }
  // across wavefronts through LDS
  const int wave = tid / RA_WAVE, lane = tid % RA_WAVE;
  if (lane < DLP) {
#pragma unroll
    for (int h = 0; h < G; ++h) {
#pragma unroll
      for (int j = 0; j < 8; ++j) lds_o[wave][h][lane * 8 + j] = acc[h][j];
      if (lane == 0) {
        lds_ml[wave][h][0] = m[h];
        lds_ml[wave][h][1] = l[h];
      }
    }
  }
  __syncthreads();
  constexpr int NW = FD_THREADS / RA_WAVE;
  for (int idx = tid; idx < G * DL * 8; idx += FD_THREADS) {
    const int h = idx / (DL * 8), e = idx % (DL * 8);
    float mn = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) mn = fmaxf(mn, lds_ml[w][h][0]);
    float lt = 0.f, ot = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float c = (mn == -INFINITY) ? 0.f : fast_exp2(lds_ml[w][h][0] - mn);
      lt += lds_ml[w][h][1] * c;
      ot += lds_o[w][h][e] * c;
    }
    const int head = kvh * G + h;
    if (n_splits == 1) {
      out[(size_t)t * out_stride + (size_t)head * d + e] = from_f32<bf16_t>(ot / lt);
    } else {
      const size_t row = ((size_t)li * Hq + head) * n_splits + split;
      part_o[row * d + e] = ot;
      if (e == 0) {
        part_ml[row * 2] = mn;
        part_ml[row * 2 + 1] = lt;
      }
    }
  }
}

// merge the splits of one (token, head): fixed order, float
__global__ void flash_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                          bf16_t* __restrict__ out, int out_stride,
                                          const int* __restrict__ token_list, int Hq, int d, int n_splits) {
  const int head = blockIdx.x, li = blockIdx.y;
  const int t = token_list ? token_list[li] : li;
  const size_t row0 = ((size_t)li * Hq + head) * n_splits;
  float mn = -INFINITY;
  for (int s = 0; s < n_splits; ++s) mn = fmaxf(mn, part_ml[(row0 + s) * 2]);
  float lt = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float ms = part_ml[(row0 + s) * 2];
    lt += (ms == -INFINITY) ? 0.f : part_ml[(row0 + s) * 2 + 1] * fast_exp2(ms - mn);
  }
  for (int e = threadIdx.x; e < d; e += blockDim.x) {
    float o = 0.f;
    for (int s = 0; s < n_splits; ++s) {
      const float ms = part_ml[(row0 + s) * 2];
      if (ms != -INFINITY) o += part_o[(row0 + s) * d + e] * fast_exp2(ms - mn);
    }
    out[(size_t)t * out_stride + (size_t)head * d + e] = from_f32<bf16_t>(o / lt);
  }
}

template <int DLP>
static int launch_fd(int G, dim3 grid, hipStream_t stream, const bf16_t* q, int q_stride, bf16_t* out,
                     int out_stride, const bf16_t* kc, const bf16_t* vc, const int* tables, int max_blocks,
                     const int* token_list, const int* seq_of_token, const int* positions, int block_size,
                     int Hkv, int d, float scale_log2, int window, int n_splits, float* part_o,
                     float* part_ml) {
#define RA_FD(GG)                                                                                    \
  case GG:                                                                                           \
    flash_decode_kernel<DLP, GG><<<grid, FD_THREADS, 0, stream>>>(                                   \
        q, q_stride, out, out_stride, kc, vc, tables, max_blocks, token_list, seq_of_token,          \
        positions, block_size, Hkv, d, scale_log2, window, n_splits, part_o, part_ml);               \
    break;
  switch (G) {
    RA_FD(1) RA_FD(2) RA_FD(3) RA_FD(4) RA_FD(5) RA_FD(6) RA_FD(7) RA_FD(8)
    default:
      return ra_fail("attention_decode: %d query heads per KV head (this kernel takes 1..8)", G);
  }
#undef RA_FD
  RA_LAUNCH_CHECK("attention_decode");
  return 0;
}

// 1 if the kernel takes these sizes, else 0 (the caller then uses the plain kernel)
extern "C" int ra_attention_decode_supports(int Hq, int Hkv, int d) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return 0;
  const int G = Hq / Hkv;
  return (G >= 1 && G <= 8 && d % 8 == 0 && d >= 16 && d <= 256) ? 1 : 0;
}

extern "C" int ra_attention_decode(const void* q, int q_stride, void* out, int out_stride,
                                   const void* kcache, const void* vcache, const int* block_tables,
                                   int max_blocks, const int* token_list, const int* seq_of_token,
                                   const int* positions, int n_tokens, int block_size, int Hq, int Hkv,
                                   int d, float scale, int window, int n_splits, float* part_o,
                                   float* part_ml, hipStream_t stream) {
  RA_CHECK(n_tokens > 0, "attention_decode: no tokens");
  RA_CHECK(ra_attention_decode_supports(Hq, Hkv, d),
           "attention_decode: unsupported sizes (%d query heads, %d KV heads, head size %d)", Hq, Hkv, d);
  RA_CHECK(block_size > 0 && max_blocks > 0 && window >= 0, "attention_decode: bad cache geometry");
  RA_CHECK(n_splits >= 1 && n_splits <= 256, "attention_decode: %d splits outside 1..256", n_splits);
  RA_CHECK(n_splits == 1 || (part_o && part_ml), "attention_decode: split-KV needs the partial buffers");
  RA_CHECK(q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)kcache % 16) == 0 &&
               ((uintptr_t)vcache % 16) == 0,
           "attention_decode: operands must be 16-byte aligned");
  RA_CHECK(n_tokens <= 65535 && Hkv <= 65535, "attention_decode: grid too large");
  const int G = Hq / Hkv;
  const int DL = d / 8;
  dim3 grid(n_splits, Hkv, n_tokens);
  const float scale_log2 = scale * 1.4426950408889634f;
  int rc;
#define RA_ARGS                                                                                       \
  G, grid, stream, (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kcache,      \
      (const bf16_t*)vcache, block_tables, max_blocks, token_list, seq_of_token, positions,          \
      block_size, Hkv, d, scale_log2, window, n_splits, part_o, part_ml
  if (DL <= 2) rc = launch_fd<2>(RA_ARGS);
  else if (DL <= 4) rc = launch_fd<4>(RA_ARGS);
  else if (DL <= 8) rc = launch_fd<8>(RA_ARGS);
  else if (DL <= 16) rc = launch_fd<16>(RA_ARGS);
  else rc = launch_fd<32>(RA_ARGS);
#undef RA_ARGS
  if (rc) return rc;
  if (n_splits > 1) {
    dim3 mg(Hq, n_tokens);
    flash_decode_merge_kernel<<<mg, 64, 0, stream>>>(part_o, part_ml, (bf16_t*)out, out_stride,
                                                     token_list, Hq, d, n_splits);
    RA_LAUNCH_CHECK("attention_decode merge");
  }
  return 0;
}
