// Row kernels of the step: embedding rows, fused residual-add + RMSNorm,
// fused per-head q/k norm + rotation + cache write, SiLU gate.
// Sums of squares, rsqrt, rotation angles and the residual sum are float;
// one rounding at the store.
#include "common.h"
#include "reinfer_hip.h"

thread_local char ra_error_text[512] = {0};

int ra_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(ra_error_text, sizeof(ra_error_text), fmt, ap);
  va_end(ap);
  return 1;
}

extern "C" const char* ra_last_error(void) { return ra_error_text; }

int ra_cu_count(void) {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = n;
  }
  return cus[dev];
}
extern "C" int ra_abi_version(void) { return RA_ABI_VERSION; }

// ---------------------------------------------------------------------------
// embedding rows into the float residual stream: out[t, :] = table[ids[t], :]
// (reference: gather_row, crates/cuda/kernels/dense_kernels.cu:329-336)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int h) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * h;
  float* o = out + (size_t)t * h;
  for (int i = threadIdx.x; i < h; i += blockDim.x) o[i] = to_f32(row[i]);
}

extern "C" int ra_embed(const void* table, int table_dtype, const int* ids, float* out, int n_tokens,
                        int hidden, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && hidden > 0, "embed: empty input (%d tokens, width %d)", n_tokens, hidden);
  if (table_dtype == RA_F32)
    embed_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)table, ids, out, hidden);
  else if (table_dtype == RA_BF16)
    embed_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const bf16_t*)table, ids, out, hidden);
  else
    return ra_fail("embed: unknown dtype tag %d", table_dtype);
  RA_LAUNCH_CHECK("embed");
  return 0;
}

// ---------------------------------------------------------------------------
// Fused residual add + RMSNorm (any width).
//   in place (rows == null):  resid[r] += delta[r];  out[r] = rms(resid[r]) * w
//   gathered (rows != null):  out[i] = rms(resid[rows[i]] + delta[rows[i]]) * w
// y = x * rsqrt(mean(x^2) + eps) * w   (crates/cuda/kernels/dense_kernels.cu:59-88,
// fused add form :257-274; there limited to n <= 1024 and one row).
// ---------------------------------------------------------------------------
template <typename TA, typename TW>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TA* __restrict__ delta,
                                   const TW* __restrict__ w, TA* __restrict__ out,
                                   const int* __restrict__ rows, int h, float eps) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * h;
  const TA* dl = delta ? delta + src * h : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    float v = x[i];
    if (dl) {
      v += to_f32(dl[i]);
      if (!rows) x[i] = v;      // the same thread reads it back below
    }
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float rstd = rsqrtf(ss / (float)h + eps);
  TA* o = out + (size_t)r * h;
  for (int i = threadIdx.x; i < h; i += blockDim.x) {
    float v = x[i];
    if (dl && rows) v += to_f32(dl[i]);
    o[i] = from_f32<TA>(v * rstd * to_f32(w[i]));
  }
}

// The same for rows that fit the workgroup's registers (width a multiple of 4, at
// most threads * 16): one read of the row, the sum in registers, one write. A
// decode step runs this on a handful of rows, so its time is the chain of memory
// round trips, not bandwidth; the plain kernel above reads the row a second time.
typedef float f32x4_raw __attribute__((ext_vector_type(4)));

template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ f32x4_raw load(const float* p) { return *(const f32x4_raw*)p; }
  static __device__ __forceinline__ void store(float* p, f32x4_raw v) { *(f32x4_raw*)p = v; }
};
template <> struct Vec4<bf16_t> {
  static __device__ __forceinline__ f32x4_raw load(const bf16_t* p) {
    const bf16x4_t v = *(const bf16x4_t*)p;
    return (f32x4_raw){(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
  }
  static __device__ __forceinline__ void store(bf16_t* p, f32x4_raw v) {
    *(bf16x4_t*)p = (bf16x4_t){(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
  }
};

#define NORM_CH 4       // chunks of 4 elements a thread keeps

template <typename TA, typename TW>
__global__ void add_rmsnorm_reg_kernel(float* __restrict__ resid, const TA* __restrict__ delta,
                                       const TW* __restrict__ w, TA* __restrict__ out,
                                       const int* __restrict__ rows, int h, float eps) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  float* x = resid + src * h;
  const TA* dl = delta ? delta + src * h : nullptr;
  f32x4_raw v[NORM_CH], wv[NORM_CH];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NORM_CH; ++j) {
    const int i = (threadIdx.x + j * blockDim.x) * 4;
    v[j] = (f32x4_raw){0.f, 0.f, 0.f, 0.f};
    wv[j] = v[j];
    if (i < h) {
      v[j] = Vec4<float>::load(x + i);
      if (dl) v[j] += Vec4<TA>::load(dl + i);
      wv[j] = Vec4<TW>::load(w + i);
    }
  }
#pragma unroll
  for (int j = 0; j < NORM_CH; ++j) {
    const int i = (threadIdx.x + j * blockDim.x) * 4;
    if (i < h) {
      if (dl && !rows) Vec4<float>::store(x + i, v[j]);
      ss += v[j][0] * v[j][0] + v[j][1] * v[j][1] + v[j][2] * v[j][2] + v[j][3] * v[j][3];
    }
  }
  ss = block_sum(ss, red);
  const float rstd = rsqrtf(ss / (float)h + eps);
  TA* o = out + (size_t)r * h;
#pragma unroll
  for (int j = 0; j < NORM_CH; ++j) {
    const int i = (threadIdx.x + j * blockDim.x) * 4;
    if (i < h) Vec4<TA>::store(o + i, v[j] * rstd * wv[j]);
  }
}

extern "C" int ra_add_rmsnorm(float* resid, const void* delta, const void* weight, int weight_dtype,
                              void* out, int act_dtype, const int* rows, int n_rows, int hidden,
                              float eps, hipStream_t stream) {
  RA_CHECK(n_rows > 0 && hidden > 0, "add_rmsnorm: empty input (%d rows, width %d)", n_rows, hidden);
  int threads = hidden >= 2048 ? 512 : 256;
  const bool aligned = hidden % 4 == 0 && ((uintptr_t)resid % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                       ((uintptr_t)weight % 16) == 0 && ((uintptr_t)delta % 16) == 0;
  bool in_regs = aligned && hidden <= 1024 * 4 * NORM_CH;
  if (in_regs) {
    threads = 64;
    while (threads * 4 * NORM_CH < hidden) threads *= 2;
    if (hidden >= 2048 && threads < 256) threads = 256;
  }
#define RA_GO(TA, TW)                                                                                  \
  do {                                                                                                 \
    if (in_regs)                                                                                       \
      add_rmsnorm_reg_kernel<TA, TW><<<n_rows, threads, 0, stream>>>(                                  \
          resid, (const TA*)delta, (const TW*)weight, (TA*)out, rows, hidden, eps);                    \
    else                                                                                               \
      add_rmsnorm_kernel<TA, TW><<<n_rows, threads, 0, stream>>>(resid, (const TA*)delta,             \
                                                                 (const TW*)weight, (TA*)out, rows,    \
                                                                 hidden, eps);                         \
  } while (0)
  if (act_dtype == RA_F32 && weight_dtype == RA_F32) RA_GO(float, float);
  else if (act_dtype == RA_BF16 && weight_dtype == RA_BF16) RA_GO(bf16_t, bf16_t);
  else if (act_dtype == RA_BF16 && weight_dtype == RA_F32) RA_GO(bf16_t, float);
  else return ra_fail("add_rmsnorm: unsupported dtypes (activations %d, weight %d)", act_dtype, weight_dtype);
#undef RA_GO
  RA_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------
// Fused per-head RMSNorm of q and k, rotation, and cache write.
// qkv: [T, (Hq + 2 Hkv) * d]; q heads are normalised + rotated in place, k heads
// are normalised + rotated and stored at the token's cache slot, v heads are
// copied there. One wavefront per (token, head).
//   head norm: u * rsqrt(mean(u^2) + eps) * g, one g[d] for all heads, before the
//     rotation (crates/cuda/kernels/dense_kernels.cu:92-123; engine.rs:4122-4147)
//   rotation: pairs (j, j + R/2) [style 0, half split] or (2j, 2j+1) [style 1],
//     angle = pos * inv_freq[j] (dense_kernels.cu:125-139)
//   cache: [block][kv head][block_size * d] in the tiled order of cache_k_index /
//     cache_v_index (write: dense_kernels.cu:298-318)
// ---------------------------------------------------------------------------
#define QK_WAVES 4
#define QK_MAX_D 512

// The q/k/v product as the K ranges of a split product left it, not yet added (parts null: qkv holds the
// finished product and q is rotated in place): float [n_ranges][T][width], added here in range order, with
// the row factor of an RMSNorm carried by that product (in_ss null: none); the rotated q then goes to q_out.
struct QkSums {
  const float* parts;
  int n_ranges;
  size_t range_stride;     // T * width
  const float* in_ss;      // [in_parts][T]
  int in_parts;
  float in_eps, in_inv_width;
  void* q_out;             // [T][q_stride] in the activations' type
  int q_stride;
};

template <typename TA, typename TW>
__global__ void qk_norm_rope_cache_kernel(TA* __restrict__ qkv, const TW* __restrict__ q_w,
                                          const TW* __restrict__ k_w, float eps,
                                          const int* __restrict__ positions,
                                          const float* __restrict__ inv_freq, int rotary_dim,
                                          int rope_style, const int* __restrict__ slots,
                                          TA* __restrict__ kcache, TA* __restrict__ vcache,
                                          int block_size, int Hq, int Hkv, int d, QkSums sm) {
  __shared__ float buf[QK_WAVES][QK_MAX_D];
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int t = blockIdx.y;
  const int head = blockIdx.x * QK_WAVES + wave;
  const int n_heads = Hq + 2 * Hkv;
  const bool live = head < n_heads;
  TA* u = qkv + ((size_t)t * n_heads + (live ? head : 0)) * d;
  const bool is_q = head < Hq;
  const bool is_k = !is_q && head < Hq + Hkv;
  const int kvh = is_q ? 0 : (is_k ? head - Hq : head - Hq - Hkv);
  const int slot = slots[t];
  TA* slab = nullptr;           // the (block, kv head) slab a k or v head goes to
  int off = 0;                  // its slot there
  if (live && !is_q && slot >= 0) {
    const size_t blk = (size_t)(slot / block_size);
    off = slot % block_size;
    slab = (is_k ? kcache : vcache) + (blk * Hkv + kvh) * (size_t)block_size * d;
  }
  float* b = buf[wave];
  float ss = 0.f;
  if (live) {
    if (sm.parts) {
      float row = 1.f;
      if (sm.in_ss) {
        float tsum = 0.f;                      // the lanes share the parts out: a lane's ascending, then the lanes
        for (int p = lane; p < sm.in_parts; p += RA_WAVE) tsum += sm.in_ss[(size_t)p * gridDim.y + t];
        tsum = wave_sum(tsum);
        row = rsqrtf(tsum * sm.in_inv_width + sm.in_eps);
      }
      const float* src = sm.parts + ((size_t)t * n_heads + head) * d;
      for (int i = lane; i < d; i += RA_WAVE) {
        float v = 0.f;                         // range order; six ranges' values asked for in one trip
        constexpr int U = 6;
        for (int r0 = 0; r0 < sm.n_ranges; r0 += U) {
          float tv[U];
#pragma unroll
          for (int j = 0; j < U; ++j) tv[j] = src[(size_t)min(r0 + j, sm.n_ranges - 1) * sm.range_stride + i];
#pragma unroll
          for (int j = 0; j < U; ++j) v += r0 + j < sm.n_ranges ? tv[j] : 0.f;
        }
        v *= row;
        b[i] = v;
        ss += v * v;
      }
    } else {
      for (int i = lane; i < d; i += RA_WAVE) {
        float v = to_f32(u[i]);
        b[i] = v;
        ss += v * v;
      }
    }
  }
  __syncthreads();
  if (!live) return;
  if (!is_q && !is_k) {          // v head: plain copy
    if (slab)
      for (int i = lane; i < d; i += RA_WAVE) slab[cache_v_index(off, i, d)] = from_f32<TA>(b[i]);
    return;
  }
  const TW* w = is_q ? q_w : k_w;
  float rstd = 1.f;
  if (w) {
    ss = wave_sum(ss);
    rstd = rsqrtf(ss / (float)d + eps);
  }
  if (!is_q && !slab) return;
  // where element i of the head goes: in place for q, the cache slab for k
  TA* q_to = sm.parts ? (TA*)sm.q_out + (size_t)t * sm.q_stride + (size_t)head * d : u;
  auto put = [&](int i, float v) {
    if (is_q) q_to[i] = from_f32<TA>(v);
    else slab[cache_k_index(off, i, d)] = from_f32<TA>(v);
  };
  const float pos = (float)positions[t];
  const int half = rotary_dim / 2;
  for (int j = lane; j < half; j += RA_WAVE) {
    const int i0 = rope_style == 0 ? j : 2 * j;
    const int i1 = rope_style == 0 ? j + half : 2 * j + 1;
    float a = b[i0] * rstd, c = b[i1] * rstd;
    if (w) {
      a *= to_f32(w[i0]);
      c *= to_f32(w[i1]);
    }
    float sn, cs;
    sincosf(pos * inv_freq[j], &sn, &cs);
    put(i0, a * cs - c * sn);
    put(i1, a * sn + c * cs);
  }
  for (int i = rotary_dim + lane; i < d; i += RA_WAVE) {
    float a = b[i] * rstd;
    if (w) a *= to_f32(w[i]);
    put(i, a);
  }
}

// The same for few tokens of the common shape (half-split rotation over the whole head, head size 64,
// 128 or 256, the product already added): one wave per (token, head), and one trip to memory. A decode
// step's launch of this kernel does almost no work, so its time is the trips to memory that wait for
// each other; here the token's slot and position, the head's elements, the norm weights and the
// frequencies are all asked for before the first of them is used. A lane holds elements lane + 64 k: for
// EPL >= 2 both members of its rotation pairs (j, j + d/2); for EPL = 1 the partner sits 32 lanes away.
// An element as its bits in a register of its own: nothing is computed on a loaded value (a conversion,
// a packing of two halves) before the last load is out.
__device__ __forceinline__ unsigned raw_bits(const float* p, int i) { return ((const unsigned*)p)[i]; }
__device__ __forceinline__ unsigned raw_bits(const bf16_t* p, int i) { return (unsigned)((const unsigned short*)p)[i]; }
template <typename T> __device__ __forceinline__ float raw_value(unsigned bits);
template <> __device__ __forceinline__ float raw_value<float>(unsigned bits) { return __uint_as_float(bits); }
template <> __device__ __forceinline__ float raw_value<bf16_t>(unsigned bits) { return __uint_as_float(bits << 16); }

template <typename TA, typename TW, int EPL, bool NORM>
__global__ void __launch_bounds__(QK_WAVES * RA_WAVE)
qk_norm_rope_cache_head_kernel(TA* __restrict__ qkv, const TW* __restrict__ q_w, const TW* __restrict__ k_w,
                               float eps, const int* __restrict__ positions, const float* __restrict__ inv_freq,
                               const int* __restrict__ slots, TA* __restrict__ kcache, TA* __restrict__ vcache,
                               int block_size, int Hq, int Hkv) {
  constexpr int d = 64 * EPL;
  constexpr int NF = EPL >= 2 ? EPL / 2 : 1;
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / RA_WAVE);      // the same in every lane
  const int t = blockIdx.y;
  const int head = blockIdx.x * QK_WAVES + wave;
  const int n_heads = Hq + 2 * Hkv;
  if (head >= n_heads) return;
  TA* u = qkv + ((size_t)t * n_heads + head) * d;
  const bool is_q = head < Hq;
  const bool is_k = !is_q && head < Hq + Hkv;
  const TW* w = is_q ? q_w : k_w;              // a v head reads k's weights and drops them
  // ---- every load, then the first use
  const int slot = slots[t];
  const int posi = positions[t];
  unsigned xr[EPL], wr[EPL];
  float fr[NF];
#pragma unroll
  for (int k = 0; k < EPL; ++k) xr[k] = raw_bits(u, lane + 64 * k);
#pragma unroll
  for (int k = 0; k < EPL; ++k) wr[k] = NORM ? raw_bits(w, lane + 64 * k) : 0u;
#pragma unroll
  for (int k = 0; k < NF; ++k) fr[k] = inv_freq[EPL >= 2 ? lane + 64 * k : (lane & 31)];
  asm volatile("" ::: "memory");               // no load moves below this line, into the branches that follow
  // ----
  const int kvh = is_q ? 0 : (is_k ? head - Hq : head - Hq - Hkv);
  if (!is_q && slot < 0) return;               // nothing to store for this token
  const size_t blk = slot >= 0 ? (size_t)(slot / block_size) : 0;
  const int off = slot >= 0 ? slot % block_size : 0;
  TA* slab = is_q ? nullptr : (is_k ? kcache : vcache) + (blk * Hkv + kvh) * (size_t)block_size * d;
  float x[EPL];
#pragma unroll
  for (int k = 0; k < EPL; ++k) x[k] = raw_value<TA>(xr[k]);
  if (!is_q && !is_k) {                        // v head: copy into the V tile order
#pragma unroll
    for (int k = 0; k < EPL; ++k) slab[cache_v_index(off, lane + 64 * k, d)] = from_f32<TA>(x[k]);
    return;
  }
  if (NORM) {
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < EPL; ++k) ss += x[k] * x[k];
    ss = wave_sum(ss);
    const float rstd = rsqrtf(ss / (float)d + eps);
#pragma unroll
    for (int k = 0; k < EPL; ++k) x[k] = x[k] * rstd * raw_value<TW>(wr[k]);
  }
  const float pos = (float)posi;
  float y[EPL];
  if (EPL >= 2) {
#pragma unroll
    for (int k = 0; k < NF; ++k) {             // pair (lane + 64 k, lane + 64 k + d/2)
      float sn, cs;
      sincosf(pos * fr[k], &sn, &cs);
      const float a = x[k], c = x[k + NF];
      y[k] = a * cs - c * sn;
      y[k + NF] = a * sn + c * cs;
    }
  } else {
    float sn, cs;
    sincosf(pos * fr[0], &sn, &cs);
    const float other = __shfl_xor(x[0], 32, RA_WAVE);
    y[0] = lane < 32 ? x[0] * cs - other * sn : other * sn + x[0] * cs;
  }
#pragma unroll
  for (int k = 0; k < EPL; ++k) {
    const int i = lane + 64 * k;
    if (is_q) u[i] = from_f32<TA>(y[k]);
    else slab[cache_k_index(off, i, d)] = from_f32<TA>(y[k]);
  }
}

// 16 bytes of a row, as floats
template <typename T> struct Row16;
template <> struct Row16<float> {
  static constexpr int E = 4;
  static __device__ __forceinline__ void widen(f32x4_raw v, float* o) {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = v[i];
  }
  static __device__ __forceinline__ void load(const float* p, float* o) {
    const f32x4_raw v = *(const f32x4_raw*)p;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = v[i];
  }
  static __device__ __forceinline__ void store(float* p, const float* v) {
    *(f32x4_raw*)p = (f32x4_raw){v[0], v[1], v[2], v[3]};
  }
};
template <> struct Row16<bf16_t> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void widen(f32x4_raw raw, float* o) {
    const bf16x8_t v = __builtin_bit_cast(bf16x8_t, raw);
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (float)v[i];
  }
  static __device__ __forceinline__ void load(const bf16_t* p, float* o) {
    const bf16x8_t v = *(const bf16x8_t*)p;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (float)v[i];
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float* v) {
    bf16x8_t o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (bf16_t)v[i];
    *(bf16x8_t*)p = o;
  }
};

// The same for the common shape (half-split rotation over the whole head, head
// size a power of two between 16 and 256): one workgroup per token. The sines and
// cosines of the token's angles are computed once, in LDS, for all heads (the
// plain kernel computes them per head); a head is spread over LPH lanes, each
// holding 16 bytes of either half of the head: rotation pairs (j..j+E-1, j+d/2..j+d/2+E-1).
//
// What it lasts is how its accesses reach memory, not its arithmetic (timed with parts left out at 8192
// tokens of 48 heads of 128: neither the sines nor the barrier count). With 8 bytes a lane the reads ran at
// 3.0 TB/s, with 16 at 5. A token's keys and values go into tiles in which the same elements of
// neighbouring slots lie side by side: written token by token they are pieces of 16 bytes (keys) or single
// elements (values), each a request of its own. So four tokens in a row whose slots are s .. s + 3 with s a
// multiple of 4 (the usual case inside a prompt) share the work on their keys and values: workgroup i of
// the four takes KV heads i, i + 4, ... of all four tokens, lays the rotated keys and the values out in
// LDS as the tiles want them and writes runs of 64 bytes (keys) and whole 128-byte lines (values).
// 8192 tokens: 68 -> 55 us with 16-byte accesses and the XCD order below, -> 50 with the shared tiles, -> 46
// with the query rows asked for before the angles (2048 tokens, one round of workgroups: 15.3 -> 13.5 us).
// Dynamic LDS: the sines of four tokens (4 * d floats) and the two staging areas (qk_token_lds below).
template <typename TA, typename TW, int LPH>
__global__ void __launch_bounds__(256)
qk_norm_rope_cache_token_kernel(TA* __restrict__ qkv, const TW* __restrict__ q_w, const TW* __restrict__ k_w,
                                float eps, const int* __restrict__ positions,
                                const float* __restrict__ inv_freq, const int* __restrict__ slots,
                                TA* __restrict__ kcache, TA* __restrict__ vcache, int block_size, int Hq,
                                int Hkv, int d, int T, int share) {
  constexpr int E = Row16<TA>::E;
  constexpr int ROWS = 256 / LPH;              // head rows a pass of the workgroup
  extern __shared__ __attribute__((aligned(16))) unsigned char qk_lds[];
  const int half = d / 2;
  float* cs = (float*)qk_lds;                  // [4][half]
  float* sn = cs + 4 * half;                   // [4][half]
  // Sixteen tokens in a row write into the same lines of the cache (a tile's 16 slots lie side by side) and
  // workgroups go round the chip's XCDs, each with an L2 of its own: a run of 16 tokens is given to one
  // XCD (workgroup w runs on XCD w % RA_XCDS), so that the pieces meet in one L2. The grid is padded to
  // runs for all XCDs; a workgroup past the last token has nothing to do.
  const int w_xcd = blockIdx.x % RA_XCDS, w_k = blockIdx.x / RA_XCDS;
  const int t = ((w_k / 16) * RA_XCDS + w_xcd) * 16 + w_k % 16;
  if (t >= T) return;
  const int n_heads = Hq + 2 * Hkv;
  const int sub = threadIdx.x / LPH, ln = threadIdx.x % LPH;
  const int j0 = ln * E;                       // pairs j0..j0+E-1
  const int slot = slots[t];
  // which of four tokens this one is follows from its slot, not from its place in the step: a portion
  // that begins behind a few single tokens still finds its groups
  const int me = slot >= 0 ? (slot & 3) : 0, t0 = t - me;
  // the first pass's query rows are asked for before anything they do not hang on is waited for
  f32x4_raw first_a = {}, first_c = {};
  if (sub < Hq) {
    const TA* u = qkv + ((size_t)t * n_heads + sub) * d;
    first_a = *(const f32x4_raw*)(u + j0);
    first_c = *(const f32x4_raw*)(u + half + j0);
  }
  bool quad = share && slot >= 0 && t0 >= 0 && t0 + 3 < T;      // the same in every thread of the workgroup
  const int s0 = slot - me;
  if (quad) quad = slots[t0] == s0 && slots[t0 + 1] == s0 + 1 && slots[t0 + 2] == s0 + 2 && slots[t0 + 3] == s0 + 3;
  if (quad) {
    for (int idx = threadIdx.x; idx < 4 * half; idx += blockDim.x) {
      const int tok = idx / half, j = idx % half;
      sincosf((float)positions[t0 + tok] * inv_freq[j], &sn[idx], &cs[idx]);
    }
  } else {
    const float pos = (float)positions[t];
    for (int j = threadIdx.x; j < half; j += blockDim.x) sincosf(pos * inv_freq[j], &sn[me * half + j], &cs[me * half + j]);
  }
  __syncthreads();

  // one head row: norm and rotation with the angles of token `tok` of the four
  auto turn_held = [&](f32x4_raw raw_a, f32x4_raw raw_c, const TW* w, int tok, float* ra, float* rc) {
    float a[E], c[E];
    Row16<TA>::widen(raw_a, a);
    Row16<TA>::widen(raw_c, c);
    if (w) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < E; ++i) ss += a[i] * a[i];
#pragma unroll
      for (int i = 0; i < E; ++i) ss += c[i] * c[i];
#pragma unroll
      for (int m = LPH / 2; m > 0; m >>= 1) ss += __shfl_xor(ss, m, RA_WAVE);
      const float rstd = rsqrtf(ss / (float)d + eps);
#pragma unroll
      for (int i = 0; i < E; ++i) {
        a[i] = a[i] * rstd * to_f32(w[j0 + i]);
        c[i] = c[i] * rstd * to_f32(w[half + j0 + i]);
      }
    }
    const float* csr = cs + tok * half + j0;
    const float* snr = sn + tok * half + j0;
#pragma unroll
    for (int i = 0; i < E; ++i) {
      ra[i] = a[i] * csr[i] - c[i] * snr[i];
      rc[i] = a[i] * snr[i] + c[i] * csr[i];
    }
  };
  auto turn = [&](const TA* u, const TW* w, int tok, float* ra, float* rc) {
    turn_held(*(const f32x4_raw*)(u + j0), *(const f32x4_raw*)(u + half + j0), w, tok, ra, rc);
  };

  // the token's own query heads, in place
  for (int head = sub; head < Hq; head += ROWS) {
    TA* u = qkv + ((size_t)t * n_heads + head) * d;
    float ra[E], rc[E];
    if (head == sub) turn_held(first_a, first_c, q_w, me, ra, rc);
    else turn(u, q_w, me, ra, rc);
    Row16<TA>::store(u + j0, ra);
    Row16<TA>::store(u + half + j0, rc);
  }

  if (!quad) {                                 // its own keys and values, piece by piece
    if (slot < 0) return;                      // nothing to store for this token
    const size_t blk = (size_t)(slot / block_size);
    const int off = slot % block_size;
    for (int r = sub; r < 2 * Hkv; r += ROWS) {
      const bool is_k = r < Hkv;
      const int kvh = is_k ? r : r - Hkv;
      const TA* u = qkv + ((size_t)t * n_heads + Hq + r) * d;
      TA* slab = (is_k ? kcache : vcache) + (blk * Hkv + kvh) * (size_t)block_size * d;
      if (is_k) {                              // the elements of one 8-chunk are contiguous in the K tile
        float ra[E], rc[E];
        turn(u, k_w, me, ra, rc);
        Row16<TA>::store(slab + cache_k_index(off, j0, d), ra);
        Row16<TA>::store(slab + cache_k_index(off, half + j0, d), rc);
      } else {
        float a[E], c[E];
        Row16<TA>::load(u + j0, a);
        Row16<TA>::load(u + half + j0, c);
#pragma unroll
        for (int i = 0; i < E; ++i) {
          slab[cache_v_index(off, j0 + i, d)] = from_f32<TA>(a[i]);
          slab[cache_v_index(off, half + j0 + i, d)] = from_f32<TA>(c[i]);
        }
      }
    }
    return;
  }

  // KV heads me, me + 4, ... of the four tokens: into LDS in tile order, then out in whole runs.
  //   keys    kst[m][chunk][token][8]      = the K tile's [chunk][slot][8] over the four slots
  //   values  vst[m][e / 16][e % 16][token] = the V tile's [e / 16][slot / 4][e % 16][slot % 4] of this quad
  const int n_mine = (Hkv - me + 3) / 4;       // may be 0
  const int n_max = (Hkv + 3) / 4;
  TA* kst = (TA*)(sn + 4 * half);
  TA* vst = kst + (size_t)n_max * d * 4;
  for (int r = sub; r < n_mine * 8; r += ROWS) {
    const int m = r >> 3, tok = r & 3;
    const bool is_k = (r & 4) == 0;
    const int kvh = me + 4 * m;
    const TA* u = qkv + ((size_t)(t0 + tok) * n_heads + Hq + (is_k ? 0 : Hkv) + kvh) * d;
    if (is_k) {
      float ra[E], rc[E];
      turn(u, k_w, tok, ra, rc);
      TA* dst = kst + (size_t)m * d * 4;
      // element e of the row -> ((e / 8) * 4 + tok) * 8 + e % 8; the E elements of a lane lie in one chunk
      Row16<TA>::store(dst + ((j0 >> 3) * 4 + tok) * 8 + (j0 & 7), ra);
      Row16<TA>::store(dst + (((half + j0) >> 3) * 4 + tok) * 8 + ((half + j0) & 7), rc);
    } else {
      float a[E], c[E];
      Row16<TA>::load(u + j0, a);
      Row16<TA>::load(u + half + j0, c);
      TA* dst = vst + (size_t)m * d * 4;
#pragma unroll
      for (int i = 0; i < E; ++i) {
        dst[(j0 + i) * 4 + tok] = from_f32<TA>(a[i]);
        dst[(half + j0 + i) * 4 + tok] = from_f32<TA>(c[i]);
      }
    }
  }
  __syncthreads();
  constexpr int PIECE = 16 / (int)sizeof(TA);  // elements of a 16-byte piece
  const size_t blk = (size_t)(s0 / block_size);
  const int off0 = s0 % block_size;            // a multiple of 4: the four slots lie in one tile
  const size_t tile_at = (size_t)(off0 >> 4) * 16 * d;
  const int per_head = d * 4 / PIECE;          // pieces of a head's four tokens
  for (int idx = threadIdx.x; idx < n_mine * per_head * 2; idx += blockDim.x) {
    const bool is_k = idx < n_mine * per_head;
    const int i2 = is_k ? idx : idx - n_mine * per_head;
    const int m = i2 / per_head, e4 = (i2 % per_head) * PIECE;     // element among the head's d * 4
    const int kvh = me + 4 * m;
    TA* slab = (is_k ? kcache : vcache) + (blk * Hkv + kvh) * (size_t)block_size * d + tile_at;
    const TA* src = (is_k ? kst : vst) + (size_t)m * d * 4 + e4;
    // keys: chunk c = e4 / 32 holds 32 elements of the four tokens, at (c * 16 + off0 % 16) * 8 in the tile;
    // values: group g = e4 / 64 holds 64, at ((g * 4 + (off0 % 16) / 4) * 16) * 4
    const size_t at = is_k ? (size_t)((e4 >> 5) * 16 + (off0 & 15)) * 8 + (e4 & 31)
                           : (size_t)((e4 >> 6) * 4 + ((off0 & 15) >> 2)) * 64 + (e4 & 63);
    *(f32x4_raw*)(slab + at) = *(const f32x4_raw*)src;
  }
}

// Bytes of dynamic LDS of the per-token kernel: the sines and cosines of four tokens and, where four
// tokens share their keys and values, the two staging areas.
static size_t qk_token_lds(int Hkv, int d, size_t elem, bool share) {
  return (size_t)4 * d * sizeof(float) + (share ? (size_t)2 * ((Hkv + 3) / 4) * d * 4 * elem : 0);
}

static int qk_norm_rope_cache_impl(void* qkv, int act_dtype, const void* q_weight, const void* k_weight,
                                   int weight_dtype, float eps, const int* positions,
                                   const float* inv_freq, int rotary_dim, int rope_style,
                                   const int* slots, void* kcache, void* vcache, int block_size,
                                   int n_tokens, int Hq, int Hkv, int d, const QkSums& sm, hipStream_t stream) {
  RA_CHECK(n_tokens > 0, "qk_norm_rope_cache: no tokens");
  RA_CHECK(Hq > 0 && Hkv > 0 && d > 0, "qk_norm_rope_cache: bad head sizes (%d, %d, %d)", Hq, Hkv, d);
  RA_CHECK(d <= QK_MAX_D, "qk_norm_rope_cache: head size %d above the supported %d", d, QK_MAX_D);
  RA_CHECK(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0,
           "qk_norm_rope_cache: rotary width %d must be even and <= head size %d", rotary_dim, d);
  RA_CHECK(rope_style == 0 || rope_style == 1, "qk_norm_rope_cache: unknown rotation style %d", rope_style);
  RA_CHECK((q_weight == nullptr) == (k_weight == nullptr), "qk_norm_rope_cache: q and k norm weights go together");
  RA_CHECK(block_size > 0 && block_size % 16 == 0 && d % 16 == 0,
           "qk_norm_rope_cache: the cache is tiled 16 x 16: block size %d and head size %d must be multiples of 16",
           block_size, d);
  RA_CHECK(n_tokens <= 65535, "qk_norm_rope_cache: %d tokens in one launch (max 65535)", n_tokens);
  // the per-token kernel takes half-split rotation over the whole head, d in {16, 32, 64, 128, 256};
  // with few tokens (decode) a wave per head spreads over more of the chip (measured at 32 heads of 128:
  // 3.2 against 4.4 us at 64 tokens, 3.9 against 4.7 at 128, 6.2 against 5.4 at 255)
  const bool pow2 = (d & (d - 1)) == 0 && d >= 16 && d <= 256;
  if (!sm.parts && pow2 && n_tokens >= 192 && rope_style == 0 && rotary_dim == d && ((uintptr_t)qkv % 16) == 0 &&
      (q_weight == nullptr || (((uintptr_t)q_weight % 16) == 0 && ((uintptr_t)k_weight % 16) == 0))) {
    // four tokens share their keys and values where the staging areas leave room for eight workgroups a CU
    const bool share = qk_token_lds(Hkv, d, act_dtype == RA_F32 ? 4 : 2, true) <= 16384;
#define RA_TOK2(TA, TW, LPH)                                                                              \
  qk_norm_rope_cache_token_kernel<TA, TW, LPH>                                                            \
      <<<(n_tokens + 16 * RA_XCDS - 1) / (16 * RA_XCDS) * (16 * RA_XCDS), 256,                            \
         qk_token_lds(Hkv, d, sizeof(TA), share), stream>>>(                                              \
      (TA*)qkv, (const TW*)q_weight, (const TW*)k_weight, eps, positions, inv_freq, slots, (TA*)kcache,  \
      (TA*)vcache, block_size, Hq, Hkv, d, n_tokens, share ? 1 : 0)
  /* lanes a head: 16 bytes of either half a lane (SH: 0 for 4-byte elements, 1 for 2-byte ones) */
#define RA_TOK(TA, TW, SH)                           \
  do {                                               \
    if (d == 16) RA_TOK2(TA, TW, (2 >> SH));         \
    else if (d == 32) RA_TOK2(TA, TW, (4 >> SH));    \
    else if (d == 64) RA_TOK2(TA, TW, (8 >> SH));    \
    else if (d == 128) RA_TOK2(TA, TW, (16 >> SH));  \
    else RA_TOK2(TA, TW, (32 >> SH));                \
  } while (0)
    if (act_dtype == RA_F32 && weight_dtype == RA_F32) RA_TOK(float, float, 0);
    else if (act_dtype == RA_BF16 && weight_dtype == RA_BF16) RA_TOK(bf16_t, bf16_t, 1);
    else if (act_dtype == RA_BF16 && weight_dtype == RA_F32) RA_TOK(bf16_t, float, 1);
    else return ra_fail("qk_norm_rope_cache: unsupported dtypes (activations %d, weight %d)", act_dtype, weight_dtype);
#undef RA_TOK
#undef RA_TOK2
    RA_LAUNCH_CHECK("qk_norm_rope_cache");
    return 0;
  }
  dim3 grid((Hq + 2 * Hkv + QK_WAVES - 1) / QK_WAVES, n_tokens);
  if (!sm.parts && (d == 64 || d == 128 || d == 256) && rope_style == 0 && rotary_dim == d) {
#define RA_HEAD2(TA, TW, EPL)                                                                             \
  do {                                                                                                    \
    if (q_weight)                                                                                         \
      qk_norm_rope_cache_head_kernel<TA, TW, EPL, true><<<grid, QK_WAVES * RA_WAVE, 0, stream>>>(         \
          (TA*)qkv, (const TW*)q_weight, (const TW*)k_weight, eps, positions, inv_freq, slots, (TA*)kcache, \
          (TA*)vcache, block_size, Hq, Hkv);                                                              \
    else                                                                                                  \
      qk_norm_rope_cache_head_kernel<TA, TW, EPL, false><<<grid, QK_WAVES * RA_WAVE, 0, stream>>>(        \
          (TA*)qkv, (const TW*)q_weight, (const TW*)k_weight, eps, positions, inv_freq, slots, (TA*)kcache, \
          (TA*)vcache, block_size, Hq, Hkv);                                                              \
  } while (0)
#define RA_HEAD(TA, TW)                      \
  do {                                       \
    if (d == 64) RA_HEAD2(TA, TW, 1);        \
    else if (d == 128) RA_HEAD2(TA, TW, 2);  \
    else RA_HEAD2(TA, TW, 4);                \
  } while (0)
    if (act_dtype == RA_F32 && weight_dtype == RA_F32) RA_HEAD(float, float);
    else if (act_dtype == RA_BF16 && weight_dtype == RA_BF16) RA_HEAD(bf16_t, bf16_t);
    else if (act_dtype == RA_BF16 && weight_dtype == RA_F32) RA_HEAD(bf16_t, float);
    else return ra_fail("qk_norm_rope_cache: unsupported dtypes (activations %d, weight %d)", act_dtype, weight_dtype);
#undef RA_HEAD
#undef RA_HEAD2
    RA_LAUNCH_CHECK("qk_norm_rope_cache");
    return 0;
  }
#define RA_GO(TA, TW)                                                                              \
  qk_norm_rope_cache_kernel<TA, TW><<<grid, QK_WAVES * RA_WAVE, 0, stream>>>(                      \
      (TA*)qkv, (const TW*)q_weight, (const TW*)k_weight, eps, positions, inv_freq, rotary_dim,   \
      rope_style, slots, (TA*)kcache, (TA*)vcache, block_size, Hq, Hkv, d, sm)
  if (act_dtype == RA_F32 && weight_dtype == RA_F32) RA_GO(float, float);
  else if (act_dtype == RA_BF16 && weight_dtype == RA_BF16) RA_GO(bf16_t, bf16_t);
  else if (act_dtype == RA_BF16 && weight_dtype == RA_F32) RA_GO(bf16_t, float);
  else return ra_fail("qk_norm_rope_cache: unsupported dtypes (activations %d, weight %d)", act_dtype, weight_dtype);
#undef RA_GO
  RA_LAUNCH_CHECK("qk_norm_rope_cache");
  return 0;
}

extern "C" int ra_qk_norm_rope_cache(void* qkv, int act_dtype, const void* q_weight, const void* k_weight,
                                     int weight_dtype, float eps, const int* positions,
                                     const float* inv_freq, int rotary_dim, int rope_style,
                                     const int* slots, void* kcache, void* vcache, int block_size,
                                     int n_tokens, int Hq, int Hkv, int d, hipStream_t stream) {
  RA_CHECK(qkv != nullptr, "qk_norm_rope_cache: no q/k/v rows");
  const QkSums none = {};
  return qk_norm_rope_cache_impl(qkv, act_dtype, q_weight, k_weight, weight_dtype, eps, positions, inv_freq,
                                 rotary_dim, rope_style, slots, kcache, vcache, block_size, n_tokens, Hq, Hkv, d,
                                 none, stream);
}

// The same from the float partial results of a product cut into K ranges ([n_ranges][n_tokens][width],
// width = (Hq + 2 Hkv) d), which are added here, in range order, instead of by a kernel of their own; with
// in_ss ([in_parts][n_tokens] partial sums of squares, eps, width) the rows are also scaled by the RMSNorm
// that product carried. The rotated q goes to q_out ([n_tokens][q_stride], the cache's type).
extern "C" int ra_qk_norm_rope_cache_sums(const float* parts, int n_ranges, const float* in_ss, int in_parts,
                                          float in_eps, int in_width, void* q_out, int q_stride, int act_dtype,
                                          const void* q_weight, const void* k_weight, int weight_dtype,
                                          float eps, const int* positions, const float* inv_freq,
                                          int rotary_dim, int rope_style, const int* slots, void* kcache,
                                          void* vcache, int block_size, int n_tokens, int Hq, int Hkv, int d,
                                          hipStream_t stream) {
  RA_CHECK(parts && n_ranges >= 1 && q_out, "qk_norm_rope_cache_sums: partial results and a place for q are needed");
  RA_CHECK(q_stride >= Hq * d, "qk_norm_rope_cache_sums: q rows of %d elements do not hold %d heads of %d", q_stride, Hq, d);
  RA_CHECK(in_ss == nullptr || (in_parts > 0 && in_width > 0 && in_eps >= 0.f),
           "qk_norm_rope_cache_sums: row sums need parts (%d), width (%d) and eps", in_parts, in_width);
  QkSums sm = {};
  sm.parts = parts;
  sm.n_ranges = n_ranges;
  sm.range_stride = (size_t)n_tokens * (size_t)(Hq + 2 * Hkv) * (size_t)d;
  sm.in_ss = in_ss;
  sm.in_parts = in_parts;
  sm.in_eps = in_eps;
  sm.in_inv_width = in_ss ? 1.f / (float)in_width : 0.f;
  sm.q_out = q_out;
  sm.q_stride = q_stride;
  return qk_norm_rope_cache_impl(nullptr, act_dtype, q_weight, k_weight, weight_dtype, eps, positions, inv_freq,
                                 rotary_dim, rope_style, slots, kcache, vcache, block_size, n_tokens, Hq, Hkv, d,
                                 sm, stream);
}

// ---------------------------------------------------------------------------
// SiLU gate: out[t, i] = silu(g[t, i]) * u[t, i], silu(g) = g / (1 + exp(-g))
// (crates/cuda/kernels/dense_kernels.cu:202-213). gate_up is [T, 2I]; with
// group == 0 gate is columns [0, I) and up [I, 2I); with group > 0 the two are
// interleaved in runs of `group` columns, as the gated product kernel wants them.
// ---------------------------------------------------------------------------
template <typename TA>
__global__ void silu_mul_kernel(const TA* __restrict__ gu, TA* __restrict__ out, int I, int group, size_t total) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; idx < total; idx += stride) {
    const size_t t = idx / I;
    const int i = (int)(idx - t * I);
    const size_t gi = group > 0 ? (size_t)(i / group) * 2 * group + i % group : (size_t)i;
    const size_t ui = group > 0 ? gi + group : (size_t)I + i;
    const float g = to_f32(gu[t * 2 * I + gi]);
    const float u = to_f32(gu[t * 2 * I + ui]);
    out[idx] = from_f32<TA>(g / (1.f + expf(-g)) * u);
  }
}

// eight outputs a thread, 16-byte loads and stores; I a multiple of 8, group 0 or a multiple of 8
template <typename TA>
__global__ void silu_mul_vec_kernel(const TA* __restrict__ gu, TA* __restrict__ out, int I, int group, size_t total8) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const int I8 = I / 8;
  for (; idx < total8; idx += stride) {
    const size_t t = idx / I8;
    const int i = (int)(idx - t * I8) * 8;
    const size_t gi = group > 0 ? (size_t)(i / group) * 2 * group + i % group : (size_t)i;
    const size_t ui = group > 0 ? gi + group : (size_t)I + i;
    const TA* row = gu + t * 2 * I;
    f32x4_raw g0 = Vec4<TA>::load(row + gi), g1 = Vec4<TA>::load(row + gi + 4);
    f32x4_raw u0 = Vec4<TA>::load(row + ui), u1 = Vec4<TA>::load(row + ui + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      g0[e] = g0[e] / (1.f + expf(-g0[e])) * u0[e];
      g1[e] = g1[e] / (1.f + expf(-g1[e])) * u1[e];
    }
    Vec4<TA>::store(out + idx * 8, g0);
    Vec4<TA>::store(out + idx * 8 + 4, g1);
  }
}

extern "C" int ra_silu_mul(const void* gate_up, void* out, int act_dtype, int n_tokens, int intermediate,
                           int group, hipStream_t stream) {
  RA_CHECK(n_tokens > 0 && intermediate > 0, "silu_mul: empty input");
  RA_CHECK(group >= 0 && (group == 0 || intermediate % group == 0),
           "silu_mul: width %d is not a whole number of runs of %d", intermediate, group);
  const size_t total = (size_t)n_tokens * intermediate;
  if (intermediate % 8 == 0 && group % 8 == 0 && ((uintptr_t)gate_up % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
      (act_dtype == RA_F32 || act_dtype == RA_BF16)) {
    const size_t total8 = total / 8;
    size_t vb = (total8 + 255) / 256;
    if (vb > 65535 * 4) vb = 65535 * 4;
    if (act_dtype == RA_F32)
      silu_mul_vec_kernel<float><<<(unsigned)vb, 256, 0, stream>>>((const float*)gate_up, (float*)out, intermediate, group, total8);
    else
      silu_mul_vec_kernel<bf16_t><<<(unsigned)vb, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, intermediate, group, total8);
    RA_LAUNCH_CHECK("silu_mul");
    return 0;
  }
  size_t blocks = (total + 255) / 256;
  if (blocks > 65535 * 4) blocks = 65535 * 4;
  if (act_dtype == RA_F32)
    silu_mul_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out, intermediate, group, total);
  else if (act_dtype == RA_BF16)
    silu_mul_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, intermediate, group, total);
  else
    return ra_fail("silu_mul: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("silu_mul");
  return 0;
}
