// Plain paged attention for any batch: one wavefront per (token, query head).
// It is the attention of the 32-bit path and the twin that the tiled kernels
// are checked against. Scores, maximum, exponentials, their sum and the
// weighted sum of values are float.
//
//   s_t = scale * (q . K_t) for keys t in [lo, p] of the token's own request,
//   lo = max(0, p - window + 1) if window > 0 else 0; softmax with the running
//   maximum subtracted; o = sum_t P_t V_t.
//   Query head a reads KV head a / (Hq / Hkv).
// (crates/cuda/kernels/decode_gqa_kernels.cu:69-136; plain form
//  crates/cuda/tests/engine_vs_cpu.rs:205-241)
#include "common.h"
#include "reinfer_hip.h"

template <typename TA>
__global__ void attention_plain_kernel(const TA* __restrict__ q, int q_stride, TA* __restrict__ out,
                                       int out_stride, const TA* __restrict__ kcache,
                                       const TA* __restrict__ vcache,
                                       const int* __restrict__ block_tables, int max_blocks,
                                       const int* __restrict__ token_list,
                                       const int* __restrict__ seq_of_token,
                                       const int* __restrict__ positions, int block_size, int Hq,
                                       int Hkv, int d, float scale, int window) {
  extern __shared__ float lds[];          // q vector [d], then probabilities [64]
  float* qs = lds;
  float* ps = lds + d;
  const int lane = threadIdx.x;
  const int a = blockIdx.x;
  const int t = token_list ? token_list[blockIdx.y] : blockIdx.y;
  const int kvh = a / (Hq / Hkv);
  const int seq = seq_of_token[t];
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int* table = block_tables + (size_t)seq * max_blocks;
  const TA* qv = q + (size_t)t * q_stride + (size_t)a * d;
  for (int i = lane; i < d; i += RA_WAVE) qs[i] = to_f32(qv[i]);
  __syncthreads();

  const int n_acc = (d + RA_WAVE - 1) / RA_WAVE;   // output elements per lane (<= 8)
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int base = lo; base <= p; base += RA_WAVE) {
    const int key = base + lane;
    float s = -INFINITY;
    if (key <= p) {
      const int blk = table[key / block_size];
      const TA* kr = kcache + ((size_t)blk * Hkv + kvh) * block_size * d;
      const int off = key % block_size;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot += qs[i] * to_f32(kr[cache_k_index(off, i, d)]);
      s = dot * scale;
    }
    const float cmax = wave_max(s);
    const float m_new = fmaxf(m, cmax);
    const float pr = (key <= p) ? expf(s - m_new) : 0.f;
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + wave_sum(pr);
    m = m_new;
    __syncthreads();                 // ps of the previous chunk is no longer read
    ps[lane] = pr;
    __syncthreads();
    const int n_keys = (p - base + 1 < RA_WAVE) ? p - base + 1 : RA_WAVE;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      if (r < n_acc) {
        const int i = r * RA_WAVE + lane;
        float sum = 0.f;
        if (i < d) {
          for (int kk = 0; kk < n_keys; ++kk) {
            const int key2 = base + kk;
            const int blk = table[key2 / block_size];
            const TA* vr = vcache + ((size_t)blk * Hkv + kvh) * block_size * d;
            sum += ps[kk] * to_f32(vr[cache_v_index(key2 % block_size, i, d)]);
          }
        }
        acc[r] = acc[r] * corr + sum;
      }
    }
  }
  TA* o = out + (size_t)t * out_stride + (size_t)a * d;
  const float inv = 1.f / l;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    if (r < n_acc) {
      const int i = r * RA_WAVE + lane;
      if (i < d) o[i] = from_f32<TA>(acc[r] * inv);
    }
  }
}

extern "C" int ra_attention_plain(const void* q, int q_stride, void* out, int out_stride,
                                  const void* kcache, const void* vcache, int act_dtype,
                                  const int* block_tables, int max_blocks, const int* token_list,
                                  const int* seq_of_token, const int* positions, int n_tokens, int block_size, int Hq, int Hkv,
                                  int d, float scale, int window, hipStream_t stream) {
  RA_CHECK(n_tokens > 0, "attention_plain: no tokens");
  RA_CHECK(Hq > 0 && Hkv > 0 && Hq % Hkv == 0, "attention_plain: %d query heads do not divide into %d groups", Hq, Hkv);
  RA_CHECK(d > 0 && d <= 512, "attention_plain: head size %d outside 1..512", d);
  RA_CHECK(block_size > 0 && block_size % 16 == 0 && d % 16 == 0 && max_blocks > 0,
           "attention_plain: the cache is tiled 16 x 16: block size %d and head size %d must be multiples of 16",
           block_size, d);
  RA_CHECK(window >= 0, "attention_plain: negative window");
  RA_CHECK(n_tokens <= 65535, "attention_plain: %d tokens in one launch (max 65535)", n_tokens);
  dim3 grid(Hq, n_tokens);
  const size_t lds = (size_t)(d + RA_WAVE) * sizeof(float);
  if (act_dtype == RA_F32)
    attention_plain_kernel<float><<<grid, RA_WAVE, lds, stream>>>(
        (const float*)q, q_stride, (float*)out, out_stride, (const float*)kcache, (const float*)vcache,
        block_tables, max_blocks, token_list, seq_of_token, positions, block_size, Hq, Hkv, d, scale, window);
  else if (act_dtype == RA_BF16)
    attention_plain_kernel<bf16_t><<<grid, RA_WAVE, lds, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kcache,
        (const bf16_t*)vcache, block_tables, max_blocks, token_list, seq_of_token, positions, block_size,
        Hq, Hkv, d, scale, window);
  else
    return ra_fail("attention_plain: unknown dtype tag %d", act_dtype);
  RA_LAUNCH_CHECK("attention_plain");
  return 0;
}
