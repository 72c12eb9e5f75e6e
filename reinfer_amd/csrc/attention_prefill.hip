// Paged flash attention for prompt portions, bfloat16, on the matrix cores.
//
// A workgroup (4 wavefronts) takes one tile of up to 64 consecutive query tokens
// of one request and one query head; wavefront w owns 16 of the queries. Keys
// and values come from the request's block table: earlier context and the
// portion's own tokens alike (they were stored before this kernel runs), 64
// keys a tile, staged through LDS: K as [key][d], V transposed as [d][key], so
// that both products contract over a register-contiguous axis.
//
//   S^T[key][query] = K . Q^T        v_mfma_f32_16x16x32_bf16, contraction over d
//   online softmax per query column (float; running maximum, sum)
//   O^T[d][query]  += V^T . P        contraction over 32 keys; the probabilities
//                                    are the MFMA's second operand straight from
//                                    the score registers (two score tiles packed)
//
// Causal: query at position p sees keys <= p (and > p - window if a window is
// set). The reference's prompt attention is a vendored library kernel that sees
// only the prompt itself, from position 0 (crates/cuda/src/fmha.rs:574-686;
// crates/cuda/kernels/fmha_kernels.cu:96); this one is written here and reads
// earlier context from the cache, so a prompt can be cut anywhere.
#include "common.h"
#include "reinfer_hip.h"

#define FP_THREADS 256
#define FP_QT 64          // queries per workgroup
#define FP_KT 64          // keys per tile
#define FP_KPAD 8         // bf16 elements of padding per LDS row

__device__ __forceinline__ float fp_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int DMAX>
__global__ void __launch_bounds__(FP_THREADS)
flash_prefill_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                     const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
                     const int* __restrict__ block_tables, int max_blocks,
                     const int* __restrict__ tile_info,      // per tile: seq, first token row, n queries, first position
                     int block_size, int Hq, int Hkv, int d, float scale_log2, int window) {
  constexpr int NDT = DMAX / 32;       // 32-wide d tiles of the score product
  constexpr int NOT = DMAX / 16;       // 16-wide d tiles of the output
  constexpr int KROW = DMAX + FP_KPAD;
  constexpr int VROW = FP_KT + FP_KPAD;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[FP_KT * KROW];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[DMAX * VROW];

  const int tid = threadIdx.x;
  const int lane = tid & (RA_WAVE - 1), wave = tid / RA_WAVE;
  const int r = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x, head = blockIdx.y;
  const int kvh = head / (Hq / Hkv);
  const int seq = tile_info[tile * 4 + 0];
  const int row0 = tile_info[tile * 4 + 1];
  const int nq = tile_info[tile * 4 + 2];
  const int pos0 = tile_info[tile * 4 + 3];
  const int* table = block_tables + (size_t)seq * max_blocks;
  const int DL = d / 8;

  // this lane's query column: query 16 * wave + r
  const int qi = wave * 16 + r;
  const bool q_live = qi < nq;
  const int q_pos = pos0 + qi;
  const int q_lo = (window > 0 && q_pos - window + 1 > 0) ? q_pos - window + 1 : 0;
  bf16x8_t qreg[NDT];
  {
    const int qrow = row0 + (q_live ? qi : nq - 1);
    const bf16_t* qp = q + (size_t)qrow * q_stride + (size_t)head * d;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const int e = dt * 32 + g * 8;
      qreg[dt] = (e < d) ? *(const bf16x8_t*)(qp + e) : (bf16x8_t){0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  f32x4_t acc[NOT];
#pragma unroll
  for (int i = 0; i < NOT; ++i) acc[i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // keys this tile of queries can see
  const int last_pos = pos0 + nq - 1;
  const int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int kt_begin = first_key / FP_KT * FP_KT;

  for (int k0 = kt_begin; k0 <= last_pos; k0 += FP_KT) {
    __syncthreads();                       // the previous tile is no longer read
    // stage K and V^T: 64 keys x d/8 chunks of 16 bytes
    for (int c = tid; c < FP_KT * DL; c += FP_THREADS) {
      const int kk = c / DL, dc = c % DL;
      const int key = k0 + kk;
      bf16x8_t kv = {0, 0, 0, 0, 0, 0, 0, 0}, vv = kv;
      if (key <= last_pos && key >= first_key) {    // outside: zeros, never a stale block's bits
        const int blk = table[key / block_size];
        const size_t off = (((size_t)blk * Hkv + kvh) * block_size + key % block_size) * d + dc * 8;
        kv = *(const bf16x8_t*)(kcache + off);
        vv = *(const bf16x8_t*)(vcache + off);
      }
      *(bf16x8_t*)(Ks + kk * KROW + dc * 8) = kv;
#pragma unroll
      for (int j = 0; j < 8; ++j) Vt[(dc * 8 + j) * VROW + kk] = vv[j];
    }
    __syncthreads();

    // a wavefront whose live queries all lie before this tile has nothing to add
    // (it still meets the barriers at the top of the next round)
    if (wave * 16 >= nq || pos0 + min(wave * 16 + 15, nq - 1) < k0) continue;

    // scores S^T[key][query] for 4 sub-tiles of 16 keys
    f32x4_t s[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      s[ks] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        const int e = dt * 32 + g * 8;
        if (dt * 32 < d) {
          bf16x8_t a = (e < d) ? *(const bf16x8_t*)(Ks + (ks * 16 + r) * KROW + e)
                               : (bf16x8_t){0, 0, 0, 0, 0, 0, 0, 0};
          s[ks] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qreg[dt], s[ks], 0, 0, 0);
        }
      }
    }
    // mask, scale, tile maximum of this lane's query column
    float tmax = -INFINITY;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = k0 + ks * 16 + 4 * g + i;
        const bool ok = q_live && key <= q_pos && key >= q_lo;
        const float v = ok ? s[ks][i] * scale_log2 : -INFINITY;
        s[ks][i] = v;
        tmax = fmaxf(tmax, v);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, RA_WAVE));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, RA_WAVE));
    const float mn = fmaxf(m, tmax);
    // a column with nothing visible so far keeps m = -inf and adds zeros
    const float base = (mn == -INFINITY) ? 0.f : mn;
    const float corr = (mn == -INFINITY) ? 1.f : fp_exp2(m - mn);
    float psum = 0.f;
    bf16x8_t pb[2];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = fp_exp2(s[ks][i] - base);      // masked: exp2(-inf) = 0
        psum += p;
        pb[ks / 2][(ks % 2) * 4 + i] = from_f32<bf16_t>(p);
      }
    l = l * corr + psum;
    m = mn;
#pragma unroll
    for (int ot = 0; ot < NOT; ++ot)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[ot][i] *= corr;
    // O^T[d][query] += V^T[d][key] P[key][query], 32 keys per instruction:
    // k-slots (g, j): j < 4 -> key 4g + j of the first sub-tile, j >= 4 -> of the second
#pragma unroll
    for (int kp = 0; kp < 2; ++kp) {
#pragma unroll
      for (int ot = 0; ot < NOT; ++ot) {
        if (ot * 16 < d) {
          const bf16_t* vrow = Vt + (ot * 16 + r) * VROW + kp * 32 + 4 * g;
          const bf16x4_t lo4 = *(const bf16x4_t*)(vrow);
          const bf16x4_t hi4 = *(const bf16x4_t*)(vrow + 16);
          const bf16x8_t a = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
          acc[ot] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[kp], acc[ot], 0, 0, 0);
        }
      }
    }
  }
  // the lane groups hold partial sums of l over their own keys
  l += __shfl_xor(l, 16, RA_WAVE);
  l += __shfl_xor(l, 32, RA_WAVE);
  if (!q_live) return;
  const float inv = 1.f / l;
  bf16_t* op = out + (size_t)(row0 + qi) * out_stride + (size_t)head * d;
#pragma unroll
  for (int ot = 0; ot < NOT; ++ot) {
    const int e = ot * 16 + 4 * g;
    if (e < d) {
      bf16x4_t o4 = {from_f32<bf16_t>(acc[ot][0] * inv), from_f32<bf16_t>(acc[ot][1] * inv),
                     from_f32<bf16_t>(acc[ot][2] * inv), from_f32<bf16_t>(acc[ot][3] * inv)};
      *(bf16x4_t*)(op + e) = o4;
    }
  }
}

extern "C" int ra_attention_prefill_supports(int Hq, int Hkv, int d) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return 0;
  return (d % 16 == 0 && d >= 16 && d <= 128) ? 1 : 0;   // LDS tiles are sized for d <= 128
}

extern "C" int ra_attention_prefill_tile(void) { return FP_QT; }

extern "C" int ra_attention_prefill(const void* q, int q_stride, void* out, int out_stride,
                                    const void* kcache, const void* vcache, const int* block_tables,
                                    int max_blocks, const int* tile_info, int n_tiles, int block_size,
                                    int Hq, int Hkv, int d, float scale, int window, hipStream_t stream) {
  RA_CHECK(n_tiles > 0, "attention_prefill: no query tiles");
  RA_CHECK(ra_attention_prefill_supports(Hq, Hkv, d),
           "attention_prefill: unsupported sizes (%d query heads, %d KV heads, head size %d)", Hq, Hkv, d);
  RA_CHECK(block_size > 0 && max_blocks > 0 && window >= 0, "attention_prefill: bad cache geometry");
  RA_CHECK(q_stride % 8 == 0 && out_stride % 4 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 8) == 0 &&
               ((uintptr_t)kcache % 16) == 0 && ((uintptr_t)vcache % 16) == 0,
           "attention_prefill: operands must be 16-byte aligned");
  RA_CHECK(Hq <= 65535, "attention_prefill: too many heads for one launch");
  dim3 grid(n_tiles, Hq);
  const float scale_log2 = scale * 1.4426950408889634f;
#define RA_FP(DM)                                                                                     \
  flash_prefill_kernel<DM><<<grid, FP_THREADS, 0, stream>>>(                                          \
      (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kcache,                    \
      (const bf16_t*)vcache, block_tables, max_blocks, tile_info, block_size, Hq, Hkv, d, scale_log2, \
      window)
  if (d <= 32) RA_FP(32);
  else if (d <= 64) RA_FP(64);
  else RA_FP(128);
#undef RA_FP
  RA_LAUNCH_CHECK("attention_prefill");
  return 0;
}
