// Paged flash attention for prompt portions, bfloat16, on the matrix cores.
//
// A workgroup (4 waves) takes one tile of consecutive query tokens of one
// request and up to NC query heads that share a KV head. A wave owns NC column
// tiles of 16: QT runs of 16 queries times HG heads (QT * HG <= NC), so every
// key and value it reads from LDS feeds NC MFMAs. Keys and values come from the
// request's block table, earlier context and the portion's own tokens alike
// (they were stored before this kernel runs), 64 keys a round, copied to LDS
// as the cache holds them: tiles of 16 slots in MFMA operand order
// (cache_k_index / cache_v_index), so the copy is linear and every operand read
// from LDS is a contiguous run with no bank conflict. The next round's tiles
// are fetched into registers while this one is multiplied.
//
//   S^T[key][column] = K . Q^T        v_mfma_f32_16x16x32_bf16, contraction over d
//   online softmax per column (float; running maximum, sum), once per 64 keys
//   O^T[d][column]  += V^T . P        contraction over 32 keys; the probabilities
//                                     are the MFMA's second operand straight from
//                                     the score registers (two score tiles packed)
//
// Causal: a query at position p sees keys <= p (and > p - window if a window is
// set). The reference's prompt attention is a vendored library kernel that sees
// only the prompt itself, from position 0 (crates/cuda/src/fmha.rs:574-686;
// crates/cuda/kernels/fmha_kernels.cu:96); this one is written here and reads
// earlier context from the cache, so a prompt can be cut anywhere.
#include "common.h"
#include "reinfer_hip.h"

#define FP_THREADS 256
#define FP_WAVES 4
#define FP_KT 64          // keys per round

__device__ __forceinline__ float fp_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// how the heads of a group and the queries are spread over a wave's column tiles
struct FpShape {
  int nc;      // column tiles a wave holds (template parameter)
  int hg;      // heads of one KV head per workgroup
  int qt;      // runs of 16 queries per wave
};
static FpShape fp_shape(int Hq, int Hkv, int d) {
  FpShape s;
  const int G = Hq / Hkv;
  s.nc = d <= 128 ? 4 : 2;
  s.hg = 1;
  for (int h = 1; h <= s.nc; ++h)
    if (G % h == 0) s.hg = h;
  s.qt = s.nc / s.hg;
  return s;
}

template <int DMAX, int NC>
__global__ void __launch_bounds__(FP_THREADS)
flash_prefill_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                     const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
                     const int* __restrict__ block_tables, int max_blocks,
                     const int* __restrict__ tile_info,      // per tile: seq, first token row, n queries, first position
                     int block_size, int Hq, int Hkv, int d, int HG, int QT, float scale_log2, int window) {
  constexpr int NDT = DMAX / 32;       // 32-wide d tiles of the score product
  constexpr int NOT = DMAX / 16;       // 16-row d tiles of the output
  constexpr int NPRE = (FP_KT * DMAX / 8) / FP_THREADS;     // 16-byte chunks a thread fetches per operand
  __shared__ __attribute__((aligned(16))) bf16_t Ks[FP_KT * DMAX];       // 4 tiles of 16 * d
  __shared__ __attribute__((aligned(16))) bf16_t Vs[FP_KT * DMAX];

  const int tid = threadIdx.x;
  const int lane = tid & (RA_WAVE - 1), wave = tid / RA_WAVE;
  const int r = lane & 15, g = lane >> 4;
  const int G = Hq / Hkv;
  const int n_hgrp = G / HG;
  const int tile = gridDim.x - 1 - blockIdx.x;          // later tiles see more keys: start them first
  const int kvh = blockIdx.y / n_hgrp, hgrp = blockIdx.y % n_hgrp;
  const int seq = tile_info[tile * 4 + 0];
  const int row0 = tile_info[tile * 4 + 1];
  const int nq = tile_info[tile * 4 + 2];
  const int pos0 = tile_info[tile * 4 + 3];
  const int* table = block_tables + (size_t)seq * max_blocks;

  // column tile j of this wave: queries (wave * QT + j / HG) * 16 + r, head hgrp * HG + j % HG
  const int n_real = QT * HG;
  int qi[NC];
  bool q_live[NC];
  bf16x8_t qreg[NC][NDT];
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    qi[j] = (wave * QT + j / HG) * 16 + r;
    q_live[j] = j < n_real && qi[j] < nq;
    const int head = kvh * G + hgrp * HG + j % HG;
    const bf16_t* qp = q + (size_t)(row0 + (q_live[j] ? qi[j] : 0)) * q_stride + (size_t)head * d;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const int e = dt * 32 + g * 8;
      qreg[j][dt] = (q_live[j] && e < d) ? *(const bf16x8_t*)(qp + e) : (bf16x8_t){0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  f32x4_t acc[NC][NOT];
  float m[NC], l[NC];
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    m[j] = -INFINITY;
    l[j] = 0.f;
#pragma unroll
    for (int i = 0; i < NOT; ++i) acc[j][i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  }

  // keys this tile of queries can see, and this wave's share of them
  const int last_pos = pos0 + nq - 1;
  const int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int kt_begin = first_key / FP_KT * FP_KT;
  const int w_q0 = wave * QT * 16;                              // first query of the wave
  const int w_first_pos = pos0 + w_q0;
  const int w_last_pos = pos0 + min(w_q0 + QT * 16, nq) - 1;    // < w_first_pos if the wave has no query

  // fetch of one round into registers: the four 16-slot tiles of K and of V, chunk by chunk
  const int tile_chunks = 2 * d;                 // 16-byte chunks of a tile
  bf16x8_t kpre[NPRE], vpre[NPRE];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int u = 0; u < NPRE; ++u) {
      const int c = tid + u * FP_THREADS;
      const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
      kpre[u] = zero;
      vpre[u] = zero;
      if (c < 4 * tile_chunks) {
        const int tt = c / tile_chunks, w = c % tile_chunks;
        const int kt = k0 + tt * 16;
        if (kt <= last_pos && kt + 15 >= first_key) {
          const int blk = table[kt / block_size];
          const size_t src = ((size_t)blk * Hkv + kvh) * block_size * d + (size_t)((kt % block_size) >> 4) * 16 * d + w * 8;
          kpre[u] = *(const bf16x8_t*)(kcache + src);
          vpre[u] = *(const bf16x8_t*)(vcache + src);
          // slots of the tile outside the visible range may hold anything (a freed block's bits): zero them
          if (kt + 15 > last_pos || kt < first_key) {
            const int kkey = kt + (w & 15);                      // K chunk w: 8 elements of slot w % 16
            if (kkey > last_pos || kkey < first_key) kpre[u] = zero;
#pragma unroll
            for (int e = 0; e < 8; ++e) {                        // V chunk w: slots 4 ((w / 8) % 4) + e % 4
              const int vkey = kt + ((w >> 3) & 3) * 4 + (e & 3);
              if (vkey > last_pos || vkey < first_key) vpre[u][e] = (bf16_t)0.f;
            }
          }
        }
      }
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int u = 0; u < NPRE; ++u) {
      const int c = tid + u * FP_THREADS;
      if (c < 4 * tile_chunks) {
        *(bf16x8_t*)(Ks + c * 8) = kpre[u];
        *(bf16x8_t*)(Vs + c * 8) = vpre[u];
      }
    }
  };

  fetch(kt_begin);
  for (int k0 = kt_begin; k0 <= last_pos; k0 += FP_KT) {
    __syncthreads();                       // the previous round is no longer read
    stage();
    __syncthreads();
    if (k0 + FP_KT <= last_pos) fetch(k0 + FP_KT);

    // a wave whose queries all lie before this round, or that has none, has nothing to add
    if (w_last_pos < w_first_pos || w_last_pos < k0) continue;
    if (window > 0 && k0 + FP_KT - 1 < w_first_pos - window + 1) continue;

    // scores S^T[key][column] for 4 sub-tiles of 16 keys
    f32x4_t s[4][NC];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int j = 0; j < NC; ++j) s[ks][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        if (dt * 32 < d) {
          const int e = dt * 32 + g * 8;
          const bf16x8_t a = (e < d) ? *(const bf16x8_t*)(Ks + ks * 16 * d + ((dt * 4 + g) * 16 + r) * 8)
                                     : (bf16x8_t){0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
          for (int j = 0; j < NC; ++j)
            s[ks][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qreg[j][dt], s[ks][j], 0, 0, 0);
        }
      }
    }
    // a round strictly inside every query's view needs no mask
    const bool inner = k0 + FP_KT - 1 <= w_first_pos && w_q0 + QT * 16 <= nq && n_real == NC &&
                       (window <= 0 || k0 >= w_last_pos - window + 1);
    bf16x8_t pb[NC][2];
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      const int q_pos = pos0 + qi[j];
      const int q_lo = (window > 0 && q_pos - window + 1 > 0) ? q_pos - window + 1 : 0;
      float tmax = -INFINITY;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = s[ks][j][i] * scale_log2;
          if (!inner) {
            const int key = k0 + ks * 16 + 4 * g + i;
            if (!(q_live[j] && key <= q_pos && key >= q_lo)) v = -INFINITY;
          }
          s[ks][j][i] = v;
          tmax = fmaxf(tmax, v);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, RA_WAVE));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, RA_WAVE));
      const float mn = fmaxf(m[j], tmax);
      // a column with nothing visible so far keeps m = -inf and adds zeros
      const float base = (mn == -INFINITY) ? 0.f : mn;
      const float corr = (mn == -INFINITY) ? 1.f : fp_exp2(m[j] - mn);
      float psum = 0.f;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = fp_exp2(s[ks][j][i] - base);      // masked: exp2(-inf) = 0
          psum += p;
          pb[j][ks / 2][(ks % 2) * 4 + i] = from_f32<bf16_t>(p);
        }
      l[j] = l[j] * corr + psum;
      m[j] = mn;
      if (__any(corr != 1.f)) {
#pragma unroll
        for (int ot = 0; ot < NOT; ++ot)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[j][ot][i] *= corr;
      }
    }
    // O^T[d][column] += V^T[d][key] P[key][column], 32 keys per instruction:
    // k-slots (g, e): e < 4 -> key 4g + e of the first 16-key tile, e >= 4 -> of the second
#pragma unroll
    for (int kp = 0; kp < 2; ++kp) {
#pragma unroll
      for (int ot = 0; ot < NOT; ++ot) {
        if (ot * 16 < d) {
          const bf16_t* v0 = Vs + (2 * kp) * 16 * d + ((ot * 4 + g) * 16 + r) * 4;
          const bf16x4_t lo4 = *(const bf16x4_t*)(v0);
          const bf16x4_t hi4 = *(const bf16x4_t*)(v0 + 16 * d);
          const bf16x8_t a = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
#pragma unroll
          for (int j = 0; j < NC; ++j)
            acc[j][ot] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[j][kp], acc[j][ot], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    // the lane groups hold partial sums of l over their own keys
    float lt = l[j];
    lt += __shfl_xor(lt, 16, RA_WAVE);
    lt += __shfl_xor(lt, 32, RA_WAVE);
    if (!q_live[j]) continue;
    const float inv = 1.f / lt;
    const int head = kvh * G + hgrp * HG + j % HG;
    bf16_t* op = out + (size_t)(row0 + qi[j]) * out_stride + (size_t)head * d;
#pragma unroll
    for (int ot = 0; ot < NOT; ++ot) {
      const int e = ot * 16 + 4 * g;
      if (e < d) {
        bf16x4_t o4 = {from_f32<bf16_t>(acc[j][ot][0] * inv), from_f32<bf16_t>(acc[j][ot][1] * inv),
                       from_f32<bf16_t>(acc[j][ot][2] * inv), from_f32<bf16_t>(acc[j][ot][3] * inv)};
        *(bf16x4_t*)(op + e) = o4;
      }
    }
  }
}

extern "C" int ra_attention_prefill_supports(int Hq, int Hkv, int d, int block_size) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return 0;
  return (d % 16 == 0 && d >= 16 && d <= 256 && block_size > 0 && block_size % 16 == 0) ? 1 : 0;
}

// queries per workgroup tile for these sizes
extern "C" int ra_attention_prefill_tile(int Hq, int Hkv, int d) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || d <= 0) return 64;
  return FP_WAVES * 16 * fp_shape(Hq, Hkv, d).qt;
}

extern "C" int ra_attention_prefill(const void* q, int q_stride, void* out, int out_stride,
                                    const void* kcache, const void* vcache, const int* block_tables,
                                    int max_blocks, const int* tile_info, int n_tiles, int block_size,
                                    int Hq, int Hkv, int d, float scale, int window, hipStream_t stream) {
  RA_CHECK(n_tiles > 0, "attention_prefill: no query tiles");
  RA_CHECK(ra_attention_prefill_supports(Hq, Hkv, d, block_size),
           "attention_prefill: unsupported sizes (%d query heads, %d KV heads, head size %d, block %d)", Hq,
           Hkv, d, block_size);
  RA_CHECK(max_blocks > 0 && window >= 0, "attention_prefill: bad cache geometry");
  RA_CHECK(q_stride % 8 == 0 && out_stride % 4 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 8) == 0 &&
               ((uintptr_t)kcache % 16) == 0 && ((uintptr_t)vcache % 16) == 0,
           "attention_prefill: operands must be 16-byte aligned");
  const FpShape sh = fp_shape(Hq, Hkv, d);
  const int G = Hq / Hkv;
  const int gy = Hkv * (G / sh.hg);
  RA_CHECK(gy <= 65535, "attention_prefill: too many heads for one launch");
  dim3 grid(n_tiles, gy);
  const float scale_log2 = scale * 1.4426950408889634f;
#define RA_FP(DM, NCC)                                                                                \
  flash_prefill_kernel<DM, NCC><<<grid, FP_THREADS, 0, stream>>>(                                     \
      (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kcache,                    \
      (const bf16_t*)vcache, block_tables, max_blocks, tile_info, block_size, Hq, Hkv, d, sh.hg,      \
      sh.qt, scale_log2, window)
  if (d <= 64) RA_FP(64, 4);
  else if (d <= 128) RA_FP(128, 4);
  else RA_FP(256, 2);
#undef RA_FP
  RA_LAUNCH_CHECK("attention_prefill");
  return 0;
}
