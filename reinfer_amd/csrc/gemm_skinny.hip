// Weight-streaming product for few rows (decode):  C[M,N] = A[M,K] . W[N,K]^T,
// M <= 64, bfloat16 in, float accumulation on the matrix cores.
//
// The step is bound by reading W once from HBM, so every global load is laid
// out for the memory pipeline, not for the MFMA: one wave instruction covers a
// few rows times a contiguous run of 16*LPR bytes (16 bytes a lane, adjacent
// lanes adjacent in memory). The MFMA wants lane (r, g) to hold row r, k-chunk
// g, which read straight from memory makes 64 scattered 16-byte requests per
// instruction; measured on MI355X that pattern tops out near 9 TB/s out of the
// cache against 26 TB/s for contiguous runs, and weights plus activations
// together hit it. So both operands go registers -> LDS (row-contiguous,
// padded pitch) -> registers in MFMA layout, in a tile private to the wave: no
// workgroup barrier in the loop, only the wave's own LDS ordering.
//
// A workgroup owns 16*NT output features. Its waves split K: wave w takes the
// k-runs w, w + WAVES, ... of U*32 elements, so together they walk each weight
// row, from a start that differs from workgroup to workgroup, once round. Loads for the next run are in flight while the current
// one is multiplied. The waves' partial sums are added through LDS in a fixed
// order (deterministic; no atomics).
//
// Epilogues: plain (+ bias); the SiLU gate of a feed-forward whose gate and
// up rows are interleaved in groups of 8 (tile rows 0-7 gate, 8-15 up of the
// same 8 features): out[m, 8*tile + j] = silu(gate_j) * up_j, which saves the
// [M, 2I] round trip and a launch; or accumulation into a float matrix
// (C += A . W^T: the residual add of an output projection).
//
// RMSNorm around the product, without a kernel of its own: y = rstd[m] * ((x .* w) . W^T), so the
// norm's column weight can be applied by whoever wrote x and its row factor after the product.
// A product that adds into the residual stream (epilogue 2) can also write bf16(stream * w) for the
// norm that follows and, a workgroup, the sum of squares of its 16*NT columns of each row
// ("emit"); the next product takes those partial sums, adds them in a fixed order and scales its
// result rows by rsqrt(sum / width + eps) ("row sums"). (Normalising a float input inside the
// consuming product instead was tried and measured slower: every workgroup re-reads the rows in
// float and must finish the sums before its first MFMA.)
//
// The reference's own decode product is a thread-per-column split-K GEMV with a
// second reduce launch (crates/cuda/kernels/gemm_m1.cu:63-235).
#include "common.h"
#include "reinfer_hip.h"

enum { EPI_PLAIN = 0, EPI_SILU_PAIRS = 1, EPI_ACCUM = 2 };

// RMSNorm carried by the products around it (all pointers may be null)
struct SkinnyNorm {
  const float* in_ss;      // [in_parts, M] partial sums of squares of the rows behind A
  int in_parts;
  float in_eps, in_inv_width;
  const void* out_w;       // [N] weight of the norm that follows (epilogue 2 only)
  int out_w_f32;           // 1: float, 0: bfloat16
  bf16_t* out_x;           // [M, out_ldx] bf16(C_new * out_w)
  int out_ldx;
  float* out_ss;           // [workgroups, M] sums of squares of C_new over the workgroup's columns
};

template <int MT, int NT, int WAVES, int U, int EPI, typename TO>
__global__ void __launch_bounds__(WAVES * RA_WAVE)
gemm_skinny_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W,
                   const bf16_t* __restrict__ bias, TO* __restrict__ C, int ldc, int M, int N, int K,
                   SkinnyNorm nf) {
  constexpr int KS = U * 32;                 // k elements per wave run
  constexpr int LPR = U * 4;                 // lanes per row segment (16 bytes each)
  constexpr int RPI = RA_WAVE / LPR;         // rows per load instruction
  constexpr int NI = 16 / RPI;               // load instructions per 16-row tile
  constexpr int PITCH = KS + 8;              // LDS row pitch in elements: 16 bytes of padding
  constexpr int TILE = 16 * PITCH;
  constexpr int STAGE = (NT + MT) * TILE;    // staged elements per wave
  constexpr int RED = (WAVES - 1) * NT * MT * RA_WAVE * 4 * 2;   // partial sums, in bf16 units
  constexpr int LDS_ELEMS = (WAVES * STAGE > RED) ? WAVES * STAGE : RED;
  __shared__ __attribute__((aligned(16))) bf16_t lds[LDS_ELEMS];
  __shared__ float row_ss[WAVES][MT * 16];   // each wave's share of the rows' sums of squares

  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int r = lane & 15, g = lane >> 4;              // MFMA operand layout
  const int lr = lane / LPR, lc = lane % LPR;          // load layout
  const int n0 = blockIdx.x * (16 * NT);
  bf16_t* my = lds + wave * STAGE;

  const bf16_t* wp[NT][NI];
  const bf16_t* ap[MT][NI];
  bool aok[MT][NI];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      int n = n0 + nt * 16 + i * RPI + lr;
      n = n < N ? n : N - 1;                 // rows past the end are computed and dropped
      wp[nt][i] = W + (size_t)n * K + lc * 8;
    }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      int m = mt * 16 + i * RPI + lr;
      aok[mt][i] = m < M;                    // rows past M are zeros, not loaded
      m = m < M ? m : M - 1;
      ap[mt][i] = A + (size_t)m * lda + lc * 8;
    }
  f32x4_t acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8_t wr[NT][NI], ar[MT][NI];
  auto gload = [&](int k0) {
    const bool ok = k0 + lc * 8 < K;         // K is a multiple of 8: a chunk is in or out as a whole
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < NI; ++i) wr[nt][i] = ok ? *(const bf16x8_t*)(wp[nt][i] + k0) : zero;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < NI; ++i) ar[mt][i] = (ok && aok[mt][i]) ? *(const bf16x8_t*)(ap[mt][i] + k0) : zero;
  };

  // A workgroup's waves walk K together, a span of WAVES runs a step. Workgroups start at different
  // steps and wrap round: in step, the rows read at one moment (a whole K apart from each other, at
  // the same offset) fall on few memory channels. A run past K loads nothing and multiplies zeros.
  const int span = WAVES * KS;
  const int n_steps = (K + span - 1) / span;
  // (Measured: a gain where the grid is larger than the chip holds at once or K is long; a small loss
  // at 6144 x 4096, where all workgroups run side by side and share the activations they read in step.)
  const int rot = (gridDim.x > 512 || K > 8192) ? (int)((blockIdx.x * 7u) % (unsigned)n_steps) : 0;
  auto k_of = [&](int step) {
    const int q = step + rot < n_steps ? step + rot : step + rot - n_steps;
    return q * span + wave * KS;
  };
  gload(k_of(0));
  // This wave's share of the rows' partial sums, p = 4 wave + g, + 4 WAVES, ...: the first SS_HELD of a
  // lane are asked for here, behind the first weights, and not touched before the loop is over, so
  // that no wait for them holds up the weight stream; any further ones are read after the loop.
  constexpr int SS_HELD = 8;
  float ss_held[MT][SS_HELD];
  if (nf.in_ss) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
#pragma unroll
      for (int j = 0; j < SS_HELD; ++j) {
        const int p = wave * 4 + g + j * WAVES * 4;
        ss_held[mt][j] = (m < M && p < nf.in_parts) ? nf.in_ss[(size_t)p * M + m] : 0.f;
      }
    }
  }
  for (int step = 0; step < n_steps; ++step) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < NI; ++i)
        *(bf16x8_t*)(my + nt * TILE + (i * RPI + lr) * PITCH + lc * 8) = wr[nt][i];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < NI; ++i)
        *(bf16x8_t*)(my + (NT + mt) * TILE + (i * RPI + lr) * PITCH + lc * 8) = ar[mt][i];
    // the tile is the wave's own: its LDS operations complete in order, so waiting
    // for them is all the ordering the re-layout needs
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (step + 1 < n_steps) gload(k_of(step + 1));
    bf16x8_t a[NT][U], b[MT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        a[nt][u] = *(const bf16x8_t*)(my + nt * TILE + r * PITCH + u * 32 + g * 8);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        b[mt][u] = *(const bf16x8_t*)(my + (NT + mt) * TILE + r * PITCH + u * 32 + g * 8);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt][u], b[mt][u], acc[nt][mt], 0, 0, 0);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // reads done before the next run overwrites the tile
  }

  if (nf.in_ss) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
      float t = 0.f;
#pragma unroll
      for (int j = 0; j < SS_HELD; ++j) t += ss_held[mt][j];
      if (m < M)
        for (int p = wave * 4 + g + SS_HELD * WAVES * 4; p < nf.in_parts; p += WAVES * 4)
          t += nf.in_ss[(size_t)p * M + m];
      t += __shfl_xor(t, 16, RA_WAVE);
      t += __shfl_xor(t, 32, RA_WAVE);
      if (g == 0) row_ss[wave][mt * 16 + r] = t;
    }
  }
  // add the waves' partial sums: wave w > 0 writes, wave 0 adds in order 1, 2, ...
  __syncthreads();                           // the staging tiles are dead; their LDS is reused
  float* red = (float*)lds;
  if (wave > 0) {
    float* dst = red + (size_t)(wave - 1) * NT * MT * RA_WAVE * 4;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[((nt * MT + mt) * 4 + i) * RA_WAVE + lane] = acc[nt][mt][i];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int w = 1; w < WAVES; ++w) {
    const float* src = red + (size_t)(w - 1) * NT * MT * RA_WAVE * 4;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[nt][mt][i] += src[((nt * MT + mt) * 4 + i) * RA_WAVE + lane];
  }
  // lane (r, g) holds C[feature 4g + i of the tile][token r]
  if (nf.in_ss) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) t += row_ss[w][mt * 16 + r];
      const float rstd = rsqrtf(t * nf.in_inv_width + nf.in_eps);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[nt][mt][i] *= rstd;
    }
  }
  if (EPI == EPI_ACCUM && nf.out_x) {
    // the sum goes into the stream; the norm that follows gets bf16(sum * weight) and this
    // workgroup's part of each row's sum of squares
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
      float ss = 0.f;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + nt * 16 + 4 * g + i;
          if (m >= M || n >= N) continue;
          float v = acc[nt][mt][i];
          if (bias) v += to_f32(bias[n]);
          v += to_f32(C[(size_t)m * ldc + n]);           // this thread alone owns (m, n)
          C[(size_t)m * ldc + n] = from_f32<TO>(v);
          const float w = nf.out_w_f32 ? ((const float*)nf.out_w)[n] : to_f32(((const bf16_t*)nf.out_w)[n]);
          nf.out_x[(size_t)m * nf.out_ldx + n] = from_f32<bf16_t>(v * w);
          ss += v * v;
        }
      ss += __shfl_xor(ss, 16, RA_WAVE);
      ss += __shfl_xor(ss, 32, RA_WAVE);
      if (g == 0 && m < M) nf.out_ss[(size_t)blockIdx.x * M + m] = ss;
    }
    return;
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
      if (EPI == EPI_ACCUM) {
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + nt * 16 + 4 * g + i;
          if (n >= N) continue;
          float v = acc[nt][mt][i];
          if (bias) v += to_f32(bias[n]);
          C[(size_t)m * ldc + n] = from_f32<TO>(to_f32(C[(size_t)m * ldc + n]) + v);   // this thread alone owns (m, n)
        }
      } else if (EPI == EPI_PLAIN) {
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + nt * 16 + 4 * g + i;
          if (n >= N) continue;
          float v = acc[nt][mt][i];
          if (bias) v += to_f32(bias[n]);
          C[(size_t)m * ldc + n] = from_f32<TO>(v);
        }
      } else {
        // rows 0-7 of the tile are gate, 8-15 up of the same features: the up value of
        // gate row 4g + i sits in lane (r, g + 2), same i
        float up[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) up[i] = __shfl_xor(acc[nt][mt][i], 32, RA_WAVE);
        if (m >= M || g >= 2) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int f = (n0 / 16 + nt) * 8 + 4 * g + i;
          if (2 * f >= N) continue;          // N = 2 I
          const float gt = acc[nt][mt][i];
          C[(size_t)m * ldc + f] = from_f32<TO>(gt / (1.f + __expf(-gt)) * up[i]);
        }
      }
    }
}

template <int MT, int NT, int WAVES, int U>
static int launch_skinny(const void* A, int lda, const void* W, const void* bias, void* C, int ldc,
                         int out_dtype, int epilogue, int M, int N, int K, const SkinnyNorm& nf,
                         hipStream_t stream) {
  const int grid = (N + 16 * NT - 1) / (16 * NT);
#define RA_GO(EPI, TO)                                                                     \
  gemm_skinny_kernel<MT, NT, WAVES, U, EPI, TO><<<grid, WAVES * RA_WAVE, 0, stream>>>(     \
      (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, (TO*)C, ldc, M, N, K, nf)
  if (epilogue == EPI_SILU_PAIRS) {
    if (out_dtype == RA_BF16) RA_GO(EPI_SILU_PAIRS, bf16_t);
    else RA_GO(EPI_SILU_PAIRS, float);
  } else if (epilogue == EPI_ACCUM) {
    RA_GO(EPI_ACCUM, float);
  } else {
    if (out_dtype == RA_BF16) RA_GO(EPI_PLAIN, bf16_t);
    else RA_GO(EPI_PLAIN, float);
  }
#undef RA_GO
  RA_LAUNCH_CHECK("gemm_skinny");
  return 0;
}

extern "C" int ra_gemm_skinny_max_rows(void) { return 64; }

// Output features a workgroup owns at M rows and N features: the unit of the emitted partial sums.
static int skinny_features(int M, int N) { return (M > 32 && N > 8192) ? 32 : 16; }

extern "C" int ra_gemm_skinny_row_parts(int M, int N) {
  const int f = skinny_features(M, N);
  return (N + f - 1) / f;
}

extern "C" int ra_gemm_skinny_normed(const void* A, const void* W, const void* bias, void* C, int out_dtype,
                                     int epilogue, int M, int N, int K, int lda, int ldc, const float* in_ss,
                                     int in_parts, float in_eps, int in_width, const void* out_w,
                                     int out_w_dtype, void* out_x, int out_ldx, float* out_ss,
                                     hipStream_t stream) {
  RA_CHECK(M > 0 && N > 0 && K > 0, "gemm_skinny: empty product (%d, %d, %d)", M, N, K);
  RA_CHECK(M <= 64, "gemm_skinny: %d rows; this kernel takes at most 64", M);
  RA_CHECK(K % 8 == 0 && lda % 8 == 0, "gemm_skinny: K (%d) and the row stride (%d) must be multiples of 8", K, lda);
  RA_CHECK(epilogue == EPI_PLAIN || epilogue == EPI_SILU_PAIRS || epilogue == EPI_ACCUM, "gemm_skinny: unknown epilogue %d", epilogue);
  RA_CHECK(epilogue != EPI_ACCUM || out_dtype == RA_F32, "gemm_skinny: accumulation is into a float matrix");
  const int n_out = epilogue == EPI_SILU_PAIRS ? N / 2 : N;
  RA_CHECK(epilogue != EPI_SILU_PAIRS || (N % 16 == 0 && bias == nullptr),
           "gemm_skinny: the gated epilogue needs N (%d) in whole tiles of 16 and no bias", N);
  RA_CHECK(lda >= K && ldc >= n_out, "gemm_skinny: row strides (%d, %d) below the row lengths (%d, %d)", lda, ldc, K, n_out);
  RA_CHECK(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_skinny: operands must be 16-byte aligned");
  RA_CHECK(out_dtype == RA_BF16 || out_dtype == RA_F32, "gemm_skinny: unknown output dtype tag %d", out_dtype);
  SkinnyNorm nf = {};
  if (in_ss) {
    RA_CHECK(in_parts > 0 && in_width > 0 && in_eps >= 0.f, "gemm_skinny: row sums need parts (%d), width (%d) and eps", in_parts, in_width);
    nf.in_ss = in_ss;
    nf.in_parts = in_parts;
    nf.in_eps = in_eps;
    nf.in_inv_width = 1.f / (float)in_width;
  }
  if (out_x || out_ss || out_w) {
    RA_CHECK(epilogue == EPI_ACCUM, "gemm_skinny: only the accumulating epilogue emits for a norm");
    RA_CHECK(M <= 16, "gemm_skinny: with %d rows the other product kernel emits for a norm (this one up to 16)", M);
    RA_CHECK(out_x && out_ss && out_w, "gemm_skinny: emitting needs the norm weight, the scaled copy and the partial sums");
    RA_CHECK(out_w_dtype == RA_BF16 || out_w_dtype == RA_F32, "gemm_skinny: unknown norm weight dtype tag %d", out_w_dtype);
    RA_CHECK(out_ldx >= N, "gemm_skinny: the scaled copy's row stride (%d) is below %d", out_ldx, N);
    nf.out_w = out_w;
    nf.out_w_f32 = out_w_dtype == RA_F32;
    nf.out_x = (bf16_t*)out_x;
    nf.out_ldx = out_ldx;
    nf.out_ss = out_ss;
  }
  if (M <= 16) return launch_skinny<1, 1, 8, 4>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, stream);
  if (M <= 32) return launch_skinny<2, 1, 8, 4>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, stream);
  // 33..64 rows: with few output features, 16 a workgroup keep all CUs busy; with many, 32 a
  // workgroup halve the activations each one re-reads (measured at N = 4096 and 24576)
  if (skinny_features(M, N) == 16)
    return launch_skinny<4, 1, 8, 2>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, stream);
  return launch_skinny<4, 2, 8, 2>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, stream);
}

extern "C" int ra_gemm_skinny(const void* A, const void* W, const void* bias, void* C, int out_dtype,
                              int epilogue, int M, int N, int K, int lda, int ldc, hipStream_t stream) {
  return ra_gemm_skinny_normed(A, W, bias, C, out_dtype, epilogue, M, N, K, lda, ldc, nullptr, 0, 0.f, 0, nullptr,
                               0, nullptr, 0, nullptr, stream);
}
