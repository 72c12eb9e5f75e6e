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
// row front to back. Loads for the next run are in flight while the current
// one is multiplied. The waves' partial sums are added through LDS in a fixed
// order (deterministic; no atomics).
//
// Epilogues: plain (+ bias); the SiLU gate of a feed-forward whose gate and
// up rows are interleaved in groups of 8 (tile rows 0-7 gate, 8-15 up of the
// same 8 features): out[m, 8*tile + j] = silu(gate_j) * up_j, which saves the
// [M, 2I] round trip and a launch; or accumulation into a float matrix
// (C += A . W^T: the residual add of an output projection).
// (RMSNorm of a float input inside this kernel was tried and measured slower
// than the separate norm kernel: every workgroup re-reads the rows in float.)
//
// The reference's own decode product is a thread-per-column split-K GEMV with a
// second reduce launch (crates/cuda/kernels/gemm_m1.cu:63-235).
#include "common.h"
#include "reinfer_hip.h"

enum { EPI_PLAIN = 0, EPI_SILU_PAIRS = 1, EPI_ACCUM = 2 };

template <int MT, int NT, int WAVES, int U, int EPI, typename TO>
__global__ void __launch_bounds__(WAVES * RA_WAVE)
gemm_skinny_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W,
                   const bf16_t* __restrict__ bias, TO* __restrict__ C, int ldc, int M, int N, int K) {
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

  const int span = WAVES * KS;
  int k0 = wave * KS;
  if (k0 < K) gload(k0);
  for (; k0 < K; k0 += span) {
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
    if (k0 + span < K) gload(k0 + span);
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
                         int out_dtype, int epilogue, int M, int N, int K, hipStream_t stream) {
  const int grid = (N + 16 * NT - 1) / (16 * NT);
#define RA_GO(EPI, TO)                                                                     \
  gemm_skinny_kernel<MT, NT, WAVES, U, EPI, TO><<<grid, WAVES * RA_WAVE, 0, stream>>>(     \
      (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, (TO*)C, ldc, M, N, K)
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

extern "C" int ra_gemm_skinny(const void* A, const void* W, const void* bias, void* C, int out_dtype,
                              int epilogue, int M, int N, int K, int lda, int ldc, hipStream_t stream) {
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
  if (M <= 16) return launch_skinny<1, 1, 8, 4>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, stream);
  if (M <= 32) return launch_skinny<2, 1, 8, 4>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, stream);
  // 33..64 rows: with few output features, 16 a workgroup keep all CUs busy; with many, 32 a
  // workgroup halve the activations each one re-reads (measured at N = 4096 and 24576)
  if (N <= 8192) return launch_skinny<4, 1, 8, 2>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, stream);
  return launch_skinny<4, 2, 8, 2>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, stream);
}
