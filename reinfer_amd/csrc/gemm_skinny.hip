// Weight-streaming product for few rows (decode):  C[M,N] = A[M,K] . W[N,K]^T,
// M <= 64, bfloat16 in, float accumulation on the matrix cores.
//
// The weight tile is the MFMA's first operand: 16 output features x 32 k per
// instruction, each lane loading 16 bytes (8 k) of one weight row straight from
// HBM into registers, so every weight byte is read once and never touches LDS.
// The activations are the second operand (16 tokens x 32 k, L2-resident).
// A workgroup owns 16*NT output features; its wavefronts take interleaved
// k-tiles (wave w: tiles w, w + WAVES, ...) so that together they read each
// weight row in one contiguous run, and their partial sums are added through
// LDS in a fixed order (deterministic; no atomics).
//
// The reference's own decode product is a thread-per-column split-K GEMV with a
// second reduce launch (crates/cuda/kernels/gemm_m1.cu:63-235); this one keeps
// the reduce inside the workgroup and uses v_mfma_f32_16x16x32_bf16.
#include "common.h"
#include "reinfer_hip.h"

template <int MT, int NT, int WAVES, int U, typename TO>
__global__ void __launch_bounds__(WAVES * RA_WAVE)
gemm_skinny_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W,
                   const bf16_t* __restrict__ bias, TO* __restrict__ C, int ldc, int M, int N, int K) {
  __shared__ float red[(WAVES - 1) * NT * MT * RA_WAVE * 4];
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (16 * NT);

  const bf16_t* wrow[NT];
  const bf16_t* arow[MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int n = n0 + nt * 16 + r;
    n = n < N ? n : N - 1;                  // rows past the end are computed and dropped
    wrow[nt] = W + (size_t)n * K;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = mt * 16 + r;
    m = m < M ? m : M - 1;
    arow[mt] = A + (size_t)m * lda;
  }
  f32x4_t acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const int ktiles = (K + 31) / 32;
  const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int kt = wave; kt < ktiles; kt += WAVES * U) {
    bf16x8_t a[NT][U], b[MT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (kt + u * WAVES) * 32 + g * 8;
      const bool ok = k < K;                 // K is a multiple of 8: a chunk is in or out as a whole
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) a[nt][u] = ok ? *(const bf16x8_t*)(wrow[nt] + k) : zero;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[mt][u] = ok ? *(const bf16x8_t*)(arow[mt] + k) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nt][u], b[mt][u], acc[nt][mt], 0, 0, 0);
  }

  // add the wavefronts' partial sums: wave w > 0 writes, wave 0 adds in order 1, 2, ...
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
  // C[row = feature 4g + i][col = token r] of each 16x16 tile
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
      if (m >= M) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + nt * 16 + 4 * g + i;
        if (n >= N) continue;
        float v = acc[nt][mt][i];
        if (bias) v += to_f32(bias[n]);
        C[(size_t)m * ldc + n] = from_f32<TO>(v);
      }
    }
}

template <int MT, int NT, int WAVES, int U>
static int launch_skinny(const void* A, int lda, const void* W, const void* bias, void* C, int ldc,
                         int out_dtype, int M, int N, int K, hipStream_t stream) {
  const int grid = (N + 16 * NT - 1) / (16 * NT);
  if (out_dtype == RA_BF16)
    gemm_skinny_kernel<MT, NT, WAVES, U, bf16_t><<<grid, WAVES * RA_WAVE, 0, stream>>>(
        (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, (bf16_t*)C, ldc, M, N, K);
  else
    gemm_skinny_kernel<MT, NT, WAVES, U, float><<<grid, WAVES * RA_WAVE, 0, stream>>>(
        (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, (float*)C, ldc, M, N, K);
  RA_LAUNCH_CHECK("gemm_skinny");
  return 0;
}

extern "C" int ra_gemm_skinny_max_rows(void) { return 64; }

extern "C" int ra_gemm_skinny(const void* A, const void* W, const void* bias, void* C, int out_dtype,
                              int M, int N, int K, int lda, int ldc, hipStream_t stream) {
  RA_CHECK(M > 0 && N > 0 && K > 0, "gemm_skinny: empty product (%d, %d, %d)", M, N, K);
  RA_CHECK(M <= 64, "gemm_skinny: %d rows; this kernel takes at most 64", M);
  RA_CHECK(K % 8 == 0 && lda % 8 == 0, "gemm_skinny: K (%d) and the row stride (%d) must be multiples of 8", K, lda);
  RA_CHECK(lda >= K && ldc >= N, "gemm_skinny: row strides (%d, %d) below the row lengths (%d, %d)", lda, ldc, K, N);
  RA_CHECK(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_skinny: operands must be 16-byte aligned");
  RA_CHECK(out_dtype == RA_BF16 || out_dtype == RA_F32, "gemm_skinny: unknown output dtype tag %d", out_dtype);
  if (M <= 16) return launch_skinny<1, 1, 8, 4>(A, lda, W, bias, C, ldc, out_dtype, M, N, K, stream);
  if (M <= 32) return launch_skinny<2, 1, 8, 4>(A, lda, W, bias, C, ldc, out_dtype, M, N, K, stream);
  return launch_skinny<4, 2, 4, 2>(A, lda, W, bias, C, ldc, out_dtype, M, N, K, stream);
}
