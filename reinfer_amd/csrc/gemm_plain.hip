// Plain tiled matrix product  C[M,N] = A[M,K] . W[N,K]^T (+ bias[N]),
// float accumulation with ordinary FMA (no matrix-core instruction, no
// reduced-precision mode): the product of the true 32-bit path and the twin of
// the MFMA kernels. Both operands are row-major with K contiguous, which is how
// checkpoints store a projection ([out, in]); the reference transposes at load
// instead (crates/cuda/src/engine.rs:6523-6540) and calls cublasGemmEx with
// float accumulation (crates/cuda/src/gemm.rs:226-292).
#include "common.h"
#include "reinfer_hip.h"

#define TM 64
#define TN 64
#define TK 16

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
gemm_plain_kernel(const TI* __restrict__ A, const TI* __restrict__ W, const TI* __restrict__ bias,
                  TO* __restrict__ C, int M, int N, int K, int lda, int ldc) {
  __shared__ float As[TK][TM + 4];
  __shared__ float Ws[TK][TN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int tr = (tid / 16) * 4, tc = (tid % 16) * 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += TK) {
    // 64 rows x 16 k per operand = 1024 elements, 4 per thread
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + e * 256;
      const int r = idx / TK, kk = idx % TK;
      const int k = k0 + kk;
      As[kk][r] = (m0 + r < M && k < K) ? to_f32(A[(size_t)(m0 + r) * lda + k]) : 0.f;
      Ws[kk][r] = (n0 + r < N && k < K) ? to_f32(W[(size_t)(n0 + r) * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][tr + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tc + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + tr + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tc + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += to_f32(bias[n]);
      C[(size_t)m * ldc + n] = from_f32<TO>(v);
    }
  }
}

extern "C" int ra_gemm_plain(const void* A, const void* W, const void* bias, void* C, int in_dtype,
                             int out_dtype, int M, int N, int K, int lda, int ldc, hipStream_t stream) {
  RA_CHECK(M > 0 && N > 0 && K > 0, "gemm_plain: empty product (%d, %d, %d)", M, N, K);
  RA_CHECK(lda >= K && ldc >= N, "gemm_plain: row strides (%d, %d) below the row lengths (%d, %d)", lda, ldc, K, N);
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  RA_CHECK(grid.y <= 65535, "gemm_plain: %d rows in one launch", M);
#define RA_GO(TI, TO)                                                                         \
  gemm_plain_kernel<TI, TO><<<grid, 256, 0, stream>>>((const TI*)A, (const TI*)W, (const TI*)bias, \
                                                      (TO*)C, M, N, K, lda, ldc)
  if (in_dtype == RA_F32 && out_dtype == RA_F32) RA_GO(float, float);
  else if (in_dtype == RA_BF16 && out_dtype == RA_BF16) RA_GO(bf16_t, bf16_t);
  else if (in_dtype == RA_BF16 && out_dtype == RA_F32) RA_GO(bf16_t, float);
  else return ra_fail("gemm_plain: unsupported dtypes (in %d, out %d)", in_dtype, out_dtype);
#undef RA_GO
  RA_LAUNCH_CHECK("gemm_plain");
  return 0;
}
