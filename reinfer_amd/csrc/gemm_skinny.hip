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

// What follows the walk over K in both kernels below: the waves' partial sums added in a fixed order,
// the carried norm's row factor, the epilogue. `ss_held` are the first SS_HELD partial sums of squares
// of this lane's row (asked for before the walk); `pre`, if filled, holds the values of C that this
// thread will add to (epilogue 2) and the following norm's weights of its columns (`pre`), asked for
// before the walk so that no trip to memory is left at the end.
constexpr int SS_HELD = 8;
template <int NT, int MT>
struct SkinnyAhead {
  bool have_c, have_w;         // wave-uniform
  float c[NT][MT][4];          // C[token r][feature 4g + i of tile nt]
  unsigned w[NT][4];           // the next norm's weight of the same features: float bits, or bfloat16 bits
};
template <int MT, int NT, int WAVES, int EPI, typename TO>
__device__ __forceinline__ void skinny_finish(f32x4_t (&acc)[NT][MT], const float (&ss_held)[MT][SS_HELD],
                                              const SkinnyAhead<NT, MT>& pre, bf16_t* lds,
                                              float (*row_ss)[MT * 16],
                                              const bf16_t* __restrict__ bias, TO* __restrict__ C, int ldc,
                                              int M, int N, int n0, const SkinnyNorm& nf) {
  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int r = lane & 15, g = lane >> 4;
  if (nf.in_ss) {
    // In the persistent kernel this runs once a tile, and a wave may write row_ss for the next tile while
    // wave 0 still reads it for this one, with no barrier between: that is safe because what is written
    // does not depend on the tile (the sums of squares of the input rows are the same for every feature
    // tile), so the racing write stores the value that is already there.
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
          v += pre.have_c ? pre.c[nt][mt][i] : to_f32(C[(size_t)m * ldc + n]);           // this thread alone owns (m, n)
          C[(size_t)m * ldc + n] = from_f32<TO>(v);
          const float w = pre.have_w ? __uint_as_float(nf.out_w_f32 ? pre.w[nt][i] : pre.w[nt][i] << 16)
                                     : (nf.out_w_f32 ? ((const float*)nf.out_w)[n] : to_f32(((const bf16_t*)nf.out_w)[n]));
          nf.out_x[(size_t)m * nf.out_ldx + n] = from_f32<bf16_t>(v * w);
          ss += v * v;
        }
      ss += __shfl_xor(ss, 16, RA_WAVE);
      ss += __shfl_xor(ss, 32, RA_WAVE);
      if (g == 0 && m < M) nf.out_ss[(size_t)(n0 / (16 * NT)) * M + m] = ss;      // the tile's number: a workgroup may take several
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
          const float c0 = pre.have_c ? pre.c[nt][mt][i] : to_f32(C[(size_t)m * ldc + n]);
          C[(size_t)m * ldc + n] = from_f32<TO>(c0 + v);   // this thread alone owns (m, n)
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
  float ss_held[MT][SS_HELD] = {};
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

  SkinnyAhead<NT, MT> none;
  none.have_c = none.have_w = false;
  skinny_finish<MT, NT, WAVES, EPI, TO>(acc, ss_held, none, lds, row_ss, bias, C, ldc, M, N, n0, nf);
}

// Up to 16 rows: the same product with a wave's loads DEPTH runs ahead, in workgroups that stay. A
// launch of the decode step is short (a few microseconds of streaming), so what it costs beside the
// streaming is trips to memory that wait for each other, and workgroups that start when others end
// and pay those trips again. Here nothing waits that does not have to:
//  - the grid is what the chip holds at once (the host sees to that); a workgroup takes the tiles
//    b, b + grid, ... and its ring of loads runs on across tile ends, so the weight stream of a
//    wave never stops between tiles;
//  - everything a wave needs first (the values of C it will add to, the next norm's weights, the
//    carried norm's partial sums, then its first DEPTH runs of weights and activations) is asked
//    for at once behind the kernel's arguments, and nothing of it is touched before it is needed;
//  - every load is unconditional (a chunk past K, a row past M or a run past the end reads the
//    matrix's first bytes and is replaced by zeros when it is used): no branch around a load, so the
//    waits count loads exactly;
//  - the run DEPTH ahead is asked for as soon as a run's registers are free.
// A tile's runs are padded to a multiple of DEPTH (runs of zeros), so that a tile ends where a round
// of the ring ends. MROWS = rows of A that are loaded (4, 8 or 16: the least that holds M).
template <int NT, int WAVES, int U, int DEPTH, int OCC, int MROWS, int EPI, typename TO>
__global__ void __launch_bounds__(WAVES * RA_WAVE, OCC)
gemm_skinny_deep_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W,
                        const bf16_t* __restrict__ bias, TO* __restrict__ C, int ldc, int M, int N, int K,
                        SkinnyNorm nf) {
  constexpr int MT = (MROWS + 15) / 16;            // row tiles of A
  constexpr int KS = U * 32;
  constexpr int LPR = U * 4;
  constexpr int RPI = RA_WAVE / LPR;
  constexpr int NI = 16 / RPI;
  constexpr int MI = (MROWS + RPI - 1) / RPI;      // load instructions that cover the rows of A
  constexpr int MZ = MT * 16 / RPI;                // load instructions that would cover every row tile
  constexpr int PITCH = KS + 8;
  constexpr int TILE = 16 * PITCH;
  constexpr int STAGE = (NT + MT) * TILE;
  constexpr int RED = (WAVES - 1) * NT * MT * RA_WAVE * 4 * 2;     // in bf16 units
  __shared__ __attribute__((aligned(16))) bf16_t lds[WAVES * STAGE];
  __shared__ __attribute__((aligned(16))) bf16_t red[RED];          // its own: the next tile's runs are staged meanwhile
  __shared__ float row_ss[WAVES][MT * 16];

  const int lane = threadIdx.x & (RA_WAVE - 1);
  const int wave = threadIdx.x / RA_WAVE;
  const int r = lane & 15, g = lane >> 4;              // MFMA operand layout
  const int lr = lane / LPR, lc = lane % LPR;          // load layout
  bf16_t* my = lds + wave * STAGE;

  const int span = WAVES * KS;
  const int n_steps = (K + span - 1) / span;
  const int n_steps_p = (n_steps + DEPTH - 1) / DEPTH * DEPTH;
  const int n_tiles = (N + 16 * NT - 1) / (16 * NT);
  const int stride_n = (int)gridDim.x * 16 * NT;
  const int n_mine = (n_tiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
  const int total = n_mine * n_steps_p;
  // Workgroups start their walk over K at different runs and wrap round where many run side by side:
  // in step, the rows read at one moment, a whole K apart, fall on few memory channels.
  const int rot = (n_tiles > 512 || K > 8192) ? (int)((blockIdx.x * 7u) % (unsigned)n_steps) : 0;

  // Both operands are read through buffer descriptors: a load whose offset lies past the descriptor's end
  // returns zeros and touches no memory, so rows past N or M, chunks past K, padding runs and runs past
  // the workgroup's last tile are loads like any other (they count in order) that cost nothing.
  constexpr unsigned NOWHERE = 0xFFFFFFF0u;
  const __amdgpu_buffer_rsrc_t w_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(W), 0, (int)((size_t)N * K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t a_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(A), 0, (int)(((size_t)(M - 1) * lda + K) * 2), 0x00020000);
  unsigned a_off[MI];                      // byte offset of this lane's chunk in run 0, or NOWHERE
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = i * RPI + lr;
    a_off[i] = m < M ? (unsigned)(((size_t)m * lda + lc * 8) * 2) : NOWHERE;
  }

  // what the end of the first tile needs from memory, asked for first (loads complete in order: behind the
  // weights they would make the first run wait for all of them) and not touched before the walk is
  // over (any arithmetic on it would wait for it); indices are clamped, so no branch guards a load
  SkinnyAhead<NT, MT> pre;
  pre.have_c = EPI == EPI_ACCUM && wave == 0;
  pre.have_w = pre.have_c && nf.out_w != nullptr;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) pre.c[nt][mt][i] = 0.f;
      pre.w[nt][i] = 0u;
    }
  if (EPI == EPI_ACCUM && pre.have_c) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r < M ? mt * 16 + r : M - 1;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          int n = (int)blockIdx.x * 16 * NT + nt * 16 + 4 * g + i;
          n = n < N ? n : N - 1;
          pre.c[nt][mt][i] = ((const float*)C)[(size_t)m * ldc + n];
        }
    }
    if (pre.have_w) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          int n = (int)blockIdx.x * 16 * NT + nt * 16 + 4 * g + i;
          n = n < N ? n : N - 1;
          pre.w[nt][i] = nf.out_w_f32 ? ((const unsigned*)nf.out_w)[n] : (unsigned)((const unsigned short*)nf.out_w)[n];
        }
    }
  }
  float ss_held[MT][SS_HELD] = {};
  if (nf.in_ss) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int ss_m = mt * 16 + r < M ? mt * 16 + r : M - 1;
#pragma unroll
      for (int j = 0; j < SS_HELD; ++j) {
        int p = wave * 4 + g + j * WAVES * 4;
        p = p < nf.in_parts ? p : nf.in_parts - 1;
        ss_held[mt][j] = nf.in_ss[(size_t)p * M + ss_m];
      }
    }
  }

  // the ring: run q of this workgroup (tile q / n_steps_p, step q % n_steps_p) sits in slot q % DEPTH
  bf16x8_t wr[DEPTH][NT][NI], ar[DEPTH][MI];
  int l_q = 0, l_step = 0, l_n0 = (int)blockIdx.x * 16 * NT;        // where the loads are
  // `d` is a constant after unrolling: the ring of registers is indexed statically
#define RA_DEEP_LOAD(d)                                                                        \
  do {                                                                                         \
    int kk_ = K;                          /* a padding run, or past the end: nothing is read */ \
    if (l_q < total && l_step < n_steps) {                                                     \
      const int q_ = l_step + rot < n_steps ? l_step + rot : l_step + rot - n_steps;           \
      kk_ = q_ * span + wave * KS + lc * 8;                                                    \
    }                                                                                          \
    const bool ok_ = kk_ < K;             /* K is a multiple of 8: a chunk is in or out as a whole */ \
    _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                          \
      _Pragma("unroll") for (int i = 0; i < NI; ++i) {                                         \
        const int n_ = l_n0 + nt * 16 + i * RPI + lr;                                          \
        const unsigned off_ = (ok_ && n_ < N) ? (unsigned)(((size_t)n_ * K + kk_) * 2) : NOWHERE; \
        wr[d][nt][i] = __builtin_bit_cast(bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, off_, 0, 0)); \
      }                                                                                        \
    _Pragma("unroll") for (int i = 0; i < MI; ++i) {                                           \
      const unsigned off_ = (ok_ && a_off[i] != NOWHERE) ? a_off[i] + (unsigned)(kk_ - lc * 8) * 2u : NOWHERE; \
      ar[d][i] = __builtin_bit_cast(bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, off_, 0, 0)); \
    }                                                                                          \
    ++l_q;                                                                                     \
    if (++l_step == n_steps_p) {                                                               \
      l_step = 0;                                                                              \
      l_n0 += stride_n;                                                                        \
    }                                                                                          \
  } while (0)

#pragma unroll
  for (int d = 0; d < DEPTH; ++d) RA_DEEP_LOAD(d);

  f32x4_t acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // rows of the A tiles that no load instruction covers stay zero
#pragma unroll
  for (int i = MI; i < MZ; ++i) *(bf16x8_t*)(my + NT * TILE + (i * RPI + lr) * PITCH + lc * 8) = zero;

  int c_step = 0, c_n0 = (int)blockIdx.x * 16 * NT;                 // where the products are
  for (int base = 0; base < total; base += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < NI; ++i)
          *(bf16x8_t*)(my + nt * TILE + (i * RPI + lr) * PITCH + lc * 8) = wr[d][nt][i];
#pragma unroll
      for (int i = 0; i < MI; ++i)
        *(bf16x8_t*)(my + NT * TILE + (i * RPI + lr) * PITCH + lc * 8) = ar[d][i];
      // the tile is the wave's own: its LDS operations complete in order
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      RA_DEEP_LOAD(d);
      bf16x8_t a[NT][U], b[MT][U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) a[nt][u] = *(const bf16x8_t*)(my + nt * TILE + r * PITCH + u * 32 + g * 8);
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
    c_step += DEPTH;
    if (c_step < n_steps_p) continue;
    // a tile is complete
    if (base < n_steps_p) {
      // What was asked for ahead is first touched here: an empty volatile statement per value keeps the
      // compiler from moving arithmetic on it (and with it the wait for it) up in front of the walk.
      if (EPI == EPI_ACCUM && pre.have_c) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) asm volatile("" : "+v"(pre.c[nt][mt][i]));
            asm volatile("" : "+v"(pre.w[nt][i]));
          }
      }
      if (nf.in_ss) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int j = 0; j < SS_HELD; ++j) {
            asm volatile("" : "+v"(ss_held[mt][j]));
            if (!(mt * 16 + r < M && wave * 4 + g + j * WAVES * 4 < nf.in_parts)) ss_held[mt][j] = 0.f;
          }
      }
    } else {
      pre.have_c = pre.have_w = false;      // only the first tile's values were asked for ahead
    }
    skinny_finish<MT, NT, WAVES, EPI, TO>(acc, ss_held, pre, red, row_ss, bias, C, ldc, M, N, c_n0, nf);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    c_step = 0;
    c_n0 += stride_n;
  }
#undef RA_DEEP_LOAD
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

static int skinny_cus() { return ra_cu_count(); }

template <int NT, int WAVES, int U, int DEPTH, int OCC, int MROWS>
static int launch_deep(const void* A, int lda, const void* W, const void* bias, void* C, int ldc, int out_dtype,
                       int epilogue, int M, int N, int K, const SkinnyNorm& nf, int grid, hipStream_t stream) {
#define RA_GO(EPI, TO)                                                                              \
  gemm_skinny_deep_kernel<NT, WAVES, U, DEPTH, OCC, MROWS, EPI, TO><<<grid, WAVES * RA_WAVE, 0, stream>>>(  \
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

// Up to 16 rows. All workgroups of a launch run side by side: two a CU, eight waves each with two runs
// in flight, each workgroup taking every grid-th tile of 16 features. (Measured on the Qwen3-8B shape's
// products at 1, 8 and 16 rows against four runs in flight with one workgroup a CU, four waves a
// workgroup with four workgroups a CU, and sixteen waves: within 3 % of each other, this one ahead.)
template <int MROWS>
static int launch_deep_rows(const void* A, int lda, const void* W, const void* bias, void* C, int ldc, int out_dtype,
                            int epilogue, int M, int N, int K, const SkinnyNorm& nf, hipStream_t stream) {
  const int n_tiles = (N + 15) / 16, cus = skinny_cus();
  const int grid = n_tiles < 2 * cus ? n_tiles : 2 * cus;
  // a wave's runs are 128 k long, or 64 where that splits K more evenly over the eight waves (2560 = 2.5
  // x 1024 would leave half of the waves idle in every tile's last run)
  const int runs128 = (K + 1023) / 1024, runs64 = (K + 511) / 512;
  if (runs64 * 512 < runs128 * 1024)
    return launch_deep<1, 8, 2, 2, 2, MROWS>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, grid, stream);
  return launch_deep<1, 8, 4, 2, 2, MROWS>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, grid, stream);
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
    RA_CHECK(out_x && out_ss && out_w, "gemm_skinny: emitting needs the norm weight, the scaled copy and the partial sums");
    RA_CHECK(out_w_dtype == RA_BF16 || out_w_dtype == RA_F32, "gemm_skinny: unknown norm weight dtype tag %d", out_w_dtype);
    RA_CHECK(out_ldx >= N, "gemm_skinny: the scaled copy's row stride (%d) is below %d", out_ldx, N);
    nf.out_w = out_w;
    nf.out_w_f32 = out_w_dtype == RA_F32;
    nf.out_x = (bf16_t*)out_x;
    nf.out_ldx = out_ldx;
    nf.out_ss = out_ss;
  }
  // the kernel for up to 16 rows reads through buffer descriptors, whose offsets are 32 bits
  const bool small = (size_t)N * K * 2 < 0xFFFFFF00ull && ((size_t)(M - 1) * lda + K) * 2 < 0xFFFFFF00ull;
  if (M <= 4 && small) return launch_deep_rows<4>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, stream);
  if (M <= 8 && small) return launch_deep_rows<8>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, stream);
  if (M <= 16 && small) return launch_deep_rows<16>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, stream);
  if (M <= 16) return launch_skinny<1, 1, 8, 4>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, stream);
  if (small && skinny_features(M, N) == 16) {
    // 17..64 rows, 16 features a workgroup: one workgroup a CU, runs of 64 k
    const int n_tiles = (N + 15) / 16, cus = skinny_cus();
    const int grid = n_tiles < cus ? n_tiles : cus;
    if (M <= 32) return launch_deep<1, 8, 2, 2, 1, 32>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, grid, stream);
    if (M <= 48) return launch_deep<1, 8, 2, 2, 1, 48>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, grid, stream);
    return launch_deep<1, 8, 2, 2, 1, 64>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, nf, grid, stream);
  }
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
