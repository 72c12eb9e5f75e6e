// Weight-streaming product for up to 64 rows (the faster of the two from 17 rows on, and for wide gated
// products below that):  C[M,N] = A[M,K] . W[N,K]^T, bfloat16 in, float
// accumulation on the matrix cores.
//
// With more than one row tile the activations weigh as much as the weights: a workgroup that
// owns 16 features and splits K over its waves (gemm_skinny.hip) reads all of A, once a wave
// slice, and with its registers full of row tiles it keeps too few bytes in flight to cover the
// memory latency (measured at 64 rows: 3 TB/s). Here the eight waves of a workgroup split the
// features instead, 16 each, and walk K together: a run of 128 k of A is loaded once for the
// whole workgroup into LDS (two buffers, one barrier a run), every wave streams its own 16
// weight rows (contiguous 256-byte runs, re-laid through a tile of its own into MFMA layout),
// and loads run three runs ahead of the matrix cores (more was measured: no faster).
// A wave owns its 16 features over the
// workgroup's whole K range, so there is nothing to add between waves.
//
// Where N gives too few workgroups of 128 features to fill the chip, K is cut into S ranges
// (grid.y); each writes its float partial result and a second kernel adds them in range order
// and applies the epilogue: deterministic, no atomics. In that form only, the kernel also takes 65 to
// 128 rows (six or eight row tiles): a product over a long K that adds into the residual stream is
// faster so than the library's product followed by the add. Epilogues as in gemm_skinny.hip: plain
// (+ bias), SiLU gate over interleaved gate/up rows (S = 1 only), C += (float).
//
// An RMSNorm can ride on these products as on gemm_skinny's (y = rstd[m] * ((x .* w) . W^T)): the
// row factor is applied in the epilogue of whichever kernel finishes the product; the scaled copy
// and the partial sums of squares for the norm that follows an accumulating product are written by
// the adding kernel, which such a product then always runs: one partial sum per row and 1024 columns.
#include "common.h"
#include "reinfer_hip.h"

enum { WEPI_PLAIN = 0, WEPI_SILU_PAIRS = 1, WEPI_ACCUM = 2, WEPI_PARTIAL = 3 };

// RMSNorm carried by the product (all pointers may be null): see gemm_skinny.hip
struct WideNorm {
  const float* in_ss;      // [in_parts, M] partial sums of squares of the rows behind A
  int in_parts;
  float in_eps, in_inv_width;
  const void* out_w;       // [N] weight of the norm that follows (adding kernel only)
  int out_w_f32;
  bf16_t* out_x;           // [M, out_ldx] bf16(C_new * out_w)
  int out_ldx;
  float* out_ss;           // [ceil(N / 1024), M] sums of squares of C_new over 1024 columns
  float out_eps;           // >= 0 with out_ss null: the adding kernel finishes the norm, out_x = bf16(norm(C_new) * out_w)
};

#define GW_KS 128                      // k elements of a run
#define GW_PITCH (GW_KS + 8)           // LDS row pitch in elements: 16 bytes of padding
#ifndef GW_DEPTH
#define GW_DEPTH 3                      // runs in flight ahead of the matrix cores
#endif

// WV waves a workgroup (8 or 6: 128 or 96 features; the host picks what fills the chip evenly)
template <int MT, int WV>
struct GwRegs {
  bf16x8_t w[4];                                     // this wave's 16 weight rows x 128 k: 4 rows an instruction
  bf16x8_t a[(MT * 16 + WV * 4 - 1) / (WV * 4)];     // the workgroup's MT*16 rows x 128 k: 4 WV rows a pass
};

template <int MT, int WV, int EPI, typename TO>
__global__ void __launch_bounds__(WV * RA_WAVE)
gemm_wide_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W,
                 const bf16_t* __restrict__ bias, TO* __restrict__ C, int ldc, int M, int N, int K,
                 int k_per_split, WideNorm nf) {
  constexpr int RP = WV * 4;                     // rows of the A tile a pass of the whole workgroup loads
  constexpr int AP = (MT * 16 + RP - 1) / RP;
  constexpr int ATILE = (MT * 16 + 1) * GW_PITCH;   // one row more: where loads of rows past the tile are put
  constexpr int WTILE = 16 * GW_PITCH;
  __shared__ __attribute__((aligned(16))) bf16_t lds_a[2 * ATILE];
  __shared__ __attribute__((aligned(16))) bf16_t lds_w[WV * WTILE];

  const int tid = threadIdx.x;
  const int lane = tid & (RA_WAVE - 1), wave = tid / RA_WAVE;
  const int r = lane & 15, g = lane >> 4;        // MFMA operand layout
  const int lr = lane >> 4, lc = lane & 15;      // weight loads: 16 lanes a row, 4 rows an instruction
  const int ar = tid >> 4, ac = tid & 15;        // A loads: 16 threads a row, RP rows a pass
  const int n0 = (blockIdx.x * WV + wave) * 16;
  const int kb = blockIdx.y * k_per_split;
  const int ke = min(K, kb + k_per_split);
  const int n_runs = (ke - kb + GW_KS - 1) / GW_KS;
  bf16_t* my_w = lds_w + wave * WTILE;

  // Both operands are read through buffer descriptors: a load whose offset lies past the descriptor's
  // end returns zeros and touches no memory. Rows past N or M, chunks past the K range and the padding
  // runs are then loads like any other: no branch stands around a load, the waits count loads exactly,
  // and a run is used while the two behind it are still on their way. The weights' descriptor starts at
  // the workgroup's first row; both descriptors span less than 2 GiB, and an offset with its top bit set
  // is past their end whatever is added to it (made by arithmetic, not by a choice: the compiler turns a
  // choice between two offsets into a branch with a load in each arm).
  constexpr unsigned NOWHERE = 0x80000000u;
  const int nb = blockIdx.x * WV * 16;
  const int w_rows = min(N - nb, WV * 16);
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(W) + (size_t)nb * K, 0, (int)((size_t)w_rows * K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(A), 0, (int)(((size_t)(M - 1) * lda + K) * 2), 0x00020000);
  unsigned w_off[4], a_off[AP];                  // byte offset of this lane's chunk at k = 0, or NOWHERE
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = wave * 16 + i * 4 + lr;        // rows past the end are zeros; their results are dropped
    w_off[i] = n < w_rows ? (unsigned)(((size_t)n * K + lc * 8) * 2) : NOWHERE;
  }
#pragma unroll
  for (int ps = 0; ps < AP; ++ps) {
    const int m = ps * RP + ar;
    a_off[ps] = (m < M && m < MT * 16) ? (unsigned)(((size_t)m * lda + ac * 8) * 2) : NOWHERE;
  }

  // Workgroups start their walk over K at different runs (and wrap round): if all walked in step, the
  // rows read at one moment, a whole K apart from each other, would fall on few memory channels.
  const int rot = (int)((blockIdx.x * 7u + blockIdx.y * 3u) % (unsigned)n_runs);
  auto gload = [&](GwRegs<MT, WV>& R, int run) {
    // a padding run starts at the range's end: every chunk of it is out
    const int k = kb + (run < n_runs ? (run + rot < n_runs ? run + rot : run + rot - n_runs) * GW_KS : ke - kb);
    // K and the split are multiples of 8: a chunk is in or out as a whole; the top bit where it is out
    const unsigned w_out = (unsigned)((ke - 1 - (k + lc * 8)) >> 31) << 31;
    const unsigned a_out = (unsigned)((ke - 1 - (k + ac * 8)) >> 31) << 31;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned off = (w_off[i] + (unsigned)k * 2u) | w_out;
      R.w[i] = __builtin_bit_cast(bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, off, 0, 0));
    }
#pragma unroll
    for (int ps = 0; ps < AP; ++ps) {
      const unsigned off = (a_off[ps] + (unsigned)k * 2u) | a_out;
      R.a[ps] = __builtin_bit_cast(bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, off, 0, 0));
    }
  };

  f32x4_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  // one run: registers -> LDS, ask for the run GW_DEPTH ahead into the same registers, barrier, multiply
  auto step = [&](GwRegs<MT, WV>& R, int run) {
    bf16_t* abuf = lds_a + (run & 1) * ATILE;
#pragma unroll
    for (int i = 0; i < 4; ++i) *(bf16x8_t*)(my_w + (i * 4 + lr) * GW_PITCH + lc * 8) = R.w[i];
#pragma unroll
    for (int ps = 0; ps < AP; ++ps)      // no branch in the loop: the waits for loads stay exact
      *(bf16x8_t*)(abuf + min(ps * RP + ar, MT * 16) * GW_PITCH + ac * 8) = R.a[ps];
    gload(R, run + GW_DEPTH);
    // A buffer (run & 1) was last read in run - 2; every wave has passed the barrier of run - 1
    // since, so it is free. This barrier makes the tile whole before anyone reads it.
    __syncthreads();
#pragma unroll
    for (int u = 0; u < GW_KS / 32; ++u) {
      const bf16x8_t a = *(const bf16x8_t*)(my_w + r * GW_PITCH + u * 32 + g * 8);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8_t b = *(const bf16x8_t*)(abuf + (mt * 16 + r) * GW_PITCH + u * 32 + g * 8);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
      }
    }
    // the weight tile is the wave's own and is overwritten by the next run: its reads must be done
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  };

  GwRegs<MT, WV> R[GW_DEPTH];                       // indexed by constants only once unrolled: registers
#pragma unroll
  for (int d = 0; d < GW_DEPTH; ++d) {
    gload(R[d], d);
    // the runs are asked for in the order in which they are used (left alone, the scheduler asks for the
    // first run last, and the loop then waits for every load at its head)
    __builtin_amdgcn_sched_barrier(0);
  }
  // The carried norm's partial sums of row mt*16 + r: the waves and their lane groups share the parts out
  // (lane group g of wave w takes parts 4 w + g, 4 w + g + 4 WV, ...); the first GW_HELD of a lane are asked
  // for here, behind the first weights, and not touched before the loop is over, so that no wait for them
  // holds up the weight stream (a producer with 16 columns a workgroup leaves 256 of them for a width of
  // 4096: 8 a lane and row tile with eight waves); any further ones are read after the loop. The waves'
  // sums meet in LDS, in wave order.
  constexpr int GW_HELD = MT == 1 ? 16 : 8;
  constexpr int PSTEP = 4 * WV;
  __shared__ float row_ss[WV][MT * 16];
  const int p0 = 4 * wave + g;
  float held[MT][GW_HELD];
  if (EPI != WEPI_PARTIAL && nf.in_ss) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r < M ? mt * 16 + r : M - 1;       // clamped: no branch around the load
#pragma unroll
      for (int j = 0; j < GW_HELD; ++j) {
        const int p = p0 + PSTEP * j < nf.in_parts ? p0 + PSTEP * j : nf.in_parts - 1;
        held[mt][j] = nf.in_ss[(size_t)p * M + m];
      }
    }
  }
  // Whole groups of GW_DEPTH runs in the loop, the runs left over behind it: padding the range with runs of
  // zeros instead costs a short range half as much again (four runs became six), and a condition out here
  // costs the loop's waits nothing. The loads that a step asks for past the range's end are out as a whole.
  const int n_whole = n_runs / GW_DEPTH * GW_DEPTH;
  for (int run = 0; run < n_whole; run += GW_DEPTH) {  // the same in every thread of the workgroup
#pragma unroll
    for (int d = 0; d < GW_DEPTH; ++d) step(R[d], run + d);
  }
#pragma unroll
  for (int d = 0; d < GW_DEPTH - 1; ++d)
    if (n_whole + d < n_runs) step(R[d], n_whole + d);
  if (EPI != WEPI_PARTIAL && nf.in_ss) {
    // first touched here: an empty volatile statement per value keeps the compiler from moving
    // arithmetic on it, and with it the wait for it, up in front of the loop
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < GW_HELD; ++j) {
        asm volatile("" : "+v"(held[mt][j]));
        if (!(mt * 16 + r < M && p0 + PSTEP * j < nf.in_parts)) held[mt][j] = 0.f;
      }
    // a fixed order: a lane's parts ascending, the lane groups, then the waves
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
      float t = 0.f;
#pragma unroll
      for (int j = 0; j < GW_HELD; ++j) t += held[mt][j];
      if (m < M)
        for (int p = p0 + PSTEP * GW_HELD; p < nf.in_parts; p += PSTEP) t += nf.in_ss[(size_t)p * M + m];
      t += __shfl_xor(t, 16, RA_WAVE);
      t += __shfl_xor(t, 32, RA_WAVE);
      if (g == 0) row_ss[wave][mt * 16 + r] = t;
    }
    __syncthreads();
  }

  // lane (r, g) holds C[feature n0 + 4g + i][token mt*16 + r]
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r;
    if (EPI != WEPI_PARTIAL && nf.in_ss) {               // a split product is scaled when its parts are added
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < WV; ++w) t += row_ss[w][mt * 16 + r];
      const float rstd = rsqrtf(t * nf.in_inv_width + nf.in_eps);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[mt][i] *= rstd;
    }
    if (EPI == WEPI_PARTIAL) {
      if (m >= M) continue;
      float* P = (float*)C + ((size_t)blockIdx.y * M + m) * N;
      if ((N & 3) == 0 && n0 + 4 * g + 3 < N) {
        *(f32x4_t*)(P + n0 + 4 * g) = acc[mt];
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + 4 * g + i;
          if (n < N) P[n] = acc[mt][i];
        }
      }
    } else if (EPI == WEPI_ACCUM || EPI == WEPI_PLAIN) {
      if (m >= M) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 4 * g + i;
        if (n >= N) continue;
        float v = acc[mt][i];
        if (bias) v += to_f32(bias[n]);
        if (EPI == WEPI_ACCUM) v += to_f32(C[(size_t)m * ldc + n]);      // this thread alone owns (m, n)
        C[(size_t)m * ldc + n] = from_f32<TO>(v);
      }
    } else {
      // rows 0-7 of the wave's tile are gate, 8-15 up of the same features: the up value of
      // gate row 4g + i sits in lane (r, g + 2), same i
      float up[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) up[i] = __shfl_xor(acc[mt][i], 32, RA_WAVE);
      if (m >= M || g >= 2) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int f = (n0 / 16) * 8 + 4 * g + i;
        if (2 * f >= N) continue;              // N = 2 I
        const float gt = acc[mt][i];
        C[(size_t)m * ldc + f] = from_f32<TO>(gt / (1.f + __expf(-gt)) * up[i]);
      }
    }
  }
}

// C = epilogue(sum over s of P[s]) for the K ranges of a split product, in range order; a workgroup
// takes 1024 columns of one row. The carried norm's row factor and, for the norm that follows an
// accumulating product, the scaled copy and the workgroup's sum of squares are applied here.
template <int EPI, typename TO>
__global__ void __launch_bounds__(256)
gemm_wide_reduce_kernel(const float* __restrict__ P, int S, const bf16_t* __restrict__ bias,
                        TO* __restrict__ C, int ldc, int M, int N, WideNorm nf) {
  __shared__ float red[17];
  const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
  const int m = blockIdx.y;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (n < N) {
    const bool whole = n + 3 < N && (N & 3) == 0;
    if (whole) {
      // six ranges' values are asked for in one trip and then added in range order (one by one, the loop
      // made a trip a range)
      constexpr int U = 6;
      for (int s0 = 0; s0 < S; s0 += U) {
        f32x4_t t[U];
#pragma unroll
        for (int j = 0; j < U; ++j)
          t[j] = *(const f32x4_t*)(P + ((size_t)min(s0 + j, S - 1) * M + m) * N + n);
#pragma unroll
        for (int j = 0; j < U; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] += s0 + j < S ? t[j][i] : 0.f;
      }
    } else {
      for (int s = 0; s < S; ++s) {
        const float* p = P + ((size_t)s * M + m) * N + n;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) v[i] += p[i];
      }
    }
  }
  float rstd = 1.f;
  if (nf.in_ss) {                              // the same for every thread: the threads share the parts out
    float t = 0.f;
    for (int p = threadIdx.x; p < nf.in_parts; p += blockDim.x) t += nf.in_ss[(size_t)p * M + m];
    rstd = rsqrtf(block_sum(t, red) * nf.in_inv_width + nf.in_eps);
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (n + i >= N) continue;
    float x = v[i] * rstd;
    if (bias) x += to_f32(bias[n + i]);
    if (EPI == WEPI_ACCUM) x += to_f32(C[(size_t)m * ldc + n + i]);
    C[(size_t)m * ldc + n + i] = from_f32<TO>(x);
    if (EPI == WEPI_ACCUM && nf.out_x) {
      const float w = nf.out_w_f32 ? ((const float*)nf.out_w)[n + i] : to_f32(((const bf16_t*)nf.out_w)[n + i]);
      nf.out_x[(size_t)m * nf.out_ldx + n + i] = from_f32<bf16_t>(x * w);
      ss += x * x;
    }
  }
  if (EPI == WEPI_ACCUM && nf.out_x) {        // the same for every thread of the workgroup
    ss = block_sum(ss, red);
    if (threadIdx.x == 0) nf.out_ss[(size_t)blockIdx.x * M + m] = ss;
  }
}

// The same with a whole row a workgroup, which then also finishes the RMSNorm that follows an accumulating
// product: out_x = bf16(C_new * rsqrt(mean(C_new^2) + out_eps) * out_w). For the rows above those that the
// weight-streaming products take (65 to 128 requests decoding), where the products behind the norm are the
// library's and cannot apply a row factor: the norm then costs no kernel of its own. 1024 threads a row, each
// with CH chunks of 4 columns (N <= 4096 CH, N a multiple of 4): with few workgroups it is the loads in flight
// that count (256 threads with four chunks each, one after the other: 11 us against 7).
template <int CH>
__global__ void __launch_bounds__(1024)
gemm_wide_reduce_rows_kernel(const float* __restrict__ P, int S, const bf16_t* __restrict__ bias,
                             float* __restrict__ C, int ldc, int M, int N, WideNorm nf) {
  __shared__ float red[17];
  const int m = blockIdx.x;
  float rstd = 1.f;
  if (nf.in_ss) {                              // the same for every thread: the threads share the parts out
    float t = 0.f;
    for (int p = threadIdx.x; p < nf.in_parts; p += blockDim.x) t += nf.in_ss[(size_t)p * M + m];
    rstd = rsqrtf(block_sum(t, red) * nf.in_inv_width + nf.in_eps);
  }
  float x[CH][4];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int n = (c * 1024 + threadIdx.x) * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) x[c][i] = 0.f;
    if (n >= N) continue;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    constexpr int U = 6;                       // ranges asked for in one trip, added in range order
    for (int s0 = 0; s0 < S; s0 += U) {
      f32x4_t t[U];
#pragma unroll
      for (int j = 0; j < U; ++j) t[j] = *(const f32x4_t*)(P + ((size_t)min(s0 + j, S - 1) * M + m) * N + n);
#pragma unroll
      for (int j = 0; j < U; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] += s0 + j < S ? t[j][i] : 0.f;
    }
    const f32x4_t c0 = *(const f32x4_t*)(C + (size_t)m * ldc + n);
    f32x4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float y = v[i] * rstd;
      if (bias) y += to_f32(bias[n + i]);
      y += c0[i];
      o[i] = y;
      x[c][i] = y;
      ss += y * y;
    }
    *(f32x4_t*)(C + (size_t)m * ldc + n) = o;
  }
  const float rout = rsqrtf(block_sum(ss, red) / (float)N + nf.out_eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int n = (c * 1024 + threadIdx.x) * 4;
    if (n >= N) continue;
    bf16x4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float w = nf.out_w_f32 ? ((const float*)nf.out_w)[n + i] : to_f32(((const bf16_t*)nf.out_w)[n + i]);
      o[i] = from_f32<bf16_t>(x[c][i] * rout * w);
    }
    *(bf16x4_t*)(nf.out_x + (size_t)m * nf.out_ldx + n) = o;
  }
}

// How [M, N, K] is cut: waves a workgroup (5 to 8, 16 features each) and K ranges. With many features
// one range, and the workgroup width that fills the chip's 256 CUs most evenly (24576 features: 256
// workgroups of 96; 19456: 244 of 80; 51200: 458 of 112). With few features 128 a workgroup and as many K ranges as
// give one workgroup a CU or fewer, each range a multiple of the run.
static void gw_split(int epilogue, int M, int N, int K, int* waves, int* S, int* k_per_split, bool* partial = nullptr,
                     bool emits = false) {
  if (partial) *partial = emits;                       // the adding kernel writes what the next norm needs
  const int cus = ra_cu_count(), fill = cus - cus / 4;  // workgroups that keep the chip busy: three quarters of its CUs
  const int cb8 = (N + 127) / 128;
  *waves = 8;
  *S = 1;
  *k_per_split = (K + GW_KS - 1) / GW_KS * GW_KS;
  if ((cb8 >= fill && !emits) || epilogue == WEPI_SILU_PAIRS) {
    // The width whose workgroups fill whole rounds of the chip's CUs (256 on MI355X) best: 5 to 8 waves from 17 rows
    // on, 6 or 8 below (there the odd widths were slower inside a decode step although faster alone, and
    // a shape that neither 6 nor 8 fills well goes to gemm_skinny: ra_gemm_wide_preferred). A narrower
    // workgroup stages the activations more often, so it must fill the rounds clearly better (with many
    // rounds, as for a vocabulary, the widths differ little in that and the widest stays). Measured
    // inside decode steps, against 6 or 8 waves at every row count: 51200 x 5120 gated, 64 layers: -4 % a step
    // at 1 and 8 rows, -2 % at 64; 19456 x 2560, 36 layers: -1.7 % at 1 row, -1 % at 64.
    double best = -1.0;
    for (int wv = 8; wv >= 5; --wv) {
      if (M <= 16 && (wv == 7 || wv == 5)) continue;
      const int cb = (N + wv * 16 - 1) / (wv * 16);
      const double e = (double)cb / (((cb + cus - 1) / cus) * cus);
      if (e > best * 1.03) {
        best = e;
        *waves = wv;
      }
    }
    return;
  }
  // As many ranges as fill the chip's CUs once and no more: workgroups of a second, part-filled round last as
  // long as those of the first (64 rows, 10240 x 5120: 4 ranges, 320 workgroups, 34 us; 3 ranges, 240
  // workgroups, 26 us; 5120 x 25600: 8 ranges 77 us, 6 ranges 55 us). A range is four runs or more (shorter
  // ones are all start and end), and there are at most 12 (each is a float plane to write and read again).
  int s = cus / cb8;
  if (s > 12) s = 12;
  while (s > 1 && K / s < 4 * GW_KS) --s;
  if (s < 1) s = 1;
  int kps = (K + s - 1) / s;
  kps = (kps + GW_KS - 1) / GW_KS * GW_KS;
  *S = (K + kps - 1) / kps;
  *k_per_split = kps;
  if (partial) *partial = emits || *S > 1;
}

// 1 where this kernel beats ra_gemm_skinny (measured on MI355X at 4 to 64 rows): from 17 rows on,
// except a small product whose K has to be cut (4096 x 4096: the second launch costs more than the
// shared activations save); from 9 rows for the gated product of a wide feed-forward.
extern "C" int ra_gemm_wide_preferred(int epilogue, int M, int N, int K) {
  if (M < 1 || M > 128) return 0;
  int waves, S, kps;
  gw_split(epilogue, M, N, K, &waves, &S, &kps);
  // sizes are priced a CU: a product is "large" where every CU has more than 128 KiB of weights to stream
  // (on 256 CUs: more than 4096 x 4096 bfloat16)
  const int cus = ra_cu_count(), fill = cus - cus / 4;
  const bool large = (long)N * K * 2 > 131072L * cus;
  // 65 to 128 rows: the library's products are as fast or faster (151936 x 4096 at 128 rows: 285 us against
  // 400) but for a product that adds into the residual stream over a long K, which this kernel cuts into
  // ranges (4096 x 12288 at 96 / 128 rows: 37 / 43 us against 59 / 70 for the library's product and the add)
  // (and from exactly 128 KiB a CU on: 4096 x 4096 at 96 / 128 rows 19.7 / 22.0 us with the adding kernel, which
  // also does the add, against 17.2 / 19.3 for the library's product, whose result the norm kernel then adds)
  if (M > 64) return (epilogue == WEPI_ACCUM && S > 1 && (long)N * K * 2 >= 131072L * cus) ? 1 : 0;
  // from 9 to 16 rows the gated product of a wide feed-forward (up to 8 rows the other kernel, whose
  // workgroups stay and keep two runs a wave in flight, is ahead: 24576 x 4096 36 us against 37, 51200 x
  // 5120 91 to 97 against 101 to 103): one K range, enough workgroups to fill the
  // chip (measured at 16 rows, 24576 x 4096: 37 us against 41) and to fill whole rounds of it
  // (400 workgroups would leave a third of the CUs with half the work: the other kernel's many small
  // ones are then faster); and from 9 rows a plain product over a vocabulary (151936 features at 16 rows,
  // K = 2560 / 4096 / 5120: 148 / 237 / 280 us against 170 / 239 / 327)
  const int cb = (N + waves * 16 - 1) / (waves * 16);
  if (M < 17) {
    if (epilogue == WEPI_SILU_PAIRS)
      return (M > 8 && S == 1 && cb >= fill && cb * 10 >= ((cb + cus - 1) / cus) * cus * 8) ? 1 : 0;
    return (epilogue == WEPI_PLAIN && M > 8 && S == 1 && cb >= 3 * cus) ? 1 : 0;
  }
  return (S == 1 || large) ? 1 : 0;
}

// Floats of scratch that ra_gemm_wide needs for this product (0: none).
extern "C" long ra_gemm_wide_scratch(int epilogue, int M, int N, int K, int emits) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int waves, S, kps;
  bool partial;
  gw_split(epilogue, M, N, K, &waves, &S, &kps, &partial, emits != 0);
  return partial ? (long)S * M * N : 0;
}

// Partial sums a row that an emitting product writes for the norm that follows an [M, N] result.
extern "C" int ra_gemm_wide_row_parts(int N) { return (N + 1023) / 1024; }

// the second half of a product cut into K ranges: adds them in range order and applies the epilogue
static int launch_wide_reduce(const void* bias, void* C, int ldc, int out_dtype, int epilogue, int M, int N, int S,
                              const float* scratch, const WideNorm& nf, hipStream_t stream) {
  if (nf.out_x && !nf.out_ss) {                // a whole row a workgroup: the norm that follows is finished here
    if (N <= 4096) gemm_wide_reduce_rows_kernel<1><<<M, 1024, 0, stream>>>(scratch, S, (const bf16_t*)bias, (float*)C, ldc, M, N, nf);
    else if (N <= 8192) gemm_wide_reduce_rows_kernel<2><<<M, 1024, 0, stream>>>(scratch, S, (const bf16_t*)bias, (float*)C, ldc, M, N, nf);
    else gemm_wide_reduce_rows_kernel<4><<<M, 1024, 0, stream>>>(scratch, S, (const bf16_t*)bias, (float*)C, ldc, M, N, nf);
    RA_LAUNCH_CHECK("gemm_wide reduce rows");
    return 0;
  }
  const dim3 rg((N + 1023) / 1024, M);
#define RA_GR(EPI, TO) \
  gemm_wide_reduce_kernel<EPI, TO><<<rg, 256, 0, stream>>>(scratch, S, (const bf16_t*)bias, (TO*)C, ldc, M, N, nf)
  if (epilogue == WEPI_ACCUM) RA_GR(WEPI_ACCUM, float);
  else if (out_dtype == RA_BF16) RA_GR(WEPI_PLAIN, bf16_t);
  else RA_GR(WEPI_PLAIN, float);
#undef RA_GR
  RA_LAUNCH_CHECK("gemm_wide reduce");
  return 0;
}

// 65 to 128 rows: only as K ranges and the adding kernel (six or eight row tiles, workgroups of eight waves)
template <int MT>
static int launch_wide_ranges(const void* A, int lda, const void* W, const void* bias, void* C, int ldc, int out_dtype,
                              int epilogue, int M, int N, int K, int S, int kps, float* scratch, const WideNorm& nf,
                              hipStream_t stream) {
  RA_CHECK(((size_t)(M - 1) * lda + K) * 2 < 0x7FFFFF00ull && (size_t)128 * K * 2 < 0x7FFFFF00ull,
           "gemm_wide: rows of %d (stride %d) are too long for this kernel", K, lda);
  const WideNorm none = {};
  gemm_wide_kernel<MT, 8, WEPI_PARTIAL, float><<<dim3((N + 127) / 128, S), 8 * RA_WAVE, 0, stream>>>(
      (const bf16_t*)A, lda, (const bf16_t*)W, nullptr, scratch, N, M, N, K, kps, none);
  RA_LAUNCH_CHECK("gemm_wide");
  return launch_wide_reduce(bias, C, ldc, out_dtype, epilogue, M, N, S, scratch, nf, stream);
}

template <int MT, int WV>
static int launch_wide(const void* A, int lda, const void* W, const void* bias, void* C, int ldc, int out_dtype,
                       int epilogue, int M, int N, int K, int S, int kps, bool partial, float* scratch,
                       const WideNorm& nf, hipStream_t stream) {
  const dim3 grid((N + WV * 16 - 1) / (WV * 16), S);
  // the kernel reads through buffer descriptors that must span less than 2 GiB: the activations, and a
  // workgroup's 16 WV rows of weights
  RA_CHECK(((size_t)(M - 1) * lda + K) * 2 < 0x7FFFFF00ull && (size_t)WV * 16 * K * 2 < 0x7FFFFF00ull,
           "gemm_wide: rows of %d (stride %d) are too long for this kernel", K, lda);
#define RA_GW(EPI, TO, OUT, LD)                                                                 \
  gemm_wide_kernel<MT, WV, EPI, TO><<<grid, WV * RA_WAVE, 0, stream>>>(                         \
      (const bf16_t*)A, lda, (const bf16_t*)W, (const bf16_t*)bias, (TO*)(OUT), LD, M, N, K, kps, nf)
  if (partial) {
    RA_GW(WEPI_PARTIAL, float, scratch, N);
    RA_LAUNCH_CHECK("gemm_wide");
    return launch_wide_reduce(bias, C, ldc, out_dtype, epilogue, M, N, S, scratch, nf, stream);
  }
  if (epilogue == WEPI_SILU_PAIRS) {
    if (out_dtype == RA_BF16) RA_GW(WEPI_SILU_PAIRS, bf16_t, C, ldc);
    else RA_GW(WEPI_SILU_PAIRS, float, C, ldc);
  } else if (epilogue == WEPI_ACCUM) {
    RA_GW(WEPI_ACCUM, float, C, ldc);
  } else {
    if (out_dtype == RA_BF16) RA_GW(WEPI_PLAIN, bf16_t, C, ldc);
    else RA_GW(WEPI_PLAIN, float, C, ldc);
  }
#undef RA_GW
  RA_LAUNCH_CHECK("gemm_wide");
  return 0;
}

extern "C" int ra_gemm_wide_normed(const void* A, const void* W, const void* bias, void* C, int out_dtype,
                                   int epilogue, int M, int N, int K, int lda, int ldc, float* scratch,
                                   long scratch_floats, const float* in_ss, int in_parts, float in_eps,
                                   int in_width, const void* out_w, int out_w_dtype, void* out_x, int out_ldx,
                                   float* out_ss, float out_eps, hipStream_t stream) {
  RA_CHECK(M > 0 && N > 0 && K > 0, "gemm_wide: empty product (%d, %d, %d)", M, N, K);
  RA_CHECK(M <= 128, "gemm_wide: %d rows; this kernel takes at most 128", M);
  RA_CHECK(K % 8 == 0 && lda % 8 == 0, "gemm_wide: K (%d) and the row stride (%d) must be multiples of 8", K, lda);
  RA_CHECK(epilogue == WEPI_PLAIN || epilogue == WEPI_SILU_PAIRS || epilogue == WEPI_ACCUM,
           "gemm_wide: unknown epilogue %d", epilogue);
  RA_CHECK(epilogue != WEPI_ACCUM || out_dtype == RA_F32, "gemm_wide: accumulation is into a float matrix");
  const int n_out = epilogue == WEPI_SILU_PAIRS ? N / 2 : N;
  RA_CHECK(epilogue != WEPI_SILU_PAIRS || (N % 16 == 0 && bias == nullptr),
           "gemm_wide: the gated epilogue needs N (%d) in whole tiles of 16 and no bias", N);
  RA_CHECK(lda >= K && ldc >= n_out, "gemm_wide: row strides (%d, %d) below the row lengths (%d, %d)", lda, ldc, K, n_out);
  RA_CHECK(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_wide: operands must be 16-byte aligned");
  RA_CHECK(out_dtype == RA_BF16 || out_dtype == RA_F32, "gemm_wide: unknown output dtype tag %d", out_dtype);
  WideNorm nf = {};
  if (in_ss) {
    RA_CHECK(in_parts > 0 && in_width > 0 && in_eps >= 0.f, "gemm_wide: row sums need parts (%d), width (%d) and eps", in_parts, in_width);
    nf.in_ss = in_ss;
    nf.in_parts = in_parts;
    nf.in_eps = in_eps;
    nf.in_inv_width = 1.f / (float)in_width;
  }
  const bool emits = out_x || out_ss || out_w;
  const bool finishes = emits && !out_ss;      // the adding kernel finishes the norm that follows
  if (emits) {
    RA_CHECK(epilogue == WEPI_ACCUM, "gemm_wide: only the accumulating epilogue emits for a norm");
    RA_CHECK(out_x && out_w && (out_ss || out_eps >= 0.f),
             "gemm_wide: emitting needs the norm weight, the scaled copy and the partial sums (or, to finish the norm, its eps)");
    RA_CHECK(!finishes || (N % 4 == 0 && N <= 16384 && ldc % 4 == 0 && out_ldx % 4 == 0 && ((uintptr_t)C % 16) == 0 &&
                           ((uintptr_t)out_x % 8) == 0),
             "gemm_wide: finishing the norm takes rows of up to 16384 columns in steps of 4 (%d, strides %d and %d)", N, ldc, out_ldx);
    RA_CHECK(out_w_dtype == RA_BF16 || out_w_dtype == RA_F32, "gemm_wide: unknown norm weight dtype tag %d", out_w_dtype);
    RA_CHECK(out_ldx >= N, "gemm_wide: the scaled copy's row stride (%d) is below %d", out_ldx, N);
    nf.out_w = out_w;
    nf.out_w_f32 = out_w_dtype == RA_F32;
    nf.out_x = (bf16_t*)out_x;
    nf.out_ldx = out_ldx;
    nf.out_ss = out_ss;
    nf.out_eps = out_eps;
  }
  const long need = ra_gemm_wide_scratch(epilogue, M, N, K, emits);
  RA_CHECK(need == 0 || (scratch && scratch_floats >= need && ((uintptr_t)scratch % 16) == 0),
           "gemm_wide: this product needs %ld floats of scratch, got %ld", need, scratch_floats);
  int waves, S, kps;
  bool partial;
  gw_split(epilogue, M, N, K, &waves, &S, &kps, &partial, emits);
  if (M > 64) {
    RA_CHECK(partial && epilogue != WEPI_SILU_PAIRS,
             "gemm_wide: with %d rows only a product that is cut into K ranges (64 rows otherwise)", M);
    if (M <= 96) return launch_wide_ranges<6>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, S, kps, scratch, nf, stream);
    return launch_wide_ranges<8>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, S, kps, scratch, nf, stream);
  }
#define RA_GWW(MT, WV) launch_wide<MT, WV>(A, lda, W, bias, C, ldc, out_dtype, epilogue, M, N, K, S, kps, partial, scratch, nf, stream)
#define RA_GWL(MT) return waves == 5 ? RA_GWW(MT, 5) : waves == 6 ? RA_GWW(MT, 6) : waves == 7 ? RA_GWW(MT, 7) : RA_GWW(MT, 8)
  if (M <= 16) RA_GWL(1);
  if (M <= 32) RA_GWL(2);
  if (M <= 48) RA_GWL(3);
  RA_GWL(4);
#undef RA_GWL
#undef RA_GWW
}

// K ranges that ra_gemm_wide_partial cuts [M, N, K] into (its result has that many [M, N] float planes).
extern "C" int ra_gemm_wide_ranges(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  int waves, S, kps;
  bool partial;
  gw_split(WEPI_PLAIN, M, N, K, &waves, &S, &kps, &partial, true);
  return S;
}

// Only the first half of a split product: P[s][m][n] = A[m, range s] . W[n, range s]^T, float, for a
// consumer that adds the ranges itself (in range order) instead of the adding kernel.
extern "C" int ra_gemm_wide_partial(const void* A, const void* W, float* P, long p_floats, int M, int N, int K,
                                    int lda, hipStream_t stream) {
  RA_CHECK(M > 0 && N > 0 && K > 0, "gemm_wide: empty product (%d, %d, %d)", M, N, K);
  RA_CHECK(M <= 64, "gemm_wide: %d rows; this kernel takes at most 64", M);
  RA_CHECK(K % 8 == 0 && lda % 8 == 0 && lda >= K, "gemm_wide: K (%d) and the row stride (%d) must be multiples of 8", K, lda);
  RA_CHECK(((uintptr_t)A % 16) == 0 && ((uintptr_t)W % 16) == 0 && ((uintptr_t)P % 16) == 0,
           "gemm_wide: operands must be 16-byte aligned");
  int waves, S, kps;
  bool partial;
  gw_split(WEPI_PLAIN, M, N, K, &waves, &S, &kps, &partial, true);
  RA_CHECK(P && p_floats >= (long)S * M * N, "gemm_wide: %d ranges of [%d, %d] need %ld floats, got %ld", S, M, N,
           (long)S * M * N, p_floats);
  const WideNorm nf = {};
#define RA_GWP(MT, WV)                                                                                  \
  gemm_wide_kernel<MT, WV, WEPI_PARTIAL, float><<<dim3((N + WV * 16 - 1) / (WV * 16), S), WV * RA_WAVE, 0, stream>>>( \
      (const bf16_t*)A, lda, (const bf16_t*)W, nullptr, P, N, M, N, K, kps, nf)
#define RA_GWPM(MT) RA_GWP(MT, 8)          /* a product cut into K ranges has workgroups of 8 waves */
  if (M <= 16) RA_GWPM(1);
  else if (M <= 32) RA_GWPM(2);
  else if (M <= 48) RA_GWPM(3);
  else RA_GWPM(4);
#undef RA_GWPM
#undef RA_GWP
  RA_LAUNCH_CHECK("gemm_wide partial");
  return 0;
}

extern "C" int ra_gemm_wide(const void* A, const void* W, const void* bias, void* C, int out_dtype, int epilogue,
                            int M, int N, int K, int lda, int ldc, float* scratch, long scratch_floats,
                            hipStream_t stream) {
  return ra_gemm_wide_normed(A, W, bias, C, out_dtype, epilogue, M, N, K, lda, ldc, scratch, scratch_floats,
                             nullptr, 0, 0.f, 0, nullptr, 0, nullptr, 0, nullptr, -1.f, stream);
}
