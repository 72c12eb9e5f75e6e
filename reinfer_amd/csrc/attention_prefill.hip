// Paged flash attention for prompt portions, bfloat16, on the matrix cores.
//
// A workgroup (8 waves, two a SIMD) takes one tile of consecutive query tokens of
// one request and HG query heads that share a KV head: 8 * NC column tiles of
// 16 columns, tile c = run c / HG of 16 queries, head c % HG; a wave owns NC
// adjacent column tiles, so every key and value it reads from LDS feeds NC
// MFMAs and all waves share one staged copy. Keys and values come from the
// request's block table, earlier context and the portion's own tokens alike
// (they were stored before this kernel runs), 64 keys a round, copied to LDS
// tile by tile of 16 slots in the cache's MFMA operand order (cache_k_index /
// cache_v_index; V with the two tiles of a 32-key half interleaved in runs of 8
// bytes), so every operand read from LDS is one contiguous 16-byte run a lane with
// no bank conflict. Tiles are fetched into registers two rounds ahead and staged
// into one of two LDS buffers, one barrier a round.
//
//   S^T[key][column] = K . Q^T        v_mfma_f32_16x16x32_bf16, contraction over d
//   online softmax per column (float; running maximum, sum), once per 32 keys
//   O^T[d][column]  += V^T . P        contraction over 32 keys; the probabilities
//                                     are the MFMA's second operand straight from
//                                     the score registers (two score tiles packed)
//
// The parts of a round run one after the other in a wave, and the two waves of a
// SIMD overlap little (timed with parts left out); what a wave's own instruction
// stream alternates overlaps: a column tile's output products with the next
// tile's exponentials.
//
// Causal: a query at position p sees keys <= p (and > p - window if a window is
// set). The reference's prompt attention is a vendored library kernel that sees
// only the prompt itself, from position 0 (crates/cuda/src/fmha.rs:574-686;
// crates/cuda/kernels/fmha_kernels.cu:96); this one is written here and reads
// earlier context from the cache, so a prompt can be cut anywhere.
#include <type_traits>
#include "common.h"
#include "reinfer_hip.h"

#define FP_THREADS 512
#define FP_WAVES 8
#define FP_KT 64          // keys per round

__device__ __forceinline__ float fp_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// how the heads of a group and the queries are spread over a wave's column tiles
struct FpShape {
  int nc;      // column tiles a wave holds (template parameter)
  int hg;      // heads of one KV head per workgroup: 4, 2 or 1
  int runs;    // runs of 16 queries per workgroup
};
static FpShape fp_shape(int Hq, int Hkv, int d) {
  FpShape s;
  const int G = Hq / Hkv;
  s.nc = d <= 128 ? 2 : 1;
  s.hg = (G % 4 == 0) ? 4 : (G % 2 == 0) ? 2 : 1;
  s.runs = FP_WAVES * s.nc / s.hg;
  return s;
}

// A listed tile may be one of several parts of a query tile, each with a range of keys (split.ranges, three
// ints a listed tile: first key, one past the last, both multiples of the round; and the part's slot, or -1
// for a tile that is whole): a part leaves its float sums (the outputs before the division, the running
// maximum and the sum of each column) in its slot, and a second kernel adds a tile's parts up. A portion
// of few queries deep in a long prompt is a handful of tiles with thousands of keys each, and a 2048-token
// prompt is one tile a CU of which the last has 32 times the keys of the first: cut by keys, the heavy
// tiles spread over the CUs that would idle.
struct FpSplit {
  const int* ranges;       // [listed tiles][3], or null: every tile is whole
  float* part_o;           // [slots][workgroups a tile][256 columns][DMAX]
  float* part_ml;          // [slots][workgroups a tile][256 columns][2]
};

// EXACT: the head size is DMAX itself, so every test against it is decided when the kernel is compiled
template <int DMAX, int NC, bool EXACT>
__global__ void __launch_bounds__(FP_THREADS)
flash_prefill_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                     const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
                     const int* __restrict__ block_tables, int max_blocks,
                     const int* __restrict__ tile_info,      // per tile: seq, first token row, n queries, first position
                     int block_size, int Hq, int Hkv, int d_arg, int HG, float scale_log2, int window,
                     FpSplit sp) {
  const int d = EXACT ? DMAX : d_arg;
  constexpr int NDT = DMAX / 32;       // 32-wide d tiles of the score product
  constexpr int NOT = DMAX / 16;       // 16-row d tiles of the output
  constexpr int NPRE = (FP_KT * DMAX / 8) / FP_THREADS;     // 16-byte chunks a thread fetches per operand
  __shared__ __attribute__((aligned(16))) bf16_t Ks2[2][FP_KT * DMAX];   // two rounds of 4 tiles of 16 * d
  __shared__ __attribute__((aligned(16))) bf16_t Vs2[2][FP_KT * DMAX];

  const int tid = threadIdx.x;
  const int lane = tid & (RA_WAVE - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / RA_WAVE);      // scalar: tests on it are branches
  const int r = lane & 15, g = lane >> 4;
  const int G = Hq / Hkv;
  const int n_hgrp = G / HG;
  // Workgroups go round the chip's XCDs, each with an L2 of its own, in the order of their numbers: the
  // (KV head, head group) is the fast index, so that with 8 of them all query tiles of one KV head run on
  // one XCD and its keys and values fill one L2 instead of all of them. Later tiles see more keys: they
  // start first.
  const int gy = Hkv * n_hgrp;
  const int by = blockIdx.x % gy;
  const int tile = gridDim.x / gy - 1 - blockIdx.x / gy;
  const int kvh = by / n_hgrp, hgrp = by % n_hgrp;
  const int seq = tile_info[tile * 4 + 0];
  const int row0 = tile_info[tile * 4 + 1];
  // n queries in the low half; above it, optionally, which of a wave's NC column tiles this workgroup
  // computes (bit j; 0 = all): a tile with many keys can be given to two workgroups, each with half of
  // the heads, so that a launch of about as many tiles as the chip has CUs does not last as long as its
  // heaviest tile while the CUs of the light ones idle.
  const int nq_word = tile_info[tile * 4 + 2];
  const int nq = nq_word & 0xffff;
  const int col_bits = (nq_word >> 16) & ((1 << NC) - 1);
  const int col_mask = col_bits ? col_bits : (1 << NC) - 1;
  const int pos0 = tile_info[tile * 4 + 3];
  const int* table = block_tables + (size_t)seq * max_blocks;

  // column tile c = wave * NC + j: queries (c / HG) * 16 + r, head hgrp * HG + c % HG
  int qi[NC];
  bool q_live[NC];
  bf16x8_t qreg[NC][NDT];
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    const int c = wave * NC + j;
    qi[j] = (c / HG) * 16 + r;
    q_live[j] = qi[j] < nq && ((col_mask >> j) & 1);
    const int head = kvh * G + hgrp * HG + c % HG;
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
    m[j] = q_live[j] ? -INFINITY : 0.f;      // a column without a query adds zeros and never asks for a new maximum
    l[j] = 0.f;
#pragma unroll
    for (int i = 0; i < NOT; ++i) acc[j][i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  }

  // keys this tile of queries can see, and this wave's share of them
  const int last_pos = pos0 + nq - 1;
  const int first_key = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  int kt_begin = first_key / FP_KT * FP_KT;
  int k_stop = last_pos;                      // the last key of this workgroup's rounds
  int slot = -1;
  if (sp.ranges) {
    kt_begin = max(kt_begin, sp.ranges[tile * 3 + 0]);
    k_stop = min(k_stop, sp.ranges[tile * 3 + 1] - 1);
    slot = sp.ranges[tile * 3 + 2];
  }
  const int w_q0 = (wave * NC / HG) * 16;                       // first query of the wave
  const int w_qend = ((wave * NC + NC - 1) / HG + 1) * 16;      // one past its last
  const int w_first_pos = pos0 + w_q0;
  const int w_last_pos = pos0 + min(w_qend, nq) - 1;            // < w_first_pos if the wave has no query

  // fetch of one round into registers: the four 16-slot tiles of K and of V, 16 bytes a thread and
  // step; tile tt_u of step u is the same for a whole wave, so its block id is a scalar load
  constexpr int TCH = 2 * DMAX;                  // 16-byte chunks of a tile, padded to the template's head size
  const int bs_shift = __builtin_ctz(block_size);      // block sizes are powers of two here
  // A fetch only issues loads, the same number every call whatever lies in range (a tile outside the
  // visible keys reads the first visible tile instead); stage() zeroes what must not be seen as it copies
  // the registers to LDS.
  struct Fetched {
    bf16x8_t kpre[NPRE], vpre[NPRE];
  };
  const int safe_kt = first_key & ~15;
  // Which of the round's four tiles a thread fetches in step u: with two steps or more, neighbouring tiles (the
  // two of a 32-key half), so that it holds both halves of every 16-byte piece of V's interleaved order and
  // writes it whole (8-byte stores 32 bytes apart fall on a quarter of the LDS banks: measured, 23 % of the
  // LDS's busy cycles were bank conflicts of those stores).
  const int tile_group = __builtin_amdgcn_readfirstlane(tid / TCH);
  auto tile_of = [&](int u) -> int { return NPRE >= 2 ? tile_group * NPRE + u : (tid + u * FP_THREADS) / TCH; };
  const int w = tid % TCH;                         // the thread's 16-byte chunk of each of its tiles
  auto fetch = [&](Fetched& F, int k0) {
#pragma unroll
    for (int u = 0; u < NPRE; ++u) {
      const int tt = __builtin_amdgcn_readfirstlane(tile_of(u));
      const int kt = k0 + tt * 16;
      const bool live = kt <= k_stop && kt + 15 >= first_key;           // wave-uniform
      const int ktl = live ? kt : safe_kt;
      const int blk = table[ktl >> bs_shift];
      const size_t tile_at = (((size_t)blk * Hkv + kvh) << bs_shift) * d + (size_t)((ktl & (block_size - 1)) >> 4) * 16 * d;
      const int wl = w < 2 * d ? w : 0;
      F.kpre[u] = *(const bf16x8_t*)(kcache + tile_at + wl * 8);
      F.vpre[u] = *(const bf16x8_t*)(vcache + tile_at + wl * 8);
    }
  };
  auto stage = [&](const Fetched& F, int k0, int buf) {
    bf16x8_t vkeep = {0, 0, 0, 0, 0, 0, 0, 0};      // the even tile's values, until the odd tile's are there
#pragma unroll
    for (int u = 0; u < NPRE; ++u) {
      const int tt = tile_of(u);
      const int kt = k0 + tt * 16;
      const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
      bf16x8_t kv = F.kpre[u], vv = F.vpre[u];
      if (!(kt <= last_pos && kt + 15 >= first_key)) {
        kv = zero;
        vv = zero;
      } else if (kt + 15 > last_pos || kt < first_key) {
        // slots of the tile outside the visible range may hold anything (a freed block's bits): zero them
        const int kkey = kt + (w & 15);                      // K chunk w: 8 elements of slot w % 16
        if (kkey > last_pos || kkey < first_key) kv = zero;
#pragma unroll
        for (int e = 0; e < 8; ++e) {                        // V chunk w: slots 4 ((w / 8) % 4) + e % 4
          const int vkey = kt + ((w >> 3) & 3) * 4 + (e & 3);
          if (vkey > last_pos || vkey < first_key) vv[e] = (bf16_t)0.f;
        }
      }
      if (w < 2 * d) {
        *(bf16x8_t*)(Ks2[buf] + (tt * 2 * d + w) * 8) = kv;
        // V: the two tiles of a half interleaved in runs of 8 bytes, so that an operand of the output
        // product (4 slots of the first tile, 4 of the second) is one 16-byte read
        bf16_t* vd = Vs2[buf] + ((tt >> 1) * 4 * d + 2 * w) * 8;
        if constexpr (NPRE >= 2) {
          if (u & 1) {
            *(bf16x8_t*)(vd) = (bf16x8_t){vkeep[0], vkeep[1], vkeep[2], vkeep[3], vv[0], vv[1], vv[2], vv[3]};
            *(bf16x8_t*)(vd + 8) = (bf16x8_t){vkeep[4], vkeep[5], vkeep[6], vkeep[7], vv[4], vv[5], vv[6], vv[7]};
          } else {
            vkeep = vv;
          }
        } else {
          *(bf16x4_t*)(vd + (tt & 1) * 4) = (bf16x4_t){vv[0], vv[1], vv[2], vv[3]};
          *(bf16x4_t*)(vd + (tt & 1) * 4 + 8) = (bf16x4_t){vv[4], vv[5], vv[6], vv[7]};
        }
      }
    }
  };

  // one round of 64 keys from LDS buffer `buf`
  auto compute = [&](int k0, int buf) {
    const bf16_t* Ks = Ks2[buf];
    const bf16_t* Vs = Vs2[buf];
    // a wave whose queries all lie before this round, or that has none, has nothing to add
    if (w_last_pos < w_first_pos || w_last_pos < k0) return;
    if (window > 0 && k0 + FP_KT - 1 < w_first_pos - window + 1) return;

    // two halves of 32 keys, each: scores, online softmax, values
#pragma unroll
    for (int kp = 0; kp < 2; ++kp) {
      const int kh = k0 + kp * 32;
      if (kh > w_last_pos) break;          // the second half may lie past the wave's last query
      // All LDS operands of the half are asked for at once, before the first matrix product: K for
      // the scores and V for the output, which does not depend on the softmax in between (left to
      // itself the compiler reads one operand, waits for it, multiplies, and so on: sixteen exposed
      // LDS latencies a half; asking first made the kernel 12 % faster). Head sizes above 128 have
      // no registers for that and read as they go.
      constexpr bool AHEAD = DMAX <= 128;
      const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
      auto k_operand = [&](int ks, int dt) -> bf16x8_t {
        const int e = dt * 32 + g * 8;
        return (e < d) ? *(const bf16x8_t*)(Ks + (kp * 2 + ks) * 16 * d + ((dt * 4 + g) * 16 + r) * 8) : zero8;
      };
      auto v_operand = [&](int ot) -> bf16x8_t {
        return (ot * 16 < d) ? *(const bf16x8_t*)(Vs + (kp * 4 * d + (ot * 4 + g) * 16 + r) * 8) : zero8;
      };
      bf16x8_t ka[AHEAD ? 2 : 1][AHEAD ? NDT : 1];
      bf16x8_t va[AHEAD ? NOT : 1];
      if constexpr (AHEAD) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
          for (int dt = 0; dt < NDT; ++dt) ka[ks][dt] = k_operand(ks, dt);
#pragma unroll
        for (int ot = 0; ot < NOT; ++ot) va[ot] = v_operand(ot);
        __builtin_amdgcn_sched_barrier(0);     // the reads stay ahead of the products
      }
      // scores S^T[key][column] for 2 sub-tiles of 16 keys, of the column tiles jlo .. jhi - 1
      f32x4_t s[2][NC];
      auto scores = [&](auto jlo_c, auto jhi_c) {
        constexpr int jlo = decltype(jlo_c)::value, jhi = decltype(jhi_c)::value;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
          for (int j = 0; j < NC; ++j) s[ks][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int dt = 0; dt < NDT; ++dt) {
            if (dt * 32 < d) {
              bf16x8_t a;
              if constexpr (AHEAD) a = ka[ks][dt];
              else a = k_operand(ks, dt);
#pragma unroll
              for (int j = jlo; j < jhi; ++j)
                s[ks][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qreg[j][dt], s[ks][j], 0, 0, 0);
            }
          }
        }
      };
      using I0 = std::integral_constant<int, 0>;
      using I1 = std::integral_constant<int, 1>;
      using IN = std::integral_constant<int, NC>;
      if (NC == 1 || col_mask == (1 << NC) - 1) scores(I0{}, IN{});
      else if (col_mask == 1) scores(I0{}, I1{});
      else scores(I1{}, IN{});
      // keys strictly inside every query's view need no mask
      const bool inner = kh + 31 <= w_first_pos && w_qend <= nq &&
                         (window <= 0 || kh >= w_last_pos - window + 1);
      if (!inner) {
#pragma unroll
        for (int j = 0; j < NC; ++j) {
          const int q_pos = pos0 + qi[j];
          const int q_lo = (window > 0 && q_pos - window + 1 > 0) ? q_pos - window + 1 : 0;
#pragma unroll
          for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int key = kh + ks * 16 + 4 * g + i;
              if (!(q_live[j] && key <= q_pos && key >= q_lo)) s[ks][j][i] = -INFINITY;
            }
        }
      }
      // Column tile by column tile: probabilities, then at once the tile's output products, so that the
      // matrix core works on them while the next tile's probabilities are computed.
#pragma unroll
      for (int j = 0; j < NC; ++j) {
        if (!((col_mask >> j) & 1)) continue;            // the other workgroup's column tile
        // Probabilities against the running maximum m first; m follows the true maximum only when
        // some probability comes out above 2^8 (the true maximum has grown by more than 8 in the
        // exponent): until then float sums and bfloat16 operands hold the larger values as well, and
        // the accumulators need no rescaling. A lane tests the 8 values it holds itself; the exchange
        // between lanes that finds a column's maximum is left to the rare branch, which the wave
        // takes as a whole, for every column: it rescales and computes the probabilities again. A
        // column that has seen no key yet (m = -inf) always takes it, so m never stays unset while
        // keys are visible.
        float p[8];
        auto probabilities = [&]() {
          const float base = (m[j] == -INFINITY) ? 0.f : m[j];
#pragma unroll
          for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              p[ks * 4 + i] = fp_exp2(fmaf(s[ks][j][i], scale_log2, -base));      // masked: exp2(-inf) = 0
        };
        probabilities();
        // the lane's sum stands for its largest value: no probability is above 2^8 unless the sum is (it is
        // needed anyway; a sum above 2^8 of smaller values only rescales a round early)
        float big = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) big += p[e];
        if (__any(!(big <= 256.f) || m[j] == -INFINITY)) {           // an overflowed or undefined value counts as large
          float tmax = fmaxf(fmaxf(fmaxf(s[0][j][0], s[0][j][1]), fmaxf(s[0][j][2], s[0][j][3])),
                             fmaxf(fmaxf(s[1][j][0], s[1][j][1]), fmaxf(s[1][j][2], s[1][j][3])));
          tmax = fmaxf(tmax, __shfl_xor(tmax, 16, RA_WAVE));
          tmax = fmaxf(tmax, __shfl_xor(tmax, 32, RA_WAVE)) * scale_log2;    // the scale is positive
          const float mn = fmaxf(m[j], tmax);
          // a column with nothing visible so far keeps m = -inf and adds zeros
          const float corr = (mn == -INFINITY) ? 1.f : fp_exp2(m[j] - mn);
          l[j] *= corr;
          m[j] = mn;
#pragma unroll
          for (int ot = 0; ot < NOT; ++ot)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[j][ot][i] *= corr;
          probabilities();
          big = 0.f;
#pragma unroll
          for (int e = 0; e < 8; ++e) big += p[e];
        }
        bf16x8_t pb;
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[e] = from_f32<bf16_t>(p[e]);
        l[j] += big;                                     // the lane's sum, of the second set where one was computed
        // O^T[d][column] += V^T[d][key] P[key][column], 32 keys per instruction:
        // k-slots (g, e): e < 4 -> key 4g + e of the first 16-key tile, e >= 4 -> of the second
#pragma unroll
        for (int ot = 0; ot < NOT; ++ot) {
          if (ot * 16 < d) {
            bf16x8_t a;
            if constexpr (AHEAD) a = va[ot];
            else a = v_operand(ot);
            acc[j][ot] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, acc[j][ot], 0, 0, 0);
          }
        }
        if (j + 1 < NC) {
          // one product, then three of the next tile's vector instructions, and so on: a wave issues
          // in order, so only alternating them lets the two kinds of work overlap
#pragma unroll
          for (int ot = 0; ot < NOT; ++ot) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     // MFMA
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);     // VALU
          }
        }
      }
    }
  };

  // Rounds alternate between two register sets and two LDS buffers; a set is fetched two rounds
  // ahead, right after it was staged. One barrier a round: it makes the staged tile whole, and a
  // wave that stages buffer b for round i has passed the barrier of round i - 1, which every wave
  // reaches only after its reads of round i - 2, the last user of buffer b.
  Fetched F0, F1;
  fetch(F0, kt_begin);
  __builtin_amdgcn_sched_barrier(0);
  fetch(F1, kt_begin + FP_KT);
  __builtin_amdgcn_sched_barrier(0);
  for (int k0 = kt_begin; k0 <= k_stop; k0 += 2 * FP_KT) {       // the bounds are the same in every thread
    stage(F0, k0, 0);
    __syncthreads();
    fetch(F0, k0 + 2 * FP_KT);
    compute(k0, 0);
    if (k0 + FP_KT > k_stop) break;
    stage(F1, k0 + FP_KT, 1);
    __syncthreads();
    fetch(F1, k0 + 3 * FP_KT);
    compute(k0 + FP_KT, 1);
  }
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    // the lane groups hold partial sums of l over their own keys
    float lt = l[j];
    lt += __shfl_xor(lt, 16, RA_WAVE);
    lt += __shfl_xor(lt, 32, RA_WAVE);
    if (slot >= 0) {
      // (a workgroup that was given some of a wave's column tiles only leaves the others' columns alone: two
      // workgroups with the halves of one part then fill one slot between them)
      if (!((col_mask >> j) & 1)) continue;
      // a part: the sums as they are, for the kernel that adds the parts (a column without a query, or one
      // that saw none of this part's keys, leaves zeros and -inf or 0 as its maximum: both weigh nothing)
      const size_t col = ((size_t)slot * gy + by) * (FP_WAVES * NC * 16) + (wave * NC + j) * 16 + r;
#pragma unroll
      for (int ot = 0; ot < NOT; ++ot)
        if (ot * 16 < d) *(f32x4_t*)(sp.part_o + col * DMAX + ot * 16 + 4 * g) = acc[j][ot];
      if (g == 0) {
        sp.part_ml[col * 2] = q_live[j] ? m[j] : -INFINITY;
        sp.part_ml[col * 2 + 1] = lt;
      }
      continue;
    }
    if (!q_live[j]) continue;
    const float inv = 1.f / lt;
    const int head = kvh * G + hgrp * HG + (wave * NC + j) % HG;
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

// The parts of one query tile added up, in part order: a wave takes one column (query, head) of one (tile,
// KV head, head group); everything it may read (the maxima and sums and the outputs of up to FPM_AHEAD parts)
// is asked for at once. merge_info, four ints a tile: first token row, queries, first slot, parts.
#define FPM_AHEAD 8
template <int DMAX>
__global__ void __launch_bounds__(256)
flash_prefill_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                           bf16_t* __restrict__ out, int out_stride, const int* __restrict__ merge_info,
                           int gy, int n_hgrp, int G, int HG, int d, int n_cols) {
  const int lane = threadIdx.x & (RA_WAVE - 1), wave = threadIdx.x / RA_WAVE;
  const int groups = n_cols / 4;                         // workgroups a (tile, KV head, head group): 4 columns each
  const int col = (blockIdx.x % groups) * 4 + wave;
  const int by = (blockIdx.x / groups) % gy, mt = blockIdx.x / groups / gy;
  const int kvh = by / n_hgrp, hgrp = by % n_hgrp;
  const int row0 = merge_info[mt * 4 + 0], nq = merge_info[mt * 4 + 1];
  const int slot0 = merge_info[mt * 4 + 2], n_parts = merge_info[mt * 4 + 3];
  constexpr int EPL = DMAX / RA_WAVE > 0 ? DMAX / RA_WAVE : 1;
  const int c = col / 16, r = col % 16;
  const int qi = (c / HG) * 16 + r;
  if (qi >= nq) return;
  const int head = kvh * G + hgrp * HG + c % HG;
  if (n_parts > FPM_AHEAD) {                             // many parts: one after the other
    float mx = -INFINITY;
    for (int p = 0; p < n_parts; ++p) mx = fmaxf(mx, part_ml[(((size_t)(slot0 + p) * gy + by) * n_cols + col) * 2]);
    float acc[EPL], lt = 0.f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[i] = 0.f;
    for (int p = 0; p < n_parts; ++p) {
      const size_t at = ((size_t)(slot0 + p) * gy + by) * n_cols + col;
      const float m1 = part_ml[at * 2];
      const float w = (m1 == -INFINITY) ? 0.f : fp_exp2(m1 - mx);
      lt += part_ml[at * 2 + 1] * w;
#pragma unroll
      for (int i = 0; i < EPL; ++i) {
        const int e = lane + i * RA_WAVE;
        if (e < d) acc[i] += part_o[at * DMAX + e] * w;
      }
    }
    const float inv = 1.f / lt;
    bf16_t* op = out + (size_t)(row0 + qi) * out_stride + (size_t)head * d;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int e = lane + i * RA_WAVE;
      if (e < d) op[e] = from_f32<bf16_t>(acc[i] * inv);
    }
    return;
  }
  float mp[FPM_AHEAD], lp[FPM_AHEAD], v[FPM_AHEAD][EPL];
#pragma unroll
  for (int p = 0; p < FPM_AHEAD; ++p) {                  // parts past the last are read again and weigh nothing
    const size_t at = ((size_t)(slot0 + min(p, n_parts - 1)) * gy + by) * n_cols + col;
    mp[p] = part_ml[at * 2];
    lp[p] = part_ml[at * 2 + 1];
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int e = lane + i * RA_WAVE;
      v[p][i] = part_o[at * DMAX + (e < d ? e : 0)];
    }
  }
  float mx = -INFINITY;
#pragma unroll
  for (int p = 0; p < FPM_AHEAD; ++p)
    if (p < n_parts) mx = fmaxf(mx, mp[p]);
  float acc[EPL], lt = 0.f;
#pragma unroll
  for (int i = 0; i < EPL; ++i) acc[i] = 0.f;
#pragma unroll
  for (int p = 0; p < FPM_AHEAD; ++p) {                  // part order: the same sum whatever ran first
    if (p >= n_parts) continue;
    const float w = (mp[p] == -INFINITY) ? 0.f : fp_exp2(mp[p] - mx);
    lt += lp[p] * w;
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[i] += v[p][i] * w;
  }
  const float inv = 1.f / lt;                            // every query sees at least its own key
  bf16_t* op = out + (size_t)(row0 + qi) * out_stride + (size_t)head * d;
#pragma unroll
  for (int i = 0; i < EPL; ++i) {
    const int e = lane + i * RA_WAVE;
    if (e < d) op[e] = from_f32<bf16_t>(acc[i] * inv);
  }
}

extern "C" int ra_attention_prefill_supports(int Hq, int Hkv, int d, int block_size) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return 0;
  return (d % 16 == 0 && d >= 16 && d <= 256 && block_size >= 16 && (block_size & (block_size - 1)) == 0) ? 1 : 0;
}

// queries per workgroup tile for these sizes
extern "C" int ra_attention_prefill_tile(int Hq, int Hkv, int d) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || d <= 0) return 64;
  return 16 * fp_shape(Hq, Hkv, d).runs;
}

// Column tiles a wave holds for these sizes (2: a tile's workgroup can be split in two by the high half of
// the tile's query count, see the kernel) and workgroups a query tile makes (KV heads x head groups).
extern "C" int ra_attention_prefill_columns(int Hq, int Hkv, int d) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || d <= 0) return 1;
  return fp_shape(Hq, Hkv, d).nc;
}
extern "C" int ra_attention_prefill_groups(int Hq, int Hkv, int d) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || d <= 0) return 1;
  return Hkv * ((Hq / Hkv) / fp_shape(Hq, Hkv, d).hg);
}

// Floats of part_o and part_ml that n_slots parts need (ra_attention_prefill_split)
extern "C" long ra_attention_prefill_part_floats(int Hq, int Hkv, int d, int n_slots, int which) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || d <= 0 || n_slots <= 0) return 0;
  const FpShape sh = fp_shape(Hq, Hkv, d);
  const long cols = (long)n_slots * Hkv * ((Hq / Hkv) / sh.hg) * FP_WAVES * sh.nc * 16;
  const int dmax = d <= 64 ? 64 : d <= 128 ? 128 : 256;
  return which == 0 ? cols * dmax : cols * 2;
}

static int fp_launch(const void* q, int q_stride, void* out, int out_stride,
                     const void* kcache, const void* vcache, const int* block_tables,
                     int max_blocks, const int* tile_info, int n_tiles, int block_size,
                     int Hq, int Hkv, int d, float scale, int window, const FpSplit& sp, const int* merge_info,
                     int n_merge, hipStream_t stream) {
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
  RA_CHECK((long)n_tiles * gy <= 0x7fffffffL, "attention_prefill: too many workgroups");
  dim3 grid(n_tiles * gy);
  const float scale_log2 = scale * 1.4426950408889634f;
#define RA_FP_GO(DM, NCC, EX)                                                                         \
  flash_prefill_kernel<DM, NCC, EX><<<grid, FP_THREADS, 0, stream>>>(                                 \
      (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kcache,                    \
      (const bf16_t*)vcache, block_tables, max_blocks, tile_info, block_size, Hq, Hkv, d, sh.hg,      \
      scale_log2, window, sp)
#define RA_FP(DM, NCC)                                                                                \
  do {                                                                                                \
    if (d == DM && DM <= 128) RA_FP_GO(DM, NCC, true); /* at 256 the exact form spills registers */   \
    else RA_FP_GO(DM, NCC, false);                                                                    \
  } while (0)
  if (d <= 64) RA_FP(64, 2);
  else if (d <= 128) RA_FP(128, 2);
  else RA_FP(256, 1);
#undef RA_FP_GO
#undef RA_FP
  RA_LAUNCH_CHECK("attention_prefill");
  if (n_merge > 0) {
    const int n_cols = FP_WAVES * sh.nc * 16;
    RA_CHECK((long)n_merge * gy * (n_cols / 4) <= 0x7fffffffL, "attention_prefill: too many tiles to add up");
#define RA_FPM(DM)                                                                                      \
  flash_prefill_merge_kernel<DM><<<n_merge * gy * (n_cols / 4), 256, 0, stream>>>(                      \
      sp.part_o, sp.part_ml, (bf16_t*)out, out_stride, merge_info, gy, G / sh.hg, G, sh.hg, d, n_cols)
    if (d <= 64) RA_FPM(64);
    else if (d <= 128) RA_FPM(128);
    else RA_FPM(256);
#undef RA_FPM
    RA_LAUNCH_CHECK("attention_prefill merge");
  }
  return 0;
}

extern "C" int ra_attention_prefill(const void* q, int q_stride, void* out, int out_stride,
                                    const void* kcache, const void* vcache, const int* block_tables,
                                    int max_blocks, const int* tile_info, int n_tiles, int block_size,
                                    int Hq, int Hkv, int d, float scale, int window, hipStream_t stream) {
  const FpSplit none = {};
  return fp_launch(q, q_stride, out, out_stride, kcache, vcache, block_tables, max_blocks, tile_info, n_tiles,
                   block_size, Hq, Hkv, d, scale, window, none, nullptr, 0, stream);
}

// The same with query tiles cut by keys: `ranges` holds three ints a listed tile (first key and one past the
// last, multiples of 64; the part's slot, or -1 for a whole tile), `merge_info` four a cut tile (first token
// row, queries, first slot, parts: its parts hold consecutive slots in key order); part_o and part_ml as
// ra_attention_prefill_part_floats() sizes them for the number of slots.
extern "C" int ra_attention_prefill_split(const void* q, int q_stride, void* out, int out_stride,
                                          const void* kcache, const void* vcache, const int* block_tables,
                                          int max_blocks, const int* tile_info, int n_tiles, const int* ranges,
                                          const int* merge_info, int n_merge, float* part_o, float* part_ml,
                                          int block_size, int Hq, int Hkv, int d, float scale, int window,
                                          hipStream_t stream) {
  RA_CHECK(ranges && merge_info && n_merge > 0 && part_o && part_ml,
           "attention_prefill_split: ranges, the list of cut tiles and the buffers for their parts are needed");
  RA_CHECK(((uintptr_t)part_o % 16) == 0, "attention_prefill_split: the parts' buffer must be 16-byte aligned");
  FpSplit sp = {};
  sp.ranges = ranges;
  sp.part_o = part_o;
  sp.part_ml = part_ml;
  return fp_launch(q, q_stride, out, out_stride, kcache, vcache, block_tables, max_blocks, tile_info, n_tiles,
                   block_size, Hq, Hkv, d, scale, window, sp, merge_info, n_merge, stream);
}
