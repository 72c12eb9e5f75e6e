// Flash-decode attention over the paged cache, bfloat16, on the matrix cores:
// one query token per (request, position); the query heads of one KV head are
// the columns of the MFMA tiles, so every key and value is read once for the
// whole group. The keys are cut into chunks; a workgroup (4 waves) takes one
// (chunk, KV head, token), its waves take 32 keys at a time:
//
//   S^T[key][head]  = K . Q^T          v_mfma_f32_16x16x32_bf16 over d
//   online softmax per head column     (float: running maximum and sum)
//   O^T[d][head]   += V^T . P          contraction over the 32 keys
//
// The cache keeps K and V in tiles of 16 slots laid out in MFMA operand order
// (cache_k_index / cache_v_index), so a wave's load of an operand is one
// contiguous run of 1 KB (K) or 512 bytes (V^T) and goes straight from memory
// into the matrix core's registers; the probabilities are the second
// product's operand as they leave the first (k-slot s of lane group g is key
// 4g + s of the first 16 keys for s < 4, of the second 16 for s >= 4, for both
// operands alike).
//
// The grid is a fixed number of workgroups, as many as the chip holds at once; every
// token has max_chunks items a KV head (those past its own number of chunks are
// empty) and workgroup w takes items w, w + grid, ...: launching one workgroup an
// item costs 13 to 20 ns each (a step of 64 requests has ten thousand) and leaves
// the last round of workgroups half empty. An item's token and chunk follow from
// its number, not from a table built from all tokens' positions first: in a
// launch that lasts some ten microseconds every trip to memory that another
// waits for shows (here: arguments, position and request, block ids, keys).
//
// Chunks of one (token, head) are merged by a second small kernel, always in
// chunk order. (Merging in the last workgroup to arrive needs device-wide
// release/acquire fences in every workgroup; on this chip each one writes back
// and invalidates a whole L2, which made the kernel nine times slower.) A token
// whose keys fit one chunk is written directly.
//
// The reference's flash decode keeps the whole score row in shared memory,
// which caps the context at (d + max_kv) * 4 <= 48 KB (crates/cuda/src/decode.rs:49-52;
// crates/cuda/kernels/decode_flash_kernels.cu:212-350), and takes one CTA per
// query head; the online form here has no such cap and shares K/V in a group.
#include "common.h"
#include "reinfer_hip.h"

// Waves a workgroup: 4 where the step has (token, KV head) pairs enough to fill the chip with small
// workgroups, 12 where it has few: a CU then has 192 KB of keys and values in flight for one work item,
// few chunks a token are enough to keep the memory busy, and a token with one chunk needs no merge.

__device__ __forceinline__ float fd_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// How one token's keys [lo, p] are cut: into at most max_chunks chunks of equal length, a whole number of
// the workgroup's rounds and at least chunk_min (a power of two; but for the rounding), from the 16-key tile that holds lo. Equal chunks of
// the token's own length, not of the longest context in the batch: no work item is a short remainder.
struct FdCut {
  int base;    // first key of chunk 0 (a multiple of 16)
  int chunk;   // keys of a chunk
  int n;       // chunks
};
// gran: keys a workgroup takes a round (its waves x 32); a chunk is a whole number of rounds
__device__ __forceinline__ FdCut fd_cut(int p, int lo, int chunk_shift, int max_chunks, int gran) {
  FdCut c;
  c.base = lo & ~15;
  const int span = p - c.base + 1;
  int want = (span + (1 << chunk_shift) - 1) >> chunk_shift;       // chunk_min = 1 << chunk_shift
  want = want < max_chunks ? want : max_chunks;
  c.chunk = ((span + want - 1) / want + gran - 1) / gran * gran;
  c.n = want;                                                      // fewer if the rounding up covers the keys sooner
  while ((c.n - 1) * c.chunk >= span) --c.n;
  return c;
}

// EXACT: the head size is DMAX itself, so every test against it is decided when the kernel is compiled
template <int DMAX, bool EXACT, int FD_WAVES>
__global__ void __launch_bounds__(FD_WAVES * RA_WAVE, (DMAX <= 128 && FD_WAVES == 4) ? 3 : 1)
flash_decode_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                    const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
                    const int* __restrict__ block_tables, int max_blocks,
                    const int* __restrict__ token_list, const int* __restrict__ seq_of_token,
                    const int* __restrict__ positions, int block_size, int Hkv, int G, int d_arg,
                    float scale_log2, int window, int chunk_shift, int max_chunks, int n_tokens,
                    int t_base, float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int FD_THREADS = FD_WAVES * RA_WAVE;
  const int d = EXACT ? DMAX : d_arg;
  constexpr int NDT = DMAX / 32;       // 32-wide d tiles of the score product
  constexpr int NOT = DMAX / 16;       // 16-row d tiles of the output
  extern __shared__ float lds[];       // [waves][G][d] outputs, then [waves][G][2] maximum and sum

  const int tid = threadIdx.x;
  const int lane = tid & (RA_WAVE - 1), wave = tid / RA_WAVE;
  const int r = lane & 15, g = lane >> 4;

  // Item i is (token i / (max_chunks * Hkv), chunk (i / Hkv) % max_chunks, KV head i % Hkv): known from
  // the item's number alone, so the first trip to memory is already the token's own position and
  // request. A token whose keys make fewer chunks leaves its last items empty (they end here).
  const int n_items = n_tokens * max_chunks * Hkv;
  for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
    const int slot = item / Hkv, kvh = item % Hkv;  // KV heads of one (token, chunk) are neighbours in memory
    const int li = slot / max_chunks, ci = slot % max_chunks;
    const int t = token_list ? token_list[li] : t_base + li;
    // seq_of_token null: every request of the step brings one token, token t is request t
    const int seq = seq_of_token ? seq_of_token[t] : t;
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const FdCut cut = fd_cut(p, lo, chunk_shift, max_chunks, FD_WAVES * 32);
    const int n_chunks = cut.n;
    if (ci >= n_chunks) continue;
    const int* table = block_tables + (size_t)seq * max_blocks;

    // second operand of the score product: column r is query head r of the group
    bf16x8_t qreg[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const int e = dt * 32 + g * 8;
      qreg[dt] = (bf16x8_t){0, 0, 0, 0, 0, 0, 0, 0};
      if (r < G && e < d) qreg[dt] = *(const bf16x8_t*)(q + (size_t)t * q_stride + (size_t)(kvh * G + r) * d + e);
    }
    f32x4_t acc[NOT];
#pragma unroll
    for (int i = 0; i < NOT; ++i) acc[i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    const int k_begin = cut.base + ci * cut.chunk;
    const int k_end = min(k_begin + cut.chunk, p + 1);
    // Block ids come through the scalar cache (the index is made uniform for the compiler) and are asked
    // for one step ahead: a vector load would queue behind the K and V loads in flight, and under load a
    // load that the K and V loads depend on costs microseconds. (The table's head fetched into LDS beside
    // the position, to save the trip that waits for the position, was measured: the barrier it needs
    // costs what the trip did.)
    auto block_of = [&](int kt_any) -> int {
      const int kt = __builtin_amdgcn_readfirstlane(kt_any);
      return (kt <= p && kt + 15 >= lo && kt < k_end) ? table[kt / block_size] : 0;
    };
    int next_blk[2];
    next_blk[0] = block_of(k_begin + wave * 32);
    next_blk[1] = block_of(k_begin + wave * 32 + 16);
    for (int k0 = k_begin + wave * 32; k0 < k_end; k0 += FD_WAVES * 32) {
      const int blk_now[2] = {next_blk[0], next_blk[1]};
      next_blk[0] = block_of(k0 + FD_WAVES * 32);
      next_blk[1] = block_of(k0 + FD_WAVES * 32 + 16);
      if (k0 + 31 < lo) continue;
      // the two 16-key tiles of this step; a tile past the last key is not touched
      bool live[2], edge[2];
      const bf16_t* kb[2];
      const bf16_t* vb[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const int kt = k0 + tt * 16;
        live[tt] = kt <= p && kt + 15 >= lo;
        edge[tt] = kt + 15 > p || kt < lo;
        const int blk = live[tt] ? blk_now[tt] : 0;
        const size_t tile = ((size_t)blk * Hkv + kvh) * block_size * d + (size_t)((kt % block_size) >> 4) * 16 * d;
        kb[tt] = kcache + tile + (g * 16 + r) * 8;        // chunk 4 dt + g of slot r
        vb[tt] = vcache + tile + (g * 16 + r) * 4;        // slots 4g..4g+3 of row 16 ot + r
      }
      bf16x8_t kreg[2][NDT];
      bf16x4_t vreg[2][NOT];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
          kreg[tt][dt] = (bf16x8_t){0, 0, 0, 0, 0, 0, 0, 0};
          if (live[tt] && dt * 32 + g * 8 < d) kreg[tt][dt] = *(const bf16x8_t*)(kb[tt] + dt * 512);
        }
#pragma unroll
        for (int ot = 0; ot < NOT; ++ot) {
          vreg[tt][ot] = (bf16x4_t){0, 0, 0, 0};
          if (live[tt] && ot * 16 < d) vreg[tt][ot] = *(const bf16x4_t*)(vb[tt] + ot * 256);
        }
      }
      f32x4_t s[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        s[tt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
          if (dt * 32 < d) s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[tt][dt], qreg[dt], s[tt], 0, 0, 0);
      }
      // mask and scale; keys outside [lo, p] get -inf, whatever bits their slots hold
      float tmax = -INFINITY;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = k0 + tt * 16 + 4 * g + i;
          const float v = (key <= p && key >= lo) ? s[tt][i] * scale_log2 : -INFINITY;
          s[tt][i] = v;
          tmax = fmaxf(tmax, v);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, RA_WAVE));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, RA_WAVE));
      const float mn = fmaxf(m, tmax);              // finite: the step holds at least one visible key
      const float corr = fd_exp2(m - mn);           // m = -inf gives 0
      bf16x8_t pb;
      float psum = 0.f;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float pr = fd_exp2(s[tt][i] - mn);  // masked: exp2(-inf) = 0
          psum += pr;
          pb[tt * 4 + i] = from_f32<bf16_t>(pr);
        }
      l = l * corr + psum;
      m = mn;
      // values of masked keys may be anything (a freed block's bits): zero them at the edges
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
        if (edge[tt]) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = k0 + tt * 16 + 4 * g + i;
            if (!(key <= p && key >= lo)) {
#pragma unroll
              for (int ot = 0; ot < NOT; ++ot) vreg[tt][ot][i] = (bf16_t)0.f;
            }
          }
        }
#pragma unroll
      for (int ot = 0; ot < NOT; ++ot) {
        if (ot * 16 < d) {
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[ot][i] *= corr;
          const bf16x8_t a = {vreg[0][ot][0], vreg[0][ot][1], vreg[0][ot][2], vreg[0][ot][3],
                              vreg[1][ot][0], vreg[1][ot][1], vreg[1][ot][2], vreg[1][ot][3]};
          acc[ot] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, acc[ot], 0, 0, 0);
        }
      }
    }
    // lane groups hold partial sums of l over their own keys
    l += __shfl_xor(l, 16, RA_WAVE);
    l += __shfl_xor(l, 32, RA_WAVE);

    // merge the waves through LDS: lane (head r, group g) holds O^T rows 16 ot + 4 g + i
    float* lds_o = lds;                                  // [waves][G][d]
    float* lds_ml = lds + FD_WAVES * G * d;              // [waves][G][2]
    if (r < G) {
#pragma unroll
      for (int ot = 0; ot < NOT; ++ot)
        if (ot * 16 < d) {
#pragma unroll
          for (int i = 0; i < 4; ++i) lds_o[((size_t)wave * G + r) * d + ot * 16 + 4 * g + i] = acc[ot][i];
        }
      if (g == 0) {
        lds_ml[(wave * G + r) * 2] = m;
        lds_ml[(wave * G + r) * 2 + 1] = l;
      }
    }
    __syncthreads();
    const size_t pair = (size_t)li * Hkv + kvh;
    const size_t prow = (pair * max_chunks + ci) * G;      // [pair][chunk][head]
    for (int idx = tid; idx < G * d; idx += FD_THREADS) {
      const int h = idx / d, e = idx % d;
      float mw = -INFINITY;
#pragma unroll
      for (int w = 0; w < FD_WAVES; ++w) mw = fmaxf(mw, lds_ml[(w * G + h) * 2]);
      float lt = 0.f, ot = 0.f;
#pragma unroll
      for (int w = 0; w < FD_WAVES; ++w) {
        const float mwv = lds_ml[(w * G + h) * 2];
        const float c = (mwv == -INFINITY) ? 0.f : fd_exp2(mwv - mw);
        lt += lds_ml[(w * G + h) * 2 + 1] * c;
        ot += lds_o[((size_t)w * G + h) * d + e] * c;
      }
      if (n_chunks == 1) {
        out[(size_t)t * out_stride + (size_t)(kvh * G + h) * d + e] = from_f32<bf16_t>(ot / lt);
      } else {
        part_o[(prow + h) * d + e] = ot;
        if (e == 0) {
          part_ml[(prow + h) * 2] = mw;
          part_ml[(prow + h) * 2 + 1] = lt;
        }
      }
    }
    __syncthreads();                                // the next item writes the same LDS
  }
}

// Merge of the chunks of one (token, head), one wave each: lane c weighs chunk c, then the lanes share
// the d outputs. With up to FDM_AHEAD chunks a token everything the wave may need (the maxima and sums
// and the partial outputs of all max_chunks rows) is asked for at once, beside the token's position,
// before the number of chunks is known: rows past it hold whatever was there and are left out by
// selection, never by a factor of zero. That is one trip to memory instead of three in a row.
#define FDM_AHEAD 16
// AHEAD = outputs a lane (1, 2 or 4: head sizes up to 64, 128, 256) of the form that asks ahead; 0: the general form
template <int AHEAD>
__global__ void __launch_bounds__(RA_WAVE)
flash_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                          bf16_t* __restrict__ out, int out_stride, const int* __restrict__ token_list,
                          const int* __restrict__ positions, int Hkv, int G, int d, int window, int chunk_shift,
                          int max_chunks, int gran, int t_base) {
  const int head = blockIdx.x, li = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = head / G, h = head % G;
  const size_t base = ((size_t)li * Hkv + kvh) * max_chunks * G + h;    // row of chunk 0; chunks are G rows apart
  const int t = token_list ? token_list[li] : t_base + li;
  if (AHEAD) {
    // max_chunks <= FDM_AHEAD, d <= 64 * AHEAD
    constexpr int EPL = AHEAD > 0 ? AHEAD : 1;
    float v[FDM_AHEAD][EPL];
    const int cl = lane < max_chunks ? lane : max_chunks - 1;
    const float mc_raw = part_ml[(base + (size_t)cl * G) * 2];
    const float lc_raw = part_ml[(base + (size_t)cl * G) * 2 + 1];
#pragma unroll
    for (int c = 0; c < FDM_AHEAD; ++c) {
      const float* po = part_o + (base + (size_t)(c < max_chunks ? c : max_chunks - 1) * G) * d;
#pragma unroll
      for (int i = 0; i < EPL; ++i) {
        const int e = lane + i * RA_WAVE;
        v[c][i] = po[e < d ? e : d - 1];
      }
    }
    const int p = positions[t];
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int n_chunks = fd_cut(p, lo, chunk_shift, max_chunks, gran).n;
    if (n_chunks == 1) return;                           // written by the first kernel
    const bool mine = lane < n_chunks;
    const float mc = mine ? mc_raw : -INFINITY, lc = mine ? lc_raw : 0.f;
    const float mt = wave_max(mc);                       // finite: every chunk saw at least one key
    const float w = mine ? fd_exp2(mc - mt) : 0.f;
    const float lt = wave_sum(lc * w);
    float acc[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) acc[i] = 0.f;
#pragma unroll
    for (int c = 0; c < FDM_AHEAD; ++c) {
      const float wc = __shfl(w, c, RA_WAVE);
      if (c < n_chunks) {                                // uniform; chunk order
#pragma unroll
        for (int i = 0; i < EPL; ++i) acc[i] += v[c][i] * wc;
      }
    }
    const float inv = 1.f / lt;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const int e = lane + i * RA_WAVE;
      if (e < d) out[(size_t)t * out_stride + (size_t)head * d + e] = from_f32<bf16_t>(acc[i] * inv);
    }
    return;
  }
  const int p = positions[t];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int n_chunks = fd_cut(p, lo, chunk_shift, max_chunks, gran).n;
  if (n_chunks == 1) return;                           // written by the first kernel
  float acc[4] = {0.f, 0.f, 0.f, 0.f};                 // d <= 256: up to 4 outputs a lane
  float mt = -INFINITY, lt = 0.f;
  for (int c0 = 0; c0 < n_chunks; c0 += RA_WAVE) {
    const int c = c0 + lane;
    float mc = -INFINITY, lc = 0.f;
    if (c < n_chunks) {
      mc = part_ml[(base + (size_t)c * G) * 2];
      lc = part_ml[(base + (size_t)c * G) * 2 + 1];
    }
    const float mn = fmaxf(mt, wave_max(mc));          // finite: every chunk saw at least one key
    const float corr = fd_exp2(mt - mn);
    const float w = (c < n_chunks) ? fd_exp2(mc - mn) : 0.f;
    lt = lt * corr + wave_sum(lc * w);
    mt = mn;
    const int n_here = min(RA_WAVE, n_chunks - c0);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] *= corr;
    // four chunks' rows are requested before the first is used
    for (int cc = 0; cc < n_here; cc += 4) {
      float v[4][4], wc[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bool ok = cc + u < n_here;
        wc[u] = ok ? __shfl(w, cc + u, RA_WAVE) : 0.f;
        const float* po = part_o + (base + (size_t)(c0 + (ok ? cc + u : cc)) * G) * d;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int e = lane + i * RA_WAVE;
          v[u][i] = (e < d) ? po[e] : 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += v[u][i] * wc[u];
    }
  }
  const float inv = 1.f / lt;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int e = lane + i * RA_WAVE;
    if (e < d) out[(size_t)t * out_stride + (size_t)head * d + e] = from_f32<bf16_t>(acc[i] * inv);
  }
}

// Workgroups of the kernel that the current device holds at once (asked once a head-size variant, waves a
// workgroup and LDS size; the answer of the first device stands for all: one kind of GPU in a process).
static int fd_resident_workgroups(int variant, int waves, size_t lds) {
  static int cached[3][2] = {{0, 0}, {0, 0}, {0, 0}};
  static size_t cached_lds[3][2] = {{0, 0}, {0, 0}, {0, 0}};
  const int wi = waves == 4 ? 0 : 1;
  if (cached[variant][wi] > 0 && cached_lds[variant][wi] == lds) return cached[variant][wi];
  int dev = 0, cus = 0, per_cu = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  hipError_t e = hipSuccess;
  // the exact form of a head size needs a few registers more than the other: ask for it
#define RA_FD_OCC(DM)                                                                                                  \
  e = waves == 4 ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, flash_decode_kernel<DM, true, 4>, 4 * RA_WAVE, lds) \
                 : hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, flash_decode_kernel<DM, true, 12>, 12 * RA_WAVE, lds)
  if (variant == 0) RA_FD_OCC(64);
  else if (variant == 1) RA_FD_OCC(128);
  else RA_FD_OCC(256);
#undef RA_FD_OCC
  if (e != hipSuccess || cus <= 0 || per_cu <= 0) return 0;
  cached[variant][wi] = cus * per_cu;
  cached_lds[variant][wi] = lds;
  return cached[variant][wi];
}

// 1 if the kernel takes these sizes, else 0 (the caller then uses the plain kernel)
extern "C" int ra_attention_decode_supports(int Hq, int Hkv, int d, int block_size) {
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0) return 0;
  const int G = Hq / Hkv;
  return (G >= 1 && G <= 16 && d % 16 == 0 && d >= 16 && d <= 256 && block_size > 0 &&
          block_size % 16 == 0) ? 1 : 0;
}

// Workgroups of the decode kernel, in its form with `waves` waves a workgroup (4 or 12), that the current
// device holds at once for these sizes (its grid); 0 if the sizes are not taken or the device cannot be
// asked. The caller cuts the keys so that the work items fill this grid once.
extern "C" int ra_attention_decode_slots(int Hq, int Hkv, int d, int waves) {
  if (!ra_attention_decode_supports(Hq, Hkv, d, 16) || (waves != 4 && waves != 12)) return 0;
  const size_t lds = (size_t)waves * (Hq / Hkv) * (d + 2) * sizeof(float);
  if (lds > 64 * 1024) return 0;
  return fd_resident_workgroups(d <= 64 ? 0 : d <= 128 ? 1 : 2, waves, lds);
}

extern "C" int ra_attention_decode(const void* q, int q_stride, void* out, int out_stride,
                                   const void* kcache, const void* vcache, const int* block_tables,
                                   int max_blocks, const int* token_list, const int* seq_of_token,
                                   const int* positions, int n_tokens, int block_size, int Hq, int Hkv,
                                   int d, float scale, int window, int chunk, int max_chunks, int waves,
                                   float* part_o, float* part_ml, hipStream_t stream) {
  RA_CHECK(n_tokens > 0, "attention_decode: no tokens");
  RA_CHECK(ra_attention_decode_supports(Hq, Hkv, d, block_size),
           "attention_decode: unsupported sizes (%d query heads, %d KV heads, head size %d, block %d)", Hq,
           Hkv, d, block_size);
  RA_CHECK(max_blocks > 0 && window >= 0, "attention_decode: bad cache geometry");
  RA_CHECK(chunk >= 128 && (chunk & (chunk - 1)) == 0, "attention_decode: chunk %d is no power of two from 128", chunk);
  if (waves == 0) waves = 4;
  RA_CHECK(waves == 4 || waves == 12, "attention_decode: workgroups of %d waves (4 or 12)", waves);
  const int chunk_shift = __builtin_ctz((unsigned)chunk);
  RA_CHECK(max_chunks >= 1 && max_chunks <= 65535, "attention_decode: %d chunks outside 1..65535", max_chunks);
  RA_CHECK(max_chunks == 1 || (part_o && part_ml),
           "attention_decode: more than one chunk needs the partial buffers");
  RA_CHECK(q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)kcache % 16) == 0 &&
               ((uintptr_t)vcache % 16) == 0,
           "attention_decode: operands must be 16-byte aligned");
  const int G = Hq / Hkv;
  const float scale_log2 = scale * 1.4426950408889634f;
  const size_t lds = (size_t)waves * G * (d + 2) * sizeof(float);
  RA_CHECK(lds <= 64 * 1024, "attention_decode: %d heads of %d per KV head need too much LDS", G, d);
  const int slots = fd_resident_workgroups(d <= 64 ? 0 : d <= 128 ? 1 : 2, waves, lds);
  RA_CHECK(slots > 0, "attention_decode: cannot size the grid (%s)", hipGetErrorString(hipGetLastError()));
  const long items_max = (long)n_tokens * Hkv * max_chunks;
  RA_CHECK(items_max < (1L << 30), "attention_decode: %ld work items in one launch", items_max);
  const int grid = (int)(items_max < slots ? items_max : slots);
#define RA_FD_GO(DM, EX, WV)                                                                          \
  flash_decode_kernel<DM, EX, WV><<<grid, WV * RA_WAVE, lds, stream>>>(                               \
      (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kcache,                    \
      (const bf16_t*)vcache, block_tables, max_blocks, token_list, seq_of_token, positions, block_size, \
      Hkv, G, d, scale_log2, window, chunk_shift, max_chunks, n_tokens, 0, part_o, part_ml)
#define RA_FD(DM)                                                                                     \
  do {                                                                                                \
    if (waves == 4) {                                                                                 \
      if (d == DM) RA_FD_GO(DM, true, 4);                                                             \
      else RA_FD_GO(DM, false, 4);                                                                    \
    } else {                                                                                          \
      if (d == DM) RA_FD_GO(DM, true, 12);                                                            \
      else RA_FD_GO(DM, false, 12);                                                                   \
    }                                                                                                 \
  } while (0)
  if (d <= 64) RA_FD(64);
  else if (d <= 128) RA_FD(128);
  else RA_FD(256);
#undef RA_FD_GO
#undef RA_FD
  RA_LAUNCH_CHECK("attention_decode");
  if (max_chunks > 1) {
    RA_CHECK(n_tokens <= 65535, "attention_decode: %d tokens in one launch of the merge (max 65535)", n_tokens);
    dim3 mg(Hq, n_tokens);
#define RA_FDM(AH)                                                                                          \
  flash_decode_merge_kernel<AH><<<mg, RA_WAVE, 0, stream>>>(part_o, part_ml, (bf16_t*)out, out_stride, token_list, \
                                                           positions, Hkv, G, d, window, chunk_shift, max_chunks, waves * 32, 0)
    if (max_chunks > FDM_AHEAD) RA_FDM(0);
    else if (d <= 64) RA_FDM(1);
    else if (d <= 128) RA_FDM(2);
    else RA_FDM(4);
#undef RA_FDM
    RA_LAUNCH_CHECK("attention_decode merge");
  }
  return 0;
}
