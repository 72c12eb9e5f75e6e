// C interface of the gfx950 kernel library. Every entry point checks its
// arguments on the host, launches on the given stream and returns 0, or
// returns non-zero with a message in ra_last_error(). Pointers are device
// memory unless said otherwise. dtype tags: 0 = float, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>

#define RA_ABI_VERSION 17

#ifdef __cplusplus
extern "C" {
#endif

const char* ra_last_error(void);
int ra_abi_version(void);

int ra_embed(const void* table, int table_dtype, const int* ids, float* out, int n_tokens, int hidden,
             hipStream_t stream);

int ra_add_rmsnorm(float* resid, const void* delta, const void* weight, int weight_dtype, void* out,
                   int act_dtype, const int* rows, int n_rows, int hidden, float eps, hipStream_t stream);

int ra_qk_norm_rope_cache(void* qkv, int act_dtype, const void* q_weight, const void* k_weight,
                          int weight_dtype, float eps, const int* positions, const float* inv_freq,
                          int rotary_dim, int rope_style, const int* slots, void* kcache, void* vcache,
                          int block_size, int n_tokens, int Hq, int Hkv, int d, hipStream_t stream);
// The same from the partial results of ra_gemm_wide_partial (added here, in range order), optionally scaled
// by the RMSNorm that product carried (in_ss [in_parts][n_tokens], eps, width); the rotated q goes to q_out.
int ra_qk_norm_rope_cache_sums(const float* parts, int n_ranges, const float* in_ss, int in_parts, float in_eps,
                               int in_width, void* q_out, int q_stride, int act_dtype, const void* q_weight,
                               const void* k_weight, int weight_dtype, float eps, const int* positions,
                               const float* inv_freq, int rotary_dim, int rope_style, const int* slots,
                               void* kcache, void* vcache, int block_size, int n_tokens, int Hq, int Hkv, int d,
                               hipStream_t stream);

// gate_up is [T, 2I]: group == 0: gate columns [0, I), up columns [I, 2I); group > 0: gate and
// up interleaved in runs of `group` columns (gate run, then the up run of the same features)
int ra_silu_mul(const void* gate_up, void* out, int act_dtype, int n_tokens, int intermediate,
                int group, hipStream_t stream);

int ra_attention_plain(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                       const void* vcache, int act_dtype, const int* block_tables, int max_blocks,
                       const int* token_list, const int* seq_of_token, const int* positions, int n_tokens,
                       int block_size,
                       int Hq, int Hkv, int d, float scale, int window, hipStream_t stream);

int ra_gemm_plain(const void* A, const void* W, const void* bias, void* C, int in_dtype, int out_dtype,
                  int M, int N, int K, int lda, int ldc, hipStream_t stream);

// bfloat16, M <= 64, K and lda multiples of 8: weight-streaming MFMA product.
// epilogue 0: C[M, N] = A . W^T (+ bias); epilogue 1: W rows are gate/up interleaved in runs of 8
// and C[M, N/2] = silu(gate) * up; epilogue 2: C is float and C += A . W^T (+ bias)
int ra_gemm_skinny_max_rows(void);
int ra_gemm_skinny(const void* A, const void* W, const void* bias, void* C, int out_dtype, int epilogue,
                   int M, int N, int K, int lda, int ldc, hipStream_t stream);
// The same with an RMSNorm carried by the products around it, y = rstd[m] * ((x .* w) . W^T):
// in_ss float [in_parts, M], if given: partial sums of squares of the rows behind A; the result
// rows are scaled by rsqrt(sum / in_width + in_eps). out_w / out_x / out_ss, if given (epilogue 2
// only, up to 16 rows): after C += ..., out_x[M, N] = bf16(C * out_w[n]) and
// out_ss[ra_gemm_skinny_row_parts(M, N), M] = each workgroup's sums of squares of its columns of C.
int ra_gemm_skinny_row_parts(int M, int N);
int ra_gemm_skinny_normed(const void* A, const void* W, const void* bias, void* C, int out_dtype,
                          int epilogue, int M, int N, int K, int lda, int ldc, const float* in_ss,
                          int in_parts, float in_eps, int in_width, const void* out_w, int out_w_dtype,
                          void* out_x, int out_ldx, float* out_ss, hipStream_t stream);

// bfloat16, up to 64 rows: the same product and epilogues with the activations shared by a
// workgroup's waves; ra_gemm_wide_preferred says where it is the faster of the two (17 rows and
// more, not the smallest products). Small N cuts K into ranges whose float partial results need
// `ra_gemm_wide_scratch(...)` floats of scratch (0: none needed). A product that is cut so may have up to
// 128 rows (ra_gemm_wide_preferred says which are worth it: adding into the stream over a long K).
int ra_gemm_wide_ranges(int M, int N, int K);          // K ranges of ra_gemm_wide_partial's result
int ra_gemm_wide_partial(const void* A, const void* W, float* P, long p_floats, int M, int N, int K, int lda,
                         hipStream_t stream);         // P[range][m][n] float, for a consumer that adds the ranges
int ra_gemm_wide_preferred(int epilogue, int M, int N, int K);
long ra_gemm_wide_scratch(int epilogue, int M, int N, int K, int emits);
int ra_gemm_wide(const void* A, const void* W, const void* bias, void* C, int out_dtype, int epilogue,
                 int M, int N, int K, int lda, int ldc, float* scratch, long scratch_floats,
                 hipStream_t stream);
// With a carried RMSNorm, as ra_gemm_skinny_normed; an emitting product always needs scratch
// (ra_gemm_wide_scratch with emits = 1) and writes out_ss[ra_gemm_wide_row_parts(N), M]. With out_ss null and
// out_eps >= 0 it finishes the norm that follows instead: out_x = bf16(norm(C_new, out_eps) * out_w), one
// workgroup a row (N a multiple of 4, at most 16384).
int ra_gemm_wide_row_parts(int N);
int ra_gemm_wide_normed(const void* A, const void* W, const void* bias, void* C, int out_dtype, int epilogue,
                        int M, int N, int K, int lda, int ldc, float* scratch, long scratch_floats,
                        const float* in_ss, int in_parts, float in_eps, int in_width, const void* out_w,
                        int out_w_dtype, void* out_x, int out_ldx, float* out_ss, float out_eps,
                        hipStream_t stream);

// The cache of a layer: K and V are [blocks][Hkv][block_size * d], every (block, KV head) slab
// in tiles of 16 slots laid out in MFMA operand order (cache_k_index, cache_v_index in common.h);
// block_size and d are multiples of 16.
//
// bfloat16 flash-decode: one query per listed token. A token's keys are cut into equal chunks of its
// own length: at most max_chunks of them, each a whole number of the workgroup's rounds (waves x 32 keys) and
// about `chunk` (a power of two, 128 or more) or longer. `waves` = waves a workgroup, 4 or 12 (0: 4): 12 where
// the step has few (token, KV head) pairs. With max_chunks > 1: part_o float [n_tokens * Hkv, max_chunks, G, d],
// part_ml float [.., 2], merged by a second kernel.
int ra_attention_decode_supports(int Hq, int Hkv, int d, int block_size);
int ra_attention_decode_slots(int Hq, int Hkv, int d, int waves);   // workgroups of its grid on this device (0: unknown)
int ra_attention_decode(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                        const void* vcache, const int* block_tables, int max_blocks,
                        const int* token_list, const int* seq_of_token, const int* positions,
                        int n_tokens, int block_size, int Hq, int Hkv, int d, float scale, int window,
                        int chunk, int max_chunks, int waves, float* part_o, float* part_ml, hipStream_t stream);

// bfloat16 flash prefill over query tiles; tile_info holds 4 ints per tile:
// request row in block_tables, first token row, number of queries (<= tile), first position.
// Where ra_attention_prefill_columns() is 2, bits 16-17 of the third may name the half of the heads a
// workgroup computes (1 or 2; 0 or 3: all): the same tile listed twice, once with each, is computed by
// two workgroups. A tile makes ra_attention_prefill_groups() workgroups.
int ra_attention_prefill_supports(int Hq, int Hkv, int d, int block_size);
int ra_attention_prefill_tile(int Hq, int Hkv, int d);
int ra_attention_prefill_columns(int Hq, int Hkv, int d);
int ra_attention_prefill_groups(int Hq, int Hkv, int d);
int ra_attention_prefill(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                         const void* vcache, const int* block_tables, int max_blocks, const int* tile_info,
                         int n_tiles, int block_size, int Hq, int Hkv, int d, float scale, int window,
                         hipStream_t stream);
// The same with query tiles cut by keys: ranges = three ints a listed tile (first key, one past the last, both
// multiples of 64; the part's slot, or -1 for a whole tile); merge_info = four ints a cut tile (first token row,
// queries, first slot, parts: a tile's parts hold consecutive slots in key order); part_o / part_ml: floats as
// ra_attention_prefill_part_floats(Hq, Hkv, d, slots, 0 / 1) says. A second kernel adds the parts up in order.
long ra_attention_prefill_part_floats(int Hq, int Hkv, int d, int n_slots, int which);
int ra_attention_prefill_split(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                               const void* vcache, const int* block_tables, int max_blocks, const int* tile_info,
                               int n_tiles, const int* ranges, const int* merge_info, int n_merge, float* part_o,
                               float* part_ml, int block_size, int Hq, int Hkv, int d, float scale, int window,
                               hipStream_t stream);

int ra_sample_slices(int vocab);
int ra_sample(const float* logits, int n_rows, int vocab, int row_stride, const float* temperature,
              const long long* seeds, const int* positions, float* scratch_val, int* scratch_idx,
              int* tokens, hipStream_t stream);

// ra_sample for callers that cannot allocate device memory (code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. The slice
// winners go to an array that the library holds on every GPU it runs on (512 KiB, until the process
// ends) instead of caller buffers; inputs and `tokens` are still the caller's. It calls no hipMalloc,
// hipFree or allocating routine; n_rows * ra_sample_slices(vocab) may be at most
// ra_sample_static_max_pairs() (65536), more is refused with a message. All calls on one GPU share that
// GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.
// ra_sample_static_prepare() looks the array's address up for the current device (once per device, under
// a lock); ra_sample_static does the same at its first call on a device, so a caller that captures its
// stream calls prepare beforehand, outside the capture.
long ra_sample_static_max_pairs(void);
int ra_sample_static_prepare(void);
int ra_sample_static(const float* logits, int n_rows, int vocab, int row_stride, const float* temperature,
                     const long long* seeds, const int* positions, int* tokens, hipStream_t stream);

// Logit bias, penalties and filters on rows of float logits, in place, before ra_sample. `rows`
// holds one record of 12 x 4 bytes per row: float temperature, top_p, min_p, repeat_penalty,
// frequency_penalty, presence_penalty; int top_k, window_off, window_len, bias_off, bias_len, pad.
// `window` holds the requests' recent tokens, row r's at [window_off, window_off + window_len), and
// its logit bias as bias_len pairs (token id, float bits) from bias_off, each id once.
int ra_filter_logits(float* logits, int n_rows, int vocab, int row_stride, const void* rows,
                     const int* window, hipStream_t stream);

// What the machine gives at best (peaks.hip; for measurement, not on the product path): one read of
// `bytes` of device memory, and `iters` iterations of bfloat16 matrix-core products on registers
// (shape 16: eight 16x16x32 an iteration; shape 32: four 32x32x16) in `waves_per_cu` waves on every CU
// (*flops: what all of them did). `sink` is 4 bytes of
// device memory that is never written in practice.
int ra_stream_read(const void* src, long bytes, void* sink, hipStream_t stream);
int ra_mfma_loop(int shape, int iters, int waves_per_cu, void* sink, double* flops, hipStream_t stream);

#ifdef __cplusplus
}
#endif
