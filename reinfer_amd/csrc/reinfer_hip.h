// C interface of the gfx950 kernel library. Every entry point checks its
// arguments on the host, launches on the given stream and returns 0, or
// returns non-zero with a message in ra_last_error(). Pointers are device
// memory unless said otherwise. dtype tags: 0 = float, 1 = bfloat16.
#pragma once
#include <hip/hip_runtime.h>

#define RA_ABI_VERSION 23

#ifdef __cplusplus
extern "C" {
#endif

const char* ra_last_error(void);
int ra_abi_version(void);

int ra_embed(const void* table, int table_dtype, const int* ids, float* out, int n_tokens, int hidden,
             float scale, hipStream_t stream);

int ra_add_rmsnorm(float* resid, const void* delta, const void* weight, int weight_dtype, void* out,
                   int act_dtype, const int* rows, int n_rows, int hidden, float eps, float delta_scale,
                   hipStream_t stream);

// The same norm in `groups` equal consecutive parts of the row, each over its own root mean square.
int ra_add_group_rmsnorm(float* resid, const void* delta, const void* weight, int weight_dtype, void* out,
                         int act_dtype, const int* rows, int n_rows, int hidden, int groups, float eps,
                         float delta_scale, hipStream_t stream);

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
// out = act(gate) * up; act 0: silu, act 1: the tanh form of gelu
int ra_act_mul(const void* gate_up, void* out, int act_dtype, int n_tokens, int intermediate, int group, int act,
               hipStream_t stream);

int ra_attention_plain(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                       const void* vcache, int act_dtype, const int* block_tables, int max_blocks,
                       const int* token_list, const int* seq_of_token, const int* positions, int n_tokens,
                       int block_size,
                       int Hq, int Hkv, int d, float scale, int window, hipStream_t stream);
// The `_mod` forms of the three attention kernels change a score between the scaled product and the softmax:
// softcap > 0: s <- softcap tanh(s / softcap); r1, r2 (float, one entry a query head, both or neither):
// s <- s - r1[h] ln(1 + r2[h] (query position - key position)); the cap first.
int ra_attention_plain_mod(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                           const void* vcache, int act_dtype, const int* block_tables, int max_blocks,
                           const int* token_list, const int* seq_of_token, const int* positions, int n_tokens,
                           int block_size, int Hq, int Hkv, int d, float scale, int window, float softcap,
                           const float* r1, const float* r2, hipStream_t stream);
// act 2 of ra_act_mul with its bound: g <- min(g, lim), u <- clamp(u, -lim, lim), out = g sigmoid(1.702 g) (u + 1)
int ra_act_mul_bounded(const void* gate_up, void* out, int act_dtype, int n_tokens, int intermediate, int group,
                       int act, float lim, hipStream_t stream);

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
int ra_attention_decode_mod(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                            const void* vcache, const int* block_tables, int max_blocks,
                            const int* token_list, const int* seq_of_token, const int* positions,
                            int n_tokens, int block_size, int Hq, int Hkv, int d, float scale, int window,
                            int chunk, int max_chunks, int waves, float* part_o, float* part_ml, float softcap,
                            const float* r1, const float* r2, hipStream_t stream);
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

int ra_attention_prefill_mod(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                             const void* vcache, const int* block_tables, int max_blocks, const int* tile_info,
                             int n_tiles, int block_size, int Hq, int Hkv, int d, float scale, int window,
                             float softcap, const float* r1, const float* r2, hipStream_t stream);
int ra_attention_prefill_split_mod(const void* q, int q_stride, void* out, int out_stride, const void* kcache,
                                   const void* vcache, const int* block_tables, int max_blocks, const int* tile_info,
                                   int n_tiles, const int* ranges, const int* merge_info, int n_merge, float* part_o,
                                   float* part_ml, int block_size, int Hq, int Hkv, int d, float scale, int window,
                                   float softcap, const float* r1, const float* r2, hipStream_t stream);

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

// ---- around the residual stream (stream.hip) ----
// resid[t, :] += table[row(t), :] with row(t) = (prev * mul_prev + id * mul_cur) mod buckets, row `buckets` for a
// request's first token (position 0). The token before a portion's first comes from last_token[state slot of the
// request], which is then set to the portion's last token; state slot -1 reads and writes nothing.
int ra_pair_hash_add(float* resid, const void* table, int table_dtype, const int* ids, const int* positions,
                     const int* seq_of_token, const int* cu_tokens, const int* state_slots, int* last_token,
                     int buckets, long long mul_prev, long long mul_cur, int n_tokens, int hidden,
                     hipStream_t stream);
// resid[t, :] += delta[t, :] + other[t, :] + vec[:]; every addend may be null
int ra_stream_add(float* resid, const void* delta, int delta_dtype, const float* other, const void* vec,
                  int vec_dtype, int n_tokens, int hidden, float delta_scale, hipStream_t stream);
// logits <- cap * tanh(logits / cap) in place
int ra_tanh_cap(float* logits, int n_rows, int vocab, int row_stride, float cap, hipStream_t stream);

// ---- attention over a shared latent (latent.hip) ----
// proj rows hold H query heads ([D unrotated | R rotated] each) from column q_off and [c_raw (rank) | kr (R)] from
// column dkv_off. Writes the cache row [rms(c_raw) * c_weight | rot(kr) | 0...] of Dp (a multiple of 16) elements in
// the K and V tile layouts of one KV head at slots[t] (-1: nothing), and q_lat[t, h, rank:Dp] = [rot(q_h's rotated
// part) | 0...]. Rotation: the first rot_dims of an R-wide part, half-split pairs, angle pos * inv_freq[i].
int ra_latent_prep(const void* proj, int act_dtype, int ld, int q_off, int dkv_off, const void* c_weight,
                   int weight_dtype, float eps, const int* positions, const float* inv_freq, int rot_dims, int R,
                   int rank, int H, int D, void* q_lat, int Dp, const int* slots, void* kcache, void* vcache,
                   int block_size, int n_tokens, hipStream_t stream);
// out[t, h * o_head + n] = sum_k x[t, h * x_head + k] * W[h, k, n] (* sigmoid(gate[t, h * N + n]) if gate, or
// * sigmoid(gate[t, h]) with gate_per_head: one number a head)
int ra_head_linear(const void* x, int ldx, int x_head, const void* W, void* out, int ldo, int o_head,
                   const void* gate, int ldg, int gate_per_head, int act_dtype, int n_tokens, int H, int N, int K,
                   hipStream_t stream);

// ---- mixture of experts (moe.hip) ----
// the `top` (<= 64) largest of each row of float logits [n_tokens, experts] (row stride ld) in falling order into
// ids [n_tokens, top] (ties: the lower expert first), their softmax over the chosen alone into weights [n_tokens, top]
int ra_moe_topk(const float* logits, int ld, int experts, int top, int* ids, float* weights, int n_tokens,
                hipStream_t stream);
// act[t, e * ff + j] = weight(t, e) * relu(up[t, e * ff + j])^2 for chosen experts, 0 for the others
int ra_moe_relu2_scale(const void* up, void* act, int act_dtype, const int* ids, const float* weights, int top,
                       int experts, int ff, int n_tokens, hipStream_t stream);

// Few tokens: only the chosen experts' rows are read. w_up [experts * ff, width], w_down [width, experts * ff];
// act[t * top + j, f] = weights[t, j] * relu(w_up[ids[t, j] * ff + f, :] . x[t, :])^2, then
// y[t, n] = sum_j w_down[n, ids[t, j] * ff : ...] . act[t * top + j, :], added into resid (float [n_tokens, width])
// or written to out ([n_tokens, width], the activations' dtype): exactly one of the two is given
int ra_moe_up_chosen(const void* x, int ldx, const void* w_up, const int* ids, const float* weights, void* act,
                     int act_dtype, int n_tokens, int top, int experts, int ff, int width, hipStream_t stream);
int ra_moe_down_chosen(const void* act, const void* w_down, const int* ids, float* resid, void* out, int act_dtype,
                       int n_tokens, int top, int experts, int ff, int width, hipStream_t stream);

// sigmoid scores, groups of experts of which the best `kept` stay (a group's score: the sum of its `group_top`
// largest), then the `top` largest; weights = score * scale, not renormalised
int ra_moe_route_sigmoid(const float* logits, int ld, int experts, int top, int groups, int kept, int group_top,
                         float scale, int* ids, float* weights, int n_tokens, hipStream_t stream);
// gu [n_tokens, 2 (experts ff + shared)]: [gate | up] an expert, the shared expert's behind them;
// act [n_tokens, experts ff + shared] = weight * silu(gate) * up (0 for experts not chosen, weight 1 for the shared one)
int ra_moe_silu_gate_scale(const void* gu, void* act, int act_dtype, const int* ids, const float* weights, int top,
                           int experts, int ff, int shared, int n_tokens, hipStream_t stream);

// The same with the shared expert's weight sigmoid(shared_logit[t * ld_logit]) (float; null: weight 1); chosen ids
// of `experts` or more name no matrices and are skipped
int ra_moe_silu_gate_scale_shared(const void* gu, void* act, int act_dtype, const int* ids, const float* weights,
                                  int top, int experts, int ff, int shared, const float* shared_logit, int ld_logit,
                                  int n_tokens, hipStream_t stream);
// softmax scores over all `experts` router outputs; the choice is by score + correction (float [experts], may be
// null) inside the `kept` best of `groups` groups of neighbours (a group's score: its largest choice score); the
// weights are the chosen scores over their sum + norm_eps
int ra_moe_route_softmax(const float* logits, int ld, int experts, int top, int groups, int kept,
                         const float* correction, float norm_eps, int* ids, float* weights, int n_tokens,
                         hipStream_t stream);
// y[t, :] += (sum of weights[t, j] with ids[t, j] >= experts) * x[t, :]: chosen ids past the experts stand for the
// identity
int ra_moe_identity_add(void* y, int ldy, const void* x, int ldx, int act_dtype, const int* ids, const float* weights,
                        int top, int experts, int n_tokens, int width, hipStream_t stream);

// Few tokens, gated experts: only the chosen experts' rows are read, and the shared expert's. w_gate_up
// [2 (experts ff + shared), width], [gate; up] an expert, the shared expert's last; w_down [width, experts ff + shared].
// act [n_tokens, top ff + shared]: act[t, j ff + f] = weights[t, j] silu(gate) up of expert ids[t, j] (0 for an id of
// `experts` or more), behind them the shared expert's, times sigmoid(shared_logit[t * ld_logit]) (null: 1). Then
// out[t, n] = sum_j w_down[n, ids[t, j] ff : ...] . act[t, j ff : ...] + w_down[n, experts ff :] . act[t, top ff :]
//             + (sum of weights[t, j] with ids[t, j] >= experts) * x[t, n]
int ra_moe_gate_up_chosen(const void* x, int ldx, const void* w_gate_up, const int* ids, const float* weights,
                          const float* shared_logit, int ld_logit, void* act, int act_dtype, int n_tokens, int top,
                          int experts, int ff, int shared, int width, hipStream_t stream);
int ra_moe_down_gated_chosen(const void* act, const void* w_down, const int* ids, const float* weights, const void* x,
                             int ldx, void* out, int act_dtype, int n_tokens, int top, int experts, int ff, int shared,
                             int width, hipStream_t stream);

// ids[t, j] = table[token_ids[t], j] (table int32 [vocabulary, top]); weights[t, j] = 1 / top
int ra_moe_table_route(const int* token_ids, const int* table, int top, int* ids, float* weights, int n_tokens,
                       hipStream_t stream);

// ---- sublayer.hip: the stream as an operand, results that enter behind a norm, norms over runs of columns, turns ----
int ra_stream_cast(const float* x, void* out, int act_dtype, long n, hipStream_t stream);
// y = sum_i scales[i] xs[i]; normed: y <- y / rms(y) * weight (weight_stride 1: a vector, 0: one number);
// resid (float, or null) += y; copy (or null) = the new stream, or without resid the result, in copy_dtype
int ra_sum_norm_add(const void* const* xs, const float* scales, int n, int in_dtype, const float* weight,
                    int weight_stride, int normed, float eps, int n_tokens, int hidden, float* resid, void* copy,
                    int copy_dtype, hipStream_t stream);
int ra_span_rmsnorm(void* x, int act_dtype, long ld, int n_tokens, int n_spans, const int* col0, const int* width,
                    const int* count, const float* const* w, float eps, hipStream_t stream);
int ra_turn_heads(void* x, int act_dtype, long ld, int n_tokens, int heads, int head_stride, int width, int style,
                  const int* positions, const float* inv_freq, float sign, const void* gate, long ldg, int gate_stride,
                  hipStream_t stream);

// C += acc_scale * (A . W^T) through the weight-streaming kernels (bfloat16 operands, float C; the limits of
// ra_gemm_skinny / ra_gemm_wide with the accumulating epilogue)
int ra_gemm_skinny_scaled(const void* A, const void* W, float* C, int M, int N, int K, int lda, int ldc,
                          float acc_scale, hipStream_t stream);
int ra_gemm_wide_scaled(const void* A, const void* W, float* C, int M, int N, int K, int lda, int ldc, float* scratch,
                        long scratch_floats, float acc_scale, hipStream_t stream);

// ---- recurrent mixers (recurrent.hip) ----
// floats of state a request slot holds for the scan kernels; kind 0: matrix memory, 1: delta rule, 2: wkv, 3: a memory
// fading by a constant a head; -1: sizes not taken
long ra_scan_state_floats(int kind, int heads, int key_dim, int value_dim);
// max_q_len: the most tokens a request brings (0: unknown; it only sizes the chunks that are staged)
// gates [n_tokens, 2 heads] float pre-activations (input | forget); gates3 [n_tokens, 3 heads] scratch for the
// decay, input and threshold factors made from them; proj rows hold q, k (heads x key_dim) and v (heads x value_dim)
// at the given column offsets; out float [n_tokens, heads * value_dim]
int ra_matrix_memory_scan(const void* proj, int act_dtype, int ld, int q_off, int k_off, int v_off, const float* gates,
                          float* gates3, const float* gate_bias, float* state, long slot_stride, const int* cu_tokens,
                          const int* state_slots, const int* fresh, int n_seqs, int n_tokens, int max_q_len, int heads,
                          int key_dim, int value_dim, float gate_cap, float q_scale, float denom_eps, float* out,
                          hipStream_t stream);
// proj rows hold q | k (key_heads x key_dim each) | v (heads x value_dim) from column 0; filt float [channels, taps];
// the filter's tail lies at tail_off floats in a request's state slot; qkv float [n_tokens, channels]
int ra_delta_rule_prepare(const void* proj, int act_dtype, int ld, const float* filt, float* state, long slot_stride,
                          long tail_off, const int* seq_of_token, const int* cu_tokens, const int* state_slots,
                          const int* fresh, int n_seqs, int n_tokens, int key_heads, int key_dim, int heads,
                          int value_dim, int taps, float unit_eps, float q_scale, float* qkv, hipStream_t stream);
// gates [n_tokens, 2 heads] float pre-activations (b | a), turned into (beta | decay) in place
int ra_delta_rule_scan(const float* qkv, int ld, float* gates, const float* a_log, const float* dt_bias, float* state,
                       long slot_stride, const int* cu_tokens, const int* state_slots, const int* fresh, int n_seqs,
                       int n_tokens, int max_q_len, int heads, int key_heads, int key_dim, int value_dim, float* out,
                       hipStream_t stream);
// kind 2 of ra_scan_state_floats. proj rows hold r, k and v (heads x dim each) at the given column offsets; decay
// float [n_tokens, >= heads dim] holds the decays' pre-activations z, the decay being exp(-exp(z + w0)); u float
// [heads dim] is the bonus of the current token: o = (S + diag(u) k v^T)^T r, then S <- diag(decay) S + k v^T
int ra_wkv_scan(const void* proj, int act_dtype, int ld, int r_off, int k_off, int v_off, const float* decay, int ldw,
                const float* w0, const float* u, float* state, long slot_stride, const int* cu_tokens,
                const int* state_slots, const int* fresh, int n_seqs, int n_tokens, int max_q_len, int heads, int dim,
                float* out, hipStream_t stream);
// kind 3 of ra_scan_state_floats. proj rows hold q, k (heads x key_dim each) and v (heads x value_dim) at the given
// column offsets, before their silu (applied here, in float); decays float [heads]: S <- decays[h] S + k v^T, then
// o = S^T q
int ra_decay_scan(const void* proj, int act_dtype, int ld, int q_off, int k_off, int v_off, const float* decays,
                  float* state, long slot_stride, const int* cu_tokens, const int* state_slots, const int* fresh,
                  int n_seqs, int n_tokens, int max_q_len, int heads, int key_dim, int value_dim, float* out,
                  hipStream_t stream);
int ra_head_norm_gate(const float* read, const float* weight, int per_head_weight, const void* gate, int ldg,
                      int act_dtype, int silu, float eps, int n_tokens, int heads, int value_dim, void* out,
                      hipStream_t stream);
int ra_normed_mean(const void* const* xs, const float* const* ws, int n, int act_dtype, float eps, int n_tokens,
                   int hidden, void* out, float* resid, float scale, hipStream_t stream);

// ---- around a mixer that reads the token before (shift.hip) ----
// out[t, j width + e] = h[t, e] + (prev(t)[e] - h[t, e]) * mu[j, e] for j < n_mix; prev(t) is row t - 1 inside a
// portion and, for a portion's first row, the row kept at keep_off floats in the request's state slot (zeros at a
// request's start; state slot -1 reads zeros and keeps nothing). The slot then takes the portion's last row.
// single_tokens != 0 promises that every request of the step brings one token (one launch instead of two).
int ra_token_shift(const void* h, int ldh, const void* mu, int mu_dtype, int n_mix, float* state, long slot_stride,
                   long keep_off, const int* seq_of_token, const int* cu_tokens, const int* state_slots,
                   const int* fresh, void* out, int ldo, int act_dtype, int n_seqs, int n_tokens, int width,
                   int single_tokens, hipStream_t stream);
// resid[t, e] += sigmoid(gates[t, e]) * a[t, e] + sigmoid(gates[t, width + e]) * b[t, e]; b may be null
int ra_gated_stream_add(float* resid, const void* gates, int ldg, int gate_dtype, const void* a, int a_dtype,
                        const void* b, int b_dtype, int n_tokens, int width, hipStream_t stream);
// out[r, :] = x[r, :] / sqrt(mean(x[r, :]^2) + eps) * weight over rows of activations ldx / ldo apart
int ra_rows_rmsnorm(const void* x, int ldx, const void* weight, int weight_dtype, void* out, int ldo, int act_dtype,
                    int n_rows, int width, float eps, hipStream_t stream);
int ra_tanh_rows(void* x, int act_dtype, long n, hipStream_t stream);

#ifdef __cplusplus
}
#endif
