// C entry points of the kernel library.  Every function takes the HIP stream
// to launch on, returns 0 on success and nonzero after leaving a message for
// pa_last_error().  `dtype` codes: 0 = float32, 1 = bfloat16.  All pointers
// are device pointers unless said otherwise; nothing here allocates.
#pragma once
#ifdef __cplusplus
extern "C" {
#endif

const char* pa_last_error();
int pa_device_arch(char* out, int cap);
int pa_num_compute_units();

// A kernel that only reads: `bytes` (a multiple of 16) from src by `blocks` workgroups; out holds a word per
// workgroup.  For measuring the rate at which this device streams memory.
int pa_stream_read(void* stream, const void* src, long bytes, void* out, int blocks);
// out[t, :] = table[ids[t], :]
int pa_embed_gather(void* stream, int dtype, const int* ids, const void* table, void* out, int tokens, int hidden,
                    int vocab);
// ids[dst[i]] = sampled[src[i]] for i < n with src[i] >= 0 (token ids handed from one step to the next on the device).
int pa_carry_tokens(void* stream, const int* sampled, const int* src, const int* dst, int* ids, int n, int sampled_rows,
                    int tokens);
// Clears row slots[i] of data [num_rows, row_bytes] for every sequence i < nseq with fresh[i] != 0 and slots[i] >= 0:
// per-request state of fixed size starts from zero, decided on the device (so a captured step can do it).
int pa_zero_fresh_rows(void* stream, void* data, long row_bytes, const int* slots, const int* fresh, int nseq,
                       int num_rows);
// RMSNorm of x (+ residual, which then receives the sum) with a 32-bit weight;
// with `rows`, output row r comes from input row rows[r] and the residual is left alone.
int pa_rmsnorm(void* stream, int dtype, const void* x, void* residual, const float* w, void* out, const int* rows,
               int nrows, int hidden, float eps);
// The same with x given as `slices` 32-bit partial sums [slices, rows, hidden], slice_stride elements apart (what
// pa_gemm_mid leaves of a product cut along its inner size): they are added in order as they are loaded.
int pa_rmsnorm_slices(void* stream, int dtype, const float* parts, int slices, long slice_stride, void* residual,
                      const float* w, void* out, const int* rows, int nrows, int hidden, float eps);
// out[t, c] = act(gate_up[t, 2c]) * gate_up[t, 2c + 1]   (columns alternate gate_j, up_j); act: 0 SiLU, 1 GELU in its
// tanh form.  The products' gated epilogues take the same choice as epilogue code 1 + act.
int pa_silu_mul(void* stream, int dtype, const void* gate_up, void* out, int tokens, int inter, int act);
int pa_gather_rows(void* stream, int dtype, const void* x, const int* rows, void* out, int nrows, int width);
int pa_add_bias(void* stream, int dtype, void* y, const float* b, int tokens, int width);
int pa_to_f32(void* stream, int dtype, const void* x, float* out, long total);

// qkv [tokens, (nh + 2 nkv) * hd] -> q_out [tokens, nh, hd] (normed, rotated) and, where slots[t] >= 0,
// K (normed, rotated) into a cache laid out [page, nkv, page_size, hd] and V into one laid out
// [page, nkv, hd, page_size]; slot = page * page_size + offset.
int pa_qknorm_rope_kv(void* stream, int dtype, const void* qkv, const float* q_weight, const float* k_weight,
                      const float* cos_table, const float* sin_table, const int* positions, const int* slots,
                      void* q_out, void* k_cache, void* v_cache, int tokens, int nh, int nkv, int hd, int rot,
                      int page_size, float eps);

// pa_qknorm_rope_kv from the rotary frequencies alone (inv_freq [rot / 2], the angle position * inv_freq[j] taken in
// 32-bit in the kernel: no tables, no longest position); v_from_k: qkv is [tokens, (nh + nkv) * hd] and the cached
// value of a head is its key as projected, before norm and rotation.  q_scale (or null) [nh]: every query head times
// its number, in 32-bit before it is rounded (a temperature per head).
int pa_qknorm_rope_kv_freq(void* stream, int dtype, const void* qkv, const float* q_weight, const float* k_weight,
                           const float* inv_freq, const int* positions, const int* slots, void* q_out, void* k_cache,
                           void* v_cache, int tokens, int nh, int nkv, int hd, int rot, int page_size, float eps,
                           int v_from_k, const float* q_scale);

// C[m, n] = X[m, k] W[n, k]^T, bfloat16 with 32-bit accumulation, by hipBLASLt called directly; `workspace` is
// device memory its kernels may use.  The first call with a shape makes and keeps that shape's plan in host memory.
int pa_gemm_library(void* stream, const void* x, const void* w, void* c, int m, int n, int k, long ldx, long ldc,
                    void* workspace, long workspace_bytes);
// C[m, n] = A[m, k] W[n, k]^T (+ bias[n]), true 32-bit arithmetic.
int pa_gemm_plain(void* stream, int in_dtype, int out_dtype, const void* a, const void* w, const float* bias, void* c,
                  int m, int n, int k, long lda, long ldw, long ldc);

// C[m, n] = X[m, k] W[n, k]^T for a weight of few rows (n <= 256), bfloat16 operands (k a multiple of 8), 32-bit sums
// and result: what a router's scores want at any number of rows.
int pa_gemm_narrow(void* stream, const void* x, const void* w, float* c, int m, int n, int k, long ldx, long ldc);
// C[m, n] = X[m, k] W[n, k]^T for m <= 64 in bfloat16 (32-bit accumulation); out_dtype 0 = float32, 1 = bfloat16.
// epilogue 0: (+ bias[n]); 1: C[m, n/2] = silu(gate) * up for a weight whose rows alternate gate_j, up_j.
// tiled 1: w is the weight as pa_pack_tiles lays it out.
int pa_gemm_skinny_slices(int k, int slices);
int pa_gemm_skinny_sliced(void* stream, const void* x, const void* w, const float* bias, float* parts, int m, int n, int k,
                          long ldx, int slices, int waves);
int pa_gemm_skinny(void* stream, int out_dtype, int epilogue, const void* x, const void* w, const float* bias, void* c,
                   int m, int n, int k, long ldx, long ldc, int tiled);
// C[m, n] = X[m, k] W[n, k]^T for m <= 128 from the weight in tiles, X staged through LDS and W streamed by
// `waves` wavefronts a workgroup, 16 rows of W each (3, 4, 5, 6 or 8; 0: chosen from the weight's shape; the same
// bits at every number).  slices 1: as pa_gemm_skinny (epilogue 0 (+ bias) / 1 SiLU * up).
// slices > 1 (epilogue 0): the inner size is cut into that many slices, each left as 32-bit sums in
// parts [slices, m, n] (pa_gemm_mid_parts floats; the bias in the first) for the reader to add in order, and c is
// not written.  pa_gemm_mid_slices: the number of slices that suits an [n, k] weight.
int pa_gemm_mid_slices(int n, int k);
long pa_gemm_mid_parts(int m, int n, int slices);
int pa_gemm_mid(void* stream, int out_dtype, int epilogue, const void* x, const void* w, const float* bias, void* c,
                float* parts, int m, int n, int k, long ldx, long ldc, int slices, int waves);
// pa_gemm_mid's gated product of up to 16 rows with the residual add and RMSNorm in front of it, done as X is staged:
// res_out = x + res (another buffer than res), c = act(gate) * up of rmsnorm(x + res; gain, eps) W^T.
int pa_gemm_mid_normed(void* stream, int epilogue, const void* x, const void* res, const float* gain, float eps,
                       void* res_out, const void* w, void* c, int m, int n, int k, long ldx, long ldc, int waves);
// C = X W^T for any number of rows from the weight in tiles, the output tiled both ways (gemm_tall.hip): 16 mt rows
// of X by 64 nt rows of W a workgroup (mt, nt = 0, 0: the launcher's choice, what pa_gemm_tall_shape puts into
// out[0], out[1]).  epilogue 0: C (+ bias) in bfloat16; 1: C[m, n/2] = silu(gate) * up.  slices > 1 (epilogue 0): parts
// [slices, m, n] as pa_gemm_mid leaves them, c not written.
void pa_gemm_tall_shape(int m, int n, int k, int slices, int* out);
int pa_gemm_tall(void* stream, int epilogue, const void* x, const void* w, const float* bias, void* c, float* parts,
                 int m, int n, int k, long ldx, long ldc, int slices, int mt, int nt);
// out[i] = parts[0, i] + parts[1, i] + ..; out_dtype 0 = float32, 1 = bfloat16; total = rows * columns.
int pa_sum_slices(void* stream, int out_dtype, const float* parts, void* out, int slices, long total);
// out[tile][step][half][g][r][8] = w[16 tile + r][64 step + 16 g + 8 half ..], zero-padded: ceil(n/16) * ceil(k/64) * 1024 elements.
int pa_pack_tiles(void* stream, const void* w, void* out, int n, int k);

// Paged causal attention, one query token per (seq_of_token[t], positions[t]); window 0 = all keys.
// softcap (here and in the matrix-core entry points): 0 = none; > 0 bends every scaled score to
// softcap * tanh(score / softcap) before the softmax.
int pa_attn_generic(void* stream, int dtype, const void* q, const void* k_cache, const void* v_cache,
                    const int* block_table, int table_stride, const int* seq_of_token, const int* positions, void* out,
                    int tokens, int nh, int nkv, int hd, int page_size, int window, float scale, float softcap);

// pa_attn_generic with a sink per head (sink [nh], 32-bit, in the units of the scaled scores): the softmax divides
// by sum_j exp(s_j) + exp(sink_h).
int pa_attn_generic_sink(void* stream, int dtype, const void* q, const void* k_cache, const void* v_cache,
                         const int* block_table, int table_stride, const int* seq_of_token, const int* positions, void* out,
                         int tokens, int nh, int nkv, int hd, int page_size, int window, float scale, float softcap,
                         const float* sink);

// Matrix-core attention in bfloat16 (K cache [page, nkv, page_size, hd], V cache [page, nkv, hd, page_size]).
// seq_ids lists the sequences of the step a call handles; cu_q[s] is the first packed token row of sequence s,
// context_lens[s] its tokens in the cache after the step.  Decode takes sequences that feed one token and cuts
// each one's keys into splits of split_keys; workspace must hold pa_attn_decode_workspace(...) floats.
// The two decode entry points take seq_ids = null for the sequences 0 .. nseq - 1 (a step of single tokens only).
int pa_attn_mfma_supports(int hd, int page_size);
long pa_attn_decode_workspace(int nseq, int nh, int hd, int max_splits);
int pa_attn_decode(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                   int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                   float* workspace, int nseq, int nh, int nkv, int hd, int page_size, int window, float scale,
                   float softcap, int split_keys, int max_splits);
// pa_qknorm_rope_kv + pa_attn_decode in one kernel for steps of single tokens: takes the merged projection,
// norms and rotates the queries in place of loading them, and writes each token's key and value first.
int pa_attn_decode_fused(void* stream, const void* qkv, const float* q_weight, const float* k_weight,
                         const float* cos_table, const float* sin_table, const int* slots, float eps,
                         void* kc, void* vc, const int* block_table, int table_stride, const int* seq_ids, const int* cu_q,
                         const int* context_lens, void* out, float* workspace, int nseq, int nh, int nkv, int hd,
                         int page_size, int window, float scale, float softcap, int split_keys, int max_splits);
int pa_attn_decode_fused_supports(int nh, int nkv, int hd, int rot, int page_size);
int pa_attn_prefill(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                    int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                    int nseq, int max_q_len, int min_prefix, int nh, int nkv, int hd, int page_size, int window,
                    float scale, float softcap);
// pa_attn_decode and pa_attn_prefill with a sink per head (sink [nh], 32-bit, in the units of the scaled scores; null:
// none): a head's softmax divides by sum_j exp(s_j) + exp(sink_h).
int pa_attn_decode_sink(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                        int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                        float* workspace, int nseq, int nh, int nkv, int hd, int page_size, int window, float scale,
                        float softcap, const float* sink, int split_keys, int max_splits);
int pa_attn_prefill_sink(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                         int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                         int nseq, int max_q_len, int min_prefix, int nh, int nkv, int hd, int page_size, int window,
                         float scale, float softcap, const float* sink);
// min_prefix: the fewest keys any sequence has before its portion (0 if unknown), a hint for the cut of the work.
// The same with the cut of the work given (for tests and measurements): tiles in pairs, heads a wavefront (1, 2, 4),
// head groups a workgroup (1, 2), keys staged in LDS; -1 leaves one to the launcher.
int pa_attn_prefill_cut(void* stream, const void* q, const void* kc, const void* vc, const int* block_table,
                        int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                        int nseq, int max_q_len, int min_prefix, int nh, int nkv, int hd, int page_size, int window,
                        float scale, float softcap, int paired, int heads, int groups, int staged);

// out[r] = index of the largest of logits[r, :], the lowest index among equals.
// scratch: pa_argmax_scratch(rows, vocab) floats (none for narrow rows).
int pa_argmax_scratch(int rows, int vocab);
int pa_argmax(void* stream, const float* logits, int* out, float* scratch, int rows, int vocab);
// pa_argmax without a scratch argument and without any allocation, for callers that cannot allocate (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
// reference.  The candidates of wide rows go to an array inside the library, pa_argmax_static_capacity() floats
// (65,536 = 256 KB) on every GPU the library runs on, held until the process ends; rows * ceil(vocab / 2048) * 2
// must fit it (64 rows of 151,936 entries take 9,600), else the call is refused.  The first call on a GPU looks
// up where that GPU's copy lies (make it before a capture begins).  Nothing in the array has to be cleared between
// calls: what the second launch reads the first has written.  All calls on a GPU share the one array: calls
// that overlap there (two streams, two threads) race, calls in order on one stream do not.
int pa_argmax_static_capacity();
int pa_argmax_static(void* stream, const float* logits, int* out, int rows, int vocab);

// Per row: temperature < 1e-7 -> argmax; else a draw from softmax(logits / T) kept to the top_k largest
// (0 = all) and to the shortest descending prefix of mass top_p (>= 1 = all), at the uniform number uniform[r] in [0, 1).
int pa_sample(void* stream, const float* logits, const float* temperature, const int* top_k, const float* top_p,
              const float* uniform, int* out, int rows, int vocab);
// The same choice for long rows with every pass spread over the chip; modes: bit 0 some row may have a top-k,
// bit 1 some row may have a top-p.  workspace: pa_sample_wide_workspace(rows, vocab) bytes, 16-byte aligned.
long pa_sample_wide_workspace(int rows, int vocab);
// lp[r] = logits[r, ids[r]] - logsumexp(logits[r]) (0 where ids[r] < 0); for k > 0 also the entries among the row's
// k largest with their log-probabilities, ties at the k-th value included, unsorted, at most cap a row:
// top_v / top_i [rows, cap], count [rows].
int pa_logprobs(void* stream, const float* logits, const int* ids, float* lp, float* top_v, int* top_i, int* count,
                int rows, int vocab, int k, int cap);
int pa_sample_wide(void* stream, const float* logits, const float* temperature, const int* top_k, const float* top_p,
                   const float* uniform, int* out, void* workspace, int rows, int vocab, int modes);

// ---- a residual stream kept in 32-bit; activations the gated epilogues do not have (rowwise_wide.hip) ----
// RMSNorm of x (+ residual): the residual is 32-bit and receives the unrounded sum (unless `rows`); x and out are of
// `dtype`; x may be given as `slices` 32-bit partial sums [slices, rows, hidden] instead (then x is null).
int pa_rmsnorm_wide(void* stream, int dtype, const void* x, const float* parts, int slices, long slice_stride,
                    float* residual, const float* w, void* out, const int* rows, int nrows, int hidden, float eps);
// gate_up [tokens, 2 inter], columns alternating gate_j, up_j -> out [tokens, inter]:
// g = min(g, limit), u = clamp(u, -limit, limit), g * sigmoid(alpha g) * (u + 1)
int pa_clamped_gate(void* stream, int dtype, const void* gate_up, void* out, int tokens, int inter, float limit, float alpha);
// out = max(x, 0)^2
int pa_relu_squared(void* stream, int dtype, const void* x, void* out, long total);

// residual (32-bit) += y * rsqrt(mean(y^2) + eps) * w, y = x (of `dtype`) or `slices` partial sums; copy (or null,
// of `dtype`) receives the new residual rounded: a branch's output normed and added to the stream.
int pa_rmsnorm_branch(void* stream, int dtype, const void* x, const float* parts, int slices, long slice_stride,
                      float* residual, const float* w, void* copy, int nrows, int hidden, float eps);
// out[t, i] = o[t, i] * rsqrt(mean(o[t]^2) + eps) * w[i] * sigmoid(gate[t, i]); o 32-bit, gate and out of `dtype`,
// gate rows gate_stride elements apart.
int pa_gated_rmsnorm(void* stream, int dtype, const float* o, const void* gate, long gate_stride, const float* w, void* out,
                     int nrows, int width, float eps);

// ---- linear attention with a decaying state (lightning.hip) ----
// S_t = decay[h] S_(t-1) + k_t v_t^T, out[t, h, :] = S_t^T q_t; q, k [heads, dim] and v [heads, vdim] of token t at
// qkv[t * ld + q_off / k_off / v_off ..] of `dtype`, passed through act (0 none, 1 SiLU); state [slots, heads, dim,
// vdim] 32-bit; sequence s owns rows cu_q[s] .. cu_q[s + 1] and slot state_slots[s]; out [tokens, heads, vdim] 32-bit.
int pa_lightning_attn(void* stream, int dtype, const void* qkv, long ld, int q_off, int k_off, int v_off, const float* decay,
                      float* state, const int* state_slots, const int* cu_q, float* out, int nseq, int tokens, int heads,
                      int dim, int vdim, int act, int max_len, int min_len);
// The same for the step's sequences of exactly one token (a small kernel for decode steps; the same bits); with
// min_len 2 above the two together cover a step.
int pa_lightning_step(void* stream, int dtype, const void* qkv, long ld, int q_off, int k_off, int v_off, const float* decay,
                      float* state, const int* state_slots, const int* cu_q, float* out, int nseq, int heads, int dim,
                      int vdim, int act);
// max_len > 0 above: sequences of more tokens are left alone, for the call below (min_len: shorter ones too).  The sequences seq_ids[0 .. nlisted)
// with more than `chunk` tokens (a multiple of 16 up to 256; at most max_len each) in chunks that the whole chip
// works on at once: three passes (each chunk from a zero state, the states chained in order, what came before a chunk
// added).  work: pa_lightning_attn_workspace(...) 32-bit words.
long pa_lightning_attn_workspace(int nlisted, int tokens, int heads, int dim, int vdim, int chunk);
int pa_lightning_attn_chunked(void* stream, int dtype, const void* qkv, long ld, int q_off, int k_off, int v_off,
                              const float* decay, float* state, const int* state_slots, const int* cu_q, const int* seq_ids,
                              float* out, float* work, int nlisted, int tokens, int max_len, int heads, int dim, int vdim,
                              int act, int chunk);

// ---- attention through a latent (latent.hip) ----
// in [tokens, q_rank + rank + rot]: cq_out [tokens, q_rank] = RMSNorm(first part) * wq; into the cache row slots[t]
// ([rank + rot] elements a token): RMSNorm(second part) * wc, then the third part with its first rot_dims elements
// rotated in pairs (2i, 2i+1) by the angle position * inv_freq[i].  slots null: nothing is cached.  cache_t (or null):
// [pages, rank, page_size], the normed latent once more with the token's offset in its page running fastest.
int pa_latent_prep(void* stream, int dtype, const void* in, const float* wq, const float* wc, const float* inv_freq,
                   const int* positions, const int* slots, void* cq_out, void* cache, void* cache_t, int page_size,
                   int tokens, int q_rank, int rank, int rot, int rot_dims, float eps, long in_stride);
// out [rows, rank] = the first `rank` elements of the cached vectors [pages, page, width] at (seq[i], pos[i]) through the
// block table: latents back out of their pages, for a product over them.
int pa_latent_gather(void* stream, int dtype, const void* cache, const int* block_table, int table_stride, const int* seq,
                     const int* pos, void* out, int rows, int rank, int width, int page_size);
// in [tokens, heads, in_stride] -> out [tokens, heads, out_stride]: `width` elements from in_off to out_off of every
// head, the first rot_dims of them rotated in pairs
int pa_rotate_pairs(void* stream, int dtype, const void* in, void* out, const float* inv_freq, const int* positions,
                    int tokens, int heads, int in_stride, int in_off, int out_stride, int out_off, int width, int rot_dims);
// y[t, h, n] = sum_k x[t, h, k] wt[h, k, n]; strides in elements
int pa_head_linear(void* stream, int dtype, const void* x, const void* wt, void* y, int tokens, int heads, int K, int N,
                   long xs_t, long xs_h, long ys_t, long ys_h);
// q [tokens, heads, rank + rot], cache [pages, page_size, rank + rot], sink [heads] or null -> out [tokens, heads, rank]
int pa_latent_attn(void* stream, int dtype, const void* q, const void* cache, const float* sink, const int* block_table,
                   int table_stride, const int* seq_of_token, const int* positions, void* out, int tokens, int nh, int rank,
                   int rot, int page_size, int window, float scale);
// The same on the matrix cores (latent_mfma.hip; bfloat16): the sequences seq_ids[0..n_seqs) (null: 0..n_seqs) with
// cu_q[s+1] - cu_q[s] tokens each (at most max_q_len) ending at context_lens[s].  n_splits > 1, for sequences of one
// token: keys in splits of split_keys, partials in ws (pa_latent_attn_mfma_workspace 32-bit words), merged in split order;
// wave_splits: a split is a wavefront that reads the cache directly (many sequences) instead of a workgroup that stages it.
int pa_latent_attn_mfma_supports(int rank, int rot, int page_size);
long pa_latent_attn_mfma_workspace(int n_seqs, int nh, int rank, int n_splits);
int pa_latent_attn_mfma(void* stream, const void* q, const void* cache, const void* cache_t, const float* sink, const int* block_table,
                        int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out, void* ws,
                        int n_seqs, int max_q_len, int nh, int rank, int rot, int page_size, int window, float scale,
                        int split_keys, int n_splits, int wave_splits);

// ---- experts (moe.hip) ----
int pa_moe_choices_by_table(void* stream, const int* ids, const int* table, int* choice, int tokens, int top, int vocab,
                            int experts);
int pa_moe_order(void* stream, const int* choice, int entries, int experts, int* counts, int* offsets, int* order, int* place);
int pa_moe_linear(void* stream, int x_dtype, int w_dtype, int y_dtype, const void* x, const void* wt, void* y,
                  const int* offsets, const int* order, int entries, int experts, int top, int K, int N, int from_tokens,
                  int act);
// out[t] = (base_scale ? base_scale[t] : 1) * base[t] + sum_j w[t, j] * y[place[t * top + j]]
// With `into` (a 32-bit stream [tokens, width]): into[t] += other[t] (or null) + that sum, unrounded, and nothing goes to out.
int pa_moe_combine(void* stream, int dtype, const float* y, const int* place, const float* weights, float weight,
                   const void* base, const float* base_scale, void* out, int tokens, int top, int width, float* into,
                   const void* other);
// A router: logits [tokens, ld] (32-bit; the first `experts` columns), s = softmax(logits); the `top` experts with the
// largest s + correction[e] (correction null: none) -> choice [tokens, top]; weights [tokens, top] = their s over the
// sum of the chosen s (+ 1e-20), times scale.  gate_out (or null) [tokens] = sigmoid(logits[t, gate_col]), a gate a
// token for a shared expert, from one more column of the same product.
// bias (or null) [experts] is added to the logits first.  by_logit: the choice goes by the logits themselves (+ bias; no
// correction) and the weights are the softmax over the chosen logits alone, times scale.
int pa_moe_route(void* stream, const float* logits, int ld, const float* correction, int* choice, float* weights,
                 float* gate_out, int tokens, int experts, int top, float scale, int gate_col, const float* bias, int by_logit);
// The same two products on the matrix cores (grouped_mfma.hip; bfloat16 operands, K a multiple of 8): the weight as
// stored, [group, N, K].
// act 2 (here only): the weight's rows alternate gate_j, up_j and y [entries, N / 2] receives the clamped gated pair
// g * sigmoid(alpha g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit).  act 3: the same rows, the
// plain gated pair silu(gate) * up.
int pa_moe_linear_mfma(void* stream, int y_dtype, const void* x, const void* w, void* y, const int* offsets, const int* order,
                       int entries, int experts, int top, int K, int N, int from_tokens, int act, float limit, float alpha);
int pa_head_linear_mfma(void* stream, const void* x, const void* w, void* y, int tokens, int heads, int K, int N, long xs_t,
                        long xs_h, long ys_t, long ys_h);

// ---- statistics over parts of a row (rowwise_groups.hip) ----
// Around a 32-bit stream: with y, residual[r] += norm_g(y[r]) * w_add; with out, out[r] = norm_g(residual[row]) * w_out
// (row = rows[r] when rows is given, which goes without y).  norm_g: the row in `groups` equal consecutive parts, each
// over its own sqrt(mean(part^2) + eps).
int pa_group_norm_step(void* stream, int dtype, const void* y, const float* w_add, float* residual, const float* w_out,
                       void* out, const int* rows, int nrows, int hidden, int groups, float eps);
// out = a N(z) + b N(z^2) + c N(z^3) + e, z = x (+ bias), N(u) = u / sqrt(mean(u^2) + eps) over the row; coeff (a, b, c, e).
int pa_poly_norm(void* stream, int dtype, const void* x, const float* bias, const float* coeff, void* out, int nrows,
                 int width, float eps);
// out[r, h, :] = o[r, h, :] / sqrt(mean(o[r, h, :]^2) + eps) * w (null: none; vdim elements shared by the heads)
//                * act(gate[r, h, :]) * scale;  act 0 sigmoid, 1 silu.
int pa_head_norm_gate(void* stream, int dtype, const float* o, const void* gate, long gate_stride, const float* w, void* out,
                      long out_stride, int nrows, int heads, int vdim, float eps, int act, float scale);

// ---- attention with a window that keeps first tokens, a bias by distance, a gate a head (attention_masked.hip) ----
int pa_attn_masked(void* stream, int dtype, const void* q, const void* k_cache, const void* v_cache, const int* block_table,
                   int table_stride, const int* seq_of_token, const int* positions, void* out, long out_stride, int tokens,
                   int nh, int nkv, int hd, int vd, int page_size, int window, int keep_first, float scale, float softcap,
                   const float* slopes, const float* sink, const void* gate, long gate_stride, float out_scale, const int* cu_q,
                   const int* context_lens, int nseq, int max_q_len, int nv);
int pa_attn_masked_mfma_supports(int hd, int vd, int page_size);
int pa_qkv_prepare(void* stream, int dtype, const void* p, long stride, int q_off, int k_off, int v_off, const float* qw,
                   const float* kw, const int* slots, void* q_out, void* k_cache, void* v_cache, int tokens, int nh, int nkv,
                   int hd, int vd, int page_size, float eps);

// ---- the gated delta rule and what stands in front of a recurrence (delta_rule.hip) ----
int pa_delta_prepare(void* stream, int dtype, const void* p, long stride, int off, int b_off, const float* w, int taps,
                     float* conv_state, const int* seq_of_token, const int* cu_q, const int* state_slots, const void* a,
                     long a_stride, int a_off, const float* a_log, const float* dt_bias, float* out, float* decay, float* beta,
                     int tokens, int nseq, int heads, int kvh, int d, int e);
int pa_gated_delta(void* stream, const float* x, const float* decay, const float* beta, float* state, const int* state_slots,
                   const int* cu_q, float* out, int nseq, int heads, int kvh, int d, int e);
int pa_rotate_halves_f32(void* stream, int dtype, const void* p, long stride, int q_off, int k_off, int v_off,
                         const float* inv_freq, const int* positions, float* out, int tokens, int heads, int d, int e, int rot,
                         float k_scale);

// ---- parts around a 32-bit stream, in front of and behind attention (stream_parts.hip) ----
int pa_pair_embed(void* stream, int dtype, const int* ids, const int* positions, const int* seq_of_token, const int* cu_q,
                  const int* state_slots, int* prev_state, const void* table, const void* pair, float* out, int tokens,
                  int hidden, int vocab, int buckets, long mul_prev, long mul_cur, float scale);
int pa_time_conv_add(void* stream, int dtype, const void* h, const float* w, float* state, const int* seq_of_token,
                     const int* cu_q, const int* state_slots, void* out, int tokens, int nseq, int channels, int taps,
                     int all_single);
int pa_stream_add_row(void* stream, float* x, const float* row, int tokens, int hidden);
int pa_stream_add_branches(void* stream, int dtype, float* x, const void* a, const void* b, long total);
int pa_qkv_rope_prepare(void* stream, int dtype, const void* p, long stride, int q_off, int k_off, int v_off,
                        const float* inv_freq, const int* positions, const int* slots, const float* q_scale, void* q_out,
                        void* k_cache, void* v_cache, int tokens, int nq, int nk, int nv, int hd, int vd, int rot, int pairs,
                        int page_size);
int pa_diff_combine(void* stream, int dtype, const void* a, void* out, int tokens, int heads, int vd, float lambda, float eps,
                    float scale);
int pa_sigmoid_gate(void* stream, int dtype, const void* o, long o_stride, const void* gate, long gate_stride, void* out,
                    int rows, int width);
int pa_cap_logits(void* stream, float* x, long total, float cap);

#ifdef __cplusplus
}
#endif
