// C entry points of the gfx950 kernel library. Every pointer is device memory
// unless named host_*. Every entry validates its sizes, launches on `stream`
// and returns IMPARO_OK (0), IMPARO_BAD_ARGUMENT (1, nothing launched) or
// IMPARO_LAUNCH_FAILED (2). dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* imparo_stream;

// The hash of the sources this library was built from, as the build computed it.
const char* imparo_hip_source_hash();

// Loads the code of every kernel file onto the current device. The runtime would load each file's
// code when one of its kernels is first launched, which a stream under graph capture cannot do: call
// this once per device before the first capture.
int imparo_load_code(void);

// x[t, :] = table[ids[t], :] as float32.
int imparo_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* x,
                        int n_tokens, int width, int vocab, imparo_stream stream);

// ids[dst[i]] = src[src_index[i]] for i < n, clamped into [0, vocab): token ids sampled by the
// step before that are still on the device. The caller guarantees dst[i] < len(ids) and
// src_index[i] < len(src).
int imparo_place_tokens(int32_t* ids, const int32_t* dst, const int32_t* src, const int32_t* src_index,
                        int n, int vocab, imparo_stream stream);

// Row-wise RMS norm. For output row i the source row is rows ? rows[i] : i.
// If delta is given the row is x + delta[0] + delta[1] + ... first (n_delta
// slices, each [n_x_rows, width], added in order); with write_back (rows must
// be null) the sum is stored to x. out[i, :] = v * rsqrt(mean(v^2) + eps) * weight.
int imparo_rms_norm(float* x, const float* delta, int n_delta, int n_x_rows, const int32_t* rows, const float* weight,
                    void* out, int out_dtype, int n_rows, int width, float eps, int write_back,
                    imparo_stream stream);

// Y[m, n] = X[m, k] . W[n, k]^T (+ bias[n], float32, may be null), float32
// accumulate. X and W share `dtype`. epilogue 0: Y is [m, n]. epilogue 1
// (SwiGLU): W's rows alternate gate, up; Y is [m, n/2] with
// Y[m, j] = silu(y[m, 2j]) * y[m, 2j+1].
// `slices` > 1 (only the number imparo_gemm_slices gives, float32 out, epilogue 0): K is cut into
// that many slices and Y is [slices, m, n], slice s holding the sum over its part of K (the bias
// in slice 0); the consumer adds the slices in order.
int imparo_gemm(const void* x, const void* w, const float* bias, void* y, int dtype, int out_dtype,
                int m, int n, int k, int epilogue, int slices, imparo_stream stream);
int imparo_gemm_slices(int m, int n, int k, int dtype);
// epilogue 2 (float32 out, `slices` 1): Y[m, n] += the product (+ bias), each element of Y read where it
// is stored. Only for shapes for which imparo_gemm_adds gives 1 (many rows, a K the tile kernel takes).
int imparo_gemm_adds(int m, int n, int k, int dtype);
// imparo_gemm with the kernel named by the caller instead of chosen by the library: for tests and
// measurements, so that every kernel can be met at any shape (the numbers are listed in gemm.hip).
// Nothing in the library keeps the choice: it is this call's argument.
int imparo_gemm_variant(const void* x, const void* w, const float* bias, void* y, int dtype, int out_dtype,
                        int m, int n, int k, int epilogue, int slices, int variant, imparo_stream stream);

// Per (token, head): RMS norm over the head (weight null: none), NeoX rotation
// with angles pos * inv_freq[i] over the first 2*n_freq dims (n_freq 0: none): pair i is dims
// (i, i + n_freq), or with `interleaved` dims (2i, 2i + 1).
// qkv is float32 [n_tokens, (heads + 2*kv_heads) * head_dim]; q goes to q_out
// [n_tokens, heads, head_dim], k and v into the paged cache at each token's
// position: page = table[row_of_token[t] * table_stride + pos / page_size].
// Cache layout [n_pages, kv_heads, page_size, head_dim]; with v_transposed the V
// cache is [n_pages, kv_heads, head_dim, page_size]. write_kv 0 skips the cache.
int imparo_qk_norm_rope_store(const float* qkv, const float* q_weight, const float* k_weight, float eps,
                              const float* inv_freq, int n_freq, int interleaved,
                              const int32_t* positions, const int32_t* row_of_token,
                              const int32_t* block_table, int table_stride, int page_size,
                              void* q_out, void* k_cache, void* v_cache, int dtype, int write_kv,
                              int n_tokens, int heads, int kv_heads, int head_dim, int n_pages,
                              int v_transposed, imparo_stream stream);

// Causal grouped-query attention over the paged cache; one query per (token,
// head); keys lo..pos with lo = max(0, pos + 1 - window) (window 0: all keys; window < 0: the keys of the query's
// own chunk, lo = pos - pos % -window; the matrix-core attention kernels below read `window` the same way).
int imparo_attention(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                     const int32_t* positions, const int32_t* row_of_token,
                     const int32_t* block_table, int table_stride, int page_size,
                     int n_tokens, int heads, int kv_heads, int head_dim, int n_pages,
                     float scale, int window, int v_transposed, imparo_stream stream);

// imparo_attention_decode and imparo_attention_prefill (below) with the softmax weights kept to float32
// through the product with the values: a weight goes in as its bfloat16 rounding plus, through a second
// product, the bfloat16 rounding of what that took off (16 bits of mantissa and more), and the
// denominator sums the weights as they are. Same arguments.
int imparo_attention_decode_exact(const void* q, const void* k_cache, const void* v_cache, void* out,
                                  float* part_o, float* part_ml, const int32_t* rows, int n_rows,
                                  const int32_t* seg_start, const int32_t* positions,
                                  const int32_t* block_table, int table_stride, int page_size,
                                  int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                                  int n_splits, imparo_stream stream);
int imparo_attention_prefill_exact(const void* q, const void* k_cache, const void* v_cache, void* out,
                                   float* part_o, float* part_ml, int n_splits,
                                   const int32_t* rows, int n_rows, int n_tiles,
                                   const int32_t* seg_start, const int32_t* seg_len, const int32_t* positions,
                                   const int32_t* block_table, int table_stride, int page_size,
                                   int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                                   imparo_stream stream);

// The two above for heads whose values have another size than their keys (value_dim): a token's row is
// heads + kv_heads units of head_dim, then kv_heads units of value_dim; the value cache holds value_dim a
// position and out is [tokens, out_ld >= heads * value_dim] (the rest of a row zeros); any head_dim up to 512. The store also takes rows of
// queries only (kv_heads 0, write_kv 0), for a layer that reads another layer's keys and values.
int imparo_qk_norm_rope_store_dv(const float* qkv, const float* q_weight, const float* k_weight, float eps,
                                 const float* inv_freq, int n_freq, int interleaved,
                                 const int32_t* positions, const int32_t* row_of_token,
                                 const int32_t* block_table, int table_stride, int page_size,
                                 void* q_out, void* k_cache, void* v_cache, int dtype, int write_kv,
                                 int n_tokens, int heads, int kv_heads, int head_dim, int value_dim, int n_pages,
                                 int v_transposed, imparo_stream stream);
int imparo_attention_dv(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                        const int32_t* positions, const int32_t* row_of_token,
                        const int32_t* block_table, int table_stride, int page_size,
                        int n_tokens, int heads, int kv_heads, int head_dim, int value_dim, int out_ld, int n_pages,
                        float scale, int window, int v_transposed, imparo_stream stream);

// ---- attention over a cached latent (absorbed form)
// Attention in which every head reads the same cached rows [pages, page, row_dim]: a key is a whole row, its value
// the row's first value_dim numbers. q [tokens, heads, row_dim], out [tokens, heads * value_dim].
int imparo_attention_latent(const void* q, const void* rows_cache, void* out, int dtype, const int32_t* positions,
                            const int32_t* row_of_token, const int32_t* block_table, int table_stride, int page_size,
                            int n_tokens, int heads, int row_dim, int value_dim, int n_pages, float scale, int window,
                            imparo_stream stream);
// Per token: the first `rank` numbers of kv_rows [tokens, rank + rot_dim] are divided by their root mean square
// (eps inside the root) and multiplied by norm_weight; the last rot_dim are turned by position (the first
// 2 n_freq of them; pair i is (i, i + n_freq), or with `interleaved` (2i, 2i + 1); angle = position *
// inv_freq[i]); the row goes to the token's place in `cache` [pages, page, rank + rot_dim] (cache null: not
// written). q_rows [tokens, heads * (dim + rot_dim)]: each head's first dim numbers go to q_plain [tokens, heads,
// dim], its last rot_dim, turned alike, to columns rank .. of q_full [tokens, heads, rank + rot_dim].
int imparo_latent_store(const float* q_rows, const float* kv_rows, const float* norm_weight, float eps,
                        const float* inv_freq, int n_freq, int interleaved, const int32_t* positions,
                        const int32_t* row_of_token, const int32_t* block_table, int table_stride, int page_size,
                        int n_pages, void* cache, void* cache_t, void* q_plain, void* q_full, int dtype, int n_tokens,
                        int heads, int dim, int rot_dim, int rank, imparo_stream stream);
// (cache_t, or null: the normed latent once more at [pages, rank, page], for the matrix-core kernel below.)
// The matrix-core form of imparo_attention_latent, bfloat16: up to 16 heads of a token are the 16 queries of a
// wave's products. rows_t [pages, rank, page] holds the latents transposed inside a page; the values are the
// latents (value_dim = rank). `_takes`: whether it is built for these sizes. `_split`: into how many parts the
// keys are cut for this many tokens (and how many keys a part holds; 1 or a multiple of 4: a block adds the parts
// of its four waves): with n_splits > 4, part_o [tokens, heads, n_splits / 4, rank] and part_ml [tokens, heads,
// n_splits / 4, 2] float32 hold the blocks' sums, merged by a second launch.
// `exact`: a softmax weight enters the product with the values as two bfloat16 numbers.
int imparo_attention_latent_tiles_takes(int row_dim, int rank, int page_size);
int imparo_attention_latent_tiles_split(int n_tokens, int heads, int max_context, int* split_keys);
int imparo_attention_latent_tiles(const void* q, const void* rows, const void* rows_t, void* out, float* part_o,
                                  float* part_ml, const int32_t* positions, const int32_t* row_of_token,
                                  const int32_t* block_table, int table_stride, int page_size, int n_pages,
                                  int n_tokens, int heads, int row_dim, int rank, float scale, int window,
                                  int split_keys, int n_splits, int exact, imparo_stream stream);
// out[t, h, :n] = W[h] in[t, h, :k] with w [heads, k, n]: a token's rows lie in_ld (out_ld) apart, a head's part
// in_hs (out_hs) apart inside a row. float32 sums in the order of k.
int imparo_head_gemm(const void* in, int in_ld, int in_hs, const void* w, int dtype, void* out, int out_dtype,
                     int out_ld, int out_hs, int n_tokens, int heads, int k, int n, imparo_stream stream);

// The same product on the matrix cores: in bfloat16, w_t [heads, n, k] (the inner size running fastest) bfloat16,
// out bfloat16 or float32; k, in_ld and in_hs multiples of 8.
int imparo_head_gemm_tiles(const void* in, int in_ld, int in_hs, const void* w_t, void* out, int out_dtype, int out_ld,
                           int out_hs, int n_tokens, int heads, int k, int n, imparo_stream stream);

// ---- a gated linear recurrence with a matrix of state a head
// Per request (row), head and token in order: q = silu(zq), f = lower + (1 - lower) sigmoid(zf),
// S <- diag(f) S + (1 - f) v^T, out = S^T q. rows [tokens, ld] float32 holds zq at q_off, zf at f_off, v at v_off,
// head by head; state [slots, heads, dim, vdim] float32; out [tokens, heads * vdim] float32. dim <= 512.
// chunk_tokens 0: one launch, a block walks a row's whole segment. Otherwise (a multiple of 8) segments are walked
// in chunks of that many tokens side by side, in three launches; max_chunks >= ceil(longest segment /
// chunk_tokens); chunk_state [n_rows * max_chunks, heads, dim, vdim] and chunk_decay [n_rows * max_chunks, heads,
// dim] float32 are scratch.
int imparo_hgrn2_scan(const float* rows, int ld, int q_off, int f_off, int v_off, const float* lower, float* state,
                      const int32_t* seg_start, const int32_t* seg_len, const int32_t* slot, float* out, int n_rows,
                      int heads, int dim, int vdim, int chunk_tokens, int max_chunks, float* chunk_state,
                      float* chunk_decay, imparo_stream stream);

// ---- recurrences with a matrix of state a head and one decay a head and token
// Per request (row), head and token in order:  S <- a S + k v^T, out = S^T q;  with `beta` the gated delta rule
// S <- a S, u = sigmoid(beta) (v - S^T k), S <- S + k u^T, out = S^T q. q, k, v are float32 rows (a token's row ld
// floats apart, heads from off on; head h reads q head h / q_div and k head h / k_div). a = decay_const[h], or
// exp(-rate[h] softplus(step[t, h] + step_bias[h])); with v_times_step v is multiplied by that softplus; with
// `skip`, out += skip[h] v (v as it came). state [slots, heads, dim, vdim] float32; out [tokens, heads * vdim]
// float32. dim <= 512. chunk_tokens 0: one launch. Otherwise (a multiple of 8; without beta) segments are walked
// in chunks side by side, in three launches; max_chunks >= ceil(longest segment / chunk_tokens); chunk_state
// [n_rows * max_chunks, heads, dim, vdim] and chunk_decay [n_rows * max_chunks, heads] float32 are scratch.
// chunk_tokens = imparo_delta_chunk_tokens() (dim at most imparo_delta_chunk_max_dim()): a segment's chunks in order,
// small products a chunk, two launches, with or without beta; chunk_state then holds [n_rows * max_chunks, heads, 2,
// chunk, chunk] floats and chunk_decay [n_rows * max_chunks, heads, 2, chunk]. With beta chunk_tokens is that or 0.
int imparo_delta_chunk_tokens(void);
int imparo_delta_chunk_max_dim(void);
int imparo_decay_scan(const float* q, int q_ld, int q_off, int q_div, const float* k, int k_ld, int k_off, int k_div,
                      const float* v, int v_ld, int v_off, const float* decay_const, const float* step, int step_ld,
                      int step_off, const float* step_bias, const float* rate, int v_times_step, const float* beta,
                      int beta_ld, int beta_off, const float* skip, float* state, const int32_t* seg_start,
                      const int32_t* seg_len, const int32_t* slot, float* out, int n_rows, int heads, int dim, int vdim,
                      int chunk_tokens, int max_chunks, float* chunk_state, float* chunk_decay, imparo_stream stream);
// Heads of `dim` columns from `off` on in float32 rows, in place: divided by sqrt(sum of squares + unit_eps) if
// `unit`, the first 2 n_freq dimensions rotated by position (pairs (i, i + n_freq), or neighbours if interleaved),
// multiplied by scale_first (heads below n_first) or scale_rest.
int imparo_head_prepare(float* rows, int ld, int off, int n_tokens, int heads, int dim, int unit, float unit_eps,
                        const float* inv_freq, int n_freq, int interleaved, const int32_t* positions, int n_first,
                        float scale_first, float scale_rest, imparo_stream stream);
// A row of `width` float32 values in `groups` equal parts, with g = silu(gate[t, gate_off + c]) (gate null: 1):
// gate_first: (x g) / rms_part(x g) * w; otherwise x / rms_part(x) * w * g (w null: 1).
int imparo_gated_group_norm(const float* x, const float* gate, int gate_ld, int gate_off, const float* w, void* out,
                            int out_dtype, int n_tokens, int width, int groups, float eps, int gate_first,
                            imparo_stream stream);
// out[t, j] = g sigmoid(alpha g) (u + 1), g = min(gu[t, j], limit), u = clamp(gu[t, hidden + j], -limit, limit);
// columns from `hidden` to out_ld are zero.
int imparo_clamped_glu(const float* gu, void* out, int out_dtype, int n_tokens, int hidden, int out_ld, float limit,
                       float alpha, imparo_stream stream);
// out[t] = factor (rms_norm(a[t]) wa + rms_norm(b[t]) wb); a and b float32 [slices, tokens, width], added in order.
int imparo_normed_sum(const float* a, int a_slices, const float* wa, const float* b, int b_slices, const float* wb,
                      float* out, int n_tokens, int width, float eps, float factor, imparo_stream stream);
// out[t] += sigmoid(z[t, z_col]) * (the sum of y's slices)[t].
int imparo_gated_row_add(float* out, const float* y, int y_slices, const float* z, int z_ld, int z_col, int n_tokens,
                         int width, imparo_stream stream);

// ---- pieces of a parallel block with gated sublayers
// x += a * sigmoid(gates[:, :width]) (+ b * sigmoid(gates[:, width : 2 width]), b may be null); with `copy`
// the new x is also stored there in copy_dtype. x float32 [tokens, width]; a and b float32 [slices, tokens, width],
// their slices added in order; gates float32 [tokens, gate_ld].
int imparo_gated_sum(float* x, const float* a, int a_slices, const float* b, int b_slices, const float* gates,
                     int gate_ld, void* copy, int copy_dtype, int n_tokens, int width, imparo_stream stream);
// out[t, j] = gelu_tanh(z[t, j]) * table[ids[t], offset + j] for j < dim, zero for dim <= j < out_ld.
int imparo_side_gate(const float* z, const void* table, int table_dtype, int table_ld, int offset, const int32_t* ids,
                     int vocab, void* out, int out_dtype, int n_tokens, int dim, int out_ld, imparo_stream stream);
// x[i] += y[i] for i < n.
int imparo_add_rows(float* x, const float* y, long long n, imparo_stream stream);
// out[i] = x[rows ? rows[i] : i] in out_dtype: float32 rows as a product reads them (rows null: all n_out rows).
int imparo_cast_rows(const float* x, const int32_t* rows, void* out, int out_dtype, int n_out, int width,
                     imparo_stream stream);

// Matrix-core attention, bfloat16, V cache transposed, page_size a power of two
// >= 16, head_dim a multiple of 16 up to 128.
// Decode: one query token per listed row (rows[i] indexes seg_start); the key
// range is split in pieces of 256 keys whose partial results go through
// part_o [n_rows, heads, n_splits, head_dim] and part_ml [n_rows, heads,
// n_splits, 2]; n_splits >= ceil(longest context / 256).
int imparo_attention_decode_split(void);      // keys per split
int imparo_attention_prefill_tile(void);      // queries per tile that n_tiles counts
int imparo_attention_decode(const void* q, const void* k_cache, const void* v_cache, void* out,
                            float* part_o, float* part_ml, const int32_t* rows, int n_rows,
                            const int32_t* seg_start, const int32_t* positions,
                            const int32_t* block_table, int table_stride, int page_size,
                            int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                            int n_splits, imparo_stream stream);

// The same for a step whose rows' keys and values are not in the cache yet: qkv is the fused
// projection's float32 rows [tokens, (heads + 2 kv_heads) x head_dim] (q heads, k heads, v heads). The
// launch norms each head of q and k (weights [head_dim], or both null: no norm), rotates them
// (inv_freq [n_freq] with 2 n_freq = head_dim, pairs (i, i + n_freq) or with `interleaved`
// (2i, 2i + 1); n_freq 0: no rotation), attends over the cached keys before each row's position and
// the new key, and with write_kv puts the new key and value into their page (V pages transposed).
// It replaces imparo_qk_norm_rope_store + imparo_attention_decode for such a step, in one launch less.
// Head sizes 64 and 128 (imparo_attention_decode_qkv_takes); a layer that reads another layer's cache
// finds the row's key there already and takes the two-launch form.
int imparo_attention_decode_qkv_takes(int head_dim, int n_freq);
int imparo_attention_decode_qkv_pays(int n_rows, int n_splits);   // few rows over not too many splits: the one launch is the faster way
int imparo_attention_decode_qkv(const float* qkv, const float* q_weight, const float* k_weight, float eps,
                                const float* inv_freq, int n_freq, int interleaved, void* k_cache, void* v_cache,
                                int write_kv, void* out, float* part_o, float* part_ml, const int32_t* rows,
                                int n_rows, const int32_t* seg_start, const int32_t* positions,
                                const int32_t* block_table, int table_stride, int page_size, int heads,
                                int kv_heads, int head_dim, int n_pages, float scale, int window, int n_splits,
                                imparo_stream stream);

// imparo_attention_decode for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the
// reference. The splits' partial results go through a buffer of IMPARO_STATIC_SCRATCH_BYTES that the
// library holds itself on every GPU it runs on (until the process ends) instead of part_o / part_ml;
// the call allocates and frees nothing. rows x heads x n_splits x (head_dim + 2) floats (the first
// part rounded up to 64 floats) must fit, else nothing is launched, a line on stderr says what was
// asked for, and IMPARO_SCRATCH_TOO_SMALL (3) is returned. All calls on one GPU share that GPU's
// buffer: calls that overlap there (two streams, two threads) race; calls on one stream do not.
// The buffer keeps the last call's contents; no call relies on them. The first call on a device
// looks the buffer's address up (no allocation, but not a stream operation: make it outside a capture).
#define IMPARO_STATIC_SCRATCH_BYTES (16u << 20)
int imparo_attention_decode_static(const void* q, const void* k_cache, const void* v_cache, void* out,
                                   const int32_t* rows, int n_rows,
                                   const int32_t* seg_start, const int32_t* positions,
                                   const int32_t* block_table, int table_stride, int page_size,
                                   int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                                   int n_splits, imparo_stream stream);

// Prompt portions: the listed rows' segments in tiles of 64 queries;
// n_tiles = sum over the rows of ceil(seg_len / 64). n_splits (from
// imparo_attention_prefill_splits, or 1) parts of each block's keys, merged by a
// second launch; then part_o holds [tokens, heads, n_splits, head_dim] floats
// and part_ml [tokens, heads, n_splits, 2], tokens counted over the whole batch.
// `max_context` is the bound on the contexts that imparo_attention_prefill itself goes by: what its
// block table can hold, table_stride x page_size (both lay a launch out from that one number).
int imparo_attention_prefill_splits(int n_tiles, int heads, int kv_heads, int head_dim, int max_context);
int imparo_attention_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                             float* part_o, float* part_ml, int n_splits,
                             const int32_t* rows, int n_rows, int n_tiles,
                             const int32_t* seg_start, const int32_t* seg_len, const int32_t* positions,
                             const int32_t* block_table, int table_stride, int page_size,
                             int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                             imparo_stream stream);

// Gated short convolution over each request's segment, continuing from its
// state slot. bcx float32 [n_tokens, 3*width] = [B | C | x]. state float32
// [n_slots, taps-1, width], oldest first. seg_start[r], seg_len[r], slot[r]
// describe request r's tokens in the batch. out[t] = C_t * (sum_k w[ch,k] *
// seq[t+k] + bias[ch]).
int imparo_short_conv(const float* bcx, const float* weight, const float* bias, const float* state,
                      const int32_t* row_of_token, const int32_t* seg_start, const int32_t* slot,
                      void* out, int out_dtype, int n_tokens, int width, int taps, int n_slots, int n_rows,
                      imparo_stream stream);

// The same for a batch in which every request brings exactly one token, output
// and state update in one launch: n_tokens == n_rows, token r belongs to row r.
int imparo_short_conv_decode(const float* bcx, const float* weight, const float* bias, float* state,
                             const int32_t* slot, void* out, int out_dtype, int n_rows, int width, int taps,
                             int n_slots, imparo_stream stream);

// The conv mixer's input projection and imparo_short_conv_decode in one launch, for at most 16
// single-token rows: x [m, k] and w [3 e, k] bfloat16, in_bias [3 e] or null, conv_w [e, taps],
// conv_b [e] or null, slot [m] (distinct). out [m, e]; the state is shifted in place.
int imparo_in_proj_conv_decode(const void* x, const void* w, const float* in_bias, const float* conv_w,
                               const float* conv_b, float* state, const int32_t* slot, void* out, int out_dtype,
                               int m, int e, int k, int taps, int n_slots, imparo_stream stream);

// The same on activations that are the residual stream times a norm's weight, each row still to be
// scaled: ssq_in [n_parts, 16] holds the partial sums of squares of the stream's rows and the launch
// multiplies B, C and x of row r by rsqrt(sum_p ssq_in[p][r] / k + eps). ssq_in null: as above.
int imparo_in_proj_conv_decode_normed(const void* x, const float* ssq_in, int n_parts, float eps, const void* w,
                                      const float* in_bias, const float* conv_w, const float* conv_b, float* state,
                                      const int32_t* slot, void* out, int out_dtype, int m, int e, int k, int taps,
                                      int n_slots, imparo_stream stream);

// Products for a step of at most 16 rows with a norm of the residual stream folded into them
// (decode_rows.hip). x [m, k] and w [n, k] bfloat16, k a multiple of 8, bias float32 [n] or null.
// With ssq_in [n_parts, 16] and eps, x is the stream times a norm's weight, each row still to be
// scaled, and row r's result is multiplied by rsqrt(sum_p ssq_in[p][r] / k + eps) at the end, in float32.
// epilogue 0: y [m, n] in out_dtype; 1: SwiGLU, y [m, n/2] (rows of w alternate gate, up);
// 2: x_io [m, n] float32 += the result, in place, and ssq_out [imparo_rows_parts(n), 16] receives the
// partial sums of squares of the new rows (entries of rows >= m are zero); with weighted_by [n] (the
// weight of the norm that reads the stream next), weighted_out [m, n] bfloat16 receives the new rows
// times it. A block sums the whole of K, in an order that depends on k alone.
int imparo_rows_parts(int n);
int imparo_rows_gemm(const void* x, const float* ssq_in, int n_parts, float eps, const void* w, const float* bias,
                     void* y, int out_dtype, float* x_io, float* ssq_out, void* weighted_out, const float* weighted_by,
                     int m, int n, int k, int epilogue, imparo_stream stream);

// state' = the last taps-1 rows of (state ++ B*x) for every request; runs after
// imparo_short_conv on the same stream.
int imparo_short_conv_state(const float* bcx, float* state, const int32_t* seg_start, const int32_t* seg_len,
                            const int32_t* slot, int n_rows, int n_tokens, int width, int taps, int n_slots,
                            imparo_stream stream);

// out[r] = smallest index of the maximum of logits[r, :]; NaN never wins.
int imparo_argmax_rows(const float* logits, int32_t* out, int n_rows, int vocab, imparo_stream stream);

// out[r] = the first index whose cumulative softmax(logits[r]/temperature[r])
// reaches uniform[r]; temperature <= 0 is argmax.
int imparo_sample_rows(const float* logits, const float* temperature, const float* uniform, int32_t* out,
                       int n_rows, int vocab, imparo_stream stream);

// Fills n float32 values (or n int32 values of the same bits) without a memset node.
int imparo_fill_f32(float* p, float value, int64_t n, imparo_stream stream);

// The fixed-size state of one slot, every site in one launch: for site i, per_slot[i] float32
// values at base[i] (a device address) + slot * per_slot[i] are set to value[i]. base, per_slot
// and value are device arrays of n_sites entries that the caller built from tensors it owns.
int imparo_fill_sites(const uint64_t* base, const int64_t* per_slot, const float* value, int n_sites, int slot,
                      imparo_stream stream);

// ---- row-wise kernels of layers that norm in groups, shift tokens, add a sinusoid or use a polynomial activation
// x[t, 2i] = table[ids[t], 2i] + sin(positions[t] * inv_freq[i]), x[t, 2i + 1] = ... + cos(the same angle).
int imparo_embed_sinusoid(const void* table, int table_dtype, const int32_t* ids, const int32_t* positions,
                          const float* inv_freq, float* x, int n_tokens, int width, int vocab, imparo_stream stream);
// imparo_rms_norm with the row cut into `groups` equal consecutive parts, each divided by its own root mean
// square. With shift_mix [width] (rows of one token each, row i's request in slot[i]; rows must be null):
// out = h + (prev - h) * mix with prev = shift_state[slot[i]], which then becomes h (float32 [slots, width]).
int imparo_group_rms_norm(float* x, const float* delta, int n_delta, int n_x_rows, const int32_t* rows,
                          const float* weight, void* out, int out_dtype, int n_rows, int width, int groups, float eps,
                          int write_back, const float* shift_mix, float* shift_state, const int32_t* slot,
                          imparo_stream stream);
// out[t] = h[t] + (prev - h[t]) * mix, prev the row before inside a request's segment and state[slot] at its
// first token; afterwards state[slot] = the segment's last row of h. h float32 [tokens, width].
int imparo_token_shift(const float* h, const float* mix, float* state, const int32_t* row_of_token,
                       const int32_t* seg_start, const int32_t* seg_len, const int32_t* slot, void* out, int out_dtype,
                       int n_tokens, int n_rows, int width, imparo_stream stream);
// out = a N(z) + b N(z^2) + c N(z^3) + e with N(v) = v / sqrt(mean(v^2) + eps) over a token's `width` values;
// coef = {a, b, c, e} on the device. Columns width .. out_ld of out become zero.
int imparo_poly_norm(const float* z, int z_ld, const float* coef, void* out, int out_dtype, int out_ld, int n_tokens,
                     int width, float eps, imparo_stream stream);

// ---- selective state-space mixer
// y[t, c] = act(bias[c] + sum_k weight[c, k] u[t - (taps - 1) + k, c]) per request, zeros before its start;
// state [slots, taps - 1, channels] float32 holds each request's last inputs and is advanced. u rows lie u_ld
// floats apart. single_tokens: every row brings one token (one launch instead of two).
int imparo_causal_conv(const float* u, int u_ld, const float* weight, const float* bias, float* state,
                       const int32_t* row_of_token, const int32_t* seg_start, const int32_t* seg_len,
                       const int32_t* slot, void* out, int out_dtype, int n_tokens, int n_rows, int channels, int taps,
                       int silu, int single_tokens, imparo_stream stream);
// S[c, n] <- exp(dt A[c, n]) S[c, n] + dt x[c] B[n]; y[c] = sum_n S[c, n] C[n] + D[c] x[c]; out = y * silu(z);
// dt = softplus(dt_raw), taken in place (dt_raw [n_tokens, channels] holds the steps afterwards). bc rows are [B | C] float32; state [slots, channels, n_state] float32. n_chunks 1:
// every segment in one piece; more (at least ceil(longest segment / imparo_selective_scan_chunk())): chunks of a
// segment run side by side through scratch, n_rows * (n_chunks * channels * (n_state + 1) + channels * n_state) floats.
int imparo_selective_scan_chunk(void);
int imparo_selective_scan(float* dt_raw, const void* x, const float* bc, const float* z, int z_ld,
                          const float* A, const float* D, float* state, const int32_t* seg_start,
                          const int32_t* seg_len, const int32_t* slot, void* out, int dtype, float* scratch,
                          int n_chunks, int n_tokens, int n_rows, int channels, int n_state, imparo_stream stream);

// ---- differential attention (two softmax maps a head over shared values)
// rows_in float32 [tokens, ld] = [q: heads x 2 x dim | k: kv_heads x 2 x dim | v: kv_heads x vdim | ...];
// q_out [tokens, heads, 2, dim] = q * (1 + temp_coef * ln(floor((pos + 1) / temp_every) + 1)) (temp_every 0:
// none); with write_kv, k and v go into their pages: K [n_pages, 2 kv_heads, page_size, dim], V [n_pages,
// kv_heads, page_size, vdim].
int imparo_diff_qkv_store(const float* rows_in, int ld, const int32_t* positions, const int32_t* row_of_token,
                          const int32_t* block_table, int table_stride, int page_size, void* q_out, void* k_cache,
                          void* v_cache, int dtype, int write_kv, int n_tokens, int heads, int kv_heads, int dim,
                          int vdim, int n_pages, float temp_coef, int temp_every, imparo_stream stream);
// Per (token, head): a_m = softmax_j(q_m . k_m[j] * scale) v[j] over the keys lo..pos, o = a_1 - lambda a_2,
// out = o / sqrt(mean(o^2) + eps) * out_scale * sigmoid(gate) (gate null: no gate). n_splits > 1 walks the
// keys in pieces of imparo_diff_attention_split() through `part` (tokens x heads x n_splits x (2 vdim + 4) floats).
int imparo_diff_attention_split(void);
// below > 0: only the tokens of rows (seg_len per row) that bring fewer than `below` tokens.
int imparo_diff_attention(const void* q, const void* k_cache, const void* v_cache, const float* gate, int gate_ld,
                          void* out, float* part, int dtype, const int32_t* positions, const int32_t* row_of_token,
                          const int32_t* block_table, int table_stride, int page_size, int n_tokens, int heads,
                          int kv_heads, int dim, int vdim, int n_pages, float scale, int window, float lambda,
                          float eps, float out_scale, int n_splits, const int32_t* seg_len, int below,
                          imparo_stream stream);
// The same on the matrix cores, for rows that bring portions: bfloat16, pages of a multiple of 16 positions, dim
// and vdim multiples of 4 up to 128 (imparo_diff_attention_tiles_takes). A block takes
// imparo_diff_attention_tile() queries of one row and one head; rows of fewer than min_len tokens are skipped.
// With dim and vdim multiples of 8 and pages of a power of two, a block stages every tile of keys and values once
// in LDS for its four waves; otherwise every wave reads its operands itself.
int imparo_diff_attention_tile(void);
int imparo_diff_attention_tiles_takes(int page_size, int dim, int vdim);
int imparo_diff_attention_tiles(const void* q, const void* k_cache, const void* v_cache, const float* gate,
                                int gate_ld, void* out, const int32_t* positions, const int32_t* seg_start,
                                const int32_t* seg_len, const int32_t* block_table, int table_stride, int page_size,
                                int n_rows, int max_seg_len, int heads, int kv_heads, int dim, int vdim, int n_pages,
                                float scale, int window, float lambda, float eps, float out_scale, int min_len,
                                imparo_stream stream);

// ---------------------------------------------------------------------------------------------
// A model's step as one call. A program is the model's run order as a list of operations over a
// float32 residual stream: the embedding, then per layer a norm, a mixer, a norm and a
// feed-forward, then the norm and head of the wanted rows. Each operation launches the kernels
// above, chosen by the batch's shape exactly as a caller of the single entry points would choose
// them; what the program saves is the caller's time between launches. The reference issues a
// step's kernels from one native routine as well
// (/root/reference/crates/imparo-model/src/lfm2/workflow_gpu.rs:317-1633).
//
// Scratch lives in regions that the caller binds: the program names them (imparo_program_region_*),
// says how many bytes of each a step needs (imparo_program_needs) and refuses to run with
// IMPARO_SCRATCH_TOO_SMALL, before any launch, when a bound region is too small for the step.
// Nothing here allocates device memory.
typedef struct ImparoProgram ImparoProgram;

// A projection Y = X . W^T (+ bias): W is [n, k] in `dtype`, bias float32 [n] or null.
typedef struct {
    const void* weight;
    const float* bias;
    int32_t dtype, n, k;
} ImparoLinearDesc;

typedef struct {
    ImparoLinearDesc qkv, out;           // fused q | k | v projection, output projection
    const float* q_norm;                 // per-head RMS norm weights [head_dim], both null: no norm
    const float* k_norm;
    float norm_eps;
    const float* inv_freq;               // [n_freq] or null
    int32_t n_freq, interleaved;
    int32_t heads, kv_heads, head_dim;
    float scale;
    int32_t window;                      // 0: every key
    void* k_cache;                       // this call's cache site
    void* v_cache;
    int32_t n_pages, v_transposed, group; // group: which of the step's block tables
    int32_t owns_cache;                  // 0: reads a cache that an earlier call of the step has written
} ImparoAttentionDesc;

typedef struct {
    ImparoLinearDesc in_proj, out_proj;
    const float* conv_weight;            // [width, taps]
    const float* conv_bias;              // [width] or null
    int32_t width, taps;
    float* state;                        // [n_slots, taps - 1, width]
    int32_t n_slots;
} ImparoShortConvDesc;

typedef struct {
    ImparoLinearDesc gate_up, down;      // gate and up rows alternate in gate_up
} ImparoSwigluDesc;

// One batch: device arrays as imparo_cache_pack lays them out (any placement), and the sizes the
// host knows. tables[g] is [n_rows, table_width] for cache group g.
#define IMPARO_MAX_GROUPS 8
typedef struct {
    const int32_t* tokens;               // [n_tokens]
    const int32_t* positions;            // [n_tokens]
    const int32_t* row_of_token;         // [n_tokens]
    const int32_t* seg_start;            // [n_rows]
    const int32_t* seg_len;              // [n_rows]
    const int32_t* slot;                 // [n_rows]
    const int32_t* single_rows;          // [n_single]: rows that bring one token
    const int32_t* portion_rows;         // [n_portion]: rows that bring more
    const int32_t* want_rows;            // [n_want]: places in the packed batch whose logits are wanted
    const int32_t* tables[IMPARO_MAX_GROUPS];
    int32_t n_groups, table_width;
    int32_t n_tokens, n_rows, n_want, n_single, n_portion;
    int32_t max_seg_len, max_context;    // longest segment; longest context after the step (a bound will do)
    int32_t portion_tiles;               // sum over the portion rows of ceil(tokens / imparo_attention_prefill_tile())
} ImparoStepArgs;

ImparoProgram* imparo_program_new(int engine_dtype, int page_size);
void imparo_program_delete(ImparoProgram* p);
// In a step of at most 16 single tokens a norm of the stream can be folded into the products around
// it (decode_rows.hip): mode 0 never, 1 where imparo_rows_fold_pays says so (the default), 2 wherever
// the operations allow. Folding changes results by rounding only.
int imparo_program_set_fold(ImparoProgram* p, int mode);
int imparo_rows_fold_pays(int m, int n, int k);
// Operations, in run order. Each returns IMPARO_OK or IMPARO_BAD_ARGUMENT (sizes that do not fit).
int imparo_program_embedding(ImparoProgram* p, const void* table, int table_dtype, int vocab, int width);
// h = norm(stream + what the last mixer or feed-forward left pending), in out_dtype; the sum goes back to the stream
int imparo_program_norm(ImparoProgram* p, const float* weight, float eps, int width, int out_dtype);
int imparo_program_attention(ImparoProgram* p, const ImparoAttentionDesc* d);
int imparo_program_short_conv(ImparoProgram* p, const ImparoShortConvDesc* d);
int imparo_program_swiglu(ImparoProgram* p, const ImparoSwigluDesc* d);
// logits = head(norm(stream + pending) at the wanted rows); the stream is left as it is
int imparo_program_head(ImparoProgram* p, const float* norm_weight, float eps, int width, const ImparoLinearDesc* head);

int imparo_program_n_regions(const ImparoProgram* p);
const char* imparo_program_region_name(const ImparoProgram* p, int region);
int imparo_program_bind(ImparoProgram* p, int region, void* ptr, int64_t bytes);
// needs[region] = bytes of each region that a step of this shape uses (0: not used)
int imparo_program_needs(ImparoProgram* p, const ImparoStepArgs* args, int64_t* needs);
// Runs the step on `stream`. *logits = where the float32 [n_want, vocab] logits are (inside the
// "logits" region), or null if nothing is wanted. IMPARO_SCRATCH_TOO_SMALL: nothing was launched,
// imparo_program_needs says what to bind. Any other failure: imparo_program_error names the operation.
int imparo_program_run(ImparoProgram* p, const ImparoStepArgs* args, float** logits, imparo_stream stream);
const char* imparo_program_error(const ImparoProgram* p);

// x[t] = table[ids[t]] * scale (float32 product).
int imparo_embed_gather_scaled(const void* table, int table_dtype, const int32_t* ids, float* x,
                               int n_tokens, int width, int vocab, float scale, imparo_stream stream);

// ---- a routed feed-forward (mixture of experts)
// route: scores = softmax(logits[t, :n_router]) (scoring 0) or the sigmoid of each output (scoring 1); the `top`
// largest of score + correction are chosen (of equal ones the lowest index), choice [tokens, top] holds their
// indices and weight [tokens, top] their scores.
// Beyond that: a token's logits lie logits_ld floats apart (at least n_router); with groups > 1 (at most 64) the
// outputs form that many equal groups of neighbours, a group's score is the sum of its two largest choice scores
// (score + correction) and only outputs of the `keep` best groups can be chosen; with `normalize` the chosen scores
// are divided by their sum + 1e-20; the weights are multiplied by `scale` at the end.
int imparo_moe_route(const float* logits, const float* correction, int32_t* choice, float* weight,
                     int n_tokens, int n_router, int top, int scoring, int logits_ld, int groups, int keep,
                     int normalize, float scale, imparo_stream stream);
// hidden[slot, j] = silu(w g) * (w u), g = gu[slot, j], u = gu[slot, half + j], w = weight[entry_of_slot[slot]]
// (weight null: 1): the hidden values of gated experts without biases that read w times their input, from the
// stacked gate and up products of the input itself. gu float32 [n_slots, 2 half].
int imparo_moe_gated(const float* gu, const float* weight, const int32_t* entry_of_slot, void* hidden, int out_dtype,
                     int n_slots, int half, imparo_stream stream);
// plan: entries are (token, choice) pairs in row-major order; those whose expert is below n_experts get a slot,
// an expert's slots side by side (slot_of_entry, -1 for the others; entry_of_slot), and `tiles` [max_tiles, 3]
// lists (expert, first slot, rows <= tile_rows) of every tile of rows, expert -1 past the list's end.
int imparo_moe_tile_rows(int n_entries, int n_experts, int dtype);
int imparo_moe_max_tiles(int n_entries, int n_experts, int tile_rows);
int imparo_moe_plan(const int32_t* choice, int n_entries, int n_experts, int tile_rows,
                    int32_t* slot_of_entry, int32_t* entry_of_slot, int32_t* tiles, int max_tiles,
                    imparo_stream stream);
// product: out[slot, :n] = epilogue(a[row(slot), :k] . w[expert(slot), :n, :k]); row(slot) is the slot, or with
// gather_div > 0 entry_of_slot[slot] / gather_div. epilogue 0: none, 1: max(z, 0)^2. bfloat16 operands (k a
// multiple of 8, out bfloat16 or float32; tile_rows 16, 64 or 128) or float32 throughout (tile_rows 64).
int imparo_moe_gemm(const void* a, int a_ld, int gather_div, const int32_t* entry_of_slot, const void* w,
                    void* out, int out_dtype, int dtype, const int32_t* tiles, int max_tiles, int tile_rows,
                    int n, int k, int epilogue, imparo_stream stream);
// combine: out[t] = sum_j weight[t, j] * (y[slot of (t, j)] if choice[t, j] < n_experts else h[t]), j in order
// (weight null: every weight is 1).
int imparo_moe_combine(const float* y, const void* h, int h_dtype, const int32_t* choice,
                       const float* weight, const int32_t* slot_of_entry, float* out, int n_tokens,
                       int width, int top, int n_experts, imparo_stream stream);

// route and plan in one launch, for at most imparo_moe_route_plan_tokens() tokens (a decode step)
int imparo_moe_route_plan_tokens(void);
int imparo_moe_route_plan(const float* logits, const float* correction, int32_t* choice, float* weight,
                          int n_tokens, int n_router, int top, int scoring, int n_experts, int tile_rows,
                          int32_t* slot_of_entry, int32_t* entry_of_slot, int32_t* tiles, int max_tiles,
                          int logits_ld, int groups, int keep, int normalize, float scale, imparo_stream stream);

// A norm on what a sublayer returns, its add into the stream, and the next norm, in one launch:
// x[r] += rms_norm(sum of delta's slices [n_delta, n_rows_x, width])[r] * w_post; with w_next,
// out[i] = rms_norm(x[r]) * w_next. r = rows[i] (then x is left as it is), or i.
int imparo_post_norm_add(float* x, const float* delta, int n_delta, int n_rows_x, const int32_t* rows,
                         const float* w_post, float eps_post, const float* w_next, float eps_next,
                         void* out, int out_dtype, int n_out, int width, imparo_stream stream);

// imparo_post_norm_add with the delta made in the launch from a routed feed-forward's rows: what
// imparo_moe_combine would have written, added up in the same order.
int imparo_post_norm_add_moe(float* x, const float* y, const void* h, int h_dtype, const int32_t* choice,
                             const float* weight, const int32_t* slot_of_entry, int top, int n_experts,
                             int n_rows_x, const int32_t* rows, const float* w_post, float eps_post,
                             const float* w_next, float eps_next, void* out, int out_dtype, int n_out,
                             int width, imparo_stream stream);

#ifdef __cplusplus
}
#endif
