// Attention over a cached latent (keys and values are up-projections of one small vector a token,
// plus one rotated key part that all heads share), in its absorbed form: the cache keeps a row
// [latent | rotated key part] a position; a query carries W_uk^T q_unrotated next to its rotated part,
// so that a score is one dot product with a cached row; the weighted sum of latents goes through W_uv
// afterwards. Two kernels here, the attention itself is the wave kernel over shared rows:
//   latent_store  norms the latent, rotates the shared key part and writes the row into its page;
//                 rotates every head's rotated query part and lays the queries out for what follows
//   head_gemm     out[t, h, :] = W[h] in[t, h, :], a small product per head (the two absorbed
//                 up-projections), float32 sums in the order k = 0, 1, 2, ...
#include "common.h"

#include <algorithm>
#include "api.h"

#define LAT_MAX_FREQ 256

// x: this thread's view of a vector whose first 2 n_freq entries turn; d its index. Halves: pair i is
// (i, i + n_freq); neighbours: (2i, 2i + 1). (u, v) -> (u cos - v sin, v cos + u sin).
__device__ __forceinline__ float turned(const float* __restrict__ x, int d, int n_freq, int interleaved,
                                        const float* __restrict__ sn, const float* __restrict__ cs) {
    if (d >= 2 * n_freq) return x[d];
    if (interleaved) {
        const int i = d >> 1;
        return (d & 1) ? x[d] * cs[i] + x[d - 1] * sn[i] : x[d] * cs[i] - x[d + 1] * sn[i];
    }
    if (d < n_freq) return x[d] * cs[d] - x[d + n_freq] * sn[d];
    const int i = d - n_freq;
    return x[d] * cs[i] + x[i] * sn[i];
}

// One block a token. q_rows [tokens, heads * (dim + rot_dim)] float32, kv_rows [tokens, rank + rot_dim] float32.
// q_plain [tokens, heads, dim] gets the unrotated parts, q_full [tokens, heads, rank + rot_dim] the rotated
// parts at columns rank .. (the first rank columns are written by the product that follows).
template <typename T>
__global__ __launch_bounds__(256) void k_latent_store(const float* __restrict__ q_rows, const float* __restrict__ kv_rows,
                                                      const float* __restrict__ norm_weight, float eps,
                                                      const float* __restrict__ inv_freq, int n_freq, int interleaved,
                                                      const int32_t* __restrict__ positions,
                                                      const int32_t* __restrict__ row_of_token,
                                                      const int32_t* __restrict__ block_table, int table_stride,
                                                      int page_size, int n_pages, T* __restrict__ cache,
                                                      T* __restrict__ cache_t, T* __restrict__ q_plain, T* __restrict__ q_full, int heads, int dim,
                                                      int rot_dim, int rank) {
    __shared__ float sn[LAT_MAX_FREQ], cs[LAT_MAX_FREQ];
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const int pos = positions[t];
    for (int i = threadIdx.x; i < n_freq; i += blockDim.x) rotation_of(pos, inv_freq[i], sn[i], cs[i]);
    const float* kv = kv_rows + (size_t)t * (rank + rot_dim);
    float ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) ss += kv[i] * kv[i];
    ss = block_sum(ss, scratch);             // (its barriers also publish the sines and cosines)
    const float scale = 1.0f / sqrtf(ss / (float)rank + eps);
    if (cache) {
        const int page = block_table[(size_t)row_of_token[t] * table_stride + pos / page_size];
        if (page >= 0 && page < n_pages) {
            T* dst = cache + ((size_t)page * page_size + (pos % page_size)) * (rank + rot_dim);
            for (int i = threadIdx.x; i < rank; i += blockDim.x) store_f32<T>(dst, i, kv[i] * scale * norm_weight[i]);
            for (int d = threadIdx.x; d < rot_dim; d += blockDim.x)
                store_f32<T>(dst, rank + d, turned(kv + rank, d, n_freq, interleaved, sn, cs));
            if (cache_t) {      // the latent once more, [page, rank, position]: the values as the matrix-core kernel reads them
                T* dst_t = cache_t + (size_t)page * rank * page_size + (pos % page_size);
                for (int i = threadIdx.x; i < rank; i += blockDim.x)
                    store_f32<T>(dst_t, (size_t)i * page_size, kv[i] * scale * norm_weight[i]);
            }
        }
    }
    const int per = dim + rot_dim;
    for (int i = threadIdx.x; i < heads * per; i += blockDim.x) {
        const int h = i / per, d = i - h * per;
        const float* qh = q_rows + (size_t)t * heads * per + (size_t)h * per;
        if (d < dim)
            store_f32<T>(q_plain, ((size_t)t * heads + h) * dim + d, qh[d]);
        else
            store_f32<T>(q_full, ((size_t)t * heads + h) * (rank + rot_dim) + rank + (d - dim),
                         turned(qh + dim, d - dim, n_freq, interleaved, sn, cs));
    }
}

extern "C" int imparo_latent_store(const float* q_rows, const float* kv_rows, const float* norm_weight, float eps,
                                   const float* inv_freq, int n_freq, int interleaved, const int32_t* positions,
                                   const int32_t* row_of_token, const int32_t* block_table, int table_stride,
                                   int page_size, int n_pages, void* cache, void* cache_t, void* q_plain, void* q_full, int dtype,
                                   int n_tokens, int heads, int dim, int rot_dim, int rank, imparo_stream stream) {
    if (!q_rows || !kv_rows || !norm_weight || !positions || !q_plain || !q_full) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || heads < 1 || dim < 1 || rot_dim < 0 || rank < 1) return IMPARO_BAD_ARGUMENT;
    if (n_freq < 0 || n_freq > LAT_MAX_FREQ || 2 * n_freq > rot_dim || (n_freq && !inv_freq)) return IMPARO_BAD_ARGUMENT;
    if (cache_t && !cache) return IMPARO_BAD_ARGUMENT;
    if (cache && (!row_of_token || !block_table || table_stride < 1 || page_size < 1 || n_pages < 1)) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == IMPARO_F32)
        k_latent_store<float><<<n_tokens, 256, 0, s>>>(q_rows, kv_rows, norm_weight, eps, inv_freq, n_freq, interleaved,
                                                       positions, row_of_token, block_table, table_stride, page_size,
                                                       n_pages, (float*)cache, (float*)cache_t, (float*)q_plain, (float*)q_full, heads, dim,
                                                       rot_dim, rank);
    else if (dtype == IMPARO_BF16)
        k_latent_store<bf16_t><<<n_tokens, 256, 0, s>>>(q_rows, kv_rows, norm_weight, eps, inv_freq, n_freq, interleaved,
                                                        positions, row_of_token, block_table, table_stride, page_size,
                                                        n_pages, (bf16_t*)cache, (bf16_t*)cache_t, (bf16_t*)q_plain, (bf16_t*)q_full, heads,
                                                        dim, rot_dim, rank);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// out[t, h, n] = sum_k w[h, k, n] in[t, h, k]: a block takes HG_ROWS tokens of one head, the tokens' rows in LDS
// as float32, a thread the outputs n = thread, thread + 256, ... for all of them (w lies [heads, k, n], so the
// threads of a wave read neighbouring numbers). in rows lie in_ld apart and a head's part in_hs apart inside a
// row; out likewise.
#define HG_ROWS 16
template <typename T, typename TOut>
__global__ __launch_bounds__(256) void k_head_gemm(const T* __restrict__ in, int in_ld, int in_hs,
                                                   const T* __restrict__ w, TOut* __restrict__ out, int out_ld,
                                                   int out_hs, int n_tokens, int K, int N) {
    extern __shared__ float rows[];          // [HG_ROWS][K]
    const int h = blockIdx.y;
    const int t0 = blockIdx.x * HG_ROWS;
    const int n_rows = min(HG_ROWS, n_tokens - t0);
    for (int i = threadIdx.x; i < HG_ROWS * K; i += blockDim.x) {
        const int r = i / K, k = i - r * K;
        rows[i] = r < n_rows ? load_f32<T>(in, (size_t)(t0 + r) * in_ld + (size_t)h * in_hs + k) : 0.f;
    }
    __syncthreads();
    const T* wh = w + (size_t)h * K * N;
    for (int n = threadIdx.x; n < N; n += blockDim.x) {
        float acc[HG_ROWS];
#pragma unroll
        for (int r = 0; r < HG_ROWS; ++r) acc[r] = 0.f;
        for (int k = 0; k < K; ++k) {
            const float wv = load_f32<T>(wh, (size_t)k * N + n);
#pragma unroll
            for (int r = 0; r < HG_ROWS; ++r) acc[r] = fmaf(rows[r * K + k], wv, acc[r]);
        }
#pragma unroll
        for (int r = 0; r < HG_ROWS; ++r)
            if (r < n_rows) store_f32<TOut>(out, (size_t)(t0 + r) * out_ld + (size_t)h * out_hs + n, acc[r]);
    }
}

extern "C" int imparo_head_gemm(const void* in, int in_ld, int in_hs, const void* w, int dtype, void* out, int out_dtype,
                                int out_ld, int out_hs, int n_tokens, int heads, int k, int n, imparo_stream stream) {
    if (!in || !w || !out || n_tokens < 0 || heads < 1 || k < 1 || n < 1) return IMPARO_BAD_ARGUMENT;
    if (in_hs < k || in_ld < (heads - 1) * in_hs + k || out_hs < n || out_ld < (heads - 1) * out_hs + n)
        return IMPARO_BAD_ARGUMENT;
    const size_t lds = (size_t)HG_ROWS * k * sizeof(float);
    if (lds > 64 * 1024) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((n_tokens + HG_ROWS - 1) / HG_ROWS, heads);
    if (dtype == IMPARO_F32 && out_dtype == IMPARO_F32)
        k_head_gemm<float, float><<<grid, 256, lds, s>>>((const float*)in, in_ld, in_hs, (const float*)w, (float*)out,
                                                         out_ld, out_hs, n_tokens, k, n);
    else if (dtype == IMPARO_BF16 && out_dtype == IMPARO_BF16)
        k_head_gemm<bf16_t, bf16_t><<<grid, 256, lds, s>>>((const bf16_t*)in, in_ld, in_hs, (const bf16_t*)w,
                                                           (bf16_t*)out, out_ld, out_hs, n_tokens, k, n);
    else if (dtype == IMPARO_BF16 && out_dtype == IMPARO_F32)
        k_head_gemm<bf16_t, float><<<grid, 256, lds, s>>>((const bf16_t*)in, in_ld, in_hs, (const bf16_t*)w, (float*)out,
                                                          out_ld, out_hs, n_tokens, k, n);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// ---------------------------------------------------------------- the matrix-core kernel
// A wave takes up to 16 heads of one token as the 16 queries of its products (32 heads, as two such sets, where
// a token has more than 16: every loaded tile then feeds twice the products): every head reads the same
// rows, so one tile of keys serves them all, and they share one range of keys. Keys are walked in tiles of
// 32 at absolute multiples of 32:
//   S^T[key][head] = rows . Q^T     A = 16 bytes of a cached row a lane, B = Q^T in registers. Row m of
//                                   product t stands for key 8 (m / 4) + 4 t + m % 4, so that the 8 scores
//                                   a lane ends up with are the keys 8 (lane / 16) .. + 7,
//   O^T[dim][head] += V^T . P^T     A = 16 bytes of the transposed copy of the latents (8 keys of one
//                                   dimension), B = the lane's 8 softmax weights as they are.
// With `exact` a weight enters the second product as two bfloat16 numbers (its rounding and what the
// rounding lost). With n_splits > 1 a wave takes the keys [split * split_keys, (split + 1) * split_keys)
// of its range and writes an unnormed part (sum, maximum, weight sum); k_latent_merge adds the parts.
typedef float lat_f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 lat_bf16x8 __attribute__((ext_vector_type(8)));
union LatFrag {
    uint4 u;
    lat_bf16x8 v;
};

#define LAT_WAVES 4

__device__ __forceinline__ uint32_t lat_pack2(float a, float b) { return f32x2_to_bf16x2(a, b); }

__device__ __forceinline__ float lat_bf16_value(float a) { return __uint_as_float((uint32_t)f32_to_bf16(a) << 16); }

template <int NK, int NV, int QT>
__global__ __launch_bounds__(LAT_WAVES * WAVE, QT == 1 ? 2 : 1) void k_latent_attention_tiles(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ rows, const bf16_t* __restrict__ rows_t,
    bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ row_of_token,
    const int32_t* __restrict__ block_table, int table_stride, int page_shift, int n_pages, int n_tokens, int heads,
    int row_dim, int rank, float scale, int window, int split_keys, int n_splits, int exact) {
    // (what a wave shares is said to be the same in all of its lanes, so that it is kept and computed once a wave)
    const int lane = threadIdx.x & (WAVE - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int c = lane & 15, g = lane >> 4;
    const int head_groups = (heads + 16 * QT - 1) / (16 * QT);
    const long long total = (long long)n_tokens * head_groups * n_splits;
    const long long id = (long long)blockIdx.x * LAT_WAVES + wave;
    if (id >= total) return;                       // (with parts the waves come in whole blocks: all reach the barrier below)
    const int split = (int)(id % n_splits);
    const long long rest = id / n_splits;
    const int t = n_tokens - 1 - (int)(rest % n_tokens);    // late tokens of a prompt, with the most keys, start first
    const int h0 = (int)(rest / n_tokens) * 16 * QT + c;   // this lane's heads: h0, h0 + 16, ...
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
    const int k_lo = n_splits > 1 ? max(lo, split * split_keys) : lo;
    const int k_hi = n_splits > 1 ? min(pos, (split + 1) * split_keys - 1) : pos;
    const int page_size = 1 << page_shift, page_mask = page_size - 1;
    const int32_t* table = block_table + (size_t)row_of_token[t] * table_stride;

    LatFrag qf[QT][NK];
    lat_f32x4 o[QT][NV];
    float m[QT], l[QT];
#pragma unroll
    for (int u = 0; u < QT; ++u) {
        const int h = h0 + 16 * u;
        const bool live = h < heads;
        const bf16_t* qrow = q + ((size_t)t * heads + (live ? h : 0)) * row_dim;
#pragma unroll
        for (int dk = 0; dk < NK; ++dk) {
            const int d0 = dk * 32 + 8 * g;
            qf[u][dk].u = (live && d0 < row_dim) ? *reinterpret_cast<const uint4*>(qrow + d0) : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int dt = 0; dt < NV; ++dt) o[u][dt] = lat_f32x4{0.f, 0.f, 0.f, 0.f};
        m[u] = -INFINITY;
        l[u] = 0.f;
    }

    if (k_lo <= k_hi) {
        for (int base = k_lo & ~31; base <= k_hi; base += 32) {
            // a tile lies in one page (pages hold a multiple of 32 positions), and a part of it is in the range:
            // addresses are held inside that part, so that no lane reads outside the tile's own page
            const int page = min(max(table[base >> page_shift], 0), n_pages - 1);
            const int t_lo = max(k_lo, base), t_hi = min(k_hi, base + 31);
            LatFrag kf[2][NK];
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
                const int key = min(max(base + 8 * (c >> 2) + 4 * t2 + (c & 3), t_lo), t_hi);
                const bf16_t* krow = rows + ((size_t)page * page_size + (key & page_mask)) * row_dim;
#pragma unroll
                for (int dk = 0; dk < NK; ++dk)     // beyond the row: its last 8 again, against zeros of the query
                    kf[t2][dk].u = *reinterpret_cast<const uint4*>(krow + min(dk * 32 + 8 * g, row_dim - 8));
            }
            const int kg = base + 8 * g;            // this lane's 8 keys in both products' results
            LatFrag vf[NV];
            {
                const int kgc = min(max(kg, t_lo & ~7), t_hi & ~7);
                const bf16_t* vbase = rows_t + (size_t)page * rank * page_size + (kgc & page_mask);
#pragma unroll
                for (int dt = 0; dt < NV; ++dt)
                    vf[dt].u = *reinterpret_cast<const uint4*>(vbase + (size_t)min(dt * 16 + c, rank - 1) * page_size);
            }
            lat_f32x4 s[QT][2];
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2) {
#pragma unroll
                for (int u = 0; u < QT; ++u) s[u][t2] = lat_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int dk = 0; dk < NK; ++dk)
#pragma unroll
                    for (int u = 0; u < QT; ++u)
                        s[u][t2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t2][dk].v, qf[u][dk].v, s[u][t2], 0, 0, 0);
            }
            if (base < k_lo || base + 31 > k_hi) {  // what a page holds beyond the range may be anything: zeros instead
                uint32_t keep[4];
#pragma unroll
                for (int j2 = 0; j2 < 4; ++j2) {
                    const int k0 = kg + 2 * j2;
                    keep[j2] = ((k0 >= k_lo && k0 <= k_hi) ? 0x0000ffffu : 0u) |
                               ((k0 + 1 >= k_lo && k0 + 1 <= k_hi) ? 0xffff0000u : 0u);
                }
#pragma unroll
                for (int dt = 0; dt < NV; ++dt)
                    vf[dt].u = make_uint4(vf[dt].u.x & keep[0], vf[dt].u.y & keep[1], vf[dt].u.z & keep[2], vf[dt].u.w & keep[3]);
            }
#pragma unroll
            for (int u = 0; u < QT; ++u) {
                float sv[8];
                float tile_max = -INFINITY;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int key = kg + j;
                    sv[j] = (key >= k_lo && key <= k_hi) ? s[u][j >> 2][j & 3] * scale : -INFINITY;
                    tile_max = fmaxf(tile_max, sv[j]);
                }
                tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE));
                tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE));
                const float m_new = fmaxf(m[u], tile_max);  // finite: every tile holds a key of the range
                const float corr = __expf(m[u] - m_new);
                float p[8], p_sum = 0.f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    p[j] = __expf(sv[j] - m_new);
                    p_sum += p[j];
                }
                l[u] = l[u] * corr + p_sum;         // a lane's own 8 keys; the four lanes of a head are added at the end
                if (__builtin_amdgcn_ballot_w64(m_new != m[u])) {   // (no head's maximum moved: every factor is 1)
#pragma unroll
                    for (int dt = 0; dt < NV; ++dt) o[u][dt] *= corr;
                }
                m[u] = m_new;
                LatFrag ph;
                ph.u = make_uint4(lat_pack2(p[0], p[1]), lat_pack2(p[2], p[3]), lat_pack2(p[4], p[5]), lat_pack2(p[6], p[7]));
#pragma unroll
                for (int dt = 0; dt < NV; ++dt)
                    o[u][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, ph.v, o[u][dt], 0, 0, 0);
                if (exact) {
                    float r[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) r[j] = p[j] - lat_bf16_value(p[j]);
                    LatFrag pl;
                    pl.u = make_uint4(lat_pack2(r[0], r[1]), lat_pack2(r[2], r[3]), lat_pack2(r[4], r[5]), lat_pack2(r[6], r[7]));
#pragma unroll
                    for (int dt = 0; dt < NV; ++dt)
                        o[u][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pl.v, o[u][dt], 0, 0, 0);
                }
            }
        }
    }
    if (n_splits > 1) {
        // The block's four waves hold four neighbouring parts of one token's keys (n_splits is a multiple of 4, and
        // such launches take 16 heads a wave): waves 1 .. 3 leave theirs in LDS, wave 0 adds the four in order.
        extern __shared__ float lat_parts[];         // [3][NV * 4 + 2][64]
        constexpr int PER = (NV * 4 + 2) * WAVE;
        float lu = l[0];
        lu += __shfl_xor(lu, 16, WAVE);
        lu += __shfl_xor(lu, 32, WAVE);
        if (wave > 0) {
            float* mine = lat_parts + (size_t)(wave - 1) * PER;
#pragma unroll
            for (int dt = 0; dt < NV; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) mine[(dt * 4 + i) * WAVE + lane] = o[0][dt][i];
            mine[NV * 4 * WAVE + lane] = m[0];
            mine[(NV * 4 + 1) * WAVE + lane] = lu;
        }
        __syncthreads();
        if (wave > 0 || h0 >= heads) return;
        float top = m[0], wt[LAT_WAVES];
#pragma unroll
        for (int w = 1; w < LAT_WAVES; ++w) top = fmaxf(top, lat_parts[(size_t)(w - 1) * PER + NV * 4 * WAVE + lane]);
        wt[0] = m[0] == -INFINITY ? 0.f : __expf(m[0] - top);
        float sum = wt[0] * lu;
#pragma unroll
        for (int w = 1; w < LAT_WAVES; ++w) {
            const float mw = lat_parts[(size_t)(w - 1) * PER + NV * 4 * WAVE + lane];
            wt[w] = mw == -INFINITY ? 0.f : __expf(mw - top);
            sum += wt[w] * lat_parts[(size_t)(w - 1) * PER + (NV * 4 + 1) * WAVE + lane];
        }
        const int parts = n_splits / LAT_WAVES, part = split / LAT_WAVES;
        const size_t row = (size_t)t * heads + h0;
        const float inv = parts == 1 ? (sum > 0.f ? 1.0f / sum : 0.f) : 1.0f;
#pragma unroll
        for (int dt = 0; dt < NV; ++dt) {
            const int d = dt * 16 + 4 * g;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[i] = wt[0] * o[0][dt][i];
#pragma unroll
                for (int w = 1; w < LAT_WAVES; ++w) v[i] += wt[w] * lat_parts[(size_t)(w - 1) * PER + (dt * 4 + i) * WAVE + lane];
                v[i] *= inv;
            }
            if (d >= rank) continue;                 // (rank is a multiple of 8: a lane's four numbers are in or out together)
            if (parts == 1)
                *reinterpret_cast<uint2*>(out + row * rank + d) = make_uint2(lat_pack2(v[0], v[1]), lat_pack2(v[2], v[3]));
            else
                *reinterpret_cast<float4*>(part_o + (row * parts + part) * rank + d) = make_float4(v[0], v[1], v[2], v[3]);
        }
        if (parts > 1 && g == 0) {
            part_ml[(row * parts + part) * 2] = top;
            part_ml[(row * parts + part) * 2 + 1] = sum;
        }
        return;
    }
#pragma unroll
    for (int u = 0; u < QT; ++u) {
        float lu = l[u];
        lu += __shfl_xor(lu, 16, WAVE);
        lu += __shfl_xor(lu, 32, WAVE);
        const int h = h0 + 16 * u;
        if (h >= heads) continue;
        const float inv = lu > 0.f ? 1.0f / lu : 0.f;
        bf16_t* dst = out + ((size_t)t * heads + h) * rank;     // (rank is a multiple of 8: a lane's four numbers are in or out together)
#pragma unroll
        for (int dt = 0; dt < NV; ++dt) {
            const int d = dt * 16 + 4 * g;
            if (d < rank)
                *reinterpret_cast<uint2*>(dst + d) = make_uint2(lat_pack2(o[u][dt][0] * inv, o[u][dt][1] * inv),
                                                                lat_pack2(o[u][dt][2] * inv, o[u][dt][3] * inv));
        }
    }
}

// out[row, d] = sum_s w_s part_o[row, s, d] / sum_s w_s l_s with w_s = exp(m_s - max m), the parts in order.
// A thread takes four neighbouring numbers of a row (rank is a multiple of 8).
__global__ void k_latent_merge(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                               bf16_t* __restrict__ out, long long n_rows, int n_splits, int rank) {
    const int quads = rank / 4;
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_rows * quads) return;
    const long long row = i / quads;
    const int d = (int)(i - row * quads) * 4;
    const float* ml = part_ml + row * n_splits * 2;
    float top = -INFINITY;
    for (int s = 0; s < n_splits; ++s) top = fmaxf(top, ml[2 * s]);
    float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
    float den = 0.f;
    for (int s = 0; s < n_splits; ++s) {
        const float ms = ml[2 * s];
        if (ms == -INFINITY) continue;
        const float w = __expf(ms - top);
        const float4 part = *reinterpret_cast<const float4*>(part_o + (row * n_splits + s) * rank + d);
        num.x += w * part.x;
        num.y += w * part.y;
        num.z += w * part.z;
        num.w += w * part.w;
        den += w * ml[2 * s + 1];
    }
    const float inv = den > 0.f ? 1.0f / den : 0.f;
    *reinterpret_cast<uint2*>(out + row * rank + d) = make_uint2(lat_pack2(num.x * inv, num.y * inv), lat_pack2(num.z * inv, num.w * inv));
}

// The sizes the matrix-core kernel is built for: latents of up to 256 numbers in steps of 8 (value tiles of
// 16: 2, 4, 8 or 16 of them), rows (latent and rotated key part) of up to 32 (tiles / 2 + 2) numbers in
// steps of 8, pages of a power of two from 32 on.
static int latent_tiles_shape(int row_dim, int rank, int* nk, int* nv) {
    if (rank < 8 || rank > 256 || rank % 8 || row_dim % 8 || row_dim < rank) return 0;
    const int v = rank <= 32 ? 2 : rank <= 64 ? 4 : rank <= 128 ? 8 : 16;
    const int k = (row_dim + 31) / 32;
    if (k > v / 2 + 2) return 0;
    *nv = v;
    *nk = k <= v / 2 + 1 ? v / 2 + 1 : v / 2 + 2;
    return 1;
}

extern "C" int imparo_attention_latent_tiles_takes(int row_dim, int rank, int page_size) {
    int nk, nv;
    return page_size >= 32 && (page_size & (page_size - 1)) == 0 && latent_tiles_shape(row_dim, rank, &nk, &nv);
}

// Into how many parts the keys of a launch are cut, and how many keys a part holds: few tokens over long
// contexts would leave most of the chip idle. Parts lie at absolute multiples of their size.
// 32 heads a wave where the launch fills the chip that way; few tokens are better spread over more waves.
static int latent_heads_a_wave(int n_tokens, int heads) {
    return heads > 16 && (long long)n_tokens * ((heads + 31) / 32) >= 512 ? 32 : 16;
}

extern "C" int imparo_attention_latent_tiles_split(int n_tokens, int heads, int max_context, int* split_keys) {
    const int per = latent_heads_a_wave(n_tokens, heads);
    const long long items = (long long)n_tokens * ((heads + per - 1) / per);
    int want = items >= 512 ? 1 : (int)((512 + items - 1) / items);
    int keys = ((max_context + want - 1) / want + 63) / 64 * 64;
    if (keys < 64) keys = 64;
    int n = max_context <= keys ? 1 : (max_context + keys - 1) / keys;
    if (n > 1) n = (n + LAT_WAVES - 1) / LAT_WAVES * LAT_WAVES;    // a block's waves take neighbouring parts and add them
    if (split_keys) *split_keys = keys;
    return n;
}

template <int NK, int NV, int QT>
static void launch_latent_tiles(const void* q, const void* rows, const void* rows_t, void* out, float* part_o,
                                float* part_ml, const int32_t* positions, const int32_t* row_of_token,
                                const int32_t* block_table, int table_stride, int page_shift, int n_pages, int n_tokens,
                                int heads, int row_dim, int rank, float scale, int window, int split_keys, int n_splits,
                                int exact, hipStream_t s) {
    const long long waves = (long long)n_tokens * ((heads + 16 * QT - 1) / (16 * QT)) * n_splits;
    const unsigned blocks = (unsigned)((waves + LAT_WAVES - 1) / LAT_WAVES);
    const size_t lds = n_splits > 1 ? (size_t)(LAT_WAVES - 1) * (NV * 4 + 2) * WAVE * sizeof(float) : 0;
    k_latent_attention_tiles<NK, NV, QT><<<blocks, LAT_WAVES * WAVE, lds, s>>>(
        (const bf16_t*)q, (const bf16_t*)rows, (const bf16_t*)rows_t, (bf16_t*)out, part_o, part_ml, positions,
        row_of_token, block_table, table_stride, page_shift, n_pages, n_tokens, heads, row_dim, rank, scale, window,
        split_keys, n_splits, exact);
}

// q [tokens, heads, row_dim], rows [pages, page, row_dim], rows_t [pages, rank, page] (the latents once more,
// transposed inside a page), out [tokens, heads * rank], all bfloat16. n_splits and split_keys as
// imparo_attention_latent_tiles_split gives them for a max_context that bounds every position + 1; with
// n_splits > 1, part_o [tokens, heads, n_splits, rank] and part_ml [tokens, heads, n_splits, 2] float32.
extern "C" int imparo_attention_latent_tiles(const void* q, const void* rows, const void* rows_t, void* out,
                                             float* part_o, float* part_ml, const int32_t* positions,
                                             const int32_t* row_of_token, const int32_t* block_table, int table_stride,
                                             int page_size, int n_pages, int n_tokens, int heads, int row_dim, int rank,
                                             float scale, int window, int split_keys, int n_splits, int exact,
                                             imparo_stream stream) {
    if (!q || !rows || !rows_t || !out || !positions || !row_of_token || !block_table) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || heads < 1 || table_stride < 1 || n_pages < 1 || window < 0) return IMPARO_BAD_ARGUMENT;
    int nk = 0, nv = 0;
    if (!imparo_attention_latent_tiles_takes(row_dim, rank, page_size) || !latent_tiles_shape(row_dim, rank, &nk, &nv))
        return IMPARO_BAD_ARGUMENT;
    if (n_splits < 1 || (n_splits > 1 && (!part_o || !part_ml || split_keys < 32 || split_keys % 32))) return IMPARO_BAD_ARGUMENT;
    if (n_splits > 1 && (long long)n_splits * split_keys > 0x7fffffffLL) return IMPARO_BAD_ARGUMENT;
    if (n_splits > 1 && (n_splits % LAT_WAVES || latent_heads_a_wave(n_tokens, heads) != 16)) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    hipStream_t s = (hipStream_t)stream;
#define LAT_CASE(K, V)                                                                                               \
    if (nk == K && nv == V) {                                                                                        \
        if (latent_heads_a_wave(n_tokens, heads) == 32)                                                                       \
            launch_latent_tiles<K, V, 2>(q, rows, rows_t, out, part_o, part_ml, positions, row_of_token, block_table, \
                                         table_stride, page_shift, n_pages, n_tokens, heads, row_dim, rank, scale,    \
                                         window, split_keys, n_splits, exact, s);                                    \
        else                                                                                                         \
            launch_latent_tiles<K, V, 1>(q, rows, rows_t, out, part_o, part_ml, positions, row_of_token, block_table, \
                                         table_stride, page_shift, n_pages, n_tokens, heads, row_dim, rank, scale,    \
                                         window, split_keys, n_splits, exact, s);                                    \
    }
    LAT_CASE(2, 2) LAT_CASE(3, 2) LAT_CASE(3, 4) LAT_CASE(4, 4) LAT_CASE(5, 8) LAT_CASE(6, 8) LAT_CASE(9, 16) LAT_CASE(10, 16)
#undef LAT_CASE
    if (launch_status() != IMPARO_OK) return IMPARO_LAUNCH_FAILED;
    if (n_splits > LAT_WAVES) {
        const long long n = (long long)n_tokens * heads * (rank / 4);
        k_latent_merge<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(part_o, part_ml, (bf16_t*)out, (long long)n_tokens * heads,
                                                                  n_splits / LAT_WAVES, rank);
    }
    return launch_status();
}

// The per-head product on the matrix cores, bfloat16: w_t [heads, n, k] keeps a head's matrix with the inner
// size running fastest, as both operands of a 16x16x32 product want it. A wave makes 16 outputs of one head
// for 16 tokens: O^T[n][token] = W_t . in^T, so that a lane ends up with 4 neighbouring outputs of one token.
template <typename TOut>
__global__ __launch_bounds__(LAT_WAVES * WAVE) void k_head_gemm_tiles(const bf16_t* __restrict__ in, int in_ld, int in_hs,
                                                                      const bf16_t* __restrict__ w_t, TOut* __restrict__ out,
                                                                      int out_ld, int out_hs, int n_tokens, int K, int N) {
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int c = lane & 15, g = lane >> 4;
    const int h = blockIdx.y;
    const int token = blockIdx.x * 16 + c;
    const bool live = token < n_tokens;
    const bf16_t* brow = in + (size_t)(live ? token : 0) * in_ld + (size_t)h * in_hs;
    TOut* dst = out + (size_t)(live ? token : 0) * out_ld + (size_t)h * out_hs;
    const bool quads = out_ld % 4 == 0 && out_hs % 4 == 0;      // every head's outputs start where four of them align
    // the launch's waves share a head's tiles of 16 outputs among them (many tokens: few, long-lived waves)
    for (int n_base = (blockIdx.z * LAT_WAVES + wave) * 16; n_base < N; n_base += gridDim.z * LAT_WAVES * 16) {
        const bf16_t* arow = w_t + ((size_t)h * N + min(n_base + c, N - 1)) * K;
        lat_f32x4 acc = lat_f32x4{0.f, 0.f, 0.f, 0.f};
        for (int k0 = 0; k0 < K; k0 += 32) {
            const int kk = k0 + 8 * g;
            LatFrag a, b;
            a.u = kk < K ? *reinterpret_cast<const uint4*>(arow + kk) : make_uint4(0u, 0u, 0u, 0u);
            b.u = (kk < K && live) ? *reinterpret_cast<const uint4*>(brow + kk) : make_uint4(0u, 0u, 0u, 0u);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc, 0, 0, 0);
        }
        if (!live) continue;
        const int n0 = n_base + 4 * g;
        if (quads && n0 + 3 < N) {                   // a lane's four outputs in one store
            if constexpr (sizeof(TOut) == 2)
                *reinterpret_cast<uint2*>(dst + n0) = make_uint2(lat_pack2(acc[0], acc[1]), lat_pack2(acc[2], acc[3]));
            else
                *reinterpret_cast<float4*>(dst + n0) = make_float4(acc[0], acc[1], acc[2], acc[3]);
            continue;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n0 + i < N) store_f32<TOut>(dst, n0 + i, acc[i]);
    }
}

// in [tokens, .] bfloat16 (a token's rows in_ld apart, a head's part in_hs apart, both multiples of 8, as is k),
// w_t [heads, n, k] bfloat16, out bfloat16 or float32.
extern "C" int imparo_head_gemm_tiles(const void* in, int in_ld, int in_hs, const void* w_t, void* out, int out_dtype,
                                      int out_ld, int out_hs, int n_tokens, int heads, int k, int n,
                                      imparo_stream stream) {
    if (!in || !w_t || !out || n_tokens < 0 || heads < 1 || k < 8 || n < 1) return IMPARO_BAD_ARGUMENT;
    if (k % 8 || in_ld % 8 || in_hs % 8) return IMPARO_BAD_ARGUMENT;
    if (in_hs < k || in_ld < (heads - 1) * in_hs + k || out_hs < n || out_ld < (heads - 1) * out_hs + n)
        return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    const int n_tiles = (n + 15) / 16;
    const int all_z = (n_tiles + LAT_WAVES - 1) / LAT_WAVES;
    const long long xy = (long long)((n_tokens + 15) / 16) * heads;
    const int z = (int)std::min<long long>(all_z, std::max<long long>(1, (2048 + xy - 1) / xy));
    const dim3 grid((n_tokens + 15) / 16, heads, z);
    if (grid.y > 65535 || grid.z > 65535) return IMPARO_BAD_ARGUMENT;
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == IMPARO_BF16)
        k_head_gemm_tiles<bf16_t><<<grid, LAT_WAVES * WAVE, 0, s>>>((const bf16_t*)in, in_ld, in_hs, (const bf16_t*)w_t,
                                                                   (bf16_t*)out, out_ld, out_hs, n_tokens, k, n);
    else if (out_dtype == IMPARO_F32)
        k_head_gemm_tiles<float><<<grid, LAT_WAVES * WAVE, 0, s>>>((const bf16_t*)in, in_ld, in_hs, (const bf16_t*)w_t,
                                                                  (float*)out, out_ld, out_hs, n_tokens, k, n);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (a stream under capture cannot).
int imparo_load_code_latent_attention() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_latent_store<float>)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
