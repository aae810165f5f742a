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
                                                      T* __restrict__ q_plain, T* __restrict__ q_full, int heads, int dim,
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
                                   int page_size, int n_pages, void* cache, void* q_plain, void* q_full, int dtype,
                                   int n_tokens, int heads, int dim, int rot_dim, int rank, imparo_stream stream) {
    if (!q_rows || !kv_rows || !norm_weight || !positions || !q_plain || !q_full) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || heads < 1 || dim < 1 || rot_dim < 0 || rank < 1) return IMPARO_BAD_ARGUMENT;
    if (n_freq < 0 || n_freq > LAT_MAX_FREQ || 2 * n_freq > rot_dim || (n_freq && !inv_freq)) return IMPARO_BAD_ARGUMENT;
    if (cache && (!row_of_token || !block_table || table_stride < 1 || page_size < 1 || n_pages < 1)) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == IMPARO_F32)
        k_latent_store<float><<<n_tokens, 256, 0, s>>>(q_rows, kv_rows, norm_weight, eps, inv_freq, n_freq, interleaved,
                                                       positions, row_of_token, block_table, table_stride, page_size,
                                                       n_pages, (float*)cache, (float*)q_plain, (float*)q_full, heads, dim,
                                                       rot_dim, rank);
    else if (dtype == IMPARO_BF16)
        k_latent_store<bf16_t><<<n_tokens, 256, 0, s>>>(q_rows, kv_rows, norm_weight, eps, inv_freq, n_freq, interleaved,
                                                        positions, row_of_token, block_table, table_stride, page_size,
                                                        n_pages, (bf16_t*)cache, (bf16_t*)q_plain, (bf16_t*)q_full, heads,
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

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (a stream under capture cannot).
int imparo_load_code_latent_attention() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_latent_store<float>)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
