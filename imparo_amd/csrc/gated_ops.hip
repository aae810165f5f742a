// Elementwise pieces of a parallel block with gated sublayers and a per-layer token input:
//   gated_sum   x += a * sigmoid(ga) (+ b * sigmoid(gb)); optionally also x in another dtype, for a
//               product that reads the stream itself
//   side_gate   g[t, j] = gelu_tanh(z[t, j]) * table[token[t], offset + j]
//   add_rows    x += y
//   cast_rows   the stream's rows (all, or chosen ones) in another dtype
// All sums and activations in float32, one order per element whatever the batch.
#include "common.h"
#include "api.h"

__device__ __forceinline__ float sigmoid_f32(float z) { return 1.0f / (1.0f + expf(-z)); }

__device__ __forceinline__ float gelu_tanh_f32(float z) {
    const float inner = 0.79788456080286535588f * (z + 0.044715f * z * z * z);
    return 0.5f * z * (1.0f + tanhf(inner));
}

// gates [tokens, gate_ld]: columns 0 .. width are the first sublayer's, width .. 2 width the second's. a and b
// may come as sums over slices of a product's inner size, [slices, tokens, width], added here in order.
template <typename TCopy>
__global__ void k_gated_sum(float* __restrict__ x, const float* __restrict__ a, int a_slices,
                            const float* __restrict__ b, int b_slices, const float* __restrict__ gates, int gate_ld,
                            TCopy* __restrict__ copy, int width, long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / width;
    const int c = (int)(i - t * width);
    float av = a[i];
    for (int s = 1; s < a_slices; ++s) av += a[(long long)s * total + i];
    float sum = av * sigmoid_f32(gates[t * gate_ld + c]);
    if (b) {
        float bv = b[i];
        for (int s = 1; s < b_slices; ++s) bv += b[(long long)s * total + i];
        sum += bv * sigmoid_f32(gates[t * gate_ld + width + c]);
    }
    const float v = x[i] + sum;
    x[i] = v;
    if (copy) store_f32<TCopy>(copy, (size_t)i, v);
}

extern "C" int imparo_gated_sum(float* x, const float* a, int a_slices, const float* b, int b_slices,
                                const float* gates, int gate_ld, void* copy, int copy_dtype, int n_tokens, int width,
                                imparo_stream stream) {
    if (!x || !a || !gates || n_tokens < 0 || width < 1 || gate_ld < (b ? 2 * width : width)) return IMPARO_BAD_ARGUMENT;
    if (a_slices < 1 || (b && b_slices < 1)) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    const long long total = (long long)n_tokens * width;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (copy && copy_dtype == IMPARO_BF16)
        k_gated_sum<bf16_t><<<blocks, 256, 0, s>>>(x, a, a_slices, b, b_slices, gates, gate_ld, (bf16_t*)copy, width, total);
    else if (!copy || copy_dtype == IMPARO_F32)
        k_gated_sum<float><<<blocks, 256, 0, s>>>(x, a, a_slices, b, b_slices, gates, gate_ld, (float*)copy, width, total);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

template <typename TTable, typename TOut>
__global__ void k_side_gate(const float* __restrict__ z, const TTable* __restrict__ table, int table_ld, int offset,
                            const int32_t* __restrict__ ids, int vocab, TOut* __restrict__ out, int dim, int out_ld,
                            long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / out_ld;
    const int j = (int)(i - t * out_ld);
    float g = 0.f;                       // columns dim .. out_ld are filled with zeros
    if (j < dim) {
        const int id = min(max(ids[t], 0), vocab - 1);
        g = gelu_tanh_f32(z[t * dim + j]) * load_f32<TTable>(table, (size_t)id * table_ld + offset + j);
    }
    store_f32<TOut>(out, (size_t)i, g);
}

extern "C" int imparo_side_gate(const float* z, const void* table, int table_dtype, int table_ld, int offset,
                                const int32_t* ids, int vocab, void* out, int out_dtype, int n_tokens, int dim,
                                int out_ld, imparo_stream stream) {
    if (!z || !table || !ids || !out || n_tokens < 0 || dim < 1 || out_ld < dim || vocab < 1) return IMPARO_BAD_ARGUMENT;
    if (offset < 0 || offset + dim > table_ld) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    const long long total = (long long)n_tokens * out_ld;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
#define SIDE_LAUNCH(TT, TO)                                                                                          \
    k_side_gate<TT, TO><<<blocks, 256, 0, s>>>(z, (const TT*)table, table_ld, offset, ids, vocab, (TO*)out, dim,    \
                                               out_ld, total)
    if (table_dtype == IMPARO_BF16 && out_dtype == IMPARO_BF16) SIDE_LAUNCH(bf16_t, bf16_t);
    else if (table_dtype == IMPARO_BF16 && out_dtype == IMPARO_F32) SIDE_LAUNCH(bf16_t, float);
    else if (table_dtype == IMPARO_F32 && out_dtype == IMPARO_F32) SIDE_LAUNCH(float, float);
    else if (table_dtype == IMPARO_F32 && out_dtype == IMPARO_BF16) SIDE_LAUNCH(float, bf16_t);
    else return IMPARO_BAD_ARGUMENT;
#undef SIDE_LAUNCH
    return launch_status();
}

__global__ void k_add_rows(float* __restrict__ x, const float* __restrict__ y, long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) x[i] += y[i];
}

extern "C" int imparo_add_rows(float* x, const float* y, long long n, imparo_stream stream) {
    if (!x || !y || n < 0) return IMPARO_BAD_ARGUMENT;
    if (n == 0) return IMPARO_OK;
    k_add_rows<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(x, y, n);
    return launch_status();
}

// out[i] = x[rows ? rows[i] : i] in out's dtype: the stream's rows as a product reads them, without a norm.
template <typename TOut>
__global__ void k_cast_rows(const float* __restrict__ x, const int32_t* __restrict__ rows, TOut* __restrict__ out,
                            int width, long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / width;
    const long long src = rows ? (long long)rows[t] * width + (i - t * width) : i;
    store_f32<TOut>(out, (size_t)i, x[src]);
}

extern "C" int imparo_cast_rows(const float* x, const int32_t* rows, void* out, int out_dtype, int n_out, int width,
                                imparo_stream stream) {
    if (!x || !out || n_out < 0 || width < 1) return IMPARO_BAD_ARGUMENT;
    if (out_dtype != IMPARO_F32 && out_dtype != IMPARO_BF16) return IMPARO_BAD_ARGUMENT;
    const long long n = (long long)n_out * width;
    if (n == 0) return IMPARO_OK;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (out_dtype == IMPARO_BF16)
        k_cast_rows<bf16_t><<<blocks, 256, 0, (hipStream_t)stream>>>(x, rows, (bf16_t*)out, width, n);
    else
        k_cast_rows<float><<<blocks, 256, 0, (hipStream_t)stream>>>(x, rows, (float*)out, width, n);
    return launch_status();
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (a stream under capture cannot).
int imparo_load_code_gated_ops() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_add_rows)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
