// A gated linear recurrence with a matrix of state a head (HGRN2): per head, with q = silu(zq),
// f = lower + (1 - lower) sigmoid(zf) and values v,
//   S <- diag(f) S + (1 - f) v^T,   o = S^T q,
// S [dim, vdim] float32 per request and head, carried from token to token. Gates, the state and every sum
// are float32 whatever the engine's dtype.
//
// A block takes one request's segment, one head and a run of value columns. A thread keeps a slice of one
// column of S in registers: KS neighbouring lanes share a column (each up to 16 of its dim entries), so that
// o's sum over dim ends with a few exchanges inside a wave and nothing meets across waves per token. The
// tokens' q, f and v come through LDS eight tokens at a time, with the activations taken once per element.
// Every sum runs in an order that dim alone decides: a token's result does not depend on how its
// sequence was cut into steps or on what else is in the batch.
//
// A long segment is walked in three launches instead, so that its chunks of tokens run side by side (the
// recurrence is linear in S: after a chunk, S = (product of the chunk's f) S_before + what the chunk makes of
// a zero state): every chunk but the last makes its end state from zero and the product of its gates; one
// thread a state entry then carries the true state from chunk to chunk, leaving each chunk the state it
// starts from; every chunk runs again from there and writes its tokens' results, the last one the state.
#include "common.h"
#include "api.h"

#define HG2_KPT 16            // entries of a column a thread keeps at most
#define HG2_TOKENS 8          // tokens staged in LDS at once
#define HG2_THREADS 256
#define HG2_MAX_DIM 512

__device__ __forceinline__ float hg2_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

// MODE 0: a segment from its request's state to its end. With chunks (blockIdx.x = row * max_chunks + chunk):
// MODE 1: a chunk that is not the segment's last, from a zero state: its end state goes to chunk_state, the
// product of its gates to chunk_decay, no results; MODE 2: a chunk from the state chunk_state holds for it,
// with results; the last chunk writes the request's state.
template <int KS, int MODE>
__global__ __launch_bounds__(HG2_THREADS) void k_hgrn2_scan(
    const float* __restrict__ rows, int ld, int q_off, int f_off, int v_off, const float* __restrict__ lower,
    float* __restrict__ state, const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
    const int32_t* __restrict__ slot, float* __restrict__ out, int heads, int dim, int vdim, int kpt,
    int chunk_tokens, int max_chunks, float* __restrict__ chunk_state, float* __restrict__ chunk_decay) {
    constexpr int VB = HG2_THREADS / KS;                 // value columns of a block
    __shared__ float sq[HG2_TOKENS][HG2_MAX_DIM], sf[HG2_TOKENS][HG2_MAX_DIM], sv[HG2_TOKENS][VB];
    const int r = MODE == 0 ? blockIdx.x : blockIdx.x / max_chunks;
    const int chunk = MODE == 0 ? 0 : blockIdx.x - r * max_chunks;
    const int h = blockIdx.y, v0 = blockIdx.z * VB;
    const int tid = threadIdx.x, ks = tid % KS, vl = tid / KS;
    const int v = v0 + vl;
    const bool live = v < vdim;
    const int n_all = seg_len[r];
    const int n_chunks = MODE == 0 ? 1 : (n_all + chunk_tokens - 1) / chunk_tokens;
    if (MODE == 1 && chunk >= n_chunks - 1) return;      // (the whole block)
    if (MODE == 2 && chunk >= n_chunks) return;
    const int first = seg_start[r] + (MODE == 0 ? 0 : chunk * chunk_tokens);
    const int n = MODE == 0 ? n_all : min(chunk_tokens, n_all - chunk * chunk_tokens);
    const int dkp = KS * kpt;                            // dim, filled up to whole slices
    float* S_at = state + (((size_t)slot[r] * heads + h) * dim) * vdim;
    float* C_at = MODE == 0 ? nullptr : chunk_state + (((size_t)blockIdx.x * heads + h) * dim) * vdim;
    float S[HG2_KPT], decay[MODE == 1 ? HG2_KPT : 1];
#pragma unroll
    for (int j = 0; j < HG2_KPT; ++j) {
        const int k = ks * kpt + j;
        if constexpr (MODE == 1) {
            S[j] = 0.f;
            decay[j] = 1.f;
        } else {
            S[j] = (j < kpt && k < dim && live) ? (MODE == 0 ? S_at : C_at)[(size_t)k * vdim + v] : 0.f;
        }
    }
    for (int t0 = 0; t0 < n; t0 += HG2_TOKENS) {
        const int nt = min(HG2_TOKENS, n - t0);
        __syncthreads();                                 // the last batch has been read
        for (int i = tid; i < nt * dkp; i += HG2_THREADS) {
            const int tok = i / dkp, k = i - tok * dkp;
            float q = 0.f, f = 1.f;                      // beyond dim: a state that stays zero
            if (k < dim) {
                const float* row = rows + (size_t)(first + t0 + tok) * ld;
                const float zq = row[q_off + h * dim + k], zf = row[f_off + h * dim + k];
                const float lo = lower[h * dim + k];
                q = zq * hg2_sigmoid(zq);
                f = lo + (1.0f - lo) * hg2_sigmoid(zf);
            }
            sq[tok][k] = q;
            sf[tok][k] = f;
        }
        for (int i = tid; i < nt * VB; i += HG2_THREADS) {
            const int tok = i / VB, c = i - tok * VB;
            sv[tok][c] = (v0 + c) < vdim ? rows[(size_t)(first + t0 + tok) * ld + v_off + h * vdim + v0 + c] : 0.f;
        }
        __syncthreads();
        for (int tok = 0; tok < nt; ++tok) {
            const float val = sv[tok][vl];
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < HG2_KPT; ++j) {
                if (j < kpt) {
                    const float f = sf[tok][ks * kpt + j];
                    S[j] = f * S[j] + (1.0f - f) * val;
                    if constexpr (MODE == 1)
                        decay[j] *= f;
                    else
                        acc = fmaf(S[j], sq[tok][ks * kpt + j], acc);
                }
            }
            if (MODE != 1) {
#pragma unroll
                for (int off = 1; off < KS; off <<= 1) acc += __shfl_xor(acc, off, WAVE);
                if (ks == 0 && live) out[(size_t)(first + t0 + tok) * heads * vdim + (size_t)h * vdim + v] = acc;
            }
        }
    }
    if (MODE == 2 && chunk != n_chunks - 1) return;
    float* end_at = MODE == 1 ? C_at : S_at;
#pragma unroll
    for (int j = 0; j < HG2_KPT; ++j) {
        const int k = ks * kpt + j;
        if (j < kpt && k < dim && live) end_at[(size_t)k * vdim + v] = S[j];
        if constexpr (MODE == 1)
            if (j < kpt && k < dim && vl == 0 && blockIdx.z == 0)
                chunk_decay[((size_t)blockIdx.x * heads + h) * dim + k] = decay[j];
    }
}

// One thread a state entry: the request's state walks over the chunks' ends; chunk_state[chunk] turns from
// "what the chunk makes of a zero state" into "the state the chunk starts from".
__global__ void k_hgrn2_carry(float* __restrict__ chunk_state, const float* __restrict__ chunk_decay,
                              const float* __restrict__ state, const int32_t* __restrict__ seg_len,
                              const int32_t* __restrict__ slot, int n_rows, int heads, int dim, int vdim, int chunk_tokens,
                              int max_chunks) {
    const long long per_row = (long long)heads * dim * vdim;
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_rows * per_row) return;
    const int r = (int)(i / per_row);
    const long long e = i - r * per_row;                 // (head, state row, value column)
    const long long hk = e / vdim;                       // (head, state row)
    const int n_chunks = (seg_len[r] + chunk_tokens - 1) / chunk_tokens;
    float S = state[(size_t)slot[r] * per_row + e];
    for (int c = 0; c < n_chunks; ++c) {
        float* at = chunk_state + ((size_t)r * max_chunks + c) * per_row + e;
        const bool more = c < n_chunks - 1;
        const float made = more ? *at : 0.f;
        *at = S;
        if (more) S = chunk_decay[((size_t)r * max_chunks + c) * heads * dim + hk] * S + made;
    }
}

// rows [tokens, ld] float32 holds a token's zq at q_off, zf (bias added) at f_off, v at v_off, each head by
// head; state [slots, heads, dim, vdim] float32; out [tokens, heads * vdim] float32 (before the head norm).
// chunk_tokens 0: one launch. Otherwise a multiple of 8, with max_chunks >= ceil(longest segment / chunk_tokens),
// chunk_state [n_rows * max_chunks, heads, dim, vdim] and chunk_decay [n_rows * max_chunks, heads, dim] float32.
extern "C" int imparo_hgrn2_scan(const float* rows, int ld, int q_off, int f_off, int v_off, const float* lower,
                                 float* state, const int32_t* seg_start, const int32_t* seg_len, const int32_t* slot,
                                 float* out, int n_rows, int heads, int dim, int vdim, int chunk_tokens, int max_chunks,
                                 float* chunk_state, float* chunk_decay, imparo_stream stream) {
    if (!rows || !lower || !state || !seg_start || !seg_len || !slot || !out) return IMPARO_BAD_ARGUMENT;
    if (chunk_tokens < 0 || chunk_tokens % HG2_TOKENS) return IMPARO_BAD_ARGUMENT;
    if (chunk_tokens && (max_chunks < 1 || !chunk_state || !chunk_decay)) return IMPARO_BAD_ARGUMENT;
    if (n_rows < 0 || heads < 1 || dim < 1 || dim > HG2_MAX_DIM || vdim < 1) return IMPARO_BAD_ARGUMENT;
    if (q_off < 0 || f_off < 0 || v_off < 0 || ld < q_off + heads * dim || ld < f_off + heads * dim ||
        ld < v_off + heads * vdim)
        return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    int ks = 1;
    while ((dim + ks - 1) / ks > HG2_KPT) ks *= 2;
    const int kpt = (dim + ks - 1) / ks;
    hipStream_t s = (hipStream_t)stream;
    const int vb = HG2_THREADS / ks;
    const int chunks = chunk_tokens ? max_chunks : 1;
    if ((long long)n_rows * chunks > 0x7fffffffLL) return IMPARO_BAD_ARGUMENT;
    const dim3 grid(n_rows * chunks, heads, (vdim + vb - 1) / vb);
#define HG2_PASS(KS, MODE)                                                                                           \
    k_hgrn2_scan<KS, MODE><<<grid, HG2_THREADS, 0, s>>>(rows, ld, q_off, f_off, v_off, lower, state, seg_start,      \
                                                        seg_len, slot, out, heads, dim, vdim, kpt, chunk_tokens,     \
                                                        max_chunks, chunk_state, chunk_decay)
#define HG2_LAUNCH(KS)                                                                                               \
    if (!chunk_tokens) {                                                                                             \
        HG2_PASS(KS, 0);                                                                                             \
    } else {                                                                                                         \
        HG2_PASS(KS, 1);                                                                                             \
        const long long entries = (long long)n_rows * heads * dim * vdim;                                            \
        k_hgrn2_carry<<<(unsigned)((entries + 255) / 256), 256, 0, s>>>(chunk_state, chunk_decay, state, seg_len,    \
                                                                        slot, n_rows, heads, dim, vdim,              \
                                                                        chunk_tokens, max_chunks);                   \
        HG2_PASS(KS, 2);                                                                                             \
    }
    switch (ks) {
        case 1: HG2_LAUNCH(1); break;
        case 2: HG2_LAUNCH(2); break;
        case 4: HG2_LAUNCH(4); break;
        case 8: HG2_LAUNCH(8); break;
        case 16: HG2_LAUNCH(16); break;
        case 32: HG2_LAUNCH(32); break;
        default: return IMPARO_BAD_ARGUMENT;
    }
#undef HG2_LAUNCH
#undef HG2_PASS
    return launch_status();
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (a stream under capture cannot).
int imparo_load_code_hgrn2() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_hgrn2_scan<1, 0>)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
