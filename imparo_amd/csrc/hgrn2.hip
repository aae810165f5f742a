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
#include "common.h"
#include "api.h"

#define HG2_KPT 16            // entries of a column a thread keeps at most
#define HG2_TOKENS 8          // tokens staged in LDS at once
#define HG2_THREADS 256
#define HG2_MAX_DIM 256

__device__ __forceinline__ float hg2_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

template <int KS>
__global__ __launch_bounds__(HG2_THREADS) void k_hgrn2_scan(
    const float* __restrict__ rows, int ld, int q_off, int f_off, int v_off, const float* __restrict__ lower,
    float* __restrict__ state, const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
    const int32_t* __restrict__ slot, float* __restrict__ out, int heads, int dim, int vdim, int kpt) {
    constexpr int VB = HG2_THREADS / KS;                 // value columns of a block
    __shared__ float sq[HG2_TOKENS][HG2_MAX_DIM], sf[HG2_TOKENS][HG2_MAX_DIM], sv[HG2_TOKENS][VB];
    const int r = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * VB;
    const int tid = threadIdx.x, ks = tid % KS, vl = tid / KS;
    const int v = v0 + vl;
    const bool live = v < vdim;
    const int first = seg_start[r], n = seg_len[r];
    const int dkp = KS * kpt;                            // dim, filled up to whole slices
    float* S_at = state + (((size_t)slot[r] * heads + h) * dim) * vdim;
    float S[HG2_KPT];
#pragma unroll
    for (int j = 0; j < HG2_KPT; ++j) {
        const int k = ks * kpt + j;
        S[j] = (j < kpt && k < dim && live) ? S_at[(size_t)k * vdim + v] : 0.f;
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
                    acc = fmaf(S[j], sq[tok][ks * kpt + j], acc);
                }
            }
#pragma unroll
            for (int off = 1; off < KS; off <<= 1) acc += __shfl_xor(acc, off, WAVE);
            if (ks == 0 && live) out[(size_t)(first + t0 + tok) * heads * vdim + (size_t)h * vdim + v] = acc;
        }
    }
#pragma unroll
    for (int j = 0; j < HG2_KPT; ++j) {
        const int k = ks * kpt + j;
        if (j < kpt && k < dim && live) S_at[(size_t)k * vdim + v] = S[j];
    }
}

// rows [tokens, ld] float32 holds a token's zq at q_off, zf (bias added) at f_off, v at v_off, each head by
// head; state [slots, heads, dim, vdim] float32; out [tokens, heads * vdim] float32 (before the head norm).
extern "C" int imparo_hgrn2_scan(const float* rows, int ld, int q_off, int f_off, int v_off, const float* lower,
                                 float* state, const int32_t* seg_start, const int32_t* seg_len, const int32_t* slot,
                                 float* out, int n_rows, int heads, int dim, int vdim, imparo_stream stream) {
    if (!rows || !lower || !state || !seg_start || !seg_len || !slot || !out) return IMPARO_BAD_ARGUMENT;
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
    const dim3 grid(n_rows, heads, (vdim + vb - 1) / vb);
#define HG2_LAUNCH(KS)                                                                                               \
    k_hgrn2_scan<KS><<<grid, HG2_THREADS, 0, s>>>(rows, ld, q_off, f_off, v_off, lower, state, seg_start, seg_len,   \
                                                  slot, out, heads, dim, vdim, kpt)
    switch (ks) {
        case 1: HG2_LAUNCH(1); break;
        case 2: HG2_LAUNCH(2); break;
        case 4: HG2_LAUNCH(4); break;
        case 8: HG2_LAUNCH(8); break;
        case 16: HG2_LAUNCH(16); break;
        default: return IMPARO_BAD_ARGUMENT;
    }
#undef HG2_LAUNCH
    return launch_status();
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (a stream under capture cannot).
int imparo_load_code_hgrn2() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_hgrn2_scan<1>)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
