// Recurrences with a matrix of state a head and one decay a head and token:
//   S <- a S + k v^T,                 o = S^T q                  (a linear attention with decay)
//   S <- a S;  u = b (v - S^T k);  S <- S + k u^T,  o = S^T q    (the gated delta rule)
// S [dim, vdim] float32 per request and head, carried from token to token. The decay a is a constant of
// the head, or exp(-rate_h softplus(raw + bias_h)) of a projected number (the step; the values may be
// multiplied by that step, as a state-space layer does, and the head's result may take D_h x on top). b is
// the sigmoid of a projected number. Heads may share queries and keys in groups of neighbours (q_div, k_div
// heads read one). Decays, steps, gates, the state and every sum are float32 whatever the engine's dtype.
//
// A block takes one request's segment, one head and a run of value columns. A thread keeps a slice of one
// column of S in registers: KS neighbouring lanes share a column, so that the sums over dim (the delta
// rule's S^T k, every o) end with a few exchanges inside a wave. The tokens' q, k, v and scalars come
// through LDS eight tokens at a time. Every sum runs in an order that dim alone decides.
//
// A long segment of the first form is walked in three launches, its chunks side by side (the recurrence
// is linear in S with a scalar factor: after a chunk S = (product of the chunk's a) S_before + what the chunk
// makes of a zero state). The delta rule's transition is a matrix (a (I - b k k^T)): its long segments take the
// form in chunks further down (a triangle solved a chunk, then the chunks in order), short ones this walk.
//
// Beside it: what such mixers do to a head before the walk (unit length, rotation, a factor) and to the
// heads behind it (a gate and a norm in groups of the row).
#include "common.h"
#include "api.h"

#define DS_KPT 16             // entries of a column a thread keeps at most
#define DS_TOKENS 8           // tokens staged in LDS at once
#define DS_MAX_THREADS 256
#define DS_MAX_DIM 512

__device__ __forceinline__ float ds_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float ds_silu(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float ds_softplus(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

struct DecayScanArgs {
    const float* q; int q_ld, q_off, q_div;      // head h reads q head h / q_div
    const float* k; int k_ld, k_off, k_div;
    const float* v; int v_ld, v_off;
    const float* decay_const;                    // [heads], or null: the decay comes from `step`
    const float* step; int step_ld, step_off;    // raw steps [tokens, heads]
    const float* step_bias;                      // [heads]
    const float* rate;                           // [heads]: a = exp(-rate softplus(raw + bias))
    int v_times_step;                            // v <- softplus(raw + bias) v
    const float* beta; int beta_ld, beta_off;    // raw [tokens, heads], the delta rule's only
    const float* skip;                           // [heads] or null: o += skip_h v (v as it came)
    float* state;                                // [slots, heads, dim, vdim]
    const int32_t* seg_start; const int32_t* seg_len; const int32_t* slot;
    float* out;                                  // [tokens, heads * vdim]
    int heads, dim, vdim, kpt;
    int chunk_tokens, max_chunks;
    float* chunk_state;                          // [rows * max_chunks, heads, dim, vdim]
    float* chunk_decay;                          // [rows * max_chunks, heads]
};

// MODE 0: a segment from its request's state to its end. With chunks (blockIdx.x = row * max_chunks + chunk):
// MODE 1: a chunk that is not the segment's last, from a zero state: its end state goes to chunk_state, the
// product of its decays to chunk_decay, no results; MODE 2: a chunk from the state chunk_state holds for it,
// with results; the last chunk writes the request's state.
// V4: a thread's slice is whole 16-byte pieces, read as such.
template <int KS, int MODE, bool DELTA, bool V4>
__global__ __launch_bounds__(DS_MAX_THREADS) void k_decay_scan(const DecayScanArgs A) {
    __shared__ __attribute__((aligned(16))) float sq[DS_TOKENS][DS_MAX_DIM], sk[DS_TOKENS][DS_MAX_DIM];
    __shared__ float sv[DS_TOKENS][DS_MAX_THREADS];
    __shared__ float sa[DS_TOKENS], sb[DS_TOKENS], sdt[DS_TOKENS];
    const int VB = blockDim.x / KS;                      // value columns of a block
    const int r = MODE == 0 ? blockIdx.x : blockIdx.x / A.max_chunks;
    const int chunk = MODE == 0 ? 0 : blockIdx.x - r * A.max_chunks;
    const int h = blockIdx.y, v0 = blockIdx.z * VB;
    const int tid = threadIdx.x, ks = tid % KS, vl = tid / KS;
    const int v = v0 + vl;
    const int heads = A.heads, dim = A.dim, vdim = A.vdim, kpt = A.kpt;
    const bool live = v < vdim;
    const int n_all = A.seg_len[r];
    const int n_chunks = MODE == 0 ? 1 : (n_all + A.chunk_tokens - 1) / A.chunk_tokens;
    if (MODE == 1 && chunk >= n_chunks - 1) return;      // (the whole block)
    if (MODE == 2 && chunk >= n_chunks) return;
    const int first = A.seg_start[r] + (MODE == 0 ? 0 : chunk * A.chunk_tokens);
    const int n = MODE == 0 ? n_all : min(A.chunk_tokens, n_all - chunk * A.chunk_tokens);
    const int dkp = KS * kpt;                            // dim, filled up to whole slices
    const int qh = h / A.q_div, kh = h / A.k_div;
    float* S_at = A.state + (((size_t)A.slot[r] * heads + h) * dim) * vdim;
    float* C_at = MODE == 0 ? nullptr : A.chunk_state + (((size_t)blockIdx.x * heads + h) * dim) * vdim;
    float S[DS_KPT];
    float decay_all = 1.f;
#pragma unroll
    for (int j = 0; j < DS_KPT; ++j) {
        const int k = ks * kpt + j;
        if constexpr (MODE == 1)
            S[j] = 0.f;
        else
            S[j] = (j < kpt && k < dim && live) ? (MODE == 0 ? S_at : C_at)[(size_t)k * vdim + v] : 0.f;
    }
    const float skip = A.skip ? A.skip[h] : 0.f;
    for (int t0 = 0; t0 < n; t0 += DS_TOKENS) {
        const int nt = min(DS_TOKENS, n - t0);
        __syncthreads();                                 // the last batch has been read
        for (int i = tid; i < nt * dkp; i += blockDim.x) {
            const int tok = i / dkp, k = i - tok * dkp;
            const size_t t = (size_t)(first + t0 + tok);
            sq[tok][k] = k < dim ? A.q[t * A.q_ld + A.q_off + qh * dim + k] : 0.f;   // beyond dim: a state that stays zero
            sk[tok][k] = k < dim ? A.k[t * A.k_ld + A.k_off + kh * dim + k] : 0.f;
        }
        for (int i = tid; i < nt * VB; i += blockDim.x) {
            const int tok = i / VB, c = i - tok * VB;
            sv[tok][c] = (v0 + c) < vdim ? A.v[(size_t)(first + t0 + tok) * A.v_ld + A.v_off + h * vdim + v0 + c] : 0.f;
        }
        if (tid < nt) {
            const size_t t = (size_t)(first + t0 + tid);
            float a, dt = 1.f;
            if (A.decay_const) {
                a = A.decay_const[h];
            } else {
                dt = ds_softplus(A.step[t * A.step_ld + A.step_off + h] + A.step_bias[h]);
                a = expf(-A.rate[h] * dt);
            }
            sa[tid] = a;
            sdt[tid] = A.v_times_step ? dt : 1.f;
            sb[tid] = DELTA ? ds_sigmoid(A.beta[t * A.beta_ld + A.beta_off + h]) : 1.f;
        }
        __syncthreads();
        for (int tok = 0; tok < nt; ++tok) {
            const float a = sa[tok];
            const float raw = sv[tok][vl];
            float val = raw * sdt[tok];
            float acc = 0.f;
            float kk[DS_KPT], qq[DS_KPT];
            if constexpr (V4) {
#pragma unroll
                for (int j = 0; j < DS_KPT; j += 4)
                    if (j < kpt) {
                        const float4 k4 = *reinterpret_cast<const float4*>(&sk[tok][ks * kpt + j]);
                        const float4 q4 = *reinterpret_cast<const float4*>(&sq[tok][ks * kpt + j]);
                        kk[j] = k4.x, kk[j + 1] = k4.y, kk[j + 2] = k4.z, kk[j + 3] = k4.w;
                        qq[j] = q4.x, qq[j + 1] = q4.y, qq[j + 2] = q4.z, qq[j + 3] = q4.w;
                    }
            } else {
#pragma unroll
                for (int j = 0; j < DS_KPT; ++j)
                    if (j < kpt) {
                        kk[j] = sk[tok][ks * kpt + j];
                        qq[j] = sq[tok][ks * kpt + j];
                    }
            }
            if constexpr (DELTA) {
                float seen = 0.f;
#pragma unroll
                for (int j = 0; j < DS_KPT; ++j)
                    if (j < kpt) {
                        S[j] *= a;
                        seen = fmaf(S[j], kk[j], seen);
                    }
#pragma unroll
                for (int off = 1; off < KS; off <<= 1) seen += __shfl_xor(seen, off, WAVE);
                val = sb[tok] * (val - seen);
#pragma unroll
                for (int j = 0; j < DS_KPT; ++j)
                    if (j < kpt) {
                        S[j] = fmaf(kk[j], val, S[j]);
                        acc = fmaf(S[j], qq[j], acc);
                    }
            } else {
#pragma unroll
                for (int j = 0; j < DS_KPT; ++j)
                    if (j < kpt) {
                        S[j] = fmaf(kk[j], val, a * S[j]);
                        if constexpr (MODE != 1) acc = fmaf(S[j], qq[j], acc);
                    }
                if constexpr (MODE == 1) decay_all *= a;
            }
            if (MODE != 1) {
#pragma unroll
                for (int off = 1; off < KS; off <<= 1) acc += __shfl_xor(acc, off, WAVE);
                if (ks == 0 && live)
                    A.out[(size_t)(first + t0 + tok) * heads * vdim + (size_t)h * vdim + v] = fmaf(skip, raw, acc);
            }
        }
    }
    if (MODE == 2 && chunk != n_chunks - 1) return;
    float* end_at = MODE == 1 ? C_at : S_at;
#pragma unroll
    for (int j = 0; j < DS_KPT; ++j) {
        const int k = ks * kpt + j;
        if (j < kpt && k < dim && live) end_at[(size_t)k * vdim + v] = S[j];
    }
    if (MODE == 1 && tid == 0 && blockIdx.z == 0) A.chunk_decay[(size_t)blockIdx.x * heads + h] = decay_all;
}

// One thread a state entry: the request's state walks over the chunks' ends; chunk_state[chunk] turns from
// "what the chunk makes of a zero state" into "the state the chunk starts from".
__global__ void k_decay_carry(float* __restrict__ chunk_state, const float* __restrict__ chunk_decay,
                              const float* __restrict__ state, const int32_t* __restrict__ seg_len,
                              const int32_t* __restrict__ slot, int n_rows, int heads, int dim, int vdim,
                              int chunk_tokens, int max_chunks) {
    const long long per_head = (long long)dim * vdim, per_row = per_head * heads;
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_rows * per_row) return;
    const int r = (int)(i / per_row);
    const long long e = i - r * per_row;
    const int h = (int)(e / per_head);
    const int n_chunks = (seg_len[r] + chunk_tokens - 1) / chunk_tokens;
    float S = state[(size_t)slot[r] * per_row + e];
    for (int c = 0; c < n_chunks; ++c) {
        float* at = chunk_state + ((size_t)r * max_chunks + c) * per_row + e;
        const bool more = c < n_chunks - 1;
        const float made = more ? *at : 0.f;
        *at = S;
        if (more) S = fmaf(chunk_decay[((size_t)r * max_chunks + c) * heads + h], S, made);
    }
}

// ---------------------------------------------------------------- the delta rule in chunks
// Inside a chunk of DC tokens that starts from the state S0, with g_t the product of the decays from the
// chunk's start up to token t:
//   u_t = b_t (v_t - g_t S0^T k_t - sum_{j<t} (g_t / g_j) (k_t . k_j) u_j)        (I + L) U = diag(b) (V - P),
//   o_t = g_t S0^T q_t + sum_{j<=t} (g_t / g_j) (q_t . k_j) u_j                     O = Qs + M U,
//   S_end = g_last S0 + sum_j (g_last / g_j) k_j u_j^T.
// A first launch makes, for every chunk of every segment and head side by side, T = (I + L)^-1 diag(b) (a lower
// triangle, by forward substitution, a column a thread), M and the logarithms of g (sums of -rate * step, so
// that every ratio is the exponential of a difference and at most one). A second launch walks a segment's
// chunks in order with the state in LDS, a block a (segment, head, run of DVB value columns): four small
// products a chunk on the vector units, every sum in an order the sizes alone decide. Tokens past a segment's
// end count as k = q = 0, b = 0 and a decay of one: they change nothing.
#define DC 32                 // tokens a chunk
#define DVB 32                // value columns a block of the walk
#define DMAXK 128             // state rows a head at most, in this form

// PLAIN: the recurrence without the delta rule's correction (b = 1, no triangle): M, log g and the steps only.
template <bool PLAIN>
__global__ __launch_bounds__(256) void k_delta_chunk_prepare(const DecayScanArgs A) {
    __shared__ float sk[DC][DMAXK + 1], sq[DC][DMAXK + 1], sL[PLAIN ? 1 : DC][DC + 1], lg[DC], sb[DC];
    const int r = blockIdx.x / A.max_chunks, chunk = blockIdx.x - r * A.max_chunks, h = blockIdx.y;
    const int tid = threadIdx.x, dim = A.dim, heads = A.heads;
    const int n_all = A.seg_len[r];
    if (chunk * DC >= n_all) return;                     // (the whole block)
    const int first = A.seg_start[r] + chunk * DC, n = min(DC, n_all - chunk * DC);
    const int qh = h / A.q_div, kh = h / A.k_div;
    for (int i = tid; i < DC * dim; i += 256) {
        const int t = i / dim, k = i - t * dim;
        const size_t row = (size_t)(first + min(t, n - 1));
        const float kv = A.k[row * A.k_ld + A.k_off + kh * dim + k], qv = A.q[row * A.q_ld + A.q_off + qh * dim + k];
        sk[t][k] = t < n ? kv : 0.f;
        sq[t][k] = t < n ? qv : 0.f;
    }
    if (tid < DC) {
        float la = 0.f, b = 0.f, dt = 1.f;
        if (tid < n) {
            const size_t row = (size_t)(first + tid);
            if (A.decay_const) {
                la = logf(fmaxf(A.decay_const[h], 1e-30f));
            } else {
                dt = ds_softplus(A.step[row * A.step_ld + A.step_off + h] + A.step_bias[h]);
                la = -A.rate[h] * dt;
            }
            if constexpr (!PLAIN) b = ds_sigmoid(A.beta[row * A.beta_ld + A.beta_off + h]);
        }
        lg[tid] = la;
        sb[tid] = b;
        // the steps, for a walk that multiplies its values by them
        A.chunk_decay[((size_t)blockIdx.x * A.heads + h) * (2 * DC) + DC + tid] = dt;
    }
    __syncthreads();
    if (tid == 0) {
        float sum = 0.f;
        for (int t = 0; t < DC; ++t) {
            sum += lg[t];
            lg[t] = sum;
        }
    }
    __syncthreads();
    const size_t at = ((size_t)blockIdx.x * heads + h);
    float* T_out = A.chunk_state + at * (2 * DC * DC);
    float* M_out = T_out + DC * DC;
    for (int i = tid; i < DC * DC; i += 256) {
        const int t = i / DC, j = i - t * DC;
        float kk = 0.f, qk = 0.f;
        if (j <= t) {
            for (int k = 0; k < dim; ++k) {
                if constexpr (!PLAIN) kk = fmaf(sk[t][k], sk[j][k], kk);
                qk = fmaf(sq[t][k], sk[j][k], qk);
            }
            const float w = expf(lg[t] - lg[j]);
            kk *= w * sb[t];
            qk *= w;
        }
        if constexpr (!PLAIN) sL[t][j] = j < t ? kk : 0.f;
        M_out[i] = qk;
    }
    if (tid < DC) A.chunk_decay[at * (2 * DC) + tid] = lg[tid];
    if constexpr (PLAIN) return;
    __syncthreads();
    if (tid < DC) {
        // column tid of (I + L)^-1 by forward substitution, then times b of that column
        float x[DC];
#pragma unroll
        for (int t = 0; t < DC; ++t) {
            float acc = t == tid ? 1.f : 0.f;
#pragma unroll
            for (int j = 0; j < t; ++j) acc = fmaf(-sL[t][j], x[j], acc);
            x[t] = acc;
        }
        const float b = sb[tid];
#pragma unroll
        for (int t = 0; t < DC; ++t) T_out[t * DC + tid] = x[t] * b;
    }
}

// What a block of the walk asks of memory for one chunk, in registers: asked for while the chunk before is worked on.
#define DPIECES (DC * DMAXK / 256)        // elements of a chunk's K (and Q) a thread brings at most
struct DeltaFetch {
    float k[DPIECES], q[DPIECES], t[DC * DC / 256], m[DC * DC / 256], v[DC / 8], dt[DC / 8], l, last;
};

template <int VB, bool PLAIN>
__global__ __launch_bounds__(256) void k_delta_chunk_scan(const DecayScanArgs A) {
    constexpr int KLD = DMAXK + 4;                       // floats between two tokens' rows: whole 16-byte pieces
    constexpr int NG = 256 / VB;                         // threads a value column: each takes every NG-th token
    constexpr int TPT = DC / NG;                         // tokens of a chunk a thread takes
    constexpr int KPT = DMAXK / NG;                      // state rows of its column a thread takes at most
    __shared__ __attribute__((aligned(16))) float sk[DC][KLD], sq[DC][KLD];
    __shared__ float sS[DMAXK][VB], sU[DC][VB], sT[PLAIN ? 1 : DC][DC], sM[DC][DC], sg[DC], sw[DC];
    float (*sR)[VB] = reinterpret_cast<float (*)[VB]>(&sq[0][0]);        // R lies where Q lay, once Q has been used
    const int r = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * VB;
    const int tid = threadIdx.x, v = tid % VB, g = tid / VB;
    const int heads = A.heads, dim = A.dim, vdim = A.vdim;
    const int dim4 = (dim + 3) & ~3;
    const bool live = v0 + v < vdim;
    const int n_all = A.seg_len[r], n_chunks = (n_all + DC - 1) / DC;
    const int qh = h / A.q_div, kh = h / A.k_div;
    float* S_at = A.state + (((size_t)A.slot[r] * heads + h) * dim) * vdim;
    for (int i = tid; i < dim4 * VB; i += 256) {
        const int k = i / VB, c = i - k * VB;
        sS[k][c] = (k < dim && (v0 + c) < vdim) ? S_at[(size_t)k * vdim + v0 + c] : 0.f;
    }
    // which (token, state row) of a chunk's K and Q this thread brings: the same for every chunk
    int piece_t[DPIECES];
#pragma unroll
    for (int it = 0; it < DPIECES; ++it) piece_t[it] = min((tid + 256 * it) / dim4, DC - 1);
    DeltaFetch f;
    // every address is clamped into the segment (no load under a branch); what lies beyond is zeroed when it is used
    auto fetch = [&](int chunk) {
        const int first = A.seg_start[r] + chunk * DC, n = min(DC, n_all - chunk * DC);
        const size_t at = ((size_t)(r * A.max_chunks + chunk) * heads + h);
        const float* T_in = A.chunk_state + at * (2 * DC * DC);
#pragma unroll
        for (int it = 0; it < DPIECES; ++it) {
            const int t = piece_t[it], k = min(max(tid + 256 * it - t * dim4, 0), dim - 1);
            const size_t row = (size_t)(first + min(t, n - 1));
            f.k[it] = A.k[row * A.k_ld + A.k_off + kh * dim + k];
            f.q[it] = A.q[row * A.q_ld + A.q_off + qh * dim + k];
        }
#pragma unroll
        for (int it = 0; it < DC * DC / 256; ++it) {
            if constexpr (!PLAIN) f.t[it] = T_in[tid + 256 * it];
            f.m[it] = T_in[DC * DC + tid + 256 * it];
        }
        f.l = A.chunk_decay[at * (2 * DC) + (tid & (DC - 1))];
        f.last = A.chunk_decay[at * (2 * DC) + DC - 1];
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
            const int t = min(g + NG * i, n - 1);
            f.v[i] = A.v[(size_t)(first + t) * A.v_ld + A.v_off + h * vdim + min(v0 + v, vdim - 1)];
            f.dt[i] = A.chunk_decay[at * (2 * DC) + DC + t];
        }
    };
    fetch(0);
    const int kpt = (((dim4 + NG - 1) / NG) + 3) & ~3;   // this thread's state rows: kpt from g * kpt on
    const float skip = (PLAIN && A.skip) ? A.skip[h] : 0.f;
    for (int chunk = 0; chunk < n_chunks; ++chunk) {
        const int first = A.seg_start[r] + chunk * DC, n = min(DC, n_all - chunk * DC);
        __syncthreads();                                 // the chunk before has been used, the state is whole
#pragma unroll
        for (int it = 0; it < DPIECES; ++it) {
            const int i = tid + 256 * it, t = piece_t[it], k = i - t * dim4;
            if (i < DC * dim4) {
                const bool on = t < n && k < dim;
                sk[t][k] = on ? f.k[it] : 0.f;
                sq[t][k] = on ? f.q[it] : 0.f;
            }
        }
#pragma unroll
        for (int it = 0; it < DC * DC / 256; ++it) {
            const int i = tid + 256 * it;
            if constexpr (!PLAIN) sT[i / DC][i % DC] = f.t[it];
            sM[i / DC][i % DC] = f.m[it];
        }
        if (tid < DC) {
            sg[tid] = expf(f.l);
            sw[tid] = expf(f.last - f.l);
        }
        float vt[TPT], dts[TPT];
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
            vt[i] = (g + NG * i < n && live) ? f.v[i] : 0.f;
            dts[i] = f.dt[i];
        }
        __syncthreads();
        fetch(min(chunk + 1, n_chunks - 1));             // on its way while this chunk is worked on (no load under a branch)
        // what the state says of the chunk's keys and queries
        float p[TPT], s[TPT];
#pragma unroll
        for (int i = 0; i < TPT; ++i) p[i] = s[i] = 0.f;
#pragma unroll 4
        for (int k = 0; k < dim4; k += 4) {
            const float s0 = sS[k][v], s1 = sS[k + 1][v], s2 = sS[k + 2][v], s3 = sS[k + 3][v];
#pragma unroll
            for (int i = 0; i < TPT; ++i) {
                const float4 kk = *reinterpret_cast<const float4*>(&sk[g + NG * i][k]);
                const float4 qq = *reinterpret_cast<const float4*>(&sq[g + NG * i][k]);
                if constexpr (!PLAIN) p[i] = fmaf(kk.w, s3, fmaf(kk.z, s2, fmaf(kk.y, s1, fmaf(kk.x, s0, p[i]))));
                s[i] = fmaf(qq.w, s3, fmaf(qq.z, s2, fmaf(qq.y, s1, fmaf(qq.x, s0, s[i]))));
            }
        }
        __syncthreads();                                 // K and Q have been used: R goes where Q lay, K takes its weights
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
            const int t = g + NG * i;
            if constexpr (PLAIN)
                sU[t][v] = A.v_times_step ? vt[i] * dts[i] : vt[i];     // no correction: what is written is the value itself
            else
                sR[t][v] = vt[i] - sg[t] * p[i];
            s[i] *= sg[t];
        }
        for (int i = tid; i < DC * dim4; i += 256) sk[i / dim4][i % dim4] *= sw[i / dim4];
        __syncthreads();
        // (T and M are zero above their diagonals: the sums run over the whole chunk, so that the reads of
        // several steps can be under way at once; a product with zero adds nothing)
        if constexpr (!PLAIN) {
            float u[TPT];
#pragma unroll
            for (int i = 0; i < TPT; ++i) u[i] = 0.f;
#pragma unroll 8
            for (int j = 0; j < DC; ++j) {
                const float rv = sR[j][v];
#pragma unroll
                for (int i = 0; i < TPT; ++i) u[i] = fmaf(sT[g + NG * i][j], rv, u[i]);
            }
#pragma unroll
            for (int i = 0; i < TPT; ++i) sU[g + NG * i][v] = u[i];
            __syncthreads();
        }
#pragma unroll 8
        for (int j = 0; j < DC; ++j) {
            const float uv = sU[j][v];
#pragma unroll
            for (int i = 0; i < TPT; ++i) s[i] = fmaf(sM[g + NG * i][j], uv, s[i]);
        }
#pragma unroll
        for (int i = 0; i < TPT; ++i) {
            const int t = g + NG * i;
            if (t < n && live)
                A.out[(size_t)(first + t) * heads * vdim + (size_t)h * vdim + v0 + v] = PLAIN ? fmaf(skip, vt[i], s[i]) : s[i];
        }
        // the state behind the chunk: this thread's rows of its column
        const float g_last = sg[DC - 1];
        float acc[KPT];
#pragma unroll
        for (int m = 0; m < KPT; ++m) acc[m] = (m < kpt && g * kpt + m < dim4) ? g_last * sS[g * kpt + m][v] : 0.f;
#pragma unroll 4
        for (int j = 0; j < DC; ++j) {
            const float u = sU[j][v];
#pragma unroll
            for (int m = 0; m < KPT; m += 4)
                if (m < kpt && g * kpt + m < dim4) {
                    const float4 w = *reinterpret_cast<const float4*>(&sk[j][g * kpt + m]);
                    acc[m] = fmaf(w.x, u, acc[m]);
                    acc[m + 1] = fmaf(w.y, u, acc[m + 1]);
                    acc[m + 2] = fmaf(w.z, u, acc[m + 2]);
                    acc[m + 3] = fmaf(w.w, u, acc[m + 3]);
                }
        }
#pragma unroll
        for (int m = 0; m < KPT; ++m)
            if (m < kpt && g * kpt + m < dim4) sS[g * kpt + m][v] = acc[m];
    }
    __syncthreads();
    for (int i = tid; i < dim * VB; i += 256) {
        const int k = i / VB, c = i - k * VB;
        if (v0 + c < vdim) S_at[(size_t)k * vdim + v0 + c] = sS[k][c];
    }
}

extern "C" int imparo_delta_chunk_tokens() { return DC; }
extern "C" int imparo_delta_chunk_max_dim() { return DMAXK; }

extern "C" int imparo_decay_scan(const float* q, int q_ld, int q_off, int q_div, const float* k, int k_ld, int k_off,
                                 int k_div, const float* v, int v_ld, int v_off, const float* decay_const,
                                 const float* step, int step_ld, int step_off, const float* step_bias,
                                 const float* rate, int v_times_step, const float* beta, int beta_ld, int beta_off,
                                 const float* skip, float* state, const int32_t* seg_start, const int32_t* seg_len,
                                 const int32_t* slot, float* out, int n_rows, int heads, int dim, int vdim,
                                 int chunk_tokens, int max_chunks, float* chunk_state, float* chunk_decay,
                                 imparo_stream stream) {
    if (!q || !k || !v || !state || !seg_start || !seg_len || !slot || !out) return IMPARO_BAD_ARGUMENT;
    if (!decay_const && (!step || !step_bias || !rate)) return IMPARO_BAD_ARGUMENT;
    if (v_times_step && decay_const) return IMPARO_BAD_ARGUMENT;
    if (chunk_tokens < 0 || chunk_tokens % DS_TOKENS) return IMPARO_BAD_ARGUMENT;
    if (chunk_tokens && (max_chunks < 1 || !chunk_state || !chunk_decay)) return IMPARO_BAD_ARGUMENT;
    if (chunk_tokens && beta && (chunk_tokens != DC || dim > DMAXK || decay_const)) return IMPARO_BAD_ARGUMENT;
    if (chunk_tokens == DC && dim > DMAXK) return IMPARO_BAD_ARGUMENT;
    if (n_rows < 0 || heads < 1 || dim < 1 || dim > DS_MAX_DIM || vdim < 1) return IMPARO_BAD_ARGUMENT;
    if (q_div < 1 || k_div < 1 || heads % q_div || heads % k_div) return IMPARO_BAD_ARGUMENT;
    if (q_off < 0 || k_off < 0 || v_off < 0 || q_ld < q_off + heads / q_div * dim || k_ld < k_off + heads / k_div * dim ||
        v_ld < v_off + heads * vdim)
        return IMPARO_BAD_ARGUMENT;
    if (step && (step_off < 0 || step_ld < step_off + heads)) return IMPARO_BAD_ARGUMENT;
    if (beta && (beta_off < 0 || beta_ld < beta_off + heads)) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    int ks = 1;
    while ((dim + ks - 1) / ks > DS_KPT) ks *= 2;
    const int kpt = (dim + ks - 1) / ks;
    hipStream_t s = (hipStream_t)stream;
    // a block is as many value columns as fill it, in whole waves
    int threads = (ks * vdim + WAVE - 1) / WAVE * WAVE;
    threads = threads > DS_MAX_THREADS ? DS_MAX_THREADS : threads;
    const int vb = threads / ks;
    const int chunks = chunk_tokens ? max_chunks : 1;
    if ((long long)n_rows * chunks > 0x7fffffffLL) return IMPARO_BAD_ARGUMENT;
    const dim3 grid(n_rows * chunks, heads, (vdim + vb - 1) / vb);
    const DecayScanArgs args{q, q_ld, q_off, q_div, k, k_ld, k_off, k_div, v, v_ld, v_off, decay_const,
                             step, step_ld, step_off, step_bias, rate, v_times_step, beta, beta_ld, beta_off, skip,
                             state, seg_start, seg_len, slot, out, heads, dim, vdim, kpt,
                             chunk_tokens, max_chunks, chunk_state, chunk_decay};
    if (chunk_tokens == DC && dim <= DMAXK) {
        // the chunks of a segment in order, small products a chunk: chunk_state holds T and M of every chunk,
        // chunk_decay the logarithms of its decays and its steps
        if (beta && (v_times_step || skip)) return IMPARO_BAD_ARGUMENT;
        const dim3 pgrid(n_rows * max_chunks, heads);
        if (beta) k_delta_chunk_prepare<false><<<pgrid, 256, 0, s>>>(args);
        else k_delta_chunk_prepare<true><<<pgrid, 256, 0, s>>>(args);
        // few blocks (a segment, few heads): narrower runs of columns make more of them
        // (a column's arithmetic is the same whatever the width of its run: the same bits)
        const long long rh = (long long)n_rows * heads;
#define DCS(VB)                                                                                                      \
    if (beta) k_delta_chunk_scan<VB, false><<<dim3(n_rows, heads, (vdim + VB - 1) / VB), 256, 0, s>>>(args);        \
    else k_delta_chunk_scan<VB, true><<<dim3(n_rows, heads, (vdim + VB - 1) / VB), 256, 0, s>>>(args)
        if (rh * ((vdim + DVB - 1) / DVB) >= 512 || vdim <= 8) { DCS(DVB); }
        else if (rh * ((vdim + 15) / 16) >= 512) { DCS(16); }
        else { DCS(8); }
#undef DCS
        return launch_status();
    }
#define DS_PASS(KS, MODE, DELTA)                                                                                     \
    if (kpt % 4 == 0)                                                                                                \
        k_decay_scan<KS, MODE, DELTA, true><<<grid, threads, 0, s>>>(args);                                         \
    else                                                                                                             \
        k_decay_scan<KS, MODE, DELTA, false><<<grid, threads, 0, s>>>(args)
#define DS_LAUNCH(KS)                                                                                                \
    if (beta) {                                                                                                      \
        DS_PASS(KS, 0, true);                                                                                        \
    } else if (!chunk_tokens) {                                                                                      \
        DS_PASS(KS, 0, false);                                                                                       \
    } else {                                                                                                         \
        DS_PASS(KS, 1, false);                                                                                       \
        const long long entries = (long long)n_rows * heads * dim * vdim;                                            \
        k_decay_carry<<<(unsigned)((entries + 255) / 256), 256, 0, s>>>(chunk_state, chunk_decay, state, seg_len,    \
                                                                        slot, n_rows, heads, dim, vdim,              \
                                                                        chunk_tokens, max_chunks);                   \
        DS_PASS(KS, 2, false);                                                                                       \
    }
    switch (ks) {
        case 1: DS_LAUNCH(1); break;
        case 2: DS_LAUNCH(2); break;
        case 4: DS_LAUNCH(4); break;
        case 8: DS_LAUNCH(8); break;
        case 16: DS_LAUNCH(16); break;
        case 32: DS_LAUNCH(32); break;
        default: return IMPARO_BAD_ARGUMENT;
    }
#undef DS_LAUNCH
#undef DS_PASS
    return launch_status();
}

// ---------------------------------------------------------------- a head before the walk
// One wave per (token, head) over rows [tokens, ld] float32, in place: head j is the `dim` columns from
// off + j dim. `unit`: the head is divided by sqrt(sum of its squares + unit_eps). Then the first 2 n_freq
// dimensions are rotated by position (pairs (i, i + n_freq), or neighbours (2i, 2i + 1)), then the head is
// multiplied by scale_first (heads below n_first) or scale_rest.
__global__ void k_head_prepare(float* __restrict__ rows, int ld, int off, int n_tokens, int heads, int dim, int unit,
                               float unit_eps, const float* __restrict__ inv_freq, int n_freq, int interleaved,
                               const int32_t* __restrict__ positions, int n_first, float scale_first,
                               float scale_rest) {
    const int lane = threadIdx.x & (WAVE - 1);
    const long long id = (long long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (id >= (long long)n_tokens * heads) return;
    const int t = (int)(id / heads), j = (int)(id - (long long)t * heads);
    float* x = rows + (size_t)t * ld + off + (size_t)j * dim;
    float f = j < n_first ? scale_first : scale_rest;
    if (unit) {
        float ss = 0.f;
        for (int i = lane; i < dim; i += WAVE) ss = fmaf(x[i], x[i], ss);
        f *= 1.0f / sqrtf(wave_sum(ss) + unit_eps);
    }
    const int pos = n_freq ? positions[t] : 0;
    for (int i = lane; i < n_freq; i += WAVE) {
        const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + n_freq;
        float sn, cs;
        rotation_of(pos, inv_freq[i], sn, cs);
        const float a = x[ia], b = x[ib];
        x[ia] = (a * cs - b * sn) * f;
        x[ib] = (b * cs + a * sn) * f;
    }
    for (int i = 2 * n_freq + lane; i < dim; i += WAVE) x[i] *= f;
}

extern "C" int imparo_head_prepare(float* rows, int ld, int off, int n_tokens, int heads, int dim, int unit,
                                   float unit_eps, const float* inv_freq, int n_freq, int interleaved,
                                   const int32_t* positions, int n_first, float scale_first, float scale_rest,
                                   imparo_stream stream) {
    if (!rows || n_tokens < 0 || heads < 1 || dim < 1 || off < 0 || ld < off + heads * dim) return IMPARO_BAD_ARGUMENT;
    if (n_freq < 0 || 2 * n_freq > dim || (n_freq && (!inv_freq || !positions))) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    const long long waves = (long long)n_tokens * heads;
    k_head_prepare<<<(unsigned)((waves + 3) / 4), 4 * WAVE, 0, (hipStream_t)stream>>>(
        rows, ld, off, n_tokens, heads, dim, unit, unit_eps, inv_freq, n_freq, interleaved, positions, n_first,
        scale_first, scale_rest);
    return launch_status();
}

// ---------------------------------------------------------------- the heads behind the walk
// out[t, c] for a row of `width` values in `groups` equal parts: with y = x[t, c] and g = silu(gate[t, c]),
//   gate_first: (y g) / rms_part(y g) * w[c];   otherwise: y / rms_part(y) * w[c] * g     (w null: 1).
// A wave takes a part; for long parts a block does, with the part in registers (PER values a thread, every load
// asked for before any is used, the gate's activation taken once).
template <typename TOut>
__global__ __launch_bounds__(256) void k_gated_group_norm(const float* __restrict__ x, const float* __restrict__ gate,
                                                          int gate_ld, int gate_off, const float* __restrict__ w,
                                                          TOut* __restrict__ out, int n_tokens, int width, int groups,
                                                          float eps, int gate_first) {
    const int part = width / groups;
    const long long id = (long long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    const int first = threadIdx.x & (WAVE - 1);
    if (id >= (long long)n_tokens * groups) return;
    const int t = (int)(id / groups), g = (int)(id - (long long)t * groups);
    const float* xr = x + (size_t)t * width + (size_t)g * part;
    const float* gr = gate ? gate + (size_t)t * gate_ld + gate_off + (size_t)g * part : nullptr;
    float ss = 0.f;
#pragma unroll 4
    for (int i = first; i < part; i += WAVE) {
        float y = xr[i];
        if (gate_first && gr) y *= ds_silu(gr[i]);
        ss = fmaf(y, y, ss);
    }
    ss = wave_sum(ss);
    const float rs = 1.0f / sqrtf(ss / (float)part + eps);
#pragma unroll 4
    for (int i = first; i < part; i += WAVE) {
        float y = xr[i];
        const float gv = gr ? ds_silu(gr[i]) : 1.f;
        if (gate_first) y *= gv;
        y = y * rs * (w ? w[(size_t)g * part + i] : 1.f);
        if (!gate_first) y *= gv;
        store_f32<TOut>(out, (size_t)t * width + (size_t)g * part + i, y);
    }
}

template <typename TOut, int PER>
__global__ __launch_bounds__(256) void k_gated_group_norm_block(const float* __restrict__ x, const float* __restrict__ gate,
                                                                int gate_ld, int gate_off, const float* __restrict__ w,
                                                                TOut* __restrict__ out, int width, int groups, float eps,
                                                                int gate_first) {
    __shared__ float scratch[16];
    const int part = width / groups;
    const int t = blockIdx.x / groups, g = blockIdx.x - t * groups;
    const float* xr = x + (size_t)t * width + (size_t)g * part;
    const float* gr = gate ? gate + (size_t)t * gate_ld + gate_off + (size_t)g * part : nullptr;
    float y[PER], gv[PER], wv[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = min((int)threadIdx.x + j * 256, part - 1);
        y[j] = xr[i];
        gv[j] = gr ? gr[i] : 0.f;
        wv[j] = w ? w[(size_t)g * part + i] : 1.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        gv[j] = gr ? ds_silu(gv[j]) : 1.f;
        if (gate_first) y[j] *= gv[j];
        if ((int)threadIdx.x + j * 256 < part) ss = fmaf(y[j], y[j], ss);
    }
    const float rs = 1.0f / sqrtf(block_sum(ss, scratch) / (float)part + eps);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + j * 256;
        float v = y[j] * rs * wv[j];
        if (!gate_first) v *= gv[j];
        if (i < part) store_f32<TOut>(out, (size_t)t * width + (size_t)g * part + i, v);
    }
}

extern "C" int imparo_gated_group_norm(const float* x, const float* gate, int gate_ld, int gate_off, const float* w,
                                       void* out, int out_dtype, int n_tokens, int width, int groups, float eps,
                                       int gate_first, imparo_stream stream) {
    if (!x || !out || n_tokens < 0 || width < 1 || groups < 1 || width % groups) return IMPARO_BAD_ARGUMENT;
    if (gate && (gate_off < 0 || gate_ld < gate_off + width)) return IMPARO_BAD_ARGUMENT;
    if (out_dtype != IMPARO_F32 && out_dtype != IMPARO_BF16) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const long long parts = (long long)n_tokens * groups;
    if (parts > 0x7fffffffLL) return IMPARO_BAD_ARGUMENT;
    const int part = width / groups;
    if (part > 512 && part <= 256 * 64) {
#define GGN_BLOCK(T, PER)                                                                                            \
    k_gated_group_norm_block<T, PER><<<(unsigned)parts, 256, 0, s>>>(x, gate, gate_ld, gate_off, w, (T*)out, width, \
                                                                     groups, eps, gate_first)
#define GGN_PER(T)                                                                                                   \
    if (part <= 256 * 4) GGN_BLOCK(T, 4);                                                                            \
    else if (part <= 256 * 8) GGN_BLOCK(T, 8);                                                                       \
    else if (part <= 256 * 16) GGN_BLOCK(T, 16);                                                                     \
    else if (part <= 256 * 32) GGN_BLOCK(T, 32);                                                                     \
    else GGN_BLOCK(T, 64)
        if (out_dtype == IMPARO_BF16) { GGN_PER(bf16_t); } else { GGN_PER(float); }
#undef GGN_PER
#undef GGN_BLOCK
        return launch_status();
    }
    const unsigned blocks = (unsigned)((parts + 3) / 4);
    if (out_dtype == IMPARO_BF16)
        k_gated_group_norm<bf16_t><<<blocks, 256, 0, s>>>(x, gate, gate_ld, gate_off, w, (bf16_t*)out, n_tokens, width,
                                                          groups, eps, gate_first);
    else
        k_gated_group_norm<float><<<blocks, 256, 0, s>>>(x, gate, gate_ld, gate_off, w, (float*)out, n_tokens, width,
                                                         groups, eps, gate_first);
    return launch_status();
}

// ---------------------------------------------------------------- a gated unit with bounds
// gu [tokens, 2 hidden] float32 holds a token's gate values and, `hidden` further on, its up values:
// g = min(gate, limit), u = clamp(up, -limit, limit), out = g sigmoid(alpha g) (u + 1).
template <typename TOut>
__global__ void k_clamped_glu(const float* __restrict__ gu, TOut* __restrict__ out, long long n, int hidden,
                              int out_ld, float limit, float alpha) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long long t = i / out_ld;
    const int j = (int)(i - t * out_ld);
    float y = 0.f;                                        // columns past `hidden` fill a row up with zeros
    if (j < hidden) {
        const float g = fminf(gu[t * 2 * hidden + j], limit);
        const float u = fminf(fmaxf(gu[t * 2 * hidden + hidden + j], -limit), limit);
        y = g * ds_sigmoid(alpha * g) * (u + 1.0f);
    }
    store_f32<TOut>(out, (size_t)i, y);
}

extern "C" int imparo_clamped_glu(const float* gu, void* out, int out_dtype, int n_tokens, int hidden, int out_ld,
                                  float limit, float alpha, imparo_stream stream) {
    if (!gu || !out || n_tokens < 0 || hidden < 1 || out_ld < hidden) return IMPARO_BAD_ARGUMENT;
    if (out_dtype != IMPARO_F32 && out_dtype != IMPARO_BF16) return IMPARO_BAD_ARGUMENT;
    const long long n = (long long)n_tokens * out_ld;
    if (n == 0) return IMPARO_OK;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (out_dtype == IMPARO_BF16)
        k_clamped_glu<bf16_t><<<blocks, 256, 0, (hipStream_t)stream>>>(gu, (bf16_t*)out, n, hidden, out_ld, limit, alpha);
    else
        k_clamped_glu<float><<<blocks, 256, 0, (hipStream_t)stream>>>(gu, (float*)out, n, hidden, out_ld, limit, alpha);
    return launch_status();
}

// ---------------------------------------------------------------- sums of mixers and of experts
// out[t, c] (+)= sum_i f_i * rms_norm(a_i[t])[c] * w_i[c] over up to two inputs (each maybe in slices that
// are added in order first): the results of mixers that run side by side, each normed over the row.
// PER: values of the row a thread keeps in registers (256 threads x PER cover the width): every slice is read
// once, and the loads of a slice are asked for together.
template <int PER>
__global__ __launch_bounds__(256) void k_normed_sum(const float* __restrict__ a, int a_slices, const float* __restrict__ wa,
                                                    const float* __restrict__ b, int b_slices, const float* __restrict__ wb,
                                                    float* __restrict__ out, int n_tokens, int width, float eps,
                                                    float factor) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const size_t stride = (size_t)n_tokens * width, row = (size_t)t * width;
    float ya[PER], yb[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) ya[j] = yb[j] = 0.f;
    for (int s = 0; s < a_slices; ++s)
#pragma unroll
        for (int j = 0; j < PER; ++j) ya[j] += a[s * stride + row + min((int)threadIdx.x + j * 256, width - 1)];
    for (int s = 0; s < b_slices; ++s)
#pragma unroll
        for (int j = 0; j < PER; ++j) yb[j] += b[s * stride + row + min((int)threadIdx.x + j * 256, width - 1)];
    float ssa = 0.f, ssb = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j)
        if ((int)threadIdx.x + j * 256 < width) {
            ssa = fmaf(ya[j], ya[j], ssa);
            ssb = fmaf(yb[j], yb[j], ssb);
        }
    const float ra = 1.0f / sqrtf(block_sum(ssa, scratch) / (float)width + eps);
    const float rb = 1.0f / sqrtf(block_sum(ssb, scratch) / (float)width + eps);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + j * 256;
        if (i < width) out[row + i] = factor * (ya[j] * ra * wa[i] + yb[j] * rb * wb[i]);
    }
}

extern "C" int imparo_normed_sum(const float* a, int a_slices, const float* wa, const float* b, int b_slices,
                                 const float* wb, float* out, int n_tokens, int width, float eps, float factor,
                                 imparo_stream stream) {
    if (!a || !b || !wa || !wb || !out || a_slices < 1 || b_slices < 1 || n_tokens < 0 || width < 1 || width > 16384)
        return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
#define NSUM(PER) k_normed_sum<PER><<<n_tokens, 256, 0, s>>>(a, a_slices, wa, b, b_slices, wb, out, n_tokens, width, eps, factor)
    const int per = (width + 255) / 256;
    if (per <= 1) NSUM(1);
    else if (per <= 2) NSUM(2);
    else if (per <= 4) NSUM(4);
    else if (per <= 8) NSUM(8);
    else if (per <= 16) NSUM(16);
    else if (per <= 32) NSUM(32);
    else NSUM(64);
#undef NSUM
    return launch_status();
}

// out[t, c] += sigmoid(z[t, z_col]) * sum over slices of y[s, t, c]: an expert that every token uses, weighed by
// one gate a token.
__global__ void k_gated_row_add(float* __restrict__ out, const float* __restrict__ y, int y_slices,
                                const float* __restrict__ z, int z_ld, int z_col, int n_tokens, int width) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (long long)n_tokens * width) return;
    const long long t = i / width;
    float s = 0.f;
    for (int k = 0; k < y_slices; ++k) s += y[(size_t)k * n_tokens * width + i];
    out[i] = fmaf(ds_sigmoid(z[t * z_ld + z_col]), s, out[i]);
}

extern "C" int imparo_gated_row_add(float* out, const float* y, int y_slices, const float* z, int z_ld, int z_col,
                                    int n_tokens, int width, imparo_stream stream) {
    if (!out || !y || !z || y_slices < 1 || z_col < 0 || z_ld <= z_col || n_tokens < 0 || width < 1)
        return IMPARO_BAD_ARGUMENT;
    const long long n = (long long)n_tokens * width;
    if (n == 0) return IMPARO_OK;
    k_gated_row_add<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(out, y, y_slices, z, z_ld, z_col,
                                                                                n_tokens, width);
    return launch_status();
}

int imparo_load_code_decay_scan() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_decay_carry)) == hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
