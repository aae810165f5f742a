// A routed feed-forward (mixture of experts) in five launches:
//   route    softmax over the router's outputs, the choice of `top` of them by score + correction,
//            the weights (the scores themselves, as they are), one wave a token;
//   plan     one block: how many (token, choice) entries each expert got, a slot for every entry
//            (the entries of one expert side by side), and the list of row tiles the products walk;
//   product  twice: a tile of one expert's slots times that expert's matrix (up with the activation
//            in its epilogue, then down), on the matrix cores in bfloat16, plain fused multiply-adds
//            in float32; the grid is sized by a bound that the host knows (no count comes back);
//   combine  a token's result: its chosen experts' rows times their weights, added in the order of
//            the choice; an expert past the last real one passes the token's input through.
// Which slot an entry gets depends on the order in which threads arrive; no result does: a row of
// a product is summed over k in one order wherever the row lies in its tile, and a token's sum
// over its experts runs in the order of its own choice.
#include "common.h"
#include "api.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define MOE_MAX_ROUTER 512          // router outputs (experts of both kinds)
#define MOE_MAX_EXPERTS 1024        // real experts the plan kernel keeps counters for
#define MOE_MAX_TOP 16
#define MOE_SCORE_SOFTMAX 0         // scores = softmax over all router outputs
#define MOE_SCORE_SIGMOID 1         // scores = sigmoid of each output

extern "C" int imparo_moe_max_tiles(int n_entries, int n_experts, int tile_rows);

// ---------------------------------------------------------------- route
// What a router may do beyond scoring and choosing. logits_ld: floats between two tokens' logits (at least
// n_router; further columns belong to someone else). groups > 1: the router outputs form that many equal
// groups of neighbours, a group's score is the sum of its two largest choice scores (score + correction), and
// only outputs of the `keep` best groups can be chosen (of equal groups the lowest). normalize: the chosen
// scores are divided by their sum + 1e-20. scale: the weights are multiplied by it at the end.
struct MoeRouteRules {
    int logits_ld, groups, keep, normalize;
    float scale;
};

__device__ __forceinline__ void moe_route_token(const float* __restrict__ logits, const float* __restrict__ correction,
                                                int32_t* __restrict__ choice, float* __restrict__ weight, int t,
                                                int n_router, int top, int scoring, const MoeRouteRules rules) {
    const int lane = threadIdx.x & (WAVE - 1);
    constexpr int PER = MOE_MAX_ROUTER / WAVE;
    float z[PER], pick[PER];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = lane + j * WAVE;
        z[j] = i < n_router ? logits[(size_t)t * rules.logits_ld + i] : -INFINITY;
        m = fmaxf(m, z[j]);
    }
    if (scoring == MOE_SCORE_SIGMOID) {
        // every output scored by itself
#pragma unroll
        for (int j = 0; j < PER; ++j) z[j] = (lane + j * WAVE) < n_router ? 1.0f / (1.0f + expf(-z[j])) : 0.f;
    } else {
        m = wave_max(m);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            z[j] = (lane + j * WAVE) < n_router ? expf(z[j] - m) : 0.f;
            sum += z[j];
        }
        sum = wave_sum(sum);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int j = 0; j < PER; ++j) z[j] *= inv;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = lane + j * WAVE;
        pick[j] = i < n_router ? z[j] + (correction ? correction[i] : 0.f) : -INFINITY;
    }
    if (rules.groups > 1) {
        // lane g scores group g (at most 64 groups): the sum of its two largest choice scores, read from
        // the lanes that hold them; then `keep` rounds of a wave-wide argmax mark the groups that stay
        const int per = n_router / rules.groups;
        float gscore = -INFINITY;
        {
            float b1 = -INFINITY, b2 = -INFINITY;
            for (int e = 0; e < per; ++e) {
                // every lane reads output (lane * per + e) of its own group; lanes beyond the groups read output 0
                const int i = lane < rules.groups ? lane * per + e : 0;
                float v = -INFINITY;
#pragma unroll
                for (int j = 0; j < PER; ++j) {
                    const float got = __shfl(pick[j], i & (WAVE - 1), WAVE);
                    if (i / WAVE == j) v = got;
                }
                if (v > b1) { b2 = b1; b1 = v; } else if (v > b2) { b2 = v; }
            }
            if (lane < rules.groups) gscore = per > 1 ? b1 + b2 : b1;
        }
        unsigned long long kept = 0ull;
        for (int k = 0; k < rules.keep; ++k) {
            float best = gscore;
            int at = lane < rules.groups ? lane : 0x7fffffff;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float ob = __shfl_xor(best, off, WAVE);
                const int oa = __shfl_xor(at, off, WAVE);
                if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
            }
            if (at < rules.groups) kept |= 1ull << at;
            if (lane == at) gscore = -INFINITY;
        }
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = lane + j * WAVE;
            if (i < n_router && !((kept >> (i / per)) & 1ull)) pick[j] = -INFINITY;
        }
    }
    float chosen_sum = 0.f;
    for (int k = 0; k < top; ++k) {
        // the largest choice score that is left; of equal ones the lowest index
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = lane + j * WAVE;
            if (pick[j] > best) { best = pick[j]; at = i; }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, WAVE);
            const int oa = __shfl_xor(at, off, WAVE);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < PER; ++j)
            if (lane + j * WAVE == at) { s = z[j]; pick[j] = -INFINITY; }
        s = wave_sum(s);           // one lane holds it
        chosen_sum += s;
        if (lane == 0) {
            choice[(size_t)t * top + k] = at;
            weight[(size_t)t * top + k] = s;
        }
    }
    if (rules.normalize || rules.scale != 1.0f) {
        const float f = (rules.normalize ? 1.0f / (chosen_sum + 1e-20f) : 1.0f) * rules.scale;
        if (lane == 0)
            for (int k = 0; k < top; ++k) weight[(size_t)t * top + k] *= f;
    }
}

__global__ void k_moe_route(const float* __restrict__ logits, const float* __restrict__ correction,
                            int32_t* __restrict__ choice, float* __restrict__ weight, int n_tokens, int n_router,
                            int top, int scoring, const MoeRouteRules rules) {
    const int t = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (t < n_tokens) moe_route_token(logits, correction, choice, weight, t, n_router, top, scoring, rules);
}

static bool moe_rules_fit(const MoeRouteRules& r, int n_router, int top) {
    if (r.logits_ld < n_router || r.groups < 1 || r.groups > WAVE || n_router % r.groups) return false;
    if (r.groups > 1 && (r.keep < 1 || r.keep > r.groups || r.keep * (n_router / r.groups) < top)) return false;
    return r.scale == r.scale;
}

extern "C" int imparo_moe_route(const float* logits, const float* correction, int32_t* choice, float* weight,
                                int n_tokens, int n_router, int top, int scoring, int logits_ld, int groups, int keep,
                                int normalize, float scale, imparo_stream stream) {
    if (!logits || !choice || !weight || n_tokens < 0) return IMPARO_BAD_ARGUMENT;
    const MoeRouteRules rules{logits_ld, groups, keep, normalize, scale};
    if (!moe_rules_fit(rules, n_router, top)) return IMPARO_BAD_ARGUMENT;
    if (scoring != MOE_SCORE_SOFTMAX && scoring != MOE_SCORE_SIGMOID) return IMPARO_BAD_ARGUMENT;
    if (n_router < 1 || n_router > MOE_MAX_ROUTER || top < 1 || top > n_router || top > MOE_MAX_TOP)
        return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    k_moe_route<<<(n_tokens + 3) / 4, 4 * WAVE, 0, (hipStream_t)stream>>>(logits, correction, choice, weight, n_tokens,
                                                                         n_router, top, scoring, rules);
    return launch_status();
}

// ---------------------------------------------------------------- plan
// tiles[3 i ..]: expert, first slot, rows of tile i; expert -1 where the list has ended.
struct MoePlanShared {
    int count[MOE_MAX_EXPERTS], first[MOE_MAX_EXPERTS], first_tile[MOE_MAX_EXPERTS + 1];
};

__device__ __forceinline__ void moe_plan_block(MoePlanShared& sh, const int32_t* __restrict__ choice, int n_entries,
                                               int n_experts, int tile_rows, int32_t* __restrict__ slot_of_entry,
                                               int32_t* __restrict__ entry_of_slot, int32_t* __restrict__ tiles,
                                               int max_tiles) {
    int* count = sh.count;
    int* first = sh.first;
    int* first_tile = sh.first_tile;
    const int tid = threadIdx.x;
    for (int e = tid; e < n_experts; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int i = tid; i < n_entries; i += blockDim.x) {
        const int e = choice[i];
        if (e >= 0 && e < n_experts) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int slots = 0, n_tiles = 0;
        for (int e = 0; e < n_experts; ++e) {
            first[e] = slots;
            first_tile[e] = n_tiles;
            slots += count[e];
            n_tiles += (count[e] + tile_rows - 1) / tile_rows;
        }
        first_tile[n_experts] = n_tiles;
    }
    __syncthreads();
    for (int e = tid; e < n_experts; e += blockDim.x) {
        const int n = count[e];
        int i = first_tile[e];
        for (int r = 0; r < n && i < max_tiles; r += tile_rows, ++i) {
            tiles[3 * i] = e;
            tiles[3 * i + 1] = first[e] + r;
            tiles[3 * i + 2] = min(tile_rows, n - r);
        }
    }
    for (int i = first_tile[n_experts] + tid; i < max_tiles; i += blockDim.x) {
        tiles[3 * i] = -1;
        tiles[3 * i + 1] = 0;
        tiles[3 * i + 2] = 0;
    }
    __syncthreads();
    for (int e = tid; e < n_experts; e += blockDim.x) count[e] = 0;      // now the cursor of each expert
    __syncthreads();
    for (int i = tid; i < n_entries; i += blockDim.x) {
        const int e = choice[i];
        int slot = -1;
        if (e >= 0 && e < n_experts) {
            slot = first[e] + atomicAdd(&count[e], 1);
            entry_of_slot[slot] = i;
        }
        slot_of_entry[i] = slot;
    }
}

__global__ __launch_bounds__(1024) void k_moe_plan(const int32_t* __restrict__ choice, int n_entries, int n_experts,
                                                   int tile_rows, int32_t* __restrict__ slot_of_entry,
                                                   int32_t* __restrict__ entry_of_slot, int32_t* __restrict__ tiles,
                                                   int max_tiles) {
    __shared__ MoePlanShared sh;
    moe_plan_block(sh, choice, n_entries, n_experts, tile_rows, slot_of_entry, entry_of_slot, tiles, max_tiles);
}

// Route and plan in one launch, for the few tokens of a decode step: the block's waves route the tokens in
// turn, then the block plans what they chose.
#define MOE_ROUTE_PLAN_TOKENS 64
__global__ __launch_bounds__(1024) void k_moe_route_plan(const float* __restrict__ logits,
                                                         const float* __restrict__ correction,
                                                         int32_t* __restrict__ choice, float* __restrict__ weight,
                                                         int n_tokens, int n_router, int top, int scoring,
                                                         const MoeRouteRules rules, int n_experts, int tile_rows,
                                                         int32_t* __restrict__ slot_of_entry,
                                                         int32_t* __restrict__ entry_of_slot,
                                                         int32_t* __restrict__ tiles, int max_tiles) {
    __shared__ MoePlanShared sh;
    for (int t = threadIdx.x / WAVE; t < n_tokens; t += blockDim.x / WAVE)
        moe_route_token(logits, correction, choice, weight, t, n_router, top, scoring, rules);
    __threadfence_block();
    __syncthreads();
    moe_plan_block(sh, choice, n_tokens * top, n_experts, tile_rows, slot_of_entry, entry_of_slot, tiles, max_tiles);
}

extern "C" int imparo_moe_route_plan_tokens() { return MOE_ROUTE_PLAN_TOKENS; }

extern "C" int imparo_moe_route_plan(const float* logits, const float* correction, int32_t* choice, float* weight,
                                     int n_tokens, int n_router, int top, int scoring, int n_experts, int tile_rows,
                                     int32_t* slot_of_entry, int32_t* entry_of_slot, int32_t* tiles, int max_tiles,
                                     int logits_ld, int groups, int keep, int normalize, float scale,
                                     imparo_stream stream) {
    if (!logits || !choice || !weight || !slot_of_entry || !entry_of_slot || !tiles) return IMPARO_BAD_ARGUMENT;
    const MoeRouteRules rules{logits_ld, groups, keep, normalize, scale};
    if (!moe_rules_fit(rules, n_router, top)) return IMPARO_BAD_ARGUMENT;
    if (scoring != MOE_SCORE_SOFTMAX && scoring != MOE_SCORE_SIGMOID) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || n_tokens > MOE_ROUTE_PLAN_TOKENS) return IMPARO_BAD_ARGUMENT;
    if (n_router < 1 || n_router > MOE_MAX_ROUTER || top < 1 || top > n_router || top > MOE_MAX_TOP)
        return IMPARO_BAD_ARGUMENT;
    if (n_experts < 0 || n_experts > MOE_MAX_EXPERTS || tile_rows < 1) return IMPARO_BAD_ARGUMENT;
    if (max_tiles < imparo_moe_max_tiles(n_tokens * top, n_experts, tile_rows)) return IMPARO_SCRATCH_TOO_SMALL;
    if (n_tokens == 0) return IMPARO_OK;
    k_moe_route_plan<<<1, 1024, 0, (hipStream_t)stream>>>(logits, correction, choice, weight, n_tokens, n_router, top,
                                                          scoring, rules, n_experts, tile_rows, slot_of_entry, entry_of_slot,
                                                          tiles, max_tiles);
    return launch_status();
}

extern "C" int imparo_moe_max_tiles(int n_entries, int n_experts, int tile_rows) {
    if (n_entries <= 0 || tile_rows <= 0) return 0;
    return (n_entries + tile_rows - 1) / tile_rows + (n_experts < n_entries ? n_experts : n_entries);
}

// Rows of a product's tile for this many entries over this many experts: the wide tile where an
// expert's share fills it, the narrow one else (many experts), tiles of 16 for the few entries of a decode step.
extern "C" int imparo_moe_tile_rows(int n_entries, int n_experts, int dtype) {
    if (dtype != IMPARO_BF16) return 64;
    if (n_entries <= 128) return 16;          // a decode step: the experts' matrices are streamed once, few rows each
    return (n_experts > 0 && n_entries / n_experts >= 96) ? 128 : 64;
}

extern "C" int imparo_moe_plan(const int32_t* choice, int n_entries, int n_experts, int tile_rows,
                               int32_t* slot_of_entry, int32_t* entry_of_slot, int32_t* tiles, int max_tiles,
                               imparo_stream stream) {
    if (!choice || !slot_of_entry || !entry_of_slot || !tiles || n_entries < 0) return IMPARO_BAD_ARGUMENT;
    if (n_experts < 0 || n_experts > MOE_MAX_EXPERTS || tile_rows < 1) return IMPARO_BAD_ARGUMENT;
    if (max_tiles < imparo_moe_max_tiles(n_entries, n_experts, tile_rows)) return IMPARO_SCRATCH_TOO_SMALL;
    if (n_entries == 0) return IMPARO_OK;
    k_moe_plan<<<1, 1024, 0, (hipStream_t)stream>>>(choice, n_entries, n_experts, tile_rows, slot_of_entry,
                                                    entry_of_slot, tiles, max_tiles);
    return launch_status();
}

// ---------------------------------------------------------------- products
#define MOE_EPI_NONE 0
#define MOE_EPI_RELU2 1        // max(z, 0)^2

__device__ __forceinline__ float moe_epilogue(float v, int epi) {
    if (epi == MOE_EPI_RELU2) {
        v = fmaxf(v, 0.f);
        v *= v;
    }
    return v;
}

// out[slot, n] = epi(sum_k a[row(slot), k] * w[expert, n, k]) for the slots of one tile. row(slot) is the
// slot itself, or with gather_div the token of the slot's entry (entry / gather_div). Four waves as 2 x 2,
// each WM x WN products of 32 x 32; K in steps of 64 through two LDS stages, the next step's loads in
// registers while this one is multiplied. K is a multiple of 8.
template <int WM, int WN, typename TOut>
__global__ __launch_bounds__(256) void k_moe_gemm_bf16(const bf16_t* __restrict__ A, int a_ld, int gather_div,
                                                       const int32_t* __restrict__ entry_of_slot,
                                                       const bf16_t* __restrict__ W, TOut* __restrict__ out,
                                                       const int32_t* __restrict__ tiles, int N, int K, int epi) {
    constexpr int TM = 64 * WM, TN = 64 * WN, LD = 72, BK = 64;
    __shared__ __attribute__((aligned(16))) bf16_t As[2][TM * LD];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[2][TN * LD];
    const int expert = tiles[3 * blockIdx.x];
    if (expert < 0) return;
    const int row0 = tiles[3 * blockIdx.x + 1], rows = tiles[3 * blockIdx.x + 2];
    const int n0 = blockIdx.y * TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const bf16_t* Wb = W + (size_t)expert * N * K;
    const int kc = (tid & 7) * 8;
    const bf16_t* pa[TM / 32];
    const bf16_t* pb[TN / 32];
#pragma unroll
    for (int j = 0; j < TM / 32; ++j) {
        const int slot = row0 + min((tid >> 3) + 32 * j, rows - 1);
        const int src = gather_div ? entry_of_slot[slot] / gather_div : slot;
        pa[j] = A + (size_t)src * a_ld;
    }
#pragma unroll
    for (int j = 0; j < TN / 32; ++j) pb[j] = Wb + (size_t)min(n0 + (tid >> 3) + 32 * j, N - 1) * K;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    // two sets of registers, each holding one K-step's loads: a step's loads are asked for two steps ahead
    u32x4 ra0[TM / 32], rb0[TN / 32], ra1[TM / 32], rb1[TN / 32];
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const int nk = (K + BK - 1) / BK;
    // the loads of K-step kt into registers; what lies beyond K comes as zeros (K is a multiple of 8, so a
    // piece of 8 is inside or outside as a whole) from an address inside the row; a step past the last
    // reads the last again and is never stored
#define MOE_FETCH(kt, ra, rb)                                                                                       \
    {                                                                                                               \
        const int k_ = min((kt), nk - 1) * BK + kc;                                                                 \
        const bool in_ = k_ < K;                                                                                    \
        const int kk_ = in_ ? k_ : 0;                                                                               \
        _Pragma("unroll") for (int j = 0; j < TM / 32; ++j) {                                                       \
            const u32x4 v_ = *reinterpret_cast<const u32x4*>(pa[j] + kk_);                                          \
            ra[j] = in_ ? v_ : zero;                                                                                \
        }                                                                                                           \
        _Pragma("unroll") for (int j = 0; j < TN / 32; ++j) {                                                       \
            const u32x4 v_ = *reinterpret_cast<const u32x4*>(pb[j] + kk_);                                          \
            rb[j] = in_ ? v_ : zero;                                                                                \
        }                                                                                                           \
    }
#define MOE_STASH(buf_, ra, rb)                                                                                     \
    {                                                                                                               \
        _Pragma("unroll") for (int j = 0; j < TM / 32; ++j)                                                         \
            *reinterpret_cast<u32x4*>(&As[buf_][((tid >> 3) + 32 * j) * LD + kc]) = ra[j];                          \
        _Pragma("unroll") for (int j = 0; j < TN / 32; ++j)                                                         \
            *reinterpret_cast<u32x4*>(&Bs[buf_][((tid >> 3) + 32 * j) * LD + kc]) = rb[j];                          \
    }
#define MOE_MULTIPLY(buf_)                                                                                          \
    _Pragma("unroll") for (int ks = 0; ks < BK / 16; ++ks) {                                                        \
        bf16x8 fa[WM], fb[WN];                                                                                      \
        _Pragma("unroll") for (int i = 0; i < WM; ++i)                                                              \
            fa[i] = *reinterpret_cast<const bf16x8*>(&As[buf_][a_base + i * 32 * LD + ks * 16]);                    \
        _Pragma("unroll") for (int j = 0; j < WN; ++j)                                                              \
            fb[j] = *reinterpret_cast<const bf16x8*>(&Bs[buf_][b_base + j * 32 * LD + ks * 16]);                    \
        _Pragma("unroll") for (int i = 0; i < WM; ++i)                                                              \
            _Pragma("unroll") for (int j = 0; j < WN; ++j)                                                          \
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);              \
    }
    f32x16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    const int a_base = (wm * 32 * WM + (lane & 31)) * LD + (lane >> 5) * 8;
    const int b_base = (wn * 32 * WN + (lane & 31)) * LD + (lane >> 5) * 8;
    MOE_FETCH(0, ra0, rb0);
    MOE_FETCH(1, ra1, rb1);
    MOE_STASH(0, ra0, rb0);
    MOE_FETCH(2, ra0, rb0);
    __syncthreads();
    // step kt is multiplied out of stage kt % 2 while step kt + 1 goes from its registers into the other
    // stage and those registers take the loads of step kt + 3
    for (int kt = 0; kt < nk; kt += 2) {
        MOE_MULTIPLY(0);
        if (kt + 1 < nk) MOE_STASH(1, ra1, rb1);
        MOE_FETCH(kt + 3, ra1, rb1);
        __syncthreads();
        if (kt + 1 < nk) {
            MOE_MULTIPLY(1);
            if (kt + 2 < nk) MOE_STASH(0, ra0, rb0);
            MOE_FETCH(kt + 4, ra0, rb0);
            __syncthreads();
        }
    }
#undef MOE_FETCH
#undef MOE_STASH
#undef MOE_MULTIPLY
    // a lane holds column lane % 32 of a 32 x 32 product, rows 8 (r / 4) + 4 (lane / 32) + r % 4
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) {
            const int n = n0 + wn * 32 * WN + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = wm * 32 * WM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m < rows && n < N) store_f32<TOut>(out, (size_t)(row0 + m) * N + n, moe_epilogue(acc[i][j][r], epi));
            }
        }
}

// Few rows an expert (a decode step): a block takes 16 outputs of one expert and up to 16 slots. The expert's
// 16 weight rows are the M side of 16x16x32 products and go from memory straight into the operand registers,
// K cut over the block's four waves and, inside a wave, walked in runs of 64 with four runs' loads in flight
// (a lane takes 16 consecutive k of its row, so that four lanes read a row's 128 bytes side by side; the
// slots' rows are read with the same k order, which is all a dot product asks for). The waves' partial sums
// meet in LDS and are added in wave order.
template <typename TOut>
__global__ __launch_bounds__(256) void k_moe_gemm_rows16(const bf16_t* __restrict__ A, int a_ld, int gather_div,
                                                         const int32_t* __restrict__ entry_of_slot,
                                                         const bf16_t* __restrict__ W, TOut* __restrict__ out,
                                                         const int32_t* __restrict__ tiles, int N, int K, int epi) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    __shared__ f32x4 part[4][WAVE];
    const int expert = tiles[3 * blockIdx.x];
    if (expert < 0) return;
    const int row0 = tiles[3 * blockIdx.x + 1], rows = tiles[3 * blockIdx.x + 2];
    const int n0 = blockIdx.y * 16;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const bf16_t* wrow = W + ((size_t)expert * N + min(n0 + c, N - 1)) * K;
    const int slot = row0 + min(c, rows - 1);
    const bf16_t* arow = A + (size_t)(gather_div ? entry_of_slot[slot] / gather_div : slot) * a_ld;
    // this wave's part of K, in whole runs of 64
    const int runs = (K + 63) / 64;
    const int per_wave = (runs + 3) / 4;
    const int run_lo = wave * per_wave, run_hi = min(runs, run_lo + per_wave);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    const u32x4 zero = {0u, 0u, 0u, 0u};
    for (int r0 = run_lo; r0 < run_hi; r0 += 4) {
        u32x4 w[4][2], a[4][2];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int k = min(r0 + u, run_hi - 1) * 64 + g * 16 + h * 8;
                const bool in = k < K && r0 + u < run_hi;
                const int kk = k < K ? k : 0;
                const u32x4 wv = *reinterpret_cast<const u32x4*>(wrow + kk);
                const u32x4 av = *reinterpret_cast<const u32x4*>(arow + kk);
                w[u][h] = in ? wv : zero;
                a[u][h] = in ? av : zero;
            }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w[u][h]),
                                                              __builtin_bit_cast(bf16x8, a[u][h]), acc, 0, 0, 0);
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave != 0) return;
    f32x4 total = part[0][lane];
#pragma unroll
    for (int w2 = 1; w2 < 4; ++w2) {
        const f32x4 p = part[w2][lane];
#pragma unroll
        for (int i = 0; i < 4; ++i) total[i] += p[i];
    }
    // a lane holds slot c, outputs n0 + 4 g + i
    if (c < rows) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + 4 * g + i;
            if (n < N) store_f32<TOut>(out, (size_t)(row0 + c) * N + n, moe_epilogue(total[i], epi));
        }
    }
}

// The same in float32: a tile of 64 slots by 64 outputs, K in steps of 16 through LDS, every output
// summed over k = 0, 1, 2, ... by fused multiply-adds, whatever the tile holds beside it.
__global__ __launch_bounds__(256) void k_moe_gemm_f32(const float* __restrict__ A, int a_ld, int gather_div,
                                                      const int32_t* __restrict__ entry_of_slot,
                                                      const float* __restrict__ W, float* __restrict__ out,
                                                      const int32_t* __restrict__ tiles, int N, int K, int epi) {
    constexpr int TM = 64, TN = 64, BK = 16, LD = 68;
    __shared__ float As[BK][LD], Bs[BK][LD];
    const int expert = tiles[3 * blockIdx.x];
    if (expert < 0) return;
    const int row0 = tiles[3 * blockIdx.x + 1], rows = tiles[3 * blockIdx.x + 2];
    const int n0 = blockIdx.y * TN;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    const float* Wb = W + (size_t)expert * N * K;
    const float* pa[4];
    const float* pb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = (tid >> 4) + 16 * j;
        const int slot = row0 + min(r, rows - 1);
        const int src = gather_div ? entry_of_slot[slot] / gather_div : slot;
        pa[j] = A + (size_t)src * a_ld;
        pb[j] = Wb + (size_t)min(n0 + r, N - 1) * K;
    }
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += BK) {
        const int k = k0 + tx;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            As[tx][(tid >> 4) + 16 * j] = k < K ? pa[j][k] : 0.f;
            Bs[tx][(tid >> 4) + 16 * j] = k < K ? pb[j][k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = ty * 4 + i, n = n0 + tx * 4 + j;
            if (m < rows && n < N) out[(size_t)(row0 + m) * N + n] = moe_epilogue(acc[i][j], epi);
        }
}

extern "C" int imparo_moe_gemm(const void* a, int a_ld, int gather_div, const int32_t* entry_of_slot, const void* w,
                               void* out, int out_dtype, int dtype, const int32_t* tiles, int max_tiles, int tile_rows,
                               int n, int k, int epilogue, imparo_stream stream) {
    if (!a || !w || !out || !tiles || max_tiles < 0 || n < 1 || k < 1 || a_ld < k || gather_div < 0)
        return IMPARO_BAD_ARGUMENT;
    if (gather_div && !entry_of_slot) return IMPARO_BAD_ARGUMENT;
    if (epilogue != MOE_EPI_NONE && epilogue != MOE_EPI_RELU2) return IMPARO_BAD_ARGUMENT;
    if (max_tiles == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == IMPARO_F32) {
        if (out_dtype != IMPARO_F32 || tile_rows != 64) return IMPARO_BAD_ARGUMENT;
        k_moe_gemm_f32<<<dim3(max_tiles, (n + 63) / 64), 256, 0, s>>>((const float*)a, a_ld, gather_div, entry_of_slot,
                                                                     (const float*)w, (float*)out, tiles, n, k, epilogue);
        return launch_status();
    }
    if (dtype != IMPARO_BF16 || k % 8 || a_ld % 8 || ((uintptr_t)a | (uintptr_t)w) % 16) return IMPARO_BAD_ARGUMENT;
#define MOE_LAUNCH(WM, WN, TO)                                                                                       \
    k_moe_gemm_bf16<WM, WN, TO><<<dim3(max_tiles, (n + 64 * WN - 1) / (64 * WN)), 256, 0, s>>>(                      \
        (const bf16_t*)a, a_ld, gather_div, entry_of_slot, (const bf16_t*)w, (TO*)out, tiles, n, k, epilogue)
    if (tile_rows == 16) {
        const dim3 grid16(max_tiles, (n + 15) / 16);
        if (out_dtype == IMPARO_BF16)
            k_moe_gemm_rows16<bf16_t><<<grid16, 256, 0, s>>>((const bf16_t*)a, a_ld, gather_div, entry_of_slot,
                                                             (const bf16_t*)w, (bf16_t*)out, tiles, n, k, epilogue);
        else if (out_dtype == IMPARO_F32)
            k_moe_gemm_rows16<float><<<grid16, 256, 0, s>>>((const bf16_t*)a, a_ld, gather_div, entry_of_slot,
                                                            (const bf16_t*)w, (float*)out, tiles, n, k, epilogue);
        else
            return IMPARO_BAD_ARGUMENT;
    } else if (tile_rows == 128) {
        if (out_dtype == IMPARO_BF16) MOE_LAUNCH(2, 2, bf16_t);
        else if (out_dtype == IMPARO_F32) MOE_LAUNCH(2, 2, float);
        else return IMPARO_BAD_ARGUMENT;
    } else if (tile_rows == 64) {
        if (n >= 128) {
            if (out_dtype == IMPARO_BF16) MOE_LAUNCH(1, 2, bf16_t);
            else if (out_dtype == IMPARO_F32) MOE_LAUNCH(1, 2, float);
            else return IMPARO_BAD_ARGUMENT;
        } else {
            if (out_dtype == IMPARO_BF16) MOE_LAUNCH(1, 1, bf16_t);
            else if (out_dtype == IMPARO_F32) MOE_LAUNCH(1, 1, float);
            else return IMPARO_BAD_ARGUMENT;
        }
    } else {
        return IMPARO_BAD_ARGUMENT;
    }
#undef MOE_LAUNCH
    return launch_status();
}

// ---------------------------------------------------------------- gated experts
// hidden[slot, j] = silu(w g) * (w u) with g = gu[slot, j], u = gu[slot, half + j] (an expert's gate and up
// rows stacked in one product) and w the weight of the slot's entry (null: 1): an expert without biases that
// reads w * h has w times the products of h. Columns j >= ff (a hidden width filled up for the product
// that follows) hold zeros in gu already and give zeros.
template <typename TOut>
__global__ void k_moe_gated(const float* __restrict__ gu, const float* __restrict__ weight,
                            const int32_t* __restrict__ entry_of_slot, int n_entries, TOut* __restrict__ hidden,
                            int half, long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long slot = i / half;
    const int j = (int)(i - slot * half);
    float w = 1.0f;
    if (weight) {
        const int e = entry_of_slot[slot];          // a row behind the last slot names no entry
        w = (e >= 0 && e < n_entries) ? weight[e] : 0.f;
    }
    const float g = w * gu[slot * 2 * half + j], u = w * gu[slot * 2 * half + half + j];
    store_f32<TOut>(hidden, (size_t)i, g / (1.0f + expf(-g)) * u);
}

// n_slots: the entries that got a slot are the first ones of gu and hidden; where some entries have none
// (experts past the last real one) the rows behind the last slot are computed from whatever gu holds and
// never read.
extern "C" int imparo_moe_gated(const float* gu, const float* weight, const int32_t* entry_of_slot, void* hidden,
                                int out_dtype, int n_slots, int half, imparo_stream stream) {
    if (!gu || !hidden || n_slots < 0 || half < 1 || (weight && !entry_of_slot)) return IMPARO_BAD_ARGUMENT;
    if (n_slots == 0) return IMPARO_OK;
    const long long total = (long long)n_slots * half;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == IMPARO_F32)
        k_moe_gated<float><<<blocks, 256, 0, s>>>(gu, weight, entry_of_slot, n_slots, (float*)hidden, half, total);
    else if (out_dtype == IMPARO_BF16)
        k_moe_gated<bf16_t><<<blocks, 256, 0, s>>>(gu, weight, entry_of_slot, n_slots, (bf16_t*)hidden, half, total);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// ---------------------------------------------------------------- combine
// out[t] = sum over the token's choices, in their order, of weight * (the expert's row, or for an
// expert past the last real one the token's input).
template <typename T>
__global__ void k_moe_combine(const float* __restrict__ y, const T* __restrict__ h, const int32_t* __restrict__ choice,
                              const float* __restrict__ weight, const int32_t* __restrict__ slot_of_entry,
                              float* __restrict__ out, int width, int top, int n_experts) {
    const int t = blockIdx.x;
    __shared__ int slot[MOE_MAX_TOP];
    __shared__ float w[MOE_MAX_TOP];
    if (threadIdx.x < top) {
        const int e = choice[(size_t)t * top + threadIdx.x];
        slot[threadIdx.x] = e < n_experts ? slot_of_entry[(size_t)t * top + threadIdx.x] : -1;
        w[threadIdx.x] = weight ? weight[(size_t)t * top + threadIdx.x] : 1.0f;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const float v = slot[k] >= 0 ? y[(size_t)slot[k] * width + i] : load_f32<T>(h, (size_t)t * width + i);
            acc = fmaf(w[k], v, acc);
        }
        out[(size_t)t * width + i] = acc;
    }
}

extern "C" int imparo_moe_combine(const float* y, const void* h, int h_dtype, const int32_t* choice,
                                  const float* weight, const int32_t* slot_of_entry, float* out, int n_tokens,
                                  int width, int top, int n_experts, imparo_stream stream) {
    if (!y || !h || !choice || !slot_of_entry || !out || n_tokens < 0 || width < 1) return IMPARO_BAD_ARGUMENT;
    if (top < 1 || top > MOE_MAX_TOP || n_experts < 0) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const int threads = width >= 1024 ? 256 : 64;
    if (h_dtype == IMPARO_F32)
        k_moe_combine<float><<<n_tokens, threads, 0, s>>>(y, (const float*)h, choice, weight, slot_of_entry, out, width,
                                                          top, n_experts);
    else if (h_dtype == IMPARO_BF16)
        k_moe_combine<bf16_t><<<n_tokens, threads, 0, s>>>(y, (const bf16_t*)h, choice, weight, slot_of_entry, out,
                                                           width, top, n_experts);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// ---------------------------------------------------------------- a norm on what a sublayer returns
// x[row] += d / sqrt(mean(d^2) + eps_post) * w_post, d = the sum of the delta's slices in order; then,
// with w_next, out[row] = x[row] / sqrt(mean(x[row]^2) + eps_next) * w_next. One block a row, the row in
// registers between the passes, every sum in float32 and in an order that the width alone decides. With `rows`
// only those rows are taken and the stream is left as it is (the rows whose logits are wanted).
// PER: values of the row a thread keeps in registers (the block's threads x PER cover the width); every
// load of the row (the delta's slices, the stream, both weights) is asked for before any is used.
// What a routed feed-forward leaves for this launch to combine instead of a finished delta: the experts'
// rows y [slots, width], the feed-forward's input h (for experts that pass it through), and per token its
// choice, weights and slots. delta[t] = sum_j weight[t, j] * (y[slot] or h[t]), j in the order of the choice.
struct MoeRows {
    const float* y;
    const void* h;
    const int32_t* choice;
    const float* weight;
    const int32_t* slot_of_entry;
    int h_is_bf16, top, n_experts;
};

template <typename TOut, int PER>
__global__ __launch_bounds__(256) void k_post_norm_add(float* __restrict__ x, const float* __restrict__ delta,
                                                       int n_delta, size_t delta_stride, MoeRows moe,
                                                       const int32_t* __restrict__ rows,
                                                       const float* __restrict__ w_post, float eps_post,
                                                       const float* __restrict__ w_next, float eps_next,
                                                       TOut* __restrict__ out, int width, int write_back) {
    __shared__ float scratch[16];
    const int i_out = blockIdx.x;
    const size_t src = (size_t)(rows ? rows[i_out] : i_out) * width;
    float d[PER], xv[PER], wp[PER], wn[PER];
    if (moe.y) {
        __shared__ int slot[MOE_MAX_TOP];
        __shared__ float wt[MOE_MAX_TOP];
        const size_t t = src / width;
        if ((int)threadIdx.x < moe.top) {
            const int e = moe.choice[t * moe.top + threadIdx.x];
            slot[threadIdx.x] = e < moe.n_experts ? moe.slot_of_entry[t * moe.top + threadIdx.x] : -1;
            wt[threadIdx.x] = moe.weight[t * moe.top + threadIdx.x];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < PER; ++j) d[j] = 0.f;
        for (int k = 0; k < moe.top; ++k) {
            const int sl = slot[k];
            const float w = wt[k];
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                const int ii = min((int)threadIdx.x + j * 256, width - 1);
                const float v = sl >= 0 ? moe.y[(size_t)sl * width + ii]
                                        : (moe.h_is_bf16 ? load_f32<bf16_t>((const bf16_t*)moe.h, src + ii)
                                                         : load_f32<float>((const float*)moe.h, src + ii));
                d[j] = fmaf(w, v, d[j]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + j * 256;
        const int ii = min(i, width - 1);
        if (!moe.y) d[j] = delta[src + ii];
        xv[j] = x[src + ii];
        wp[j] = w_post[ii];
        wn[j] = w_next ? w_next[ii] : 0.f;
    }
    for (int s = 1; s < n_delta && !moe.y; ++s)
#pragma unroll
        for (int j = 0; j < PER; ++j) d[j] += delta[(size_t)s * delta_stride + src + min((int)threadIdx.x + j * 256, width - 1)];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j)
        if (threadIdx.x + j * 256 < width) ss = fmaf(d[j], d[j], ss);
    const float r1 = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps_post);
    ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + j * 256;
        xv[j] = xv[j] + d[j] * r1 * wp[j];
        if (i < width) {
            if (write_back) x[src + i] = xv[j];
            ss = fmaf(xv[j], xv[j], ss);
        }
    }
    if (!w_next) {
        // no norm follows: with an output, the new rows themselves go there in its dtype
        if (out)
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                const int i = threadIdx.x + j * 256;
                if (i < width) store_f32<TOut>(out, (size_t)i_out * width + i, xv[j]);
            }
        return;
    }
    const float r2 = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps_next);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = threadIdx.x + j * 256;
        if (i < width) store_f32<TOut>(out, (size_t)i_out * width + i, xv[j] * r2 * wn[j]);
    }
}

static int post_norm_add_launch(float* x, const float* delta, int n_delta, MoeRows moe, int n_rows_x,
                                const int32_t* rows, const float* w_post, float eps_post, const float* w_next,
                                float eps_next, void* out, int out_dtype, int n_out, int width, imparo_stream stream) {
    if (!x || (!delta && !moe.y) || !w_post || n_delta < 1 || n_rows_x < 0 || n_out < 0 || width < 1 || width > 16384)
        return IMPARO_BAD_ARGUMENT;
    if (w_next && !out) return IMPARO_BAD_ARGUMENT;
    if (!rows && n_out != n_rows_x) return IMPARO_BAD_ARGUMENT;
    if (n_out == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const size_t stride = (size_t)n_rows_x * width;
    const int write_back = rows ? 0 : 1;
    const bool to_bf16 = out && out_dtype == IMPARO_BF16;
    if (out && out_dtype != IMPARO_BF16 && out_dtype != IMPARO_F32) return IMPARO_BAD_ARGUMENT;
#define POST_NORM(PER)                                                                                              \
    if (to_bf16)                                                                                                    \
        k_post_norm_add<bf16_t, PER><<<n_out, 256, 0, s>>>(x, delta, n_delta, stride, moe, rows, w_post, eps_post,  \
                                                           w_next, eps_next, (bf16_t*)out, width, write_back);      \
    else                                                                                                            \
        k_post_norm_add<float, PER><<<n_out, 256, 0, s>>>(x, delta, n_delta, stride, moe, rows, w_post, eps_post,   \
                                                          w_next, eps_next, (float*)out, width, write_back)
    const int per = (width + 255) / 256;
    if (per <= 1) { POST_NORM(1); }
    else if (per <= 2) { POST_NORM(2); }
    else if (per <= 4) { POST_NORM(4); }
    else if (per <= 8) { POST_NORM(8); }
    else if (per <= 16) { POST_NORM(16); }
    else if (per <= 32) { POST_NORM(32); }
    else { POST_NORM(64); }
#undef POST_NORM
    return launch_status();
}

extern "C" int imparo_post_norm_add(float* x, const float* delta, int n_delta, int n_rows_x, const int32_t* rows,
                                    const float* w_post, float eps_post, const float* w_next, float eps_next,
                                    void* out, int out_dtype, int n_out, int width, imparo_stream stream) {
    return post_norm_add_launch(x, delta, n_delta, MoeRows{}, n_rows_x, rows, w_post, eps_post, w_next, eps_next, out,
                                out_dtype, n_out, width, stream);
}

// The same with the delta made in the launch from a routed feed-forward's rows (imparo_moe_combine's sum).
extern "C" int imparo_post_norm_add_moe(float* x, const float* y, const void* h, int h_dtype, const int32_t* choice,
                                        const float* weight, const int32_t* slot_of_entry, int top, int n_experts,
                                        int n_rows_x, const int32_t* rows, const float* w_post, float eps_post,
                                        const float* w_next, float eps_next, void* out, int out_dtype, int n_out,
                                        int width, imparo_stream stream) {
    if (!y || !h || !choice || !weight || !slot_of_entry || top < 1 || top > MOE_MAX_TOP || n_experts < 0)
        return IMPARO_BAD_ARGUMENT;
    if (h_dtype != IMPARO_F32 && h_dtype != IMPARO_BF16) return IMPARO_BAD_ARGUMENT;
    const MoeRows moe{y, h, choice, weight, slot_of_entry, h_dtype == IMPARO_BF16, top, n_experts};
    return post_norm_add_launch(x, nullptr, 1, moe, n_rows_x, rows, w_post, eps_post, w_next, eps_next, out, out_dtype,
                                n_out, width, stream);
}

int imparo_load_code_moe() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_moe_plan)) == hipSuccess ? IMPARO_OK
                                                                                                       : IMPARO_LAUNCH_FAILED;
}
