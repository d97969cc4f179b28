// Kernels of a feed-forward made of many small experts of which each token uses a few (gfx950,
// wave64): the choice of experts from the router's logits, the plan that sorts (token, choice)
// pairs by expert, the products of all experts in one launch, and the weighted sum of the chosen
// experts' outputs.  Scores, weights and sums are 32-bit.  Everything is device work with launch
// sizes that depend on the step's shape only, so a step can be recorded and replayed.
//
// A pair is p = token * top + choice.  The plan gives every pair a place in an order in which the
// pairs of one expert are neighbours; the experts' products work on rows in that order (a tile of
// MOE_TM rows never spans two experts) and the weighted sum reads them back through `place`.
#include "common.h"

ROCML_LAST_ERROR_FN(moe)

constexpr int MOE_TM = 128;           // rows of a tile of the experts' products
constexpr int RT_MAX_PER_LANE = 8;    // experts per lane of the routing wave: at most 512 experts
constexpr int RT_BLOCK = 256;

// ---- routing -----------------------------------------------------------------------
// One wave per token.  s = softmax(logits) over all experts.  With groups (count > 0): the
// experts form `count` equal groups of neighbours, a group's score is its largest s, and only
// experts of the `keep` best groups can be chosen.  The `top` largest s among those are chosen
// (the lower index wins a tie), and their weights are s / (sum of the chosen s + sum_eps).
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(v, off, 64);
        int oi = __shfl_xor(i, off, 64);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
}

// sigmoid != 0: s = sigmoid(logit) by itself instead of the softmax.  correction (may be null): one number per
// expert that is added to s for the choice (of groups and of experts) only; the weights use s without it, so a
// choice score may be negative and "cannot be chosen" is minus infinity.  group_top2: a group's score is the sum
// of its two largest choice scores (of its one score in groups of one expert).
__global__ void __launch_bounds__(RT_BLOCK)
moe_route_kernel(const float* __restrict__ logits, int n_tokens, int n_experts, int top, int group_count, int group_keep,
                 float sum_eps, int* __restrict__ chosen, float* __restrict__ weight, const float* __restrict__ bias,
                 int sigmoid, const float* __restrict__ correction, int group_top2, int ld) {
    // ld: numbers between the starts of two tokens' logits (the logits may be the leading columns of a wider matrix)
    // bias (may be null): one number per expert, added to the logits first
    extern __shared__ float rt_smem[];          // [waves][n_experts]
    int wave = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
    int t = blockIdx.x * (RT_BLOCK / WAVE) + wave;
    bool live = t < n_tokens;
    float* mine = rt_smem + (size_t)wave * n_experts;
    const float* z = logits + (size_t)(live ? t : 0) * ld;
    float s[RT_MAX_PER_LANE];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < RT_MAX_PER_LANE; ++j) {
        int e = lane + j * WAVE;
        s[j] = e < n_experts ? z[e] + (bias ? bias[e] : 0.f) : -INFINITY;
        m = fmaxf(m, s[j]);
    }
    if (sigmoid) {
#pragma unroll
        for (int j = 0; j < RT_MAX_PER_LANE; ++j) s[j] = lane + j * WAVE < n_experts ? 1.0f / (1.0f + expf(-s[j])) : 0.f;
    } else {
        m = wave_max(m);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < RT_MAX_PER_LANE; ++j) {
            int e = lane + j * WAVE;
            s[j] = e < n_experts ? expf(s[j] - m) : 0.f;
            sum += s[j];
        }
        sum = wave_sum(sum);
#pragma unroll
        for (int j = 0; j < RT_MAX_PER_LANE; ++j) s[j] = s[j] / sum;
    }
    // candidates: the choice scores; minus infinity marks an expert that cannot be chosen (any more)
    float cand[RT_MAX_PER_LANE];
#pragma unroll
    for (int j = 0; j < RT_MAX_PER_LANE; ++j) {
        int e = lane + j * WAVE;
        cand[j] = e < n_experts ? s[j] + (correction ? correction[e] : 0.f) : -INFINITY;
        if (e < n_experts) mine[e] = cand[j];
    }
    if (group_count > 0) {
        __syncthreads();
        int per = n_experts / group_count;
        // group scores, one or more groups per lane
        float gs[RT_MAX_PER_LANE];
        bool kept[RT_MAX_PER_LANE];
#pragma unroll
        for (int j = 0; j < RT_MAX_PER_LANE; ++j) {
            int g = lane + j * WAVE;
            gs[j] = -INFINITY;
            kept[j] = false;
            if (g < group_count) {
                float best = mine[g * per], second = -INFINITY;
                for (int i = 1; i < per; ++i) {
                    float c = mine[g * per + i];
                    if (c > best) { second = best; best = c; }
                    else if (c > second) second = c;
                }
                gs[j] = group_top2 && per > 1 ? best + second : best;
            }
        }
        // the kept groups, best first
        for (int k = 0; k < group_keep; ++k) {
            float bv = -INFINITY;
            int bi = 0x7fffffff;
#pragma unroll
            for (int j = 0; j < RT_MAX_PER_LANE; ++j)
                if (lane + j * WAVE < group_count && !kept[j] && (gs[j] > bv || bi == 0x7fffffff)) { bv = gs[j]; bi = lane + j * WAVE; }
            wave_argmax(bv, bi);
#pragma unroll
            for (int j = 0; j < RT_MAX_PER_LANE; ++j)
                if (lane + j * WAVE == bi) kept[j] = true;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < RT_MAX_PER_LANE; ++j) {
            int g = lane + j * WAVE;
            if (g < group_count) mine[g] = kept[j] ? 1.f : 0.f;      // (scores are in registers by now)
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < RT_MAX_PER_LANE; ++j) {
            int e = lane + j * WAVE;
            if (e < n_experts && mine[e / per] == 0.f) cand[j] = -INFINITY;
        }
    }
    float total = 0.f;
    float mine_w = 0.f;
    int mine_e = 0;
    for (int k = 0; k < top; ++k) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < RT_MAX_PER_LANE; ++j)
            if (cand[j] > bv) { bv = cand[j]; bi = lane + j * WAVE; }
        wave_argmax(bv, bi);
        float sv = 0.f;
#pragma unroll
        for (int j = 0; j < RT_MAX_PER_LANE; ++j)
            if (lane + j * WAVE == bi) { cand[j] = -INFINITY; sv = s[j]; }
        sv = wave_sum(sv);            // the chosen expert's score, from the lane that holds it
        total += sv;
        if (lane == k) { mine_w = sv; mine_e = bi; }
    }
    if (live && lane < top) {
        chosen[(size_t)t * top + lane] = mine_e;
        weight[(size_t)t * top + lane] = mine_w / (total + sum_eps);
    }
}

ROCML_EXPORT int rocml_moe_route(const float* logits, int n_tokens, int n_experts, int top, int group_count, int group_keep,
                                 float sum_eps, int* chosen, float* weight, const float* bias, int sigmoid,
                                 const float* correction, int group_top2, int ld, hipStream_t stream) {
    ROCML_REQUIRE(ld >= n_experts, "moe_route: rows of %d numbers for %d experts", ld, n_experts);
    ROCML_REQUIRE(n_tokens >= 0 && n_experts > 0 && n_experts <= RT_MAX_PER_LANE * WAVE, "moe_route: %d experts (1 to %d)", n_experts,
                  RT_MAX_PER_LANE * WAVE);
    ROCML_REQUIRE(top >= 1 && top <= WAVE && top <= n_experts, "moe_route: %d chosen of %d experts", top, n_experts);
    ROCML_REQUIRE(group_count >= 0 && (group_count == 0 || (n_experts % group_count == 0 && group_keep >= 1 && group_keep <= group_count &&
                                                              top <= group_keep * (n_experts / group_count))),
                  "moe_route: %d groups of which %d are kept do not fit %d experts and %d chosen", group_count, group_keep, n_experts, top);
    ROCML_REQUIRE(logits && chosen && weight, "moe_route: missing arguments");
    if (n_tokens == 0) return 0;
    size_t lds = (size_t)(RT_BLOCK / WAVE) * n_experts * sizeof(float);
    moe_route_kernel<<<ceil_div(n_tokens, RT_BLOCK / WAVE), RT_BLOCK, lds, stream>>>(logits, n_tokens, n_experts, top, group_count,
                                                                                     group_keep, sum_eps, chosen, weight, bias,
                                                                                     sigmoid, correction, group_top2, ld);
    ROCML_CHECK_LAUNCH("moe_route");
    return 0;
}

// ---- the plan ------------------------------------------------------------------------
// One block.  offsets[e] .. offsets[e + 1] are the places of expert e's pairs; order[place] = pair,
// place[pair] = its place; tiles[2 i] and tiles[2 i + 1] are the expert and the first place of
// tile i, n_tiles[0] their number.  Which of an expert's places a pair gets is decided by atomic
// counters and may differ from run to run; every row of the products is computed by itself, so no
// result depends on it.
constexpr int PL_BLOCK = 1024;

__global__ void __launch_bounds__(PL_BLOCK)
moe_plan_kernel(const int* __restrict__ chosen, int n_pairs, int n_experts, int* __restrict__ offsets,
                int* __restrict__ order, int* __restrict__ place, int* __restrict__ tiles, int* __restrict__ n_tiles,
                int max_tiles) {
    extern __shared__ int pl_smem[];            // [n_experts] counts, then [n_experts] cursors
    int* count = pl_smem;
    int* cursor = pl_smem + n_experts;
    for (int e = threadIdx.x; e < n_experts; e += PL_BLOCK) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += PL_BLOCK) atomicAdd(&count[chosen[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, nt = 0;
        for (int e = 0; e < n_experts; ++e) {
            offsets[e] = at;
            cursor[e] = at;
            for (int r = 0; r < count[e] && nt < max_tiles; r += MOE_TM) {
                tiles[2 * nt] = e;
                tiles[2 * nt + 1] = at + r;
                ++nt;
            }
            at += count[e];
        }
        offsets[n_experts] = at;
        n_tiles[0] = nt;
    }
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += PL_BLOCK) {
        int at = atomicAdd(&cursor[chosen[p]], 1);
        order[at] = p;
        place[p] = at;
    }
}

ROCML_EXPORT int rocml_moe_plan(const int* chosen, int n_pairs, int n_experts, int* offsets, int* order, int* place,
                                int* tiles, int* n_tiles, int max_tiles, hipStream_t stream) {
    ROCML_REQUIRE(n_pairs >= 0 && n_experts > 0 && n_experts <= 4096, "moe_plan: bad sizes pairs=%d experts=%d", n_pairs, n_experts);
    // an expert's last tile may be short, so there can be one more tile per expert than whole ones
    ROCML_REQUIRE(max_tiles >= (n_pairs < n_pairs / MOE_TM + n_experts ? n_pairs : n_pairs / MOE_TM + n_experts),
                  "moe_plan: room for %d tiles is too little for %d pairs of %d experts", max_tiles, n_pairs, n_experts);
    ROCML_REQUIRE(chosen && offsets && order && place && tiles && n_tiles, "moe_plan: missing arguments");
    moe_plan_kernel<<<1, PL_BLOCK, 2 * n_experts * sizeof(int), stream>>>(chosen, n_pairs, n_experts, offsets, order, place, tiles,
                                                                           n_tiles, max_tiles);
    ROCML_CHECK_LAUNCH("moe_plan");
    return 0;
}

// ---- the experts' products -------------------------------------------------------------
// For every place r of expert e: out[r, :] = W_e a(r), W_e = w + e * w_expert_stride ([N, K],
// rows ldw apart).  a(r) is row order[r] / top of `a` when `order` is given (the rows of the
// step's tokens, gathered) and row r otherwise (rows already in the plan's order).  DUAL: a second
// matrix w2 of the same shape, and out[r, j] = act(W_e a)[j] * (W2_e a)[j] with act = silu (a gated
// feed-forward's first two products and its activation in one pass).  Block (x, y): columns
// 64 x .. 64 x + 63 of tile y; blocks beyond the plan's number of tiles leave at once.
struct MoeGemmArgs {
    const void* a;
    int lda;
    const int* order;
    int top;
    const void* w;
    const void* w2;
    long long w_expert_stride;
    int ldw;
    void* out;
    int ldo;
    int n, k;
    const int* offsets;
    const int* tiles;
    const int* n_tiles;
};

__device__ __forceinline__ float moe_silu(float z) { return z / (1.0f + expf(-z)); }

// Any sizes and types, fused multiply-add in 32-bit: the whole 32-bit path and shapes the
// matrix-core kernel refuses.  64 x 64 outputs at a time (a tile's rows in MOE_TM / 64 passes), 4 x 4
// per thread, K staged 16 at a time.
template <typename TA, typename TW, typename TO, bool DUAL>
__global__ void __launch_bounds__(256)
moe_gemm_plain_kernel(MoeGemmArgs g) {
    int tile = blockIdx.y;
    if (tile >= g.n_tiles[0]) return;
    __shared__ float as[16][64 + 4];
    __shared__ float ws[16][64 + 4];
    __shared__ float ws2[DUAL ? 16 : 1][64 + 4];
    __shared__ int src[64];
    int expert = g.tiles[2 * tile], tile_r0 = g.tiles[2 * tile + 1];
    int r_end = g.offsets[expert + 1];
    int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    int n0 = blockIdx.x * 64;
    const TA* a = (const TA*)g.a;
    const TW* w = (const TW*)g.w + (size_t)expert * g.w_expert_stride;
    const TW* w2 = DUAL ? (const TW*)g.w2 + (size_t)expert * g.w_expert_stride : nullptr;
  for (int r0 = tile_r0; r0 < min(tile_r0 + MOE_TM, r_end); r0 += 64) {
    __syncthreads();
    if (tid < 64) {
        int r = r0 + tid;
        src[tid] = r < r_end ? (g.order ? g.order[r] / g.top : r) : -1;
    }
    __syncthreads();
    float acc[4][4] = {}, acc2[DUAL ? 4 : 1][4] = {};
    for (int k0 = 0; k0 < g.k; k0 += 16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int idx = tid + i * 256;
            int kk = idx % 16, r = idx / 16;
            int gk = k0 + kk, gn = n0 + r;
            int row = src[r];
            as[kk][r] = (row >= 0 && gk < g.k) ? Elem<TA>::load(a + (size_t)row * g.lda + gk) : 0.f;
            bool w_ok = gn < g.n && gk < g.k;
            ws[kk][r] = w_ok ? Elem<TW>::load(w + (size_t)gn * g.ldw + gk) : 0.f;
            if (DUAL) ws2[kk][r] = w_ok ? Elem<TW>::load(w2 + (size_t)gn * g.ldw + gk) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float av[4], bv[4], b2[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                bv[j] = ws[kk][tx * 4 + j];
                if (DUAL) b2[j] = ws2[kk][tx * 4 + j];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
                    if (DUAL) acc2[i][j] = fmaf(av[i], b2[j], acc2[i][j]);
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int r = r0 + ty * 4 + i;
        if (r >= r_end) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int gn = n0 + tx * 4 + j;
            if (gn >= g.n) continue;
            float v = DUAL ? moe_silu(acc[i][j]) * acc2[DUAL ? i : 0][j] : acc[i][j];
            Elem<TO>::store((TO*)g.out + (size_t)r * g.ldo + gn, v);
        }
    }
  }
}

// bfloat16 operands on the matrix cores (v_mfma_f32_16x16x32_bf16), 32-bit sums.  Four waves a
// block; a wave owns 16 of the block's 64 columns and all MOE_TM rows (a weight fragment from memory
// meets MOE_TM / 16 row fragments from LDS).  The rows' activations (gathered)
// go through LDS 64 values of K at a time; a wave's weight fragments come straight from memory
// (a lane reads 16 bytes of one weight row), requested a stage ahead.  K must be a multiple of 8.
typedef __attribute__((ext_vector_type(8))) __bf16 moe_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float moe_f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t moe_u32x4_t;
constexpr int MG_KC = 64;                  // K values per stage
constexpr int MG_ROW = MG_KC / 8 + 1;      // 16-byte pieces per LDS row, one of padding

template <typename TO, bool DUAL, int NT>
__global__ void __launch_bounds__(256)
moe_gemm_mfma_kernel(MoeGemmArgs g) {
    // NT: 16-column fragments a wave owns (a block is 64 NT columns wide); a row fragment read from LDS
    // meets NT weight fragments (2 NT with a second matrix), and the LDS, which all four waves share,
    // moves 1 / NT of the bytes per product.
    int tile = blockIdx.y;
    if (tile >= g.n_tiles[0]) return;
    __shared__ moe_u32x4_t xs[2][MOE_TM * MG_ROW];
    __shared__ int src[MOE_TM];
    int expert = g.tiles[2 * tile], r0 = g.tiles[2 * tile + 1];
    int r_end = g.offsets[expert + 1];
    int tid = threadIdx.x, wave = tid / WAVE, lane = tid & (WAVE - 1);
    int n0 = (blockIdx.x * 4 + wave) * 16 * NT;
    if (tid < MOE_TM) {
        int r = r0 + tid;
        src[tid] = r < r_end ? (g.order ? g.order[r] / g.top : r) : -1;
    }
    __syncthreads();
    const bf16_t* a = (const bf16_t*)g.a;
    // a lane's weight rows (clamped to the matrix: columns beyond N are computed and not stored)
    const bf16_t* w[NT];
    const bf16_t* w2[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        size_t wrow = (size_t)expert * g.w_expert_stride + (size_t)min(n0 + nt * 16 + (lane & 15), g.n - 1) * g.ldw;
        w[nt] = (const bf16_t*)g.w + wrow;
        w2[nt] = DUAL ? (const bf16_t*)g.w2 + wrow : nullptr;
    }
    int kq = (lane >> 4) * 8;              // the lane's 8 K values inside a 32-wide step
    // the 16-byte pieces of the activations this thread stages: rows tid / 8 + 32 i
    constexpr int MT = MOE_TM / 16, XP = MOE_TM / 32, D2 = DUAL ? 1 : 0;
    int piece_k = (tid & 7) * 8;
    int rows_x[XP];
#pragma unroll
    for (int i = 0; i < XP; ++i) rows_x[i] = src[(tid >> 3) + 32 * i];
    moe_f32x4_t acc[NT][MT], acc2[DUAL ? NT : 1][DUAL ? MT : 1];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            acc[nt][i] = moe_f32x4_t{0.f, 0.f, 0.f, 0.f};
            if (DUAL) acc2[nt * D2][i * D2] = moe_f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
    const moe_u32x4_t zero = {0u, 0u, 0u, 0u};
    int n_stages = (g.k + MG_KC - 1) / MG_KC;
    moe_u32x4_t xr[XP], wf[NT][2], wf2[DUAL ? NT : 1][2];
#define MG_LOAD(stage_)                                                                                        \
    {                                                                                                          \
        int kb_ = (stage_) * MG_KC;                                                                            \
        int gk_ = kb_ + piece_k;                                                                               \
        _Pragma("unroll") for (int i = 0; i < XP; ++i)                                                         \
            xr[i] = (rows_x[i] >= 0 && gk_ < g.k) ? *(const moe_u32x4_t*)(a + (size_t)rows_x[i] * g.lda + gk_) : zero; \
        _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                                      \
            _Pragma("unroll") for (int j = 0; j < 2; ++j) {                                                    \
                int wk_ = min(kb_ + j * 32 + kq, g.k - 8);   /* beyond K the activations are zero */           \
                wf[nt][j] = *(const moe_u32x4_t*)(w[nt] + wk_);                                                \
                if (DUAL) wf2[nt * D2][j] = *(const moe_u32x4_t*)(w2[nt] + wk_);                               \
            }                                                                                                  \
    }
    MG_LOAD(0)
    for (int s = 0; s < n_stages; ++s) {
        int buf = s & 1;
#pragma unroll
        for (int i = 0; i < XP; ++i) xs[buf][((tid >> 3) + 32 * i) * MG_ROW + (tid & 7)] = xr[i];
        moe_u32x4_t wc[NT][2], wc2[DUAL ? NT : 1][2];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                wc[nt][j] = wf[nt][j];
                if (DUAL) wc2[nt * D2][j] = wf2[nt * D2][j];
            }
        __syncthreads();                   // (two buffers: the one written two stages ago is free again)
        if (s + 1 < n_stages) MG_LOAD(s + 1)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                moe_bf16x8_t xv = __builtin_bit_cast(moe_bf16x8_t, xs[buf][(mt * 16 + (lane & 15)) * MG_ROW + j * 4 + (lane >> 4)]);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(moe_bf16x8_t, wc[nt][j]), xv, acc[nt][mt], 0, 0, 0);
                    if (DUAL)
                        acc2[nt * D2][mt * D2] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(moe_bf16x8_t, wc2[nt * D2][j]), xv,
                                                                                         acc2[nt * D2][mt * D2], 0, 0, 0);
                }
            }
        }
    }
#undef MG_LOAD
    // acc[nt][mt][e]: row mt * 16 + (lane & 15) of the tile, column n0 + nt * 16 + (lane >> 4) * 4 + e
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            int r = r0 + mt * 16 + (lane & 15);
            if (r >= r_end) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                int gn = n0 + nt * 16 + (lane >> 4) * 4 + e;
                if (gn >= g.n) continue;
                float v = DUAL ? moe_silu(acc[nt][mt][e]) * acc2[nt * D2][mt * D2][e] : acc[nt][mt][e];
                Elem<TO>::store((TO*)g.out + (size_t)r * g.ldo + gn, v);
            }
        }
}

ROCML_EXPORT int rocml_moe_gemm(const void* a, int a_dtype, int lda, int a_rows, const int* order, int top, const void* w,
                                const void* w2, int w_dtype, long long w_expert_stride, int ldw, int n_experts, void* out,
                                int out_dtype, int ldo, int n_pairs, int n, int k, const int* offsets, const int* tiles,
                                const int* n_tiles, int max_tiles, int plain, hipStream_t stream) {
    ROCML_REQUIRE(n_pairs >= 0 && n > 0 && k > 0 && n_experts > 0 && top >= 1, "moe_gemm: bad sizes pairs=%d n=%d k=%d", n_pairs, n, k);
    ROCML_REQUIRE(lda >= k && ldw >= k && ldo >= n && w_expert_stride >= (long long)(n - 1) * ldw + k,
                  "moe_gemm: strides do not fit the shapes (lda=%d ldw=%d ldo=%d)", lda, ldw, ldo);
    ROCML_REQUIRE(a && w && out && offsets && tiles && n_tiles, "moe_gemm: missing arguments");
    ROCML_REQUIRE(order ? (long long)a_rows * top >= n_pairs : a_rows >= n_pairs, "moe_gemm: %d rows for %d pairs", a_rows, n_pairs);
    ROCML_REQUIRE(max_tiles >= ceil_div(n_pairs, MOE_TM) && max_tiles >= 1 && max_tiles < 65536, "moe_gemm: room for %d tiles", max_tiles);
    ROCML_REQUIRE(a_dtype == w_dtype, "moe_gemm: activations and weights must share their type");
    if (n_pairs == 0) return 0;
    MoeGemmArgs g{a, lda, order, top, w, w2, w_expert_stride, ldw, out, ldo, n, k, offsets, tiles, n_tiles};
    dim3 grid(ceil_div(n, 64), max_tiles);
    bool dual = w2 != nullptr;
    bool mfma = !plain && a_dtype == ROCML_BF16 && k % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && w_expert_stride % 8 == 0;
    if (mfma) {
        // Blocks of 128 columns where the matrix is at least that wide and there is one matrix: a row fragment
        // then meets two weight fragments either way.  (With a second matrix and 128 columns the sums need 256
        // registers beside the operands, a CU holds one block, and the pass is slower: 2,997 against 2,538 us
        // for 32,768 rows of 3072 x 4096; with one matrix 1,386 against 1,649.)
        bool wide = n >= 128 && !dual;
        dim3 mgrid(ceil_div(n, wide ? 128 : 64), max_tiles);
#define MG(TO_, DUAL_) { if (wide) moe_gemm_mfma_kernel<TO_, DUAL_, 2><<<mgrid, 256, 0, stream>>>(g); \
                         else moe_gemm_mfma_kernel<TO_, DUAL_, 1><<<mgrid, 256, 0, stream>>>(g); }
        if (dual && out_dtype == ROCML_BF16) MG(bf16_t, true)
        else if (!dual && out_dtype == ROCML_F32) MG(float, false)
        else if (dual && out_dtype == ROCML_F32) MG(float, true)
        else MG(bf16_t, false)
#undef MG
    } else if (a_dtype == ROCML_F32 && out_dtype == ROCML_F32) {
        if (dual) moe_gemm_plain_kernel<float, float, float, true><<<grid, 256, 0, stream>>>(g);
        else moe_gemm_plain_kernel<float, float, float, false><<<grid, 256, 0, stream>>>(g);
    } else if (a_dtype == ROCML_BF16 && out_dtype == ROCML_BF16) {
        if (dual) moe_gemm_plain_kernel<bf16_t, bf16_t, bf16_t, true><<<grid, 256, 0, stream>>>(g);
        else moe_gemm_plain_kernel<bf16_t, bf16_t, bf16_t, false><<<grid, 256, 0, stream>>>(g);
    } else if (a_dtype == ROCML_BF16 && out_dtype == ROCML_F32) {
        if (dual) moe_gemm_plain_kernel<bf16_t, bf16_t, float, true><<<grid, 256, 0, stream>>>(g);
        else moe_gemm_plain_kernel<bf16_t, bf16_t, float, false><<<grid, 256, 0, stream>>>(g);
    } else {
        return rocml_fail("moe_gemm: unsupported types a=%d out=%d", a_dtype, out_dtype);
    }
    ROCML_CHECK_LAUNCH("moe_gemm");
    return 0;
}

// ---- the weighted sum -------------------------------------------------------------------
// out[t, :] (+)= sum_c weight[t, c] * y[place[t * top + c], :], choices in order (32-bit).
__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ place, const float* __restrict__ weight,
                   float* __restrict__ out, int top, int n, long long total, int accumulate) {
    long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    long long t = idx / n;
    int i = (int)(idx - t * n);
    float sum = 0.f;
    for (int c = 0; c < top; ++c) sum = fmaf(weight[t * top + c], y[(size_t)place[t * top + c] * n + i], sum);
    out[idx] = accumulate ? out[idx] + sum : sum;
}

ROCML_EXPORT int rocml_moe_combine(const float* y, const int* place, const float* weight, float* out, int n_tokens, int top,
                                   int n, int accumulate, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && top >= 1 && n > 0, "moe_combine: bad sizes T=%d top=%d n=%d", n_tokens, top, n);
    ROCML_REQUIRE(y && place && weight && out, "moe_combine: missing arguments");
    long long total = (long long)n_tokens * n;
    if (total == 0) return 0;
    moe_combine_kernel<<<ceil_div(total, 256), 256, 0, stream>>>(y, place, weight, out, top, n, total, accumulate);
    ROCML_CHECK_LAUNCH("moe_combine");
    return 0;
}
