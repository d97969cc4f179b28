// Kernels of mixers that carry a state of fixed size from token to token (gfx950, wave64): the
// short causal convolution in front of a recurrence, the recurrence with one scalar decay per head
// (state-space duality), and the gated norm in equal parts behind it.  Everything here is 32-bit:
// the inputs of the recurrence, step sizes, decays, the state and the norm's statistics.
//
// A step brings, per sequence b, the tokens cu_seqlens[b] .. cu_seqlens[b + 1] - 1 of the packed
// batch, in order; the sequence's state lives in row seq_slots[b] of the state tensors and is zero
// when the sequence starts.  A step of one token per sequence and a step of a whole prompt run the
// same arithmetic per token, in the same order, so the result does not depend on how a prompt
// was cut.
#include "common.h"

ROCML_LAST_ERROR_FN(recurrent)

constexpr int RC_BLOCK = 256;

__device__ __forceinline__ float rc_silu(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float rc_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// ---- causal convolution per channel ------------------------------------------------
// out[t, c] = act(bias[c] + sum_j w[j, c] * in(t - (taps - 1) + j, c)): w is [taps, C] (a tap's weights of
// neighbouring channels lie side by side, as the threads that read them do), its last row the current token's.  Inputs before the step's first token of a sequence come from the
// sequence's state [slot, taps - 1, C] (its last taps - 1 inputs, oldest first; zeros at the
// start).  u is [T, ldu] 32-bit and the channels are its columns col0 .. col0 + C - 1.
constexpr int CONV_MAX_TAPS = 8;

__global__ void __launch_bounds__(RC_BLOCK)
causal_conv_kernel(const float* __restrict__ u, int ldu, int col0, int n_channels, int taps,
                   const float* __restrict__ w, const float* __restrict__ bias, const float* __restrict__ state,
                   const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                   const int* __restrict__ seq_slots, float* __restrict__ out, long long total, int silu) {
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx >= total) return;
    int t = (int)(idx / n_channels), c = (int)(idx - (long long)t * n_channels);
    int b = token_seq[t];
    int local = t - cu_seqlens[b];
    const float* st = state + (size_t)seq_slots[b] * (taps - 1) * n_channels;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        int src = local - (taps - 1) + j;
        float v = src >= 0 ? u[(size_t)(t - (taps - 1) + j) * ldu + col0 + c] : st[(size_t)(taps - 1 + src) * n_channels + c];
        acc = fmaf(w[(size_t)j * n_channels + c], v, acc);
    }
    out[idx] = silu ? rc_silu(acc) : acc;
}

// Four neighbouring channels per thread, as 16-byte pieces (channels, first column and row strides are
// multiples of 4): a quarter of the loads and of the index arithmetic.
typedef float cv_f4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(RC_BLOCK)
causal_conv_vec_kernel(const float* __restrict__ u, int ldu, int col0, int n_channels, int taps,
                       const float* __restrict__ w, const float* __restrict__ bias, const float* __restrict__ state,
                       const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                       const int* __restrict__ seq_slots, float* __restrict__ out, long long total4, int silu) {
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx >= total4) return;
    int c4 = n_channels / 4;
    int t = (int)(idx / c4), c = (int)(idx - (long long)t * c4) * 4;
    int b = token_seq[t];
    int local = t - cu_seqlens[b];
    const float* st = state + (size_t)seq_slots[b] * (taps - 1) * n_channels;
    cv_f4 acc = bias ? *(const cv_f4*)(bias + c) : cv_f4{0.f, 0.f, 0.f, 0.f};
    cv_f4 v[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        if (j >= taps) break;
        int src = local - (taps - 1) + j;
        v[j] = src >= 0 ? *(const cv_f4*)(u + (size_t)(t - (taps - 1) + j) * ldu + col0 + c)
                        : *(const cv_f4*)(st + (size_t)(taps - 1 + src) * n_channels + c);
    }
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        if (j >= taps) break;
        cv_f4 wj = *(const cv_f4*)(w + (size_t)j * n_channels + c);
        acc.x = fmaf(wj.x, v[j].x, acc.x);
        acc.y = fmaf(wj.y, v[j].y, acc.y);
        acc.z = fmaf(wj.z, v[j].z, acc.z);
        acc.w = fmaf(wj.w, v[j].w, acc.w);
    }
    if (silu) { acc.x = rc_silu(acc.x); acc.y = rc_silu(acc.y); acc.z = rc_silu(acc.z); acc.w = rc_silu(acc.w); }
    *(cv_f4*)(out + (size_t)t * n_channels + c) = acc;
}

// The state after the step: the last taps - 1 inputs of each sequence, taken from the step's
// tokens and, where the step brought fewer, from the old state.  Runs after the outputs.
__global__ void __launch_bounds__(RC_BLOCK)
causal_conv_state_kernel(const float* __restrict__ u, int ldu, int col0, int n_channels, int taps,
                         float* __restrict__ state, const int* __restrict__ cu_seqlens,
                         const int* __restrict__ seq_slots, long long total) {
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx >= total) return;
    int b = (int)(idx / n_channels), c = (int)(idx - (long long)b * n_channels);
    int first = cu_seqlens[b], n = cu_seqlens[b + 1] - first;
    float* st = state + (size_t)seq_slots[b] * (taps - 1) * n_channels;
    float keep[CONV_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        int src = n - (taps - 1) + k;
        keep[k] = src >= 0 ? u[(size_t)(first + src) * ldu + col0 + c] : st[(size_t)(taps - 1 + src) * n_channels + c];
    }
#pragma unroll
    for (int k = 0; k < CONV_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        st[(size_t)k * n_channels + c] = keep[k];
    }
}

// A step of one token per sequence: output and new state in one launch.  A thread takes W channels
// (1, or 4 as a 16-byte piece) of one sequence, reads its kept inputs, forms the output and moves
// the kept inputs up by one.
template <int W>
__global__ void __launch_bounds__(RC_BLOCK)
causal_conv_step_kernel(const float* __restrict__ u, int ldu, int col0, int n_channels, int taps,
                        const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ state,
                        const int* __restrict__ seq_slots, float* __restrict__ out, long long total, int silu) {
    typedef float vec_t __attribute__((ext_vector_type(W)));
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx >= total) return;
    int cw = n_channels / W;
    int b = (int)(idx / cw), c = (int)(idx - (long long)b * cw) * W;
    float* st = state + (size_t)seq_slots[b] * (taps - 1) * n_channels;
    vec_t v[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        if (j >= taps) break;
        v[j] = j < taps - 1 ? *(const vec_t*)(st + (size_t)j * n_channels + c) : *(const vec_t*)(u + (size_t)b * ldu + col0 + c);
    }
#pragma unroll
    for (int e = 0; e < W; ++e) {
        float acc = bias ? bias[c + e] : 0.f;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; ++j) {
            if (j >= taps) break;
            float in = W == 1 ? ((const float*)&v[j])[0] : ((const float*)&v[j])[e];
            acc = fmaf(w[(size_t)j * n_channels + c + e], in, acc);
        }
        out[(size_t)b * n_channels + c + e] = silu ? rc_silu(acc) : acc;
    }
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        if (j >= taps - 1) break;
        *(vec_t*)(st + (size_t)j * n_channels + c) = v[j + 1];
    }
}

ROCML_EXPORT int rocml_causal_conv(const float* u, int ldu, int col0, int n_tokens, int n_channels, int taps,
                                   const float* w, const float* bias, float* state, int n_slots,
                                   const int* token_seq, const int* cu_seqlens, const int* seq_slots, int n_seqs,
                                   float* out, int silu, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && n_channels > 0 && n_seqs >= 0 && n_slots > 0, "causal_conv: bad sizes T=%d C=%d B=%d", n_tokens,
                  n_channels, n_seqs);
    ROCML_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "causal_conv: %d taps (1 to %d)", taps, CONV_MAX_TAPS);
    ROCML_REQUIRE(col0 >= 0 && ldu >= col0 + n_channels, "causal_conv: row stride %d too small for columns %d..%d", ldu, col0,
                  col0 + n_channels);
    ROCML_REQUIRE(u && w && out && token_seq && cu_seqlens && seq_slots && (taps == 1 || state), "causal_conv: missing arguments");
    if (n_tokens == 0 || n_seqs == 0) return 0;
    long long total = (long long)n_tokens * n_channels;
    if (n_tokens == n_seqs) {
        // one token per sequence (every sequence brings at least one): token b is sequence b's
        bool vec4 = n_channels % 4 == 0 && col0 % 4 == 0 && ldu % 4 == 0 && (((uintptr_t)u | (uintptr_t)state) & 15) == 0;
        if (vec4)
            causal_conv_step_kernel<4><<<ceil_div(total / 4, RC_BLOCK), RC_BLOCK, 0, stream>>>(u, ldu, col0, n_channels, taps, w, bias,
                                                                                             state, seq_slots, out, total / 4, silu);
        else
            causal_conv_step_kernel<1><<<ceil_div(total, RC_BLOCK), RC_BLOCK, 0, stream>>>(u, ldu, col0, n_channels, taps, w, bias,
                                                                                         state, seq_slots, out, total, silu);
        ROCML_CHECK_LAUNCH("causal_conv step");
        return 0;
    }
    bool vec = n_channels % 4 == 0 && col0 % 4 == 0 && ldu % 4 == 0 && (((uintptr_t)u | (uintptr_t)out | (uintptr_t)state | (uintptr_t)bias | (uintptr_t)w) & 15) == 0;
    if (vec)
        causal_conv_vec_kernel<<<ceil_div(total / 4, RC_BLOCK), RC_BLOCK, 0, stream>>>(u, ldu, col0, n_channels, taps, w, bias, state,
                                                                                       token_seq, cu_seqlens, seq_slots, out, total / 4, silu);
    else
        causal_conv_kernel<<<ceil_div(total, RC_BLOCK), RC_BLOCK, 0, stream>>>(u, ldu, col0, n_channels, taps, w, bias, state, token_seq,
                                                                               cu_seqlens, seq_slots, out, total, silu);
    ROCML_CHECK_LAUNCH("causal_conv");
    if (taps > 1) {
        long long st_total = (long long)n_seqs * n_channels;
        causal_conv_state_kernel<<<ceil_div(st_total, RC_BLOCK), RC_BLOCK, 0, stream>>>(u, ldu, col0, n_channels, taps, state,
                                                                                       cu_seqlens, seq_slots, st_total);
        ROCML_CHECK_LAUNCH("causal_conv state");
    }
    return 0;
}

// ---- the recurrence ----------------------------------------------------------------
// Per head a (group g = a / (H / G)) and token t, with x_t [P], B_t and C_t [N] from xbc (rows of
// [x: H * P | B: G * N | C: G * N]) and the raw step size from column dt_col0 + a of dtsrc:
//     dt = softplus(raw + dt_bias[a]),  S <- exp(-exp(A_log[a]) dt) S + dt B_t x_t^T,
//     y_t = S^T C_t + D[a] x_t.
// The columns of S (one per value p) do not depend on each other: a block takes one sequence, one
// head and SC_PT values and walks the sequence's tokens in order.  Thread (pair of columns, r) keeps
// the state entries n = r * NI .. r * NI + NI - 1 of its two columns in registers (2 NI numbers); the
// 16 threads of a column pair sit in one row of 16 lanes and add up their parts of S^T C with four
// cross-lane additions inside the row, in a fixed order.  Tokens come through LDS tc at a time, B and
// C rows padded with zeros to 16 NI numbers so that a thread reads its NI numbers as whole vectors.
// State layout: [slot, H, P, N].
typedef float sc_f4 __attribute__((ext_vector_type(4)));      // 16 bytes as a native vector
constexpr int SC_R = 16, SC_PP = 2, SC_PT = RC_BLOCK / SC_R * SC_PP, SC_MAX_TC = 32, SC_U = 4;

// sum over the 16 lanes of a row, the same in every lane: lanes 1 apart, 2 apart, mirrored inside a
// half row, mirrored inside the row
__device__ __forceinline__ float row16_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false));
    return v;
}

// A thread's NI state entries of one column, n = r * NI ..: as 16-byte pieces where NI is a multiple of 4 and
// the state is exactly 16 NI long (one load instruction of a wave then touches 16 memory lines, not 64).
template <int NI>
__device__ __forceinline__ void sc_load_state(float (&s)[NI], const float* col, int r, int n_state, bool p_ok) {
    if (NI % 4 == 0 && n_state == SC_R * NI) {
#pragma unroll
        for (int i = 0; i < NI; i += 4) {
            sc_f4 v = p_ok ? *(const sc_f4*)(col + r * NI + i) : sc_f4{0.f, 0.f, 0.f, 0.f};
            s[i] = v.x; s[i + 1] = v.y; s[i + 2] = v.z; s[i + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int n = r * NI + i;
            s[i] = (p_ok && n < n_state) ? col[n] : 0.f;
        }
    }
}

template <int NI>
__device__ __forceinline__ void sc_store_state(const float (&s)[NI], float* col, int r, int n_state, bool p_ok) {
    if (!p_ok) return;
    if (NI % 4 == 0 && n_state == SC_R * NI) {
#pragma unroll
        for (int i = 0; i < NI; i += 4) *(sc_f4*)(col + r * NI + i) = sc_f4{s[i], s[i + 1], s[i + 2], s[i + 3]};
    } else {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int n = r * NI + i;
            if (n < n_state) col[n] = s[i];
        }
    }
}

template <int NI, bool VEC>
__global__ void __launch_bounds__(RC_BLOCK)
ssd_scan_kernel(const float* __restrict__ xbc, int ldx, const float* __restrict__ dtsrc, int lddt, int dt_col0,
                const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
                float* __restrict__ state, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots,
                float* __restrict__ y, int n_heads, int head_dim, int n_state, int n_groups, int tc) {
    extern __shared__ float4 sc_smem4[];
    constexpr int NP = SC_R * NI;              // padded length of a B or C row
    float* bs = (float*)sc_smem4;              // [tc][NP]
    float* cs = bs + tc * NP;                  // [tc][NP]
    float* xs = cs + tc * NP;                  // [tc][SC_PT]
    float* ys = xs + tc * SC_PT;               // [tc][SC_PT]
    float* dts = ys + tc * SC_PT;              // [tc][2]: step size, decay
    int p0 = blockIdx.x * SC_PT, head = blockIdx.y, b = blockIdx.z;
    int tid = threadIdx.x, r = tid % SC_R, pl = tid / SC_R;
    int group = head / (n_heads / n_groups);
    int inner = n_heads * head_dim;
    int first = cu_seqlens[b], n_tok = cu_seqlens[b + 1] - first;
    float* st_head = state + ((size_t)seq_slots[b] * n_heads + head) * head_dim * n_state;
    float s[SC_PP][NI];
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        sc_load_state<NI>(s[j], st_head + (size_t)min(p, head_dim - 1) * n_state, r, n_state, p < head_dim);
    }
    float a_rate = expf(a_log[head]), bias = dt_bias[head], skip = d_skip[head];
    // VEC (rows of the inputs and the sizes are multiples of 4 numbers): a chunk's operands are asked
    // for as 16-byte pieces, all at once, while the chunk before it is worked on, and reach LDS when
    // that is done; a block is alone on its CU for most launches, and a chunk's loads one after the
    // other, with nothing to do meanwhile, would take longer than its arithmetic.
    constexpr int PF = VEC ? (SC_MAX_TC * NP / 4 + RC_BLOCK - 1) / RC_BLOCK : 1;
    sc_f4 pre_b[PF], pre_c[PF], pre_x;
    float pre_dt = 0.f;
    const sc_f4 zero4 = {0.f, 0.f, 0.f, 0.f};
    pre_x = zero4;
#define SC_PREFETCH(c0_)                                                                                         \
    {                                                                                                            \
        int nt_ = min(tc, n_tok - (c0_));                                                                        \
        _Pragma("unroll") for (int j = 0; j < PF; ++j) {                                                         \
            int i4 = tid + j * RC_BLOCK, tt = i4 / (NP / 4), n = (i4 - tt * (NP / 4)) * 4;                       \
            bool ok = tt < nt_ && n < n_state;                                                                   \
            const float* row = xbc + (size_t)(first + (c0_) + (ok ? tt : 0)) * ldx + inner + (size_t)group * n_state + (ok ? n : 0); \
            pre_b[j] = ok ? *(const sc_f4*)row : zero4;                                                         \
            pre_c[j] = ok ? *(const sc_f4*)(row + (size_t)n_groups * n_state) : zero4;                          \
        }                                                                                                        \
        {                                                                                                        \
            int tt = tid / (SC_PT / 4), pp = (tid - tt * (SC_PT / 4)) * 4;                                       \
            bool ok = tt < nt_ && p0 + pp < head_dim;                                                            \
            pre_x = ok ? *(const sc_f4*)(xbc + (size_t)(first + (c0_) + tt) * ldx + (size_t)head * head_dim + p0 + pp) : zero4; \
        }                                                                                                        \
        pre_dt = tid < nt_ ? dtsrc[(size_t)(first + (c0_) + tid) * lddt + dt_col0 + head] : 0.f;                 \
    }
    if (VEC && n_tok > 0) SC_PREFETCH(0)
    for (int c0 = 0; c0 < n_tok; c0 += tc) {
        int nt = min(tc, n_tok - c0);
        int nt_up = (nt + SC_U - 1) / SC_U * SC_U;
        __syncthreads();                          // the previous chunk's outputs have been written out
        if (VEC) {
            // (rows past the chunk's end were fetched as zeros: a step of zero and a decay of one leave the state alone)
#pragma unroll
            for (int j = 0; j < PF; ++j) {
                int i4 = tid + j * RC_BLOCK;
                if (i4 < tc * (NP / 4)) {
                    ((sc_f4*)bs)[i4] = pre_b[j];
                    ((sc_f4*)cs)[i4] = pre_c[j];
                }
            }
            if (tid < tc * (SC_PT / 4)) ((sc_f4*)xs)[tid] = pre_x;
            if (tid < tc) {
                float dt = tid < nt ? rc_softplus(pre_dt + bias) : 0.f;
                dts[2 * tid] = dt;
                dts[2 * tid + 1] = tid < nt ? expf(-a_rate * dt) : 1.f;
            }
            __syncthreads();
            if (c0 + tc < n_tok) SC_PREFETCH(c0 + tc)
        } else {
            for (int i = tid; i < nt * NP; i += RC_BLOCK) {
                int tt = i / NP, n = i - tt * NP;
                const float* row = xbc + (size_t)(first + c0 + tt) * ldx + inner + (size_t)group * n_state + n;
                bool ok = n < n_state;
                bs[i] = ok ? row[0] : 0.f;
                cs[i] = ok ? row[(size_t)n_groups * n_state] : 0.f;
            }
            for (int i = tid; i < nt * SC_PT; i += RC_BLOCK) {
                int tt = i / SC_PT, pp = i - tt * SC_PT;
                xs[i] = p0 + pp < head_dim ? xbc[(size_t)(first + c0 + tt) * ldx + (size_t)head * head_dim + p0 + pp] : 0.f;
            }
            if (tid < nt) {
                float dt = rc_softplus(dtsrc[(size_t)(first + c0 + tid) * lddt + dt_col0 + head] + bias);
                dts[2 * tid] = dt;
                dts[2 * tid + 1] = expf(-a_rate * dt);
            }
            // tokens that fill the chunk up to a multiple of SC_U: a step of zero and a decay of one
            for (int i = nt * NP + tid; i < nt_up * NP; i += RC_BLOCK) { bs[i] = 0.f; cs[i] = 0.f; }
            for (int i = nt * SC_PT + tid; i < nt_up * SC_PT; i += RC_BLOCK) xs[i] = 0.f;
            if (tid >= nt && tid < nt_up) { dts[2 * tid] = 0.f; dts[2 * tid + 1] = 1.f; }
            __syncthreads();
        }
        // SC_U tokens at a time: all their operands are read before the first is used and their sums
        // across lanes run side by side, so that a wave alone on its SIMD does not wait for every
        // load and every cross-lane step in turn.  Tokens past the chunk's end leave the state as it is.
        for (int t0 = 0; t0 < nt; t0 += SC_U) {
            float2 dd[SC_U], xv[SC_U];
            float bv[SC_U][NI], cv[SC_U][NI];
#pragma unroll
            for (int u = 0; u < SC_U; ++u) {
                int tt = t0 + u;
                dd[u] = *(const float2*)(dts + 2 * tt);
                xv[u] = *(const float2*)(xs + tt * SC_PT + pl * SC_PP);
                const float* bt = bs + tt * NP + r * NI;
                const float* ct = cs + tt * NP + r * NI;
                if (NI % 4 == 0) {
#pragma unroll
                    for (int i = 0; i < NI; i += 4) {
                        float4 b4 = *(const float4*)(bt + i), c4 = *(const float4*)(ct + i);
                        bv[u][i] = b4.x; bv[u][i + 1] = b4.y; bv[u][i + 2] = b4.z; bv[u][i + 3] = b4.w;
                        cv[u][i] = c4.x; cv[u][i + 1] = c4.y; cv[u][i + 2] = c4.z; cv[u][i + 3] = c4.w;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NI; ++i) { bv[u][i] = bt[i]; cv[u][i] = ct[i]; }
                }
            }
            float part0[SC_U], part1[SC_U];
#pragma unroll
            for (int u = 0; u < SC_U; ++u) {
                float dec = dd[u].y, dtx0 = dd[u].x * xv[u].x, dtx1 = dd[u].x * xv[u].y;
                float q0 = 0.f, q1 = 0.f;
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    s[0][i] = fmaf(dec, s[0][i], dtx0 * bv[u][i]);
                    s[1][i] = fmaf(dec, s[1][i], dtx1 * bv[u][i]);
                    q0 = fmaf(s[0][i], cv[u][i], q0);
                    q1 = fmaf(s[1][i], cv[u][i], q1);
                }
                part0[u] = q0;
                part1[u] = q1;
            }
#pragma unroll
            for (int u = 0; u < SC_U; ++u) {
                part0[u] = row16_sum(part0[u]);
                part1[u] = row16_sum(part1[u]);
            }
            if (r == 0) {
#pragma unroll
                for (int u = 0; u < SC_U; ++u)
                    *(float2*)(ys + (t0 + u) * SC_PT + pl * SC_PP) =
                        make_float2(fmaf(skip, xv[u].x, part0[u]), fmaf(skip, xv[u].y, part1[u]));
            }
        }
        __syncthreads();
        for (int i = tid; i < nt * SC_PT; i += RC_BLOCK) {
            int tt = i / SC_PT, pp = i - tt * SC_PT;
            if (p0 + pp < head_dim) y[(size_t)(first + c0 + tt) * inner + (size_t)head * head_dim + p0 + pp] = ys[i];
        }
    }
#undef SC_PREFETCH
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        sc_store_state<NI>(s[j], st_head + (size_t)min(p, head_dim - 1) * n_state, r, n_state, p < head_dim);
    }
}

// A step of one token per sequence: the same arithmetic for that token without the chunks: a thread
// reads its NI numbers of B and C and its two values of x straight from memory, next to its state
// entries, and nothing waits at a barrier.  Token b is sequence b's.
template <int NI>
__global__ void __launch_bounds__(RC_BLOCK)
ssd_step_kernel(const float* __restrict__ xbc, int ldx, const float* __restrict__ dtsrc, int lddt, int dt_col0,
                const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
                float* __restrict__ state, const int* __restrict__ seq_slots, float* __restrict__ y, int n_heads,
                int head_dim, int n_state, int n_groups, int vec_rows) {
    int p0 = blockIdx.x * SC_PT, head = blockIdx.y, b = blockIdx.z;
    int tid = threadIdx.x, r = tid % SC_R, pl = tid / SC_R;
    int group = head / (n_heads / n_groups);
    int inner = n_heads * head_dim;
    float* st_head = state + ((size_t)seq_slots[b] * n_heads + head) * head_dim * n_state;
    const float* row = xbc + (size_t)b * ldx;
    const float* brow = row + inner + (size_t)group * n_state;
    const float* crow = brow + (size_t)n_groups * n_state;
    float s[SC_PP][NI], bv[NI], cv[NI], xv[SC_PP];
    // (B and C are read like a column of the state; their rows start on 16 bytes where the vector form is taken:
    // the caller checks the strides)
    sc_load_state<NI>(bv, brow, r, vec_rows ? n_state : -1, true);
    sc_load_state<NI>(cv, crow, r, vec_rows ? n_state : -1, true);
    if (!vec_rows) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int n = r * NI + i;
            bool ok = n < n_state;
            bv[i] = ok ? brow[n] : 0.f;
            cv[i] = ok ? crow[n] : 0.f;
        }
    }
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        sc_load_state<NI>(s[j], st_head + (size_t)min(p, head_dim - 1) * n_state, r, n_state, p < head_dim);
    }
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        xv[j] = p < head_dim ? row[(size_t)head * head_dim + p] : 0.f;
    }
    float dt = rc_softplus(dtsrc[(size_t)b * lddt + dt_col0 + head] + dt_bias[head]);
    float dec = expf(-expf(a_log[head]) * dt), skip = d_skip[head];
    float part[SC_PP];
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        float dtx = dt * xv[j], q = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            s[j][i] = fmaf(dec, s[j][i], dtx * bv[i]);
            q = fmaf(s[j][i], cv[i], q);
        }
        part[j] = row16_sum(q);
    }
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        if (p >= head_dim) continue;
        if (r == 0) y[(size_t)b * inner + (size_t)head * head_dim + p] = fmaf(skip, xv[j], part[j]);
        sc_store_state<NI>(s[j], st_head + (size_t)p * n_state, r, n_state, true);
    }
}

ROCML_EXPORT int rocml_ssd_scan(const float* xbc, int ldx, const float* dtsrc, int lddt, int dt_col0,
                                const float* dt_bias, const float* a_log, const float* d_skip, float* state, int n_slots,
                                const int* cu_seqlens, const int* seq_slots, int n_seqs, int n_tokens, float* y,
                                int n_heads, int head_dim, int n_state, int n_groups, hipStream_t stream) {
    ROCML_REQUIRE(n_heads > 0 && head_dim > 0 && n_state > 0 && n_groups > 0 && n_heads % n_groups == 0,
                  "ssd_scan: bad sizes heads=%d head=%d state=%d groups=%d", n_heads, head_dim, n_state, n_groups);
    ROCML_REQUIRE(n_state <= 16 * SC_R, "ssd_scan: a state of %d exceeds %d", n_state, 16 * SC_R);
    ROCML_REQUIRE(ldx >= n_heads * head_dim + 2 * n_groups * n_state, "ssd_scan: input rows of %d are too short", ldx);
    ROCML_REQUIRE(dt_col0 >= 0 && lddt >= dt_col0 + n_heads, "ssd_scan: step-size rows of %d are too short", lddt);
    ROCML_REQUIRE(xbc && dtsrc && dt_bias && a_log && d_skip && state && cu_seqlens && seq_slots && y && n_slots > 0,
                  "ssd_scan: missing arguments");
    ROCML_REQUIRE(n_seqs >= 0 && n_seqs < 65536 && n_heads < 65536, "ssd_scan: too many sequences or heads for one launch");
    if (n_seqs == 0 || n_tokens == 0) return 0;
    dim3 grid(ceil_div(head_dim, SC_PT), n_heads, n_seqs);
    int ni = ceil_div(n_state, SC_R);
    ni = ni <= 4 ? ni : ni <= 6 ? 6 : ni <= 8 ? 8 : ni <= 12 ? 12 : 16;
    if (n_tokens == n_seqs) {          // one token per sequence (every sequence of a step brings at least one)
#define STEP(NI_)                                                                                              \
    ssd_step_kernel<NI_><<<grid, RC_BLOCK, 0, stream>>>(xbc, ldx, dtsrc, lddt, dt_col0, dt_bias, a_log, d_skip, state, \
                                                        seq_slots, y, n_heads, head_dim, n_state, n_groups, vec_rows)
        // B and C rows as 16-byte pieces: every row and every group's part starts on a multiple of 4 numbers
        int vec_rows = ldx % 4 == 0 && (n_heads * head_dim) % 4 == 0 && n_state % 4 == 0 && ((uintptr_t)xbc & 15) == 0;
        switch (ni) {
            case 1: STEP(1); break;
            case 2: STEP(2); break;
            case 3: STEP(3); break;
            case 4: STEP(4); break;
            case 6: STEP(6); break;
            case 8: STEP(8); break;
            case 12: STEP(12); break;
            default: STEP(16); break;
        }
#undef STEP
        ROCML_CHECK_LAUNCH("ssd_scan step");
        return 0;
    }
    int tc = ni <= 8 ? SC_MAX_TC : SC_MAX_TC / 2;          // 48 KB of LDS at most
    size_t lds = (size_t)(2 * tc * SC_R * ni + 2 * tc * SC_PT + 2 * tc) * sizeof(float);
    // whole 16-byte pieces: every row of x, B and C starts on a multiple of 4 numbers and ends on one
    bool vec = ldx % 4 == 0 && head_dim % 4 == 0 && n_state % 4 == 0 && ((uintptr_t)xbc & 15) == 0;
#define SCAN(NI_)                                                                                              \
    {                                                                                                          \
        if (vec)                                                                                               \
            ssd_scan_kernel<NI_, true><<<grid, RC_BLOCK, lds, stream>>>(xbc, ldx, dtsrc, lddt, dt_col0, dt_bias, a_log, d_skip, \
                                                                        state, cu_seqlens, seq_slots, y, n_heads, head_dim, \
                                                                        n_state, n_groups, tc);                \
        else                                                                                                   \
            ssd_scan_kernel<NI_, false><<<grid, RC_BLOCK, lds, stream>>>(xbc, ldx, dtsrc, lddt, dt_col0, dt_bias, a_log, d_skip, \
                                                                         state, cu_seqlens, seq_slots, y, n_heads, head_dim, \
                                                                         n_state, n_groups, tc);               \
    }
    switch (ni) {
        case 1: SCAN(1); break;
        case 2: SCAN(2); break;
        case 3: SCAN(3); break;
        case 4: SCAN(4); break;
        case 6: SCAN(6); break;
        case 8: SCAN(8); break;
        case 12: SCAN(12); break;
        default: SCAN(16); break;
    }
#undef SCAN
    ROCML_CHECK_LAUNCH("ssd_scan");
    return 0;
}

// ---- the matrix memory (mLSTM) --------------------------------------------------------
// Per head and token t, with q_t (times q_scale), k_t [dk] and v_t [dv] from columns of the 32-bit projection and
// the raw gates i~, f~ from two more of its columns:
//     i = cap tanh((i~ + bi) / cap),   f = logsigmoid(cap tanh((f~ + bf) / cap)),
//     m' = max(f + m, i),   a = exp(f + m - m'),   b = exp(i - m'),
//     S <- a S + b k v^T,   n <- a n + b k,   o = S^T q / (max(|n . q|, exp(-m')) + floor).
// The columns of S (one per value) do not depend on each other, and n is one more such column whose value is
// always 1: a block takes one sequence, one head and SC_PT values, and walks the sequence's tokens in order, as
// the recurrence above does.  Thread (pair of columns, r) keeps entries d = r * NI .. of its two columns and of n in
// registers; the 16 threads of a pair add their parts of S^T q and n . q with cross-lane additions inside their
// row of 16 lanes.  Every block of a head keeps n and m for itself (a block never reads what another writes in
// the same launch).  State layouts: S [slot, H, dv, dk] (a column's dk entries side by side), n [slot, H, tiles, dk],
// m [slot, H, tiles], tiles = ceil(dv / SC_PT); all zero when a sequence starts.  A step of one token per sequence
// and a step of a prompt run the same arithmetic per token.
__device__ __forceinline__ float rc_logsigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// VEC (rows of the projection, the columns' first numbers and the sizes are multiples of 4 numbers): a chunk's
// operands are asked for as 16-byte pieces, all at once, while the chunk before it is worked on, and reach LDS when
// that is done.  U tokens are worked on at a time: their operands are all read from LDS first and their sums across
// lanes run side by side; the gates' recurrence (m, and the two factors of every token) runs ahead of them in
// every thread; the quotients are formed for the whole chunk afterwards, by all threads at once.  A token past the chunk's end has keys of zero, a forget gate of one and an input gate of zero
// (log gates 0 and -infinity): it leaves S, n and m as they are, bit for bit.
template <int NI, bool VEC>
__global__ void __launch_bounds__(RC_BLOCK)
mlstm_scan_kernel(const float* __restrict__ proj, int ld, int q_col0, int k_col0, int v_col0, int i_col0, int f_col0,
                  const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, float q_scale, float floor_,
                  float* __restrict__ s_state, float* __restrict__ n_state, float* __restrict__ m_state,
                  const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots, float* __restrict__ out,
                  int n_heads, int dk, int dv, int tiles) {
    extern __shared__ float4 ml_smem4[];
    constexpr int NP = SC_R * NI;              // padded length of a q or k row
    constexpr int TC = NI <= 8 ? 32 : 16;      // tokens of a chunk
    constexpr int U = NI <= 8 ? 4 : 2;         // tokens worked on at a time
    float* ks = (float*)ml_smem4;              // [TC][NP]
    float* qs = ks + TC * NP;                  // [TC][NP]
    float* vs = qs + TC * NP;                  // [TC][SC_PT]
    float* os = vs + TC * SC_PT;               // [TC][SC_PT]
    float* gs = os + TC * SC_PT;               // [TC][2]: log input gate, log forget gate
    float* dn = gs + 2 * TC;                   // [TC][2]: n . q and m after the token, for the quotient
    int tile = blockIdx.x, p0 = tile * SC_PT, head = blockIdx.y, b = blockIdx.z;
    int tid = threadIdx.x, r = tid % SC_R, pl = tid / SC_R;
    int first = cu_seqlens[b], n_tok = cu_seqlens[b + 1] - first;
    size_t slot_head = (size_t)seq_slots[b] * n_heads + head;
    float* st_head = s_state + slot_head * dv * dk;
    float* n_mine = n_state + (slot_head * tiles + tile) * dk;
    float s[SC_PP][NI], nn[NI];
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        sc_load_state<NI>(s[j], st_head + (size_t)min(p, dv - 1) * dk, r, dk, p < dv);
    }
    sc_load_state<NI>(nn, n_mine, r, dk, true);
    float m = m_state[slot_head * tiles + tile];
    float bi = i_bias ? i_bias[head] : 0.f, bf = f_bias ? f_bias[head] : 0.f;
    constexpr int PF = VEC ? (TC * NP / 4 + RC_BLOCK - 1) / RC_BLOCK : 1;
    sc_f4 pre_k[PF], pre_q[PF], pre_v;
    float pre_i = 0.f, pre_f = 0.f;
    const sc_f4 zero4 = {0.f, 0.f, 0.f, 0.f};
    pre_v = zero4;
#define ML_PREFETCH(c0_)                                                                                         \
    {                                                                                                            \
        int nt_ = min(TC, n_tok - (c0_));                                                                        \
        _Pragma("unroll") for (int j = 0; j < PF; ++j) {                                                         \
            int i4 = tid + j * RC_BLOCK, tt = i4 / (NP / 4), d = (i4 - tt * (NP / 4)) * 4;                       \
            bool ok = tt < nt_ && d < dk;                                                                        \
            const float* row = proj + (size_t)(first + (c0_) + (ok ? tt : 0)) * ld + (size_t)head * dk + (ok ? d : 0); \
            pre_k[j] = ok ? *(const sc_f4*)(row + k_col0) : zero4;                                              \
            pre_q[j] = ok ? *(const sc_f4*)(row + q_col0) : zero4;                                              \
        }                                                                                                        \
        {                                                                                                        \
            int tt = tid / (SC_PT / 4), pp = (tid - tt * (SC_PT / 4)) * 4;                                       \
            bool ok = tt < nt_ && p0 + pp < dv;                                                                  \
            pre_v = ok ? *(const sc_f4*)(proj + (size_t)(first + (c0_) + tt) * ld + v_col0 + (size_t)head * dv + p0 + pp) : zero4; \
        }                                                                                                        \
        if (tid < nt_) {                                                                                         \
            const float* row = proj + (size_t)(first + (c0_) + tid) * ld;                                        \
            pre_i = row[i_col0 + head];                                                                          \
            pre_f = row[f_col0 + head];                                                                          \
        }                                                                                                        \
    }
    if (VEC && n_tok > 0) ML_PREFETCH(0)
    for (int c0 = 0; c0 < n_tok; c0 += TC) {
        int nt = min(TC, n_tok - c0);
        int nt_up = (nt + U - 1) / U * U;
        __syncthreads();                          // the previous chunk's outputs have been written out
        if (VEC) {
#pragma unroll
            for (int j = 0; j < PF; ++j) {
                int i4 = tid + j * RC_BLOCK;
                if (i4 < TC * (NP / 4)) {
                    ((sc_f4*)ks)[i4] = pre_k[j];
                    ((sc_f4*)qs)[i4] = pre_q[j] * q_scale;
                }
            }
            if (tid < TC * (SC_PT / 4)) ((sc_f4*)vs)[tid] = pre_v;
            if (tid < TC) {
                gs[2 * tid] = tid < nt ? cap * tanhf((pre_i + bi) / cap) : -INFINITY;
                gs[2 * tid + 1] = tid < nt ? rc_logsigmoid(cap * tanhf((pre_f + bf) / cap)) : 0.f;
            }
            __syncthreads();
            if (c0 + TC < n_tok) ML_PREFETCH(c0 + TC)
        } else {
            for (int i = tid; i < nt_up * NP; i += RC_BLOCK) {
                int tt = i / NP, d = i - tt * NP;
                bool ok = tt < nt && d < dk;
                const float* row = proj + (size_t)(first + c0 + (ok ? tt : 0)) * ld + (size_t)head * dk + (ok ? d : 0);
                ks[i] = ok ? row[k_col0] : 0.f;
                qs[i] = ok ? row[q_col0] * q_scale : 0.f;
            }
            for (int i = tid; i < nt_up * SC_PT; i += RC_BLOCK) {
                int tt = i / SC_PT, pp = i - tt * SC_PT;
                vs[i] = (tt < nt && p0 + pp < dv) ? proj[(size_t)(first + c0 + tt) * ld + v_col0 + (size_t)head * dv + p0 + pp] : 0.f;
            }
            if (tid < nt_up) {
                const float* row = proj + (size_t)(first + c0 + min(tid, nt - 1)) * ld;
                gs[2 * tid] = tid < nt ? cap * tanhf((row[i_col0 + head] + bi) / cap) : -INFINITY;
                gs[2 * tid + 1] = tid < nt ? rc_logsigmoid(cap * tanhf((row[f_col0 + head] + bf) / cap)) : 0.f;
            }
            __syncthreads();
        }
        for (int t0 = 0; t0 < nt; t0 += U) {
            float2 xv[U];
            float kv[U][NI], qv[U][NI], fa[U], fb[U], mt[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                int tt = t0 + u;
                float2 g = *(const float2*)(gs + 2 * tt);
                // m' = max(f + m, i); of the two factors e^(f + m - m') and e^(i - m') one is e^0 and the other e^(-|i - (f + m)|)
                float fm = g.y + m, d = g.x - fm, e = expf(-fabsf(d));
                fa[u] = d > 0.f ? e : 1.f;
                fb[u] = d > 0.f ? 1.f : e;
                m = fmaxf(fm, g.x);
                mt[u] = m;
                xv[u] = *(const float2*)(vs + tt * SC_PT + pl * SC_PP);
                const float* kt = ks + tt * NP + r * NI;
                const float* qt = qs + tt * NP + r * NI;
                if (NI % 4 == 0) {
#pragma unroll
                    for (int i = 0; i < NI; i += 4) {
                        float4 k4 = *(const float4*)(kt + i), q4 = *(const float4*)(qt + i);
                        kv[u][i] = k4.x; kv[u][i + 1] = k4.y; kv[u][i + 2] = k4.z; kv[u][i + 3] = k4.w;
                        qv[u][i] = q4.x; qv[u][i + 1] = q4.y; qv[u][i + 2] = q4.z; qv[u][i + 3] = q4.w;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NI; ++i) { kv[u][i] = kt[i]; qv[u][i] = qt[i]; }
                }
            }
            float part0[U], part1[U], partn[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float a = fa[u], bb = fb[u], bv0 = bb * xv[u].x, bv1 = bb * xv[u].y, q0 = 0.f, q1 = 0.f, nq = 0.f;
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    s[0][i] = fmaf(a, s[0][i], bv0 * kv[u][i]);
                    s[1][i] = fmaf(a, s[1][i], bv1 * kv[u][i]);
                    nn[i] = fmaf(a, nn[i], bb * kv[u][i]);
                    q0 = fmaf(s[0][i], qv[u][i], q0);
                    q1 = fmaf(s[1][i], qv[u][i], q1);
                    nq = fmaf(nn[i], qv[u][i], nq);
                }
                part0[u] = q0;
                part1[u] = q1;
                partn[u] = nq;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                part0[u] = row16_sum(part0[u]);
                part1[u] = row16_sum(part1[u]);
                partn[u] = row16_sum(partn[u]);
            }
            if (r == 0) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    *(float2*)(os + (t0 + u) * SC_PT + pl * SC_PP) = make_float2(part0[u], part1[u]);
                    if (tid == 0) *(float2*)(dn + 2 * (t0 + u)) = make_float2(partn[u], mt[u]);
                }
            }
        }
        __syncthreads();
        // the quotients, all threads at once: S^T q / (max(|n . q|, e^(-m)) + floor)
        for (int i = tid; i < nt * SC_PT; i += RC_BLOCK) {
            int tt = i / SC_PT, pp = i - tt * SC_PT;
            float2 nm = *(const float2*)(dn + 2 * tt);
            float den = fmaxf(fabsf(nm.x), expf(-nm.y)) + floor_;
            if (p0 + pp < dv) out[(size_t)(first + c0 + tt) * n_heads * dv + (size_t)head * dv + p0 + pp] = os[i] / den;
        }
    }
#undef ML_PREFETCH
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        sc_store_state<NI>(s[j], st_head + (size_t)min(p, dv - 1) * dk, r, dk, p < dv);
    }
    if (pl == 0) sc_store_state<NI>(nn, n_mine, r, dk, true);
    if (tid == 0) m_state[slot_head * tiles + tile] = m;
}

// A step of one token per sequence: the same arithmetic for that token without the chunks: a thread reads its
// entries of k and q and its two values of v straight from memory, next to its state entries, and nothing waits at
// a barrier.  Token b is sequence b's.
template <int NI>
__global__ void __launch_bounds__(RC_BLOCK)
mlstm_step_kernel(const float* __restrict__ proj, int ld, int q_col0, int k_col0, int v_col0, int i_col0, int f_col0,
                  const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, float q_scale, float floor_,
                  float* __restrict__ s_state, float* __restrict__ n_state, float* __restrict__ m_state,
                  const int* __restrict__ seq_slots, float* __restrict__ out, int n_heads, int dk, int dv, int tiles,
                  int vec_rows) {
    int tile = blockIdx.x, p0 = tile * SC_PT, head = blockIdx.y, b = blockIdx.z;
    int tid = threadIdx.x, r = tid % SC_R, pl = tid / SC_R;
    size_t slot_head = (size_t)seq_slots[b] * n_heads + head;
    float* st_head = s_state + slot_head * dv * dk;
    float* n_mine = n_state + (slot_head * tiles + tile) * dk;
    const float* row = proj + (size_t)b * ld;
    const float* krow = row + k_col0 + (size_t)head * dk;
    const float* qrow = row + q_col0 + (size_t)head * dk;
    float s[SC_PP][NI], nn[NI], kv[NI], qv[NI];
    // (k and q are read like a column of the state; their rows start on 16 bytes where the vector form is taken:
    // the caller checks the strides)
    sc_load_state<NI>(kv, krow, r, vec_rows ? dk : -1, true);
    sc_load_state<NI>(qv, qrow, r, vec_rows ? dk : -1, true);
    if (!vec_rows) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            int d = r * NI + i;
            bool ok = d < dk;
            kv[i] = ok ? krow[d] : 0.f;
            qv[i] = ok ? qrow[d] : 0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) qv[i] *= q_scale;
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        sc_load_state<NI>(s[j], st_head + (size_t)min(p, dv - 1) * dk, r, dk, p < dv);
    }
    sc_load_state<NI>(nn, n_mine, r, dk, true);
    float m = m_state[slot_head * tiles + tile];
    float xv[SC_PP];
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        xv[j] = p < dv ? row[v_col0 + (size_t)head * dv + p] : 0.f;
    }
    float gi = cap * tanhf((row[i_col0 + head] + (i_bias ? i_bias[head] : 0.f)) / cap);
    float gf = rc_logsigmoid(cap * tanhf((row[f_col0 + head] + (f_bias ? f_bias[head] : 0.f)) / cap));
    float fm = gf + m, d = gi - fm, e = expf(-fabsf(d));
    float a = d > 0.f ? e : 1.f, bb = d > 0.f ? 1.f : e;
    m = fmaxf(fm, gi);
    float em = expf(-m);
    float bv0 = bb * xv[0], bv1 = bb * xv[1], q0 = 0.f, q1 = 0.f, nq = 0.f;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        s[0][i] = fmaf(a, s[0][i], bv0 * kv[i]);
        s[1][i] = fmaf(a, s[1][i], bv1 * kv[i]);
        nn[i] = fmaf(a, nn[i], bb * kv[i]);
        q0 = fmaf(s[0][i], qv[i], q0);
        q1 = fmaf(s[1][i], qv[i], q1);
        nq = fmaf(nn[i], qv[i], nq);
    }
    q0 = row16_sum(q0);
    q1 = row16_sum(q1);
    nq = row16_sum(nq);
    float den = fmaxf(fabsf(nq), em) + floor_;
#pragma unroll
    for (int j = 0; j < SC_PP; ++j) {
        int p = p0 + pl * SC_PP + j;
        if (p >= dv) continue;
        if (r == 0) out[(size_t)b * n_heads * dv + (size_t)head * dv + p] = (j == 0 ? q0 : q1) / den;
        sc_store_state<NI>(s[j], st_head + (size_t)p * dk, r, dk, true);
    }
    if (pl == 0) sc_store_state<NI>(nn, n_mine, r, dk, true);
    if (tid == 0) m_state[slot_head * tiles + tile] = m;
}

ROCML_EXPORT int rocml_mlstm_tile() { return SC_PT; }

ROCML_EXPORT int rocml_mlstm_scan(const float* proj, int ld, int q_col0, int k_col0, int v_col0, int i_col0, int f_col0,
                                  const float* i_bias, const float* f_bias, float cap, float q_scale, float floor_,
                                  float* s_state, float* n_state, float* m_state, int n_slots, const int* cu_seqlens,
                                  const int* seq_slots, int n_seqs, int n_tokens, float* out, int n_heads, int dk, int dv,
                                  hipStream_t stream) {
    ROCML_REQUIRE(n_heads > 0 && dk > 0 && dv > 0 && cap > 0.f, "mlstm_scan: bad sizes heads=%d dk=%d dv=%d cap=%g", n_heads,
                  dk, dv, (double)cap);
    ROCML_REQUIRE(dk <= 16 * SC_R, "mlstm_scan: a key size of %d exceeds %d", dk, 16 * SC_R);
    ROCML_REQUIRE(q_col0 >= 0 && k_col0 >= 0 && v_col0 >= 0 && i_col0 >= 0 && f_col0 >= 0 && ld >= q_col0 + n_heads * dk &&
                      ld >= k_col0 + n_heads * dk && ld >= v_col0 + n_heads * dv && ld >= i_col0 + n_heads && ld >= f_col0 + n_heads,
                  "mlstm_scan: rows of %d are too short for their columns", ld);
    ROCML_REQUIRE(proj && s_state && n_state && m_state && cu_seqlens && seq_slots && out && n_slots > 0,
                  "mlstm_scan: missing arguments");
    ROCML_REQUIRE(n_seqs >= 0 && n_seqs < 65536 && n_heads < 65536, "mlstm_scan: too many sequences or heads for one launch");
    if (n_seqs == 0 || n_tokens == 0) return 0;
    int tiles = ceil_div(dv, SC_PT);
    dim3 grid(tiles, n_heads, n_seqs);
    int ni = ceil_div(dk, SC_R);
    ni = ni <= 4 ? ni : ni <= 6 ? 6 : ni <= 8 ? 8 : ni <= 12 ? 12 : 16;
    if (n_tokens == n_seqs) {          // one token per sequence (every sequence of a step brings at least one)
        // k and q rows as 16-byte pieces: every row and every head's part starts on a multiple of 4 numbers
        int vec_rows = ld % 4 == 0 && dk % 4 == 0 && q_col0 % 4 == 0 && k_col0 % 4 == 0 && ((uintptr_t)proj & 15) == 0;
#define MSTEP(NI_)                                                                                                     \
    mlstm_step_kernel<NI_><<<grid, RC_BLOCK, 0, stream>>>(proj, ld, q_col0, k_col0, v_col0, i_col0, f_col0, i_bias, f_bias, cap, \
                                                          q_scale, floor_, s_state, n_state, m_state, seq_slots, out, n_heads, dk, \
                                                          dv, tiles, vec_rows)
        switch (ni) {
            case 1: MSTEP(1); break;
            case 2: MSTEP(2); break;
            case 3: MSTEP(3); break;
            case 4: MSTEP(4); break;
            case 6: MSTEP(6); break;
            case 8: MSTEP(8); break;
            case 12: MSTEP(12); break;
            default: MSTEP(16); break;
        }
#undef MSTEP
        ROCML_CHECK_LAUNCH("mlstm_scan step");
        return 0;
    }
    int tc = ni <= 8 ? 32 : 16;
    size_t lds = (size_t)(2 * tc * SC_R * ni + 2 * tc * SC_PT + 4 * tc) * sizeof(float);
    // whole 16-byte pieces: every row of q, k and v starts on a multiple of 4 numbers and ends on one
    bool vec = ld % 4 == 0 && dk % 4 == 0 && dv % 4 == 0 && q_col0 % 4 == 0 && k_col0 % 4 == 0 && v_col0 % 4 == 0 &&
               ((uintptr_t)proj & 15) == 0;
#define MSCAN(NI_)                                                                                                     \
    {                                                                                                                  \
        if (vec)                                                                                                       \
            mlstm_scan_kernel<NI_, true><<<grid, RC_BLOCK, lds, stream>>>(proj, ld, q_col0, k_col0, v_col0, i_col0, f_col0, i_bias, \
                                                                          f_bias, cap, q_scale, floor_, s_state, n_state, m_state, \
                                                                          cu_seqlens, seq_slots, out, n_heads, dk, dv, tiles);  \
        else                                                                                                           \
            mlstm_scan_kernel<NI_, false><<<grid, RC_BLOCK, lds, stream>>>(proj, ld, q_col0, k_col0, v_col0, i_col0, f_col0, i_bias, \
                                                                           f_bias, cap, q_scale, floor_, s_state, n_state, m_state, \
                                                                           cu_seqlens, seq_slots, out, n_heads, dk, dv, tiles); \
    }
    switch (ni) {
        case 1: MSCAN(1); break;
        case 2: MSCAN(2); break;
        case 3: MSCAN(3); break;
        case 4: MSCAN(4); break;
        case 6: MSCAN(6); break;
        case 8: MSCAN(8); break;
        case 12: MSCAN(12); break;
        default: MSCAN(16); break;
    }
#undef MSCAN
    ROCML_CHECK_LAUNCH("mlstm_scan");
    return 0;
}

// ---- norm of every head, gain, output gate ---------------------------------------------
// out[t, h * dv + j] = o / sqrt(mean over the head's dv values of o^2 + eps) * gain[h * dv + j] * sigmoid(g[t, g_col0 + h * dv + j]):
// o [T, H * dv] and g (rows of ldg numbers) 32-bit, the statistics 32-bit; a wave per (token, head).
template <typename TO>
__global__ void __launch_bounds__(RC_BLOCK)
head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ g, int ldg, int g_col0,
                      const float* __restrict__ gain, TO* __restrict__ out, long long n_rows, int n_heads, int dv, float eps, int silu) {
    int lane = threadIdx.x & (WAVE - 1);
    long long row = (long long)blockIdx.x * (RC_BLOCK / WAVE) + threadIdx.x / WAVE;
    if (row >= n_rows) return;
    long long t = row / n_heads;
    int h = (int)(row - t * n_heads);
    const float* src = o + (size_t)row * dv;
    float ss = 0.f;
    for (int j = lane; j < dv; j += WAVE) ss = fmaf(src[j], src[j], ss);
    float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
    const float* gr = g + (size_t)t * ldg + g_col0 + (size_t)h * dv;
    for (int j = lane; j < dv; j += WAVE) {
        float gate = 1.0f / (1.0f + expf(-gr[j]));
        if (silu) gate *= gr[j];
        Elem<TO>::store(out + (size_t)row * dv + j, src[j] * inv * (gain ? gain[(size_t)h * dv + j] : 1.0f) * gate);
    }
}

__device__ __forceinline__ void rc_store4(float* p, float a, float b, float c, float d) { *(sc_f4*)p = sc_f4{a, b, c, d}; }
__device__ __forceinline__ void rc_store4(bf16_t* p, float a, float b, float c, float d) {
    uint2 v;
    v.x = f32x2_to_bf16x2(a, b);
    v.y = f32x2_to_bf16x2(c, d);
    *(uint2*)p = v;
}

// Heads of up to 512 values that are multiples of 4, rows that start on 16 bytes: the head stays in registers as
// 16-byte pieces between the sum and the product, and gate and gain are read the same way.
template <typename TO>
__global__ void __launch_bounds__(RC_BLOCK)
head_norm_gate_vec_kernel(const float* __restrict__ o, const float* __restrict__ g, int ldg, int g_col0,
                          const float* __restrict__ gain, TO* __restrict__ out, long long n_rows, int n_heads, int dv, float eps, int silu) {
    int lane = threadIdx.x & (WAVE - 1);
    long long row = (long long)blockIdx.x * (RC_BLOCK / WAVE) + threadIdx.x / WAVE;
    if (row >= n_rows) return;
    long long t = row / n_heads;
    int h = (int)(row - t * n_heads);
    int nv = dv / 4;
    const sc_f4* src = (const sc_f4*)(o + (size_t)row * dv);
    const sc_f4* gr = (const sc_f4*)(g + (size_t)t * ldg + g_col0 + (size_t)h * dv);
    const sc_f4* wr = gain ? (const sc_f4*)(gain + (size_t)h * dv) : nullptr;
    const sc_f4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const sc_f4 one4 = {1.f, 1.f, 1.f, 1.f};
    sc_f4 v[2], z[2], w[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        int c = lane + k * WAVE;
        bool ok = c < nv;
        v[k] = ok ? src[c] : zero4;
        z[k] = ok ? gr[c] : zero4;
        w[k] = (ok && wr) ? wr[c] : one4;
    }
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        ss = fmaf(v[k].x, v[k].x, ss); ss = fmaf(v[k].y, v[k].y, ss);
        ss = fmaf(v[k].z, v[k].z, ss); ss = fmaf(v[k].w, v[k].w, ss);
    }
    float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        int c = lane + k * WAVE;
        if (c >= nv) continue;
        TO* dst = out + (size_t)row * dv + 4 * (size_t)c;
        // (the gate: sigmoid(z), or z sigmoid(z))
        float g0 = 1.0f / (1.0f + expf(-z[k].x)), g1 = 1.0f / (1.0f + expf(-z[k].y));
        float g2 = 1.0f / (1.0f + expf(-z[k].z)), g3 = 1.0f / (1.0f + expf(-z[k].w));
        if (silu) { g0 *= z[k].x; g1 *= z[k].y; g2 *= z[k].z; g3 *= z[k].w; }
        float r0 = v[k].x * inv * w[k].x * g0;
        float r1 = v[k].y * inv * w[k].y * g1;
        float r2 = v[k].z * inv * w[k].z * g2;
        float r3 = v[k].w * inv * w[k].w * g3;
        rc_store4(dst, r0, r1, r2, r3);
    }
}

// Heads of at most 128 values (multiples of 4): G lanes a head, a 16-byte piece a lane, 64 / G heads a wave, the sum of
// squares across the G lanes; a wave per head would leave most of its lanes idle there.
template <typename TO, int G>
__global__ void __launch_bounds__(RC_BLOCK)
head_norm_gate_pack_kernel(const float* __restrict__ o, const float* __restrict__ g, int ldg, int g_col0,
                           const float* __restrict__ gain, TO* __restrict__ out, long long n_rows, int n_heads, int dv, float eps, int silu) {
    long long row = ((long long)blockIdx.x * RC_BLOCK + threadIdx.x) / G;
    int c = threadIdx.x % G;
    bool ok = row < n_rows && 4 * c < dv;
    long long t = ok ? row / n_heads : 0;
    int h = ok ? (int)(row - t * n_heads) : 0;
    const sc_f4 zero4 = {0.f, 0.f, 0.f, 0.f};
    const sc_f4 one4 = {1.f, 1.f, 1.f, 1.f};
    sc_f4 v = ok ? *(const sc_f4*)(o + (size_t)row * dv + 4 * c) : zero4;
    sc_f4 z = ok ? *(const sc_f4*)(g + (size_t)t * ldg + g_col0 + (size_t)h * dv + 4 * c) : zero4;
    sc_f4 w = (ok && gain) ? *(const sc_f4*)(gain + (size_t)h * dv + 4 * c) : one4;
    float ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, v.w * v.w)));
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    float inv = 1.0f / sqrtf(ss / (float)dv + eps);
    if (!ok) return;
    float g0 = 1.0f / (1.0f + expf(-z.x)), g1 = 1.0f / (1.0f + expf(-z.y));
    float g2 = 1.0f / (1.0f + expf(-z.z)), g3 = 1.0f / (1.0f + expf(-z.w));
    if (silu) { g0 *= z.x; g1 *= z.y; g2 *= z.z; g3 *= z.w; }
    rc_store4(out + (size_t)row * dv + 4 * c, v.x * inv * w.x * g0, v.y * inv * w.y * g1, v.z * inv * w.z * g2, v.w * inv * w.w * g3);
}

template <typename TO>
static void launch_head_norm_gate_pack(const float* o, const float* g, int ldg, int g_col0, const float* gain, TO* out, long long rows,
                                       int n_heads, int dv, float eps, int silu, hipStream_t stream) {
    int lanes = dv / 4 <= 4 ? 4 : dv / 4 <= 8 ? 8 : dv / 4 <= 16 ? 16 : 32;
    int grid = ceil_div(rows * lanes, RC_BLOCK);
    if (lanes == 4) head_norm_gate_pack_kernel<TO, 4><<<grid, RC_BLOCK, 0, stream>>>(o, g, ldg, g_col0, gain, out, rows, n_heads, dv, eps, silu);
    else if (lanes == 8) head_norm_gate_pack_kernel<TO, 8><<<grid, RC_BLOCK, 0, stream>>>(o, g, ldg, g_col0, gain, out, rows, n_heads, dv, eps, silu);
    else if (lanes == 16) head_norm_gate_pack_kernel<TO, 16><<<grid, RC_BLOCK, 0, stream>>>(o, g, ldg, g_col0, gain, out, rows, n_heads, dv, eps, silu);
    else head_norm_gate_pack_kernel<TO, 32><<<grid, RC_BLOCK, 0, stream>>>(o, g, ldg, g_col0, gain, out, rows, n_heads, dv, eps, silu);
}

// gate_act: 0 the gate is sigmoid(g), 1 it is silu(g) = g sigmoid(g).  gain may be null (ones).
ROCML_EXPORT int rocml_head_norm_gate(const float* o, const float* g, int ldg, int g_col0, const float* gain, void* out,
                                      int out_dtype, int n_tokens, int n_heads, int dv, float eps, int gate_act, hipStream_t stream) {
    ROCML_REQUIRE(gate_act == 0 || gate_act == 1, "head_norm_gate: unknown gate activation %d", gate_act);
    ROCML_REQUIRE(n_tokens >= 0 && n_heads > 0 && dv > 0 && g_col0 >= 0 && ldg >= g_col0 + n_heads * dv && o && g && out,
                  "head_norm_gate: bad arguments T=%d heads=%d dv=%d ld=%d", n_tokens, n_heads, dv, ldg);
    long long rows = (long long)n_tokens * n_heads;
    if (rows == 0) return 0;
    int grid = ceil_div(rows, RC_BLOCK / WAVE);
    bool vec = dv % 4 == 0 && dv <= 8 * WAVE && ldg % 4 == 0 && g_col0 % 4 == 0 && (uintptr_t)o % 16 == 0 && (uintptr_t)g % 16 == 0 &&
               (uintptr_t)gain % 16 == 0 && (uintptr_t)out % 16 == 0;
    if (vec && dv <= 128 && out_dtype == ROCML_F32)
        launch_head_norm_gate_pack<float>(o, g, ldg, g_col0, gain, (float*)out, rows, n_heads, dv, eps, gate_act, stream);
    else if (vec && dv <= 128 && out_dtype == ROCML_BF16)
        launch_head_norm_gate_pack<bf16_t>(o, g, ldg, g_col0, gain, (bf16_t*)out, rows, n_heads, dv, eps, gate_act, stream);
    else if (vec && out_dtype == ROCML_F32)
        head_norm_gate_vec_kernel<float><<<grid, RC_BLOCK, 0, stream>>>(o, g, ldg, g_col0, gain, (float*)out, rows, n_heads, dv, eps, gate_act);
    else if (vec && out_dtype == ROCML_BF16)
        head_norm_gate_vec_kernel<bf16_t><<<grid, RC_BLOCK, 0, stream>>>(o, g, ldg, g_col0, gain, (bf16_t*)out, rows, n_heads, dv, eps, gate_act);
    else if (out_dtype == ROCML_F32)
        head_norm_gate_kernel<float><<<grid, RC_BLOCK, 0, stream>>>(o, g, ldg, g_col0, gain, (float*)out, rows, n_heads, dv, eps, gate_act);
    else if (out_dtype == ROCML_BF16)
        head_norm_gate_kernel<bf16_t><<<grid, RC_BLOCK, 0, stream>>>(o, g, ldg, g_col0, gain, (bf16_t*)out, rows, n_heads, dv, eps, gate_act);
    else return rocml_fail("head_norm_gate: unknown dtype code %d", out_dtype);
    ROCML_CHECK_LAUNCH("head_norm_gate");
    return 0;
}

// ---- gated norm in equal parts ------------------------------------------------------
// out[t, i] = v / sqrt(mean over i's part of v^2 + eps) * gain[i],  v = y[t, i] * silu(z[t, i]):
// the gate comes before the norm, and each of the `parts` equal parts of a row has a root mean
// square of its own.  z is 32-bit in rows of ldz numbers starting at column z_col0.
__device__ __forceinline__ float rc_block_sum(float v, float* scratch) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < RC_BLOCK / WAVE; ++w) total += scratch[w];
    return total;
}

template <typename TO>
__global__ void __launch_bounds__(RC_BLOCK)
gated_part_norm_kernel(const float* __restrict__ y, const float* __restrict__ z, int ldz, int z_col0,
                       const float* __restrict__ gain, TO* __restrict__ out, int n, int parts, float eps) {
    __shared__ float scratch[RC_BLOCK / WAVE];
    int t = blockIdx.x, part = blockIdx.y;
    int width = n / parts, i0 = part * width;
    const float* yr = y + (size_t)t * n + i0;
    const float* zr = z + (size_t)t * ldz + z_col0 + i0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += RC_BLOCK) {
        float v = yr[i] * rc_silu(zr[i]);
        ss = fmaf(v, v, ss);
    }
    float inv = 1.0f / sqrtf(rc_block_sum(ss, scratch) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += RC_BLOCK) {
        float v = yr[i] * rc_silu(zr[i]);
        Elem<TO>::store(out + (size_t)t * n + i0 + i, v * inv * gain[i0 + i]);
    }
}

// Parts of up to 2048 values that are multiples of 4: a wave takes a part (the waves of a token's block take
// its parts in turn), keeps it in registers as 16-byte pieces and sums without a barrier.
constexpr int GP_MAX_VEC = 8;

template <typename TO, int VEC>
__global__ void __launch_bounds__(RC_BLOCK)
gated_part_norm_vec_kernel(const float* __restrict__ y, const float* __restrict__ z, int ldz, int z_col0,
                           const float* __restrict__ gain, TO* __restrict__ out, int n, int parts, float eps) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    int t = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
    int width = n / parts, w4 = width / 4;
    for (int part = blockIdx.y * (RC_BLOCK / WAVE) + wave; part < parts; part += gridDim.y * (RC_BLOCK / WAVE)) {
        int i0 = part * width;
        const float* yr = y + (size_t)t * n + i0;
        const float* zr = z + (size_t)t * ldz + z_col0 + i0;
        f4 v[VEC], g[VEC];
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            int i = lane + j * WAVE;
            bool ok = i < w4;
            f4 yy = ok ? ((const f4*)yr)[i] : f4{0.f, 0.f, 0.f, 0.f};
            f4 zz = ok ? ((const f4*)zr)[i] : f4{0.f, 0.f, 0.f, 0.f};
            g[j] = ok ? ((const f4*)(gain + i0))[i] : f4{0.f, 0.f, 0.f, 0.f};
            v[j].x = yy.x * rc_silu(zz.x); v[j].y = yy.y * rc_silu(zz.y);
            v[j].z = yy.z * rc_silu(zz.z); v[j].w = yy.w * rc_silu(zz.w);
            ss = fmaf(v[j].x, v[j].x, ss); ss = fmaf(v[j].y, v[j].y, ss);
            ss = fmaf(v[j].z, v[j].z, ss); ss = fmaf(v[j].w, v[j].w, ss);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
        float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            int i = lane + j * WAVE;
            if (i >= w4) continue;
            TO* o = out + (size_t)t * n + i0 + 4 * i;
            Elem<TO>::store(o, v[j].x * inv * g[j].x);
            Elem<TO>::store(o + 1, v[j].y * inv * g[j].y);
            Elem<TO>::store(o + 2, v[j].z * inv * g[j].z);
            Elem<TO>::store(o + 3, v[j].w * inv * g[j].w);
        }
    }
}

ROCML_EXPORT int rocml_gated_part_norm(const float* y, const float* z, int ldz, int z_col0, const float* gain, void* out,
                                       int out_dtype, int n_rows, int n, int parts, float eps, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n > 0 && parts > 0 && n % parts == 0, "gated_part_norm: %d values do not fall into %d equal parts", n,
                  parts);
    ROCML_REQUIRE(z_col0 >= 0 && ldz >= z_col0 + n, "gated_part_norm: gate rows of %d are too short", ldz);
    ROCML_REQUIRE(parts < 65536, "gated_part_norm: too many parts");
    if (n_rows == 0) return 0;
    ROCML_REQUIRE(out_dtype == ROCML_F32 || out_dtype == ROCML_BF16, "gated_part_norm: unknown dtype code %d", out_dtype);
    int width = n / parts;
    if (width % 4 == 0 && width <= 4 * WAVE * GP_MAX_VEC && ldz % 4 == 0 && z_col0 % 4 == 0 &&
        (((uintptr_t)y | (uintptr_t)z | (uintptr_t)gain) & 15) == 0) {
        int vec = ceil_div(width / 4, WAVE);
        dim3 vgrid(n_rows, min(ceil_div(parts, RC_BLOCK / WAVE), 1024));
#define GPV(TO_, V_) gated_part_norm_vec_kernel<TO_, V_><<<vgrid, RC_BLOCK, 0, stream>>>(y, z, ldz, z_col0, gain, (TO_*)out, n, parts, eps)
#define GPV_BY_VEC(TO_) { if (vec <= 1) GPV(TO_, 1); else if (vec <= 2) GPV(TO_, 2); else if (vec <= 4) GPV(TO_, 4); else GPV(TO_, 8); }
        if (out_dtype == ROCML_F32) GPV_BY_VEC(float)
        else GPV_BY_VEC(bf16_t)
#undef GPV_BY_VEC
#undef GPV
        ROCML_CHECK_LAUNCH("gated_part_norm");
        return 0;
    }
    dim3 grid(n_rows, parts);
    if (out_dtype == ROCML_F32)
        gated_part_norm_kernel<float><<<grid, RC_BLOCK, 0, stream>>>(y, z, ldz, z_col0, gain, (float*)out, n, parts, eps);
    else if (out_dtype == ROCML_BF16)
        gated_part_norm_kernel<bf16_t><<<grid, RC_BLOCK, 0, stream>>>(y, z, ldz, z_col0, gain, (bf16_t*)out, n, parts, eps);
    else return rocml_fail("gated_part_norm: unknown dtype code %d", out_dtype);
    ROCML_CHECK_LAUNCH("gated_part_norm");
    return 0;
}

// ---- recurrences with a decay per key channel ---------------------------------------------
// Per head a state S [dk, dv] that starts at zero, decays row by row and takes the outer product of the
// token's key and value: S <- diag(w_t) S + k_t v_t^T.  Two ways to read it:
//   after the update (a retention):        o_t = S_t^T q_t, with w_t one constant per head;
//   before it, with a bonus on the token:  o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t, with w_t per token and channel.
// The columns of S (one per value) do not depend on each other: a block takes (sequence, head, 16 CPL values).  The
// 16 lanes of a row of lanes hold CPL neighbouring columns, lane l the R entries l R .. l R + R - 1 of each: what a
// lane reads of q, k and the decays serves CPL columns, which is what keeps the walk off the LDS's bandwidth.  The
// tokens' rows (q, k, the decays and the block's values) come in chunks of 16 tokens through LDS: every thread owns
// up to SLOTS columns of a chunk's rows, requests the next chunk's numbers into registers before it works on this
// one, and writes them to LDS when this one is done, so the walk over the tokens waits for memory once.  Inside a
// chunk four tokens are worked on at a time: their 4 CPL partial sums per lane are added across the row of lanes so
// that every lane ends with one whole sum (halving exchanges), which it writes.  w_offset: the decays come as logits
// x and are exp(-exp(x + offset)), formed on the way into LDS.  The state is stored column by column,
// [slot, head, dv, dk].  Everything is 32-bit.
constexpr int DS_LANES = 16;     // lanes that share a column
constexpr int DS_GROUPS = 16;    // rows of lanes in a block
constexpr int DS_THREADS = DS_GROUPS * DS_LANES;
constexpr int DS_CHUNK = 16;     // tokens of a chunk (8: 4 to 7 % slower on 8 x 2,048 tokens, 32: 9 to 25 %)
constexpr int DS_TOKENS = 4;     // tokens whose sums cross the lanes together

struct DecayScanArgs {
    const float* q; int ldq; int q_col0;
    const float* k; int ldk; int k_col0;
    const float* v; int ldv; int v_col0;
    const float* w; int ldw; int w_col0;      // per token and channel, or null
    const float* w_offset;                     // [H * dk] or null: w holds logits x, the decay is exp(-exp(x + offset))
    const float* head_decay;                   // [H], or null (then w)
    const float* bonus;                        // [H * dk], or null: the state is read after its update
    float* state; const int* cu_seqlens; const int* seq_slots;
    float* out; int n_heads; int dk; int dv;
};

// R: entries of a column per lane (dk <= 16 R).  CPL: columns per lane.  BONUS: a decay per token and channel and a
// bonus, the state read before its update; else one decay per head, the state read after it.
// A token's row in LDS has a fixed layout, whatever dk: q, k (and the decays) padded to 16 R numbers each, the block's
// 16 CPL values, and without BONUS the token's decay (the head's, or one for the rows beyond the sequence's last
// token, which then leave the state as it is: with BONUS their decays are one and their keys zero).  A lane reads its
// R numbers of each part as whole vectors at fixed offsets, without a bound to check.
template <int R, int CPL, bool BONUS>
__global__ void __launch_bounds__(DS_THREADS)
decay_scan_kernel(DecayScanArgs a) {
    constexpr int ARRAYS = BONUS ? 3 : 2;
    constexpr int DKP = DS_LANES * R;
    constexpr int TILE = DS_GROUPS * CPL;                            // columns of a block
    constexpr int ROW = ARRAYS * DKP + TILE + (BONUS ? 0 : 4);
    constexpr int SLOTS = (ROW + DS_THREADS - 1) / DS_THREADS;
    constexpr int NV = DS_TOKENS * CPL;                              // sums of a lane per group of tokens
    __shared__ __attribute__((aligned(16))) float ds_rows[DS_CHUNK * ROW];
    int b = blockIdx.x, h = blockIdx.y, tile = blockIdx.z;
    int tid = threadIdx.x;
    int l = tid % DS_LANES, c = tid / DS_LANES;
    int dk = a.dk;
    int col0 = tile * TILE + c * CPL;
    int first = a.cu_seqlens[b], n = a.cu_seqlens[b + 1] - first;
    float hd = BONUS ? 0.f : a.head_decay[h];
    // the columns of a chunk's rows that this thread brings in: where they come from, per slot
    const float* src[SLOTS];
    int src_ld[SLOTS];
    float offset[SLOTS], beyond[SLOTS], fixed[SLOTS];
    bool is_logit[SLOTS];
#pragma unroll
    for (int m = 0; m < SLOTS; ++m) {
        int x = tid + m * DS_THREADS;
        src[m] = nullptr;
        src_ld[m] = 0;
        offset[m] = 0.f;
        beyond[m] = 0.f;           // what rows beyond the sequence's last token hold
        fixed[m] = 0.f;            // what a column without a source holds
        is_logit[m] = false;
        int part = x / DKP, ch = x - part * DKP;
        if (part < ARRAYS) {
            if (ch < dk) {
                size_t e = (size_t)h * dk + ch;
                if (part == 0) { src[m] = a.q + a.q_col0 + e; src_ld[m] = a.ldq; }
                else if (part == 1) { src[m] = a.k + a.k_col0 + e; src_ld[m] = a.ldk; }
                else {
                    src[m] = a.w + a.w_col0 + e;
                    src_ld[m] = a.ldw;
                    beyond[m] = 1.f;
                    if (a.w_offset) { is_logit[m] = true; offset[m] = a.w_offset[e]; }
                }
            }
        } else if (x < ARRAYS * DKP + TILE) {
            int vc = tile * TILE + (x - ARRAYS * DKP);
            if (vc < a.dv) { src[m] = a.v + a.v_col0 + (size_t)h * a.dv + vc; src_ld[m] = a.ldv; }
        } else {
            fixed[m] = hd;
            beyond[m] = 1.f;
        }
    }
    float* st = a.state + ((size_t)a.seq_slots[b] * a.n_heads + h) * a.dv * dk;
    float s[CPL][R], u[R];
    // (a lane's R entries of a column lie side by side: 16-byte pieces where the sizes allow)
    bool wide = R % 4 == 0 && dk % 4 == 0 && ((uintptr_t)a.state & 15) == 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int i = l * R + r;
        u[r] = (BONUS && i < dk) ? a.bonus[(size_t)h * dk + i] : 0.f;
    }
    if (wide) {
        if constexpr (R % 4 == 0) {
#pragma unroll
            for (int p = 0; p < CPL; ++p)
#pragma unroll
                for (int r4 = 0; r4 < R / 4; ++r4) {
                    int i = l * R + 4 * r4;
                    float4 z = {0.f, 0.f, 0.f, 0.f};
                    float4 v4 = (col0 + p < a.dv && i < dk) ? *(const float4*)(st + (size_t)(col0 + p) * dk + i) : z;
                    s[p][4 * r4] = v4.x; s[p][4 * r4 + 1] = v4.y; s[p][4 * r4 + 2] = v4.z; s[p][4 * r4 + 3] = v4.w;
                }
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int i = l * R + r;
#pragma unroll
            for (int p = 0; p < CPL; ++p) s[p][r] = (col0 + p < a.dv && i < dk) ? st[(size_t)(col0 + p) * dk + i] : 0.f;
        }
    }
    // what a token does to the lane's columns: qq, kk, ww the lane's R numbers of the token's rows, vv its columns' values
    auto token = [&](const float (&qq)[R], const float (&kk)[R], const float (&ww)[R], const float (&vv)[CPL], float dec, float* sums) {
        if constexpr (BONUS) {
            // (S + diag(u) k v^T)^T q = S^T q + v (u . k q): the second part is the same for every column
            float ukq = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r) ukq = fmaf(u[r] * kk[r], qq[r], ukq);
#pragma unroll
            for (int p = 0; p < CPL; ++p) {
                float sum = ukq * vv[p];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    sum = fmaf(s[p][r], qq[r], sum);
                    s[p][r] = fmaf(ww[r], s[p][r], kk[r] * vv[p]);
                }
                sums[p] = sum;
            }
        } else {
#pragma unroll
            for (int p = 0; p < CPL; ++p) {
                float sum = 0.f;
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    s[p][r] = fmaf(dec, s[p][r], kk[r] * vv[p]);
                    sum = fmaf(s[p][r], qq[r], sum);
                }
                sums[p] = sum;
            }
        }
    };
    auto keep_state = [&]() {
        if (wide) {
            if constexpr (R % 4 == 0) {
#pragma unroll
                for (int p = 0; p < CPL; ++p)
#pragma unroll
                    for (int r4 = 0; r4 < R / 4; ++r4) {
                        int i = l * R + 4 * r4;
                        if (col0 + p < a.dv && i < dk)
                            *(float4*)(st + (size_t)(col0 + p) * dk + i) = float4{s[p][4 * r4], s[p][4 * r4 + 1], s[p][4 * r4 + 2], s[p][4 * r4 + 3]};
                    }
            }
            return;
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int i = l * R + r;
#pragma unroll
            for (int p = 0; p < CPL; ++p)
                if (col0 + p < a.dv && i < dk) st[(size_t)(col0 + p) * dk + i] = s[p][r];
        }
    };
    if (n == 1) {
        // One token (a decode step): its numbers come straight from memory, beside the state's; the same arithmetic.
        float qq[R], kk[R], ww[R], vv[CPL], sums[CPL];
        size_t t = (size_t)first;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            int i = l * R + r;
            bool in = i < dk;
            size_t e = (size_t)h * dk + i;
            qq[r] = in ? a.q[t * a.ldq + a.q_col0 + e] : 0.f;
            kk[r] = in ? a.k[t * a.ldk + a.k_col0 + e] : 0.f;
            ww[r] = 0.f;
            if constexpr (BONUS) {
                if (in) {
                    float x = a.w[t * a.ldw + a.w_col0 + e];
                    ww[r] = a.w_offset ? expf(-expf(x + a.w_offset[e])) : x;
                }
            }
        }
#pragma unroll
        for (int p = 0; p < CPL; ++p) vv[p] = col0 + p < a.dv ? a.v[t * a.ldv + a.v_col0 + (size_t)h * a.dv + col0 + p] : 0.f;
        token(qq, kk, ww, vv, hd, sums);
#pragma unroll
        for (int p = 0; p < CPL; ++p) sums[p] = row16_sum(sums[p]);
        float out_val = sums[0];
#pragma unroll
        for (int p = 1; p < CPL; ++p) out_val = l == p ? sums[p] : out_val;
        if (l < CPL && col0 + l < a.dv) a.out[t * a.n_heads * a.dv + (size_t)h * a.dv + col0 + l] = out_val;
        keep_state();
        return;
    }
    float next[SLOTS][DS_CHUNK];
    auto request = [&](int t0) {
#pragma unroll
        for (int m = 0; m < SLOTS; ++m)
#pragma unroll
            for (int j = 0; j < DS_CHUNK; ++j)
                next[m][j] = (src[m] && t0 + j < n) ? src[m][(size_t)(first + t0 + j) * src_ld[m]] : 0.f;
    };
    request(0);
    for (int t0 = 0; t0 < n; t0 += DS_CHUNK) {
#pragma unroll
        for (int m = 0; m < SLOTS; ++m) {
            int x = tid + m * DS_THREADS;
            if (x < ROW) {
#pragma unroll
                for (int j = 0; j < DS_CHUNK; ++j) {
                    float val = next[m][j];
                    if (BONUS && is_logit[m]) val = expf(-expf(val + offset[m]));
                    if (!src[m]) val = fixed[m];
                    if (t0 + j >= n) val = beyond[m];
                    ds_rows[j * ROW + x] = val;
                }
            }
        }
        __syncthreads();
        if (t0 + DS_CHUNK < n) request(t0 + DS_CHUNK);
        int here = min(DS_CHUNK, n - t0);
        const float* mine = ds_rows + l * R;
        for (int j0 = 0; j0 < here; j0 += DS_TOKENS) {
            float acc[NV];
#pragma unroll
            for (int jj = 0; jj < DS_TOKENS; ++jj) {
                const float* tok = mine + (j0 + jj) * ROW;
                float qq[R], kk[R], ww[R], vv[CPL];
                if constexpr (R % 4 == 0) {
#pragma unroll
                    for (int r4 = 0; r4 < R / 4; ++r4) {
                        float4 q4 = *(const float4*)(tok + 4 * r4);
                        float4 k4 = *(const float4*)(tok + DKP + 4 * r4);
                        qq[4 * r4] = q4.x; qq[4 * r4 + 1] = q4.y; qq[4 * r4 + 2] = q4.z; qq[4 * r4 + 3] = q4.w;
                        kk[4 * r4] = k4.x; kk[4 * r4 + 1] = k4.y; kk[4 * r4 + 2] = k4.z; kk[4 * r4 + 3] = k4.w;
                        if constexpr (BONUS) {
                            float4 w4 = *(const float4*)(tok + 2 * DKP + 4 * r4);
                            ww[4 * r4] = w4.x; ww[4 * r4 + 1] = w4.y; ww[4 * r4 + 2] = w4.z; ww[4 * r4 + 3] = w4.w;
                        }
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        qq[r] = tok[r];
                        kk[r] = tok[DKP + r];
                        if constexpr (BONUS) ww[r] = tok[2 * DKP + r];
                    }
                }
                const float* vals = ds_rows + (j0 + jj) * ROW + ARRAYS * DKP;
                if constexpr (CPL == 4) {
                    float4 v4 = *(const float4*)(vals + c * CPL);
                    vv[0] = v4.x; vv[1] = v4.y; vv[2] = v4.z; vv[3] = v4.w;
                } else {
#pragma unroll
                    for (int p = 0; p < CPL; ++p) vv[p] = vals[c * CPL + p];
                }
                float dec = 0.f;
                if constexpr (!BONUS) dec = vals[TILE];
                token(qq, kk, ww, vv, dec, acc + jj * CPL);
            }
#pragma unroll
            for (int i = 0; i < NV; ++i) acc[i] = row16_sum(acc[i]);
            float out_val = acc[0];
#pragma unroll
            for (int i = 1; i < NV; ++i) out_val = l == i ? acc[i] : out_val;
            int jj = l / CPL, p = l - jj * CPL;
            if (l < NV && j0 + jj < here && col0 + p < a.dv)
                a.out[(size_t)(first + t0 + j0 + jj) * a.n_heads * a.dv + (size_t)h * a.dv + col0 + p] = out_val;
        }
        __syncthreads();                         // the rows are rewritten by the next chunk
    }
    keep_state();
}

template <int R, int CPL>
static void launch_decay_scan_cols(const DecayScanArgs& a, int n_seqs, hipStream_t stream) {
    dim3 grid(n_seqs, a.n_heads, ceil_div(a.dv, DS_GROUPS * CPL));
    if (a.bonus) decay_scan_kernel<R, CPL, true><<<grid, DS_THREADS, 0, stream>>>(a);
    else decay_scan_kernel<R, CPL, false><<<grid, DS_THREADS, 0, stream>>>(a);
}

template <int R>
static void launch_decay_scan(const DecayScanArgs& a, int n_seqs, hipStream_t stream) {
        // Two columns per lane (a lane's reads of q, k and the decays then serve both) where blocks of 16 columns would be
    // more than two a CU: measured on 8 x 2,048 tokens of 32 heads of 64 x 64 at 0.76 ms against 1.06 with one column
    // and 0.76 with four; a single sequence, whose blocks are fewer than the CUs, is faster with one (0.47 against 0.52).
    long long blocks = (long long)n_seqs * a.n_heads * ceil_div(a.dv, DS_GROUPS);
    if (R <= 8 && a.dv > DS_GROUPS && blocks > 2ll * cu_count()) launch_decay_scan_cols<R, R <= 8 ? 2 : 1>(a, n_seqs, stream);
    else launch_decay_scan_cols<R, 1>(a, n_seqs, stream);
}

ROCML_EXPORT int rocml_decay_scan(const float* q, int ldq, int q_col0, const float* k, int ldk, int k_col0, const float* v,
                                  int ldv, int v_col0, const float* w, int ldw, int w_col0, const float* w_offset,
                                  const float* head_decay, const float* bonus, float* state, int n_slots, const int* cu_seqlens,
                                  const int* seq_slots, int n_seqs, int n_tokens, float* out, int n_heads, int dk, int dv,
                                  hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && n_slots > 0 && n_heads > 0 && dk > 0 && dv > 0, "decay_scan: bad sizes T=%d B=%d H=%d",
                  n_tokens, n_seqs, n_heads);
    ROCML_REQUIRE(dk <= 16 * DS_LANES, "decay_scan: a key size of %d exceeds %d", dk, 16 * DS_LANES);
    ROCML_REQUIRE(q && k && v && state && cu_seqlens && seq_slots && out, "decay_scan: missing arguments");
    ROCML_REQUIRE((w != nullptr) != (head_decay != nullptr) && (w != nullptr) == (bonus != nullptr),
                  "decay_scan: a decay per token and channel with a bonus, or one decay per head without");
    ROCML_REQUIRE(!w_offset || w, "decay_scan: an offset goes with decays given as logits");
    ROCML_REQUIRE(q_col0 >= 0 && k_col0 >= 0 && v_col0 >= 0 && ldq >= q_col0 + n_heads * dk && ldk >= k_col0 + n_heads * dk &&
                      ldv >= v_col0 + n_heads * dv && (!w || (w_col0 >= 0 && ldw >= w_col0 + n_heads * dk)),
                  "decay_scan: a row stride is too small for its columns");
    if (n_tokens == 0 || n_seqs == 0) return 0;
    DecayScanArgs a{q, ldq, q_col0, k, ldk, k_col0, v, ldv, v_col0, w, ldw, w_col0, w_offset, head_decay, bonus, state, cu_seqlens,
                    seq_slots, out, n_heads, dk, dv};
    int r = ceil_div(dk, DS_LANES);
    if (r <= 1) launch_decay_scan<1>(a, n_seqs, stream);
    else if (r <= 2) launch_decay_scan<2>(a, n_seqs, stream);
    else if (r <= 4) launch_decay_scan<4>(a, n_seqs, stream);
    else if (r <= 8) launch_decay_scan<8>(a, n_seqs, stream);
    else launch_decay_scan<16>(a, n_seqs, stream);
    ROCML_CHECK_LAUNCH("decay_scan");
    return 0;
}

// ---- rotation of heads inside a 32-bit matrix --------------------------------------------
// Columns col0 .. col0 + n_heads * d - 1 of buf [T, ld]: of every head the first `rot` numbers turn, number i with
// number i + rot/2 by the angle whose cosine and sine stand in column i of the tables [T, rot/2]; then every number
// of the heads is multiplied by `scale` (heads from `heads_first` on by `scale_rest`: queries and keys that lie side by
// side go through one launch).  In place; a thread owns a pair (or one number beyond the rotated part).
__global__ void __launch_bounds__(RC_BLOCK)
rotate_rows_kernel(float* __restrict__ buf, int ld, int col0, int n_heads, int d, int rot, const float* __restrict__ cos_t,
                   const float* __restrict__ sin_t, float scale, int heads_first, float scale_rest, long long total) {
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx >= total) return;
    int half = rot / 2, per_head = d - half;
    long long th = idx / per_head;
    int e = (int)(idx - th * per_head);
    long long t = th / n_heads;
    int h = (int)(th - t * n_heads);
    float* row = buf + (size_t)t * ld + col0 + (size_t)h * d;
    if (h >= heads_first) scale = scale_rest;
    if (e < half) {
        float c = cos_t[(size_t)t * half + e], s = sin_t[(size_t)t * half + e];
        float x = row[e], y = row[e + half];
        row[e] = (x * c - y * s) * scale;
        row[e + half] = (y * c + x * s) * scale;
    } else {
        row[e + half] *= scale;
    }
}

ROCML_EXPORT int rocml_rotate_rows(float* buf, int ld, int col0, int n_tokens, int n_heads, int d, int rot, const float* cos_t,
                                   const float* sin_t, float scale, int heads_first, float scale_rest, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && n_heads > 0 && d > 0 && rot >= 0 && rot % 2 == 0 && rot <= d, "rotate_rows: bad sizes heads=%d d=%d rot=%d",
                  n_heads, d, rot);
    ROCML_REQUIRE(buf && col0 >= 0 && ld >= col0 + n_heads * d && (rot == 0 || (cos_t && sin_t)), "rotate_rows: bad arguments");
    long long total = (long long)n_tokens * n_heads * (d - rot / 2);
    if (total == 0) return 0;
    rotate_rows_kernel<<<ceil_div(total, RC_BLOCK), RC_BLOCK, 0, stream>>>(buf, ld, col0, n_heads, d, rot, cos_t, sin_t, scale,
                                                                           heads_first, scale_rest, total);
    ROCML_CHECK_LAUNCH("rotate_rows");
    return 0;
}

// ---- mixes of a token's input with the previous token's ------------------------------------
// out[m, t, :] = h_t + (h_(t-1) - h_t) * mu[m, :] for every one of the n_mix rows of mu, in 32-bit, written in out's
// type.  Before a sequence's first token of the step stands the sequence's kept row (state [slot, n], zeros at its
// start); the thread that reads it also writes the sequence's last row of the step there, so nobody reads a row
// that another thread has replaced.
template <typename T>
__global__ void __launch_bounds__(RC_BLOCK)
shift_mix_kernel(const T* __restrict__ h, int n, const float* __restrict__ mu, int n_mix, float* __restrict__ state,
                 const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_slots,
                 T* __restrict__ out, long long total, long long mix_stride) {
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx >= total) return;
    long long t = idx / n;
    int c = (int)(idx - t * n);
    int b = token_seq[t];
    int first = cu_seqlens[b];
    float cur = Elem<T>::load(h + idx), prev;
    if (t == first) {
        float* st = state + (size_t)seq_slots[b] * n + c;
        prev = *st;
        *st = Elem<T>::load(h + (size_t)(cu_seqlens[b + 1] - 1) * n + c);
    } else {
        prev = Elem<T>::load(h + idx - n);
    }
    float d = prev - cur;
    for (int m = 0; m < n_mix; ++m) Elem<T>::store(out + m * mix_stride + idx, fmaf(d, mu[(size_t)m * n + c], cur));
}

ROCML_EXPORT int rocml_shift_mix(const void* h, int dtype, int n_tokens, int n, const float* mu, int n_mix, float* state, int n_slots,
                                 const int* token_seq, const int* cu_seqlens, const int* seq_slots, int n_seqs, void* out,
                                 hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && n > 0 && n_mix > 0 && n_slots > 0 && n_seqs >= 0, "shift_mix: bad sizes T=%d n=%d mixes=%d", n_tokens, n, n_mix);
    ROCML_REQUIRE(h && mu && state && token_seq && cu_seqlens && seq_slots && out, "shift_mix: missing arguments");
    long long total = (long long)n_tokens * n;
    if (total == 0) return 0;
    int grid = ceil_div(total, RC_BLOCK);
    if (dtype == ROCML_F32)
        shift_mix_kernel<float><<<grid, RC_BLOCK, 0, stream>>>((const float*)h, n, mu, n_mix, state, token_seq, cu_seqlens, seq_slots,
                                                             (float*)out, total, total);
    else if (dtype == ROCML_BF16)
        shift_mix_kernel<bf16_t><<<grid, RC_BLOCK, 0, stream>>>((const bf16_t*)h, n, mu, n_mix, state, token_seq, cu_seqlens, seq_slots,
                                                              (bf16_t*)out, total, total);
    else return rocml_fail("shift_mix: unknown dtype code %d", dtype);
    ROCML_CHECK_LAUNCH("shift_mix");
    return 0;
}

// ---- small maps between two products ------------------------------------------------------
// out = tanh(x) in out's type (the middle of a decay's two small matrices), and
// out = exp(-exp(x + offset[c])) in 32-bit (the decay itself, per token and channel).
template <typename T>
__global__ void __launch_bounds__(RC_BLOCK)
tanh_kernel(const float* __restrict__ x, T* __restrict__ out, long long total) {
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx < total) Elem<T>::store(out + idx, tanhf(x[idx]));
}

ROCML_EXPORT int rocml_tanh(const float* x, void* out, int out_dtype, long long total, hipStream_t stream) {
    ROCML_REQUIRE(total >= 0 && x && out, "tanh: bad arguments");
    if (total == 0) return 0;
    int grid = ceil_div(total, RC_BLOCK);
    if (out_dtype == ROCML_F32) tanh_kernel<float><<<grid, RC_BLOCK, 0, stream>>>(x, (float*)out, total);
    else if (out_dtype == ROCML_BF16) tanh_kernel<bf16_t><<<grid, RC_BLOCK, 0, stream>>>(x, (bf16_t*)out, total);
    else return rocml_fail("tanh: unknown dtype code %d", out_dtype);
    ROCML_CHECK_LAUNCH("tanh");
    return 0;
}

__global__ void __launch_bounds__(RC_BLOCK)
double_exp_decay_kernel(float* __restrict__ x, const float* __restrict__ offset, int n, long long total) {
    long long idx = (long long)blockIdx.x * RC_BLOCK + threadIdx.x;
    if (idx < total) x[idx] = expf(-expf(x[idx] + offset[idx % n]));
}

ROCML_EXPORT int rocml_double_exp_decay(float* x, const float* offset, int n_rows, int n, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n > 0 && x && offset, "double_exp_decay: bad arguments");
    long long total = (long long)n_rows * n;
    if (total == 0) return 0;
    double_exp_decay_kernel<<<ceil_div(total, RC_BLOCK), RC_BLOCK, 0, stream>>>(x, offset, n, total);
    ROCML_CHECK_LAUNCH("double_exp_decay");
    return 0;
}
