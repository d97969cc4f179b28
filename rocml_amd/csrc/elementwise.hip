// Memory-bound kernels of the decoder for gfx950 (wave64): embedding gather, RMSNorm,
// SwiGLU, rotation tables, and the fused per-head norm + rotation + cache append.
// Norm statistics, angles and the SiLU are computed in 32-bit (angles in 64-bit) whatever
// the storage type is.
#include "common.h"

ROCML_LAST_ERROR_FN(elementwise)

constexpr int EW_BLOCK = 256;

// ---- embedding -------------------------------------------------------------------
// out[t, :] = float(table[ids[t], :]) * scale  (rocml-kernels/kernels/embedding.hip:6-18;
// the reference has no scale, callers pass 1).
// With a table of positions ([max_pos, hidden], same type): the row of the token's position is
// added, not scaled.
template <typename T>
__global__ void embed_gather_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int hidden, int vocab, float scale,
                                    const T* __restrict__ pos_table, const int* __restrict__ positions, int max_pos) {
    int t = blockIdx.x;
    int id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const T* row = table + (size_t)id * hidden;
    float* o = out + (size_t)t * hidden;
    if (pos_table) {
        int p = positions[t];
        p = p < 0 ? 0 : (p >= max_pos ? max_pos - 1 : p);
        const T* prow = pos_table + (size_t)p * hidden;
        for (int i = threadIdx.x; i < hidden; i += EW_BLOCK) o[i] = fmaf(Elem<T>::load(row + i), scale, Elem<T>::load(prow + i));
        return;
    }
    for (int i = threadIdx.x; i < hidden; i += EW_BLOCK) o[i] = Elem<T>::load(row + i) * scale;
}

ROCML_EXPORT int rocml_embed_gather(const void* table, int table_dtype, const int* ids, float* out,
                                    int n_tokens, int hidden, int vocab, float scale,
                                    const void* pos_table, const int* positions, int max_pos,
                                    hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0, "embed_gather: bad sizes T=%d H=%d V=%d",
                  n_tokens, hidden, vocab);
    ROCML_REQUIRE(!pos_table || (positions && max_pos > 0), "embed_gather: a table of positions needs the positions");
    if (n_tokens == 0) return 0;
    if (table_dtype == ROCML_F32)
        embed_gather_kernel<float><<<n_tokens, EW_BLOCK, 0, stream>>>((const float*)table, ids, out,
                                                                      hidden, vocab, scale, (const float*)pos_table, positions, max_pos);
    else if (table_dtype == ROCML_BF16)
        embed_gather_kernel<bf16_t><<<n_tokens, EW_BLOCK, 0, stream>>>((const bf16_t*)table, ids, out,
                                                                       hidden, vocab, scale, (const bf16_t*)pos_table, positions, max_pos);
    else
        return rocml_fail("embed_gather: unknown dtype code %d", table_dtype);
    ROCML_CHECK_LAUNCH("embed_gather");
    return 0;
}

// ---- block reduction -------------------------------------------------------------
// Sum over a block of EW_BLOCK threads in a fixed order: lanes by butterfly, waves in order.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    int wave = threadIdx.x / WAVE;
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < EW_BLOCK / WAVE; ++w) total += scratch[w];
    return total;
}

// ---- RMSNorm ---------------------------------------------------------------------
// out[r, i] = x[src(r), i] * (1/sqrt(sum(x^2)/n + eps)) * gain[i]
// (rocml-kernels/kernels/rmsnorm.hip:18-42).  `rows` optionally gathers source rows.
// With `partials` ([n_splits][rows of x][n], the split-K partial sums of the product whose
// result belongs to x) the kernel first forms x + sum of the partials in split order, which is
// the residual sum the reference does in a kernel of its own
// (rocml-kernels/kernels/elementwise.hip:7-12), writes it back to x unless rows are gathered,
// and normalises that.
template <typename TO>
__global__ void rmsnorm_kernel(float* x, const float* __restrict__ gain, TO* __restrict__ out,
                               const int* __restrict__ rows, int n, float eps,
                               const float* __restrict__ partials, int n_splits, long long split_stride) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    int r = blockIdx.x;
    int src = rows ? rows[r] : r;
    float* xin = x + (size_t)src * n;
    TO* o = out + (size_t)r * n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
        float v = xin[i];
        for (int sp = 0; sp < n_splits; ++sp) v += partials[sp * split_stride + (size_t)src * n + i];
        if (n_splits > 0 && !rows) xin[i] = v;
        ss = fmaf(v, v, ss);
    }
    float total = block_sum(ss, scratch);
    float inv = 1.0f / sqrtf(total / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
        float v = xin[i];
        if (rows) for (int sp = 0; sp < n_splits; ++sp) v += partials[sp * split_stride + (size_t)src * n + i];
        Elem<TO>::store(o + i, v * inv * gain[i]);
    }
}

// Same result for rows of up to 8192 values that are a multiple of 4: the row stays in
// registers between the two passes and all loads are issued at once (a loop of single loads
// waits for each one in turn, which is what a one-row decode step would spend its time on).
constexpr int RN_MAX_VEC = 8;

__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
    *(float4*)p = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store4(bf16_t* p, float a, float b, float c, float d) {
    uint2 v;
    v.x = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
    v.y = (uint32_t)f32_to_bf16(c) | ((uint32_t)f32_to_bf16(d) << 16);
    *(uint2*)p = v;
}

template <typename TO, int RN_VEC>
__global__ void __launch_bounds__(EW_BLOCK)
rmsnorm_vec_kernel(float* x, const float* __restrict__ gain, TO* __restrict__ out,
                   const int* __restrict__ rows, int n, float eps, const float* __restrict__ partials,
                   int n_splits, long long split_stride) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    int r = blockIdx.x;
    int src = rows ? rows[r] : r;
    float4* xin = (float4*)(x + (size_t)src * n);
    const float4* g4 = (const float4*)gain;
    TO* o = out + (size_t)r * n;
    int nv = n / 4;
    float4 v[RN_VEC], g[RN_VEC];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < RN_VEC; ++j) {
        int idx = threadIdx.x + j * EW_BLOCK;
        bool ok = idx < nv;
        v[j] = xin[ok ? idx : 0];
        g[j] = g4[ok ? idx : 0];
        if (!ok) v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (n_splits > 0) {
        const float4* p4 = (const float4*)(partials + (size_t)src * n);
        long long stride4 = split_stride / 4;
        constexpr int GROUP = 32 / RN_VEC;              // splits whose loads are in flight together
        for (int sp = 0; sp < n_splits; sp += GROUP) {  // loads of a group all issued, added in split order
            float4 a[GROUP][RN_VEC];
#pragma unroll
            for (int q = 0; q < GROUP; ++q)
#pragma unroll
                for (int j = 0; j < RN_VEC; ++j) {
                    int idx = threadIdx.x + j * EW_BLOCK;
                    int safe = idx < nv ? idx : 0;
                    a[q][j] = p4[(sp + q < n_splits ? sp + q : sp) * stride4 + safe];
                }
#pragma unroll
            for (int q = 0; q < GROUP; ++q)
#pragma unroll
                for (int j = 0; j < RN_VEC; ++j) {
                    if ((int)threadIdx.x + j * EW_BLOCK >= nv || sp + q >= n_splits) continue;
                    v[j].x += a[q][j].x; v[j].y += a[q][j].y; v[j].z += a[q][j].z; v[j].w += a[q][j].w;
                }
        }
        if (!rows) {
#pragma unroll
            for (int j = 0; j < RN_VEC; ++j) {
                int idx = threadIdx.x + j * EW_BLOCK;
                if (idx < nv) xin[idx] = v[j];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < RN_VEC; ++j)
        ss = fmaf(v[j].x, v[j].x, fmaf(v[j].y, v[j].y, fmaf(v[j].z, v[j].z, fmaf(v[j].w, v[j].w, ss))));
    float total = block_sum(ss, scratch);
    float inv = 1.0f / sqrtf(total / (float)n + eps);
#pragma unroll
    for (int j = 0; j < RN_VEC; ++j) {
        int idx = threadIdx.x + j * EW_BLOCK;
        if (idx < nv)
            store4(o + 4 * idx, v[j].x * inv * g[j].x, v[j].y * inv * g[j].y, v[j].z * inv * g[j].z,
                   v[j].w * inv * g[j].w);
    }
}

ROCML_EXPORT int rocml_rmsnorm(float* x, const float* gain, void* out, int out_dtype, const int* rows,
                               int n_rows, int n, float eps, const float* partials, int n_splits,
                               long long split_stride, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n > 0, "rmsnorm: bad sizes rows=%d n=%d", n_rows, n);
    ROCML_REQUIRE(eps > 0.f, "rmsnorm: eps must be positive, got %g", (double)eps);
    ROCML_REQUIRE(n_splits >= 0 && (n_splits == 0 || (partials && split_stride > 0)),
                  "rmsnorm: partial sums need a pointer and a stride");
    if (n_rows == 0) return 0;
    bool vec = n % 4 == 0 && n <= 4 * RN_MAX_VEC * EW_BLOCK && (uintptr_t)x % 16 == 0 &&
               (uintptr_t)gain % 16 == 0 && (uintptr_t)out % 16 == 0 &&
               (n_splits == 0 || ((uintptr_t)partials % 16 == 0 && split_stride % 4 == 0));
#define RN_ARGS rows, n, eps, partials, n_splits, split_stride
    bool small = n <= 4 * 4 * EW_BLOCK;      // rows of up to 4096 values: 4 vectors per thread
    if (vec && out_dtype == ROCML_F32 && small)
        rmsnorm_vec_kernel<float, 4><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (float*)out, RN_ARGS);
    else if (vec && out_dtype == ROCML_F32)
        rmsnorm_vec_kernel<float, 8><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (float*)out, RN_ARGS);
    else if (vec && out_dtype == ROCML_BF16 && small)
        rmsnorm_vec_kernel<bf16_t, 4><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (bf16_t*)out, RN_ARGS);
    else if (vec && out_dtype == ROCML_BF16)
        rmsnorm_vec_kernel<bf16_t, 8><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (bf16_t*)out, RN_ARGS);
    else if (out_dtype == ROCML_F32)
        rmsnorm_kernel<float><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (float*)out, RN_ARGS);
    else if (out_dtype == ROCML_BF16)
        rmsnorm_kernel<bf16_t><<<n_rows, EW_BLOCK, 0, stream>>>(x, gain, (bf16_t*)out, RN_ARGS);
    else
        return rocml_fail("rmsnorm: unknown dtype code %d", out_dtype);
#undef RN_ARGS
    ROCML_CHECK_LAUNCH("rmsnorm");
    return 0;
}

// ---- gated activation ------------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, inter + i],  silu(g) = g / (1 + exp(-g))
// (rocml-kernels/kernels/silu_mul.hip:12-20).  Gate and up halves lie side by side in a row.
// With `interleaved` a row holds (gate_0, up_0, gate_1, up_1, ...), the order the fused product
// epilogue wants its weight rows in.
// act: 0 silu, 1 relu (max(g, 0)), 2 gelu with the tanh form 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))),
// 3 g sigmoid(1.702 g).
__device__ __forceinline__ float gate_activation(float g, int act) {
    if (act == 1) return fmaxf(g, 0.f);
    if (act == 3) return g / (1.0f + expf(-1.702f * g));      // g sigmoid(1.702 g)
    if (act == 2) return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    return g / (1.0f + expf(-g));
}

// limit > 0: g is cut off above at limit and u is held inside [-limit, limit] first; up_offset is
// added to u (after the limit).
template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int inter,
                              long long total, int interleaved, int act, float limit, float up_offset) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    long long t = idx / inter;
    int i = (int)(idx - t * inter);
    const TI* row = gu + (size_t)t * 2 * inter;
    float g = Elem<TI>::load(row + (interleaved ? 2 * i : i));
    float u = Elem<TI>::load(row + (interleaved ? 2 * i + 1 : inter + i));
    if (limit > 0.f) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
    }
    Elem<TO>::store(out + idx, gate_activation(g, act) * (u + up_offset));
}

ROCML_EXPORT int rocml_swiglu(const void* gu, int in_dtype, void* out, int out_dtype, int n_tokens,
                              int inter, int interleaved, int act, float limit, float up_offset, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && inter > 0, "swiglu: bad sizes T=%d I=%d", n_tokens, inter);
    ROCML_REQUIRE(act >= 0 && act <= 3, "swiglu: unknown activation %d (0 silu, 1 relu, 2 gelu_tanh, 3 sigmoid_1702)", act);
    ROCML_REQUIRE(limit >= 0.f, "swiglu: the limit must not be negative (0: none)");
    long long total = (long long)n_tokens * inter;
    if (total == 0) return 0;
    int grid = ceil_div(total, EW_BLOCK);
    if (in_dtype == ROCML_F32 && out_dtype == ROCML_F32)
        swiglu_kernel<float, float><<<grid, EW_BLOCK, 0, stream>>>((const float*)gu, (float*)out, inter, total, interleaved, act, limit, up_offset);
    else if (in_dtype == ROCML_F32 && out_dtype == ROCML_BF16)
        swiglu_kernel<float, bf16_t><<<grid, EW_BLOCK, 0, stream>>>((const float*)gu, (bf16_t*)out, inter, total, interleaved, act, limit, up_offset);
    else if (in_dtype == ROCML_BF16 && out_dtype == ROCML_BF16)
        swiglu_kernel<bf16_t, bf16_t><<<grid, EW_BLOCK, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, inter, total, interleaved, act, limit, up_offset);
    else
        return rocml_fail("swiglu: unsupported dtype pair in=%d out=%d", in_dtype, out_dtype);
    ROCML_CHECK_LAUNCH("swiglu");
    return 0;
}

// ---- rotation tables -------------------------------------------------------------
// cos/sin of pos * inv_freq[i] for every token of a step, angle formed in 64-bit so that the
// 32-bit table is exact to rounding (the reference forms the angle in 32-bit,
// rocml-kernels/kernels/rope.hip:23-27).  inv_freq[i] = theta^(-2i/rot_dim) comes from the host.
__global__ void rope_table_kernel(const int* __restrict__ pos, const double* __restrict__ inv_freq,
                                  float* __restrict__ cos_t, float* __restrict__ sin_t, int half,
                                  long long total, float scale) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    long long t = idx / half;
    int i = (int)(idx - t * half);
    double a = (double)pos[t] * inv_freq[i];
    cos_t[idx] = (float)cos(a) * scale;       // scale: one factor on every cosine and sine (1: none)
    sin_t[idx] = (float)sin(a) * scale;
}

ROCML_EXPORT int rocml_rope_table(const int* pos, const double* inv_freq, float* cos_t, float* sin_t,
                                  int n_tokens, int half, float scale, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && half > 0, "rope_table: bad sizes T=%d half=%d", n_tokens, half);
    long long total = (long long)n_tokens * half;
    if (total == 0) return 0;
    rope_table_kernel<<<ceil_div(total, EW_BLOCK), EW_BLOCK, 0, stream>>>(pos, inv_freq, cos_t, sin_t,
                                                                           half, total, scale);
    ROCML_CHECK_LAUNCH("rope_table");
    return 0;
}

// ---- per-head norm + rotation + cache append -------------------------------------
// One wave per (token, head row) of the packed projection output [T, (Hq + 2 Hkv) * D]:
// q and k rows are normalised over D with one gain vector each
// (rocml/src/forward/attention.rs:105-123), rotated with NEOX pairing (i, i + rot/2)
// (rocml-kernels/kernels/rope.hip:18-33); with n_splits > 1 the input is the projection's split-K
// partial sums [n_splits][T, ld], summed here in split order; q goes to q_out, k and v go straight into the
// paged cache at the token's position (rocml-kernels/kernels/chunk_reshape.hip:37-74 is the
// reference's separate scatter).  Cache layout: keys [page, Hkv, page_size, D], values
// transposed inside a page [page, Hkv, D, page_size] (what the MFMA attention kernels read).
constexpr int QK_MAX_PER_LANE = 8;   // D <= 512

// A query's stretch with its position: 1 + coef * ln(floor((p + 1) / every) + 1); every = 0: none.
__device__ __forceinline__ float query_temperature(int pos, float coef, int every) {
    return every > 0 ? 1.0f + coef * logf((float)((pos + 1) / every + 1)) : 1.0f;
}
constexpr int QK_WAVES = EW_BLOCK / WAVE;

// LOCAL_PAIR: the whole head is rotated and a lane holds at least two values, so both values of a
// pair (e, e + d/2) are in the same lane and no exchange through LDS is needed.
template <typename TI, typename TO, int QK_PER_LANE, bool LOCAL_PAIR>
__global__ void qk_norm_rope_append_kernel(
    const TI* __restrict__ qkv, int ld, int n_tokens, int hq, int hkv, int d,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot,
    TO* __restrict__ q_out, TO* __restrict__ kcache, TO* __restrict__ vcache,
    const int* __restrict__ block_table, int bt_width, const int* __restrict__ token_seq,
    const int* __restrict__ token_pos, int page_size, int write_kv, int n_splits, long long split_stride,
    int rows_per_token, int pairing, int first_row, const float* __restrict__ bias, int dv,
    float qt_coef, int qt_every, const float* __restrict__ span_inv, int span_self) {
    // span_inv (may be null): [T, 2], the norm's factor of a token's whole q row and whole k row; the gains then
    // have one number per column of the q (k) projection, and a head takes its own part of them.  span_self: the
    // same norm, but every wave forms its row's factor itself (few tokens: one launch less).
    // qt_coef, qt_every: the queries' stretch with their position (after the norm); every = 0: none.
    // bias (may be null): one number per column of the packed row, added to the projection's sums.
    // dv: the size of a value head; the value rows start behind the Hq + Hkv rows of d numbers.
    extern __shared__ float stage[];   // [QK_WAVES][d]
    int wave = threadIdx.x / WAVE;
    int lane = threadIdx.x & (WAVE - 1);
    long long row = (long long)blockIdx.x * QK_WAVES + wave;
    bool active = row < (long long)n_tokens * rows_per_token;
    int t = active ? (int)(row / rows_per_token) : 0;
    int r = first_row + (active ? (int)(row - (long long)t * rows_per_token) : 0);     // first_row = hq: no q rows
    int kind = r < hq ? 0 : (r < hq + hkv ? 1 : 2);   // q, k, v
    if (!write_kv && kind != 0) active = false;
    int width = kind == 2 ? dv : d;
    size_t col0 = kind == 2 ? (size_t)(hq + hkv) * d + (size_t)(r - hq - hkv) * dv : (size_t)r * d;
    const TI* src = qkv + (size_t)t * ld + col0;
    float v[QK_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < QK_PER_LANE; ++j) {
        int e = lane + j * WAVE;
        bool ok = active && e < width;
        float val = Elem<TI>::load(ok ? src + e : qkv);
        if (bias && ok) val += bias[col0 + e];
        // split-K partial sums of the projection, added in split order
        // (four loads in flight at a time)
        for (int sp = 1; sp < n_splits; sp += 4) {
            const TI* p = ok ? src + e : qkv;
            float a0 = Elem<TI>::load(ok ? p + sp * split_stride : qkv);
            float a1 = Elem<TI>::load(ok && sp + 1 < n_splits ? p + (sp + 1) * split_stride : qkv);
            float a2 = Elem<TI>::load(ok && sp + 2 < n_splits ? p + (sp + 2) * split_stride : qkv);
            float a3 = Elem<TI>::load(ok && sp + 3 < n_splits ? p + (sp + 3) * split_stride : qkv);
            val += a0;
            if (sp + 1 < n_splits) val += a1;
            if (sp + 2 < n_splits) val += a2;
            if (sp + 3 < n_splits) val += a3;
        }
        v[j] = ok ? val : 0.f;
        ss = fmaf(v[j], v[j], ss);
    }
    const float* gain = kind == 0 ? q_gain : (kind == 1 ? k_gain : nullptr);
    if (gain) {
        float inv;
        if (span_inv) {
            inv = span_inv[(size_t)t * 2 + kind];
            gain += (size_t)(kind == 0 ? r : r - hq) * d;
        } else if (span_self) {
            int w0 = kind == 0 ? 0 : hq * d, wn = kind == 0 ? hq * d : hkv * d;
            const TI* whole = qkv + (size_t)t * ld + w0;
            // (the numbers are added in the order of the kernel that forms the factors for many tokens, so that a
            // token's factor does not depend on how many tokens its step has: span_self = 2 is that kernel's order
            // for rows in 16-byte pieces, a lane taking four neighbours at a time)
            float s2 = 0.f;
            if (span_self == 2) {
                for (int c = lane * 4; c < wn; c += WAVE * 4) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float val = Elem<TI>::load(whole + c + e) + (bias ? bias[w0 + c + e] : 0.f);
                        s2 = fmaf(val, val, s2);
                    }
                }
            } else {
                for (int c = lane; c < wn; c += WAVE) {
                    float val = Elem<TI>::load(whole + c) + (bias ? bias[w0 + c] : 0.f);
                    s2 = fmaf(val, val, s2);
                }
            }
            inv = 1.0f / sqrtf(wave_sum(s2) / (float)wn + eps);
            gain += (size_t)(kind == 0 ? r : r - hq) * d;
        } else {
            inv = 1.0f / sqrtf(wave_sum(ss) / (float)d + eps);
        }
#pragma unroll
        for (int j = 0; j < QK_PER_LANE; ++j) {
            int e = lane + j * WAVE;
            if (e < d) v[j] = v[j] * inv * gain[e];
        }
    }
    if (qt_every > 0 && kind == 0) {
        float temp = query_temperature(token_pos[t], qt_coef, qt_every);
#pragma unroll
        for (int j = 0; j < QK_PER_LANE; ++j) v[j] *= temp;
    }
    bool rotate = cos_t != nullptr && kind != 2;
    if (LOCAL_PAIR) {
        if (rotate) {
            constexpr int HJ = QK_PER_LANE / 2 > 0 ? QK_PER_LANE / 2 : 1;
            const float* c = cos_t + (size_t)t * (d / 2);
            const float* s = sin_t + (size_t)t * (d / 2);
#pragma unroll
            for (int j = 0; j < HJ; ++j) {
                int e = lane + j * WAVE;                     // pair (e, e + d/2) = values j and j + HJ
                float cs = c[e], sn = s[e], lo = v[j], hi = v[j + HJ];
                v[j] = lo * cs - hi * sn;
                v[j + HJ] = lo * sn + hi * cs;
            }
        }
    } else {
        float* mine = stage + (size_t)wave * d;
        if (rotate) {
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) {
                int e = lane + j * WAVE;
                if (e < d) mine[e] = v[j];
            }
        }
        __syncthreads();
        if (rotate) {
            int half = rot / 2;
            const float* c = cos_t + (size_t)t * half;
            const float* s = sin_t + (size_t)t * half;
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) {
                int e = lane + j * WAVE;
                if (e < rot) {
                    if (pairing == 1) {
                        // neighbours (2i, 2i + 1) are a pair, angle i
                        float cs = c[e >> 1], sn = s[e >> 1], other = mine[e ^ 1];
                        v[j] = (e & 1) ? other * sn + v[j] * cs : v[j] * cs - other * sn;
                    } else if (e < half) {
                        v[j] = v[j] * c[e] - mine[e + half] * s[e];
                    } else {
                        v[j] = mine[e - half] * s[e - half] + v[j] * c[e - half];
                    }
                }
            }
        }
    }
    if (!active) return;
    TO* dst;
    if (kind == 0) {
        dst = q_out + ((size_t)t * hq + r) * d;
    } else {
        int head = kind == 1 ? r - hq : r - hq - hkv;
        int pos = token_pos[t];
        int page = block_table[(size_t)token_seq[t] * bt_width + pos / page_size];
        if (page < 0) return;
        if (kind == 2) {
            // values are stored transposed inside a page: [page, Hkv, Dv, page_size]
            TO* vdst = vcache + ((size_t)page * hkv + head) * dv * page_size + pos % page_size;
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) {
                int e = lane + j * WAVE;
                if (e < dv) Elem<TO>::store(vdst + (size_t)e * page_size, v[j]);
            }
            return;
        }
        dst = kcache + (((size_t)page * hkv + head) * page_size + pos % page_size) * d;
    }
#pragma unroll
    for (int j = 0; j < QK_PER_LANE; ++j) {
        int e = lane + j * WAVE;
        if (e < d) Elem<TO>::store(dst + e, v[j]);
    }
}

// Prompts: q and k rows of many tokens.  A wave takes ROWS rows and issues the loads of all of
// them before it works on the first (one row per wave leaves too few bytes in flight and too
// many tiny blocks to dispatch).  Only the case LOCAL_PAIR describes: whole head rotated, both
// values of a pair in one lane, complete projections (no partial sums).
template <typename TI, typename TO, int QK_PER_LANE, int ROWS>
__global__ void __launch_bounds__(EW_BLOCK)
qk_norm_rope_rows_kernel(
    const TI* __restrict__ qkv, int ld, int n_tokens, int hq, int hkv, int d,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    TO* __restrict__ q_out, TO* __restrict__ kcache, const int* __restrict__ block_table, int bt_width,
    const int* __restrict__ token_seq, const int* __restrict__ token_pos, int page_size, int rows_per_token,
    int first_row, const float* __restrict__ bias, float qt_coef, int qt_every, const float* __restrict__ span_inv) {
    constexpr int HJ = QK_PER_LANE / 2;
    int wave = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
    long long total = (long long)n_tokens * rows_per_token;
    long long row0 = ((long long)blockIdx.x * QK_WAVES + wave) * ROWS;
    float v[ROWS][QK_PER_LANE], cs[ROWS][HJ], sn[ROWS][HJ];
    int tok[ROWS], rr[ROWS];
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        long long row = min(row0 + i, total - 1);            // rows past the end repeat the last one, not stored
        tok[i] = (int)(row / rows_per_token);
        rr[i] = first_row + (int)(row - (long long)tok[i] * rows_per_token);
        const TI* src = qkv + (size_t)tok[i] * ld + (size_t)rr[i] * d;
#pragma unroll
        for (int j = 0; j < QK_PER_LANE; ++j) v[i][j] = Elem<TI>::load(src + lane + j * WAVE);
        if (bias) {
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) v[i][j] += bias[(size_t)rr[i] * d + lane + j * WAVE];
        }
        if (cos_t) {
#pragma unroll
            for (int j = 0; j < HJ; ++j) {
                cs[i][j] = cos_t[(size_t)tok[i] * (d / 2) + lane + j * WAVE];
                sn[i][j] = sin_t[(size_t)tok[i] * (d / 2) + lane + j * WAVE];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
        bool is_q = rr[i] < hq;
        const float* gain = is_q ? q_gain : k_gain;
        if (gain) {
            float inv;
            if (span_inv) {          // the norm spans the token's whole q (k) row: its factor is given, the gain is the head's part
                inv = span_inv[(size_t)tok[i] * 2 + (is_q ? 0 : 1)];
                gain += (size_t)(is_q ? rr[i] : rr[i] - hq) * d;
            } else {
                float ss = 0.f;
#pragma unroll
                for (int j = 0; j < QK_PER_LANE; ++j) ss = fmaf(v[i][j], v[i][j], ss);
                inv = 1.0f / sqrtf(wave_sum(ss) / (float)d + eps);
            }
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) v[i][j] = v[i][j] * inv * gain[lane + j * WAVE];
        }
        if (qt_every > 0 && is_q) {
            float temp = query_temperature(token_pos[tok[i]], qt_coef, qt_every);
#pragma unroll
            for (int j = 0; j < QK_PER_LANE; ++j) v[i][j] *= temp;
        }
        if (cos_t) {
#pragma unroll
            for (int j = 0; j < HJ; ++j) {
                float lo = v[i][j], hi = v[i][j + HJ];
                v[i][j] = lo * cs[i][j] - hi * sn[i][j];
                v[i][j + HJ] = lo * sn[i][j] + hi * cs[i][j];
            }
        }
        if (row0 + i >= total) continue;
        TO* dst;
        if (is_q) {
            dst = q_out + ((size_t)tok[i] * hq + rr[i]) * d;
        } else {
            int pos = token_pos[tok[i]];
            int page = block_table[(size_t)token_seq[tok[i]] * bt_width + pos / page_size];
            if (page < 0) continue;
            dst = kcache + (((size_t)page * hkv + (rr[i] - hq)) * page_size + pos % page_size) * d;
        }
#pragma unroll
        for (int j = 0; j < QK_PER_LANE; ++j) Elem<TO>::store(dst + lane + j * WAVE, v[i][j]);
    }
}

// Values of many tokens at once (prompts): a block takes 64 consecutive tokens of the packed
// batch, one key/value head and 32 of its values, stages them in LDS and writes them transposed.
// In the transposed page a token is one 2- or 4-byte column; written token by token every store
// would touch a cache line of its own, written this way the 64 lanes of a wave store 64
// neighbouring positions of one row (they are neighbours wherever the tokens are consecutive
// positions of one sequence inside one page, which is the rule in a prompt).
constexpr int VT_TOKENS = 64, VT_VALUES = 32;

template <typename TI, typename TO>
__global__ void __launch_bounds__(EW_BLOCK)
v_append_tile_kernel(const TI* __restrict__ qkv, int ld, int n_tokens, int v_col0, int hkv, int d,
                     TO* __restrict__ vcache, const int* __restrict__ block_table, int bt_width,
                     const int* __restrict__ token_seq, const int* __restrict__ token_pos, int page_size,
                     const float* __restrict__ bias) {
    __shared__ float vt_stage[VT_TOKENS][VT_VALUES + 1];
    int t0 = blockIdx.x * VT_TOKENS, head = blockIdx.y, e0 = blockIdx.z * VT_VALUES;
    int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    // thread -> (token tid/32 + 8*i, value tid%32): 128 contiguous bytes per token row
    float tmp[VT_TOKENS * VT_VALUES / EW_BLOCK];
#pragma unroll
    for (int i = 0; i < VT_TOKENS * VT_VALUES / EW_BLOCK; ++i) {
        int j = min(t0 + (tid >> 5) + (EW_BLOCK / VT_VALUES) * i, n_tokens - 1), e = min(e0 + (tid & 31), d - 1);
        tmp[i] = Elem<TI>::load(qkv + (size_t)j * ld + v_col0 + (size_t)head * d + e);
        if (bias) tmp[i] += bias[v_col0 + (size_t)head * d + e];
    }
#pragma unroll
    for (int i = 0; i < VT_TOKENS * VT_VALUES / EW_BLOCK; ++i) vt_stage[(tid >> 5) + (EW_BLOCK / VT_VALUES) * i][tid & 31] = tmp[i];
    __syncthreads();
    int t = t0 + lane;
    if (t >= n_tokens) return;
    int pos = token_pos[t];
    int page = block_table[(size_t)token_seq[t] * bt_width + pos / page_size];
    if (page < 0) return;
    TO* dst = vcache + ((size_t)page * hkv + head) * d * page_size + pos % page_size;
#pragma unroll
    for (int i = 0; i < VT_VALUES / (EW_BLOCK / WAVE); ++i) {
        int el = wave + (EW_BLOCK / WAVE) * i;
        if (e0 + el < d) Elem<TO>::store(dst + (size_t)(e0 + el) * page_size, vt_stage[lane][el]);
    }
}

ROCML_EXPORT int rocml_qk_norm_rope_append(
    const void* qkv, int in_dtype, int ld, int n_tokens, int hq, int hkv, int d, const float* q_gain,
    const float* k_gain, float eps, const float* cos_t, const float* sin_t, int rot, int pairing, void* q_out,
    void* kcache, void* vcache, int out_dtype, const int* block_table, int bt_width,
    const int* token_seq, const int* token_pos, int page_size, int write_kv, int n_splits,
    long long split_stride, const float* bias, int dv, float qt_coef, int qt_every, const float* span_inv, int span_self,
    hipStream_t stream) {
    // span_self: the norm spans a token's whole q row and whole k row as with span_inv, and the kernel forms the
    // factors itself (a step of few tokens)
    // span_inv (may be null): [T, 2] factors of a norm over a token's whole q row and whole k row (qk_span_stats);
    // q_gain and k_gain then have hq * d and hkv * d numbers.
    // bias (may be null): [ld] numbers added to the projection's sums; dv (0: d): value head size.
    // qt_coef, qt_every: a query at position p is multiplied by 1 + coef ln(floor((p + 1) / every) + 1)
    // after its norm (every = 0: not).
    if (dv <= 0) dv = d;
    ROCML_REQUIRE(qt_every >= 0, "qk_norm_rope_append: the query stretch's period must not be negative");
    ROCML_REQUIRE(n_tokens >= 0 && (hq > 0 || (hq == 0 && !q_out)) && hkv > 0 && d > 0, "qk_norm_rope_append: bad sizes");
    ROCML_REQUIRE(dv <= QK_MAX_PER_LANE * WAVE, "qk_norm_rope_append: value head size %d exceeds %d", dv,
                  QK_MAX_PER_LANE * WAVE);
    ROCML_REQUIRE(n_splits >= 1 && (n_splits == 1 || (split_stride > 0 && in_dtype == ROCML_F32)),
                  "qk_norm_rope_append: partial sums must be 32-bit with a positive stride");
    ROCML_REQUIRE(d <= QK_MAX_PER_LANE * WAVE, "qk_norm_rope_append: head_dim %d exceeds %d", d,
                  QK_MAX_PER_LANE * WAVE);
    ROCML_REQUIRE(ld >= (hq + hkv) * d + hkv * dv || (!write_kv && ld >= hq * d),
                  "qk_norm_rope_append: row stride %d too small", ld);
    ROCML_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "qk_norm_rope_append: rot_dim %d must be even and <= %d", rot, d);
    ROCML_REQUIRE(pairing == 0 || pairing == 1, "qk_norm_rope_append: pairing %d (0: halves, 1: neighbours)", pairing);
    ROCML_REQUIRE(!write_kv || (page_size > 0 && bt_width > 0 && block_table && kcache && vcache),
                  "qk_norm_rope_append: cache arguments missing");
    ROCML_REQUIRE(q_out || write_kv, "qk_norm_rope_append: nothing to write");
    ROCML_REQUIRE(!(span_inv && span_self), "qk_norm_rope_append: the whole-row norm's factors are given or formed here, not both");
    ROCML_REQUIRE(!(span_inv || span_self) || (n_splits == 1 && q_gain && k_gain),
                  "qk_norm_rope_append: a norm over the whole projection needs a complete projection and both gains");
    if (n_tokens == 0) return 0;
    if (span_self)      // the order of additions of qk_span_stats for these rows (see there)
        span_self = (in_dtype == ROCML_F32 && ld % 4 == 0 && (hq * d) % 4 == 0 && (hkv * d) % 4 == 0 && (uintptr_t)qkv % 16 == 0 &&
                     (!bias || (uintptr_t)bias % 16 == 0)) ? 2 : 1;
    // prompts: the values go through the transposing tile kernel, the row kernel does q and k
    bool v_tiled = write_kv && n_splits == 1 && n_tokens >= VT_TOKENS;
    // (without q_out the q rows are left to the caller: the prefill attention that reads the
    // projection prepares its queries itself)
    int first_row = q_out ? 0 : hq;
    int rows_per_token = hq - first_row + (write_kv ? (v_tiled ? hkv : 2 * hkv) : 0);
    long long rows = (long long)n_tokens * rows_per_token;
    int widest = d > dv ? d : dv;
    int per_lane = widest <= 64 ? 1 : widest <= 128 ? 2 : widest <= 256 ? 4 : 8;     // head values per lane
    // both values of a rotation pair in one lane: whole head rotated, d = per_lane * 64
    // (and the pairs are (e, e + d/2): neighbours as pairs go through LDS)
    bool local_pair = per_lane >= 2 && (rot == 0 || (rot == d && pairing == 0)) && d == per_lane * WAVE && dv == d;
    // many rows, none of them values: several rows per wave
    bool many_rows = local_pair && per_lane <= 4 && n_splits == 1 && n_tokens >= VT_TOKENS && (v_tiled || !write_kv) && !span_self;
    constexpr int MANY = 4;
    int grid = many_rows ? ceil_div(rows, QK_WAVES * MANY) : ceil_div(rows, QK_WAVES);
    size_t lds = local_pair ? 0 : (size_t)QK_WAVES * d * sizeof(float);
#define LAUNCH_N(TI, TO, N, LP)                                                                 \
    qk_norm_rope_append_kernel<TI, TO, N, LP><<<grid, EW_BLOCK, lds, stream>>>(                 \
        (const TI*)qkv, ld, n_tokens, hq, hkv, d, q_gain, k_gain, eps, cos_t, sin_t, rot,       \
        (TO*)q_out, (TO*)kcache, (TO*)vcache, block_table, bt_width, token_seq, token_pos,      \
        page_size, write_kv, n_splits, split_stride, rows_per_token, pairing, first_row, bias, dv, qt_coef, qt_every, span_inv, span_self)
#define LAUNCH_ROWS(TI, TO, N)                                                                  \
    qk_norm_rope_rows_kernel<TI, TO, N, MANY><<<grid, EW_BLOCK, 0, stream>>>(                   \
        (const TI*)qkv, ld, n_tokens, hq, hkv, d, q_gain, k_gain, eps, rot ? cos_t : nullptr,   \
        rot ? sin_t : nullptr, (TO*)q_out, (TO*)kcache, block_table, bt_width, token_seq,       \
        token_pos, page_size, rows_per_token, first_row, bias, qt_coef, qt_every, span_inv)
#define LAUNCH(TI, TO)                                                                          \
    {                                                                                           \
        if (many_rows) { if (per_lane == 2) LAUNCH_ROWS(TI, TO, 2); else LAUNCH_ROWS(TI, TO, 4); } \
        else if (per_lane == 1) LAUNCH_N(TI, TO, 1, false);                                     \
        else if (per_lane == 2) { if (local_pair) LAUNCH_N(TI, TO, 2, true); else LAUNCH_N(TI, TO, 2, false); } \
        else if (per_lane == 4) { if (local_pair) LAUNCH_N(TI, TO, 4, true); else LAUNCH_N(TI, TO, 4, false); } \
        else { if (local_pair) LAUNCH_N(TI, TO, 8, true); else LAUNCH_N(TI, TO, 8, false); }    \
        if (v_tiled) {                                                                          \
            dim3 vgrid(ceil_div(n_tokens, VT_TOKENS), hkv, ceil_div(dv, VT_VALUES));            \
            v_append_tile_kernel<TI, TO><<<vgrid, EW_BLOCK, 0, stream>>>(                       \
                (const TI*)qkv, ld, n_tokens, (hq + hkv) * d, hkv, dv, (TO*)vcache, block_table,\
                bt_width, token_seq, token_pos, page_size, bias);                               \
        }                                                                                       \
    }
    if (in_dtype == ROCML_F32 && out_dtype == ROCML_F32) LAUNCH(float, float)
    else if (in_dtype == ROCML_F32 && out_dtype == ROCML_BF16) LAUNCH(float, bf16_t)
    else if (in_dtype == ROCML_BF16 && out_dtype == ROCML_BF16) LAUNCH(bf16_t, bf16_t)
    else return rocml_fail("qk_norm_rope_append: unsupported dtype pair in=%d out=%d", in_dtype, out_dtype);
#undef LAUNCH
#undef LAUNCH_N
#undef LAUNCH_ROWS
    ROCML_CHECK_LAUNCH("qk_norm_rope_append");
    return 0;
}

// ---- factors of a norm over a token's whole q row and whole k row ---------------------------
// inv[t, 0] = 1 / sqrt(mean over the q_width leading columns of (row + bias)^2 + eps), inv[t, 1] the same over the
// k_width columns behind them.  One wave per token; 32-bit.
template <typename TI>
__global__ void __launch_bounds__(EW_BLOCK)
qk_span_stats_kernel(const TI* __restrict__ qkv, int ld, int n_tokens, int q_width, int k_width, const float* __restrict__ bias,
                     float eps, float* __restrict__ inv) {
    // a wave per token: no barrier, and all of a lane's loads are on their way together
    int lane = threadIdx.x & (WAVE - 1);
    long long t = (long long)blockIdx.x * (EW_BLOCK / WAVE) + threadIdx.x / WAVE;
    if (t >= n_tokens) return;
    const TI* row = qkv + (size_t)t * ld;
    float sq = 0.f, sk = 0.f;
    for (int i = lane; i < q_width; i += WAVE) {
        float v = Elem<TI>::load(row + i) + (bias ? bias[i] : 0.f);
        sq = fmaf(v, v, sq);
    }
    for (int i = lane; i < k_width; i += WAVE) {
        float v = Elem<TI>::load(row + q_width + i) + (bias ? bias[q_width + i] : 0.f);
        sk = fmaf(v, v, sk);
    }
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    if (lane == 0) {
        inv[(size_t)t * 2] = 1.0f / sqrtf(sq / (float)q_width + eps);
        inv[(size_t)t * 2 + 1] = 1.0f / sqrtf(sk / (float)k_width + eps);
    }
}

// The same for 32-bit rows whose q and k parts are whole 16-byte pieces.
__global__ void __launch_bounds__(EW_BLOCK)
qk_span_stats_vec_kernel(const float* __restrict__ qkv, int ld, int n_tokens, int q_width, int k_width,
                         const float* __restrict__ bias, float eps, float* __restrict__ inv) {
    int lane = threadIdx.x & (WAVE - 1);
    long long t = (long long)blockIdx.x * (EW_BLOCK / WAVE) + threadIdx.x / WAVE;
    if (t >= n_tokens) return;
    const float4* row = (const float4*)(qkv + (size_t)t * ld);
    const float4* b4 = (const float4*)bias;
    int nq = q_width / 4, nk = k_width / 4;
    float sq = 0.f, sk = 0.f;
#pragma unroll 4
    for (int i = lane; i < nq; i += WAVE) {
        float4 v = row[i];
        if (bias) { float4 b = b4[i]; v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w; }
        sq = fmaf(v.x, v.x, sq); sq = fmaf(v.y, v.y, sq); sq = fmaf(v.z, v.z, sq); sq = fmaf(v.w, v.w, sq);
    }
#pragma unroll 4
    for (int i = lane; i < nk; i += WAVE) {
        float4 v = row[nq + i];
        if (bias) { float4 b = b4[nq + i]; v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w; }
        sk = fmaf(v.x, v.x, sk); sk = fmaf(v.y, v.y, sk); sk = fmaf(v.z, v.z, sk); sk = fmaf(v.w, v.w, sk);
    }
    sq = wave_sum(sq);
    sk = wave_sum(sk);
    if (lane == 0) {
        inv[(size_t)t * 2] = 1.0f / sqrtf(sq / (float)q_width + eps);
        inv[(size_t)t * 2 + 1] = 1.0f / sqrtf(sk / (float)k_width + eps);
    }
}

ROCML_EXPORT int rocml_qk_span_stats(const void* qkv, int dtype, int ld, int n_tokens, int q_width, int k_width,
                                     const float* bias, float eps, float* inv, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && q_width > 0 && k_width > 0 && ld >= q_width + k_width && qkv && inv,
                  "qk_span_stats: bad sizes T=%d q=%d k=%d ld=%d", n_tokens, q_width, k_width, ld);
    if (n_tokens == 0) return 0;
    int grid = ceil_div(n_tokens, EW_BLOCK / WAVE);
    bool vec = dtype == ROCML_F32 && ld % 4 == 0 && q_width % 4 == 0 && k_width % 4 == 0 && (uintptr_t)qkv % 16 == 0 &&
               (!bias || (uintptr_t)bias % 16 == 0);
    if (vec)
        qk_span_stats_vec_kernel<<<grid, EW_BLOCK, 0, stream>>>((const float*)qkv, ld, n_tokens, q_width, k_width, bias, eps, inv);
    else if (dtype == ROCML_F32)
        qk_span_stats_kernel<float><<<grid, EW_BLOCK, 0, stream>>>((const float*)qkv, ld, n_tokens, q_width, k_width, bias, eps, inv);
    else if (dtype == ROCML_BF16)
        qk_span_stats_kernel<bf16_t><<<grid, EW_BLOCK, 0, stream>>>((const bf16_t*)qkv, ld, n_tokens, q_width, k_width, bias, eps, inv);
    else return rocml_fail("qk_span_stats: unknown dtype code %d", dtype);
    ROCML_CHECK_LAUNCH("qk_span_stats");
    return 0;
}

// ---- residual add ----------------------------------------------------------------
// x += y  (rocml-kernels/kernels/elementwise.hip:7-12); parts without a fused epilogue use it.
template <typename T>
__global__ void add_into_kernel(float* __restrict__ x, const T* __restrict__ y, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx < total) x[idx] += Elem<T>::load(y + idx);
}

ROCML_EXPORT int rocml_add_into(float* x, const void* y, int y_dtype, long long total,
                                hipStream_t stream) {
    ROCML_REQUIRE(total >= 0, "add_into: negative size");
    if (total == 0) return 0;
    int grid = ceil_div(total, EW_BLOCK);
    if (y_dtype == ROCML_F32) add_into_kernel<float><<<grid, EW_BLOCK, 0, stream>>>(x, (const float*)y, total);
    else if (y_dtype == ROCML_BF16) add_into_kernel<bf16_t><<<grid, EW_BLOCK, 0, stream>>>(x, (const bf16_t*)y, total);
    else return rocml_fail("add_into: unknown dtype code %d", y_dtype);
    ROCML_CHECK_LAUNCH("add_into");
    return 0;
}

// ---- a vector added to every row -------------------------------------------------
// x[t, :] += b: a projection's bias on the way into the residual stream, or a table row that a
// schedule entry adds to the stream before it runs.
__global__ void add_row_vector_kernel(float* __restrict__ x, const float* __restrict__ b, int n, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx < total) x[idx] += b[idx % n];
}

ROCML_EXPORT int rocml_add_row_vector(float* x, const float* b, int n_rows, int n, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n > 0, "add_row_vector: bad sizes rows=%d n=%d", n_rows, n);
    long long total = (long long)n_rows * n;
    if (total == 0) return 0;
    add_row_vector_kernel<<<ceil_div(total, EW_BLOCK), EW_BLOCK, 0, stream>>>(x, b, n, total);
    ROCML_CHECK_LAUNCH("add_row_vector");
    return 0;
}

// ---- latent attention: what follows the first projection ---------------------------
// A token's row of the projection holds, side by side, q_rank numbers (the query latent),
// kv_rank numbers (the key/value latent), rot_part numbers (the key part that is rotated and
// shared by the heads) and whatever else the caller projected with the same product (a gate).
// One block per token: both latents are divided by their root mean square (32-bit, eps inside the
// root) and multiplied by their gains; the query latent goes to cq_out, the key/value latent and
// the rotated key part go into the token's row of the paged cache [page, page_size, kv_rank +
// rot_part].  Rotation: pairs (i, i + dims/2) of the first `dims` numbers of the part by the
// angle in column i of the tables [T, dims/2]; the rest of the part passes unchanged.
__device__ __forceinline__ float block_sum_256(float v, float* scratch) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE] = v;
    __syncthreads();
    float r = 0.f;
#pragma unroll
    for (int w = 0; w < EW_BLOCK / WAVE; ++w) r += scratch[w];
    return r;
}

template <typename TO>
__global__ void __launch_bounds__(EW_BLOCK)
latent_prepare_kernel(const float* __restrict__ proj, int ld, int q_rank, int kv_rank, int rot_part, int dims,
                      const float* __restrict__ q_gain, const float* __restrict__ kv_gain, float eps,
                      const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                      TO* __restrict__ cq_out, TO* __restrict__ cache, const int* __restrict__ block_table,
                      int bt_width, const int* __restrict__ token_seq, const int* __restrict__ token_pos,
                      int page_size, int write_cache) {
    __shared__ float red[EW_BLOCK / WAVE];
    int t = blockIdx.x, tid = threadIdx.x;
    const float* row = proj + (size_t)t * ld;
    float sq = 0.f, sk = 0.f;
    for (int e = tid; e < q_rank; e += EW_BLOCK) sq = fmaf(row[e], row[e], sq);
    for (int e = tid; e < kv_rank; e += EW_BLOCK) sk = fmaf(row[q_rank + e], row[q_rank + e], sk);
    float inv_q = 1.0f / sqrtf(block_sum_256(sq, red) / (float)q_rank + eps);
    float inv_k = 1.0f / sqrtf(block_sum_256(sk, red) / (float)kv_rank + eps);
    for (int e = tid; e < q_rank; e += EW_BLOCK)
        Elem<TO>::store(cq_out + (size_t)t * q_rank + e, row[e] * inv_q * q_gain[e]);
    if (!write_cache) return;
    int pos = token_pos[t];
    int page = block_table[(size_t)token_seq[t] * bt_width + pos / page_size];
    if (page < 0) return;
    TO* dst = cache + ((size_t)page * page_size + pos % page_size) * (kv_rank + rot_part);
    for (int e = tid; e < kv_rank; e += EW_BLOCK)
        Elem<TO>::store(dst + e, row[q_rank + e] * inv_k * kv_gain[e]);
    const float* kr = row + q_rank + kv_rank;
    int half = dims / 2;
    for (int e = tid; e < rot_part; e += EW_BLOCK) {
        float v = kr[e];
        if (e < half) {
            float c = cos_t[(size_t)t * half + e], s = sin_t[(size_t)t * half + e];
            v = kr[e] * c - kr[e + half] * s;
        } else if (e < dims) {
            float c = cos_t[(size_t)t * half + e - half], s = sin_t[(size_t)t * half + e - half];
            v = kr[e] * c + kr[e - half] * s;
        }
        Elem<TO>::store(dst + kv_rank + e, v);
    }
}

ROCML_EXPORT int rocml_latent_prepare(const float* proj, int ld, int n_tokens, int q_rank, int kv_rank, int rot_part,
                                      int dims, const float* q_gain, const float* kv_gain, float eps,
                                      const float* cos_t, const float* sin_t, void* cq_out, void* cache,
                                      int out_dtype, const int* block_table, int bt_width, const int* token_seq,
                                      const int* token_pos, int page_size, int write_cache, hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && q_rank > 0 && kv_rank > 0 && rot_part >= 0 && dims >= 0 && dims % 2 == 0 && dims <= rot_part,
                  "latent_prepare: bad sizes T=%d q_rank=%d kv_rank=%d rotated part=%d of which %d turn", n_tokens,
                  q_rank, kv_rank, rot_part, dims);
    ROCML_REQUIRE(ld >= q_rank + kv_rank + rot_part, "latent_prepare: rows of %d numbers, %d are needed", ld,
                  q_rank + kv_rank + rot_part);
    ROCML_REQUIRE(q_gain && kv_gain && cq_out && (dims == 0 || (cos_t && sin_t)), "latent_prepare: gains, tables or output missing");
    ROCML_REQUIRE(!write_cache || (cache && block_table && bt_width > 0 && page_size > 0 && token_seq && token_pos),
                  "latent_prepare: cache arguments missing");
    if (n_tokens == 0) return 0;
#define LAUNCH(TO)                                                                                              \
    latent_prepare_kernel<TO><<<n_tokens, EW_BLOCK, 0, stream>>>(proj, ld, q_rank, kv_rank, rot_part, dims,    \
        q_gain, kv_gain, eps, cos_t, sin_t, (TO*)cq_out, (TO*)cache, block_table, bt_width, token_seq,         \
        token_pos, page_size, write_cache)
    if (out_dtype == ROCML_F32) LAUNCH(float);
    else if (out_dtype == ROCML_BF16) LAUNCH(bf16_t);
    else return rocml_fail("latent_prepare: unknown dtype code %d", out_dtype);
#undef LAUNCH
    ROCML_CHECK_LAUNCH("latent_prepare");
    return 0;
}

// The rotated part of every query head: q [T, ldq] holds, per head, head_stride numbers of which
// those from `offset` on, rot_part of them, are the part; its rotation (as above) goes to
// out [T, ldo] at out_offset of each head's out_stride numbers.
// lead: so many numbers before the part are copied unchanged in front of it (out_offset is where they start).
template <typename TO>
__global__ void rope_heads_kernel(const float* __restrict__ q, int ldq, int head_stride, int offset, int rot_part,
                                  int dims, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                  TO* __restrict__ out, int ldo, int out_stride, int out_offset, int n_heads,
                                  int lead, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    int width = lead + rot_part;
    int e = (int)(idx % width) - lead;
    long long th = idx / width;
    int h = (int)(th % n_heads);
    long long t = th / n_heads;
    const float* src = q + (size_t)t * ldq + (size_t)h * head_stride + offset;
    if (e < 0) {
        Elem<TO>::store(out + (size_t)t * ldo + (size_t)h * out_stride + out_offset + lead + e, src[e]);
        return;
    }
    int half = dims / 2;
    float v = src[e];
    if (e < half) {
        v = src[e] * cos_t[t * half + e] - src[e + half] * sin_t[t * half + e];
    } else if (e < dims) {
        v = src[e] * cos_t[t * half + e - half] + src[e - half] * sin_t[t * half + e - half];
    }
    Elem<TO>::store(out + (size_t)t * ldo + (size_t)h * out_stride + out_offset + lead + e, v);
}

ROCML_EXPORT int rocml_rope_heads(const float* q, int ldq, int head_stride, int offset, int rot_part, int dims,
                                  const float* cos_t, const float* sin_t, void* out, int out_dtype, int ldo,
                                  int out_stride, int out_offset, int n_tokens, int n_heads, int lead,
                                  hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && n_heads > 0 && rot_part >= 0 && dims >= 0 && dims % 2 == 0 && dims <= rot_part,
                  "rope_heads: bad sizes T=%d H=%d part=%d dims=%d", n_tokens, n_heads, rot_part, dims);
    ROCML_REQUIRE(lead >= 0 && offset >= lead && offset + rot_part <= head_stride && ldq >= n_heads * head_stride &&
                      out_offset >= 0 && out_offset + lead + rot_part <= out_stride && ldo >= n_heads * out_stride,
                  "rope_heads: the part (and what is copied before it) does not lie inside the heads");
    ROCML_REQUIRE(dims == 0 || (cos_t && sin_t), "rope_heads: rotation tables missing");
    long long total = (long long)n_tokens * n_heads * (lead + rot_part);
    if (total == 0) return 0;
    int grid = ceil_div(total, EW_BLOCK);
    if (out_dtype == ROCML_F32)
        rope_heads_kernel<float><<<grid, EW_BLOCK, 0, stream>>>(q, ldq, head_stride, offset, rot_part, dims, cos_t, sin_t,
                                                                (float*)out, ldo, out_stride, out_offset, n_heads, lead, total);
    else if (out_dtype == ROCML_BF16)
        rope_heads_kernel<bf16_t><<<grid, EW_BLOCK, 0, stream>>>(q, ldq, head_stride, offset, rot_part, dims, cos_t, sin_t,
                                                                 (bf16_t*)out, ldo, out_stride, out_offset, n_heads, lead, total);
    else return rocml_fail("rope_heads: unknown dtype code %d", out_dtype);
    ROCML_CHECK_LAUNCH("rope_heads");
    return 0;
}

// y[t, i] = y[t, i] * sigmoid(g[t, i / group]) with g 32-bit in rows of ldg numbers: an output gate,
// one number per value (group = 1) or one per run of `group` values (a head).
template <typename T>
__global__ void sigmoid_gate_kernel(T* __restrict__ y, const float* __restrict__ g, int ldg, int n, int group, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    long long t = idx / n;
    int i = (int)(idx - t * n);
    float gate = 1.0f / (1.0f + expf(-g[(size_t)t * ldg + i / group]));
    Elem<T>::store(y + idx, Elem<T>::load(y + idx) * gate);
}

ROCML_EXPORT int rocml_sigmoid_gate(void* y, int dtype, const float* g, int ldg, int n_rows, int n, int group, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n > 0 && group > 0 && n % group == 0 && ldg >= n / group,
                  "sigmoid_gate: bad sizes rows=%d n=%d group=%d ld=%d", n_rows, n, group, ldg);
    long long total = (long long)n_rows * n;
    if (total == 0) return 0;
    int grid = ceil_div(total, EW_BLOCK);
    if (dtype == ROCML_F32) sigmoid_gate_kernel<float><<<grid, EW_BLOCK, 0, stream>>>((float*)y, g, ldg, n, group, total);
    else if (dtype == ROCML_BF16) sigmoid_gate_kernel<bf16_t><<<grid, EW_BLOCK, 0, stream>>>((bf16_t*)y, g, ldg, n, group, total);
    else return rocml_fail("sigmoid_gate: unknown dtype code %d", dtype);
    ROCML_CHECK_LAUNCH("sigmoid_gate");
    return 0;
}

// ---- latent attention, prompts: the rows a step's queries can see, as a dense matrix ---------
// A prompt step may expand keys and values per head for the positions its queries see (the step's own
// tokens and up to window - 1 cached ones per sequence) and run the attention kernels for separate
// heads over them.  The positions of sequence b are [lo_b, end_b), lo_b = max(0, start_b - window + 1)
// (0 without a window); they lie in the sequence's pages fp_b .. lp_b, which get scratch pages
// base_b .. in sequence order.  latent_window_plan (one block) writes the scratch block table
// [n_seqs, width] (page index of the sequence -> scratch page, -1 elsewhere) and, per scratch page, the
// latent pool page it mirrors, its first position and the range of positions that count; latent_window_gather
// copies the rows (zeros where a position does not count) into rows [scratch page * 64 + place].
__global__ void latent_window_plan_kernel(const int* __restrict__ cu_seqlens, const int* __restrict__ token_pos,
                                          const int* __restrict__ block_table, int bt_width, int n_seqs, int window,
                                          int page_size, int* __restrict__ table, int width, int* __restrict__ src_page,
                                          int* __restrict__ first_pos, int* __restrict__ lo_pos, int* __restrict__ hi_pos,
                                          int max_pages) {
    extern __shared__ int plan_smem[];      // [n_seqs] base, [n_seqs] first page, [n_seqs] count
    int* base = plan_smem;
    int* fpage = plan_smem + n_seqs;
    int* count = plan_smem + 2 * n_seqs;
    if (threadIdx.x == 0) {
        int at = 0;
        for (int b = 0; b < n_seqs; ++b) {
            int start = token_pos[cu_seqlens[b]], end = start + cu_seqlens[b + 1] - cu_seqlens[b];
            int lo = window > 0 ? max(0, start - window + 1) : 0;
            fpage[b] = lo / page_size;
            count[b] = (end - 1) / page_size - fpage[b] + 1;
            base[b] = at;
            at += count[b];
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < max_pages; i += blockDim.x) src_page[i] = -1;
    for (int i = threadIdx.x; i < n_seqs * width; i += blockDim.x) table[i] = -1;
    __syncthreads();
    for (int b = 0; b < n_seqs; ++b) {
        int start = token_pos[cu_seqlens[b]], end = start + cu_seqlens[b + 1] - cu_seqlens[b];
        int lo = window > 0 ? max(0, start - window + 1) : 0;
        for (int i = threadIdx.x; i < count[b]; i += blockDim.x) {
            int p = fpage[b] + i, s = base[b] + i;
            if (s >= max_pages || p >= width || p >= bt_width) continue;
            table[(size_t)b * width + p] = s;
            src_page[s] = block_table[(size_t)b * bt_width + p];
            first_pos[s] = p * page_size;
            lo_pos[s] = lo;
            hi_pos[s] = end;
        }
    }
}

template <typename T>
__global__ void latent_window_gather_kernel(const T* __restrict__ cache, int row, int page_size,
                                            const int* __restrict__ src_page, const int* __restrict__ first_pos,
                                            const int* __restrict__ lo_pos, const int* __restrict__ hi_pos,
                                            T* __restrict__ out, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    int e = (int)(idx % row);
    long long r = idx / row;
    int s = (int)(r / page_size), i = (int)(r % page_size);
    int page = src_page[s];
    T v = 0;
    if (page >= 0) {
        int pos = first_pos[s] + i;
        if (pos >= lo_pos[s] && pos < hi_pos[s]) v = cache[((size_t)page * page_size + i) * row + e];
    }
    out[idx] = v;
}

ROCML_EXPORT int rocml_latent_window_plan(const int* cu_seqlens, const int* token_pos, const int* block_table, int bt_width,
                                          int n_seqs, int window, int page_size, int* table, int width, int* plan,
                                          int max_pages, hipStream_t stream) {
    // plan: 4 * max_pages ints (source page, first position, first and one past the last position that count)
    ROCML_REQUIRE(n_seqs > 0 && n_seqs <= 4096 && bt_width > 0 && width > 0 && max_pages > 0 && page_size > 0 && window >= 0,
                  "latent_window_plan: bad sizes sequences=%d width=%d pages=%d", n_seqs, width, max_pages);
    latent_window_plan_kernel<<<1, 256, 3 * n_seqs * sizeof(int), stream>>>(
        cu_seqlens, token_pos, block_table, bt_width, n_seqs, window, page_size, table, width, plan, plan + max_pages,
        plan + 2 * max_pages, plan + 3 * max_pages, max_pages);
    ROCML_CHECK_LAUNCH("latent_window_plan");
    return 0;
}

ROCML_EXPORT int rocml_latent_window_gather(const void* cache, int dtype, int row, int page_size, const int* plan,
                                            int max_pages, void* out, hipStream_t stream) {
    ROCML_REQUIRE(row > 0 && page_size > 0 && max_pages > 0, "latent_window_gather: bad sizes");
    long long total = (long long)max_pages * page_size * row;
    int grid = ceil_div(total, EW_BLOCK);
    if (dtype == ROCML_BF16)
        latent_window_gather_kernel<bf16_t><<<grid, EW_BLOCK, 0, stream>>>((const bf16_t*)cache, row, page_size, plan,
            plan + max_pages, plan + 2 * max_pages, plan + 3 * max_pages, (bf16_t*)out, total);
    else if (dtype == ROCML_F32)
        latent_window_gather_kernel<float><<<grid, EW_BLOCK, 0, stream>>>((const float*)cache, row, page_size, plan,
            plan + max_pages, plan + 2 * max_pages, plan + 3 * max_pages, (float*)out, total);
    else return rocml_fail("latent_window_gather: unknown dtype code %d", dtype);
    ROCML_CHECK_LAUNCH("latent_window_gather");
    return 0;
}

// out[t, h * n + i] = x[t, h * x_stride + i] * sigmoid(g[t, h * n + i]) (g null: a plain copy of the heads'
// leading n numbers): the heads of an attention output that is wider than the values, gated and packed.
template <typename T>
__global__ void gate_heads_kernel(const T* __restrict__ x, int ldx, int x_stride, const float* __restrict__ g, int ldg,
                                  T* __restrict__ out, int n_heads, int n, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    int i = (int)(idx % n);
    long long th = idx / n;
    int h = (int)(th % n_heads);
    long long t = th / n_heads;
    float v = Elem<T>::load(x + (size_t)t * ldx + (size_t)h * x_stride + i);
    if (g) v *= 1.0f / (1.0f + expf(-g[(size_t)t * ldg + (size_t)h * n + i]));
    Elem<T>::store(out + idx, v);
}

ROCML_EXPORT int rocml_gate_heads(const void* x, int dtype, int ldx, int x_stride, const float* g, int ldg, void* out,
                                  int n_rows, int n_heads, int n, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n_heads > 0 && n > 0 && n <= x_stride && ldx >= n_heads * x_stride && (!g || ldg >= n_heads * n),
                  "gate_heads: bad sizes rows=%d heads=%d n=%d stride=%d", n_rows, n_heads, n, x_stride);
    long long total = (long long)n_rows * n_heads * n;
    if (total == 0) return 0;
    int grid = ceil_div(total, EW_BLOCK);
    if (dtype == ROCML_F32) gate_heads_kernel<float><<<grid, EW_BLOCK, 0, stream>>>((const float*)x, ldx, x_stride, g, ldg, (float*)out, n_heads, n, total);
    else if (dtype == ROCML_BF16) gate_heads_kernel<bf16_t><<<grid, EW_BLOCK, 0, stream>>>((const bf16_t*)x, ldx, x_stride, g, ldg, (bf16_t*)out, n_heads, n, total);
    else return rocml_fail("gate_heads: unknown dtype code %d", dtype);
    ROCML_CHECK_LAUNCH("gate_heads");
    return 0;
}

// ---- norm after the sum ----------------------------------------------------------
// x[t, :] <- rms(alpha * x[t, :] + c * sum_b f_b(y_b[t, :])) * gain (without a gain: the sum
// itself, not normed), all in 32-bit, with
// f_b(y) = y / sqrt(mean(y^2) + eps) * gain_b for a branch with a gain and f_b(y) = y without.
// It is the layer wiring "the sublayer reads the stream, the norm comes after the sum", and with two
// or more branches also the sum of sublayers that ran side by side on the same input, each normed
// over the width first.  x is rewritten in place; `copy` (may be null) gets the new x in another
// type, for the products that read it next.  One block per row.
constexpr int SN_MAX_BRANCHES = 4;
struct SumNormBranches {
    const float* y[SN_MAX_BRANCHES];
    const float* gain[SN_MAX_BRANCHES];
    int n;
};

template <typename TC>
__global__ void __launch_bounds__(EW_BLOCK)
sum_norm_kernel(float* __restrict__ x, SumNormBranches br, float alpha, float c, const float* __restrict__ gain,
                float eps, int n, TC* __restrict__ copy) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    size_t row = (size_t)blockIdx.x * n;
    float inv[SN_MAX_BRANCHES];
#pragma unroll
    for (int b = 0; b < SN_MAX_BRANCHES; ++b) {
        inv[b] = 1.f;
        if (b < br.n && br.gain[b]) {
            float ss = 0.f;
            for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
                float v = br.y[b][row + i];
                ss = fmaf(v, v, ss);
            }
            inv[b] = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
        }
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
        float sum = 0.f;
#pragma unroll
        for (int b = 0; b < SN_MAX_BRANCHES; ++b)
            if (b < br.n) {
                float v = br.y[b][row + i];
                sum += br.gain[b] ? v * inv[b] * br.gain[b][i] : v;
            }
        float s = alpha != 0.f ? fmaf(alpha, x[row + i], c * sum) : c * sum;      // alpha = 0: x is not read
        x[row + i] = s;
        ss = fmaf(s, s, ss);
    }
    if (!gain && !copy) return;
    float r = gain ? 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps) : 1.f;
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) {       // a thread reads back what it wrote itself
        float v = gain ? x[row + i] * r * gain[i] : x[row + i];
        x[row + i] = v;
        if (copy) Elem<TC>::store(copy + row + i, v);
    }
}

// The same for rows of up to 8192 values that are a multiple of 4 and at most two branches: the row and
// the branches stay in registers and all loads are issued at once (a decode step's few rows would
// otherwise wait for one load after the other, pass after pass).
template <typename TC, int VEC, int NB>
__global__ void __launch_bounds__(EW_BLOCK)
sum_norm_vec_kernel(float* __restrict__ x, SumNormBranches br, float alpha, float c, const float* __restrict__ gain,
                    float eps, int n, TC* __restrict__ copy) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    size_t row = (size_t)blockIdx.x * n;
    int nv = n / 4;
    float4 xv[VEC], yv[NB][VEC], gv[NB][VEC], fg[VEC];
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        int i = threadIdx.x + j * EW_BLOCK;
        bool ok = i < nv;
        xv[j] = (ok && alpha != 0.f) ? ((const float4*)(x + row))[i] : zero4;
        fg[j] = (ok && gain) ? ((const float4*)gain)[i] : zero4;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            yv[b][j] = ok ? ((const float4*)(br.y[b] + row))[i] : zero4;
            gv[b][j] = (ok && br.gain[b]) ? ((const float4*)br.gain[b])[i] : zero4;
        }
    }
    float inv[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        inv[b] = 1.f;
        if (br.gain[b]) {
            float ss = 0.f;
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                ss = fmaf(yv[b][j].x, yv[b][j].x, ss); ss = fmaf(yv[b][j].y, yv[b][j].y, ss);
                ss = fmaf(yv[b][j].z, yv[b][j].z, ss); ss = fmaf(yv[b][j].w, yv[b][j].w, ss);
            }
            inv[b] = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        float4 sum = zero4;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            float4 v = yv[b][j];
            if (br.gain[b]) {
                sum.x += v.x * inv[b] * gv[b][j].x; sum.y += v.y * inv[b] * gv[b][j].y;
                sum.z += v.z * inv[b] * gv[b][j].z; sum.w += v.w * inv[b] * gv[b][j].w;
            } else {
                sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
            }
        }
        float4 sv;
        sv.x = alpha != 0.f ? fmaf(alpha, xv[j].x, c * sum.x) : c * sum.x;
        sv.y = alpha != 0.f ? fmaf(alpha, xv[j].y, c * sum.y) : c * sum.y;
        sv.z = alpha != 0.f ? fmaf(alpha, xv[j].z, c * sum.z) : c * sum.z;
        sv.w = alpha != 0.f ? fmaf(alpha, xv[j].w, c * sum.w) : c * sum.w;
        xv[j] = sv;
        ss = fmaf(sv.x, sv.x, ss); ss = fmaf(sv.y, sv.y, ss); ss = fmaf(sv.z, sv.z, ss); ss = fmaf(sv.w, sv.w, ss);
    }
    float r = gain ? 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps) : 1.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        int i = threadIdx.x + j * EW_BLOCK;
        if (i >= nv) continue;
        float4 v = xv[j];
        if (gain) { v.x *= r * fg[j].x; v.y *= r * fg[j].y; v.z *= r * fg[j].z; v.w *= r * fg[j].w; }
        ((float4*)(x + row))[i] = v;
        if (copy) store4(copy + row + 4 * (size_t)i, v.x, v.y, v.z, v.w);
    }
}

template <typename TC>
static bool launch_sum_norm_vec(float* x, const SumNormBranches& br, float alpha, float c, const float* gain, float eps, int n,
                                TC* copy, int n_rows, hipStream_t stream) {
    int vec = ceil_div(n / 4, EW_BLOCK);
#define SNV(V_, NB_) sum_norm_vec_kernel<TC, V_, NB_><<<n_rows, EW_BLOCK, 0, stream>>>(x, br, alpha, c, gain, eps, n, copy)
#define SNV_BY_NB(V_) { if (br.n == 1) SNV(V_, 1); else SNV(V_, 2); }
    if (vec <= 1) SNV_BY_NB(1)
    else if (vec <= 2) SNV_BY_NB(2)
    else if (vec <= 4) SNV_BY_NB(4)
    else SNV_BY_NB(8)
#undef SNV_BY_NB
#undef SNV
    return true;
}

ROCML_EXPORT int rocml_sum_norm(float* x, int n_rows, int n, float alpha, float c, int n_branches,
                                const float* const* ys, const float* const* gains, const float* gain, float eps,
                                void* copy, int copy_dtype, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n > 0, "sum_norm: bad sizes rows=%d n=%d", n_rows, n);
    ROCML_REQUIRE(n_branches >= 1 && n_branches <= SN_MAX_BRANCHES, "sum_norm: %d branches (1 to %d)", n_branches, SN_MAX_BRANCHES);
    ROCML_REQUIRE(x && ys && gains, "sum_norm: missing arguments");
    if (n_rows == 0) return 0;
    SumNormBranches br{};
    br.n = n_branches;
    for (int b = 0; b < n_branches; ++b) {
        ROCML_REQUIRE(ys[b], "sum_norm: branch %d has no values", b);
        br.y[b] = ys[b];
        br.gain[b] = gains[b];
    }
    ROCML_REQUIRE(!copy || copy_dtype == ROCML_F32 || copy_dtype == ROCML_BF16, "sum_norm: unknown dtype code %d", copy_dtype);
    if (n % 4 == 0 && n <= 4 * EW_BLOCK * RN_MAX_VEC && n_branches <= 2) {
        if (!copy || copy_dtype == ROCML_F32) launch_sum_norm_vec<float>(x, br, alpha, c, gain, eps, n, (float*)copy, n_rows, stream);
        else launch_sum_norm_vec<bf16_t>(x, br, alpha, c, gain, eps, n, (bf16_t*)copy, n_rows, stream);
        ROCML_CHECK_LAUNCH("sum_norm");
        return 0;
    }
    if (!copy || copy_dtype == ROCML_F32)
        sum_norm_kernel<float><<<n_rows, EW_BLOCK, 0, stream>>>(x, br, alpha, c, gain, eps, n, (float*)copy);
    else if (copy_dtype == ROCML_BF16)
        sum_norm_kernel<bf16_t><<<n_rows, EW_BLOCK, 0, stream>>>(x, br, alpha, c, gain, eps, n, (bf16_t*)copy);
    else return rocml_fail("sum_norm: unknown dtype code %d", copy_dtype);
    ROCML_CHECK_LAUNCH("sum_norm");
    return 0;
}

// ---- norm of a sublayer's output, added to the stream ------------------------------------------
// x[t, :] += f(y[t, :]) in 32-bit, f a layer norm, (y - mean) / sqrt(var + eps) * gain + bias with var the mean
// of the squared deviations from the mean (LAYER), or y / sqrt(mean(y^2) + eps) * gain; `copy` (may be null) gets
// the new x in another type, for the products that read it next; with next_gain it gets the root-mean-square norm
// of the new x instead, x / sqrt(mean(x^2) + next_eps) * next_gain: the norm that reads the stream next.  One block per row.
template <typename TC, bool LAYER>
__global__ void __launch_bounds__(EW_BLOCK)
norm_add_kernel(float* __restrict__ x, float* __restrict__ y, const float* __restrict__ gain,
                const float* __restrict__ bias, float eps, int n, TC* __restrict__ copy,
                const float* __restrict__ partials, int n_splits, long long split_stride, int replace,
                const float* __restrict__ next_gain, float next_eps) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    size_t row = (size_t)blockIdx.x * n;
    if (n_splits > 0) {         // y (or nothing) plus the K pieces in split order, written back: a thread reads back its own
        for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
            float v = replace ? 0.f : y[row + i];
            for (int sp = 0; sp < n_splits; ++sp) v += partials[sp * split_stride + row + i];
            y[row + i] = v;
        }
    }
    float mean = 0.f;
    if (LAYER) {
        float s = 0.f;
        for (int i = threadIdx.x; i < n; i += EW_BLOCK) s += y[row + i];
        mean = block_sum(s, scratch) / (float)n;
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
        float d = y[row + i] - mean;
        ss = fmaf(d, d, ss);
    }
    float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
        float v = (y[row + i] - mean) * inv * gain[i];
        if (LAYER && bias) v += bias[i];
        v += x[row + i];
        x[row + i] = v;
        if (copy && !next_gain) Elem<TC>::store(copy + row + i, v);
    }
    if (copy && next_gain) {        // (a thread reads back what it wrote itself)
        float s2 = 0.f;
        for (int i = threadIdx.x; i < n; i += EW_BLOCK) s2 = fmaf(x[row + i], x[row + i], s2);
        float inv2 = 1.0f / sqrtf(block_sum(s2, scratch) / (float)n + next_eps);
        for (int i = threadIdx.x; i < n; i += EW_BLOCK) Elem<TC>::store(copy + row + i, x[row + i] * inv2 * next_gain[i]);
    }
}

// The same for rows of up to 8192 values that are a multiple of 4: the row stays in registers and all
// loads are issued at once.
template <typename TC, bool LAYER, int VEC>
__global__ void __launch_bounds__(EW_BLOCK)
norm_add_vec_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ gain,
                    const float* __restrict__ bias, float eps, int n, TC* __restrict__ copy,
                    const float* __restrict__ partials, int n_splits, long long split_stride, int replace,
                    const float* __restrict__ next_gain, float next_eps) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    size_t row = (size_t)blockIdx.x * n;
    int nv = n / 4;
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 yv[VEC], xv[VEC], gv[VEC], bv[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        int i = threadIdx.x + j * EW_BLOCK;
        bool ok = i < nv;
        yv[j] = (ok && !replace) ? ((const float4*)(y + row))[i] : zero4;
        xv[j] = ok ? ((const float4*)(x + row))[i] : zero4;
        gv[j] = ok ? ((const float4*)gain)[i] : zero4;
        bv[j] = (ok && LAYER && bias) ? ((const float4*)bias)[i] : zero4;
    }
    // the K pieces of the product that made y, in split order
    for (int sp = 0; sp < n_splits; ++sp) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            int i = threadIdx.x + j * EW_BLOCK;
            if (i < nv) {
                float4 p = ((const float4*)(partials + sp * split_stride + row))[i];
                yv[j].x += p.x; yv[j].y += p.y; yv[j].z += p.z; yv[j].w += p.w;
            }
        }
    }
    float mean = 0.f;
    if (LAYER) {
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) s += (yv[j].x + yv[j].y) + (yv[j].z + yv[j].w);
        mean = block_sum(s, scratch) / (float)n;
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        if (threadIdx.x + j * EW_BLOCK < nv) {
            yv[j].x -= mean; yv[j].y -= mean; yv[j].z -= mean; yv[j].w -= mean;
        }
        ss = fmaf(yv[j].x, yv[j].x, ss); ss = fmaf(yv[j].y, yv[j].y, ss);
        ss = fmaf(yv[j].z, yv[j].z, ss); ss = fmaf(yv[j].w, yv[j].w, ss);
    }
    float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        int i = threadIdx.x + j * EW_BLOCK;
        if (i >= nv) continue;
        float4 v;
        v.x = xv[j].x + (yv[j].x * inv * gv[j].x + bv[j].x);
        v.y = xv[j].y + (yv[j].y * inv * gv[j].y + bv[j].y);
        v.z = xv[j].z + (yv[j].z * inv * gv[j].z + bv[j].z);
        v.w = xv[j].w + (yv[j].w * inv * gv[j].w + bv[j].w);
        ((float4*)(x + row))[i] = v;
        if (copy && !next_gain) store4(copy + row + 4 * (size_t)i, v.x, v.y, v.z, v.w);
        xv[j] = v;
    }
    if (copy && next_gain) {        // the norm that reads the stream next, from the row in registers
        float s2 = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            if (threadIdx.x + j * EW_BLOCK >= nv) continue;
            s2 = fmaf(xv[j].x, xv[j].x, s2); s2 = fmaf(xv[j].y, xv[j].y, s2);
            s2 = fmaf(xv[j].z, xv[j].z, s2); s2 = fmaf(xv[j].w, xv[j].w, s2);
        }
        float inv2 = 1.0f / sqrtf(block_sum(s2, scratch) / (float)n + next_eps);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            int i = threadIdx.x + j * EW_BLOCK;
            if (i >= nv) continue;
            float4 g2 = ((const float4*)next_gain)[i];
            store4(copy + row + 4 * (size_t)i, xv[j].x * inv2 * g2.x, xv[j].y * inv2 * g2.y, xv[j].z * inv2 * g2.z, xv[j].w * inv2 * g2.w);
        }
    }
}

template <typename TC, bool LAYER>
static void launch_norm_add(float* x, float* y, const float* gain, const float* bias, float eps, int n_rows, int n,
                            TC* copy, const float* partials, int n_splits, long long split_stride, int replace,
                            const float* next_gain, float next_eps, hipStream_t stream) {
    bool vec = n % 4 == 0 && n <= 4 * EW_BLOCK * RN_MAX_VEC && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0 &&
               (uintptr_t)gain % 16 == 0 && (!bias || (uintptr_t)bias % 16 == 0) && (!copy || (uintptr_t)copy % 8 == 0) &&
               (!next_gain || (uintptr_t)next_gain % 16 == 0) &&
               (n_splits == 0 || ((uintptr_t)partials % 16 == 0 && split_stride % 4 == 0));
    int v = ceil_div(n / 4, EW_BLOCK);
#define NAV(V_) norm_add_vec_kernel<TC, LAYER, V_><<<n_rows, EW_BLOCK, 0, stream>>>(x, y, gain, bias, eps, n, copy, partials, n_splits, split_stride, replace, next_gain, next_eps)
    if (!vec) norm_add_kernel<TC, LAYER><<<n_rows, EW_BLOCK, 0, stream>>>(x, y, gain, bias, eps, n, copy, partials, n_splits, split_stride, replace, next_gain, next_eps);
    else if (v <= 1) NAV(1);
    else if (v <= 2) NAV(2);
    else if (v <= 4) NAV(4);
    else NAV(8);
#undef NAV
}

// The same with the sublayer's output still in branches: y = c * sum_b y_b / sqrt(mean(y_b^2) + eps_b) * gain_b (one or two
// mixers that ran side by side, each normed over the width with a gain of its own) is formed in registers, in the
// order of operations of sum_norm, and normed and added as above.  Rows of up to 4096 values that are multiples of 4.
template <typename TC, bool LAYER, int VEC>
__global__ void __launch_bounds__(EW_BLOCK)
norm_add_branches_vec_kernel(float* __restrict__ x, const float* __restrict__ y0, const float* __restrict__ y1,
                             const float* __restrict__ g0, const float* __restrict__ g1, float c, float eps_b,
                             const float* __restrict__ gain, const float* __restrict__ bias, float eps, int n,
                             TC* __restrict__ copy) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    size_t row = (size_t)blockIdx.x * n;
    int nv = n / 4;
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 av[VEC], bv2[VEC], ga[VEC], gb[VEC], xv[VEC], gv[VEC], bv[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        int i = threadIdx.x + j * EW_BLOCK;
        bool ok = i < nv;
        av[j] = ok ? ((const float4*)(y0 + row))[i] : zero4;
        ga[j] = ok ? ((const float4*)g0)[i] : zero4;
        bv2[j] = (ok && y1) ? ((const float4*)(y1 + row))[i] : zero4;
        gb[j] = (ok && y1) ? ((const float4*)g1)[i] : zero4;
        xv[j] = ok ? ((const float4*)(x + row))[i] : zero4;
        gv[j] = ok ? ((const float4*)gain)[i] : zero4;
        bv[j] = (ok && LAYER && bias) ? ((const float4*)bias)[i] : zero4;
    }
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        s0 = fmaf(av[j].x, av[j].x, s0); s0 = fmaf(av[j].y, av[j].y, s0); s0 = fmaf(av[j].z, av[j].z, s0); s0 = fmaf(av[j].w, av[j].w, s0);
        s1 = fmaf(bv2[j].x, bv2[j].x, s1); s1 = fmaf(bv2[j].y, bv2[j].y, s1); s1 = fmaf(bv2[j].z, bv2[j].z, s1); s1 = fmaf(bv2[j].w, bv2[j].w, s1);
    }
    float inv0 = 1.0f / sqrtf(block_sum(s0, scratch) / (float)n + eps_b);
    float inv1 = y1 ? 1.0f / sqrtf(block_sum(s1, scratch) / (float)n + eps_b) : 0.f;
    float4 yv[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        float4 sum;
        sum.x = av[j].x * inv0 * ga[j].x; sum.y = av[j].y * inv0 * ga[j].y; sum.z = av[j].z * inv0 * ga[j].z; sum.w = av[j].w * inv0 * ga[j].w;
        if (y1) {
            sum.x += bv2[j].x * inv1 * gb[j].x; sum.y += bv2[j].y * inv1 * gb[j].y;
            sum.z += bv2[j].z * inv1 * gb[j].z; sum.w += bv2[j].w * inv1 * gb[j].w;
        }
        yv[j] = make_float4(c * sum.x, c * sum.y, c * sum.z, c * sum.w);
    }
    float mean = 0.f;
    if (LAYER) {
        float sm = 0.f;
#pragma unroll
        for (int j = 0; j < VEC; ++j) sm += (yv[j].x + yv[j].y) + (yv[j].z + yv[j].w);
        mean = block_sum(sm, scratch) / (float)n;
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        if (threadIdx.x + j * EW_BLOCK < nv) {
            yv[j].x -= mean; yv[j].y -= mean; yv[j].z -= mean; yv[j].w -= mean;
        }
        ss = fmaf(yv[j].x, yv[j].x, ss); ss = fmaf(yv[j].y, yv[j].y, ss);
        ss = fmaf(yv[j].z, yv[j].z, ss); ss = fmaf(yv[j].w, yv[j].w, ss);
    }
    float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        int i = threadIdx.x + j * EW_BLOCK;
        if (i >= nv) continue;
        float4 v;
        v.x = xv[j].x + (yv[j].x * inv * gv[j].x + bv[j].x);
        v.y = xv[j].y + (yv[j].y * inv * gv[j].y + bv[j].y);
        v.z = xv[j].z + (yv[j].z * inv * gv[j].z + bv[j].z);
        v.w = xv[j].w + (yv[j].w * inv * gv[j].w + bv[j].w);
        ((float4*)(x + row))[i] = v;
        if (copy) store4(copy + row + 4 * (size_t)i, v.x, v.y, v.z, v.w);
    }
}

constexpr int NAB_MAX_N = 4 * EW_BLOCK * 4;      // the widest row the kernel above keeps in registers

ROCML_EXPORT int rocml_norm_add_branches_fits(int n) { return n > 0 && n % 4 == 0 && n <= NAB_MAX_N; }

template <typename TC, bool LAYER>
static void launch_norm_add_branches(float* x, const float* y0, const float* y1, const float* g0, const float* g1, float c,
                                     float eps_b, const float* gain, const float* bias, float eps, int n_rows, int n, TC* copy,
                                     hipStream_t stream) {
    int v = ceil_div(n / 4, EW_BLOCK);
#define NAB(V_) norm_add_branches_vec_kernel<TC, LAYER, V_><<<n_rows, EW_BLOCK, 0, stream>>>(x, y0, y1, g0, g1, c, eps_b, gain, bias, eps, n, copy)
    if (v <= 1) NAB(1);
    else if (v <= 2) NAB(2);
    else NAB(4);
#undef NAB
}

ROCML_EXPORT int rocml_norm_add_branches(float* x, const float* y0, const float* y1, const float* g0, const float* g1,
                                         float c, float eps_b, int n_rows, int n, const float* gain, const float* bias,
                                         float eps, int layer, void* copy, int copy_dtype, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && x && y0 && g0 && gain && (!y1 || g1), "norm_add_branches: missing arguments");
    ROCML_REQUIRE(rocml_norm_add_branches_fits(n), "norm_add_branches: rows of %d values (a multiple of 4, at most %d)", n, NAB_MAX_N);
    ROCML_REQUIRE(!copy || copy_dtype == ROCML_F32 || copy_dtype == ROCML_BF16, "norm_add_branches: unknown dtype code %d", copy_dtype);
    const void* ptrs[] = {x, y0, y1, g0, g1, gain, bias};
    for (const void* q : ptrs) ROCML_REQUIRE((uintptr_t)q % 16 == 0, "norm_add_branches: operands must start on 16 bytes");
    ROCML_REQUIRE(!copy || (uintptr_t)copy % 8 == 0, "norm_add_branches: the copy must start on 8 bytes");
    if (n_rows == 0) return 0;
    bool half = copy && copy_dtype == ROCML_BF16;
    if (layer) {
        if (half) launch_norm_add_branches<bf16_t, true>(x, y0, y1, g0, g1, c, eps_b, gain, bias, eps, n_rows, n, (bf16_t*)copy, stream);
        else launch_norm_add_branches<float, true>(x, y0, y1, g0, g1, c, eps_b, gain, bias, eps, n_rows, n, (float*)copy, stream);
    } else {
        if (half) launch_norm_add_branches<bf16_t, false>(x, y0, y1, g0, g1, c, eps_b, gain, nullptr, eps, n_rows, n, (bf16_t*)copy, stream);
        else launch_norm_add_branches<float, false>(x, y0, y1, g0, g1, c, eps_b, gain, nullptr, eps, n_rows, n, (float*)copy, stream);
    }
    ROCML_CHECK_LAUNCH("norm_add_branches");
    return 0;
}

ROCML_EXPORT int rocml_norm_add(float* x, float* y, int n_rows, int n, const float* gain, const float* bias,
                                float eps, int layer, void* copy, int copy_dtype, const float* partials, int n_splits,
                                long long split_stride, int replace, const float* next_gain, float next_eps, hipStream_t stream) {
    // next_gain (may be null; needs copy): copy gets the new x normed, x / sqrt(mean(x^2) + next_eps) * next_gain
    ROCML_REQUIRE(!next_gain || copy, "norm_add: the next norm's output needs a place");
    // layer = 1: layer norm (mean taken off, bias added if given); 0: root-mean-square norm (bias is not read)
    // partials (may be null): [n_splits][rows][n] K pieces of the product that made y, added to y in split order first;
    // with replace they are all of y (what y holds is not read; the plain kernel uses y as its buffer)
    ROCML_REQUIRE(n_rows >= 0 && n > 0 && x && y && gain, "norm_add: bad arguments rows=%d n=%d", n_rows, n);
    ROCML_REQUIRE(n_splits >= 0 && (n_splits == 0 ? !replace : (partials && split_stride >= (long long)n_rows * n)),
                  "norm_add: %d partial sums with a stride of %lld do not fit", n_splits, split_stride);
    ROCML_REQUIRE(!copy || copy_dtype == ROCML_F32 || copy_dtype == ROCML_BF16, "norm_add: unknown dtype code %d", copy_dtype);
    if (n_rows == 0) return 0;
    bool half = copy && copy_dtype == ROCML_BF16;
    if (layer) {
        if (half) launch_norm_add<bf16_t, true>(x, y, gain, bias, eps, n_rows, n, (bf16_t*)copy, partials, n_splits, split_stride, replace, next_gain, next_eps, stream);
        else launch_norm_add<float, true>(x, y, gain, bias, eps, n_rows, n, (float*)copy, partials, n_splits, split_stride, replace, next_gain, next_eps, stream);
    } else {
        if (half) launch_norm_add<bf16_t, false>(x, y, gain, nullptr, eps, n_rows, n, (bf16_t*)copy, partials, n_splits, split_stride, replace, next_gain, next_eps, stream);
        else launch_norm_add<float, false>(x, y, gain, nullptr, eps, n_rows, n, (float*)copy, partials, n_splits, split_stride, replace, next_gain, next_eps, stream);
    }
    ROCML_CHECK_LAUNCH("norm_add");
    return 0;
}

// ---- layer norm ------------------------------------------------------------------------------
// out[r, :] = (x[src(r), :] - mean) / sqrt(var + eps) * gain + bias, var the mean of the squared deviations from
// the mean; `rows` optionally gathers source rows.  32-bit statistics, one block per row.
template <typename TO>
__global__ void __launch_bounds__(EW_BLOCK)
layernorm_kernel(const float* __restrict__ x, const int* __restrict__ rows, const float* __restrict__ gain,
                 const float* __restrict__ bias, float eps, int n, TO* __restrict__ out) {
    __shared__ float scratch[EW_BLOCK / WAVE];
    const float* xin = x + (size_t)(rows ? rows[blockIdx.x] : blockIdx.x) * n;
    TO* o = out + (size_t)blockIdx.x * n;
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) s += xin[i];
    float mean = block_sum(s, scratch) / (float)n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += EW_BLOCK) {
        float d = xin[i] - mean;
        ss = fmaf(d, d, ss);
    }
    float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += EW_BLOCK)
        Elem<TO>::store(o + i, (xin[i] - mean) * inv * gain[i] + (bias ? bias[i] : 0.f));
}

ROCML_EXPORT int rocml_layernorm(const float* x, const int* rows, int n_out, int n, const float* gain, const float* bias,
                                 float eps, void* out, int out_dtype, hipStream_t stream) {
    ROCML_REQUIRE(n_out >= 0 && n > 0 && x && gain && out, "layernorm: bad arguments rows=%d n=%d", n_out, n);
    if (n_out == 0) return 0;
    if (out_dtype == ROCML_F32) layernorm_kernel<float><<<n_out, EW_BLOCK, 0, stream>>>(x, rows, gain, bias, eps, n, (float*)out);
    else if (out_dtype == ROCML_BF16) layernorm_kernel<bf16_t><<<n_out, EW_BLOCK, 0, stream>>>(x, rows, gain, bias, eps, n, (bf16_t*)out);
    else return rocml_fail("layernorm: unknown dtype code %d", out_dtype);
    ROCML_CHECK_LAUNCH("layernorm");
    return 0;
}

// ---- an input that depends on the token's id, gated -----------------------------------------
// out[t, j] = act(g[t, j]) * table[ids[t], col0 + j] for j < dim: g 32-bit [T, dim], the table [vocab, cols] in its own
// type, act = gelu_tanh, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))) (act = 0), or the identity (act = 1).
__device__ __forceinline__ float gelu_tanh_f(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename TT, typename TO>
__global__ void token_side_gate_kernel(const float* __restrict__ g, const TT* __restrict__ table, const int* __restrict__ ids,
                                       int cols, int col0, int dim, int vocab, int act, TO* __restrict__ out, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    long long t = idx / dim;
    int j = (int)(idx - t * dim);
    int id = ids[t];
    float e = (id >= 0 && id < vocab) ? Elem<TT>::load(table + (size_t)id * cols + col0 + j) : 0.f;
    float z = g[idx];
    Elem<TO>::store(out + idx, (act == 0 ? gelu_tanh_f(z) : z) * e);
}

ROCML_EXPORT int rocml_token_side_gate(const float* g, const void* table, int table_dtype, const int* ids, int n_tokens,
                                       int cols, int col0, int dim, int vocab, int act, void* out, int out_dtype,
                                       hipStream_t stream) {
    ROCML_REQUIRE(n_tokens >= 0 && dim > 0 && col0 >= 0 && col0 + dim <= cols && vocab > 0 && g && table && ids && out,
                  "token_side_gate: bad arguments T=%d dim=%d col0=%d cols=%d", n_tokens, dim, col0, cols);
    ROCML_REQUIRE(act == 0 || act == 1, "token_side_gate: unknown activation %d", act);
    long long total = (long long)n_tokens * dim;
    if (total == 0) return 0;
    int grid = ceil_div(total, EW_BLOCK);
#define TSG(TT, TO) token_side_gate_kernel<TT, TO><<<grid, EW_BLOCK, 0, stream>>>(g, (const TT*)table, ids, cols, col0, dim, vocab, act, (TO*)out, total)
    if (table_dtype == ROCML_F32 && out_dtype == ROCML_F32) TSG(float, float);
    else if (table_dtype == ROCML_BF16 && out_dtype == ROCML_BF16) TSG(bf16_t, bf16_t);
    else if (table_dtype == ROCML_BF16 && out_dtype == ROCML_F32) TSG(bf16_t, float);
    else if (table_dtype == ROCML_F32 && out_dtype == ROCML_BF16) TSG(float, bf16_t);
    else return rocml_fail("token_side_gate: unknown dtype codes %d, %d", table_dtype, out_dtype);
#undef TSG
    ROCML_CHECK_LAUNCH("token_side_gate");
    return 0;
}

// ---- a copy of 32-bit values in another type -----------------------------------------
template <typename TO>
__global__ void convert_kernel(const float* __restrict__ x, TO* __restrict__ out, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx < total) Elem<TO>::store(out + idx, x[idx]);
}

ROCML_EXPORT int rocml_convert(const float* x, void* out, int out_dtype, long long total, hipStream_t stream) {
    ROCML_REQUIRE(total >= 0, "convert: negative size");
    if (total == 0) return 0;
    int grid = ceil_div(total, EW_BLOCK);
    if (out_dtype == ROCML_F32) convert_kernel<float><<<grid, EW_BLOCK, 0, stream>>>(x, (float*)out, total);
    else if (out_dtype == ROCML_BF16) convert_kernel<bf16_t><<<grid, EW_BLOCK, 0, stream>>>(x, (bf16_t*)out, total);
    else return rocml_fail("convert: unknown dtype code %d", out_dtype);
    ROCML_CHECK_LAUNCH("convert");
    return 0;
}

// ---- soft cap ----------------------------------------------------------------------------
// x <- cap * tanh(x / cap), in place, 32-bit (a model's logits).
__global__ void softcap_kernel(float* __restrict__ x, float cap, float inv_cap, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx < total) x[idx] = cap * tanhf(x[idx] * inv_cap);
}

ROCML_EXPORT int rocml_softcap(float* x, float cap, long long total, hipStream_t stream) {
    ROCML_REQUIRE(total >= 0 && x && cap > 0.f, "softcap: bad arguments (cap %g)", (double)cap);
    if (total == 0) return 0;
    softcap_kernel<<<ceil_div(total, EW_BLOCK), EW_BLOCK, 0, stream>>>(x, cap, 1.0f / cap, total);
    ROCML_CHECK_LAUNCH("softcap");
    return 0;
}

// ---- weighted sum of up to four matrices ------------------------------------------------------
// out <- alpha * out + sum_b w[b] * y[b], all 32-bit and of one shape (alpha 0: out is only written).
struct WeightedSumArgs {
    const float* y[4];
    float w[4];
};

__global__ void weighted_sum_kernel(float* __restrict__ out, WeightedSumArgs a, int n_branches, float alpha, long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    float acc = alpha != 0.f ? alpha * out[idx] : 0.f;
    for (int b = 0; b < n_branches; ++b) acc = fmaf(a.w[b], a.y[b][idx], acc);
    out[idx] = acc;
}

ROCML_EXPORT int rocml_weighted_sum(float* out, const float* const* ys, const float* weights, int n_branches, float alpha,
                                    long long total, hipStream_t stream) {
    ROCML_REQUIRE(total >= 0 && out && ys && weights && n_branches >= 1 && n_branches <= 4, "weighted_sum: bad arguments (%d branches)",
                  n_branches);
    if (total == 0) return 0;
    WeightedSumArgs a{};
    for (int b = 0; b < n_branches; ++b) {
        ROCML_REQUIRE(ys[b], "weighted_sum: branch %d is missing", b);
        a.y[b] = ys[b];
        a.w[b] = weights[b];
    }
    weighted_sum_kernel<<<ceil_div(total, EW_BLOCK), EW_BLOCK, 0, stream>>>(out, a, n_branches, alpha, total);
    ROCML_CHECK_LAUNCH("weighted_sum");
    return 0;
}

// ---- a matrix added row by row under a gate --------------------------------------------------
// x[t, :] += sigmoid(g[t * ldg]) * y[t, :], 32-bit: a part that every token uses, weighed by one number per token.
__global__ void row_gate_add_kernel(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ g, int ldg, int n,
                                    long long total) {
    long long idx = (long long)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (idx >= total) return;
    long long t = idx / n;
    x[idx] = fmaf(1.0f / (1.0f + expf(-g[(size_t)t * ldg])), y[idx], x[idx]);
}

ROCML_EXPORT int rocml_row_gate_add(float* x, const float* y, const float* g, int ldg, int n_rows, int n, hipStream_t stream) {
    ROCML_REQUIRE(n_rows >= 0 && n > 0 && ldg >= 1 && x && y && g, "row_gate_add: bad arguments rows=%d n=%d", n_rows, n);
    long long total = (long long)n_rows * n;
    if (total == 0) return 0;
    row_gate_add_kernel<<<ceil_div(total, EW_BLOCK), EW_BLOCK, 0, stream>>>(x, y, g, ldg, n, total);
    ROCML_CHECK_LAUNCH("row_gate_add");
    return 0;
}
