// Row-wise and element-wise kernels of the mixers and feed-forwards that are not plain attention
// and SwiGLU: the Dynamic Tanh norm, the clamped gated activation of routed experts, gated
// normalisation over groups of columns, the token shift of time-mixing layers, the per-layer token
// input, and what a latent-attention step does between its projections and the attention kernel.
//
// As everywhere: the residual stream is float; activations between kernels are float or bfloat16
// (template argument); all arithmetic is float.
#include "common.h"

#include <math.h>

__device__ __forceinline__ float pw_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float pw_silu(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float pw_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// ---- residual add + Dynamic Tanh ---------------------------------------------------------------
// Without `rows`: x[r] += residual[r] (float, written back); out[r] = tanh(alpha x[r]) * w + b.
// With `rows`: the same for x[rows[r]] + residual[rows[r]], x untouched.  No statistic of the row
// is taken, so one thread does one element.
template <typename R, typename O>
__global__ void add_dyt_kernel(float* __restrict__ x, const R* __restrict__ res, const float* __restrict__ w,
                               const float* __restrict__ b, const float* __restrict__ alpha, O* __restrict__ out,
                               const int32_t* __restrict__ rows, int H) {
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    const float a = alpha[0];
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = x[src * H + c];
        if (res) {
            v += tl_to_float(res[src * H + c]);
            if (!rows) x[src * H + c] = v;
        }
        out[(size_t)r * H + c] = tl_from_float<O>(tanhf(a * v) * w[c] + b[c]);
    }
}

extern "C" int tl_add_dyt(float* x, const void* res, int res_dtype, const float* w, const float* b, const float* alpha,
                          void* out, int out_dtype, const int32_t* rows, int n, int H, hipStream_t stream) {
    TL_CHECK_ARG(n >= 0 && H > 0, "tl_add_dyt: bad sizes n=%d H=%d", n, H);
    if (n == 0) return 0;
    dim3 grid(n), block(H >= 1024 ? 256 : 128);
#define GO(R, O) hipLaunchKernelGGL((add_dyt_kernel<R, O>), grid, block, 0, stream, x, (const R*)res, w, b, alpha, (O*)out, rows, H)
    if (res_dtype == TL_F32 && out_dtype == TL_F32) GO(float, float);
    else if (res_dtype == TL_F32 && out_dtype == TL_BF16) GO(float, bf16_t);
    else if (res_dtype == TL_BF16 && out_dtype == TL_F32) GO(bf16_t, float);
    else if (res_dtype == TL_BF16 && out_dtype == TL_BF16) GO(bf16_t, bf16_t);
    else return tl_fail("tl_add_dyt: unknown dtypes %d %d", res_dtype, out_dtype);
#undef GO
    TL_CHECK_LAUNCH("tl_add_dyt");
    return 0;
}

// ---- x += residual, and x again in the activation type -------------------------------------------
template <typename O>
__global__ void add_cast_kernel(float* __restrict__ x, const float* __restrict__ res, O* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = x[i];
    if (res) {
        v += res[i];
        x[i] = v;
    }
    out[i] = tl_from_float<O>(v);
}

extern "C" int tl_add_cast(float* x, const float* res, void* out, int out_dtype, long long n, hipStream_t stream) {
    TL_CHECK_ARG(n >= 0, "tl_add_cast: bad size");
    if (n == 0) return 0;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (out_dtype == TL_F32) hipLaunchKernelGGL(add_cast_kernel<float>, grid, block, 0, stream, x, res, (float*)out, (size_t)n);
    else if (out_dtype == TL_BF16) hipLaunchKernelGGL(add_cast_kernel<bf16_t>, grid, block, 0, stream, x, res, (bf16_t*)out, (size_t)n);
    else return tl_fail("tl_add_cast: unknown dtype %d", out_dtype);
    TL_CHECK_LAUNCH("tl_add_cast");
    return 0;
}

// ---- element-wise functions ------------------------------------------------------------------------
// kind 0: tanh; kind 1: the square of relu.  float in, float or bfloat16 out.
template <typename O>
__global__ void unary_kernel(const float* __restrict__ in, O* __restrict__ out, size_t n, int kind) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float z = in[i];
    float r;
    if (kind == 0) {
        r = tanhf(z);
    } else {
        const float p = fmaxf(z, 0.f);
        r = p * p;
    }
    out[i] = tl_from_float<O>(r);
}

extern "C" int tl_unary(const float* in, void* out, int out_dtype, long long n, int kind, hipStream_t stream) {
    TL_CHECK_ARG(n >= 0 && (kind == 0 || kind == 1), "tl_unary: bad arguments");
    if (n == 0) return 0;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (out_dtype == TL_F32) hipLaunchKernelGGL(unary_kernel<float>, grid, block, 0, stream, in, (float*)out, (size_t)n, kind);
    else if (out_dtype == TL_BF16) hipLaunchKernelGGL(unary_kernel<bf16_t>, grid, block, 0, stream, in, (bf16_t*)out, (size_t)n, kind);
    else return tl_fail("tl_unary: unknown dtype %d", out_dtype);
    TL_CHECK_LAUNCH("tl_unary");
    return 0;
}

// ---- clamped gated activation ------------------------------------------------------------------------
// gu [T, 2F] (gate columns first): g = min(gate, limit), u = clamp(up, -limit, limit),
// out = g * sigmoid(alpha g) * (u + 1).
__device__ __forceinline__ float pw_clamp_glu(float g, float u, float limit, float alpha) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * pw_sigmoid(alpha * g) * (u + 1.0f);
}

template <typename I, typename O>
__global__ void clamp_glu_kernel(const I* __restrict__ gu, O* __restrict__ out, int T, int F, float limit, float alpha) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)T * F) return;
    const size_t t = i / F, c = i - t * F;
    out[i] = tl_from_float<O>(pw_clamp_glu(tl_to_float(gu[t * 2 * F + c]), tl_to_float(gu[t * 2 * F + F + c]), limit, alpha));
}

extern "C" int tl_clamp_glu(const void* gu, int in_dtype, void* out, int out_dtype, int T, int F, float limit, float alpha,
                            hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && F > 0, "tl_clamp_glu: bad sizes");
    if (T == 0) return 0;
    dim3 grid((unsigned)(((size_t)T * F + 255) / 256)), block(256);
#define GO(I, O) hipLaunchKernelGGL((clamp_glu_kernel<I, O>), grid, block, 0, stream, (const I*)gu, (O*)out, T, F, limit, alpha)
    if (in_dtype == TL_F32 && out_dtype == TL_F32) GO(float, float);
    else if (in_dtype == TL_F32 && out_dtype == TL_BF16) GO(float, bf16_t);
    else if (in_dtype == TL_BF16 && out_dtype == TL_BF16) GO(bf16_t, bf16_t);
    else return tl_fail("tl_clamp_glu: unsupported dtypes %d %d", in_dtype, out_dtype);
#undef GO
    TL_CHECK_LAUNCH("tl_clamp_glu");
    return 0;
}

// ---- gated normalisation over groups of columns ----------------------------------------------------
// o float [T, N] in groups of `group` columns (a head, or the whole row): every group is divided by
// its root mean square (eps inside the root), times weight[c], times the gate: sigmoid(gate) for
// gate_act 0, silu(gate) for 1.  gate_act 2 puts the gate first: o * silu(gate) is what is divided by
// its root mean square, then times weight[c].  gate float [T, ldg].  One work-group per (token, group).
template <typename O>
__global__ void gated_group_norm_kernel(const float* __restrict__ o, int ldo, const float* __restrict__ weight,
                                        const float* __restrict__ gate, int ldg, O* __restrict__ out, int N, int group,
                                        float eps, int gate_act) {
    __shared__ float red[16];
    const int t = blockIdx.x, g = blockIdx.y;
    const float* row = o + (size_t)t * ldo + g * group;
    const float* grow = gate + (size_t)t * ldg + g * group;
    float ss = 0.f;
    if (gate_act == 2) {
        for (int c = threadIdx.x; c < group; c += blockDim.x) {
            const float v = row[c] * pw_silu(grow[c]);
            ss += v * v;
        }
    } else {
        for (int c = threadIdx.x; c < group; c += blockDim.x) ss += row[c] * row[c];
    }
    ss = tl_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)group + eps);
    for (int c = threadIdx.x; c < group; c += blockDim.x) {
        const int n = g * group + c;
        const float z = grow[c];
        if (gate_act == 2) {
            out[(size_t)t * N + n] = tl_from_float<O>(row[c] * pw_silu(z) * rstd * weight[n]);
        } else {
            const float gv = gate_act == 0 ? pw_sigmoid(z) : pw_silu(z);
            out[(size_t)t * N + n] = tl_from_float<O>(row[c] * rstd * weight[n] * gv);
        }
    }
}

extern "C" int tl_gated_group_norm(const float* o, int ldo, const float* weight, const float* gate, int ldg, void* out,
                                   int out_dtype, int T, int N, int group, float eps, int gate_act, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && N > 0 && group > 0 && N % group == 0 && ldo >= N && ldg >= N, "tl_gated_group_norm: bad sizes");
    if (T == 0) return 0;
    const int groups = N / group;
    TL_CHECK_ARG(groups <= 65535, "tl_gated_group_norm: %d groups are more than a launch takes", groups);
    dim3 grid(T, groups), block(group >= 256 ? 256 : 64 * tl_ceil_div(group, 64));
    if (out_dtype == TL_F32)
        hipLaunchKernelGGL(gated_group_norm_kernel<float>, grid, block, 0, stream, o, ldo, weight, gate, ldg, (float*)out, N, group, eps, gate_act);
    else if (out_dtype == TL_BF16)
        hipLaunchKernelGGL(gated_group_norm_kernel<bf16_t>, grid, block, 0, stream, o, ldo, weight, gate, ldg, (bf16_t*)out, N, group, eps, gate_act);
    else return tl_fail("tl_gated_group_norm: unknown dtype %d", out_dtype);
    TL_CHECK_LAUNCH("tl_gated_group_norm");
    return 0;
}

// ---- token shift -------------------------------------------------------------------------------------
// h [T, W]: out[s][t] = h[t] + (before[t] - h[t]) * mu[s] for `ways` mixing vectors mu [ways, W], where
// before[t] is the row above in the same sequence, and for a sequence's first row of this step the row
// kept in its state slot (zeros for a new request).  prev: float, the slot's row at prev + slot * stride.
template <typename T>
__global__ void token_shift_kernel(const T* __restrict__ h, const int32_t* __restrict__ seq_of_token,
                                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                                   const float* __restrict__ prev, long long stride, const float* __restrict__ mu,
                                   T* __restrict__ out, int Tn, int W, int ways) {
    const int t = blockIdx.x;
    const int s = seq_of_token[t];
    const bool first = q_start[s] == t;
    const float* pr = prev + (size_t)state_slots[s] * stride;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float cur = tl_to_float(h[(size_t)t * W + c]);
        const float bef = first ? pr[c] : tl_to_float(h[(size_t)(t - 1) * W + c]);
        const float d = bef - cur;
        for (int m = 0; m < ways; ++m) out[((size_t)m * Tn + t) * W + c] = tl_from_float<T>(cur + d * mu[(size_t)m * W + c]);
    }
}

// The last row each sequence brought becomes the row its slot keeps.  Runs after the kernel above.
template <typename T>
__global__ void token_shift_keep_kernel(const T* __restrict__ h, const int32_t* __restrict__ q_start,
                                        const int32_t* __restrict__ state_slots, float* __restrict__ prev, long long stride, int W) {
    const int s = blockIdx.x;
    const int last = q_start[s + 1] - 1;
    if (last < q_start[s]) return;
    float* pr = prev + (size_t)state_slots[s] * stride;
    for (int c = threadIdx.x; c < W; c += blockDim.x) pr[c] = tl_to_float(h[(size_t)last * W + c]);
}

extern "C" int tl_token_shift(const void* h, int dtype, const int32_t* seq_of_token, const int32_t* q_start,
                              const int32_t* state_slots, float* prev, long long stride, const float* mu, void* out, int T,
                              int S, int W, int ways, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && S > 0 && W > 0 && ways > 0 && stride >= W, "tl_token_shift: bad sizes");
    if (T == 0) return 0;
    dim3 block(W >= 1024 ? 256 : 128);
    if (dtype == TL_F32) {
        hipLaunchKernelGGL(token_shift_kernel<float>, dim3(T), block, 0, stream, (const float*)h, seq_of_token, q_start, state_slots, prev, stride, mu, (float*)out, T, W, ways);
        hipLaunchKernelGGL(token_shift_keep_kernel<float>, dim3(S), block, 0, stream, (const float*)h, q_start, state_slots, prev, stride, W);
    } else if (dtype == TL_BF16) {
        hipLaunchKernelGGL(token_shift_kernel<bf16_t>, dim3(T), block, 0, stream, (const bf16_t*)h, seq_of_token, q_start, state_slots, prev, stride, mu, (bf16_t*)out, T, W, ways);
        hipLaunchKernelGGL(token_shift_keep_kernel<bf16_t>, dim3(S), block, 0, stream, (const bf16_t*)h, q_start, state_slots, prev, stride, W);
    } else return tl_fail("tl_token_shift: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_token_shift");
    return 0;
}

// ---- per-layer token input: gate ---------------------------------------------------------------------
// out[t, c] = gelu_tanh(z[t, c]) * table[ids[t], col0 + c]; z float [T, D], table [V, ld].
template <typename T>
__global__ void gelu_token_gate_kernel(const float* __restrict__ z, const T* __restrict__ table, const int32_t* __restrict__ ids,
                                       T* __restrict__ out, int D, int ld, int col0, int V) {
    const int t = blockIdx.x;
    const int id = ids[t];
    for (int c = threadIdx.x; c < D; c += blockDim.x) {
        const float e = (id >= 0 && id < V) ? tl_to_float(table[(size_t)id * ld + col0 + c]) : NAN;
        out[(size_t)t * D + c] = tl_from_float<T>(pw_gelu_tanh(z[(size_t)t * D + c]) * e);
    }
}

extern "C" int tl_gelu_token_gate(const float* z, const void* table, int dtype, const int32_t* ids, void* out, int T, int D,
                                  int ld, int col0, int V, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && D > 0 && col0 >= 0 && col0 + D <= ld && V > 0, "tl_gelu_token_gate: bad sizes");
    if (T == 0) return 0;
    dim3 grid(T), block(D >= 256 ? 256 : 64);
    if (dtype == TL_F32) hipLaunchKernelGGL(gelu_token_gate_kernel<float>, grid, block, 0, stream, z, (const float*)table, ids, (float*)out, D, ld, col0, V);
    else if (dtype == TL_BF16) hipLaunchKernelGGL(gelu_token_gate_kernel<bf16_t>, grid, block, 0, stream, z, (const bf16_t*)table, ids, (bf16_t*)out, D, ld, col0, V);
    else return tl_fail("tl_gelu_token_gate: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_gelu_token_gate");
    return 0;
}

// ---- latent attention: between the projections and the attention kernel ---------------------------------
// proj float [T, ldp] holds per token: H query heads of (d plain + r rotated) columns, then the
// compressed row of `rank` columns and r columns of the one rotated key part all heads share.
// Per token (one work-group):
//   * the compressed row is divided by its root mean square (eps inside the root) and scaled by
//     norm_w: the latent c;
//   * query and key rotated parts are turned: pair (i, i + r/2) by the angle pos * freq[i], cosine and
//     sine both times `mag`;
//   * plain query parts go to q_plain [T, H*d];
//   * rotated query parts go to q_lat [T, H*D] at columns [rank, rank + r) of each head, zeros up to D
//     (the first `rank` columns are written by the product with the key expansion);
//   * the row [c | rotated key part | zeros] of D columns goes into the cache at `slot`, once token-major
//     ([pages, page, 1, D]) and once with a page's tokens innermost ([pages, 1, D, page]).
template <typename T>
__global__ void latent_prepare_kernel(const float* __restrict__ proj, int ldp, const int32_t* __restrict__ pos,
                                      const float* __restrict__ freq, float mag, const float* __restrict__ norm_w, float eps,
                                      const int32_t* __restrict__ slots, T* __restrict__ q_plain, T* __restrict__ q_lat,
                                      T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int d, int r, int rank, int D,
                                      int page) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const float* row = proj + (size_t)t * ldp;
    const float p = (float)pos[t];
    const int half = r / 2;
    // queries
    for (int idx = threadIdx.x; idx < H * d; idx += blockDim.x) {
        const int h = idx / d, c = idx - h * d;
        q_plain[(size_t)t * H * d + idx] = tl_from_float<T>(row[h * (d + r) + c]);
    }
    for (int idx = threadIdx.x; idx < H * (D - rank); idx += blockDim.x) {
        const int h = idx / (D - rank), c = idx - h * (D - rank);
        float v = 0.f;
        if (c < r) {
            const int i = c < half ? c : c - half;
            const float a = p * freq[i];
            const float cs = cosf(a) * mag, sn = sinf(a) * mag;
            const float* qr = row + h * (d + r) + d;
            v = c < half ? qr[i] * cs - qr[i + half] * sn : qr[i + half] * cs + qr[i] * sn;
        }
        q_lat[((size_t)t * H + h) * D + rank + c] = tl_from_float<T>(v);
    }
    // the latent and the shared rotated key part
    const float* kv = row + H * (d + r);
    float ss = 0.f;
    for (int c = threadIdx.x; c < rank; c += blockDim.x) ss += kv[c] * kv[c];
    ss = tl_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)rank + eps);
    const int slot = slots[t];
    if (slot < 0) return;
    const size_t pg = (size_t)slot / page, within = (size_t)slot % page;
    for (int c = threadIdx.x; c < D; c += blockDim.x) {
        float v = 0.f;
        if (c < rank) {
            v = kv[c] * rstd * norm_w[c];
        } else if (c < rank + r) {
            const int cc = c - rank;
            const int i = cc < half ? cc : cc - half;
            const float a = p * freq[i];
            const float cs = cosf(a) * mag, sn = sinf(a) * mag;
            const float* kr = kv + rank;
            v = cc < half ? kr[i] * cs - kr[i + half] * sn : kr[i + half] * cs + kr[i] * sn;
        }
        const T o = tl_from_float<T>(v);
        k_cache[(size_t)slot * D + c] = o;
        v_cache[(pg * D + c) * page + within] = o;
    }
}

extern "C" int tl_latent_prepare(const float* proj, int ldp, const int32_t* pos, const float* freq, float mag,
                                 const float* norm_w, float eps, const int32_t* slots, void* q_plain, void* q_lat,
                                 void* k_cache, void* v_cache, int dtype, int T, int H, int d, int r, int rank, int D, int page,
                                 hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && H > 0 && d > 0 && r >= 0 && r % 2 == 0 && rank > 0 && D >= rank + r && page > 0,
                 "tl_latent_prepare: bad sizes H=%d d=%d r=%d rank=%d D=%d", H, d, r, rank, D);
    TL_CHECK_ARG(ldp >= H * (d + r) + rank + r, "tl_latent_prepare: the projection's rows are too short");
    if (T == 0) return 0;
    dim3 grid(T), block(256);
    if (dtype == TL_F32)
        hipLaunchKernelGGL(latent_prepare_kernel<float>, grid, block, 0, stream, proj, ldp, pos, freq, mag, norm_w, eps, slots,
                           (float*)q_plain, (float*)q_lat, (float*)k_cache, (float*)v_cache, H, d, r, rank, D, page);
    else if (dtype == TL_BF16)
        hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, grid, block, 0, stream, proj, ldp, pos, freq, mag, norm_w, eps, slots,
                           (bf16_t*)q_plain, (bf16_t*)q_lat, (bf16_t*)k_cache, (bf16_t*)v_cache, H, d, r, rank, D, page);
    else return tl_fail("tl_latent_prepare: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_latent_prepare");
    return 0;
}

// ---- a gate per head ---------------------------------------------------------------------------------------
// o [T, H*dv] *= sigmoid(gate[t, h]) (gate float with row stride ldg), in place.
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ o, const float* __restrict__ gate, int ldg, int H, int dv) {
    const int t = blockIdx.x;
    for (int idx = threadIdx.x; idx < H * dv; idx += blockDim.x) {
        const int h = idx / dv;
        const size_t at = (size_t)t * H * dv + idx;
        o[at] = tl_from_float<T>(tl_to_float(o[at]) * pw_sigmoid(gate[(size_t)t * ldg + h]));
    }
}

extern "C" int tl_head_gate(void* o, int dtype, const float* gate, int ldg, int T, int H, int dv, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && H > 0 && dv > 0 && ldg >= H, "tl_head_gate: bad sizes");
    if (T == 0) return 0;
    dim3 grid(T), block(256);
    if (dtype == TL_F32) hipLaunchKernelGGL(head_gate_kernel<float>, grid, block, 0, stream, (float*)o, gate, ldg, H, dv);
    else if (dtype == TL_BF16) hipLaunchKernelGGL(head_gate_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)o, gate, ldg, H, dv);
    else return tl_fail("tl_head_gate: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_head_gate");
    return 0;
}

// ---- attention over wide rows -----------------------------------------------------------------------------
// Causal attention of H query heads over ONE shared key/value head whose rows are wider than the
// matrix-core kernels take (D up to 1024): the key of a cached token is its whole row of D columns, its
// value the same row.  q [T, H*D], cache rows token-major [pages, page, 1, D], out [T, H*D]; float
// arithmetic, no matrix instructions: the slow and simple way for sizes nothing else serves.
// A work-group per (token, head); wave w takes the keys j with j % 4 == w (by absolute position, so the
// same keys meet in a wave however the sequence was cut), each lane the columns lane, lane + 64, ... of
// query, key and running sum; per key a sum over the wave, then the online softmax step.  The four waves'
// sums are put together in the order of the waves.
#define WIDE_MAX_D 1024
template <typename T>
__global__ __launch_bounds__(256) void attn_wide_kernel(const T* __restrict__ q, const T* __restrict__ kc,
                                                        const int32_t* __restrict__ tables, int NB,
                                                        const int32_t* __restrict__ seq_of_token,
                                                        const int32_t* __restrict__ pos, T* __restrict__ out, int H, int D,
                                                        int page, float scale, int window) {
    constexpr int E = WIDE_MAX_D / 64;
    __shared__ float sm[4], sl[4];
    __shared__ float sacc[4][WIDE_MAX_D];
    const int t = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int s = seq_of_token[t], p = pos[t];
    const int32_t* table = tables + (size_t)s * NB;
    const T* qrow = q + ((size_t)t * H + h) * D;
    float qv[E], acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int c = lane + 64 * e;
        qv[e] = c < D ? tl_to_float(qrow[c]) * scale : 0.f;
        acc[e] = 0.f;
    }
    float m = -INFINITY, l = 0.f;
    // window > 0: keys from p - window + 1 on; a wave still takes the keys j with j % 4 == w
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    for (int j = (lo & ~3) + w + ((lo & 3) > w ? 4 : 0); j <= p; j += 4) {
        const T* krow = kc + ((size_t)table[j / page] * page + j % page) * D;
        float kv[E], dot = 0.f;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int c = lane + 64 * e;
            kv[e] = c < D ? tl_to_float(krow[c]) : 0.f;
            dot += qv[e] * kv[e];
        }
        dot = tl_wave_sum(dot);
        const float m_new = fmaxf(m, dot);
        const float corr = expf(m - m_new), pe = expf(dot - m_new);
        l = l * corr + pe;
#pragma unroll
        for (int e = 0; e < E; ++e) acc[e] = acc[e] * corr + pe * kv[e];
        m = m_new;
    }
    if (lane == 0) {
        sm[w] = m;
        sl[w] = l;
    }
#pragma unroll
    for (int e = 0; e < E; ++e) sacc[w][lane + 64 * e] = acc[e];
    __syncthreads();
    float M = fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3]));
    float f[4], L = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[i] = sm[i] > -INFINITY ? expf(sm[i] - M) : 0.f;
        L += sl[i] * f[i];
    }
    T* orow = out + ((size_t)t * H + h) * D;
    for (int c = threadIdx.x; c < D; c += 256) {
        float v = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) v += sacc[i][c] * f[i];
        orow[c] = tl_from_float<T>(L > 0.f ? v / L : 0.f);
    }
}

extern "C" int tl_attention_wide(const void* q, const void* k_cache, int dtype, const int32_t* tables, int NB,
                                 const int32_t* seq_of_token, const int32_t* pos, void* out, int T, int H, int D, int page,
                                 float scale, int window, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && H > 0 && H <= 65535 && D > 0 && D <= WIDE_MAX_D && page > 0 && NB > 0 && window >= 0,
                 "tl_attention_wide: bad sizes H=%d D=%d (rows of at most %d)", H, D, WIDE_MAX_D);
    if (T == 0) return 0;
    dim3 grid(T, H), block(256);
    if (dtype == TL_F32)
        hipLaunchKernelGGL(attn_wide_kernel<float>, grid, block, 0, stream, (const float*)q, (const float*)k_cache, tables, NB,
                           seq_of_token, pos, (float*)out, H, D, page, scale, window);
    else if (dtype == TL_BF16)
        hipLaunchKernelGGL(attn_wide_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)q, (const bf16_t*)k_cache, tables, NB,
                           seq_of_token, pos, (bf16_t*)out, H, D, page, scale, window);
    else return tl_fail("tl_attention_wide: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_attention_wide");
    return 0;
}

// ---- queries and keys normed over the whole projection, a query factor by position, the cache write ----
// proj float [T, ldp] = [q: H*d | k: G*d | v: G*dv] (biases added already).  Per token:
//   * q and k are each divided by the root mean square of their whole row (all heads at once, eps inside
//     the root) and multiplied by a weight per column (wq [H*d], wk [G*d]; null: no norm);
//   * q is multiplied by 1 + coef * ln(floor((pos + 1) / every) + 1) (every <= 0: no factor);
//   * q goes to q_out [T, H*D], every head padded with zeros from d to D;
//   * k goes into the cache at `slot` ([pages, page, G, D], zeros from d to D), v with a page's tokens
//     innermost ([pages, G, D, page], zeros from dv to D).
template <typename T>
__global__ __launch_bounds__(1024) void qk_norm_store_kernel(
    const float* __restrict__ proj, int ldp, const int32_t* __restrict__ pos, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, float coef, int every, const int32_t* __restrict__ slots,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G, int d, int dv, int D, int page) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const float* q = proj + (size_t)t * ldp;
    const float* k = q + H * d;
    const float* v = k + G * d;
    float rq = 1.f, rk = 1.f;
    if (wq) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < H * d; c += blockDim.x) ss += q[c] * q[c];
        ss = tl_block_sum(ss, red);
        rq = 1.0f / sqrtf(ss / (float)(H * d) + eps);
    }
    if (wk) {
        float ss = 0.f;
        for (int c = threadIdx.x; c < G * d; c += blockDim.x) ss += k[c] * k[c];
        ss = tl_block_sum(ss, red);
        rk = 1.0f / sqrtf(ss / (float)(G * d) + eps);
    }
    float temp = 1.f;
    if (every > 0) temp = 1.0f + coef * logf((float)((pos[t] + 1) / every) + 1.0f);
    for (int idx = threadIdx.x; idx < H * D; idx += blockDim.x) {
        const int h = idx / D, c = idx - h * D;
        float o = 0.f;
        if (c < d) {
            const int n = h * d + c;
            o = wq ? q[n] * rq * wq[n] * temp : q[n] * temp;
        }
        q_out[(size_t)t * H * D + idx] = tl_from_float<T>(o);
    }
    const int slot = slots[t];
    if (slot < 0) return;
    const size_t pg = (size_t)slot / page, within = (size_t)slot % page;
    for (int idx = threadIdx.x; idx < G * D; idx += blockDim.x) {
        const int h = idx / D, c = idx - h * D;
        float kv = 0.f, vv = 0.f;
        if (c < d) {
            const int n = h * d + c;
            kv = wk ? k[n] * rk * wk[n] : k[n];
        }
        if (c < dv) vv = v[h * dv + c];
        k_cache[(size_t)slot * G * D + idx] = tl_from_float<T>(kv);
        v_cache[(pg * G * D + idx) * page + within] = tl_from_float<T>(vv);
    }
}

extern "C" int tl_qk_norm_store(const float* proj, int ldp, const int32_t* pos, const float* wq, const float* wk, float eps,
                                float coef, int every, const int32_t* slots, void* q_out, void* k_cache, void* v_cache,
                                int dtype, int T, int H, int G, int d, int dv, int D, int page, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && H > 0 && G > 0 && d > 0 && dv > 0 && D >= d && D >= dv && page > 0,
                 "tl_qk_norm_store: bad sizes H=%d G=%d d=%d dv=%d D=%d", H, G, d, dv, D);
    TL_CHECK_ARG(ldp >= H * d + G * d + G * dv, "tl_qk_norm_store: the projection's rows are too short");
    TL_CHECK_ARG((wq == nullptr) == (wk == nullptr), "tl_qk_norm_store: queries and keys are normed together or not at all");
    if (T == 0) return 0;
    // few tokens (decode steps): a token's columns over more threads, since nothing else fills the GPU
    dim3 grid(T), block(T <= 64 && H * D >= 1024 ? 1024 : 256);
    if (dtype == TL_F32)
        hipLaunchKernelGGL(qk_norm_store_kernel<float>, grid, block, 0, stream, proj, ldp, pos, wq, wk, eps, coef, every, slots,
                           (float*)q_out, (float*)k_cache, (float*)v_cache, H, G, d, dv, D, page);
    else if (dtype == TL_BF16)
        hipLaunchKernelGGL(qk_norm_store_kernel<bf16_t>, grid, block, 0, stream, proj, ldp, pos, wq, wk, eps, coef, every, slots,
                           (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, H, G, d, dv, D, page);
    else return tl_fail("tl_qk_norm_store: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_qk_norm_store");
    return 0;
}

// ---- a weighted sum of two float tensors -------------------------------------------------------------------
// out = a * x + b * y, element by element (out may be x or y).
__global__ void scaled_sum_kernel(const float* x, const float* y, float* out, float a, float b, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a * x[i] + b * y[i];
}

extern "C" int tl_scaled_sum(const float* x, const float* y, float* out, float a, float b, long long n, hipStream_t stream) {
    TL_CHECK_ARG(n >= 0, "tl_scaled_sum: bad size");
    if (n == 0) return 0;
    hipLaunchKernelGGL(scaled_sum_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, y, out, a, b, (size_t)n);
    TL_CHECK_LAUNCH("tl_scaled_sum");
    return 0;
}

// ---- the difference of two attention maps, normed per head ---------------------------------------------------
// a [T, 2 H, D]: what attention leaves for 2 H query heads that are the two maps of H heads, ordered by
// key/value head g, then map m, then the head's place r within its group of R = H / G:
// head (2 g + m) R + r is map m of head g R + r; the first dv of its D columns count.
// out [T, H, dv]: o = a1 - lambda a2, divided by its root mean square over the dv values (eps inside
// the root), times `post`.  A wave per (token, head); float arithmetic.
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(const T* __restrict__ a, int lda, T* __restrict__ out, int n, int H,
                                                          int G, int dv, int D, float lambda, float eps, float post) {
    const int lane = threadIdx.x & 63;
    const int item = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (item >= n) return;
    const int t = item / H, h = item - t * H;
    const int R = H / G, g = h / R, r = h - g * R;
    const T* a1 = a + (size_t)t * lda + (size_t)((2 * g) * R + r) * D;
    const T* a2 = a + (size_t)t * lda + (size_t)((2 * g + 1) * R + r) * D;
    float ss = 0.f;
    for (int c = lane; c < dv; c += 64) {
        const float o = tl_to_float(a1[c]) - lambda * tl_to_float(a2[c]);
        ss += o * o;
    }
    ss = tl_wave_sum(ss);
    const float f = post / sqrtf(ss / (float)dv + eps);
    T* orow = out + ((size_t)t * H + h) * dv;
    for (int c = lane; c < dv; c += 64) orow[c] = tl_from_float<T>((tl_to_float(a1[c]) - lambda * tl_to_float(a2[c])) * f);
}

extern "C" int tl_diff_combine(const void* a, int lda, void* out, int dtype, int T, int H, int G, int dv, int D, float lambda,
                               float eps, float post, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && H > 0 && G > 0 && H % G == 0 && dv > 0 && D >= dv && lda >= 2 * H * D && eps >= 0.f,
                 "tl_diff_combine: bad sizes H=%d G=%d dv=%d D=%d", H, G, dv, D);
    TL_CHECK_ARG((long long)T * H <= 2147483647LL, "tl_diff_combine: too many rows");
    if (T == 0) return 0;
    const int n = T * H;
    dim3 grid(tl_ceil_div(n, 4)), block(256);
    if (dtype == TL_F32)
        hipLaunchKernelGGL(diff_combine_kernel<float>, grid, block, 0, stream, (const float*)a, lda, (float*)out, n, H, G, dv, D,
                           lambda, eps, post);
    else if (dtype == TL_BF16)
        hipLaunchKernelGGL(diff_combine_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)a, lda, (bf16_t*)out, n, H, G, dv, D,
                           lambda, eps, post);
    else return tl_fail("tl_diff_combine: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_diff_combine");
    return 0;
}

// ---- gated activations of a fused gate/up projection --------------------------------------------------------
// gu [T, 2F] (gate columns first): out = act(gate) * up; kind 0: act = silu, kind 1: act = the tanh form of
// gelu, 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).  float arithmetic.
template <typename I, typename O>
__global__ void glu_kernel(const I* __restrict__ gu, O* __restrict__ out, int T, int F, int kind) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)T * F) return;
    const size_t t = i / F, c = i - t * F;
    const float g = tl_to_float(gu[t * 2 * F + c]), u = tl_to_float(gu[t * 2 * F + F + c]);
    out[i] = tl_from_float<O>((kind == 1 ? pw_gelu_tanh(g) : g * pw_sigmoid(g)) * u);
}

extern "C" int tl_glu(const void* gu, int in_dtype, void* out, int out_dtype, int T, int F, int kind, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && F > 0 && (kind == 0 || kind == 1), "tl_glu: bad sizes or unknown activation %d", kind);
    if (T == 0) return 0;
    dim3 grid((unsigned)(((size_t)T * F + 255) / 256)), block(256);
#define GO(I, O) hipLaunchKernelGGL((glu_kernel<I, O>), grid, block, 0, stream, (const I*)gu, (O*)out, T, F, kind)
    if (in_dtype == TL_F32 && out_dtype == TL_F32) GO(float, float);
    else if (in_dtype == TL_F32 && out_dtype == TL_BF16) GO(float, bf16_t);
    else if (in_dtype == TL_BF16 && out_dtype == TL_BF16) GO(bf16_t, bf16_t);
    else return tl_fail("tl_glu: unsupported dtypes %d %d", in_dtype, out_dtype);
#undef GO
    TL_CHECK_LAUNCH("tl_glu");
    return 0;
}

// ---- queries and keys normed per head, neighbouring pairs turned, the cache write ---------------------------
// proj float [T, ldp] = [q: H*d | k: G*d | v: G*dv] (biases added already; no v columns with v_from_k).
// Per token, for every query head and key head:
//   * the head's d values are divided by their root mean square (eps inside the root) and multiplied by a
//     weight per dimension that all heads share (wq [d], wk [d]; null: no norm);
//   * then the pairs (2i, 2i + 1), i < rot / 2, are turned by the angle pos * freq[i], cosine and sine both
//     times `mag` (freq null or rot 0: no rotation); the angle, its cosine and sine are float;
//   * q goes to q_out [T, H*D], every head padded with zeros from d to D; k into the cache at `slot`
//     ([pages, page, G, D], zeros from d to D); v with a page's tokens innermost ([pages, G, D, page], zeros
//     from dv to D).  With v_from_k the values are the keys as projected: before norm and rotation.
// A work-group per token and four heads (of queries, keys or values, in that order); a wave takes one head, a lane
// the pairs lane and lane + 64 of it (d <= 256).  A work-group computes the token's cosines and sines once, into LDS.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_rotate_store_kernel(
    const float* __restrict__ proj, int ldp, const int32_t* __restrict__ pos, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, const float* __restrict__ freq, float mag, int rot,
    const int32_t* __restrict__ slots, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G,
    int d, int dv, int D, int page, int v_from_k) {
    __shared__ float cs[128], sn[128];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* row = proj + (size_t)t * ldp;
    const float p = (float)pos[t];
    for (int i = threadIdx.x; i < rot / 2; i += blockDim.x) {
        const float a = p * freq[i];
        cs[i] = cosf(a) * mag;
        sn[i] = sinf(a) * mag;
    }
    __syncthreads();
    const int slot = slots ? slots[t] : -1;
    const size_t pg = slot >= 0 ? (size_t)slot / page : 0, within = slot >= 0 ? (size_t)slot % page : 0;
    const int units = H + G + (v_from_k ? 0 : G);
    for (int u = blockIdx.y * 4 + wave; u < units; u += units) {       // one head per wave; written as a loop for its early exits
        const bool is_q = u < H, is_k = !is_q && u < H + G;
        const int head = is_q ? u : is_k ? u - H : u - H - G;
        const int n = (is_q || is_k) ? d : dv;                   // the values the head has
        const float* x = row + (is_q ? head * d : is_k ? H * d + head * d : (H + G) * d + head * dv);
        float raw[4], y[4];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int c = 2 * (lane + 64 * j);
            raw[2 * j] = c < n ? x[c] : 0.f;
            raw[2 * j + 1] = c + 1 < n ? x[c + 1] : 0.f;
        }
        if (!is_q && slot < 0) continue;                         // nothing to write for this token (the same for the wave)
        const float* w = is_q ? wq : is_k ? wk : nullptr;
        float rstd = 1.0f;
        if (w) {
            const float ss = tl_wave_sum(raw[0] * raw[0] + raw[1] * raw[1] + raw[2] * raw[2] + raw[3] * raw[3]);
            rstd = 1.0f / sqrtf(ss / (float)n + eps);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int i = lane + 64 * j, c = 2 * i;
            float a = raw[2 * j], b = raw[2 * j + 1];
            if (w) {
                a = c < n ? a * rstd * w[c] : 0.f;
                b = c + 1 < n ? b * rstd * w[c + 1] : 0.f;
            }
            if ((is_q || is_k) && c + 1 < rot) {
                const float ra = a * cs[i] - b * sn[i], rb = b * cs[i] + a * sn[i];
                a = ra;
                b = rb;
            }
            y[2 * j] = a;
            y[2 * j + 1] = b;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int c = 2 * (lane + 64 * j) + e;
                if (c >= D) continue;
                const T o = tl_from_float<T>(y[2 * j + e]);       // zeros beyond the head's values
                if (is_q) {
                    q_out[((size_t)t * H + head) * D + c] = o;
                } else if (is_k) {
                    k_cache[((size_t)slot * G + head) * D + c] = o;
                    if (v_from_k) v_cache[((pg * G + head) * D + c) * page + within] = tl_from_float<T>(raw[2 * j + e]);
                } else {
                    v_cache[((pg * G + head) * D + c) * page + within] = o;
                }
            }
        }
    }
}

extern "C" int tl_head_norm_rotate_store(const float* proj, int ldp, const int32_t* pos, const float* wq, const float* wk,
                                         float eps, const float* freq, float mag, int rot, const int32_t* slots, void* q_out,
                                         void* k_cache, void* v_cache, int dtype, int T, int H, int G, int d, int dv, int D,
                                         int page, int v_from_k, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && H > 0 && G >= 0 && d > 0 && dv > 0 && D >= d && D >= dv && D <= 256 && page > 0,
                 "tl_head_norm_rotate_store: bad sizes H=%d G=%d d=%d dv=%d D=%d", H, G, d, dv, D);
    TL_CHECK_ARG(rot >= 0 && rot % 2 == 0 && rot <= d && (rot == 0 || freq), "tl_head_norm_rotate_store: %d turned dimensions of %d", rot, d);
    TL_CHECK_ARG(!v_from_k || dv == d, "tl_head_norm_rotate_store: values that are the keys have the keys' size");
    TL_CHECK_ARG((wq == nullptr) == (wk == nullptr), "tl_head_norm_rotate_store: queries and keys are normed together or not at all");
    TL_CHECK_ARG(ldp >= (H + G) * d + (v_from_k ? 0 : G * dv), "tl_head_norm_rotate_store: the projection's rows are too short");
    TL_CHECK_ARG(G == 0 || (slots && k_cache && v_cache), "tl_head_norm_rotate_store: keys need their cache");
    if (T == 0) return 0;
    dim3 grid(T, tl_ceil_div(H + G + (v_from_k ? 0 : G), 4)), block(256);
    TL_CHECK_ARG(grid.y <= 65535, "tl_head_norm_rotate_store: too many heads");
#define GO(TT)                                                                                                         \
    hipLaunchKernelGGL(head_norm_rotate_store_kernel<TT>, grid, block, 0, stream, proj, ldp, pos, wq, wk, eps, freq, mag, \
                       rot, slots, (TT*)q_out, (TT*)k_cache, (TT*)v_cache, H, G, d, dv, D, page, v_from_k)
    if (dtype == TL_F32) GO(float);
    else if (dtype == TL_BF16) GO(bf16_t);
    else return tl_fail("tl_head_norm_rotate_store: unknown dtype %d", dtype);
#undef GO
    TL_CHECK_LAUNCH("tl_head_norm_rotate_store");
    return 0;
}
