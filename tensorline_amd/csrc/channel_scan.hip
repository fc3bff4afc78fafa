// Mixing along the sequence one channel at a time, with what has to be carried from step to step kept
// in the request's state slot:
//
//   tl_causal_conv   a short causal convolution per channel: out[t][c] = act(bias[c] + sum_j taps[c][j] *
//                    x[t - (K - 1) + j][c]), the last tap the current token's; inputs ahead of the step's
//                    first row come from the slot (zeros for a new request), and afterwards the slot keeps
//                    the sequence's last K - 1 inputs
//   tl_gated_scan    the real-gated linear recurrent unit: per channel r = sigmoid(gr + br), i = sigmoid(gi +
//                    bi), a = exp(-c r softplus(lam)), S <- a S + sqrt(1 - a^2) i u, out = S * gelu_tanh(y)
//
// Everything is float.  A token's result is computed by the same instructions whatever the step brings
// with it, tokens in the order of the sequence, so neither the cutting of a prompt nor the batch changes a
// bit of a result.
#include "common.h"

#include <math.h>

#define CS_MAX_TAPS 16

__device__ __forceinline__ float cs_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float cs_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float cs_gelu_tanh(float z) {
    return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// One thread per (token, channel).  kept: the slot's [K - 1][C] inputs, the oldest first.  shift != 0 (steps in
// which every sequence brings one token): the thread also renews what the slot keeps, each value moved one
// place down after it has been read, the token's input last; no other thread touches that channel of that slot.
template <typename O>
__global__ void causal_conv_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ taps,
                                   const float* __restrict__ bias, float* __restrict__ kept, long long state_stride,
                                   const int32_t* __restrict__ state_slots, const int32_t* __restrict__ seq_of_token,
                                   const int32_t* __restrict__ q_start, O* __restrict__ out, int ldo, int C, int K, int act,
                                   int shift) {
    const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int s = seq_of_token[t];
    const int r0 = q_start[s];
    float* old = kept + (size_t)state_slots[s] * state_stride;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < K; ++j) {
        const int r = t - (K - 1) + j;
        const float v = r >= r0 ? x[(size_t)r * ldx + c] : old[(size_t)(r - r0 + K - 1) * C + c];
        acc += taps[(size_t)c * K + j] * v;
        if (shift && j > 0) old[(size_t)(j - 1) * C + c] = v;
    }
    if (act == 1) acc = acc / (1.0f + expf(-acc));
    out[(size_t)t * ldo + c] = tl_from_float<O>(acc);
}

// One thread per (sequence, channel): the last K - 1 inputs of the sequence, taken from the step's rows
// and, where the step brings fewer, from what the slot kept; read first, then written.
__global__ void causal_conv_keep_kernel(const float* __restrict__ x, int ldx, float* __restrict__ kept, long long state_stride,
                                        const int32_t* __restrict__ state_slots, const int32_t* __restrict__ q_start,
                                        int C, int K) {
    const int s = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int r0 = q_start[s], r1 = q_start[s + 1];
    if (r1 <= r0) return;
    float* old = kept + (size_t)state_slots[s] * state_stride;
    float keep[CS_MAX_TAPS - 1];
#pragma unroll
    for (int j = 0; j < CS_MAX_TAPS - 1; ++j) {
        if (j < K - 1) {
            const int r = r1 - (K - 1) + j;
            keep[j] = r >= r0 ? x[(size_t)r * ldx + c] : old[(size_t)(r - r0 + K - 1) * C + c];
        }
    }
#pragma unroll
    for (int j = 0; j < CS_MAX_TAPS - 1; ++j)
        if (j < K - 1) old[(size_t)j * C + c] = keep[j];
}

// x float [T, >= C] (row stride ldx); taps float [C, K]; bias float [C] or null; kept: the slots' [K - 1, C]
// at kept + slot * state_stride; act 0: none, 1: SiLU.  out [T, >= C] float or bfloat16.  `update` != 0
// also renews what the slots keep: 1 by a second launch, after every token of the step has read the old rows;
// 2 in the same launch, for steps in which every sequence brings exactly one token (T == S).
extern "C" int tl_causal_conv(const float* x, int ldx, const float* taps, const float* bias, float* kept,
                              long long state_stride, const int32_t* state_slots, const int32_t* seq_of_token,
                              const int32_t* q_start, void* out, int out_dtype, int ldo, int T, int S, int C, int K, int act,
                              int update, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && S >= 0 && C > 0 && K >= 1 && K <= CS_MAX_TAPS, "tl_causal_conv: bad sizes C=%d taps=%d (at most %d)", C, K, CS_MAX_TAPS);
    TL_CHECK_ARG(ldx >= C && ldo >= C && state_stride >= (long long)(K - 1) * C, "tl_causal_conv: rows or the kept inputs are too short");
    TL_CHECK_ARG(S <= 65535 && tl_ceil_div(C, 256) <= 65535, "tl_causal_conv: too many sequences or channels for one launch");
    TL_CHECK_ARG(update != 2 || T == S, "tl_causal_conv: the one-launch form is for steps of one token per sequence");
    if (T == 0 || S == 0) return 0;
    const int shift = update == 2 ? 1 : 0;
    dim3 block(256), grid(T, tl_ceil_div(C, 256));
    if (out_dtype == TL_F32)
        hipLaunchKernelGGL(causal_conv_kernel<float>, grid, block, 0, stream, x, ldx, taps, bias, kept, state_stride, state_slots,
                           seq_of_token, q_start, (float*)out, ldo, C, K, act, shift);
    else if (out_dtype == TL_BF16)
        hipLaunchKernelGGL(causal_conv_kernel<bf16_t>, grid, block, 0, stream, x, ldx, taps, bias, kept, state_stride, state_slots,
                           seq_of_token, q_start, (bf16_t*)out, ldo, C, K, act, shift);
    else return tl_fail("tl_causal_conv: unknown dtype %d", out_dtype);
    TL_CHECK_LAUNCH("tl_causal_conv");
    if (update == 1 && K > 1) {
        hipLaunchKernelGGL(causal_conv_keep_kernel, dim3(tl_ceil_div(C, 256), S), block, 0, stream, x, ldx, kept, state_stride,
                           state_slots, q_start, C, K);
        TL_CHECK_LAUNCH("tl_causal_conv keep");
    }
    return 0;
}

// A work-group of sixteen waves owns GS_CH channels of one sequence and takes its rows in tiles of GS_TT tokens.
// What does not depend on the state (the gates, a, the input's factor sqrt(1 - a^2) i u, the other branch's
// gelu) is computed by all threads, an element each at a time, and left in LDS; then the first GS_CH threads
// walk the tile, one multiply-add per token and channel, and write the results.  The raw operands of the next
// tile are on their way in registers meanwhile, and LDS has two buffers, so the walk of one tile and the
// element-wise work of the next overlap.  Every element is computed by the same instructions wherever its
// token falls in a tile or a step.  The element-wise work is the larger part (five transcendental functions per
// element), which is why a work-group has few channels and many waves: at 2,048 channels there are 128
// work-groups to spread over the GPU, each with four waves per SIMD to hide the functions' latencies.
#define GS_CH 16
#define GS_TT 64
#define GS_THREADS 1024
#define GS_PER (GS_CH * GS_TT / GS_THREADS)
template <typename O>
__global__ __launch_bounds__(GS_THREADS) void gated_scan_kernel(
    const float* __restrict__ gr, const float* __restrict__ gi, int ldg, const float* __restrict__ br,
    const float* __restrict__ bi, const float* __restrict__ u, int ldu, const float* __restrict__ y, int ldy,
    const float* __restrict__ lam, float c, float* __restrict__ state, long long state_stride,
    const int32_t* __restrict__ state_slots, const int32_t* __restrict__ q_start, O* __restrict__ out, int ldo, int W,
    int bw, int bstride) {
    __shared__ float as[2][GS_TT][GS_CH], bs[2][GS_TT][GS_CH], gs[2][GS_TT][GS_CH];
    const int s = blockIdx.y, ch0 = blockIdx.x * GS_CH, tid = threadIdx.x;
    const int r0 = q_start[s], r1 = q_start[s + 1];
    if (r1 <= r0) return;
    // this thread's elements of a tile: channel ch0 + tid % GS_CH of tokens tid / GS_CH + k * (GS_THREADS / GS_CH)
    const int mc = tid % GS_CH, mt = tid / GS_CH, ch = ch0 + mc;
    const bool ch_ok = ch < W;
    const int gcol = ch_ok ? (ch / bw) * bstride + ch % bw : 0;   // where the channel's gates lie in a row of gr and gi
    const float rate = ch_ok ? c * cs_softplus(lam[ch]) : 0.f;
    const float b_r = (br && ch_ok) ? br[ch] : 0.f, b_i = (bi && ch_ok) ? bi[ch] : 0.f;
    float v_r[GS_PER], v_i[GS_PER], v_u[GS_PER], v_y[GS_PER];
    auto fetch = [&](int t0) {
#pragma unroll
        for (int k = 0; k < GS_PER; ++k) {
            const int t = t0 + mt +  k * (GS_THREADS / GS_CH);
            const bool ok = ch_ok && t < r1;
            v_r[k] = ok ? gr[(size_t)t * ldg + gcol] : 0.f;
            v_i[k] = ok ? gi[(size_t)t * ldg + gcol] : 0.f;
            v_u[k] = ok ? u[(size_t)t * ldu + ch] : 0.f;
            v_y[k] = ok ? y[(size_t)t * ldy + ch] : 0.f;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int k = 0; k < GS_PER; ++k) {
            const int tt = mt +  k * (GS_THREADS / GS_CH);
            const float r = cs_sigmoid(v_r[k] + b_r), i = cs_sigmoid(v_i[k] + b_i);
            const float a = expf(-rate * r);
            as[buf][tt][mc] = a;
            bs[buf][tt][mc] = sqrtf(1.0f - a * a) * i * v_u[k];
            gs[buf][tt][mc] = cs_gelu_tanh(v_y[k]);
        }
    };
    float* st = state + (size_t)state_slots[s] * state_stride + ch0 + tid;     // used by the walkers (tid < GS_CH) only
    const bool walker = tid < GS_CH && ch0 + tid < W;
    float S = walker ? *st : 0.f;
    fetch(r0);
    stash(0);
    __syncthreads();
    int cur = 0;
    for (int t0 = r0; t0 < r1; t0 += GS_TT) {
        const int n = min(GS_TT, r1 - t0);
        const bool more = t0 + GS_TT < r1;
        if (more) fetch(t0 + GS_TT);
        if (walker) {
            // eight tokens' factors are read from LDS at once, so that only the multiply-adds wait for each other
            for (int tt0 = 0; tt0 < n; tt0 += 8) {
                float a8[8], b8[8], g8[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    a8[k] = as[cur][tt0 + k][tid];
                    b8[k] = bs[cur][tt0 + k][tid];
                    g8[k] = gs[cur][tt0 + k][tid];
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    if (tt0 + k < n) {
                        S = a8[k] * S + b8[k];
                        out[(size_t)(t0 + tt0 + k) * ldo + ch0 + tid] = tl_from_float<O>(S * g8[k]);
                    }
                }
            }
        }
        if (more) stash(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    if (walker) *st = S;
}

// gr, gi float (row stride ldg): the gates before their bias and sigmoid, channel ch at column (ch / bw) *
// bstride + ch % bw (blocks of bw channels lie bstride apart; bw = W: side by side); br, bi float [W] or
// null; u, y float [T, >= W]; lam float [W]; c: the factor on r * softplus(lam) in -ln a.  state: a
// request's [W] at state + slot * state_stride.  out [T, >= W] float or bfloat16.
extern "C" int tl_gated_scan(const float* gr, const float* gi, int ldg, const float* br, const float* bi, const float* u,
                             int ldu, const float* y, int ldy, const float* lam, float c, float* state,
                             long long state_stride, const int32_t* state_slots, const int32_t* q_start, void* out,
                             int out_dtype, int ldo, int S, int W, int bw, int bstride, hipStream_t stream) {
    TL_CHECK_ARG(S >= 0 && W > 0 && ldu >= W && ldy >= W && ldo >= W && state_stride >= W, "tl_gated_scan: bad sizes W=%d", W);
    TL_CHECK_ARG(bw > 0 && W % bw == 0 && bstride >= bw && ldg >= (W / bw - 1) * bstride + bw,
                 "tl_gated_scan: gates in blocks of %d channels %d apart do not fit rows of %d", bw, bstride, ldg);
    TL_CHECK_ARG(S <= 65535, "tl_gated_scan: too many sequences for one launch");
    if (S == 0) return 0;
    dim3 grid(tl_ceil_div(W, GS_CH), S), block(GS_THREADS);
    if (out_dtype == TL_F32)
        hipLaunchKernelGGL(gated_scan_kernel<float>, grid, block, 0, stream, gr, gi, ldg, br, bi, u, ldu, y, ldy, lam, c, state,
                           state_stride, state_slots, q_start, (float*)out, ldo, W, bw, bstride);
    else if (out_dtype == TL_BF16)
        hipLaunchKernelGGL(gated_scan_kernel<bf16_t>, grid, block, 0, stream, gr, gi, ldg, br, bi, u, ldu, y, ldy, lam, c, state,
                           state_stride, state_slots, q_start, (bf16_t*)out, ldo, W, bw, bstride);
    else return tl_fail("tl_gated_scan: unknown dtype %d", out_dtype);
    TL_CHECK_LAUNCH("tl_gated_scan");
    return 0;
}

// ---- convolution, rotation and cache write of an attention layer's projections in one pass ------------------
// proj float [T, >= C] holds a token's projected queries, keys and values side by side (biases added):
// Hq query heads of d, Gk key heads of d, Gv value heads of dv; C = (Hq + Gk) d + Gv dv.  Each channel
// goes through its short causal convolution (taps [K, C], a tap's weights for all channels in a row, the last tap
// the current token's; the kept inputs as in tl_causal_conv), then
//   * queries and keys: the first `rot` dimensions of every head are turned in neighbouring pairs,
//     (u, v) at dimensions (2i, 2i + 1) -> (u c - v s, v c + u s) with c = mag cos(pos f_i), s = mag
//     sin(pos f_i), the angle in float (freq null or rot 0: no rotation);
//   * queries are written to q_out [T, Hq, D], zeros in columns d .. D - 1;
//   * keys go into k_cache at the token's slot ([pages, page, Gk, D]) and values into v_cache with a
//     page's tokens innermost ([pages, Gv v_rep, D, page]), every value head v_rep times in a row (a
//     key head 2g + m then finds the values of g at its own index); padding columns are not written.
// Gk = 0 (slots null): a layer that only has queries.  A thread per (token, channel); a rotated channel
// computes its neighbour's convolution as well.  shift != 0 (steps of one token per sequence): the
// thread also renews what the slot keeps, after every thread of the work-group has read (neighbours
// lie in one work-group because pairs start at even channels).
template <typename O>
__global__ __launch_bounds__(256) void conv_rotate_store_kernel(
    const float* __restrict__ proj, int ldp, const float* __restrict__ taps, float* __restrict__ kept, long long state_stride,
    const int32_t* __restrict__ state_slots, const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ pos, const float* __restrict__ freq, float mag, int rot, const int32_t* __restrict__ slots,
    O* __restrict__ q_out, O* __restrict__ k_cache, O* __restrict__ v_cache, int Hq, int Gk, int d, int Gv, int dv, int D,
    int v_rep, int page, int C, int K, int shift) {
    const int t = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    const bool live = c < C;
    if (D > d) {                                    // the queries' padding columns: zeros
        const int w = D - d;
        for (int idx = blockIdx.y * blockDim.x + threadIdx.x; idx < Hq * w; idx += blockDim.x * gridDim.y)
            q_out[((size_t)t * Hq + idx / w) * D + d + idx % w] = tl_from_float<O>(0.f);
    }
    const int s = seq_of_token[t];
    const int r0 = q_start[s];
    float* old = kept + (size_t)state_slots[s] * state_stride;
    const int qk = (Hq + Gk) * d;
    int head = 0, i = 0;
    bool turns = false;
    if (live) {
        if (c < qk) {
            head = c / d;
            i = c - head * d;
            turns = freq != nullptr && i < rot;
        } else {
            head = (c - qk) / dv;
            i = (c - qk) - head * dv;
        }
    }
    const int c2 = turns ? c - i + (i ^ 1) : c;
    float mine = 0.f, other = 0.f;
    float seen[CS_MAX_TAPS];
    if (live) {
        for (int j = 0; j < K; ++j) {
            const int r = t - (K - 1) + j;
            const float v = r >= r0 ? proj[(size_t)r * ldp + c] : old[(size_t)(r - r0 + K - 1) * C + c];
            seen[j] = v;
            mine += taps[(size_t)j * C + c] * v;
            if (turns) {
                const float v2 = r >= r0 ? proj[(size_t)r * ldp + c2] : old[(size_t)(r - r0 + K - 1) * C + c2];
                other += taps[(size_t)j * C + c2] * v2;
            }
        }
    }
    if (shift) {
        __syncthreads();
        if (live)
            for (int j = 1; j < K; ++j) old[(size_t)(j - 1) * C + c] = seen[j];
    }
    if (!live) return;
    float y = mine;
    if (turns) {
        float sn, cs;
        sincosf((float)pos[t] * freq[i >> 1], &sn, &cs);
        sn *= mag;
        cs *= mag;
        y = (i & 1) ? mine * cs + other * sn : mine * cs - other * sn;
    }
    if (c < Hq * d) {
        q_out[((size_t)t * Hq + head) * D + i] = tl_from_float<O>(y);
        return;
    }
    const int slot = slots ? slots[t] : -1;
    if (slot < 0) return;
    if (c < qk) {
        k_cache[((size_t)slot * Gk + (head - Hq)) * D + i] = tl_from_float<O>(y);
        return;
    }
    const size_t pg = (size_t)slot / page, within = (size_t)slot % page;
    for (int r = 0; r < v_rep; ++r)
        v_cache[((pg * Gv * v_rep + (size_t)head * v_rep + r) * D + i) * page + within] = tl_from_float<O>(y);
}

// The same with four neighbouring channels per thread, for head sizes that are multiples of four and rows that start
// at 16-byte borders: 16-byte loads of the projection and the kept inputs; a work-group computes the token's cosines
// and sines once (rot / 2 of them, in LDS) for all its heads; a rotated pair lies within its thread, so nothing is
// computed twice and the one-launch form needs no barrier.
template <typename O>
__device__ __forceinline__ void crs_store4(O* p, float4 v);
template <>
__device__ __forceinline__ void crs_store4<float>(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
template <>
__device__ __forceinline__ void crs_store4<bf16_t>(bf16_t* p, float4 v) {
    uint2 u;
    u.x = (uint32_t)tl_f2bf_bits(v.x) | ((uint32_t)tl_f2bf_bits(v.y) << 16);
    u.y = (uint32_t)tl_f2bf_bits(v.z) | ((uint32_t)tl_f2bf_bits(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = u;
}

template <typename O>
__global__ __launch_bounds__(256) void conv_rotate_store_vec_kernel(
    const float* __restrict__ proj, int ldp, const float* __restrict__ taps, float* __restrict__ kept, long long state_stride,
    const int32_t* __restrict__ state_slots, const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ pos, const float* __restrict__ freq, float mag, int rot, const int32_t* __restrict__ slots,
    O* __restrict__ q_out, O* __restrict__ k_cache, O* __restrict__ v_cache, int Hq, int Gk, int d, int Gv, int dv, int D,
    int v_rep, int page, int C, int K, int shift) {
    __shared__ float cs_s[128], sn_s[128];          // one cosine and sine per rotated pair of the token, times mag
    const int t = blockIdx.x;
    if (D > d) {                                    // the queries' padding columns: zeros
        const int w = D - d;
        for (int idx = blockIdx.y * blockDim.x + threadIdx.x; idx < Hq * w; idx += blockDim.x * gridDim.y)
            q_out[((size_t)t * Hq + idx / w) * D + d + idx % w] = tl_from_float<O>(0.f);
    }
    if (freq != nullptr) {
        const float p = (float)pos[t];
        for (int i = threadIdx.x; i < (rot >> 1); i += blockDim.x) {
            float sn, cs;
            sincosf(p * freq[i], &sn, &cs);
            sn_s[i] = sn * mag;
            cs_s[i] = cs * mag;
        }
        __syncthreads();
    }
    const int s = seq_of_token[t];
    const int r0 = q_start[s];
    float* old = kept + (size_t)state_slots[s] * state_stride;
    const int slot = slots ? slots[t] : -1;
    const int qk = (Hq + Gk) * d;
  for (int c = 4 * (blockIdx.y * blockDim.x + threadIdx.x); c < C; c += 4 * blockDim.x * gridDim.y) {
    float4 y = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j = 0; j < K; ++j) {
        const int r = t - (K - 1) + j;
        const float4 v = r >= r0 ? *reinterpret_cast<const float4*>(proj + (size_t)r * ldp + c)
                                 : *reinterpret_cast<const float4*>(old + (size_t)(r - r0 + K - 1) * C + c);
        const float4 w = *reinterpret_cast<const float4*>(taps + (size_t)j * C + c);
        y.x += w.x * v.x;
        y.y += w.y * v.y;
        y.z += w.z * v.z;
        y.w += w.w * v.w;
        if (shift && j > 0) *reinterpret_cast<float4*>(old + (size_t)(j - 1) * C + c) = v;
    }
    if (c < qk) {
        const int head = c / d, i = c - head * d;
        if (freq != nullptr && i < rot) {
            float sn = sn_s[i >> 1], cs = cs_s[i >> 1];
            const float a = y.x, b = y.y;
            y.x = a * cs - b * sn;
            y.y = b * cs + a * sn;
            if (i + 2 < rot) {
                sn = sn_s[(i >> 1) + 1];
                cs = cs_s[(i >> 1) + 1];
                const float a2 = y.z, b2 = y.w;
                y.z = a2 * cs - b2 * sn;
                y.w = b2 * cs + a2 * sn;
            }
        }
        if (head < Hq) crs_store4<O>(q_out + ((size_t)t * Hq + head) * D + i, y);
        else if (slot >= 0) crs_store4<O>(k_cache + ((size_t)slot * Gk + (head - Hq)) * D + i, y);
        continue;
    }
    if (slot < 0) continue;
    const int head = (c - qk) / dv, i = (c - qk) - head * dv;
    const size_t pg = (size_t)slot / page, within = (size_t)slot % page;
    const float vals[4] = {y.x, y.y, y.z, y.w};
    for (int r = 0; r < v_rep; ++r) {
        O* base = v_cache + ((pg * Gv * v_rep + (size_t)head * v_rep + r) * D + i) * page + within;
#pragma unroll
        for (int e = 0; e < 4; ++e) base[(size_t)e * page] = tl_from_float<O>(vals[e]);
    }
  }
}

// update: 1 renews the kept inputs by a second launch, 2 in the same launch (steps of one token per
// sequence, T == S; needs rot == 0 or an even d, so that a pair's channels lie in one work-group).
extern "C" int tl_conv_rotate_store(const float* proj, int ldp, const float* taps, float* kept, long long state_stride,
                                    const int32_t* state_slots, const int32_t* seq_of_token, const int32_t* q_start,
                                    const int32_t* pos, const float* freq, float mag, int rot, const int32_t* slots, void* q_out,
                                    void* k_cache, void* v_cache, int dtype, int T, int S, int Hq, int Gk, int d, int Gv, int dv,
                                    int D, int v_rep, int page, int K, int update, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && S >= 0 && Hq > 0 && Gk >= 0 && Gv >= 0 && d > 0 && dv > 0 && D >= d && D >= dv && K >= 1 &&
                     K <= CS_MAX_TAPS && v_rep >= 1,
                 "tl_conv_rotate_store: bad sizes Hq=%d Gk=%d d=%d Gv=%d dv=%d D=%d taps=%d", Hq, Gk, d, Gv, dv, D, K);
    const long long C64 = (long long)(Hq + Gk) * d + (long long)Gv * dv;
    TL_CHECK_ARG(C64 <= (1 << 24) && ldp >= C64 && state_stride >= (long long)(K - 1) * C64,
                 "tl_conv_rotate_store: rows or the kept inputs are too short");
    const int C = (int)C64;
    TL_CHECK_ARG(rot >= 0 && rot % 2 == 0 && rot <= d && (rot == 0 || freq != nullptr), "tl_conv_rotate_store: bad rotation width %d", rot);
    TL_CHECK_ARG((Gk == 0 && Gv == 0) || (slots && k_cache && v_cache && page > 0 && Gk > 0 && Gv > 0),
                 "tl_conv_rotate_store: keys and values need their caches and slots");
    TL_CHECK_ARG(T <= 2147483647 / 2 && tl_ceil_div(C, 256) <= 65535 && S <= 65535, "tl_conv_rotate_store: too large for one launch");
    TL_CHECK_ARG(update == 1 || (update == 2 && T == S && (rot == 0 || d % 2 == 0)),
                 "tl_conv_rotate_store: the one-launch form is for steps of one token per sequence");
    if (T == 0 || S == 0) return 0;
    if (rot == 0) freq = nullptr;
    const int shift = update == 2 ? 1 : 0;
    const bool vec = rot <= 256 && C % 4 == 0 && (uintptr_t)taps % 16 == 0 && d % 4 == 0 && dv % 4 == 0 && D % 4 == 0 && ldp % 4 == 0 && (uintptr_t)proj % 16 == 0 && (uintptr_t)kept % 16 == 0 &&
                     state_stride % 4 == 0 && (uintptr_t)q_out % 16 == 0 && (uintptr_t)k_cache % 16 == 0;
    if (vec && (dtype == TL_F32 || dtype == TL_BF16)) {
        dim3 vblock(256), vgrid(T, tl_ceil_div(C, 1024));
        if (dtype == TL_F32)
            hipLaunchKernelGGL(conv_rotate_store_vec_kernel<float>, vgrid, vblock, 0, stream, proj, ldp, taps, kept, state_stride,
                               state_slots, seq_of_token, q_start, pos, freq, mag, rot, slots, (float*)q_out, (float*)k_cache,
                               (float*)v_cache, Hq, Gk, d, Gv, dv, D, v_rep, page, C, K, shift);
        else
            hipLaunchKernelGGL(conv_rotate_store_vec_kernel<bf16_t>, vgrid, vblock, 0, stream, proj, ldp, taps, kept, state_stride,
                               state_slots, seq_of_token, q_start, pos, freq, mag, rot, slots, (bf16_t*)q_out, (bf16_t*)k_cache,
                               (bf16_t*)v_cache, Hq, Gk, d, Gv, dv, D, v_rep, page, C, K, shift);
        TL_CHECK_LAUNCH("tl_conv_rotate_store");
        if (update == 1 && K > 1) {
            hipLaunchKernelGGL(causal_conv_keep_kernel, dim3(tl_ceil_div(C, 256), S), dim3(256), 0, stream, proj, ldp, kept,
                               state_stride, state_slots, q_start, C, K);
            TL_CHECK_LAUNCH("tl_conv_rotate_store keep");
        }
        return 0;
    }
    dim3 block(256), grid(T, tl_ceil_div(C, 256));
    if (dtype == TL_F32)
        hipLaunchKernelGGL(conv_rotate_store_kernel<float>, grid, block, 0, stream, proj, ldp, taps, kept, state_stride, state_slots,
                           seq_of_token, q_start, pos, freq, mag, rot, slots, (float*)q_out, (float*)k_cache, (float*)v_cache, Hq,
                           Gk, d, Gv, dv, D, v_rep, page, C, K, shift);
    else if (dtype == TL_BF16)
        hipLaunchKernelGGL(conv_rotate_store_kernel<bf16_t>, grid, block, 0, stream, proj, ldp, taps, kept, state_stride,
                           state_slots, seq_of_token, q_start, pos, freq, mag, rot, slots, (bf16_t*)q_out, (bf16_t*)k_cache,
                           (bf16_t*)v_cache, Hq, Gk, d, Gv, dv, D, v_rep, page, C, K, shift);
    else return tl_fail("tl_conv_rotate_store: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("tl_conv_rotate_store");
    if (update == 1 && K > 1) {
        hipLaunchKernelGGL(causal_conv_keep_kernel, dim3(tl_ceil_div(C, 256), S), block, 0, stream, proj, ldp, kept, state_stride,
                           state_slots, q_start, C, K);
        TL_CHECK_LAUNCH("tl_conv_rotate_store keep");
    }
    return 0;
}
