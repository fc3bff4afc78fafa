// Routed experts: choice of experts per token, the tokens of each expert gathered into row tiles,
// the experts' products as one grouped launch each, and the weighted sum per token.
//
//   tl_moe_route    per token: the `top` largest router logits (lowest index wins a tie) and their weights:
//                   the softmax over those alone, scale * sigmoid of each, or their shares of the softmax
//                   over all experts                             -> expert ids, weights [T, top]
//   tl_moe_sort     the (token, choice) pairs ordered by expert and cut into row tiles of BM rows that
//                   hold one expert's pairs only                 -> order, tiles
//   tl_moe_gemm     a product per tile with its expert's matrix: gate/up with the gated activation
//                   min(g, limit) sigmoid(alpha min(g, limit)) (clamp(u, +-limit) + shift) in the epilogue
//                   (limit = infinity, alpha = 1, shift = 0: silu(g) u), or up alone with the square of relu
//                   in the epilogue (experts without gate), or down, which scatters rows back to their pairs
//   tl_moe_combine  out[t] = sum over the token's choices, in the order of its choices, of weight *
//                   row (+ a shared expert's output)
//
// A pair's row is computed alone (a row of a tile does not see the other rows) and summed over k in
// one fixed order, and a token's choices are added in one fixed order, so neither the batch nor the
// place a pair gets inside its expert's tiles changes a bit of a result.  The products run on the
// float matrix instruction (v_mfma_f32_16x16x4_f32), bfloat16 operands widened on the way into
// LDS, as the any-shape product does.
#include "common.h"

#include <math.h>

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 32

// ---- routing ------------------------------------------------------------------------------------------
// A wave per token: lane l looks at logits l, l + 64, ...; the largest not yet chosen is found by a
// butterfly over (value, index), equal values going to the lower index; lane c keeps the c-th choice.
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int ldl, int32_t* __restrict__ ids,
                                                        float* __restrict__ weights, int T, int E, int top, int mode,
                                                        float scale) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t >= T) return;
    const float* z = logits + (size_t)t * ldl;
    const int none = 0x7fffffff;
    unsigned taken = 0;                 // bit s: logit lane + 64 s is chosen already
    float my_val = 0.f;
    int my_id = 0;
    for (int c = 0; c < top; ++c) {
        float bv = 0.f;
        int be = none;
        for (int e = lane, sl = 0; e < E; e += 64, ++sl) {
            if ((taken >> sl) & 1u) continue;
            const float v = z[e];
            if (be == none || v > bv) {
                bv = v;
                be = e;
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oe = __shfl_xor(be, off, 64);
            if (oe != none && (be == none || ov > bv || (ov == bv && oe < be))) {
                bv = ov;
                be = oe;
            }
        }
        if ((be & 63) == lane) taken |= 1u << (be >> 6);
        if (lane == c) {
            my_val = bv;
            my_id = be;
        }
    }
    if (mode == 1) {                    // every chosen expert by its own score: scale * sigmoid(logit)
        if (lane < top) {
            ids[(size_t)t * top + lane] = my_id;
            weights[(size_t)t * top + lane] = scale * (1.0f / (1.0f + expf(-my_val)));
        }
        return;
    }
    const float largest = __shfl(my_val, 0, 64);
    const float ex = lane < top ? expf(my_val - largest) : 0.f;
    float sum;
    if (mode == 2) {                    // the softmax over all experts, the chosen ones' shares kept as they are
        float all = 0.f;
        for (int e = lane; e < E; e += 64) all += expf(z[e] - largest);
        sum = tl_wave_sum(all);
    } else {
        sum = tl_wave_sum(ex);
    }
    if (lane < top) {
        ids[(size_t)t * top + lane] = my_id;
        weights[(size_t)t * top + lane] = ex / sum;
    }
}

// Routing within the best groups.  Scores are s = sigmoid(logit).  The E experts form `groups` equal groups of
// neighbours; a group's score is the sum of its two largest scores (of its one score, for groups of one);
// only experts of the `keep` best groups can be chosen; of those the `top` with the largest scores are,
// weighted by their scores divided by the sum of the chosen scores (+ 1e-20).  Among equals the lower index
// wins, for groups and for experts.  A wave per token: lane l holds the scores of experts l, l + 64, ...
// (at most 16 of them) and, as lane g, the score of group g (groups <= 64).
__device__ __forceinline__ void moe_wave_best(float& bv, int& be) {   // the largest value over the wave, the lower index among equals
    const int none = 0x7fffffff;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oe = __shfl_xor(be, off, 64);
        if (oe != none && (be == none || ov > bv || (ov == bv && oe < be))) {
            bv = ov;
            be = oe;
        }
    }
}
template <int SL>      // scores a lane holds: 1 for up to 64 experts, 4 for up to 256, 16 beyond
__global__ __launch_bounds__(256) void moe_route_grouped_kernel(const float* __restrict__ logits, int ldl,
                                                                int32_t* __restrict__ ids, float* __restrict__ weights, int T,
                                                                int E, int top, int groups, int keep) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t >= T) return;
    const float* z = logits + (size_t)t * ldl;
    const int none = 0x7fffffff, per = E / groups;
    const int nsl = (E + 63) >> 6;                         // slots in use: the same for the whole wave
    float s[SL];
    int grp[SL];
#pragma unroll
    for (int sl = 0; sl < SL; ++sl) {
        const int e = lane + 64 * sl;
        const bool real = sl < nsl && e < E;
        s[sl] = real ? 1.0f / (1.0f + expf(-z[e])) : -1.0f;
        grp[sl] = real ? e / per : -1;
    }
    // group scores: per group the two largest scores over the wave (a butterfly over pairs (largest, second);
    // scores lie in (0, 1), -1 stands for none), lane g keeps group g's
    float my_group = 0.f;
    for (int g = 0; g < groups; ++g) {
        float a1 = -1.0f, a2 = -1.0f;
#pragma unroll
        for (int sl = 0; sl < SL; ++sl) {
            if (sl < nsl && grp[sl] == g) {
                const float v = s[sl];
                a2 = fmaxf(a2, fminf(a1, v));
                a1 = fmaxf(a1, v);
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float b1 = __shfl_xor(a1, off, 64), b2 = __shfl_xor(a2, off, 64);
            a2 = fmaxf(fminf(a1, b1), fmaxf(a2, b2));
            a1 = fmaxf(a1, b1);
        }
        if (lane == g) my_group = fmaxf(a1, 0.f) + fmaxf(a2, 0.f);
    }
    // the best groups
    unsigned long long kept = 0ull;
    for (int k = 0; k < keep; ++k) {
        float bv = my_group;
        int be = (lane < groups && !((kept >> lane) & 1ull)) ? lane : none;
        moe_wave_best(bv, be);
        kept |= 1ull << be;
    }
    // the best experts among them
    unsigned taken = 0;
    float my_val = 0.f;
    int my_id = 0;
    for (int c = 0; c < top; ++c) {
        float bv = 0.f;
        int be = none;
#pragma unroll
        for (int sl = 0; sl < SL; ++sl) {
            if (sl < nsl && grp[sl] >= 0 && !((taken >> sl) & 1u) && ((kept >> grp[sl]) & 1ull) && (be == none || s[sl] > bv)) {
                bv = s[sl];
                be = lane + 64 * sl;
            }
        }
        moe_wave_best(bv, be);
        if ((be & 63) == lane) taken |= 1u << (be >> 6);
        if (lane == c) {
            my_val = bv;
            my_id = be;
        }
    }
    const float sum = tl_wave_sum(lane < top ? my_val : 0.f) + 1e-20f;
    if (lane < top) {
        ids[(size_t)t * top + lane] = my_id;
        weights[(size_t)t * top + lane] = my_val / sum;
    }
}

extern "C" int tl_moe_route_grouped(const float* logits, int ldl, int32_t* ids, float* weights, int T, int E, int top,
                                    int groups, int keep, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && E > 0 && top > 0 && top <= MOE_MAX_TOP && E <= MOE_MAX_EXPERTS && ldl >= E,
                 "tl_moe_route_grouped: bad sizes E=%d top=%d", E, top);
    TL_CHECK_ARG(groups > 0 && groups <= 64 && E % groups == 0 && keep > 0 && keep <= groups && top <= keep * (E / groups),
                 "tl_moe_route_grouped: %d experts in %d groups of which %d are kept do not give %d choices", E, groups, keep, top);
    if (T == 0) return 0;
#define GO(SLV)                                                                                                     \
    hipLaunchKernelGGL(moe_route_grouped_kernel<SLV>, dim3(tl_ceil_div(T, 4)), dim3(256), 0, stream, logits, ldl, ids, \
                       weights, T, E, top, groups, keep)
    if (E <= 64) GO(1);
    else if (E <= 256) GO(4);
    else GO(MOE_MAX_EXPERTS / 64);
#undef GO
    TL_CHECK_LAUNCH("tl_moe_route_grouped");
    return 0;
}

// mode 0: weights = softmax over the chosen logits; mode 1: weights = scale * sigmoid(chosen logit);
// mode 2: weights = the chosen experts' shares of the softmax over all logits, not renormalised.
extern "C" int tl_moe_route(const float* logits, int ldl, int32_t* ids, float* weights, int T, int E, int top, int mode,
                            float scale, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && E > 0 && top > 0 && top <= E && top <= MOE_MAX_TOP && E <= MOE_MAX_EXPERTS && ldl >= E,
                 "tl_moe_route: bad sizes E=%d top=%d", E, top);
    TL_CHECK_ARG(mode >= 0 && mode <= 2, "tl_moe_route: unknown weighting %d", mode);
    if (T == 0) return 0;
    hipLaunchKernelGGL(moe_route_kernel, dim3(tl_ceil_div(T, 4)), dim3(256), 0, stream, logits, ldl, ids, weights, T, E, top, mode, scale);
    TL_CHECK_LAUNCH("tl_moe_route");
    return 0;
}

// ---- pairs ordered by expert ----------------------------------------------------------------------------
// P = T * top pairs.  order[P]: the pair at each place; places of an expert are consecutive.  A tile
// is (expert, first place, rows); tiles[0] = number of tiles, then three ints per tile.  One
// work-group; counts and cursors in LDS.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ order,
                                                         int32_t* __restrict__ tiles, int P, int E, int BM) {
    __shared__ int count[MOE_MAX_EXPERTS], first[MOE_MAX_EXPERTS], tile0[MOE_MAX_EXPERTS + 1];
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        const int e = ids[p];
        if (e >= 0 && e < E) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, nt = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = at;
            tile0[e] = nt;
            at += count[e];
            nt += (count[e] + BM - 1) / BM;
        }
        tile0[E] = nt;
        tiles[0] = nt;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        const int n = count[e];
        for (int i = 0, tl = tile0[e]; i < n; i += BM, ++tl) {
            tiles[1 + 3 * tl] = e;
            tiles[2 + 3 * tl] = first[e] + i;
            tiles[3 + 3 * tl] = min(BM, n - i);
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;      // now the cursor within the expert
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        const int e = ids[p];
        if (e >= 0 && e < E) order[first[e] + atomicAdd(&count[e], 1)] = p;
    }
}

extern "C" int tl_moe_sort(const int32_t* ids, int32_t* order, int32_t* tiles, int P, int E, int BM, hipStream_t stream) {
    TL_CHECK_ARG(P >= 0 && E > 0 && E <= MOE_MAX_EXPERTS && (BM == 16 || BM == 64), "tl_moe_sort: bad sizes P=%d E=%d BM=%d", P, E, BM);
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(P >= 1024 ? 1024 : 256), 0, stream, ids, order, tiles, P, E, BM);
    TL_CHECK_LAUNCH("tl_moe_sort");
    return 0;
}

// ---- the grouped product ----------------------------------------------------------------------------------
#define MG_THREADS 256
#define MG_KS 16
#define MG_LD (MG_KS + 4)
typedef float mg_f32x4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ float4 mg_load4(const T* __restrict__ base, bool ok, int k, int K, bool vec);
template <> __device__ __forceinline__ float4 mg_load4<float>(const float* __restrict__ base, bool ok, int k, int K, bool vec) {
    if (!ok || k >= K) return make_float4(0.f, 0.f, 0.f, 0.f);
    if (vec && k + 3 < K) return *reinterpret_cast<const float4*>(base + k);
    float4 r;
    r.x = base[k];
    r.y = (k + 1 < K) ? base[k + 1] : 0.f;
    r.z = (k + 2 < K) ? base[k + 2] : 0.f;
    r.w = (k + 3 < K) ? base[k + 3] : 0.f;
    return r;
}
template <> __device__ __forceinline__ float4 mg_load4<bf16_t>(const bf16_t* __restrict__ base, bool ok, int k, int K, bool vec) {
    if (!ok || k >= K) return make_float4(0.f, 0.f, 0.f, 0.f);
    if (vec && k + 3 < K) {
        const uint2 raw = *reinterpret_cast<const uint2*>(base + k);
        return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                           __uint_as_float(raw.y & 0xffff0000u));
    }
    float4 r;
    r.x = tl_to_float(base[k]);
    r.y = (k + 1 < K) ? tl_to_float(base[k + 1]) : 0.f;
    r.z = (k + 2 < K) ? tl_to_float(base[k + 2]) : 0.f;
    r.w = (k + 3 < K) ? tl_to_float(base[k + 3]) : 0.f;
    return r;
}

// GLU: W [E, 2 N, K] (gate rows, then up rows), A rows are the tokens of the tile's pairs
// (order[place] / top), C [P, N] by place, C = act(gate, up).  Otherwise: W [E, N, K], A [P, K] by
// place, C [P, N] by pair (order[place]).  Four waves side by side, each MB x NB blocks of 16 x 16
// (GLU: NB gate blocks and NB up blocks).
// MODE 0: down; 1: gate and up with the gated activation; 2: up alone, A rows gathered by token and C by
// place as for 1, W [E, N, K], C = max(., 0)^2.
template <typename TA, typename TW, typename TO, int MB, int NB, int MODE>
__global__ __launch_bounds__(MG_THREADS) void moe_gemm_kernel(const TA* __restrict__ A, int lda, const TW* __restrict__ W,
                                                             TO* __restrict__ C, int ldc, const int32_t* __restrict__ order,
                                                             const int32_t* __restrict__ tiles, int top, int N, int K,
                                                             int a_vec, int w_vec, float limit, float alpha, float shift) {
    constexpr bool GLU = MODE == 1, BY_TOKEN = MODE != 0;
    constexpr int BM = MB * 16, BN = 4 * NB * 16, WR = GLU ? 2 * BN : BN, NW = GLU ? 2 * NB : NB;
    constexpr int A_PIECES = BM * 4, W_PIECES = WR * 4;
    constexpr int A_PER = (A_PIECES + MG_THREADS - 1) / MG_THREADS, W_PER = (W_PIECES + MG_THREADS - 1) / MG_THREADS;
    __shared__ float As[2][BM * MG_LD];
    __shared__ float Ws[2][WR * MG_LD];
    __shared__ int arow[BM];
    if ((int)blockIdx.y >= tiles[0]) return;
    const int e = tiles[1 + 3 * blockIdx.y], place0 = tiles[2 + 3 * blockIdx.y], rows = tiles[3 + 3 * blockIdx.y];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int n0 = blockIdx.x * BN;
    for (int r = tid; r < BM; r += MG_THREADS) arow[r] = r < rows ? (BY_TOKEN ? order[place0 + r] / top : place0 + r) : -1;
    __syncthreads();
    const TW* We = W + (size_t)e * (GLU ? 2 : 1) * N * K;

    mg_f32x4 acc[MB][NW];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NW; ++j) acc[i][j] = (mg_f32x4){0.f, 0.f, 0.f, 0.f};

    float4 areg[A_PER], wreg[W_PER];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int it = 0; it < A_PER; ++it) {
            const int p = tid + it * MG_THREADS;
            const int r = p >> 2, c4 = p & 3;
            const int src = p < A_PIECES ? arow[r] : -1;
            areg[it] = mg_load4<TA>(A + (size_t)(src < 0 ? 0 : src) * lda, src >= 0, k0 + 4 * c4, K, a_vec != 0);
        }
#pragma unroll
        for (int it = 0; it < W_PER; ++it) {
            const int p = tid + it * MG_THREADS;
            const int r = p >> 2, c4 = p & 3;
            // LDS row r: gate (or plain) row n0 + r for r < BN, up row N + n0 + r - BN beyond
            const int col = (GLU && r >= BN) ? n0 + r - BN : n0 + r;
            const size_t wrow = (GLU && r >= BN) ? (size_t)N + col : (size_t)col;
            wreg[it] = mg_load4<TW>(We + wrow * K, p < W_PIECES && col < N, k0 + 4 * c4, K, w_vec != 0);
        }
    };
    auto to_lds = [&](int buf) {
#pragma unroll
        for (int it = 0; it < A_PER; ++it) {
            const int p = tid + it * MG_THREADS;
            if (p < A_PIECES) *reinterpret_cast<float4*>(&As[buf][(p >> 2) * MG_LD + 4 * (p & 3)]) = areg[it];
        }
#pragma unroll
        for (int it = 0; it < W_PER; ++it) {
            const int p = tid + it * MG_THREADS;
            if (p < W_PIECES) *reinterpret_cast<float4*>(&Ws[buf][(p >> 2) * MG_LD + 4 * (p & 3)]) = wreg[it];
        }
    };

    fetch(0);
    to_lds(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += MG_KS) {
        const bool more = k0 + MG_KS < K;
        if (more) fetch(k0 + MG_KS);
        float4 af[MB], wf[NW];
#pragma unroll
        for (int i = 0; i < MB; ++i) af[i] = *reinterpret_cast<const float4*>(&As[buf][(i * 16 + li) * MG_LD + 4 * lg]);
#pragma unroll
        for (int j = 0; j < NW; ++j) {
            const int r = (j < NB ? 0 : BN) + (wave * NB + (j < NB ? j : j - NB)) * 16 + li;
            wf[j] = *reinterpret_cast<const float4*>(&Ws[buf][r * MG_LD + 4 * lg]);
        }
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
            for (int j = 0; j < NW; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i].x, wf[j].x, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i].y, wf[j].y, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i].z, wf[j].z, acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i].w, wf[j].w, acc[i][j], 0, 0, 0);
            }
        if (more) {
            to_lds(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
    }

    // this lane holds rows 4 lg + v and column li of each block
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int n = n0 + (wave * NB + j) * 16 + li;
        if (n >= N) continue;
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int r = i * 16 + 4 * lg + v;
                if (r >= rows) continue;
                if (GLU) {
                    const float g = fminf(acc[i][j][v], limit);
                    const float u = fminf(fmaxf(acc[i][NB + j][v], -limit), limit);
                    C[(size_t)(place0 + r) * ldc + n] = tl_from_float<TO>(g * (1.0f / (1.0f + expf(-alpha * g))) * (u + shift));
                } else if (MODE == 2) {
                    const float u = fmaxf(acc[i][j][v], 0.f);
                    C[(size_t)(place0 + r) * ldc + n] = tl_from_float<TO>(u * u);
                } else {
                    C[(size_t)order[place0 + r] * ldc + n] = tl_from_float<TO>(acc[i][j][v]);
                }
            }
    }
}

// The same product for bfloat16 operands on v_mfma_f32_16x16x32_bf16 (products exact, sums in float).
// Tiles of BM x 128 matrix rows per work-group (GLU: 64 gate rows and the 64 up rows of the same
// columns), k in steps of 64 through double-buffered LDS whose rows are padded to 144 bytes, so that the
// sixteen 16-byte fragment reads of a quarter wave fall into different banks; the pieces of the next two
// steps wait in registers meanwhile (what a step costs is the chain load - registers - LDS - barrier).  Lane l = 16 g + c gives row c of a block at the eight k from 8 g on,
// as first operand (a row of A) and as second (a row of W), and holds C[4 g + v][c] in register v.
typedef __bf16 mg_bf16x8 __attribute__((ext_vector_type(8)));
#define MGB_KT 64
#define MGB_LD 72

template <int MB, int MODE>
__global__ __launch_bounds__(MG_THREADS) void moe_gemm_bf16_kernel(const bf16_t* __restrict__ A, int lda,
                                                                  const bf16_t* __restrict__ W, void* __restrict__ Cv, int ldc,
                                                                  const int32_t* __restrict__ order,
                                                                  const int32_t* __restrict__ tiles, int top, int N, int K,
                                                                  float limit, float alpha, float shift) {
    constexpr bool GLU = MODE == 1, BY_TOKEN = MODE != 0;
    constexpr int BM = MB * 16, WR = 128, BN = GLU ? 64 : 128;
    constexpr int A_PIECES = BM * 8, W_PIECES = WR * 8;
    constexpr int A_PER = (A_PIECES + MG_THREADS - 1) / MG_THREADS, W_PER = W_PIECES / MG_THREADS;
    __shared__ __attribute__((aligned(16))) uint16_t As[2][BM * MGB_LD];
    __shared__ __attribute__((aligned(16))) uint16_t Ws[2][WR * MGB_LD];
    __shared__ int arow[BM];
    if ((int)blockIdx.y >= tiles[0]) return;
    const int e = tiles[1 + 3 * blockIdx.y], place0 = tiles[2 + 3 * blockIdx.y], rows = tiles[3 + 3 * blockIdx.y];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * BN;
    for (int r = tid; r < BM; r += MG_THREADS) arow[r] = r < rows ? (BY_TOKEN ? order[place0 + r] / top : place0 + r) : -1;
    __syncthreads();
    const bf16_t* We = W + (size_t)e * (GLU ? 2 : 1) * N * K;

    mg_f32x4 acc[MB][2];
#pragma unroll
    for (int i = 0; i < MB; ++i) acc[i][0] = acc[i][1] = (mg_f32x4){0.f, 0.f, 0.f, 0.f};

    // Two steps of look-ahead: while step s is multiplied out of LDS, the pieces of steps s + 1 and s + 2
    // are in registers or on their way (two sets, used in turn).
    uint4 areg[2][A_PER], wreg[2][W_PER];
    auto fetch = [&](int k0, uint4* ar, uint4* wr) {
#pragma unroll
        for (int it = 0; it < A_PER; ++it) {
            const int p = tid + it * MG_THREADS;
            const int r = p >> 3, k = k0 + 8 * (p & 7);
            const int src = p < A_PIECES ? arow[r] : -1;
            ar[it] = (src >= 0 && k < K) ? *reinterpret_cast<const uint4*>(A + (size_t)src * lda + k) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int it = 0; it < W_PER; ++it) {
            const int p = tid + it * MG_THREADS;
            const int r = p >> 3, k = k0 + 8 * (p & 7);
            const int col = (GLU && r >= 64) ? n0 + r - 64 : n0 + r;
            const size_t wrow = (GLU && r >= 64) ? (size_t)N + col : (size_t)col;
            wr[it] = (col < N && k < K) ? *reinterpret_cast<const uint4*>(We + wrow * K + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto to_lds = [&](int buf, const uint4* ar, const uint4* wr) {
#pragma unroll
        for (int it = 0; it < A_PER; ++it) {
            const int p = tid + it * MG_THREADS;
            if (p < A_PIECES) *reinterpret_cast<uint4*>(&As[buf][(p >> 3) * MGB_LD + 8 * (p & 7)]) = ar[it];
        }
#pragma unroll
        for (int it = 0; it < W_PER; ++it) {
            const int p = tid + it * MG_THREADS;
            *reinterpret_cast<uint4*>(&Ws[buf][(p >> 3) * MGB_LD + 8 * (p & 7)]) = wr[it];
        }
    };
    // W rows of this wave's two blocks: GLU gate block `wave` and up block `wave`; else blocks 2 wave, 2 wave + 1
    const int wr0 = (GLU ? wave * 16 : wave * 32) + c, wr1 = (GLU ? 64 + wave * 16 : wave * 32 + 16) + c;
    auto multiply = [&](int buf) {
#pragma unroll
        for (int s = 0; s < MGB_KT / 32; ++s) {
            const mg_bf16x8 w0 = __builtin_bit_cast(mg_bf16x8, *reinterpret_cast<const uint4*>(&Ws[buf][wr0 * MGB_LD + 32 * s + 8 * g]));
            const mg_bf16x8 w1 = __builtin_bit_cast(mg_bf16x8, *reinterpret_cast<const uint4*>(&Ws[buf][wr1 * MGB_LD + 32 * s + 8 * g]));
#pragma unroll
            for (int i = 0; i < MB; ++i) {
                const mg_bf16x8 a = __builtin_bit_cast(mg_bf16x8, *reinterpret_cast<const uint4*>(&As[buf][(i * 16 + c) * MGB_LD + 32 * s + 8 * g]));
                acc[i][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, w0, acc[i][0], 0, 0, 0);
                acc[i][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, w1, acc[i][1], 0, 0, 0);
            }
        }
    };

    const int nsteps = (K + MGB_KT - 1) / MGB_KT;
    fetch(0, areg[0], wreg[0]);
    to_lds(0, areg[0], wreg[0]);
    if (nsteps > 1) fetch(MGB_KT, areg[0], wreg[0]);
    if (nsteps > 2) fetch(2 * MGB_KT, areg[1], wreg[1]);
    __syncthreads();
    // step s is in LDS buffer s % 2; set s % 2 holds step s + 1, the other set step s + 2
    for (int s = 0; s < nsteps; s += 2) {
        multiply(0);
        if (s + 1 < nsteps) {
            to_lds(1, areg[0], wreg[0]);
            if (s + 3 < nsteps) fetch((s + 3) * MGB_KT, areg[0], wreg[0]);
            __syncthreads();
            multiply(1);
            if (s + 2 < nsteps) {
                to_lds(0, areg[1], wreg[1]);
                if (s + 4 < nsteps) fetch((s + 4) * MGB_KT, areg[1], wreg[1]);
                __syncthreads();
            }
        }
    }

#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int r = i * 16 + 4 * g + v;
            if (r >= rows) continue;
            if (GLU) {
                const int n = n0 + wave * 16 + c;
                if (n >= N) continue;
                const float gt = fminf(acc[i][0][v], limit);
                const float up = fminf(fmaxf(acc[i][1][v], -limit), limit);
                reinterpret_cast<bf16_t*>(Cv)[(size_t)(place0 + r) * ldc + n] =
                    tl_from_float<bf16_t>(gt * (1.0f / (1.0f + expf(-alpha * gt))) * (up + shift));
            } else if (MODE == 2) {
                bf16_t* crow = reinterpret_cast<bf16_t*>(Cv) + (size_t)(place0 + r) * ldc;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int n = n0 + wave * 32 + j * 16 + c;
                    const float u = fmaxf(acc[i][j][v], 0.f);
                    if (n < N) crow[n] = tl_from_float<bf16_t>(u * u);
                }
            } else {
                float* crow = reinterpret_cast<float*>(Cv) + (size_t)order[place0 + r] * ldc;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int n = n0 + wave * 32 + j * 16 + c;
                    if (n < N) crow[n] = acc[i][j][v];
                }
            }
        }
}

// glu 1: A [T, K] tokens (row stride lda), W [E, 2N, K], C [P, N] by place, of type c_dtype.
// glu 2: the same without gate: W [E, N, K], C = max(A W^T, 0)^2.
// glu 0: A [P, K] by place, W [E, N, K], C float [P, N] by pair.  max_tiles bounds the tiles that
// tl_moe_sort can have made: P / BM + E.
extern "C" int tl_moe_gemm(const void* A, int a_dtype, int lda, const void* W, int w_dtype, void* C, int c_dtype, int ldc,
                           const int32_t* order, const int32_t* tiles, int max_tiles, int BM, int top, int N, int K, int glu,
                           float limit, float alpha, float shift, hipStream_t stream) {
    TL_CHECK_ARG(N > 0 && K > 0 && lda >= K && ldc >= N && top > 0 && (BM == 16 || BM == 64), "tl_moe_gemm: bad sizes N=%d K=%d BM=%d", N, K, BM);
    TL_CHECK_ARG(max_tiles >= 0 && max_tiles <= 65535, "tl_moe_gemm: %d row tiles are too many for one launch", max_tiles);
    TL_CHECK_ARG(glu >= 0 && glu <= 2, "tl_moe_gemm: unknown form %d", glu);
    if (max_tiles == 0) return 0;
    const size_t a_el = a_dtype == TL_F32 ? 4 : 2, w_el = w_dtype == TL_F32 ? 4 : 2;
    const int a_vec = ((uintptr_t)A % (4 * a_el) == 0 && lda % 4 == 0) ? 1 : 0;
    const int w_vec = ((uintptr_t)W % (4 * w_el) == 0 && K % 4 == 0) ? 1 : 0;
#define GO(TA, TW, TO, MB, NB, GLU)                                                                                       \
    hipLaunchKernelGGL((moe_gemm_kernel<TA, TW, TO, MB, NB, GLU>), dim3(tl_ceil_div(N, 4 * NB * 16), max_tiles),          \
                       dim3(MG_THREADS), 0, stream, (const TA*)A, lda, (const TW*)W, (TO*)C, ldc, order, tiles, top, N, K, \
                       a_vec, w_vec, limit, alpha, shift)
#define GO_BM(TA, TW, TO, GLU)                 \
    do {                                       \
        if (BM == 16) GO(TA, TW, TO, 1, 1, GLU); \
        else GO(TA, TW, TO, 4, 1, GLU);          \
    } while (0)
    const bool bf = a_dtype == TL_BF16 && w_dtype == TL_BF16 && c_dtype == (glu ? TL_BF16 : TL_F32);
    if (bf && K % 8 == 0 && lda % 8 == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0) {
#define GO_BF(MB, GLU)                                                                                                   \
    hipLaunchKernelGGL((moe_gemm_bf16_kernel<MB, GLU>), dim3(tl_ceil_div(N, GLU == 1 ? 64 : 128), max_tiles), dim3(MG_THREADS), 0, \
                       stream, (const bf16_t*)A, lda, (const bf16_t*)W, C, ldc, order, tiles, top, N, K, limit, alpha, shift)
        if (glu == 1) {
            if (BM == 16) GO_BF(1, 1);
            else GO_BF(4, 1);
        } else if (glu == 2) {
            if (BM == 16) GO_BF(1, 2);
            else GO_BF(4, 2);
        } else {
            if (BM == 16) GO_BF(1, 0);
            else GO_BF(4, 0);
        }
#undef GO_BF
        TL_CHECK_LAUNCH("tl_moe_gemm");
        return 0;
    }
    if (glu == 1) {
        if (a_dtype == TL_F32 && w_dtype == TL_F32 && c_dtype == TL_F32) GO_BM(float, float, float, 1);
        else if (a_dtype == TL_BF16 && w_dtype == TL_BF16 && c_dtype == TL_BF16) GO_BM(bf16_t, bf16_t, bf16_t, 1);
        else return tl_fail("tl_moe_gemm: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
    } else if (glu == 2) {
        if (a_dtype == TL_F32 && w_dtype == TL_F32 && c_dtype == TL_F32) GO_BM(float, float, float, 2);
        else if (a_dtype == TL_BF16 && w_dtype == TL_BF16 && c_dtype == TL_BF16) GO_BM(bf16_t, bf16_t, bf16_t, 2);
        else return tl_fail("tl_moe_gemm: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
    } else {
        if (a_dtype == TL_F32 && w_dtype == TL_F32 && c_dtype == TL_F32) GO_BM(float, float, float, 0);
        else if (a_dtype == TL_BF16 && w_dtype == TL_BF16 && c_dtype == TL_F32) GO_BM(bf16_t, bf16_t, float, 0);
        else return tl_fail("tl_moe_gemm: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
    }
#undef GO_BM
#undef GO
    TL_CHECK_LAUNCH("tl_moe_gemm");
    return 0;
}

// ---- the weighted sum per token ---------------------------------------------------------------------------------
__global__ void moe_combine_kernel(const float* __restrict__ y, const float* __restrict__ weights,
                                   const float* __restrict__ shared, const float* __restrict__ shared_gate, int ldg,
                                   float* __restrict__ out, int T, int N, int top) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)T * N) return;
    const size_t t = i / N, c = i - t * N;
    float sum = 0.f;
    for (int k = 0; k < top; ++k) sum += weights[t * top + k] * y[(t * top + k) * N + c];
    if (shared) sum += shared_gate ? shared[i] * (1.0f / (1.0f + expf(-shared_gate[t * ldg]))) : shared[i];
    out[i] = sum;
}

// shared_gate (null: none): one logit per token with row stride ldg; the shared expert's row is multiplied by its
// sigmoid before it is added.
extern "C" int tl_moe_combine(const float* y, const float* weights, const float* shared, const float* shared_gate, int ldg,
                              float* out, int T, int N, int top, hipStream_t stream) {
    TL_CHECK_ARG(T >= 0 && N > 0 && top > 0 && (!shared_gate || (shared && ldg > 0)), "tl_moe_combine: bad sizes");
    if (T == 0) return 0;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)(((size_t)T * N + 255) / 256)), dim3(256), 0, stream, y, weights,
                       shared, shared_gate, ldg, out, T, N, top);
    TL_CHECK_LAUNCH("tl_moe_combine");
    return 0;
}
