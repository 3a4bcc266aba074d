// jl_moe.hip — routed experts: the router's choice (sigmoid scores with a correction, a softmax renormalised over the chosen, or a
// softmax over the chosen logits alone), the
// rows grouped by expert, and the grouped products: up with relu^2 or plain (a gated unit's activation is its own launch), down with
// the routing weights.
#include "jl_common.h"
#include <stdlib.h>

// ---- router: one thread per token ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_route_kernel(const float *__restrict__ logits, const float *__restrict__ correction, int64_t N,
                                                         int E, int top, float scale, int32_t *__restrict__ ids,
                                                         float *__restrict__ weights, int kind, float renorm_eps) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    const float *z = logits + n * E;
    if (kind == JL_ROUTE_TOP_SOFTMAX) {
        // the largest `top` logits (ties: lowest index), found in descending order; weights = softmax over the chosen logits only
        float zmax = 0.f, den = 0.f;
        for (int s = 0; s < top; ++s) {
            int best = -1;
            float bz = 0.f;
            for (int e = 0; e < E; ++e) {
                bool taken = false;
                for (int p = 0; p < s; ++p) taken |= ids[n * top + p] == e;
                if (!taken && (best < 0 || z[e] > bz)) { best = e; bz = z[e]; }
            }
            if (s == 0) zmax = bz;
            const float w = expf(bz - zmax);
            ids[n * top + s] = best;
            weights[n * top + s] = w;
            den += w;
        }
        for (int s = 0; s < top; ++s) weights[n * top + s] = weights[n * top + s] / den * scale;
        return;
    }
    if (kind == JL_ROUTE_SOFTMAX_RENORM) {
        // scores = softmax over ALL experts; the largest `top` (ties: lowest index); weights = score / (sum of the chosen + renorm_eps)
        float zmax = -INFINITY, den = 0.f, chosen = 0.f;
        for (int e = 0; e < E; ++e) zmax = fmaxf(zmax, z[e]);
        for (int e = 0; e < E; ++e) den += expf(z[e] - zmax);
        for (int s = 0; s < top; ++s) {
            int best = -1;
            float bz = 0.f;
            for (int e = 0; e < E; ++e) {
                bool taken = false;
                for (int p = 0; p < s; ++p) taken |= ids[n * top + p] == e;
                if (!taken && (best < 0 || z[e] > bz)) { best = e; bz = z[e]; }
            }
            const float sc = expf(bz - zmax) / den;
            ids[n * top + s] = best;
            weights[n * top + s] = sc;
            chosen += sc;
        }
        for (int s = 0; s < top; ++s) weights[n * top + s] = weights[n * top + s] / (chosen + renorm_eps) * scale;
        return;
    }
    for (int s = 0; s < top; ++s) {
        int best = -1;
        float bc = 0.f, bs = 0.f;
        for (int e = 0; e < E; ++e) {
            bool taken = false;
            for (int p = 0; p < s; ++p) taken |= ids[n * top + p] == e;
            if (taken) continue;
            const float sc = 1.0f / (1.0f + expf(-z[e]));
            const float ch = sc + (correction ? correction[e] : 0.f);
            if (best < 0 || ch > bc) { best = e; bc = ch; bs = sc; }
        }
        ids[n * top + s] = best;
        weights[n * top + s] = bs * scale;
    }
}

extern "C" int jl_moe_route(const float *logits, const float *correction, int64_t N, int32_t E, int32_t top, float scale, int32_t *ids,
                            float *weights, int32_t kind, float renorm_eps, void *stream) {
    if (N <= 0) return JL_OK;
    if (!logits || !ids || !weights || E <= 0 || top <= 0 || top > E) return jl_fail(JL_E_INVALID, "jl_moe_route: null pointer or top > experts");
    if (kind < JL_ROUTE_SIGMOID || kind > JL_ROUTE_TOP_SOFTMAX) return jl_fail(JL_E_INVALID, "jl_moe_route: unknown kind %d", kind);
    moe_route_kernel<<<dim3((unsigned)((N + 255) / 256)), 256, 0, (hipStream_t)stream>>>(logits, correction, N, E, top, scale, ids, weights, kind,
                                                                                         renorm_eps);
    return jl_check_launch("moe_route_kernel");
}

// ---- grouping: one workgroup counts, scans and places (a step holds at most a few 10^5 rows) ----------------------------------------
constexpr int MOE_TM = 64;        // rows of a tile
constexpr int MOE_TN = 64;        // output columns of a tile
constexpr int MOE_TK = 32;        // depth of one LDS stage
constexpr int MOE_MAX_E = 4096;

__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t *__restrict__ ids, int64_t rows, int E, int tile_rows,
                                                          int32_t *__restrict__ perm, int32_t *__restrict__ offsets,
                                                          int32_t *__restrict__ tile_expert, int32_t *__restrict__ tile_row0, int max_tiles) {
    __shared__ int cnt[MOE_MAX_E];
    __shared__ int base[MOE_MAX_E + 1];
    for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int64_t r = threadIdx.x; r < rows; r += 1024) atomicAdd(&cnt[ids[r]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int o = 0, t = 0;
        for (int e = 0; e < E; ++e) {
            base[e] = o;
            offsets[e] = o;
            for (int r = 0; r < cnt[e]; r += tile_rows)
                if (t < max_tiles) { tile_expert[t] = e; tile_row0[t] = o + r; ++t; }
            o += cnt[e];
        }
        offsets[E] = o;
        for (; t < max_tiles; ++t) { tile_expert[t] = -1; tile_row0[t] = 0; }
    }
    __syncthreads();
    // placement: a row's place within its expert is whatever the counter says when it arrives.  The order of an expert's rows
    // changes nothing in the results (every row is computed by itself); only which tile a row lands in differs from run to run.
    for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int64_t r = threadIdx.x; r < rows; r += 1024) {
        const int e = ids[r];
        perm[base[e] + atomicAdd(&cnt[e], 1)] = (int32_t)r;
    }
}

extern "C" int jl_moe_tile_rows(void) { return MOE_TM; }

extern "C" int jl_moe_group(const int32_t *ids, int64_t N, int32_t top, int32_t E, int32_t tile_rows, int32_t *perm, int32_t *offsets,
                            int32_t *tile_expert, int32_t *tile_row0, int32_t max_tiles, void *stream) {
    if (N <= 0) return JL_OK;
    if (!ids || !perm || !offsets || !tile_expert || !tile_row0) return jl_fail(JL_E_INVALID, "jl_moe_group: null pointer");
    if (E <= 0 || E > MOE_MAX_E || top <= 0 || tile_rows <= 0 || (int64_t)max_tiles < N * top / tile_rows + E)
        return jl_fail(JL_E_INVALID, "jl_moe_group: experts must be <= %d and max_tiles >= rows / tile_rows + experts", MOE_MAX_E);
    moe_group_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(ids, N * top, E, tile_rows, perm, offsets, tile_expert, tile_row0, max_tiles);
    return jl_check_launch("moe_group_kernel");
}

// ---- grouped product, any dtype and size: a 64 x 64 tile of one expert's rows per workgroup, float FMAs ------------------------------------
struct MoeAct { int kind; float limit, alpha, shift; };       // the gated unit of JL_MOE_UP_GATED (jl_gated_act's kinds)

// GATED: W holds 2 * n_out rows per expert, gate rows on linear rows; a tile forms both products of its columns and stores the unit
template <typename T, bool GATED>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const T *__restrict__ X, const T *__restrict__ Wt, int mode, int K, int n_out, int top,
                                                        const int32_t *__restrict__ perm, const int32_t *__restrict__ offsets,
                                                        const int32_t *__restrict__ tile_expert, const int32_t *__restrict__ tile_row0,
                                                        const float *__restrict__ weights, void *__restrict__ out, MoeAct act) {
    __shared__ float Xs[MOE_TM][MOE_TK + 1];
    __shared__ float Ws[(GATED ? 2 : 1) * MOE_TN][MOE_TK + 1];
    __shared__ int rin[MOE_TM];
    const int e = tile_expert[blockIdx.x];
    if (e < 0) return;
    const int r0 = tile_row0[blockIdx.x];
    const int nr = offsets[e + 1] - r0 < MOE_TM ? offsets[e + 1] - r0 : MOE_TM;
    const int n0 = blockIdx.y * MOE_TN;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    if (tid < MOE_TM) rin[tid] = tid < nr ? (mode != 1 ? perm[r0 + tid] / top : r0 + tid) : -1;
    const T *We = Wt + (int64_t)e * (GATED ? 2 : 1) * n_out * K;
    float acc[4][4] = {};
    float acu[GATED ? 4 : 1][4] = {};
    for (int k0 = 0; k0 < K; k0 += MOE_TK) {
        __syncthreads();
        for (int i = tid; i < MOE_TM * MOE_TK; i += 256) {
            const int m = i / MOE_TK, kk = i - m * MOE_TK;
            Xs[m][kk] = (rin[m] >= 0 && k0 + kk < K) ? ld_f(X + (int64_t)rin[m] * K + k0 + kk) : 0.f;
        }
        for (int i = tid; i < MOE_TN * MOE_TK; i += 256) {
            const int n = i / MOE_TK, kk = i - n * MOE_TK;
            Ws[n][kk] = (n0 + n < n_out && k0 + kk < K) ? ld_f(We + (int64_t)(n0 + n) * K + k0 + kk) : 0.f;
            if (GATED) Ws[MOE_TN + n][kk] = (n0 + n < n_out && k0 + kk < K) ? ld_f(We + (int64_t)(n_out + n0 + n) * K + k0 + kk) : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int kk = 0; kk < MOE_TK; ++kk) {
            float av[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) av[a] = Xs[ty + 16 * a][kk];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float w = Ws[tx + 16 * c][kk];
#pragma unroll
                for (int a = 0; a < 4; ++a) acc[a][c] += av[a] * w;
                if (GATED) {
                    const float wu = Ws[MOE_TN + tx + 16 * c][kk];
#pragma unroll
                    for (int a = 0; a < 4; ++a) acu[GATED ? a : 0][c] += av[a] * wu;
                }
            }
        }
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int m = ty + 16 * a;
        if (m >= nr) continue;
        const int r = r0 + m;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int n = n0 + tx + 16 * c;
            if (n >= n_out) continue;
            if (GATED) {
                st_f((T *)out + (int64_t)r * n_out + n, gated_unit_f(acc[a][c], acu[GATED ? a : 0][c], act.kind, act.limit, act.alpha, act.shift));
            } else if (mode == JL_MOE_UP_PLAIN) {
                st_f((T *)out + (int64_t)r * n_out + n, acc[a][c]);
            } else if (mode == 0) {
                const float v = fmaxf(acc[a][c], 0.f);
                st_f((T *)out + (int64_t)r * n_out + n, v * v);
            } else {
                const int p = perm[r];
                ((float *)out)[(int64_t)p * n_out + n] = acc[a][c] * weights[p];
            }
        }
    }
}

// ---- grouped product on the matrix cores (bfloat16, K a multiple of 8) -----------------------------------------------------------------
// A 64 x 128 tile per workgroup, four wavefronts side by side over the columns: each holds two 32 x 32 accumulators (rows 0-31 and
// 32-63) and feeds v_mfma_f32_32x32x8_bf16 from LDS stages of depth 32.  Operand layout of that instruction: lane l supplies row
// (A) or column (B) l % 32 with the four consecutive depths 4 * (l / 32) ..; accumulator i of lane l is row 8 * (i / 4) + 4 * (l / 32)
// + i % 4, column l % 32.
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short bf16x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
constexpr int MM_TN = 128, MM_TK = 32, MM_LD = 36;     // LDS row stride in bf16 (72 bytes: rows 16 apart share a bank, no worse)

// GATED: the tile's 128 columns of the gate AND of the linear branch (rows n_out further on in W): every wavefront holds four
// accumulators, the A fragments serve both products, and the epilogue stores the gated unit.
template <bool GATED>
__global__ __launch_bounds__(256) void moe_gemm_mfma_kernel(const bf16_t *__restrict__ X, const bf16_t *__restrict__ Wt, int mode, int K, int n_out,
                                                             int top, const int32_t *__restrict__ perm, const int32_t *__restrict__ offsets,
                                                             const int32_t *__restrict__ tile_expert, const int32_t *__restrict__ tile_row0,
                                                             const float *__restrict__ weights, void *__restrict__ out, MoeAct act) {
    __shared__ __attribute__((aligned(16))) bf16_t As[MOE_TM * MM_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[(GATED ? 2 : 1) * MM_TN * MM_LD];
    __shared__ int rin[MOE_TM];
    const int e = tile_expert[blockIdx.x];
    if (e < 0) return;
    const int r0 = tile_row0[blockIdx.x];
    const int nr = offsets[e + 1] - r0 < MOE_TM ? offsets[e + 1] - r0 : MOE_TM;
    const int n0 = blockIdx.y * MM_TN;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    if (tid < MOE_TM) rin[tid] = tid < nr ? (mode != 1 ? perm[r0 + tid] / top : r0 + tid) : -1;
    __syncthreads();
    const bf16_t *We = Wt + (int64_t)e * (GATED ? 2 : 1) * n_out * K;
    // loaders: 8 bf16 (16 bytes) per thread and row segment; A 64 x 32 = 256 segments, B 128 x 32 = 512 segments (twice that when GATED)
    const int a_row = tid >> 2, a_seg = (tid & 3) * 8;
    const int64_t a_src = rin[a_row] >= 0 ? (int64_t)rin[a_row] * K : -1;
    f32x16_t acc0 = {0}, acc1 = {0}, acu0 = {0}, acu1 = {0};
    // a stage's rows travel from memory while the previous stage is multiplied: loaded into registers one iteration ahead
    constexpr int NB = GATED ? 4 : 2;
    uint4 av, bv[NB];
    auto fetch = [&](int k0) {
        av = make_uint4(0, 0, 0, 0);
        if (a_src >= 0 && k0 + a_seg < K) av = *(const uint4 *)(X + a_src + k0 + a_seg);
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int n = (tid >> 2) + 64 * (i & 1);
            bv[i] = make_uint4(0, 0, 0, 0);
            if (n0 + n < n_out && k0 + a_seg < K) bv[i] = *(const uint4 *)(We + (int64_t)((i >> 1) * n_out + n0 + n) * K + k0 + a_seg);
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += MM_TK) {
        __syncthreads();                                   // the previous stage's readers are done
        {
            uint2 *d = (uint2 *)(As + a_row * MM_LD + a_seg);       // rows are 72 bytes apart: 8-byte stores stay aligned
            d[0] = make_uint2(av.x, av.y);
            d[1] = make_uint2(av.z, av.w);
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            uint2 *d = (uint2 *)(Bs + ((tid >> 2) + 64 * i) * MM_LD + a_seg);     // rows 0-127: gate (or the only) columns, 128-255: linear branch
            d[0] = make_uint2(bv[i].x, bv[i].y);
            d[1] = make_uint2(bv[i].z, bv[i].w);
        }
        __syncthreads();
        if (k0 + MM_TK < K) fetch(k0 + MM_TK);
#pragma unroll
        for (int kk = 0; kk < MM_TK; kk += 8) {
            const int ko = kk + 4 * (lane >> 5);
            const bf16x4_t b = *(const bf16x4_t *)(Bs + (wave * 32 + (lane & 31)) * MM_LD + ko);
            const bf16x4_t a0 = *(const bf16x4_t *)(As + (lane & 31) * MM_LD + ko);
            const bf16x4_t a1 = *(const bf16x4_t *)(As + (32 + (lane & 31)) * MM_LD + ko);
            acc0 = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a0, b, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a1, b, acc1, 0, 0, 0);
            if (GATED) {
                const bf16x4_t bu = *(const bf16x4_t *)(Bs + (MM_TN + wave * 32 + (lane & 31)) * MM_LD + ko);
                acu0 = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a0, bu, acu0, 0, 0, 0);
                acu1 = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(a1, bu, acu1, 0, 0, 0);
            }
        }
    }
    const int n = n0 + wave * 32 + (lane & 31);
    if (n >= n_out) return;
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int m = 32 * half + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
            if (m >= nr) continue;
            const float c = half ? acc1[i] : acc0[i];
            const int r = r0 + m;
            if (GATED) {
                st_f((bf16_t *)out + (int64_t)r * n_out + n, gated_unit_f(c, half ? acu1[i] : acu0[i], act.kind, act.limit, act.alpha, act.shift));
            } else if (mode == JL_MOE_UP_PLAIN) {
                st_f((bf16_t *)out + (int64_t)r * n_out + n, c);
            } else if (mode == 0) {
                const float v = fmaxf(c, 0.f);
                st_f((bf16_t *)out + (int64_t)r * n_out + n, v * v);
            } else {
                const int p = perm[r];
                ((float *)out)[(int64_t)p * n_out + n] = c * weights[p];
            }
        }
}

static int moe_gemm_launch(const void *X, const void *Wt, int dtype, int32_t mode, int32_t K, int32_t n_out, int32_t top, const int32_t *perm,
                           const int32_t *offsets, const int32_t *tile_expert, const int32_t *tile_row0, int32_t max_tiles, const float *weights,
                           void *out, const MoeAct *act, void *stream) {
    static const bool no_mfma = getenv("JL_MOE_NO_MFMA") != nullptr;      // A/B switch for measurements
    const MoeAct none = {0, 0.f, 0.f, 0.f};
    if (!no_mfma && dtype == JL_BF16 && K % 8 == 0 && ((uintptr_t)X % 16) == 0 && ((uintptr_t)Wt % 16) == 0) {
        const dim3 mgrid((unsigned)max_tiles, (unsigned)((n_out + MM_TN - 1) / MM_TN));
        if (act)
            moe_gemm_mfma_kernel<true><<<mgrid, 256, 0, (hipStream_t)stream>>>((const bf16_t *)X, (const bf16_t *)Wt, mode, K, n_out, top, perm, offsets,
                                                                              tile_expert, tile_row0, weights, out, *act);
        else
            moe_gemm_mfma_kernel<false><<<mgrid, 256, 0, (hipStream_t)stream>>>((const bf16_t *)X, (const bf16_t *)Wt, mode, K, n_out, top, perm, offsets,
                                                                               tile_expert, tile_row0, weights, out, none);
        return jl_check_launch("moe_gemm_mfma_kernel");
    }
    const dim3 grid((unsigned)max_tiles, (unsigned)((n_out + MOE_TN - 1) / MOE_TN));
    if (act)
        JL_DISPATCH(dtype, moe_gemm_kernel<T, true><<<grid, 256, 0, (hipStream_t)stream>>>((const T *)X, (const T *)Wt, mode, K, n_out, top, perm, offsets,
                                                                                           tile_expert, tile_row0, weights, out, *act));
    else
        JL_DISPATCH(dtype, moe_gemm_kernel<T, false><<<grid, 256, 0, (hipStream_t)stream>>>((const T *)X, (const T *)Wt, mode, K, n_out, top, perm, offsets,
                                                                                            tile_expert, tile_row0, weights, out, none));
    return jl_check_launch("moe_gemm_kernel");
}

extern "C" int jl_moe_gemm(const void *X, const void *Wt, int dtype, int32_t mode, int32_t K, int32_t n_out, int32_t top,
                           const int32_t *perm, const int32_t *offsets, const int32_t *tile_expert, const int32_t *tile_row0,
                           int32_t max_tiles, const float *weights, void *out, void *stream) {
    if (max_tiles <= 0) return JL_OK;
    if (!X || !Wt || !perm || !offsets || !tile_expert || !tile_row0 || !out || (mode == 1 && !weights))
        return jl_fail(JL_E_INVALID, "jl_moe_gemm: null pointer");
    if (K <= 0 || n_out <= 0 || top <= 0 || (mode != 0 && mode != 1 && mode != JL_MOE_UP_PLAIN)) return jl_fail(JL_E_INVALID, "jl_moe_gemm: bad sizes or mode");
    return moe_gemm_launch(X, Wt, dtype, mode, K, n_out, top, perm, offsets, tile_expert, tile_row0, max_tiles, weights, out, nullptr, stream);
}

extern "C" int jl_moe_gemm_gated(const void *X, const void *Wt, int dtype, int32_t K, int32_t ff, int32_t top, const int32_t *perm,
                                 const int32_t *offsets, const int32_t *tile_expert, const int32_t *tile_row0, int32_t max_tiles, int32_t kind,
                                 float limit, float alpha, float shift, void *out, void *stream) {
    if (max_tiles <= 0) return JL_OK;
    if (!X || !Wt || !perm || !offsets || !tile_expert || !tile_row0 || !out) return jl_fail(JL_E_INVALID, "jl_moe_gemm_gated: null pointer");
    if (K <= 0 || ff <= 0 || top <= 0 || kind < JL_ACT_GELU_TANH || kind > JL_ACT_GELU_ERF)
        return jl_fail(JL_E_INVALID, "jl_moe_gemm_gated: bad sizes or kind");
    const MoeAct act = {kind, limit, alpha, shift};
    return moe_gemm_launch(X, Wt, dtype, JL_MOE_UP_PLAIN, K, ff, top, perm, offsets, tile_expert, tile_row0, max_tiles, nullptr, out, &act, stream);
}
