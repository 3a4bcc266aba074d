// jl_delta.hip — the gated delta rule: a recurrent mixer whose float state S [D, Dv] per (request slot, head) is decayed, corrected towards
// the current value along the current key, and read with the current query, token by token:
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// with q, k unit vectors per head (q also times q_scale), beta = sigmoid(b) and g = exp(-exp(A_log_h) softplus(a + dt_bias_h)) per head and
// token, and the output brought to unit RMS per head, times a weight over Dv, times silu(gate).  Everything but the inputs is float.
#include "jl_common.h"

// One workgroup per (request, head).  The columns of S are independent of each other, so column j is owned by LPC adjacent lanes, each
// with DMAX / LPC consecutive rows in registers; the two dot products of a token (k . S_j and q . S_j) are partial sums per lane joined by
// LPC - 1 exchanges.  Tokens are taken DL_TT at a time: raw queries and keys go to LDS, a wavefront per token makes them unit vectors, one
// thread per token evaluates the decay and the step size; the per-head sums of squares of the outputs are reduced once per group.
constexpr int DL_TT = 8;

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T, typename TQ, int DMAX, int LPC>
__global__ __launch_bounds__(1024) void delta_rule_kernel(const TQ *__restrict__ qkv, int64_t qkv_ld, int q_col, int k_col, int v_col,
                                                           const T *__restrict__ proj, int64_t ld, int a_col, int b_col, int g_col,
                                                           const float *__restrict__ A_log, const float *__restrict__ dt_bias,
                                                           const float *__restrict__ norm_w, const int32_t *__restrict__ seq, int H, int G, int D, int Dv,
                                                           float unit_eps, float q_scale, float eps, float *__restrict__ state, T *__restrict__ out) {
    constexpr int DPER = DMAX / LPC;
    extern __shared__ float lds[];
    float *qs = lds;                                   // [TT][DMAX]
    float *ks = qs + DL_TT * DMAX;                     // [TT][DMAX]
    float *gs = ks + DL_TT * DMAX;                     // [TT] decay
    float *bs = gs + DL_TT;                            // [TT] step size
    float *red = bs + DL_TT;                           // [TT][16]
    const int b = blockIdx.x / H, h = blockIdx.x - b * H, kh = h / (H / G);
    const int row0 = seq[4 * b], cnt = seq[4 * b + 1], pos0 = seq[4 * b + 2], slot = seq[4 * b + 3];
    if (cnt <= 0) return;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, nw = (blockDim.x + 63) >> 6;
    const int j = tid / LPC, sub = tid - j * LPC, d0 = sub * DPER;
    const bool live = j < Dv;
    const float neg_rate = -expf(A_log[h]), bias = dt_bias[h];
    float *sp = state + ((int64_t)slot * H + h) * D * Dv;
    float S[DPER];
#pragma unroll
    for (int i = 0; i < DPER; ++i) S[i] = (live && d0 + i < D && pos0 > 0) ? sp[(int64_t)(d0 + i) * Dv + j] : 0.f;

    for (int t0 = 0; t0 < cnt; t0 += DL_TT) {
        const int nt = cnt - t0 < DL_TT ? cnt - t0 : DL_TT;
        __syncthreads();
        for (int e = tid; e < nt * DMAX; e += blockDim.x) {
            const int tt = e / DMAX, d = e - tt * DMAX;
            const TQ *row = qkv + (int64_t)(row0 + t0 + tt) * qkv_ld + kh * D;
            qs[e] = d < D ? ld_f(row + q_col + d) : 0.f;
            ks[e] = d < D ? ld_f(row + k_col + d) : 0.f;
        }
        if (tid < nt) {
            const T *row = proj + (int64_t)(row0 + t0 + tid) * ld;
            gs[tid] = expf(neg_rate * softplus_f(ld_f(row + a_col + h) + bias));
            bs[tid] = 1.0f / (1.0f + expf(-ld_f(row + b_col + h)));
        }
        __syncthreads();
        for (int tt = wave; tt < nt; tt += nw) {               // unit vectors: a wavefront per token
            float sq = 0.f, sk = 0.f;
            for (int d = lane; d < D; d += 64) { const float a = qs[tt * DMAX + d], c = ks[tt * DMAX + d]; sq += a * a; sk += c * c; }
            sq = wave_sum_f32(sq);
            sk = wave_sum_f32(sk);
            const float rq = q_scale / sqrtf(sq + unit_eps), rk = 1.0f / sqrtf(sk + unit_eps);
            for (int d = lane; d < D; d += 64) { qs[tt * DMAX + d] *= rq; ks[tt * DMAX + d] *= rk; }
        }
        __syncthreads();
        float o[DL_TT];
#pragma unroll
        for (int tt = 0; tt < DL_TT; ++tt) {
            o[tt] = 0.f;
            if (tt < nt) {
                const float v = live ? ld_f(qkv + (int64_t)(row0 + t0 + tt) * qkv_ld + v_col + h * Dv + j) : 0.f;
                const float *qp = qs + tt * DMAX + d0, *kp = ks + tt * DMAX + d0;
                const float g = gs[tt], beta = bs[tt];
                float dot = 0.f;
#pragma unroll
                for (int i = 0; i < DPER; ++i) dot += kp[i] * S[i];
#pragma unroll
                for (int off = 1; off < LPC; off <<= 1) dot += __shfl_xor(dot, off, 64);
                const float u = beta * (v - g * dot);
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < DPER; ++i) {
                    S[i] = g * S[i] + kp[i] * u;
                    acc += S[i] * qp[i];
                }
#pragma unroll
                for (int off = 1; off < LPC; off <<= 1) acc += __shfl_xor(acc, off, 64);
                o[tt] = acc;
                const float ss = wave_sum_f32((live && sub == 0) ? acc * acc : 0.f);
                if (lane == 0) red[tt * 16 + wave] = ss;
            }
        }
        __syncthreads();
#pragma unroll
        for (int tt = 0; tt < DL_TT; ++tt)
            if (tt < nt && live && sub == 0) {
                float ss = 0.f;
                for (int w = 0; w < nw; ++w) ss += red[tt * 16 + w];
                const float r = 1.0f / sqrtf(ss / (float)Dv + eps);
                const int64_t n = row0 + t0 + tt;
                const float gt = ld_f(proj + n * ld + g_col + h * Dv + j);
                st_f(out + n * ((int64_t)H * Dv) + h * Dv + j, o[tt] * r * norm_w[j] * silu_f(gt));
            }
    }
    if (live)
#pragma unroll
        for (int i = 0; i < DPER; ++i)
            if (d0 + i < D) sp[(int64_t)(d0 + i) * Dv + j] = S[i];
}


// ---- long portions: the columns of S shared out over single-wavefront workgroups -------------------------------------------------------------
// A prompt's portion is a chain of cnt dependent steps per (request, head); what shortens it is less work per step and nothing to wait for
// inside it.  Here a workgroup is ONE wavefront that owns 64 / LPC columns of one head's state (grid.y walks the head's columns), so a step is
// DMAX / LPC * 3 multiply-adds per lane, and the chip runs B * H * Dv * LPC / 64 such chains side by side.  Every wavefront stages the group's
// queries and keys itself (eight lanes per token make them unit vectors) and fetches the next group's inputs into registers before it starts
// on the current one.  The outputs leave unnormalised (float): the norm over a head's Dv values spans workgroups and is delta_out_kernel's.
constexpr int DC_TT = 8;        // tokens per group = 64 lanes / 8 lanes per token in the unit-vector stage

// sum over the LPC adjacent lanes that share a column; four lanes are a quad, whose exchanges are register moves (DPP), not LDS traffic
template <int LPC>
__device__ __forceinline__ float column_sum(float v) {
    if constexpr (LPC == 4 || LPC == 8) {
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));      // quad_perm [1, 0, 3, 2]
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));      // quad_perm [2, 3, 0, 1]
        if constexpr (LPC == 8)                                                                           // lane i <-> 7 - i of each eight: the other quad's sum
            v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));
    } else {
#pragma unroll
        for (int off = 1; off < LPC; off <<= 1) v += __shfl_xor(v, off, 64);
    }
    return v;
}

template <typename T, int DMAX, int LPC>
__global__ __launch_bounds__(64) void delta_cols_kernel(const float *__restrict__ qkv, int64_t qkv_ld, int q_col, int k_col, int v_col,
                                                         const T *__restrict__ proj, int64_t ld, int a_col, int b_col, const float *__restrict__ A_log,
                                                         const float *__restrict__ dt_bias, const int32_t *__restrict__ seq, int H, int G, int D, int Dv,
                                                         float unit_eps, float q_scale, float *__restrict__ state, float *__restrict__ raw) {
    // a token's row in LDS: the LPC lanes of a column read DPER consecutive values each, DPER apart — four floats between the parts keep
    // their 16-byte reads on different banks
    constexpr int DPER = DMAX / LPC, CPW = 64 / LPC, PRE = DC_TT * DMAX / 64, ROW = DMAX + 4 * LPC;
    __shared__ float qs[DC_TT * ROW], ks[DC_TT * ROW], gs[DC_TT], bs[DC_TT];
    auto at = [](int tt, int d) { return tt * ROW + d + (d / DPER) * 4; };
    const int b = blockIdx.x / H, h = blockIdx.x - b * H, kh = h / (H / G);
    const int row0 = seq[4 * b], cnt = seq[4 * b + 1], pos0 = seq[4 * b + 2], slot = seq[4 * b + 3];
    if (cnt <= 0) return;
    const int lane = threadIdx.x, j = blockIdx.y * CPW + lane / LPC, sub = lane % LPC, d0 = sub * DPER;
    const bool live = j < Dv;
    const float neg_rate = -expf(A_log[h]), bias = dt_bias[h];
    float *sp = state + ((int64_t)slot * H + h) * D * Dv;
    float S[DPER];
#pragma unroll
    for (int i = 0; i < DPER; ++i) S[i] = (live && d0 + i < D && pos0 > 0) ? sp[(int64_t)(d0 + i) * Dv + j] : 0.f;
    float pq[PRE], pk[PRE], pv[DC_TT], pa = 0.f, pb = 0.f;
    auto fetch = [&](int t0) {
        const int nt = cnt - t0 < DC_TT ? cnt - t0 : DC_TT;
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int e = i * 64 + lane, tt = e / DMAX, d = e - tt * DMAX;
            const bool ok = tt < nt && d < D;
            const float *row = qkv + (int64_t)(row0 + t0 + tt) * qkv_ld + kh * D + d;
            pq[i] = ok ? row[q_col] : 0.f;
            pk[i] = ok ? row[k_col] : 0.f;
        }
#pragma unroll
        for (int tt = 0; tt < DC_TT; ++tt) pv[tt] = (tt < nt && live) ? qkv[(int64_t)(row0 + t0 + tt) * qkv_ld + v_col + h * Dv + j] : 0.f;
        if (lane < nt) {
            const T *row = proj + (int64_t)(row0 + t0 + lane) * ld;
            pa = ld_f(row + a_col + h);
            pb = ld_f(row + b_col + h);
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < cnt; t0 += DC_TT) {
        const int nt = cnt - t0 < DC_TT ? cnt - t0 : DC_TT;
        __syncthreads();                                        // the group before has been read
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int e = i * 64 + lane, tt = e / DMAX, d = e - tt * DMAX;
            qs[at(tt, d)] = pq[i];
            ks[at(tt, d)] = pk[i];
        }
        if (lane < nt) {
            gs[lane] = expf(neg_rate * softplus_f(pa + bias));
            bs[lane] = 1.0f / (1.0f + expf(-pb));
        }
        float v[DC_TT];
#pragma unroll
        for (int tt = 0; tt < DC_TT; ++tt) v[tt] = pv[tt];
        __syncthreads();
        {                                                       // unit vectors: eight lanes per token, its values in registers between the two passes
            const int tt = lane >> 3, s8 = lane & 7;
            float qv[DMAX / 8], kv[DMAX / 8];
            float sq = 0.f, sk = 0.f;
#pragma unroll
            for (int i = 0; i < DMAX / 8; ++i) {
                const int d = s8 + 8 * i;
                qv[i] = qs[at(tt, d)];
                kv[i] = ks[at(tt, d)];
                sq += qv[i] * qv[i];
                sk += kv[i] * kv[i];
            }
#pragma unroll
            for (int off = 1; off < 8; off <<= 1) { sq += __shfl_xor(sq, off, 64); sk += __shfl_xor(sk, off, 64); }
            const float rq = q_scale / sqrtf(sq + unit_eps), rk = 1.0f / sqrtf(sk + unit_eps);
#pragma unroll
            for (int i = 0; i < DMAX / 8; ++i) {
                const int d = s8 + 8 * i;
                qs[at(tt, d)] = qv[i] * rq;
                ks[at(tt, d)] = kv[i] * rk;
            }
        }
        __syncthreads();
        if (t0 + DC_TT < cnt) fetch(t0 + DC_TT);                // in flight while this group's steps run
#pragma unroll
        for (int tt = 0; tt < DC_TT; ++tt) {
            if (tt < nt) {
                const float *qp = qs + tt * ROW + d0 + sub * 4, *kp = ks + tt * ROW + d0 + sub * 4;
                const float g = gs[tt], beta = bs[tt];
                float dot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < DPER; ++i) dot[i & 3] += kp[i] * S[i];
                const float dsum = column_sum<LPC>((dot[0] + dot[1]) + (dot[2] + dot[3]));
                const float u = beta * (v[tt] - g * dsum);
                float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int i = 0; i < DPER; ++i) {
                    S[i] = g * S[i] + kp[i] * u;
                    acc[i & 3] += S[i] * qp[i];
                }
                const float o = column_sum<LPC>((acc[0] + acc[1]) + (acc[2] + acc[3]));
                if (live && sub == 0) raw[(int64_t)(row0 + t0 + tt) * ((int64_t)H * Dv) + h * Dv + j] = o;
            }
        }
    }
    if (live)
#pragma unroll
        for (int i = 0; i < DPER; ++i)
            if (d0 + i < D) sp[(int64_t)(d0 + i) * Dv + j] = S[i];
}

// out_h(t) = o / sqrt(mean(o^2) + eps) * norm_w * silu(gate_h(t)): a wavefront per (token, head)
template <typename T>
__global__ __launch_bounds__(256) void delta_out_kernel(const float *__restrict__ raw, const T *__restrict__ proj, int64_t ld, int g_col,
                                                         const float *__restrict__ norm_w, int64_t NH, int H, int Dv, float eps, T *__restrict__ out) {
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= NH) return;
    const int lane = threadIdx.x & 63;
    const int64_t n = r / H;
    const int h = (int)(r - n * H);
    const float *o = raw + r * Dv;
    float ss = 0.f;
    for (int c = lane; c < Dv; c += 64) ss += o[c] * o[c];
    ss = wave_sum_f32(ss);
    const float rr = 1.0f / sqrtf(ss / (float)Dv + eps);
    for (int c = lane; c < Dv; c += 64) st_f(out + r * Dv + c, o[c] * rr * norm_w[c] * silu_f(ld_f(proj + n * ld + g_col + h * Dv + c)));
}

template <typename T, int DMAX>
static int delta_cols_launch(const void *qkv, int64_t qkv_ld, int q_col, int k_col, int v_col, const void *proj, int64_t ld, int a_col, int b_col, int g_col,
                             const float *A_log, const float *dt_bias, const float *norm_w, const int32_t *seq, int B, int64_t N, int H, int G, int D, int Dv,
                             float unit_eps, float q_scale, float eps, float *state, float *raw, void *out, hipStream_t st) {
    constexpr int LPC = DMAX >= 128 ? 8 : 4;            // 16 or 32 rows of a column per lane
    const dim3 grid((unsigned)(B * H), (unsigned)((Dv + 64 / LPC - 1) / (64 / LPC)));
    delta_cols_kernel<T, DMAX, LPC><<<grid, 64, 0, st>>>((const float *)qkv, qkv_ld, q_col, k_col, v_col, (const T *)proj, ld, a_col, b_col, A_log, dt_bias, seq, H, G,
                                                         D, Dv, unit_eps, q_scale, state, raw);
    int rc = jl_check_launch("delta_cols_kernel");
    if (rc != JL_OK) return rc;
    const int64_t NH = N * H;
    delta_out_kernel<T><<<dim3((unsigned)((NH + 3) / 4)), 256, 0, st>>>(raw, (const T *)proj, ld, g_col, norm_w, NH, H, Dv, eps, (T *)out);
    return jl_check_launch("delta_out_kernel");
}

template <typename T, typename TQ, int DMAX, int LPC>
static int delta_launch(const void *qkv, int64_t qkv_ld, int q_col, int k_col, int v_col, const void *proj, int64_t ld, int a_col, int b_col, int g_col,
                        const float *A_log, const float *dt_bias, const float *norm_w, const int32_t *seq, int B, int H, int G, int D, int Dv, float unit_eps,
                        float q_scale, float eps, float *state, void *out, hipStream_t st) {
    const int threads = (Dv * LPC + 63) / 64 * 64;
    const size_t lds = (size_t)(2 * DL_TT * DMAX + 2 * DL_TT + DL_TT * 16) * 4;
    delta_rule_kernel<T, TQ, DMAX, LPC><<<dim3((unsigned)(B * H)), threads, lds, st>>>((const TQ *)qkv, qkv_ld, q_col, k_col, v_col, (const T *)proj, ld, a_col,
                                                                                      b_col, g_col, A_log, dt_bias, norm_w, seq, H, G, D, Dv, unit_eps,
                                                                                      q_scale, eps, state, (T *)out);
    return jl_check_launch("delta_rule_kernel");
}

extern "C" int jl_delta_rule(const void *qkv, int qkv_dtype, int64_t qkv_ld, int32_t q_col, int32_t k_col, int32_t v_col, const void *proj, int dtype,
                             int64_t ld, int32_t a_col, int32_t b_col, int32_t g_col, const float *A_log, const float *dt_bias, const float *norm_w,
                             const int32_t *seq, int32_t B, int64_t N, int32_t H, int32_t G, int32_t D, int32_t Dv, float unit_eps, float q_scale, float eps,
                             float *state, float *raw, void *out, void *stream) {
    if (B <= 0) return JL_OK;
    if (!qkv || !proj || !A_log || !dt_bias || !norm_w || !seq || !state || !out) return jl_fail(JL_E_INVALID, "jl_delta_rule: null pointer");
    if (H <= 0 || G <= 0 || H % G || D <= 0 || D > 256 || Dv <= 0 || Dv > 1024)
        return jl_fail(JL_E_INVALID, "jl_delta_rule: heads must be a multiple of the key heads, D <= 256, Dv <= 1024");
    if (q_col < 0 || k_col < 0 || v_col < 0 || a_col < 0 || b_col < 0 || g_col < 0 || q_col + (int64_t)G * D > qkv_ld || k_col + (int64_t)G * D > qkv_ld ||
        v_col + (int64_t)H * Dv > qkv_ld || a_col + (int64_t)H > ld || b_col + (int64_t)H > ld || g_col + (int64_t)H * Dv > ld)
        return jl_fail(JL_E_INVALID, "jl_delta_rule: columns do not fit the rows");
    hipStream_t st = (hipStream_t)stream;
    if (raw) {                                          // long portions: the state's columns shared out over single-wavefront workgroups
        if (qkv_dtype != JL_F32 || N <= 0) return jl_fail(JL_E_INVALID, "jl_delta_rule: q, k, v after their convolution are float; N rows of scratch");
#define DC_CASE(DM) JL_DISPATCH(dtype, return (delta_cols_launch<T, DM>(qkv, qkv_ld, q_col, k_col, v_col, proj, ld, a_col, b_col, g_col, A_log, dt_bias, norm_w, \
                                                                         seq, B, N, H, G, D, Dv, unit_eps, q_scale, eps, state, raw, out, st)))
        if (D <= 64) DC_CASE(64);
        else if (D <= 128) DC_CASE(128);
        else DC_CASE(256);
#undef DC_CASE
    }
    const int lpc = Dv * 4 <= 1024 ? 4 : 1;             // four lanes per column while the workgroup holds them
#define DL_ARGS qkv, qkv_ld, q_col, k_col, v_col, proj, ld, a_col, b_col, g_col, A_log, dt_bias, norm_w, seq, B, H, G, D, Dv, unit_eps, q_scale, eps, state, out, st
#define DL_CASE(N)                                                                                                        \
    do {                                                                                                                  \
        if (dtype == JL_BF16 && qkv_dtype == JL_F32) return lpc == 4 ? delta_launch<bf16_t, float, N, 4>(DL_ARGS) : delta_launch<bf16_t, float, N, 1>(DL_ARGS); \
        if (dtype == JL_F32 && qkv_dtype == JL_F32) return lpc == 4 ? delta_launch<float, float, N, 4>(DL_ARGS) : delta_launch<float, float, N, 1>(DL_ARGS);   \
        return jl_fail(JL_E_INVALID, "jl_delta_rule: q, k, v after their convolution are float");                          \
    } while (0)
    if (D <= 64) DL_CASE(64);
    else if (D <= 128) DL_CASE(128);
    else DL_CASE(256);
#undef DL_CASE
#undef DL_ARGS
    return JL_OK;
}
