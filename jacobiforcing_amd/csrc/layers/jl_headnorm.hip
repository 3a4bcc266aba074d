// jl_headnorm.hip — per-head query / key stage in front of attention: an optional rotation by position (rotate-half pairs on the first
// dimensions of every head), the RMS norm of every head's vector (with or without a weight), a position-dependent query temperature,
// several score maps per head (differential attention), the cache append; and the combination of two maps' outputs.
#include "jl_common.h"

// One workgroup per token, a wavefront per D-vector (queries first, then keys), then the values.  Vectors are written map-major.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_append_kernel(const T *__restrict__ proj, int64_t ld, int q_col, int k_col, int v_col, int H, int G,
                                                                int M, int D, int GDv, const T *__restrict__ wq, const T *__restrict__ wk, float eps,
                                                                float t_coef, int t_every, const int32_t *__restrict__ pos, T *__restrict__ q_out,
                                                                int64_t q_map_stride, T *__restrict__ k_cache, T *__restrict__ v_cache,
                                                                const int64_t *__restrict__ slot, int rot_dims, const float *__restrict__ cos_t,
                                                                const float *__restrict__ sin_t) {
    const int64_t n = blockIdx.x;
    const T *row = proj + n * ld;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t sl = slot[n];
    float temp = 1.0f;
    if (t_coef != 0.f) temp = 1.0f + t_coef * logf((float)((pos[n] + 1) / t_every + 1));
    const int nq = H * M, nk = G * M, half = rot_dims / 2;
    const float *ct = rot_dims ? cos_t + (int64_t)pos[n] * half : nullptr, *sn = rot_dims ? sin_t + (int64_t)pos[n] * half : nullptr;
    for (int vec = wave; vec < nq + nk; vec += 4) {
        const bool is_q = vec < nq;
        const int idx = is_q ? vec : vec - nq;                  // head-major index: head * M + map
        const int head = idx / M, map = idx - head * M;
        const T *src = row + (is_q ? q_col : k_col) + (int64_t)idx * D;
        // element d after the rotation: (u, v) = (d, d + half) -> (u cos - v sin, v cos + u sin); dimensions from rot_dims on pass
        auto turned = [&](int d) {
            const float x = ld_f(src + d);
            if (d >= rot_dims) return x;
            return d < half ? x * ct[d] - ld_f(src + d + half) * sn[d] : x * ct[d - half] + ld_f(src + d - half) * sn[d - half];
        };
        float ss = 0.f;
        for (int d = lane; d < D; d += 64) { const float v = turned(d); ss += v * v; }
        ss = wave_sum_f32(ss);
        const float r = 1.0f / sqrtf(ss / (float)D + eps);
        if (is_q) {
            // q_map_stride 0: [N, M, H, D]; else [M, N, H, D] with the maps q_map_stride elements apart
            T *dst = q_map_stride ? q_out + map * q_map_stride + n * ((int64_t)H * D) + (int64_t)head * D
                                  : q_out + n * ((int64_t)nq * D) + ((int64_t)map * H + head) * D;
            for (int d = lane; d < D; d += 64) st_f(dst + d, turned(d) * r * (wq ? ld_f(wq + d) : 1.0f) * temp);
        } else if (sl >= 0) {
            T *dst = k_cache + sl * ((int64_t)nk * D) + ((int64_t)map * G + head) * D;
            for (int d = lane; d < D; d += 64) st_f(dst + d, turned(d) * r * (wk ? ld_f(wk + d) : 1.0f));
        }
    }
    if (sl >= 0)
        for (int c = threadIdx.x; c < GDv; c += 256) v_cache[sl * GDv + c] = row[v_col + c];
}

// four elements at a time (8 bytes of bfloat16, 16 of float)
__device__ __forceinline__ void ld4(const float *p, float (&v)[4]) { const float4 t = *(const float4 *)p; v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
__device__ __forceinline__ void ld4(const bf16_t *p, float (&v)[4]) {
    const uint2 t = *(const uint2 *)p;
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u); v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ __forceinline__ void st4(float *p, const float (&v)[4]) { *(float4 *)p = make_float4(v[0], v[1], v[2], v[3]); }
__device__ __forceinline__ void st4(bf16_t *p, const float (&v)[4]) {
    bf16_t h[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) st_f(h + i, v[i]);
    *(uint2 *)p = make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
}

// The same with LPV lanes per D-vector (a power of two, 4 * LPV >= D, D % 4 == 0, every column offset and row stride a multiple of
// four): a wavefront normalises 64 / LPV vectors at a time, four elements per lane and load.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_append_vec_kernel(const T *__restrict__ proj, int64_t ld, int q_col, int k_col, int v_col, int H, int G,
                                                                    int M, int D, int GDv, const T *__restrict__ wq, const T *__restrict__ wk, float eps,
                                                                    float t_coef, int t_every, const int32_t *__restrict__ pos, T *__restrict__ q_out,
                                                                    int64_t q_map_stride, T *__restrict__ k_cache, T *__restrict__ v_cache,
                                                                    const int64_t *__restrict__ slot, int LPV, int rot_dims,
                                                                    const float *__restrict__ cos_t, const float *__restrict__ sin_t) {
    const int64_t n = blockIdx.x;
    const T *row = proj + n * ld;
    const int sub = threadIdx.x & (LPV - 1), group = threadIdx.x / LPV, groups = 256 / LPV;
    const int64_t sl = slot[n];
    float temp = 1.0f;
    if (t_coef != 0.f) temp = 1.0f + t_coef * logf((float)((pos[n] + 1) / t_every + 1));
    const int nq = H * M, nk = G * M, d = 4 * sub, half = rot_dims / 2;
    // the rotation's pairs (i, i + half) lie four-element groups apart (half % 4 == 0): this lane's partner group and its angles
    const bool turn = d < rot_dims;
    const int pd = d < half ? d + half : d - half;
    float cs[4] = {1.f, 1.f, 1.f, 1.f}, sn[4] = {0.f, 0.f, 0.f, 0.f};
    if (turn) {
        const int64_t a0 = (int64_t)pos[n] * half + (d < half ? d : d - half);
        ld4(cos_t + a0, cs);
        ld4(sin_t + a0, sn);
        if (d < half)                                           // first of a pair: u cos - v sin; second: v cos + u sin
#pragma unroll
            for (int i = 0; i < 4; ++i) sn[i] = -sn[i];
    }
    for (int v0 = 0; v0 < nq + nk; v0 += groups) {              // every lane takes part in the shuffles of its round
        const int vec = v0 + group;
        const bool live = vec < nq + nk && d < D;
        const bool is_q = vec < nq;
        const int idx = is_q ? vec : vec - nq;
        const int head = idx / M, map = idx - head * M;
        float x[4] = {0.f, 0.f, 0.f, 0.f};
        if (live) ld4(row + (is_q ? q_col : k_col) + (int64_t)idx * D + d, x);
        if (live && turn) {
            float p[4];
            ld4(row + (is_q ? q_col : k_col) + (int64_t)idx * D + pd, p);
#pragma unroll
            for (int i = 0; i < 4; ++i) x[i] = x[i] * cs[i] + p[i] * sn[i];
        }
        float ss = x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3];
        for (int off = LPV >> 1; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
        if (!live) continue;
        const float r = 1.0f / sqrtf(ss / (float)D + eps) * (is_q ? temp : 1.0f);
        float g[4] = {1.f, 1.f, 1.f, 1.f};
        if (is_q ? wq != nullptr : wk != nullptr) ld4((is_q ? wq : wk) + d, g);
#pragma unroll
        for (int i = 0; i < 4; ++i) x[i] = x[i] * r * g[i];
        if (is_q) {
            T *dst = q_map_stride ? q_out + map * q_map_stride + n * ((int64_t)H * D) + (int64_t)head * D
                                  : q_out + n * ((int64_t)nq * D) + ((int64_t)map * H + head) * D;
            st4(dst + d, x);
        } else if (sl >= 0) {
            st4(k_cache + sl * ((int64_t)nk * D) + ((int64_t)map * G + head) * D + d, x);
        }
    }
    if (sl >= 0)
        for (int c = threadIdx.x; c < GDv; c += 256) v_cache[sl * GDv + c] = row[v_col + c];
}

extern "C" int jl_head_norm_append(const void *proj, int dtype, int64_t N, int64_t ld, int32_t q_col, int32_t k_col, int32_t v_col, int32_t H,
                                   int32_t G, int32_t M, int32_t D, int32_t Dv, const void *wq, const void *wk, float eps, float t_coef,
                                   int32_t t_every, const int32_t *pos, void *q_out, int32_t maps_apart, void *k_cache, void *v_cache,
                                   const int64_t *slot, int32_t rot_dims, const float *cos_t, const float *sin_t, void *stream) {
    if (N <= 0) return JL_OK;
    if (!proj || !q_out || !k_cache || !v_cache || !slot) return jl_fail(JL_E_INVALID, "jl_head_norm_append: null pointer");
    if (rot_dims < 0 || rot_dims % 2 || rot_dims > D || (rot_dims && (!pos || !cos_t || !sin_t)))
        return jl_fail(JL_E_INVALID, "jl_head_norm_append: a rotation needs an even width up to D, positions and angle tables");
    if (H <= 0 || G <= 0 || M <= 0 || D <= 0 || Dv <= 0 || q_col + (int64_t)H * M * D > ld || k_col + (int64_t)G * M * D > ld || v_col + (int64_t)G * Dv > ld)
        return jl_fail(JL_E_INVALID, "jl_head_norm_append: columns do not fit the row stride");
    if (t_coef != 0.f && (!pos || t_every <= 0)) return jl_fail(JL_E_INVALID, "jl_head_norm_append: a query temperature needs positions and a period >= 1");
    if (D % 4 == 0 && D <= 256 && ld % 4 == 0 && q_col % 4 == 0 && k_col % 4 == 0 && rot_dims % 8 == 0) {
        int lpv = 1;
        while (4 * lpv < D) lpv <<= 1;
        JL_DISPATCH(dtype, head_norm_append_vec_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>(
                               (const T *)proj, ld, q_col, k_col, v_col, H, G, M, D, G * Dv, (const T *)wq, (const T *)wk, eps, t_coef, t_every, pos,
                               (T *)q_out, maps_apart ? N * (int64_t)H * D : 0, (T *)k_cache, (T *)v_cache, slot, lpv, rot_dims, cos_t, sin_t));
        return jl_check_launch("head_norm_append_vec_kernel");
    }
    JL_DISPATCH(dtype, head_norm_append_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>(
                           (const T *)proj, ld, q_col, k_col, v_col, H, G, M, D, G * Dv, (const T *)wq, (const T *)wk, eps, t_coef, t_every, pos,
                           (T *)q_out, maps_apart ? N * (int64_t)H * D : 0, (T *)k_cache, (T *)v_cache, slot, rot_dims, cos_t, sin_t));
    return jl_check_launch("head_norm_append_kernel");
}

// o = a[map 0] - lambda * a[map 1], unit RMS per head, times out_scale.  A wavefront per (token, head).
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(const float *__restrict__ m1, const float *__restrict__ m2, int64_t ld, int64_t N, int H,
                                                            int Dv, float lambda, float eps, float out_scale, T *__restrict__ out) {
    const int64_t vec = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (vec >= N * H) return;
    const int lane = threadIdx.x & 63;
    const int64_t n = vec / H;
    const int h = (int)(vec - n * H);
    const float *a1 = m1 + n * ld + (int64_t)h * Dv, *a2 = m2 + n * ld + (int64_t)h * Dv;
    float ss = 0.f;
    for (int d = lane; d < Dv; d += 64) { const float o = a1[d] - lambda * a2[d]; ss += o * o; }
    ss = wave_sum_f32(ss);
    const float r = out_scale / sqrtf(ss / (float)Dv + eps);
    for (int d = lane; d < Dv; d += 64) st_f(out + vec * Dv + d, (a1[d] - lambda * a2[d]) * r);
}

extern "C" int jl_diff_combine(const float *a1, const float *a2, int64_t ld, int64_t N, int32_t H, int32_t Dv, float lambda, float eps,
                               float out_scale, void *out, int dtype, void *stream) {
    if (N <= 0) return JL_OK;
    if (!a1 || !a2 || !out || H <= 0 || Dv <= 0 || ld < (int64_t)H * Dv) return jl_fail(JL_E_INVALID, "jl_diff_combine: null pointer or bad sizes");
    const int64_t vecs = N * H;
    JL_DISPATCH(dtype, diff_combine_kernel<T><<<dim3((unsigned)((vecs + 3) / 4)), 256, 0, (hipStream_t)stream>>>(a1, a2, ld, N, H, Dv, lambda, eps, out_scale,
                                                                                                               (T *)out));
    return jl_check_launch("diff_combine_kernel");
}
