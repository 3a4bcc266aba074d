// jl_norm.hip — embedding gather, the residual-update + RMS-norm launches (norm of the stream, norm of a sublayer's output) and the
// polynomial activation.
#include "jl_common.h"

template <typename T>
__global__ __launch_bounds__(256) void embed_scale_kernel(const T *__restrict__ embed, const int64_t *__restrict__ ids, int W,
                                                           float scale, float *__restrict__ x, float *__restrict__ x0) {
    const int64_t n = blockIdx.x;
    const T *src = embed + ids[n] * (int64_t)W;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = ld_f(src + c) * scale;
        x[n * W + c] = v;
        if (x0) x0[n * W + c] = v;
    }
}

extern "C" int jl_embed_scale(const void *embed, int dtype, const int64_t *ids, int64_t N, int32_t W, float scale, float *x, float *x0,
                              void *stream) {
    if (N <= 0) return JL_OK;
    if (!embed || !ids || !x || W <= 0) return jl_fail(JL_E_INVALID, "jl_embed_scale: null pointer or bad width");
    JL_DISPATCH(dtype, embed_scale_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>((const T *)embed, ids, W, scale, x, x0));
    return jl_check_launch("embed_scale_kernel");
}

// one workgroup per row: pass 1 forms the new residual (written back) and its sum of squares, pass 2 normalises what pass 1 wrote
template <typename T>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float *__restrict__ x, const void *__restrict__ y, int y_dtype, int y_count,
                                                           const float *__restrict__ x0, const T *__restrict__ w, float eps,
                                                           T *__restrict__ out, int W) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    float *xr = x + n * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float v = xr[c];
        if (y)
            for (int s = 0; s < y_count; ++s) v += ld_any(y, y_dtype, (n * y_count + s) * (int64_t)W + c);
        if (x0) v += x0[n * W + c];
        if (y || x0) xr[c] = v;
        ss += v * v;
    }
    if (!out) return;
    ss = block_sum_f32(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = xr[c] * r;
        st_f(out + n * W + c, w ? v * ld_f(w + c) : v);
    }
}

extern "C" int jl_add_rmsnorm(float *x, const void *y, int y_dtype, int32_t y_count, const float *x0, const void *w, float eps,
                              void *out, int dtype, int64_t N, int32_t W, void *stream) {
    if (N <= 0) return JL_OK;
    if (!x || W <= 0 || (y && y_count <= 0)) return jl_fail(JL_E_INVALID, "jl_add_rmsnorm: null pointer or bad sizes");
    JL_DISPATCH(dtype, add_rmsnorm_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>(x, y, y_dtype, y_count, x0, (const T *)w,
                                                                                                 eps, (T *)out, W));
    return jl_check_launch("add_rmsnorm_kernel");
}

// ---- several scaled addends + up to two norms of the same row (a layer whose sublayers all read one stream) ---------------------------------
// pass 1: x += sum_a scale_a * (sum over the addend's middle axis), written back, with the sum of squares; pass 2: both outputs
template <typename T>
__global__ __launch_bounds__(256) void scaled_add_norms_kernel(float *__restrict__ x, jl_addend a0, jl_addend a1, jl_addend a2, const float *__restrict__ w1,
                                                                const float *__restrict__ w2, float w_offset, float eps, T *__restrict__ out1,
                                                                T *__restrict__ out2, float *__restrict__ out2_f32, int W) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    float *xr = x + n * W;
    const jl_addend ad[3] = {a0, a1, a2};
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            if (!ad[k].y) continue;
            float u = 0.f;
            for (int s = 0; s < ad[k].count; ++s) u += ld_any(ad[k].y, ad[k].dtype, (n * ad[k].count + s) * (int64_t)W + c);
            t += ad[k].scale ? u * ad[k].scale[c] : u;
        }
        const float v = xr[c] + t;
        if (a0.y || a1.y || a2.y) xr[c] = v;
        ss += v * v;
    }
    if (!out1 && !out2 && !out2_f32) return;
    ss = block_sum_f32(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = xr[c] * r;
        if (out1) st_f(out1 + n * W + c, w1 ? v * (w_offset + w1[c]) : v);
        if (out2) st_f(out2 + n * W + c, w2 ? v * (w_offset + w2[c]) : v);
        if (out2_f32) out2_f32[n * W + c] = w2 ? v * (w_offset + w2[c]) : v;
    }
}

extern "C" int jl_scaled_add_norms(float *x, const jl_addend *addends, int32_t n_addends, const float *w1, const float *w2, float w_offset, float eps,
                                   void *out1, void *out2, float *out2_f32, int dtype, int64_t N, int32_t W, void *stream) {
    if (N <= 0) return JL_OK;
    if (!x || W <= 0 || n_addends < 0 || n_addends > 3 || (n_addends && !addends)) return jl_fail(JL_E_INVALID, "jl_scaled_add_norms: null pointer, bad width or more than 3 addends");
    jl_addend ad[3] = {{nullptr, 0, 0, nullptr}, {nullptr, 0, 0, nullptr}, {nullptr, 0, 0, nullptr}};
    for (int k = 0; k < n_addends; ++k) {
        ad[k] = addends[k];
        if (ad[k].y && ad[k].count <= 0) return jl_fail(JL_E_INVALID, "jl_scaled_add_norms: addend %d has no rows", k);
    }
    JL_DISPATCH(dtype, scaled_add_norms_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>(x, ad[0], ad[1], ad[2], w1, w2, w_offset, eps, (T *)out1,
                                                                                                      (T *)out2, out2_f32, W));
    return jl_check_launch("scaled_add_norms_kernel");
}

// ---- gated activation of a feed-forward: out[n, c] = act(z[n, g_col + c]) * lin(z[n, u_col + c]) (* sigmoid(row_gate[n])) -----------------
template <typename T>
__global__ __launch_bounds__(256) void gated_act_kernel(const T *__restrict__ z, int64_t ld, int g_col, int u_col, int F, int kind, float limit, float alpha,
                                                         float shift, const T *__restrict__ row_gate, int64_t rg_ld, T *__restrict__ out, int64_t total) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const int64_t n = e / F;
    const int c = (int)(e - n * F);
    float v = gated_unit_f(ld_f(z + n * ld + g_col + c), u_col < 0 ? 1.0f : ld_f(z + n * ld + u_col + c), kind, limit, alpha, shift);
    if (row_gate) v *= 1.0f / (1.0f + expf(-ld_f(row_gate + n * rg_ld)));
    st_f(out + e, v);
}

// 16 bytes per load and thread (4 floats, 8 bfloat16): columns, row stride and F in multiples of that
__device__ __forceinline__ void ld16(const float *p, float (&v)[4]) { const float4 t = *(const float4 *)p; v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
__device__ __forceinline__ void ld16(const bf16_t *p, float (&v)[8]) {
    const uint4 t = *(const uint4 *)p;
    const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(w[i] << 16); v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
}
__device__ __forceinline__ void st16(float *p, const float (&v)[4]) { *(float4 *)p = make_float4(v[0], v[1], v[2], v[3]); }
__device__ __forceinline__ void st16(bf16_t *p, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        bf16_t lo, hi;
        st_f(&lo, v[2 * i]);
        st_f(&hi, v[2 * i + 1]);
        w[i] = (uint32_t)lo | ((uint32_t)hi << 16);
    }
    *(uint4 *)p = make_uint4(w[0], w[1], w[2], w[3]);
}
template <typename T>
__global__ __launch_bounds__(256) void gated_act_vec_kernel(const T *__restrict__ z, int64_t ld, int g_col, int u_col, int F, int kind, float limit, float alpha,
                                                             float shift, const T *__restrict__ row_gate, int64_t rg_ld, T *__restrict__ out, int64_t vecs) {
    constexpr int VEC = 16 / sizeof(T);
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= vecs) return;
    const int per_row = F / VEC;
    const int64_t n = e / per_row;
    const int c = (int)(e - n * per_row) * VEC;
    float g[VEC], u[VEC];
    ld16(z + n * ld + g_col + c, g);
    if (u_col >= 0) ld16(z + n * ld + u_col + c, u);
    else
#pragma unroll
        for (int i = 0; i < VEC; ++i) u[i] = 1.0f;
    const float rg = row_gate ? 1.0f / (1.0f + expf(-ld_f(row_gate + n * rg_ld))) : 1.0f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) g[i] = gated_unit_f(g[i], u[i], kind, limit, alpha, shift) * rg;
    st16(out + n * F + c, g);
}

extern "C" int jl_gated_act(const void *z, int dtype, int64_t N, int64_t ld, int32_t g_col, int32_t u_col, int32_t F, int32_t kind, float limit, float alpha,
                            float shift, const void *row_gate, int64_t rg_ld, void *out, void *stream) {
    if (N <= 0) return JL_OK;
    if (!z || !out || F <= 0 || g_col < 0 || g_col + (int64_t)F > ld || u_col + (int64_t)F > ld)
        return jl_fail(JL_E_INVALID, "jl_gated_act: null pointer, or the columns do not fit the row stride");
    if (kind < JL_ACT_GELU_TANH || kind > JL_ACT_GELU_ERF) return jl_fail(JL_E_INVALID, "jl_gated_act: unknown kind %d", kind);
    if (u_col < 0) u_col = -1;
    const int vec = dtype == JL_BF16 ? 8 : 4;
    if (F % vec == 0 && g_col % vec == 0 && (u_col < 0 || u_col % vec == 0) && ld % vec == 0 && (uintptr_t)z % 16 == 0 && (uintptr_t)out % 16 == 0) {
        const int64_t vecs = N * (F / vec);
        JL_DISPATCH(dtype, gated_act_vec_kernel<T><<<dim3((unsigned)((vecs + 255) / 256)), 256, 0, (hipStream_t)stream>>>(
                               (const T *)z, ld, g_col, u_col, F, kind, limit, alpha, shift, (const T *)row_gate, rg_ld, (T *)out, vecs));
        return jl_check_launch("gated_act_vec_kernel");
    }
    const int64_t total = N * F;
    JL_DISPATCH(dtype, gated_act_kernel<T><<<dim3((unsigned)((total + 255) / 256)), 256, 0, (hipStream_t)stream>>>(
                           (const T *)z, ld, g_col, u_col, F, kind, limit, alpha, shift, (const T *)row_gate, rg_ld, (T *)out, total));
    return jl_check_launch("gated_act_kernel");
}

// ---- sublayer-output norm + residual update: one workgroup per row ------------------------------------------------------------
template <typename TY, typename TO>
__global__ __launch_bounds__(256) void norm_add_kernel(float *__restrict__ x, const TY *__restrict__ y, const float *__restrict__ g, float eps,
                                                        TO *__restrict__ out, int W) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const TY *yr = y + n * W;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) { const float v = ld_f(yr + c); ss += v * v; }
    ss = block_sum_f32(ss, red);
    const float r = g[0] / sqrtf(ss / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = x[n * W + c] + ld_f(yr + c) * r;
        x[n * W + c] = v;
        if (out) st_f(out + n * W + c, v);
    }
}

extern "C" int jl_norm_add(float *x, const void *y, int y_dtype, const float *g, float eps, void *out, int out_dtype, int64_t N, int32_t W,
                           void *stream) {
    if (N <= 0) return JL_OK;
    if (!x || !y || !g || W <= 0) return jl_fail(JL_E_INVALID, "jl_norm_add: null pointer or bad width");
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)N);
    if (y_dtype == JL_BF16) {
        if (out_dtype == JL_BF16) norm_add_kernel<bf16_t, bf16_t><<<grid, 256, 0, st>>>(x, (const bf16_t *)y, g, eps, (bf16_t *)out, W);
        else norm_add_kernel<bf16_t, float><<<grid, 256, 0, st>>>(x, (const bf16_t *)y, g, eps, (float *)out, W);
    } else {
        if (out_dtype == JL_BF16) norm_add_kernel<float, bf16_t><<<grid, 256, 0, st>>>(x, (const float *)y, g, eps, (bf16_t *)out, W);
        else norm_add_kernel<float, float><<<grid, 256, 0, st>>>(x, (const float *)y, g, eps, (float *)out, W);
    }
    return jl_check_launch("norm_add_kernel");
}

// ---- polynomial activation with unit-RMS powers: one workgroup per row --------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void polynorm_kernel(const T *__restrict__ z, int F, const float *__restrict__ coef, float eps,
                                                        T *__restrict__ out) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const T *zr = z + n * F;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int c = threadIdx.x; c < F; c += 256) {
        const float v = ld_f(zr + c), v2 = v * v, v3 = v2 * v;
        s1 += v2; s2 += v2 * v2; s3 += v3 * v3;
    }
    s1 = block_sum_f32(s1, red);
    s2 = block_sum_f32(s2, red);
    s3 = block_sum_f32(s3, red);
    const float r1 = coef[0] / sqrtf(s1 / (float)F + eps), r2 = coef[1] / sqrtf(s2 / (float)F + eps), r3 = coef[2] / sqrtf(s3 / (float)F + eps);
    const float e = coef[3];
    for (int c = threadIdx.x; c < F; c += 256) {
        const float v = ld_f(zr + c), v2 = v * v;
        st_f(out + n * F + c, v * r1 + v2 * r2 + v2 * v * r3 + e);
    }
}

extern "C" int jl_polynorm(const void *z, int dtype, int64_t N, int32_t F, const float *coef, float eps, void *out, void *stream) {
    if (N <= 0) return JL_OK;
    if (!z || !coef || !out || F <= 0) return jl_fail(JL_E_INVALID, "jl_polynorm: null pointer or bad width");
    JL_DISPATCH(dtype, polynorm_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>((const T *)z, F, coef, eps, (T *)out));
    return jl_check_launch("polynorm_kernel");
}

// ---- residual update + weighted sum over the streams of all depths + RMS norm: one workgroup per row ------------------------------------
// pass 1: y = x_in + mult * (sum of the addends) is stored as stream `depth`; v = sum_j mix[j] * stream_j (j <= depth; the last one from
// registers) is stored as x_out, with its sum of squares; pass 2: the norm of what pass 1 wrote, in `dtype` and / or unrounded.
template <typename T>
__global__ __launch_bounds__(256) void depth_mix_norm_kernel(const float *__restrict__ x_in, jl_addend a0, jl_addend a1, jl_addend a2, float mult,
                                                              float *__restrict__ streams, int64_t stream_ld, int depth, const float *__restrict__ mix,
                                                              float *__restrict__ x_out, const float *__restrict__ w, float eps, T *__restrict__ out,
                                                              float *__restrict__ out_f32, int W, const float *__restrict__ shift_mu,
                                                              const int32_t *__restrict__ seq, float *shift_tail, T *__restrict__ out_shift) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const jl_addend ad[3] = {a0, a1, a2};
    const bool update = a0.y || a1.y || a2.y || depth >= 0;
    float ss = 0.f;
    for (int c = threadIdx.x; c < W; c += 256) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            if (!ad[k].y) continue;
            float u = 0.f;
            for (int s = 0; s < ad[k].count; ++s) u += ld_any(ad[k].y, ad[k].dtype, (n * ad[k].count + s) * (int64_t)W + c);
            t += ad[k].scale ? u * ad[k].scale[c] : u;
        }
        float v = x_in[n * W + c] + mult * t;
        if (depth >= 0) {
            streams[depth * stream_ld + n * W + c] = v;
            if (mix) {
                v *= mix[depth];
                for (int j = 0; j < depth; ++j) v += mix[j] * streams[j * stream_ld + n * W + c];
            }
        }
        if (update) x_out[n * W + c] = v;
        ss += v * v;
    }
    if (!out && !out_f32 && !shift_mu) return;
    ss = block_sum_f32(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
    const float *xr = update ? x_out + n * W : x_in + n * W;
    // the token shift in the same launch, for steps in which every request brings ONE row (row n is request n): the previous token's
    // norm is the slot's tail (nothing before position 0), which this thread then replaces by its own
    int slot = 0;
    bool past = false;
    if (shift_mu) { slot = seq[4 * n + 3]; past = seq[4 * n + 2] > 0; }
    for (int c = threadIdx.x; c < W; c += 256) {
        const float v = xr[c] * r * (w ? w[c] : 1.0f);
        if (out) st_f(out + n * W + c, v);
        if (out_f32) out_f32[n * W + c] = v;
        if (shift_mu) {
            float *tl = shift_tail + (int64_t)slot * W + c;
            const float prev = past ? *tl : 0.f;
            *tl = v;
            st_f(out_shift + n * W + c, v + (prev - v) * shift_mu[c]);
        }
    }
}

// The same for widths in multiples of four with 16-byte aligned rows: a thread owns four consecutive channels per pass (16-byte loads and
// stores of floats, 8-byte ones of bfloat16).  SHIFT: the token shift of single-row steps rides along.
__device__ __forceinline__ void ld4_any(const void *p, int dtype, int64_t i, float (&v)[4]) {
    if (dtype == JL_BF16) {
        const uint2 t = *(const uint2 *)((const bf16_t *)p + i);
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u); v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    } else {
        const float4 t = *(const float4 *)((const float *)p + i);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
}
__device__ __forceinline__ void st4_f(float *p, const float (&v)[4]) { *(float4 *)p = make_float4(v[0], v[1], v[2], v[3]); }
__device__ __forceinline__ void st4_f(bf16_t *p, const float (&v)[4]) {
    bf16_t h[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) st_f(&h[i], v[i]);
    *(uint2 *)p = make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
}

template <typename T, bool SHIFT>
__global__ __launch_bounds__(256) void depth_mix_norm_vec_kernel(const float *__restrict__ x_in, jl_addend a0, jl_addend a1, jl_addend a2, float mult,
                                                                  float *__restrict__ streams, int64_t stream_ld, int depth, const float *__restrict__ mix,
                                                                  float *__restrict__ x_out, const float *__restrict__ w, float eps, T *__restrict__ out,
                                                                  float *__restrict__ out_f32, int W, const float *__restrict__ shift_mu,
                                                                  const int32_t *__restrict__ seq, float *shift_tail, T *__restrict__ out_shift) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const jl_addend ad[3] = {a0, a1, a2};
    const bool update = a0.y || a1.y || a2.y || depth >= 0;
    float ss = 0.f;
    for (int c = threadIdx.x * 4; c < W; c += 1024) {
        float t[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            if (!ad[k].y) continue;
            float u[4] = {0.f, 0.f, 0.f, 0.f};
            for (int s2 = 0; s2 < ad[k].count; ++s2) {
                float a[4];
                ld4_any(ad[k].y, ad[k].dtype, (n * ad[k].count + s2) * (int64_t)W + c, a);
#pragma unroll
                for (int i = 0; i < 4; ++i) u[i] += a[i];
            }
            if (ad[k].scale) {
                const float4 sc = *(const float4 *)(ad[k].scale + c);
                u[0] *= sc.x; u[1] *= sc.y; u[2] *= sc.z; u[3] *= sc.w;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) t[i] += u[i];
        }
        float v[4];
        ld4_any(x_in, JL_F32, n * W + c, v);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] += mult * t[i];
        if (depth >= 0) {
            st4_f(streams + depth * stream_ld + n * W + c, v);
            if (mix) {
                const float md = mix[depth];
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] *= md;
                for (int j = 0; j < depth; ++j) {
                    float sj[4];
                    ld4_any(streams, JL_F32, j * stream_ld + n * W + c, sj);
                    const float mj = mix[j];
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[i] += mj * sj[i];
                }
            }
        }
        if (update) st4_f(x_out + n * W + c, v);
#pragma unroll
        for (int i = 0; i < 4; ++i) ss += v[i] * v[i];
    }
    if (!out && !out_f32 && !SHIFT) return;
    ss = block_sum_f32(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
    const float *xr = update ? x_out + n * W : x_in + n * W;
    int slot = 0;
    bool past = false;
    if (SHIFT) { slot = seq[4 * n + 3]; past = seq[4 * n + 2] > 0; }
    for (int c = threadIdx.x * 4; c < W; c += 1024) {
        float v[4], wv[4] = {1.f, 1.f, 1.f, 1.f};
        ld4_any(xr, JL_F32, c, v);
        if (w) ld4_any(w, JL_F32, c, wv);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] *= r * wv[i];
        if (out) st4_f(out + n * W + c, v);
        if (out_f32) st4_f(out_f32 + n * W + c, v);
        if (SHIFT) {
            float *tl = shift_tail + (int64_t)slot * W + c;
            float prev[4] = {0.f, 0.f, 0.f, 0.f}, mu[4], sh[4];
            if (past) ld4_any(tl, JL_F32, 0, prev);
            st4_f(tl, v);
            ld4_any(shift_mu, JL_F32, c, mu);
#pragma unroll
            for (int i = 0; i < 4; ++i) sh[i] = v[i] + (prev[i] - v[i]) * mu[i];
            st4_f(out_shift + n * W + c, sh);
        }
    }
}

extern "C" int jl_depth_mix_norm(const float *x_in, const jl_addend *addends, int32_t n_addends, float mult, float *streams, int64_t stream_ld,
                                 int32_t depth, const float *mix, float *x_out, const float *w, float eps, void *out, int dtype, float *out_f32,
                                 int64_t N, int32_t W, const float *shift_mu, const int32_t *seq, float *shift_tail, void *out_shift, void *stream) {
    if (N <= 0) return JL_OK;
    if (shift_mu && (!seq || !shift_tail || !out_shift)) return jl_fail(JL_E_INVALID, "jl_depth_mix_norm: the token shift needs seq, tail and an output");
    if (!x_in || W <= 0 || n_addends < 0 || n_addends > 3 || (n_addends && !addends))
        return jl_fail(JL_E_INVALID, "jl_depth_mix_norm: null pointer, bad width or more than 3 addends");
    if ((depth >= 0 || n_addends) && !x_out) return jl_fail(JL_E_INVALID, "jl_depth_mix_norm: an updated stream needs x_out");
    if (depth >= 0 && (!streams || stream_ld < N * (int64_t)W)) return jl_fail(JL_E_INVALID, "jl_depth_mix_norm: streams of at least N * W floats each");
    if (depth >= 0 && x_out >= streams && x_out < streams + (int64_t)(depth + 1) * stream_ld)
        return jl_fail(JL_E_INVALID, "jl_depth_mix_norm: x_out lies inside the streams it is mixed from");
    jl_addend ad[3] = {{nullptr, 0, 0, nullptr}, {nullptr, 0, 0, nullptr}, {nullptr, 0, 0, nullptr}};
    for (int k = 0; k < n_addends; ++k) {
        ad[k] = addends[k];
        if (ad[k].y && ad[k].count <= 0) return jl_fail(JL_E_INVALID, "jl_depth_mix_norm: addend %d has no rows", k);
    }
    // every pointer the four-channel form touches starts at a 16-byte border (8 for bfloat16 rows) and every row is a multiple of four wide
    auto al = [](const void *q, uintptr_t a) { return ((uintptr_t)q % a) == 0; };
    bool vec = W % 4 == 0 && stream_ld % 4 == 0 && al(x_in, 16) && al(x_out, 16) && al(streams, 16) && al(w, 16) && al(out_f32, 16) && al(shift_mu, 16) &&
               al(shift_tail, 16) && al(out, dtype == JL_BF16 ? 8 : 16) && al(out_shift, dtype == JL_BF16 ? 8 : 16);
    for (int k = 0; k < n_addends; ++k) vec = vec && al(ad[k].y, ad[k].dtype == JL_BF16 ? 8 : 16) && al(ad[k].scale, 16);
    hipStream_t st = (hipStream_t)stream;
#define DMN_ARGS x_in, ad[0], ad[1], ad[2], mult, streams, stream_ld, depth, mix, x_out, w, eps, (T *)out, out_f32, W, shift_mu, seq, shift_tail, (T *)out_shift
    if (vec && shift_mu) JL_DISPATCH(dtype, (depth_mix_norm_vec_kernel<T, true><<<dim3((unsigned)N), 256, 0, st>>>(DMN_ARGS)));
    else if (vec) JL_DISPATCH(dtype, (depth_mix_norm_vec_kernel<T, false><<<dim3((unsigned)N), 256, 0, st>>>(DMN_ARGS)));
    else JL_DISPATCH(dtype, depth_mix_norm_kernel<T><<<dim3((unsigned)N), 256, 0, st>>>(DMN_ARGS));
#undef DMN_ARGS
    return jl_check_launch("depth_mix_norm_kernel");
}

// ---- token shift: out = h + (h of the previous token - h) * mu, the previous token of a request's first row coming from its slot ------------
// One workgroup per row.  The thread that owns channel c of a request's FIRST row is the only one that touches tail[slot, c] in the
// launch: it reads the old value (when the request has a past) and then stores the h of the request's last row of this step.
template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(const float *__restrict__ h, const float *__restrict__ mu, const int32_t *__restrict__ row_req,
                                                           const int32_t *__restrict__ seq, float *tail, int W, T *__restrict__ out) {
    const int64_t n = blockIdx.x;
    const int32_t *rec = seq + 4 * (int64_t)row_req[n];
    const int row0 = rec[0], count = rec[1], pos0 = rec[2], slot = rec[3];
    const bool first = n == row0;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float cur = h[n * W + c];
        float prev;
        if (first) {
            float *tl = tail + (int64_t)slot * W + c;
            prev = pos0 > 0 ? *tl : 0.f;
            *tl = h[(int64_t)(row0 + count - 1) * W + c];
        } else {
            prev = h[(n - 1) * W + c];
        }
        st_f(out + n * W + c, cur + (prev - cur) * mu[c]);
    }
}

extern "C" int jl_token_shift(const float *h, const float *mu, const int32_t *row_req, const int32_t *seq, float *tail, int64_t N, int32_t W,
                              void *out, int dtype, void *stream) {
    if (N <= 0) return JL_OK;
    if (!h || !mu || !row_req || !seq || !tail || !out || W <= 0) return jl_fail(JL_E_INVALID, "jl_token_shift: null pointer or bad width");
    JL_DISPATCH(dtype, token_shift_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>(h, mu, row_req, seq, tail, W, (T *)out));
    return jl_check_launch("token_shift_kernel");
}

// ---- soft cap of the logits, in place: z <- cap * tanh(z / cap) ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void softcap_kernel(float *__restrict__ z, int64_t total, float cap) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e < total) z[e] = cap * tanhf(z[e] / cap);
}

extern "C" int jl_softcap(float *z, int64_t total, float cap, void *stream) {
    if (total <= 0) return JL_OK;
    if (!z || !(cap > 0.f)) return jl_fail(JL_E_INVALID, "jl_softcap: null pointer or a cap that is not positive");
    softcap_kernel<<<dim3((unsigned)((total + 255) / 256)), 256, 0, (hipStream_t)stream>>>(z, total, cap);
    return jl_check_launch("softcap_kernel");
}
