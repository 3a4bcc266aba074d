// jl_common.h — shared by the translation units of libjf_layers.so (gfx950 / CDNA4 only): the layer kernels of the models whose
// forward is not stock PyTorch (32-bit residual stream, windowed attention with a distance bias and mixed heads, retention,
// routed experts).  Activations are float or bfloat16 (dtype code JL_F32 / JL_BF16); everything the kernels accumulate,
// normalise, exponentiate or carry from token to token is float.
#ifndef JL_COMMON_H
#define JL_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>

#include "jf_layers.h"

typedef uint16_t bf16_t;

int jl_fail(int code, const char *fmt, ...);       // records the message for jl_last_error(), returns `code`
int jl_check_launch(const char *what);

template <typename T> __device__ __forceinline__ float ld_f(const T *p);
template <> __device__ __forceinline__ float ld_f<float>(const float *p) { return *p; }
template <> __device__ __forceinline__ float ld_f<bf16_t>(const bf16_t *p) { return __uint_as_float(((uint32_t)*p) << 16); }
template <typename T> __device__ __forceinline__ void st_f(T *p, float v);
template <> __device__ __forceinline__ void st_f<float>(float *p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_f<bf16_t>(bf16_t *p, float v) {          // round to nearest even
    uint32_t u = __float_as_uint(v);
    if ((u & 0x7fffffffu) > 0x7f800000u) { *p = 0x7FC0; return; }
    u += 0x7FFFu + ((u >> 16) & 1u);
    *p = (bf16_t)(u >> 16);
}
__device__ __forceinline__ float ld_any(const void *p, int dtype, int64_t i) {
    return dtype == JL_BF16 ? ld_f((const bf16_t *)p + i) : ((const float *)p)[i];
}

__device__ __forceinline__ float wave_sum_f32(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
// sum over a workgroup of up to 1024 threads; `red` holds 16 floats of LDS.  Every thread gets the result; the order of
// the additions is fixed by the lane / wavefront numbers.
__device__ __forceinline__ float block_sum_f32(float v, float *red) {
    v = wave_sum_f32(v);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float s = 0.f;
    for (int i = 0; i < nw; ++i) s += red[i];
    return s;
}

// gated units of a feed-forward (jl_gated_act, and the grouped product that applies them in its epilogue)
// 0.5 z (1 + tanh(u)) = z sigmoid(2u), u = sqrt(2/pi) (z + 0.044715 z^3)
__device__ __forceinline__ float gelu_tanh_f(float z) {
    return z / (1.0f + expf(-1.5957691216057308f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float gelu_erf_f(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float gated_unit_f(float g, float u, int kind, float limit, float alpha, float shift) {
    if (kind == JL_ACT_GELU_TANH) return gelu_tanh_f(g) * u;
    if (kind == JL_ACT_SILU) return silu_f(g) * u;
    if (kind == JL_ACT_GELU_ERF) return gelu_erf_f(g) * u;
    g = fminf(g, limit);                                            // clamped swish: the gate capped from above, the linear branch from both sides
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-alpha * g)) * (u + shift);
}

#define JL_DISPATCH(dtype, ...)                                   \
    do {                                                          \
        if ((dtype) == JL_BF16) { typedef bf16_t T; __VA_ARGS__; } \
        else { typedef float T; __VA_ARGS__; }                    \
    } while (0)

#endif
