// jl_latent.hip — attention through a low-rank latent: the pool holds, per token, the normalised key/value latent and one rotary
// key part shared by all heads; queries are brought into the pool's coordinates (the key up-projection is applied to the query),
// attention runs over the pool with one key/value "head", and the value up-projection follows.  This file: the norms, rotations and
// packing around the library products.
#include "jl_common.h"

__device__ __forceinline__ float rot_half(const float *v, int d, int rot_dims, const float *cs, const float *sn, int pairing) {
    // value of dimension d of the rotated vector; v the unrotated vector (float, in LDS or registers)
    const int half = rot_dims >> 1;
    if (d >= rot_dims) return v[d];
    if (pairing == JL_ROT_NEIGHBOURS) {                         // dimension 2i pairs with 2i + 1
        const int i = d >> 1;
        return (d & 1) ? v[d] * cs[i] + v[d - 1] * sn[i] : v[d] * cs[i] - v[d + 1] * sn[i];
    }
    if (d < half) return v[d] * cs[d] - v[d + half] * sn[d];
    return v[d] * cs[d - half] + v[d - half] * sn[d - half];
}

template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(const T *__restrict__ proj, int64_t ld, int q_col, int Rq, int kv_col, int R, int rd,
                                                           int rot_dims, const T *__restrict__ wq, const T *__restrict__ wkv, float eps,
                                                           const int32_t *__restrict__ pos, const float *__restrict__ cos_t,
                                                           const float *__restrict__ sin_t, T *__restrict__ cq_out, T *__restrict__ pool,
                                                           const int64_t *__restrict__ slot, int pairing) {
    __shared__ float red[16];
    extern __shared__ float kr[];                               // [rd] the unrotated rotary key
    const int64_t n = blockIdx.x;
    const T *row = proj + n * ld;
    float sq = 0.f, sk = 0.f;
    for (int c = threadIdx.x; c < Rq; c += blockDim.x) { const float v = ld_f(row + q_col + c); sq += v * v; }
    for (int c = threadIdx.x; c < R; c += blockDim.x) { const float v = ld_f(row + kv_col + c); sk += v * v; }
    for (int c = threadIdx.x; c < rd; c += blockDim.x) kr[c] = ld_f(row + kv_col + R + c);
    sq = block_sum_f32(sq, red);
    sk = block_sum_f32(sk, red);                                // its barriers also publish kr
    const float rq = Rq > 0 ? 1.0f / sqrtf(sq / (float)Rq + eps) : 0.f, rk = 1.0f / sqrtf(sk / (float)R + eps);
    for (int c = threadIdx.x; c < Rq; c += blockDim.x) st_f(cq_out + n * Rq + c, ld_f(row + q_col + c) * rq * ld_f(wq + c));
    const int64_t sl = slot[n];
    if (sl < 0) return;
    T *dst = pool + sl * (int64_t)(R + rd);
    for (int c = threadIdx.x; c < R; c += blockDim.x) st_f(dst + c, ld_f(row + kv_col + c) * rk * ld_f(wkv + c));
    const float *cs = cos_t + (int64_t)pos[n] * (rot_dims >> 1), *sn = sin_t + (int64_t)pos[n] * (rot_dims >> 1);
    for (int c = threadIdx.x; c < rd; c += blockDim.x) st_f(dst + R + c, rot_half(kr, c, rot_dims, cs, sn, pairing));
}

extern "C" int jl_latent_prep(const void *proj, int dtype, int64_t N, int64_t ld, int32_t q_col, int32_t Rq, int32_t kv_col, int32_t R,
                              int32_t rd, int32_t rot_dims, const void *wq, const void *wkv, float eps, const int32_t *pos,
                              const float *cos_t, const float *sin_t, int64_t table_len, void *cq_out, void *pool, const int64_t *slot,
                              int32_t pairing, void *stream) {
    if (N <= 0) return JL_OK;
    if (!proj || !wkv || !pos || !pool || !slot || (Rq > 0 && (!wq || !cq_out))) return jl_fail(JL_E_INVALID, "jl_latent_prep: null pointer");
    if (pairing != JL_ROT_HALVES && pairing != JL_ROT_NEIGHBOURS) return jl_fail(JL_E_INVALID, "jl_latent_prep: unknown pairing %d", pairing);
    if (Rq < 0 || R <= 0 || rd < 0 || q_col + (int64_t)Rq > ld || kv_col + (int64_t)R + rd > ld)
        return jl_fail(JL_E_INVALID, "jl_latent_prep: columns do not fit the row stride");
    if (rot_dims < 0 || rot_dims > rd || (rot_dims & 1) || (rot_dims && (!cos_t || !sin_t || table_len <= 0)))
        return jl_fail(JL_E_INVALID, "jl_latent_prep: rot_dims must be even, at most rd, with angle tables");
    // narrow rows (a few hundred values per token): one wavefront per token instead of four, of which three would idle
    const int threads = (int64_t)Rq + R + rd <= 512 ? 64 : 256;
    JL_DISPATCH(dtype, latent_prep_kernel<T><<<dim3((unsigned)N), threads, (size_t)(rd > 0 ? rd : 1) * 4, (hipStream_t)stream>>>(
                           (const T *)proj, ld, q_col, Rq, kv_col, R, rd, rot_dims, (const T *)wq, (const T *)wkv, eps, pos, cos_t, sin_t,
                           (T *)cq_out, (T *)pool, slot, pairing));
    return jl_check_launch("latent_prep_kernel");
}

// one workgroup per token: q_out[n, h] = [qa[h, n, :R] | rotate(q[n, h, D:])]
template <typename T>
__global__ __launch_bounds__(256) void latent_q_pack_kernel(const T *__restrict__ qa, const T *__restrict__ q, int64_t q_ld, int64_t N, int H, int D, int R, int rd,
                                                             int rot_dims, const int32_t *__restrict__ pos, const float *__restrict__ cos_t,
                                                             const float *__restrict__ sin_t, T *__restrict__ q_out, int pairing) {
    extern __shared__ float qr[];                               // [H][rd]
    const int64_t n = blockIdx.x;
    const int Dq = D + rd, Do = R + rd;
    for (int e = threadIdx.x; e < H * rd; e += 256) { const int h = e / rd, c = e - h * rd; qr[e] = ld_f(q + n * q_ld + (int64_t)h * Dq + D + c); }
    for (int e = threadIdx.x; e < H * R; e += 256) {
        const int h = e / R, c = e - h * R;
        q_out[(n * H + h) * Do + c] = qa[((int64_t)h * N + n) * R + c];
    }
    __syncthreads();
    const float *cs = cos_t + (int64_t)pos[n] * (rot_dims >> 1), *sn = sin_t + (int64_t)pos[n] * (rot_dims >> 1);
    for (int e = threadIdx.x; e < H * rd; e += 256) {
        const int h = e / rd, c = e - h * rd;
        st_f(q_out + (n * H + h) * Do + R + c, rot_half(qr + h * rd, c, rot_dims, cs, sn, pairing));
    }
}

extern "C" int jl_latent_q_pack(const void *qa, const void *q, int64_t q_ld, int dtype, int64_t N, int32_t H, int32_t D, int32_t R, int32_t rd,
                                int32_t rot_dims, const int32_t *pos, const float *cos_t, const float *sin_t, int64_t table_len, void *q_out,
                                int32_t pairing, void *stream) {
    if (N <= 0) return JL_OK;
    if (!qa || !q || !pos || !q_out || H <= 0 || D < 0 || R <= 0 || rd < 0 || q_ld < (int64_t)H * (D + rd))
        return jl_fail(JL_E_INVALID, "jl_latent_q_pack: null pointer or bad sizes");
    if (pairing != JL_ROT_HALVES && pairing != JL_ROT_NEIGHBOURS) return jl_fail(JL_E_INVALID, "jl_latent_q_pack: unknown pairing %d", pairing);
    if (rot_dims < 0 || rot_dims > rd || (rot_dims & 1) || (rot_dims && (!cos_t || !sin_t || table_len <= 0)))
        return jl_fail(JL_E_INVALID, "jl_latent_q_pack: rot_dims must be even, at most rd, with angle tables");
    const size_t lds = (size_t)(H * rd > 0 ? H * rd : 1) * 4;
    if (lds > 48 * 1024) return jl_fail(JL_E_INVALID, "jl_latent_q_pack: %d heads x %d rotary dimensions exceed the kernel's LDS", H, rd);
    JL_DISPATCH(dtype, latent_q_pack_kernel<T><<<dim3((unsigned)N), 256, lds, (hipStream_t)stream>>>((const T *)qa, (const T *)q, q_ld, N, H, D, R, rd, rot_dims,
                                                                                                   pos, cos_t, sin_t, (T *)q_out, pairing));
    return jl_check_launch("latent_q_pack_kernel");
}

template <typename T>
__global__ __launch_bounds__(256) void heads_gate_kernel(const T *__restrict__ ov, const T *__restrict__ gate, int64_t gate_ld, int64_t N, int H, int Dv,
                                                          T *__restrict__ out) {
    const int64_t n = blockIdx.x;
    for (int e = threadIdx.x; e < H * Dv; e += 256) {
        const int h = e / Dv, d = e - h * Dv;
        float v = ld_f(ov + ((int64_t)h * N + n) * Dv + d);
        if (gate) v *= 1.0f / (1.0f + expf(-ld_f(gate + n * gate_ld + e)));
        st_f(out + n * (int64_t)(H * Dv) + e, v);
    }
}

extern "C" int jl_heads_gate(const void *ov, const void *gate, int64_t gate_ld, int dtype, int64_t N, int32_t H, int32_t Dv, void *out,
                             void *stream) {
    if (N <= 0) return JL_OK;
    if (!ov || !out || H <= 0 || Dv <= 0 || (gate && gate_ld < (int64_t)H * Dv)) return jl_fail(JL_E_INVALID, "jl_heads_gate: null pointer or bad sizes");
    JL_DISPATCH(dtype, heads_gate_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>((const T *)ov, (const T *)gate, gate_ld, N, H, Dv, (T *)out));
    return jl_check_launch("heads_gate_kernel");
}
