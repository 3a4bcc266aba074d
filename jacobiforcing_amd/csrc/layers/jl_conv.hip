// jl_conv.hip — causal depthwise convolution over time on the float residual stream, added to its input, with the last inputs of
// every request carried in its state slot (so a prompt may be cut anywhere and decoding continues token by token).
#include "jl_common.h"

// one workgroup per row; a thread per channel.  Input t - taps + 1 + j of the request comes from the step's own rows when it is
// one of them, from the slot's tail when it lies before the step, and is zero before the sequence's start.  A request with ONE row in
// the step (decoding) also moves its tail here — its only reader is this thread, which has read what it needs; requests with more
// rows leave that to causal_conv_carry_kernel, after every row has read.
template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(const float *__restrict__ x, const T *__restrict__ w, const int32_t *__restrict__ row_req,
                                                           const int32_t *__restrict__ seq, float *tail, int W, int taps,
                                                           T *__restrict__ out) {
    const int64_t n = blockIdx.x;
    const int32_t *rec = seq + 4 * (int64_t)row_req[n];
    const int row0 = rec[0], count = rec[1], pos0 = rec[2], slot = rec[3];
    const int t = (int)(n - row0), keep = taps - 1;
    for (int c = threadIdx.x; c < W; c += 256) {
        float acc = x[n * W + c];
        for (int j = 0; j < taps; ++j) {
            const int u = t - keep + j;                         // index among the step's rows of this request
            float v = 0.f;
            if (u >= 0) v = x[(int64_t)(row0 + u) * W + c];
            else if (pos0 + u >= 0) v = tail[((int64_t)slot * keep + (keep + u)) * W + c];
            acc += ld_f(w + (int64_t)c * taps + j) * v;
        }
        st_f(out + n * W + c, acc);
        if (count == 1 && keep > 0) {                           // the tail moves one place on: entry j was read before entry j - 1 is written
            float *tl = tail + (int64_t)slot * keep * W + c;
            for (int j = 1; j < keep; ++j) tl[(int64_t)(j - 1) * W] = tl[(int64_t)j * W];
            tl[(int64_t)(keep - 1) * W] = x[n * W + c];
        }
    }
}

// The same for widths in multiples of four and up to eight taps: a workgroup walks CONV_ROWS consecutive rows, a thread owns four
// channels and keeps the last TAPS - 1 inputs in registers, so that every input row is read once (plus the reach into the rows or
// the tail before the workgroup's first row, and again where a new request starts).
constexpr int CONV_ROWS = 8;
template <typename T, int TAPS>
__global__ __launch_bounds__(256) void causal_conv_rows_kernel(const float *__restrict__ x, const T *__restrict__ w, const int32_t *__restrict__ row_req,
                                                                const int32_t *__restrict__ seq, float *tail, int64_t N, int W, T *__restrict__ out) {
    constexpr int KEEP = TAPS - 1;
    const int c = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (c >= W) return;
    float wv[4][TAPS];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int j = 0; j < TAPS; ++j) wv[k][j] = ld_f(w + (int64_t)(c + k) * TAPS + j);
    float4 win[KEEP > 0 ? KEEP : 1];
    int prev_req = -1;
    const int64_t n0 = (int64_t)blockIdx.x * CONV_ROWS;
    for (int r = 0; r < CONV_ROWS && n0 + r < N; ++r) {
        const int64_t n = n0 + r;
        const int req = row_req[n];
        const int32_t *rec = seq + 4 * (int64_t)req;
        const int row0 = rec[0], count = rec[1], pos0 = rec[2], slot = rec[3];
        const int t = (int)(n - row0);
        if (req != prev_req) {                                  // the inputs before this row: earlier rows of the step, the tail, or nothing
#pragma unroll
            for (int s2 = 0; s2 < KEEP; ++s2) {
                const int u = t - KEEP + s2;
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (u >= 0) v = *(const float4 *)(x + (int64_t)(row0 + u) * W + c);
                else if (pos0 + u >= 0) v = *(const float4 *)(tail + ((int64_t)slot * KEEP + (KEEP + u)) * W + c);
                win[s2] = v;
            }
            prev_req = req;
        }
        const float4 cur = *(const float4 *)(x + n * W + c);
        float a0, a1, a2, a3;
        a0 = cur.x + wv[0][KEEP] * cur.x; a1 = cur.y + wv[1][KEEP] * cur.y; a2 = cur.z + wv[2][KEEP] * cur.z; a3 = cur.w + wv[3][KEEP] * cur.w;
#pragma unroll
        for (int s2 = 0; s2 < KEEP; ++s2) {
            a0 += wv[0][s2] * win[s2].x; a1 += wv[1][s2] * win[s2].y; a2 += wv[2][s2] * win[s2].z; a3 += wv[3][s2] * win[s2].w;
        }
        T *o = out + n * W + c;
        st_f(o, a0); st_f(o + 1, a1); st_f(o + 2, a2); st_f(o + 3, a3);
#pragma unroll
        for (int s2 = 0; s2 + 1 < KEEP; ++s2) win[s2] = win[s2 + 1];
        if (KEEP > 0) win[KEEP - 1] = cur;
        if (count == 1 && KEEP > 0) {                           // a single row moves its request's tail on (its only reader is this thread)
#pragma unroll
            for (int s2 = 0; s2 < KEEP; ++s2) *(float4 *)(tail + ((int64_t)slot * KEEP + s2) * W + c) = win[s2];
        }
    }
}

template <typename T, int TAPS>
static void conv_rows_launch(const float *x, const void *w, const int32_t *row_req, const int32_t *seq, float *tail, int64_t N, int W, void *out,
                             hipStream_t st) {
    const dim3 grid((unsigned)((N + CONV_ROWS - 1) / CONV_ROWS), (unsigned)((W / 4 + 255) / 256));
    causal_conv_rows_kernel<T, TAPS><<<grid, 256, 0, st>>>(x, (const T *)w, row_req, seq, tail, N, W, (T *)out);
}

extern "C" int jl_causal_conv(const float *x, const void *w, int dtype, const int32_t *row_req, const int32_t *seq, float *tail,
                              int64_t N, int32_t W, int32_t taps, void *out, void *stream) {
    if (N <= 0) return JL_OK;
    if (!x || !w || !row_req || !seq || !out || W <= 0 || taps < 1 || taps > JL_CONV_MAX_TAPS || (taps > 1 && !tail))
        return jl_fail(JL_E_INVALID, "jl_causal_conv: null pointer, bad width or taps outside 1..%d", JL_CONV_MAX_TAPS);
    if (W % 4 == 0 && taps <= 8) {
#define CONV_CASE(TP) case TP: JL_DISPATCH(dtype, (conv_rows_launch<T, TP>(x, w, row_req, seq, tail, N, W, out, (hipStream_t)stream))); break
        switch (taps) { CONV_CASE(1); CONV_CASE(2); CONV_CASE(3); CONV_CASE(4); CONV_CASE(5); CONV_CASE(6); CONV_CASE(7); CONV_CASE(8); }
#undef CONV_CASE
        return jl_check_launch("causal_conv_rows_kernel");
    }
    JL_DISPATCH(dtype, causal_conv_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>(x, (const T *)w, row_req, seq, tail, W, taps,
                                                                                                  (T *)out));
    return jl_check_launch("causal_conv_kernel");
}

// the tail after the step: the last taps - 1 inputs up to the step's last row.  A thread owns a channel of a request: it reads
// everything it needs before it writes.
__global__ __launch_bounds__(256) void causal_conv_carry_kernel(const float *__restrict__ x, const int32_t *__restrict__ seq,
                                                                 float *__restrict__ tail, int W, int taps) {
    const int32_t *rec = seq + 4 * (int64_t)blockIdx.y;
    const int row0 = rec[0], count = rec[1], pos0 = rec[2], slot = rec[3], keep = taps - 1;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= W || count <= 1) return;                       // a single row has moved its tail in causal_conv_kernel
    float v[JL_CONV_MAX_TAPS];
#pragma unroll
    for (int s = 0; s < JL_CONV_MAX_TAPS - 1; ++s) {
        v[s] = 0.f;
        if (s < keep) {
            const int u = count - keep + s;
            if (u >= 0) v[s] = x[(int64_t)(row0 + u) * W + c];
            else if (pos0 + u >= 0) v[s] = tail[((int64_t)slot * keep + (keep + u)) * W + c];
        }
    }
#pragma unroll
    for (int s = 0; s < JL_CONV_MAX_TAPS - 1; ++s)
        if (s < keep) tail[((int64_t)slot * keep + s) * W + c] = v[s];
}

extern "C" int jl_causal_conv_carry(const float *x, const int32_t *seq, int32_t B, float *tail, int32_t W, int32_t taps, void *stream) {
    if (B <= 0 || taps <= 1) return JL_OK;
    if (!x || !seq || !tail || W <= 0 || taps > JL_CONV_MAX_TAPS) return jl_fail(JL_E_INVALID, "jl_causal_conv_carry: null pointer or bad sizes");
    causal_conv_carry_kernel<<<dim3((unsigned)((W + 255) / 256), (unsigned)B), 256, 0, (hipStream_t)stream>>>(x, seq, tail, W, taps);
    return jl_check_launch("causal_conv_carry_kernel");
}

// ---- short causal convolution of a column range of a projection, with an activation, no residual ---------------------------------------------
//   out[t, c] = act(sum_{j < taps} w[c, j] * x[t - taps + 1 + j, col + c])        (zeros before the sequence's start; float out)
// A workgroup walks CONV_ROWS consecutive rows, a thread owns a channel and keeps the last taps - 1 inputs in registers.  The tail
// (float [slots, taps - 1, C]) is read for the inputs before the step and moved on here by requests with ONE row; requests with more rows
// leave that to short_conv_carry_kernel, enqueued after every row has read.
template <typename T, int TAPS>
__global__ __launch_bounds__(256) void short_conv_kernel(const T *__restrict__ x, int64_t ld, int col, const T *__restrict__ w, const int32_t *__restrict__ row_req,
                                                          const int32_t *__restrict__ seq, float *tail, int64_t N, int C, int act, float *__restrict__ out) {
    constexpr int KEEP = TAPS - 1;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    float wv[TAPS], win[KEEP > 0 ? KEEP : 1];
#pragma unroll
    for (int j = 0; j < TAPS; ++j) wv[j] = ld_f(w + (int64_t)c * TAPS + j);
    int prev_req = -1;
    const int64_t n0 = (int64_t)blockIdx.x * CONV_ROWS;
    for (int r = 0; r < CONV_ROWS && n0 + r < N; ++r) {
        const int64_t n = n0 + r;
        const int req = row_req[n];
        const int32_t *rec = seq + 4 * (int64_t)req;
        const int row0 = rec[0], count = rec[1], pos0 = rec[2], slot = rec[3];
        const int t = (int)(n - row0);
        if (req != prev_req) {
#pragma unroll
            for (int s2 = 0; s2 < KEEP; ++s2) {
                const int u = t - KEEP + s2;
                float v = 0.f;
                if (u >= 0) v = ld_f(x + (int64_t)(row0 + u) * ld + col + c);
                else if (pos0 + u >= 0) v = tail[((int64_t)slot * KEEP + (KEEP + u)) * C + c];
                win[s2] = v;
            }
            prev_req = req;
        }
        const float cur = ld_f(x + n * ld + col + c);
        float a = wv[KEEP] * cur;
#pragma unroll
        for (int s2 = 0; s2 < KEEP; ++s2) a += wv[s2] * win[s2];
        out[n * C + c] = act == JL_ACT_SILU ? silu_f(a) : a;
#pragma unroll
        for (int s2 = 0; s2 + 1 < KEEP; ++s2) win[s2] = win[s2 + 1];
        if (KEEP > 0) win[KEEP - 1] = cur;
        if (count == 1 && KEEP > 0) {
#pragma unroll
            for (int s2 = 0; s2 < KEEP; ++s2) tail[((int64_t)slot * KEEP + s2) * C + c] = win[s2];
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void short_conv_carry_kernel(const T *__restrict__ x, int64_t ld, int col, const int32_t *__restrict__ seq,
                                                                float *__restrict__ tail, int C, int taps) {
    const int32_t *rec = seq + 4 * (int64_t)blockIdx.y;
    const int row0 = rec[0], count = rec[1], pos0 = rec[2], slot = rec[3], keep = taps - 1;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C || count <= 1) return;
    float v[JL_CONV_MAX_TAPS];
#pragma unroll
    for (int s = 0; s < JL_CONV_MAX_TAPS - 1; ++s) {
        v[s] = 0.f;
        if (s < keep) {
            const int u = count - keep + s;
            if (u >= 0) v[s] = ld_f(x + (int64_t)(row0 + u) * ld + col + c);
            else if (pos0 + u >= 0) v[s] = tail[((int64_t)slot * keep + (keep + u)) * C + c];
        }
    }
#pragma unroll
    for (int s = 0; s < JL_CONV_MAX_TAPS - 1; ++s)
        if (s < keep) tail[((int64_t)slot * keep + s) * C + c] = v[s];
}

template <typename T, int TAPS>
static void short_conv_launch(const void *x, int64_t ld, int col, const void *w, const int32_t *row_req, const int32_t *seq, float *tail, int64_t N, int C,
                              int act, float *out, hipStream_t st) {
    const dim3 grid((unsigned)((N + CONV_ROWS - 1) / CONV_ROWS), (unsigned)((C + 255) / 256));
    short_conv_kernel<T, TAPS><<<grid, 256, 0, st>>>((const T *)x, ld, col, (const T *)w, row_req, seq, tail, N, C, act, out);
}

extern "C" int jl_short_conv(const void *x, int dtype, int64_t ld, int32_t col, const void *w, const int32_t *row_req, const int32_t *seq, int32_t B,
                             int32_t max_count, float *tail, int64_t N, int32_t C, int32_t taps, int32_t act, float *out, void *stream) {
    if (N <= 0) return JL_OK;
    if (!x || !w || !row_req || !seq || !out || C <= 0 || col < 0 || col + (int64_t)C > ld || taps < 1 || taps > 8 || (taps > 1 && !tail))
        return jl_fail(JL_E_INVALID, "jl_short_conv: null pointer, columns outside the row, or taps outside 1..8");
    if (act != JL_ACT_SILU && act != JL_ACT_NONE) return jl_fail(JL_E_INVALID, "jl_short_conv: unknown activation %d", act);
    hipStream_t st = (hipStream_t)stream;
#define CONV_CASE(TP) case TP: JL_DISPATCH(dtype, (short_conv_launch<T, TP>(x, ld, col, w, row_req, seq, tail, N, C, act, out, st))); break
    switch (taps) { CONV_CASE(1); CONV_CASE(2); CONV_CASE(3); CONV_CASE(4); CONV_CASE(5); CONV_CASE(6); CONV_CASE(7); CONV_CASE(8); }
#undef CONV_CASE
    int rc = jl_check_launch("short_conv_kernel");
    if (rc != JL_OK || taps == 1 || max_count <= 1) return rc;
    JL_DISPATCH(dtype, short_conv_carry_kernel<T><<<dim3((unsigned)((C + 255) / 256), (unsigned)B), 256, 0, st>>>((const T *)x, ld, col, seq, tail, C, taps));
    return jl_check_launch("short_conv_carry_kernel");
}
