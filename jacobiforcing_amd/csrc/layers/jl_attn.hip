// jl_attn.hip — query / key norm + paged append, and attention with a sliding window that keeps the first tokens, a bucketed
// distance bias and mixed heads, for prompt portions and single decoded tokens alike (one ragged launch).
#include "jl_common.h"
#include <stdlib.h>
#include <type_traits>

// ---- whole-projection q / k norm + append: one workgroup per token ------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_append_kernel(const T *__restrict__ proj, int64_t ld, int q_col, int k_col, int v_col,
                                                              int HD, int GD, int GDv, const T *__restrict__ wq, const T *__restrict__ wk,
                                                              float eps, T *__restrict__ q_out, T *__restrict__ k_cache,
                                                              T *__restrict__ v_cache, const int64_t *__restrict__ slot) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    const T *row = proj + n * ld;
    float sq = 0.f, sk = 0.f;
    for (int c = threadIdx.x; c < HD; c += 256) { const float v = ld_f(row + q_col + c); sq += v * v; }
    for (int c = threadIdx.x; c < GD; c += 256) { const float v = ld_f(row + k_col + c); sk += v * v; }
    sq = block_sum_f32(sq, red);
    sk = block_sum_f32(sk, red);
    const float rq = 1.0f / sqrtf(sq / (float)HD + eps), rk = 1.0f / sqrtf(sk / (float)GD + eps);
    for (int c = threadIdx.x; c < HD; c += 256) st_f(q_out + n * HD + c, ld_f(row + q_col + c) * rq * ld_f(wq + c));
    const int64_t sl = slot[n];
    if (sl < 0) return;
    for (int c = threadIdx.x; c < GD; c += 256) st_f(k_cache + sl * GD + c, ld_f(row + k_col + c) * rk * ld_f(wk + c));
    for (int c = threadIdx.x; c < GDv; c += 256) v_cache[sl * GDv + c] = row[v_col + c];
}

extern "C" int jl_qk_norm_append(const void *proj, int dtype, int64_t N, int64_t ld, int32_t q_col, int32_t k_col, int32_t v_col,
                                 int32_t H, int32_t G, int32_t D, int32_t Dv, const void *wq, const void *wk, float eps, void *q_out,
                                 void *k_cache, void *v_cache, const int64_t *slot, void *stream) {
    if (N <= 0) return JL_OK;
    if (!proj || !wq || !wk || !q_out || !k_cache || !v_cache || !slot) return jl_fail(JL_E_INVALID, "jl_qk_norm_append: null pointer");
    if (H <= 0 || G <= 0 || D <= 0 || Dv <= 0 || q_col + H * D > ld || k_col + G * D > ld || v_col + G * Dv > ld)
        return jl_fail(JL_E_INVALID, "jl_qk_norm_append: columns do not fit the row stride");
    JL_DISPATCH(dtype, qk_norm_append_kernel<T><<<dim3((unsigned)N), 256, 0, (hipStream_t)stream>>>(
                           (const T *)proj, ld, q_col, k_col, v_col, H * D, G * D, G * Dv, (const T *)wq, (const T *)wk, eps, (T *)q_out,
                           (T *)k_cache, (T *)v_cache, slot));
    return jl_check_launch("qk_norm_append_kernel");
}

// ---- attention ---------------------------------------------------------------------------------------------------------------
// One workgroup per tile of up to TQ consecutive query rows of one request, all heads (mixing the heads needs every head's
// weight of a (query, key) pair in one place).  Two sweeps over the visible keys, TK keys at a time through LDS:
//   sweep 1: scores -> running maximum and sum per (head, query);
//   sweep 2: scores again -> normalised weights -> mixed over the heads -> times the values.
// The visible keys of a tile are the kept first tokens below the window's lowest key and the window's own range; the exact
// mask is applied per (query, key).
constexpr int ATT_THREADS = 256;
constexpr int ATT_LDS_BUDGET = 144 * 1024;

struct AttShape { int TQ, TK, ACC; size_t lds; };

static bool att_shape(int H, int G, int D, int Dv, int tq_want, AttShape *o) {
    const int per_row = H * Dv;
    int acc = 16;                                       // accumulators per thread: 16 (one query row of up to 4096 outputs) or 64
    if (per_row > acc * ATT_THREADS) acc = 64;
    if (per_row > acc * ATT_THREADS) return false;
    int tq = acc * ATT_THREADS / per_row;
    if (tq > 16) tq = 16;
    if (tq_want > 0 && tq > tq_want) tq = tq_want;
    const int kvw = (D + 1 > Dv ? D + 1 : Dv) * G;
    for (; tq >= 1; tq = tq > 1 ? tq / 2 : 0) {
        for (int tk = 64; tk >= 4; tk /= 2) {
            const size_t fl = (size_t)tq * H * D + (size_t)tk * kvw + 2 * (size_t)H * tq * tk + 2 * (size_t)H * tq + (size_t)H * H + 64;
            if (fl * 4 <= (size_t)ATT_LDS_BUDGET) { o->TQ = tq; o->TK = tk; o->ACC = acc; o->lds = fl * 4; return true; }
        }
        if (tq == 1) break;
    }
    return false;
}

static bool am_fits(int dtype, int H, int G, int D, int Dv);
// the matrix-core kernel loads pool rows in 8-byte units: row strides must be multiples of four elements
static bool am_strides_ok(int64_t k_ld, int64_t v_ld) { return k_ld % 4 == 0 && v_ld % 4 == 0; }

extern "C" int64_t jl_attn_scratch_floats(int32_t n_tiles, int32_t n_rows, int32_t H, int32_t Dv, int32_t splits) {
    return splits > 1 ? (int64_t)n_tiles * splits * H * 32 * 2 + (int64_t)splits * n_rows * H * Dv : 0;
}

extern "C" int jl_attn_tile_rows(int dtype, int32_t H, int32_t G, int32_t D, int32_t Dv, int64_t k_ld, int64_t v_ld) {
    if (H <= 0 || G <= 0 || H % G || D <= 0 || Dv <= 0) return 0;
    if (am_fits(dtype, H, G, D, Dv) && am_strides_ok(k_ld, v_ld)) return 32;
    AttShape s;
    return att_shape(H, G, D, Dv, 0, &s) ? s.TQ : 0;
}

template <typename T, int ACC>
__global__ __launch_bounds__(ATT_THREADS) void attn_window_kernel(jl_attn_args a, int TK) {
    extern __shared__ float lds[];
    const int H = a.H, G = a.G, D = a.D, Dv = a.Dv, TQ = a.TQ, rep = H / G, Gv = a.Gv;
    const int tid = threadIdx.x;
    const int *tile = a.tiles + 4 * (int64_t)blockIdx.x;
    const int b = tile[0], i0 = tile[1], cnt = tile[2], row0 = tile[3];
    if (b < 0 || cnt <= 0) return;
    const int kstride = D + 1;
    const int kvw = (kstride > Dv ? kstride : Dv) * G;
    float *Qs = lds;                                    // [TQ][H][D]
    float *KV = Qs + TQ * H * D;                        // [G][TK][D+1] keys (odd row stride: no bank conflicts over the keys), then [TK][G][Dv] values
    float *S = KV + TK * kvw;                           // [H][TQ][TK]
    float *Wm = S + H * TQ * TK;                        // [H][TQ][TK]
    float *mx = Wm + H * TQ * TK;                       // [H][TQ]
    float *sm = mx + H * TQ;                            // [H][TQ]
    float *talk = sm + H * TQ;                          // [H][H]
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_max = i0 + cnt - 1;
    const int lo = i0 - window + 1 > 0 ? i0 - window + 1 : 0;
    const int kf_end = a.keep_first < lo ? a.keep_first : lo;
    const int n_keys = kf_end + (i_max + 1 - lo);
    const int *bt = a.block_tables + (int64_t)b * a.bt_stride;
    const T *q = (const T *)a.q;
    const T *kc = (const T *)a.k_cache;
    const T *vc = (const T *)a.v_cache;

    for (int e = tid; e < cnt * H * D; e += ATT_THREADS) Qs[e] = ld_f(q + (int64_t)row0 * H * D + e);
    // a sink acts like one extra score that attends to nothing: every row's statistics start from (sink, 1)
    for (int e = tid; e < H * TQ; e += ATT_THREADS) { mx[e] = a.sink ? a.sink[e / TQ] : -INFINITY; sm[e] = a.sink ? 1.f : 0.f; }
    if (a.talk) for (int e = tid; e < H * H; e += ATT_THREADS) talk[e] = a.talk[e];

    float acc[ACC];
#pragma unroll
    for (int x = 0; x < ACC; ++x) acc[x] = 0.f;

    for (int sweep = 0; sweep < 2; ++sweep) {
        for (int u0 = 0; u0 < n_keys; u0 += TK) {
            const int nk = n_keys - u0 < TK ? n_keys - u0 : TK;
            __syncthreads();                                        // the previous tile's readers are done with KV / S / Wm
            for (int e = tid; e < nk * G * D; e += ATT_THREADS) {
                const int jj = e / (G * D), r = e - jj * (G * D), c = r / D, d = r - c * D;
                const int u = u0 + jj, j = u < kf_end ? u : lo + (u - kf_end);
                const int64_t tok = (int64_t)bt[j / a.page_size] * a.page_size + j % a.page_size;
                KV[(c * TK + jj) * kstride + d] = ld_f(kc + tok * a.k_ld + r);
            }
            __syncthreads();
            for (int e = tid; e < H * cnt * nk; e += ATT_THREADS) {
                const int g = e / (cnt * nk), r = e - g * (cnt * nk), ii = r / nk, jj = r - ii * nk;
                const int u = u0 + jj, j = u < kf_end ? u : lo + (u - kf_end), i = i0 + ii;
                float s = -INFINITY;
                if (j <= i && (i - j < window || j < a.keep_first)) {
                    const float *qp = Qs + (ii * H + g) * D, *kp = KV + ((g / rep) * TK + jj) * kstride;
                    float dot = 0.f;
                    for (int d = 0; d < D; ++d) dot += qp[d] * kp[d];
                    s = dot * a.scale;
                    if (a.rel) {
                        const int n = i - j < a.lut_len ? i - j : a.lut_len - 1;
                        s += a.rel[(a.lut ? a.lut[n] : n) * H + g];
                    }
                }
                S[(g * TQ + ii) * TK + jj] = s;
            }
            __syncthreads();
            if (sweep == 0) {
                for (int e = tid; e < H * cnt; e += ATT_THREADS) {
                    const int g = e / cnt, ii = e - g * cnt;
                    const float *sp = S + (g * TQ + ii) * TK;
                    float m = mx[g * TQ + ii], l = sm[g * TQ + ii], t = m;
                    for (int jj = 0; jj < nk; ++jj) t = fmaxf(t, sp[jj]);
                    if (t > -INFINITY) {
                        l = l * __expf(m - t);                       // m = -inf: l is 0 and stays 0
                        for (int jj = 0; jj < nk; ++jj) l += expf(sp[jj] - t);
                        mx[g * TQ + ii] = t;
                        sm[g * TQ + ii] = l;
                    }
                }
                continue;
            }
            for (int e = tid; e < H * cnt * nk; e += ATT_THREADS) {
                const int g = e / (cnt * nk), r = e - g * (cnt * nk), ii = r / nk, jj = r - ii * nk;
                const int o = (g * TQ + ii) * TK + jj;
                S[o] = expf(S[o] - mx[g * TQ + ii]) / sm[g * TQ + ii];
            }
            for (int e = tid; e < nk * Gv * Dv; e += ATT_THREADS) {  // keys are no longer read: the values take their place
                const int jj = e / (Gv * Dv), r = e - jj * (Gv * Dv);
                const int u = u0 + jj, j = u < kf_end ? u : lo + (u - kf_end);
                const int64_t tok = (int64_t)bt[j / a.page_size] * a.page_size + j % a.page_size;
                KV[jj * (Gv * Dv) + r] = ld_f(vc + tok * a.v_ld + r);
            }
            __syncthreads();
            const float *Wp = S;
            if (a.talk) {
                for (int e = tid; e < H * cnt * nk; e += ATT_THREADS) {
                    const int h = e / (cnt * nk), r = e - h * (cnt * nk), ii = r / nk, jj = r - ii * nk;
                    float w = 0.f;
                    for (int g = 0; g < H; ++g) w += talk[h * H + g] * S[(g * TQ + ii) * TK + jj];
                    Wm[(h * TQ + ii) * TK + jj] = w;
                }
                __syncthreads();
                Wp = Wm;
            }
#pragma unroll
            for (int x = 0; x < ACC; ++x) {
                const int e = x * ATT_THREADS + tid;
                if (e < cnt * H * Dv) {
                    const int ii = e / (H * Dv), r = e - ii * (H * Dv), h = r / Dv, d = r - h * Dv;
                    const float *wp = Wp + (h * TQ + ii) * TK, *vp = KV + ((h / rep) % Gv) * Dv + d;
                    float s = acc[x];
                    for (int jj = 0; jj < nk; ++jj) s += wp[jj] * vp[jj * (Gv * Dv)];
                    acc[x] = s;
                }
            }
        }
    }
    T *out = (T *)a.out;
    const T *gate = (const T *)a.gate;
#pragma unroll
    for (int x = 0; x < ACC; ++x) {
        const int e = x * ATT_THREADS + tid;
        if (e < cnt * H * Dv) {
            const int ii = e / (H * Dv), r = e - ii * (H * Dv);
            float v = acc[x];
            if (gate) v *= 1.0f / (1.0f + expf(-ld_f(gate + (int64_t)(row0 + ii) * a.gate_ld + (a.gate_heads ? r / Dv : r))));
            if (a.out_dtype == JL_OUT_F32) ((float *)a.out)[(int64_t)(row0 + ii) * (H * Dv) + r] = v;
            else st_f(out + (int64_t)(row0 + ii) * (H * Dv) + r, v);
        }
    }
}

// ---- the same attention on the matrix cores (bfloat16; H <= 16, D a multiple of 8 up to 256, Dv up to 128) -----------
// A tile of 32 query rows of one request, all heads; wavefront w owns heads w * HPW .. (HPW = 1 or 2).  Keys go through LDS 32 at a
// time.  v_mfma_f32_32x32x8_bf16: lane l supplies row (A) or column (B) l % 32 with depths 4 * (l / 32) .. + 3; accumulator r of lane
// l is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.
//   sweep 1: S = Q K^T per own head; every lane keeps a running maximum and sum for its 16 rows over its column; merged over the
//            lanes at the end -> maximum and 1 / sum per (head, row) in LDS.
//   sweep 2: S again -> p = exp(s - max) / sum in float -> LDS, all heads; after a barrier every wavefront mixes the heads'
//            weights for its own heads directly in the A-operand layout (w = sum_g talk[h, g] p_g, float, rounded once to
//            bfloat16) and multiplies by the value tile.
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short am_bf16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float am_f32x16;
constexpr int AM_T = 32;
constexpr int AM_PAGES = 1024;     // page-table entries of a request kept in LDS (longer tables are read from memory)
constexpr int AM_FUSED = 0, AM_STATS = 1, AM_PV = 2;    // both sweeps in one launch; or the keys split over workgroups: statistics, then outputs

__device__ __forceinline__ short am_bf16(float v) {
    uint32_t u = __float_as_uint(v);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (short)(u >> 16);
}

__device__ __forceinline__ void am_load_tile(bf16_t *dst, int dst_row, const bf16_t *src, int src_row, int units, int jj, int r, int dj, int dr,
                                             int nk, int u0, int kf_end, int lo, const int *bt, int page_size, int page_shift, int tid,
                                             int nthr) {
    for (int e0 = tid; e0 < AM_T * units; e0 += 4 * nthr) {
        uint2 v[4];
        int off[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            v[it] = make_uint2(0, 0);
            off[it] = -1;
            if (e0 + it * nthr < AM_T * units) {
                off[it] = jj * dst_row + 4 * r;
                if (jj < nk) {
                    const int u = u0 + jj, j = u < kf_end ? u : lo + (u - kf_end);
                    const int pg = page_shift >= 0 ? j >> page_shift : j / page_size;
                    const int64_t tok = (int64_t)bt[pg] * page_size + (j - pg * page_size);
                    v[it] = *(const uint2 *)(src + tok * src_row + 4 * r);
                }
                jj += dj; r += dr;
                if (r >= units) { r -= units; ++jj; }
            }
        }
#pragma unroll
        for (int it = 0; it < 4; ++it)
            if (off[it] >= 0) *(uint2 *)(dst + off[it]) = v[it];
    }
}

// The same loader in two halves, for tiles that are fetched one iteration ahead: am_fetch issues a thread's loads (at most PF of
// them) into registers, am_stash writes them to LDS once the previous tile's readers are done.  `pages` is the request's page
// table (in LDS when it fits there).
constexpr int AM_PF = 4;
__device__ __forceinline__ void am_fetch(uint2 (&v)[AM_PF], const bf16_t *src, int src_row, int units, int jj, int r, int dj, int dr, int nk,
                                         int u0, int kf_end, int lo, const int *pages, int page_size, int page_shift, int tid, int nthr) {
#pragma unroll
    for (int it = 0; it < AM_PF; ++it) {
        v[it] = make_uint2(0, 0);
        if (tid + it * nthr < AM_T * units) {
            if (jj < nk) {
                const int u = u0 + jj, j = u < kf_end ? u : lo + (u - kf_end);
                const int pg = page_shift >= 0 ? j >> page_shift : j / page_size;
                const int64_t tok = (int64_t)pages[pg] * page_size + (j - pg * page_size);
                v[it] = *(const uint2 *)(src + tok * src_row + 4 * r);
            }
            jj += dj; r += dr;
            if (r >= units) { r -= units; ++jj; }
        }
    }
}
__device__ __forceinline__ void am_stash(const uint2 (&v)[AM_PF], bf16_t *dst, int dst_row, int units, int jj, int r, int dj, int dr, int tid,
                                         int nthr) {
#pragma unroll
    for (int it = 0; it < AM_PF; ++it)
        if (tid + it * nthr < AM_T * units) {
            *(uint2 *)(dst + jj * dst_row + 4 * r) = v[it];
            jj += dj; r += dr;
            if (r >= units) { r -= units; ++jj; }
        }
}

static size_t am_lds_bytes(int H, int G, int D, int Dv) {
    return (size_t)AM_T * (G * D + 4) * 2 + (size_t)AM_T * G * Dv * 2 + ((size_t)H * AM_T * 33 + 2 * (size_t)H * AM_T + (size_t)H * H + (size_t)H * 64 + AM_PAGES) * 4;
}

template <int HPW, int NDV>
__global__ __launch_bounds__(512) void attn_mfma_kernel(jl_attn_args a, int mode) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int H = a.H, G = a.G, D = a.D, Dv = a.Dv, rep = H / G, KROW = G * D + 4, Gv = a.Gv, VROW = Gv * Dv;
    const int tid = threadIdx.x, nthr = blockDim.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, hi = lane >> 5;
    const int *tile = a.tiles + 4 * (int64_t)blockIdx.x;
    const int b = tile[0], i0 = tile[1], cnt = tile[2], row0 = tile[3];
    if (b < 0 || cnt <= 0) return;
    bf16_t *Ks = (bf16_t *)smem;                                   // [32][G * D + 4]
    bf16_t *Vs = Ks + AM_T * KROW;                                 // [32][Gv * Dv] (room for G * Dv)
    float *Ps = (float *)(Vs + AM_T * G * Dv);                     // [H][32][33]
    float *mS = Ps + H * AM_T * 33;                                // [H][32] row maximum
    float *lS = mS + H * AM_T;                                     // [H][32] 1 / row sum
    float *talk = lS + H * AM_T;                                   // [H][H]
    float *biasS = talk + H * H;                                   // [H][64] the distance bias of a key tile: entry ii - jj + 31
    int *pageS = (int *)(biasS + H * 64);                          // [AM_PAGES] this request's page table up to the tile's last key
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_max = i0 + cnt - 1;
    const int lo = i0 - window + 1 > 0 ? i0 - window + 1 : 0;
    const int kf_end = a.keep_first < lo ? a.keep_first : lo;
    const int n_keys = kf_end + (i_max + 1 - lo);
    const int *bt = a.block_tables + (int64_t)b * a.bt_stride;
    const bf16_t *kc = (const bf16_t *)a.k_cache, *vc = (const bf16_t *)a.v_cache;
    if (a.talk) for (int e = tid; e < H * H; e += nthr) talk[e] = a.talk[e];
    const int n_pages = i_max / a.page_size + 1;
    if (n_pages <= AM_PAGES) {                                      // one trip to memory for the page table instead of one per tile
        for (int e = tid; e < n_pages; e += nthr) pageS[e] = bt[e];
        __syncthreads();
        bt = pageS;
    }
    // loaders' starting points and steps (e = tid, tid + nthr, ..: key e / units, unit e % units)
    const int kq = G * D / 4, vq = VROW / 4;
    const int jj_k0 = tid / kq, r_k0 = tid - jj_k0 * kq, dj_k = nthr / kq, dr_k = nthr - dj_k * kq;
    const int jj_v0 = tid / vq, r_v0 = tid - jj_v0 * vq, dj_v = nthr / vq, dr_v = nthr - dj_v * vq;
    const int page_shift = (a.page_size & (a.page_size - 1)) == 0 ? __builtin_ctz(a.page_size) : -1;
    // keys split over blockIdx.y (few tiles with many keys: decoding): this workgroup's share of the 32-key tiles
    const int S = a.splits > 1 ? a.splits : 1, split = blockIdx.y;
    const int per = ((n_keys + AM_T - 1) / AM_T + S - 1) / S;
    const int key_lo = split * per * AM_T, key_hi = (split + 1) * per * AM_T < n_keys ? (split + 1) * per * AM_T : n_keys;
    float *ml = a.scratch;                                          // [tiles][S][H][32][2] maximum, sum of a split
    float *po = a.scratch + (int64_t)a.n_tiles * S * H * AM_T * 2;  // [S][rows][H * Dv] a split's share of the outputs
    if (mode == AM_PV) {                                            // join the splits' statistics of this tile
        for (int e = tid; e < H * AM_T; e += nthr) {
            float M = -INFINITY, L = 0.f;
            for (int sp = 0; sp < S; ++sp) M = fmaxf(M, ml[(((int64_t)blockIdx.x * S + sp) * H * AM_T + e) * 2]);
            for (int sp = 0; sp < S; ++sp) {
                const float *p2 = ml + (((int64_t)blockIdx.x * S + sp) * H * AM_T + e) * 2;
                if (p2[0] > -INFINITY) L += p2[1] * __expf(p2[0] - M);
            }
            mS[e] = M;
            lS[e] = L > 0.f ? 1.0f / L : 0.f;
        }
    }

    float m_run[HPW][16], l_run[HPW][16];
    am_f32x16 acc[HPW][NDV];
#pragma unroll
    for (int x = 0; x < HPW; ++x)
#pragma unroll
        for (int r = 0; r < 16; ++r) { m_run[x][r] = -INFINITY; l_run[x][r] = 0.f; }
    if (a.sink && split == 0 && l32 == 0) {                         // the sink enters every row's statistics once: first share, one lane per row
#pragma unroll
        for (int x = 0; x < HPW; ++x) {
            const int g = wave * HPW + x;
            if (g < H) {
                const float sk = a.sink[g];
#pragma unroll
                for (int r = 0; r < 16; ++r) { m_run[x][r] = sk; l_run[x][r] = 1.f; }
            }
        }
    }

    // fetch one tile ahead when a thread's share of a tile fits the registers set aside for it (one head per wavefront only: with
    // two the accumulators leave no room)
    const bool ahead = HPW == 1 && AM_T * kq <= AM_PF * nthr && AM_T * vq <= AM_PF * nthr;
    uint2 pk[AM_PF], pv[AM_PF];
    // one body, instantiated per sweep (the accumulators exist in the second only, the running statistics in the first only)
    auto run_sweep = [&](auto sweep_c) {
        constexpr int sweep = decltype(sweep_c)::value;
        if (ahead && key_lo < key_hi) {
            const int nk0 = key_hi - key_lo < AM_T ? key_hi - key_lo : AM_T;
            am_fetch(pk, kc, a.k_ld, kq, jj_k0, r_k0, dj_k, dr_k, nk0, key_lo, kf_end, lo, bt, a.page_size, page_shift, tid, nthr);
            if (sweep == 1) am_fetch(pv, vc, a.v_ld, vq, jj_v0, r_v0, dj_v, dr_v, nk0, key_lo, kf_end, lo, bt, a.page_size, page_shift, tid, nthr);
        }
        for (int u0 = key_lo; u0 < key_hi; u0 += AM_T) {
            const int nk = key_hi - u0 < AM_T ? key_hi - u0 : AM_T;
            __syncthreads();                                        // the previous tile's readers are done
            if (ahead) {                                            // this tile was fetched during the previous one
                am_stash(pk, Ks, KROW, kq, jj_k0, r_k0, dj_k, dr_k, tid, nthr);
                if (sweep == 1) am_stash(pv, Vs, VROW, vq, jj_v0, r_v0, dj_v, dr_v, tid, nthr);
            } else {
                // 8-byte units: thread -> (key jj, unit r of the key's row), stepped without divisions; four loads of a thread are
                // issued before the first is stored
                am_load_tile(Ks, KROW, kc, a.k_ld, kq, jj_k0, r_k0, dj_k, dr_k, nk, u0, kf_end, lo, bt, a.page_size, page_shift, tid, nthr);
                if (sweep == 1)
                    am_load_tile(Vs, VROW, vc, a.v_ld, vq, jj_v0, r_v0, dj_v, dr_v, nk, u0, kf_end, lo, bt, a.page_size, page_shift, tid, nthr);
            }
            __syncthreads();
            if (ahead && u0 + AM_T < key_hi) {                      // the next tile's rows travel while this one is computed
                const int nk2 = key_hi - (u0 + AM_T) < AM_T ? key_hi - (u0 + AM_T) : AM_T;
                am_fetch(pk, kc, a.k_ld, kq, jj_k0, r_k0, dj_k, dr_k, nk2, u0 + AM_T, kf_end, lo, bt, a.page_size, page_shift, tid, nthr);
                if (sweep == 1) am_fetch(pv, vc, a.v_ld, vq, jj_v0, r_v0, dj_v, dr_v, nk2, u0 + AM_T, kf_end, lo, bt, a.page_size, page_shift, tid, nthr);
            }
            // this lane's key (column l32 of the tile); `straight`: the tile's keys are consecutive positions
            const int u = u0 + l32, j = u < kf_end ? u : lo + (u - kf_end);
            const bool straight = u0 >= kf_end || u0 + AM_T <= kf_end;
#pragma unroll
            for (int x = 0; x < HPW; ++x) {
                const int g = wave * HPW + x;
                if (g >= H) continue;
                const int c = g / rep;
                if (a.rel) {                                        // 63 distances occur in a 32 x 32 tile: one table lookup per lane
                    const int jt = u0 < kf_end ? u0 : lo + (u0 - kf_end);      // position of the tile's first key (a tile that crosses from
                    int n = i0 - jt + lane - 31;                                // the kept tokens into the window is handled per element)
                    n = n < 0 ? 0 : (n < a.lut_len ? n : a.lut_len - 1);
                    biasS[g * 64 + lane] = a.rel[(a.lut ? a.lut[n] : n) * H + g];
                }
                am_f32x16 sc;
#pragma unroll
                for (int r = 0; r < 16; ++r) sc[r] = 0.f;
                // queries in operand order (attn_pack_q_kernel): a step's 64 lanes read 512 consecutive bytes
                const am_bf16x4 *qp = (const am_bf16x4 *)a.q_pack + ((int64_t)blockIdx.x * H + g) * (D / 8) * 64 + lane;
                const bf16_t *kp = Ks + l32 * KROW + c * D + 4 * hi;
                if constexpr (HPW == 1) {
#pragma unroll 8
                    for (int kk = 0; kk < D; kk += 8) {              // unrolled: the query loads of eight steps are in flight together
                        const am_bf16x4 qa = qp[(kk >> 3) * 64];
                        const am_bf16x4 kb = *(const am_bf16x4 *)(kp + kk);
                        sc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(qa, kb, sc, 0, 0, 0);
                    }
                } else {                                             // two heads' accumulators leave room for fewer loads in flight
#pragma unroll 2
                    for (int kk = 0; kk < D; kk += 8) {
                        const am_bf16x4 qa = qp[(kk >> 3) * 64];
                        const am_bf16x4 kb = *(const am_bf16x4 *)(kp + kk);
                        sc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(qa, kb, sc, 0, 0, 0);
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int ii = 8 * (r >> 2) + 4 * hi + (r & 3), i = i0 + ii;
                    const bool ok = ii < cnt && l32 < nk && j <= i && (i - j < window || j < a.keep_first);
                    float s = -INFINITY;
                    if (ok) {
                        s = sc[r] * a.scale;
                        if (a.rel) {
                            if (straight) {
                                s += biasS[g * 64 + ii - l32 + 31];
                            } else {
                                const int n = i - j < a.lut_len ? i - j : a.lut_len - 1;
                                s += a.rel[(a.lut ? a.lut[n] : n) * H + g];
                            }
                        }
                    }
                    if (sweep == 0) {
                        const float t = fmaxf(m_run[x][r], s);
                        if (t > -INFINITY) {
                            l_run[x][r] = l_run[x][r] * __expf(m_run[x][r] - t) + __expf(s - t);
                            m_run[x][r] = t;
                        }
                    } else {
                        Ps[(g * AM_T + ii) * 33 + l32] = ok ? __expf(s - mS[g * AM_T + ii]) * lS[g * AM_T + ii] : 0.f;
                    }
                }
            }
            if (sweep == 0) continue;
            __syncthreads();
            // mixed weights of the own heads in the A layout (row l32, keys 8 s + 4 hi ..), times the values
#pragma unroll
            for (int sK = 0; sK < AM_T / 8; ++sK) {
                const int j0 = 8 * sK + 4 * hi;
                float w[HPW][4];
#pragma unroll
                for (int x = 0; x < HPW; ++x)
#pragma unroll
                    for (int qd = 0; qd < 4; ++qd) w[x][qd] = 0.f;
                if (a.talk) {
                    for (int g = 0; g < H; ++g) {
                        const float *pp = Ps + (g * AM_T + l32) * 33 + j0;
                        const float p0 = pp[0], p1 = pp[1], p2 = pp[2], p3 = pp[3];
#pragma unroll
                        for (int x = 0; x < HPW; ++x) {
                            const int h = wave * HPW + x;
                            const float tw = h < H ? talk[h * H + g] : 0.f;
                            w[x][0] += tw * p0; w[x][1] += tw * p1; w[x][2] += tw * p2; w[x][3] += tw * p3;
                        }
                    }
                } else {
#pragma unroll
                    for (int x = 0; x < HPW; ++x) {
                        const int h = wave * HPW + x;
                        if (h < H)
#pragma unroll
                            for (int qd = 0; qd < 4; ++qd) w[x][qd] = Ps[(h * AM_T + l32) * 33 + j0 + qd];
                    }
                }
#pragma unroll
                for (int x = 0; x < HPW; ++x) {
                    const int h = wave * HPW + x;
                    if (h >= H) continue;
                    const int c = (h / rep) % Gv;
                    const am_bf16x4 wa = {am_bf16(w[x][0]), am_bf16(w[x][1]), am_bf16(w[x][2]), am_bf16(w[x][3])};
#pragma unroll
                    for (int t = 0; t < NDV; ++t) {
                        if (32 * t >= Dv) continue;
                        const bf16_t *vp = Vs + j0 * VROW + c * Dv + 32 * t + l32;
                        const am_bf16x4 vb = {(short)vp[0], (short)vp[VROW], (short)vp[2 * VROW], (short)vp[3 * VROW]};
                        acc[x][t] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(wa, vb, acc[x][t], 0, 0, 0);
                    }
                }
            }
        }
    };
    if (mode != AM_PV) {
        run_sweep(std::integral_constant<int, 0>{});
        {
            // merge the lanes' running statistics: rows are shared by the 32 lanes of a half wavefront
#pragma unroll
            for (int x = 0; x < HPW; ++x) {
                const int g = wave * HPW + x;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float M = m_run[x][r];
#pragma unroll
                    for (int off = 16; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off, 64));
                    float L = M > -INFINITY ? l_run[x][r] * __expf(m_run[x][r] - M) : 0.f;
#pragma unroll
                    for (int off = 16; off > 0; off >>= 1) L += __shfl_xor(L, off, 64);
                    const int ii = 8 * (r >> 2) + 4 * hi + (r & 3);
                    if (l32 == 0 && g < H) {
                        if (mode == AM_STATS) {
                            float *p2 = ml + ((((int64_t)blockIdx.x * S + split) * H + g) * AM_T + ii) * 2;
                            p2[0] = M;
                            p2[1] = L;
                        } else {
                            mS[g * AM_T + ii] = M;
                            lS[g * AM_T + ii] = L > 0.f ? 1.0f / L : 0.f;
                        }
                    }
                }
            }
        }
    }
    if (mode == AM_STATS) return;
#pragma unroll
    for (int x = 0; x < HPW; ++x)
#pragma unroll
        for (int t = 0; t < NDV; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[x][t][r] = 0.f;
    run_sweep(std::integral_constant<int, 1>{});
    if (mode == AM_PV) {                                            // float shares; attn_join_kernel adds them up and gates
#pragma unroll
        for (int x = 0; x < HPW; ++x) {
            const int h = wave * HPW + x;
            if (h >= H) continue;
#pragma unroll
            for (int t = 0; t < NDV; ++t) {
                if (32 * t + l32 >= Dv) continue;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int ii = 8 * (r >> 2) + 4 * hi + (r & 3);
                    if (ii < cnt) po[((int64_t)split * a.n_rows + row0 + ii) * (H * Dv) + h * Dv + 32 * t + l32] = acc[x][t][r];
                }
            }
        }
        return;
    }
    bf16_t *out = (bf16_t *)a.out;
    const bf16_t *gate = (const bf16_t *)a.gate;
#pragma unroll
    for (int x = 0; x < HPW; ++x) {
        const int h = wave * HPW + x;
        if (h >= H) continue;
#pragma unroll
        for (int t = 0; t < NDV; ++t) {
            if (32 * t + l32 >= Dv) continue;                       // a last column tile may be partly beyond Dv: computed, never stored
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ii = 8 * (r >> 2) + 4 * hi + (r & 3);
                if (ii >= cnt) continue;
                const int col = h * Dv + 32 * t + l32;
                float v = acc[x][t][r];
                if (gate) v *= 1.0f / (1.0f + __expf(-ld_f(gate + (int64_t)(row0 + ii) * a.gate_ld + (a.gate_heads ? h : col))));
                if (a.out_dtype == JL_OUT_F32) ((float *)a.out)[(int64_t)(row0 + ii) * (H * Dv) + col] = v;
                else st_f(out + (int64_t)(row0 + ii) * (H * Dv) + col, v);
            }
        }
    }
}

// Queries of every tile in the order the A operand wants them: q_pack[tile][head][step][lane] = the four depths 8 step + 4 (lane / 32) ..
// of row lane % 32 (zeros for rows a tile does not have).  Read straight from [N, H * D], a lane's 8 bytes lie a whole row apart.
__global__ __launch_bounds__(256) void attn_pack_q_kernel(const bf16_t *__restrict__ q, const int32_t *__restrict__ tiles, int H, int D,
                                                           uint2 *__restrict__ q_pack) {
    const int *tile = tiles + 4 * (int64_t)blockIdx.x;
    const int cnt = tile[2], row0 = tile[3];
    const int steps = D / 8, per_tile = H * steps * 64;
    for (int e = threadIdx.x; e < per_tile; e += 256) {
        const int lane = e & 63, st = (e >> 6) % steps, g = (e >> 6) / steps, l32 = lane & 31, hi = lane >> 5;
        uint2 v = make_uint2(0, 0);
        if (l32 < cnt) v = *(const uint2 *)(q + (int64_t)(row0 + l32) * (H * D) + g * D + 8 * st + 4 * hi);
        q_pack[(int64_t)blockIdx.x * per_tile + e] = v;
    }
}

// out = gate * the sum of the splits' shares, in split order
__global__ __launch_bounds__(256) void attn_join_kernel(const float *__restrict__ po, int S, int64_t total, int width,
                                                         const bf16_t *__restrict__ gate, int64_t gate_ld, int gate_every,
                                                         bf16_t *__restrict__ out, int out_f32) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    float v = 0.f;
    for (int sp = 0; sp < S; ++sp) v += po[(int64_t)sp * total + e];
    if (gate) {
        const int64_t row = e / width;
        v *= 1.0f / (1.0f + __expf(-ld_f(gate + row * gate_ld + (e - row * width) / gate_every)));      // gate_every = Dv: one gate per head
    }
    if (out_f32) ((float *)out)[e] = v;
    else st_f(out + e, v);
}

static bool am_fits(int dtype, int H, int G, int D, int Dv) {
    static const bool off = getenv("JL_ATTN_NO_MFMA") != nullptr;          // A/B switch for measurements
    return !off && dtype == JL_BF16 && H <= 16 && D % 8 == 0 && D <= 640 && Dv <= 128 && Dv % 4 == 0 &&
           am_lds_bytes(H, G, D, Dv) <= (size_t)ATT_LDS_BUDGET + 8 * 1024;
}

template <int HPW, int NDV> static int am_launch(const jl_attn_args &a, hipStream_t st) {
    auto kern = attn_mfma_kernel<HPW, NDV>;
    const size_t lds = am_lds_bytes(a.H, a.G, a.D, a.Dv);
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return jl_fail(JL_E_LAUNCH, "jl_attn_window: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    }
    const int waves = (a.H + HPW - 1) / HPW;
    attn_pack_q_kernel<<<dim3((unsigned)a.n_tiles), 256, 0, st>>>((const bf16_t *)a.q, a.tiles, a.H, a.D, (uint2 *)a.q_pack);
    if (a.splits <= 1) {
        kern<<<dim3((unsigned)a.n_tiles), 64 * waves, lds, st>>>(a, AM_FUSED);
        return jl_check_launch("attn_mfma_kernel");
    }
    const dim3 grid((unsigned)a.n_tiles, (unsigned)a.splits);
    kern<<<grid, 64 * waves, lds, st>>>(a, AM_STATS);
    kern<<<grid, 64 * waves, lds, st>>>(a, AM_PV);
    const int64_t total = (int64_t)a.n_rows * a.H * a.Dv;
    attn_join_kernel<<<dim3((unsigned)((total + 255) / 256)), 256, 0, st>>>(a.scratch + (int64_t)a.n_tiles * a.splits * a.H * AM_T * 2, a.splits, total,
                                                                          a.H * a.Dv, (const bf16_t *)a.gate, a.gate_ld, a.gate_heads ? a.Dv : 1, (bf16_t *)a.out,
                                                                          a.out_dtype == JL_OUT_F32);
    return jl_check_launch("attn_mfma_kernel (split keys)");
}

template <typename T, int ACC> static int att_launch(const jl_attn_args &a, const AttShape &s, hipStream_t st) {
    auto kern = attn_window_kernel<T, ACC>;
    if (s.lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)s.lds);
        if (e != hipSuccess) return jl_fail(JL_E_LAUNCH, "jl_attn_window: cannot get %zu bytes of LDS: %s", s.lds, hipGetErrorString(e));
    }
    kern<<<dim3((unsigned)a.n_tiles), ATT_THREADS, s.lds, st>>>(a, s.TK);
    return jl_check_launch("attn_window_kernel");
}

extern "C" int jl_attn_window(const jl_attn_args *ap, void *stream) {
    if (!ap) return jl_fail(JL_E_INVALID, "jl_attn_window: null arguments");
    jl_attn_args a = *ap;
    if (a.n_tiles <= 0) return JL_OK;
    if (!a.q || !a.k_cache || !a.v_cache || !a.out || !a.block_tables || !a.tiles) return jl_fail(JL_E_INVALID, "jl_attn_window: null pointer");
    if (a.H <= 0 || a.G <= 0 || a.H % a.G || a.D <= 0 || a.Dv <= 0 || a.page_size <= 0 || a.TQ <= 0)
        return jl_fail(JL_E_INVALID, "jl_attn_window: bad head counts or sizes");
    if ((a.lut && !a.rel) || (a.rel && a.lut_len <= 0)) return jl_fail(JL_E_INVALID, "jl_attn_window: a lut needs rel, and rel needs lut_len");
    if (a.Gv <= 0) a.Gv = a.G;
    if (a.k_ld <= 0) a.k_ld = (int64_t)a.G * a.D;
    if (a.v_ld <= 0) a.v_ld = (int64_t)a.Gv * a.Dv;
    if (a.G % a.Gv || a.k_ld < (int64_t)a.G * a.D || a.v_ld < (int64_t)a.Gv * a.Dv)
        return jl_fail(JL_E_INVALID, "jl_attn_window: value heads must divide the key heads, and row strides hold a row");
    if (a.out_dtype != JL_OUT_SAME && a.out_dtype != JL_OUT_F32) return jl_fail(JL_E_INVALID, "jl_attn_window: unknown out_dtype");
    if (a.dtype == JL_F32) a.out_dtype = JL_OUT_SAME;
    hipStream_t st = (hipStream_t)stream;
    if (a.splits > 1 && (!a.scratch || a.n_rows <= 0 || !(a.TQ == AM_T && am_fits(a.dtype, a.H, a.G, a.D, a.Dv) && am_strides_ok(a.k_ld, a.v_ld))))
        return jl_fail(JL_E_INVALID, "jl_attn_window: split keys need the matrix-core kernel, a scratch and the row count");
    if (a.TQ == AM_T && am_fits(a.dtype, a.H, a.G, a.D, a.Dv) && am_strides_ok(a.k_ld, a.v_ld)) {
        if (!a.q_pack) return jl_fail(JL_E_INVALID, "jl_attn_window: the matrix-core kernel needs q_pack (n_tiles * 32 * H * D elements)");
        const int ndv = (a.Dv + 31) / 32;
#define AM_CASE(HP, ND) if ((a.H > 8 ? 2 : 1) == HP && ndv == ND) return am_launch<HP, ND>(a, st)
        AM_CASE(1, 1); AM_CASE(1, 2); AM_CASE(1, 3); AM_CASE(1, 4);
        AM_CASE(2, 1); AM_CASE(2, 2); AM_CASE(2, 3); AM_CASE(2, 4);
#undef AM_CASE
    }
    AttShape s;
    if (!att_shape(a.H, a.G, a.D, a.Dv, a.TQ, &s) || s.TQ != a.TQ)
        return jl_fail(JL_E_INVALID, "jl_attn_window: TQ %d does not fit these sizes (ask jl_attn_tile_rows)", a.TQ);
#define ATT_CASE(N) case N: JL_DISPATCH(a.dtype, return (att_launch<T, N>(a, s, st))); break
    switch (s.ACC) {
        ATT_CASE(16);
        ATT_CASE(64);
    }
#undef ATT_CASE
    return jl_fail(JL_E_INVALID, "jl_attn_window: unsupported size");
}
