// jl_attn_sweep.hip — attention in ONE sweep over the keys (running maximum and sum) on the matrix cores (bfloat16), for heads that
// come in groups sharing a key head: grouped-query attention, several score maps over the same values, and the single key/value
// head of latent attention whose values are the first Dv columns of the key rows ([latent | rotary key]).  Sliding window or plain
// causal, an optional sink in the softmax's denominator and an optional sigmoid gate on the outputs; no bias or head mixing (those
// are jl_attn.hip's).
//
// A workgroup of four wavefronts owns up to 32 rows = (query, head) pairs of one request and one group — HF = min(heads per group,
// 32) heads of 32 / HF consecutive queries — so a key tile (32 keys through LDS) serves every head of the group at once.  Per tile:
//   1. the four wavefronts each form the 32 x 32 scores over a quarter of the key width (v_mfma_f32_32x32x8_bf16; the query
//      fragments stay in registers for the whole launch) and leave their partial sums in LDS;
//   2. 8 threads per row add the partial sums, mask, update the row's maximum and sum, and write exp(s - max) as bfloat16 and the
//      rescale factor of the row;
//   3. every wavefront multiplies the weights with ITS 32-column tiles of the values (tile wave, wave + 4, ..), which sit in LDS
//      beside the keys — or ARE the keys' first columns.
// Few tiles with many keys (decoding): the key tiles of a row tile are shared out over blockIdx.z; every share leaves its
// unnormalised outputs with its maximum and sum in a scratch, and attn_sweep_join_kernel combines them.
// Accumulator r of lane l of a 32 x 32 MFMA is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32; lane l supplies row (A) or
// column (B) l % 32 with depths 4 * (l / 32) .. + 3.
#include "jl_common.h"
#include <stdlib.h>

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short as_bf16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float as_f32x16;
constexpr int AS_T = 32, AS_WAVES = 4, AS_THREADS = 64 * AS_WAVES, AS_QSTEPS = 20;      // key width <= 8 * 4 * 20 = 640
constexpr int AS_PROW = 36;                                                            // weights' row stride in LDS (bfloat16)

__device__ __forceinline__ short as_bf16(float v) {
    uint32_t u = __float_as_uint(v);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (short)(u >> 16);
}

static size_t as_lds_bytes(int D, int Dv, bool v_in_k) {
    return (size_t)AS_T * (D + 4) * 2 + (v_in_k ? 0 : (size_t)AS_T * (Dv + 4) * 2) + (size_t)AS_WAVES * AS_T * 33 * 4 + (size_t)AS_T * AS_PROW * 2 + 2 * AS_T * 4;
}

template <int NT>                                                                       // value tiles (32 columns) per wavefront: Dv <= 128 * NT
__global__ __launch_bounds__(AS_THREADS) void attn_sweep_kernel(jl_attn_args a, int HF, int TQ, int HB, int v_in_k) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int H = a.H, D = a.D, Dv = a.Dv, KROW = D + 4, VROW = v_in_k ? KROW : Dv + 4, per_group = H / a.G;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, hi = lane >> 5;
    const int *tile = a.tiles + 4 * (int64_t)blockIdx.x;
    const int b = tile[0], i0 = tile[1], cnt = tile[2], row0 = tile[3];
    if (b < 0 || cnt <= 0) return;
    const int c = blockIdx.y / HB;                                  // the group = key head; its query heads are c * per_group ..
    const int h0 = c * per_group + (blockIdx.y - c * HB) * HF, h_end = (c + 1) * per_group;
    bf16_t *Ks = (bf16_t *)smem;                                    // [32][D + 4]
    bf16_t *Vs = v_in_k ? Ks : Ks + AS_T * KROW;                    // [32][Dv + 4], or the keys' own rows
    float *Sp = (float *)(Vs + (v_in_k ? AS_T * KROW : AS_T * VROW));   // [4][32][33] partial scores
    bf16_t *Pb = (bf16_t *)(Sp + AS_WAVES * AS_T * 33);             // [32][36] weights
    float *alphaS = (float *)(Pb + AS_T * AS_PROW);                 // [32] rescale factor of the tile
    float *lS = alphaS + AS_T;                                      // [32] final sums
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_max = i0 + cnt - 1;
    const int lo = i0 - window + 1 > 0 ? i0 - window + 1 : 0;
    const int n_keys = i_max + 1 - lo;
    const int *bt = a.block_tables + (int64_t)b * a.bt_stride;
    const bf16_t *kc = (const bf16_t *)a.k_cache + (int64_t)c * D;
    const bf16_t *vc = (const bf16_t *)a.v_cache + (int64_t)(c % a.Gv) * Dv;
    const int page_shift = (a.page_size & (a.page_size - 1)) == 0 ? __builtin_ctz(a.page_size) : -1;

    // this lane's query fragments: row l32 = (query l32 / HF, head h0 + l32 % HF), key-width steps wave, wave + 4, ..
    as_bf16x4 qf[AS_QSTEPS];
    {
        const int ii = l32 / HF, hh = h0 + l32 % HF;
        const bool ok = l32 < TQ * HF && ii < cnt && hh < h_end;
        const bf16_t *qp = (const bf16_t *)a.q + ((int64_t)(row0 + ii) * H + hh) * D + 4 * hi;
#pragma unroll
        for (int x = 0; x < AS_QSTEPS; ++x) {
            const int kk = 8 * (AS_WAVES * x + wave);
            qf[x] = (as_bf16x4){0, 0, 0, 0};
            if (ok && kk < D) qf[x] = *(const as_bf16x4 *)(qp + kk);
        }
    }
    // the row this thread helps to reduce: row tid / 8, keys 4 * (tid % 8) .. + 3
    const int rr = tid >> 3, rc = (tid & 7) * 4;
    const int r_i = i0 + rr / HF;
    const bool r_ok = rr < TQ * HF && rr / HF < cnt && h0 + rr % HF < h_end;
    float m_run = -INFINITY, l_run = 0.f;
    // a sink acts like one extra score that attends to nothing: the row's statistics start from (sink, 1), in the first share of the keys only
    if (a.sink && r_ok && blockIdx.z == 0) { m_run = a.sink[h0 + rr % HF]; l_run = 1.f; }

    as_f32x16 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

    const int units = D / 4;                                        // 8-byte units per key row
    const int jj0 = tid / units, u0r = tid - jj0 * units, dj = AS_THREADS / units, dr = AS_THREADS - dj * units;
    const int vunits = Dv / 4;
    const int vj0 = tid / vunits, v0r = tid - vj0 * vunits, vdj = AS_THREADS / vunits, vdr = AS_THREADS - vdj * vunits;

    const int S = a.splits > 1 ? a.splits : 1, split = blockIdx.z;
    const int per = ((n_keys + AS_T - 1) / AS_T + S - 1) / S;       // key tiles per share
    const int key_lo = split * per * AS_T, key_hi = (split + 1) * per * AS_T < n_keys ? (split + 1) * per * AS_T : n_keys;
    for (int u0 = key_lo; u0 < key_hi; u0 += AS_T) {
        const int nk = key_hi - u0 < AS_T ? key_hi - u0 : AS_T;
        __syncthreads();                                            // the previous tile's readers are done with Ks / Pb
        {
            int jj = jj0, r = u0r;
            for (int e = tid; e < AS_T * units; e += AS_THREADS) {
                uint2 v = make_uint2(0, 0);
                if (jj < nk) {
                    const int j = lo + u0 + jj;
                    const int pg = page_shift >= 0 ? j >> page_shift : j / a.page_size;
                    const int64_t tok = (int64_t)bt[pg] * a.page_size + (j - pg * a.page_size);
                    v = *(const uint2 *)(kc + tok * a.k_ld + 4 * r);
                }
                *(uint2 *)(Ks + jj * KROW + 4 * r) = v;
                jj += dj; r += dr;
                if (r >= units) { r -= units; ++jj; }
            }
        }
        if (!v_in_k) {
            int jj = vj0, r = v0r;
            for (int e = tid; e < AS_T * vunits; e += AS_THREADS) {
                uint2 v = make_uint2(0, 0);
                if (jj < nk) {
                    const int j = lo + u0 + jj;
                    const int pg = page_shift >= 0 ? j >> page_shift : j / a.page_size;
                    const int64_t tok = (int64_t)bt[pg] * a.page_size + (j - pg * a.page_size);
                    v = *(const uint2 *)(vc + tok * a.v_ld + 4 * r);
                }
                *(uint2 *)(Vs + jj * VROW + 4 * r) = v;
                jj += vdj; r += vdr;
                if (r >= vunits) { r -= vunits; ++jj; }
            }
        }
        __syncthreads();
        {   // 1. partial scores of this wavefront's share of the key width
            as_f32x16 sc;
#pragma unroll
            for (int r = 0; r < 16; ++r) sc[r] = 0.f;
            const bf16_t *kp = Ks + l32 * KROW + 4 * hi;
#pragma unroll
            for (int x = 0; x < AS_QSTEPS; ++x) {
                const int kk = 8 * (AS_WAVES * x + wave);
                if (kk < D) sc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(qf[x], *(const as_bf16x4 *)(kp + kk), sc, 0, 0, 0);
            }
            float *sp = Sp + wave * AS_T * 33;
#pragma unroll
            for (int r = 0; r < 16; ++r) sp[(8 * (r >> 2) + 4 * hi + (r & 3)) * 33 + l32] = sc[r];
        }
        __syncthreads();
        {   // 2. full scores of 4 keys of row rr, mask, running maximum and sum, weights
            float s[4];
            float mx = -INFINITY;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int jj = rc + x, j = lo + u0 + jj;
                float v = Sp[rr * 33 + jj] + Sp[(AS_T + rr) * 33 + jj] + Sp[(2 * AS_T + rr) * 33 + jj] + Sp[(3 * AS_T + rr) * 33 + jj];
                const bool ok = r_ok && jj < nk && j <= r_i && r_i - j < window;
                s[x] = ok ? v * a.scale : -INFINITY;
                mx = fmaxf(mx, s[x]);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
            const float m_new = fmaxf(m_run, mx);
            float alpha = 1.0f, sum = 0.f;
            short pw[4] = {0, 0, 0, 0};
            if (m_new > -INFINITY) {
                alpha = __expf(m_run - m_new);                      // m_run = -inf: 0, and nothing has been accumulated yet
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const float p = __expf(s[x] - m_new);           // masked: exp(-inf) = 0
                    pw[x] = as_bf16(p);
                    sum += p;
                }
            }
            sum += __shfl_xor(sum, 1, 64);
            sum += __shfl_xor(sum, 2, 64);
            sum += __shfl_xor(sum, 4, 64);
            l_run = l_run * alpha + sum;
            m_run = m_new;
            *(as_bf16x4 *)(Pb + rr * AS_PROW + rc) = (as_bf16x4){pw[0], pw[1], pw[2], pw[3]};
            if ((tid & 7) == 0) alphaS[rr] = alpha;
        }
        __syncthreads();
        {   // 3. rescale, then weights x this wavefront's value columns
            float al[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) al[r] = alphaS[8 * (r >> 2) + 4 * hi + (r & 3)];
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[t][r] *= al[r];
#pragma unroll
            for (int sK = 0; sK < AS_T / 8; ++sK) {
                const int j0 = 8 * sK + 4 * hi;
                const as_bf16x4 wa = *(const as_bf16x4 *)(Pb + l32 * AS_PROW + j0);
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const int col = 32 * (AS_WAVES * t + wave);
                    if (col >= Dv) continue;
                    const bf16_t *vp = Vs + j0 * VROW + col + l32;
                    const as_bf16x4 vb = {(short)vp[0], (short)vp[VROW], (short)vp[2 * VROW], (short)vp[3 * VROW]};
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(wa, vb, acc[t], 0, 0, 0);
                }
            }
        }
    }
    if (S > 1) {                                                    // this share's rows: [Dv] unnormalised outputs, maximum, sum
        float *part = a.scratch + (((int64_t)split * gridDim.x + blockIdx.x) * gridDim.y + blockIdx.y) * AS_T * (int64_t)(Dv + 2);
        if ((tid & 7) == 0) { part[rr * (Dv + 2) + Dv] = m_run; part[rr * (Dv + 2) + Dv + 1] = l_run; }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = 8 * (r >> 2) + 4 * hi + (r & 3);
#pragma unroll
            for (int t = 0; t < NT; ++t)
                if (32 * (AS_WAVES * t + wave) < Dv) part[row * (Dv + 2) + 32 * (AS_WAVES * t + wave) + l32] = acc[t][r];
        }
        return;
    }
    if ((tid & 7) == 0) lS[rr] = l_run > 0.f ? 1.0f / l_run : 0.f;
    __syncthreads();
    bf16_t *out = (bf16_t *)a.out;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * hi + (r & 3);
        const int ii = row / HF, hh = h0 + row % HF;
        if (row >= TQ * HF || ii >= cnt || hh >= h_end) continue;
        const float inv = lS[row];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int col = 32 * (AS_WAVES * t + wave) + l32;
            if (col - l32 >= Dv) continue;
            const int64_t o = ((int64_t)(row0 + ii) * H + hh) * Dv + col;
            float v = acc[t][r] * inv;
            if (a.gate) v *= 1.0f / (1.0f + __expf(-ld_f((const bf16_t *)a.gate + (int64_t)(row0 + ii) * a.gate_ld + (a.gate_heads ? hh : hh * Dv + col))));
            if (a.out_dtype == JL_OUT_F32) ((float *)a.out)[o] = v;
            else st_f(out + o, v);
        }
    }
}

// out[row] = sum_s part_s[row] * exp(m_s - M) / sum_s l_s * exp(m_s - M), in share order
__global__ __launch_bounds__(256) void attn_sweep_join_kernel(jl_attn_args a, int HF, int TQ, int HB) {
    __shared__ float wS[AS_T * 64];                                 // [32][S] weight of every share of a row
    const int H = a.H, Dv = a.Dv, S = a.splits, tid = threadIdx.x;
    const int *tile = a.tiles + 4 * (int64_t)blockIdx.x;
    const int cnt = tile[2], row0 = tile[3], per_group = H / a.G, c = blockIdx.y / HB;
    const int h0 = c * per_group + (blockIdx.y - c * HB) * HF, h_end = (c + 1) * per_group;
    if (tile[0] < 0 || cnt <= 0) return;
    const int64_t share = (int64_t)gridDim.x * gridDim.y * AS_T * (Dv + 2);
    const float *base = a.scratch + ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * AS_T * (int64_t)(Dv + 2);
    if (tid < AS_T) {
        float M = -INFINITY, L = 0.f;
        for (int sp = 0; sp < S; ++sp) M = fmaxf(M, base[sp * share + tid * (Dv + 2) + Dv]);
        for (int sp = 0; sp < S; ++sp) {
            const float m = base[sp * share + tid * (Dv + 2) + Dv];
            const float w = m > -INFINITY ? __expf(m - M) : 0.f;
            wS[tid * 64 + sp] = w;
            L += w * base[sp * share + tid * (Dv + 2) + Dv + 1];
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        for (int sp = 0; sp < S; ++sp) wS[tid * 64 + sp] *= inv;
    }
    __syncthreads();
    bf16_t *out = (bf16_t *)a.out;
    for (int e = tid; e < AS_T * Dv; e += 256) {
        const int row = e / Dv, col = e - row * Dv, ii = row / HF, hh = h0 + row % HF;
        if (row >= TQ * HF || ii >= cnt || hh >= h_end) continue;
        float v = 0.f;
        for (int sp = 0; sp < S; ++sp) v += wS[row * 64 + sp] * base[sp * share + row * (Dv + 2) + col];
        const int64_t o = ((int64_t)(row0 + ii) * H + hh) * Dv + col;
        if (a.gate) v *= 1.0f / (1.0f + __expf(-ld_f((const bf16_t *)a.gate + (int64_t)(row0 + ii) * a.gate_ld + (a.gate_heads ? hh : hh * Dv + col))));
        if (a.out_dtype == JL_OUT_F32) ((float *)a.out)[o] = v;
        else st_f(out + o, v);
    }
}


// ---- the same sweep for tiles of up to 128 rows: every wavefront keeps ITS 32 rows to itself ----------------------------------------
// Long portions (prefill) fill 128 (query, head) rows per workgroup; then no partial sums or weights have to meet in LDS.  Per 32-key
// tile (keys and values through LDS, shared by the four wavefronts) a wavefront forms the TRANSPOSED scores S^T = K Q^T (A = the key
// rows from LDS, B = its query fragments from registers), so that a lane holds 16 keys of ONE row (query l32; the other 16 in lane
// l32 + 32): maximum, sum and rescale factor are per-lane numbers plus one exchange with the other half-wavefront.  Accumulator
// registers 4g .. 4g + 3 of S^T are keys 8g + 4 (l / 32) .. + 3 — exactly the four depths lane l supplies as the B operand of MFMA
// step g — so the weights go from the accumulators straight into O^T = V^T P^T (A = four keys of value column l32 from LDS).  In
// O^T a lane again holds one row's values: the rescale is one multiply per register, and four consecutive value columns of a row
// leave as one 8-byte store.  A wavefront skips the key tiles none of its rows can see.
constexpr int AR_ROWS = 128;

// four floats -> four bfloat16 (round to nearest even) through the compiler's own conversion: one packed instruction per pair
typedef __bf16 ar_bf16x4 __attribute__((ext_vector_type(4)));
typedef float ar_f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ as_bf16x4 ar_round4(float a, float b, float c, float d) {
    const ar_f32x4 f = {a, b, c, d};
    const ar_bf16x4 h = __builtin_convertvector(f, ar_bf16x4);
    return __builtin_bit_cast(as_bf16x4, h);
}

constexpr int AR_PAGES = 1024;     // page-table entries of a tile's key range kept in LDS (longer ranges are read from memory)
static size_t ar_lds_bytes(int D, int Dv, bool v_in_k) {          // two buffers of a key tile and a value tile, the page table
    return 2 * ((size_t)AS_T * (D + 4) * 2 + (v_in_k ? 0 : (size_t)AS_T * (Dv + 8) * 2)) + AR_PAGES * 4;
}

template <int QS, int NDV>                                                              // D <= 8 * QS, Dv <= 32 * NDV <= 128
__global__ __launch_bounds__(AS_THREADS, 2) void attn_rows_kernel(jl_attn_args a, int HF, int TQ, int HB, int v_in_k) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int H = a.H, D = a.D, Dv = a.Dv, KROW = D + 4, VROW = v_in_k ? KROW : Dv + 8, per_group = H / a.G;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l32 = lane & 31, hi = lane >> 5;
    const int *tile = a.tiles + 4 * (int64_t)blockIdx.x;
    const int b = tile[0], i0 = tile[1], cnt = tile[2], row0 = tile[3];
    if (b < 0 || cnt <= 0) return;
    const int c = blockIdx.y / HB;
    const int h0 = c * per_group + (blockIdx.y - c * HB) * HF, h_end = (c + 1) * per_group;
    const int buf_elems = AS_T * KROW + (v_in_k ? 0 : AS_T * VROW);  // one buffer: [32][D + 4] keys, then [32][Dv + 8] values (or the keys' own rows)
    bf16_t *buf0 = (bf16_t *)smem;
    int *pageS = (int *)(buf0 + 2 * buf_elems);
    const int window = a.window > 0 ? a.window : 0x3fffffff;
    const int i_max = i0 + cnt - 1;
    const int lo = i0 - window + 1 > 0 ? i0 - window + 1 : 0;
    const int n_keys = i_max + 1 - lo;
    const int *bt = a.block_tables + (int64_t)b * a.bt_stride;
    const bf16_t *kc = (const bf16_t *)a.k_cache + (int64_t)c * D;
    const bf16_t *vc = (const bf16_t *)a.v_cache + (int64_t)(c % a.Gv) * Dv;
    const int page_shift = (a.page_size & (a.page_size - 1)) == 0 ? __builtin_ctz(a.page_size) : -1;
    // the pages of the tile's key range: one trip to memory instead of one in front of every tile's loads
    const int pg_lo = lo / a.page_size, n_pages = i_max / a.page_size - pg_lo + 1;
    if (n_pages <= AR_PAGES) {
        for (int e = tid; e < n_pages; e += AS_THREADS) pageS[e] = bt[pg_lo + e];
        __syncthreads();
        bt = pageS - pg_lo;
    }

    // this lane's row: (query R / HF, head h0 + R % HF), R = 32 * wave + l32; both half-wavefronts hold it
    const int R = 32 * wave + l32, ii = R / HF, hh = h0 + R % HF;
    const bool ok = R < TQ * HF && ii < cnt && hh < h_end;
    const int qi = i0 + ii;
    as_bf16x4 qf[QS];
    {
        const bf16_t *qp = (const bf16_t *)a.q + ((int64_t)(row0 + ii) * H + hh) * D + 4 * hi;
#pragma unroll
        for (int x = 0; x < QS; ++x) {
            qf[x] = (as_bf16x4){0, 0, 0, 0};
            if (ok && 8 * x < D) qf[x] = *(const as_bf16x4 *)(qp + 8 * x);
        }
    }
    float m_run = -INFINITY, l_run = 0.f;
    if (a.sink && ok) { m_run = a.sink[hh]; l_run = 1.f; }           // the sink: an extra score that attends to nothing
    as_f32x16 acc[NDV];
#pragma unroll
    for (int t = 0; t < NDV; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
    // the queries this wavefront's rows belong to (none: it only helps to load)
    const int wq_first = (32 * wave) / HF, wq_last = (32 * wave + 31) / HF < cnt - 1 ? (32 * wave + 31) / HF : cnt - 1;
    const bool wave_live = 32 * wave < TQ * HF && wq_first < cnt;
    const bool wave_full = 32 * wave + 31 < TQ * HF && (32 * wave + 31) / HF < cnt && h0 + HF <= h_end;     // all 32 rows are rows of the tile

    const int units = D / 4;                                        // 8-byte units per key row
    const int jj0 = tid / units, u0r = tid - jj0 * units, dj = AS_THREADS / units, dr = AS_THREADS - dj * units;
    const int vunits = Dv / 4;
    const int vj0 = tid / vunits, v0r = tid - vj0 * vunits, vdj = AS_THREADS / vunits, vdr = AS_THREADS - vdj * vunits;

    // a tile's rows travel from memory while the previous tile is multiplied: fetched into registers one iteration ahead (a thread's
    // share of a tile is D / 32 key units and Dv / 32 value units of 8 bytes), written to LDS once the previous tile's readers are done
    constexpr int KPF = QS / 4, VPF = NDV;
    uint2 kreg[KPF], vreg[VPF];
    auto fetch = [&](int u0) {
        const int nk = n_keys - u0 < AS_T ? n_keys - u0 : AS_T;
        int jj = jj0, r = u0r;
#pragma unroll
        for (int it = 0; it < KPF; ++it) {
            kreg[it] = make_uint2(0, 0);
            if (tid + it * AS_THREADS < AS_T * units) {
                if (jj < nk) {
                    const int j = lo + u0 + jj;
                    const int pg = page_shift >= 0 ? j >> page_shift : j / a.page_size;
                    const int64_t tok = (int64_t)bt[pg] * a.page_size + (j - pg * a.page_size);
                    kreg[it] = *(const uint2 *)(kc + tok * a.k_ld + 4 * r);
                }
                jj += dj; r += dr;
                if (r >= units) { r -= units; ++jj; }
            }
        }
        if (v_in_k) return;
        jj = vj0; r = v0r;
#pragma unroll
        for (int it = 0; it < VPF; ++it) {
            vreg[it] = make_uint2(0, 0);
            if (tid + it * AS_THREADS < AS_T * vunits) {
                if (jj < nk) {
                    const int j = lo + u0 + jj;
                    const int pg = page_shift >= 0 ? j >> page_shift : j / a.page_size;
                    const int64_t tok = (int64_t)bt[pg] * a.page_size + (j - pg * a.page_size);
                    vreg[it] = *(const uint2 *)(vc + tok * a.v_ld + 4 * r);
                }
                jj += vdj; r += vdr;
                if (r >= vunits) { r -= vunits; ++jj; }
            }
        }
    };
    auto stash = [&](bf16_t *Ks) {
        bf16_t *Vs = Ks + AS_T * KROW;
        int jj = jj0, r = u0r;
#pragma unroll
        for (int it = 0; it < KPF; ++it)
            if (tid + it * AS_THREADS < AS_T * units) {
                *(uint2 *)(Ks + jj * KROW + 4 * r) = kreg[it];
                jj += dj; r += dr;
                if (r >= units) { r -= units; ++jj; }
            }
        if (v_in_k) return;
        jj = vj0; r = v0r;
#pragma unroll
        for (int it = 0; it < VPF; ++it)
            if (tid + it * AS_THREADS < AS_T * vunits) {
                *(uint2 *)(Vs + jj * VROW + 4 * r) = vreg[it];
                jj += vdj; r += vdr;
                if (r >= vunits) { r -= vunits; ++jj; }
            }
    };
    // tile t is multiplied out of buffer t % 2 while tile t + 1 goes from registers into the other buffer and tile t + 2 leaves memory:
    // one barrier per tile (a buffer is written again only after the barrier that follows its last reader)
    fetch(0);
    stash(buf0);
    if (AS_T < n_keys) fetch(AS_T);
    __syncthreads();
    for (int u0 = 0, tsel = 0; u0 < n_keys; u0 += AS_T, tsel ^= 1) {
        const int nk = n_keys - u0 < AS_T ? n_keys - u0 : AS_T;
        if (u0 > 0) {
            if (u0 + AS_T < n_keys) fetch(u0 + AS_T);
        }
        const bf16_t *Ks = buf0 + tsel * buf_elems, *Vs = v_in_k ? Ks : Ks + AS_T * KROW;
        const int j0 = lo + u0;                                     // position of the tile's first key
        // wavefront-uniform: keys all behind its last query, or all before its first query's window
        if (wave_live && j0 <= i0 + wq_last && j0 + nk - 1 >= i0 + wq_first - window + 1) {
        as_f32x16 sc;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = 0.f;
        {
            const bf16_t *kp = Ks + l32 * KROW + 4 * hi;
#pragma unroll
            for (int x = 0; x < QS; ++x)
                if (8 * x < D) sc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(*(const as_bf16x4 *)(kp + 8 * x), qf[x], sc, 0, 0, 0);
        }
        float mx = -INFINITY;
        // wavefront-uniform: a full tile whose keys every row of the wavefront sees needs no mask
        const bool inside = nk == AS_T && wave_full && j0 + AS_T - 1 <= i0 + wq_first && i0 + wq_last - j0 < window;
        if (inside) {
#pragma unroll
            for (int r = 0; r < 16; ++r) { sc[r] *= a.scale; mx = fmaxf(mx, sc[r]); }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int kk = 8 * (r >> 2) + 4 * hi + (r & 3), j = j0 + kk;
                const bool vis = ok && kk < nk && j <= qi && qi - j < window;
                sc[r] = vis ? sc[r] * a.scale : -INFINITY;
                mx = fmaxf(mx, sc[r]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        float alpha = 1.0f, sum = 0.f;
        if (m_new > -INFINITY) {
            alpha = __expf(m_run - m_new);                          // m_run = -inf: 0, and nothing has been accumulated yet
#pragma unroll
            for (int r = 0; r < 16; ++r) { sc[r] = __expf(sc[r] - m_new); sum += sc[r]; }      // masked: exp(-inf) = 0
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) sc[r] = 0.f;
        }
        sum += __shfl_xor(sum, 32, 64);
        l_run = l_run * alpha + sum;
        m_run = m_new;
        if (__any(alpha != 1.0f)) {                                 // after the first tiles a row's maximum seldom moves
#pragma unroll
            for (int t = 0; t < NDV; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[t][r] *= alpha;
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const as_bf16x4 pb = ar_round4(sc[4 * g], sc[4 * g + 1], sc[4 * g + 2], sc[4 * g + 3]);
            const bf16_t *vp = Vs + (8 * g + 4 * hi) * VROW + l32;
#pragma unroll
            for (int t = 0; t < NDV; ++t) {
                if (32 * t >= Dv) continue;
                const as_bf16x4 va = {(short)vp[32 * t], (short)vp[32 * t + VROW], (short)vp[32 * t + 2 * VROW], (short)vp[32 * t + 3 * VROW]};
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(va, pb, acc[t], 0, 0, 0);
            }
        }
        }
        if (u0 + AS_T < n_keys) stash(buf0 + (tsel ^ 1) * buf_elems);
        __syncthreads();
    }
    if (!ok) return;
    const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
    const bf16_t *gate = (const bf16_t *)a.gate;
    float gh = 1.0f;
    if (gate && a.gate_heads) gh = 1.0f / (1.0f + __expf(-ld_f(gate + (int64_t)(row0 + ii) * a.gate_ld + hh)));
    const int64_t obase = ((int64_t)(row0 + ii) * H + hh) * Dv;
#pragma unroll
    for (int t = 0; t < NDV; ++t) {
        if (32 * t >= Dv) continue;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int col = 32 * t + 8 * g + 4 * hi;                // registers 4g .. 4g + 3: four consecutive value columns
            float v[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                v[x] = acc[t][4 * g + x] * inv * gh;
                if (gate && !a.gate_heads) v[x] *= 1.0f / (1.0f + __expf(-ld_f(gate + (int64_t)(row0 + ii) * a.gate_ld + hh * Dv + col + x)));
            }
            if (a.out_dtype == JL_OUT_F32) {
                *(float4 *)((float *)a.out + obase + col) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
                bf16_t hv[4];
#pragma unroll
                for (int x = 0; x < 4; ++x) st_f(hv + x, v[x]);
                *(uint2 *)((bf16_t *)a.out + obase + col) = make_uint2((uint32_t)hv[0] | ((uint32_t)hv[1] << 16), (uint32_t)hv[2] | ((uint32_t)hv[3] << 16));
            }
        }
    }
}

static int as_heads_per_tile(int H, int G) { const int per = H / G; return per < AS_T ? per : AS_T; }
static int as_head_blocks(int H, int G) { const int per = H / G, hf = as_heads_per_tile(H, G); return (per + hf - 1) / hf; }

extern "C" int64_t jl_attn_sweep_scratch_floats(int32_t n_tiles, int32_t H, int32_t G, int32_t Dv, int32_t splits) {
    if (H <= 0 || G <= 0 || H % G) return 0;
    return splits > 1 ? (int64_t)splits * n_tiles * G * as_head_blocks(H, G) * AS_T * (Dv + 2) : 0;
}

static bool as_fits(int dtype, int H, int G, int Gv, int D, int Dv, int64_t k_ld, int64_t v_ld, bool v_in_k) {
    if (!(dtype == JL_BF16 && H >= 1 && G >= 1 && H % G == 0 && Gv >= 1 && G % Gv == 0 && D % 8 == 0 && D <= 8 * AS_WAVES * AS_QSTEPS && Dv % 32 == 0 &&
          Dv >= 32 && Dv <= 512 && k_ld % 4 == 0 && v_ld % 4 == 0 && k_ld >= (int64_t)G * D))
        return false;
    if (v_in_k) return G == 1 && Dv <= D;
    return v_ld >= (int64_t)Gv * Dv && as_lds_bytes(D, Dv, false) <= 150 * 1024;
}

extern "C" int jl_attn_sweep_tile_rows(int dtype, int32_t H, int32_t G, int32_t Gv, int32_t D, int32_t Dv, int64_t k_ld, int64_t v_ld, int32_t v_in_k) {
    if (!as_fits(dtype, H, G, Gv > 0 ? Gv : G, D, Dv, k_ld, v_in_k ? k_ld : v_ld, v_in_k != 0)) return 0;
    return AS_T / as_heads_per_tile(H, G);
}

// the 128-row form takes key widths up to 256 and value widths up to 128 (its query fragments and outputs live in registers)
static bool ar_fits(int dtype, int H, int G, int Gv, int D, int Dv, int64_t k_ld, int64_t v_ld, bool v_in_k) {
    static const bool off = getenv("JL_ATTN_NO_WIDE") != nullptr;          // A/B switch for measurements
    return !off && as_fits(dtype, H, G, Gv, D, Dv, k_ld, v_ld, v_in_k) && D <= 256 && Dv <= 128;
}

extern "C" int jl_attn_sweep_wide_tile_rows(int dtype, int32_t H, int32_t G, int32_t Gv, int32_t D, int32_t Dv, int64_t k_ld, int64_t v_ld, int32_t v_in_k) {
    if (!ar_fits(dtype, H, G, Gv > 0 ? Gv : G, D, Dv, k_ld, v_in_k ? k_ld : v_ld, v_in_k != 0)) return 0;
    return AR_ROWS / as_heads_per_tile(H, G);
}

template <int QS, int NDV> static int ar_launch(const jl_attn_args &a, int hf, int tq, int hb, bool v_in_k, hipStream_t st) {
    const dim3 grid((unsigned)a.n_tiles, (unsigned)(a.G * hb));
    attn_rows_kernel<QS, NDV><<<grid, AS_THREADS, ar_lds_bytes(a.D, a.Dv, v_in_k), st>>>(a, hf, tq, hb, v_in_k ? 1 : 0);
    return jl_check_launch("attn_rows_kernel");
}

extern "C" int jl_attn_sweep(const jl_attn_args *ap, void *stream) {
    if (!ap) return jl_fail(JL_E_INVALID, "jl_attn_sweep: null arguments");
    jl_attn_args a = *ap;
    if (a.n_tiles <= 0) return JL_OK;
    if (!a.q || !a.k_cache || !a.v_cache || !a.out || !a.block_tables || !a.tiles) return jl_fail(JL_E_INVALID, "jl_attn_sweep: null pointer");
    if (a.H <= 0 || a.G <= 0 || a.H % a.G || a.page_size <= 0) return jl_fail(JL_E_INVALID, "jl_attn_sweep: bad head counts or page size");
    if (a.Gv <= 0) a.Gv = a.G;
    if (a.k_ld <= 0) a.k_ld = (int64_t)a.G * a.D;
    const bool v_in_k = a.v_cache == a.k_cache;
    if (a.v_ld <= 0) a.v_ld = v_in_k ? a.k_ld : (int64_t)a.Gv * a.Dv;
    if (!as_fits(a.dtype, a.H, a.G, a.Gv, a.D, a.Dv, a.k_ld, a.v_ld, v_in_k))
        return jl_fail(JL_E_INVALID, "jl_attn_sweep: bfloat16, key width a multiple of 8 up to %d, value width a multiple of 32 up to 512, row strides in "
                       "multiples of 4; values inside the key rows need one key head", 8 * AS_WAVES * AS_QSTEPS);
    if (a.out_dtype != JL_OUT_SAME && a.out_dtype != JL_OUT_F32) return jl_fail(JL_E_INVALID, "jl_attn_sweep: unknown out_dtype");
    const int hf = as_heads_per_tile(a.H, a.G), hb = as_head_blocks(a.H, a.G), tq = AS_T / hf;
    if (a.TQ == AR_ROWS / hf && a.TQ != tq) {                       // tiles of up to 128 rows: every wavefront keeps its rows to itself
        if (a.splits > 1 || !ar_fits(a.dtype, a.H, a.G, a.Gv, a.D, a.Dv, a.k_ld, a.v_ld, v_in_k))
            return jl_fail(JL_E_INVALID, "jl_attn_sweep: 128-row tiles take key widths up to 256, value widths up to 128 and no shared-out keys");
        hipStream_t st = (hipStream_t)stream;
        const int qs = a.D <= 64 ? 8 : (a.D <= 128 ? 16 : 32), ndv = a.Dv <= 32 ? 1 : (a.Dv <= 64 ? 2 : 4);
#define AR_CASE(Q, N) if (qs == Q && ndv == N) return ar_launch<Q, N>(a, hf, a.TQ, hb, v_in_k, st)
        AR_CASE(8, 1); AR_CASE(8, 2); AR_CASE(8, 4);
        AR_CASE(16, 1); AR_CASE(16, 2); AR_CASE(16, 4);
        AR_CASE(32, 1); AR_CASE(32, 2); AR_CASE(32, 4);
#undef AR_CASE
    }
    if (a.TQ != tq) return jl_fail(JL_E_INVALID, "jl_attn_sweep: tiles of %d queries wanted (ask jl_attn_sweep_tile_rows)", tq);
    if (a.splits > 1 && (!a.scratch || a.splits > 64)) return jl_fail(JL_E_INVALID, "jl_attn_sweep: 2 .. 64 shares of the keys need a scratch");
    const size_t lds = as_lds_bytes(a.D, a.Dv, v_in_k);
    const dim3 grid((unsigned)a.n_tiles, (unsigned)(a.G * hb), (unsigned)(a.splits > 1 ? a.splits : 1));
    hipStream_t st = (hipStream_t)stream;
#define AS_CASE(NTV)                                                                                                              \
    case NTV: {                                                                                                                   \
        auto kern = attn_sweep_kernel<NTV>;                                                                                       \
        if (lds > 64 * 1024) {                                                                                                    \
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);         \
            if (e != hipSuccess) return jl_fail(JL_E_LAUNCH, "jl_attn_sweep: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e)); \
        }                                                                                                                         \
        kern<<<grid, AS_THREADS, lds, st>>>(a, hf, tq, hb, v_in_k ? 1 : 0);                                                       \
        break;                                                                                                                    \
    }
    switch ((a.Dv + 127) / 128) {
        AS_CASE(1) AS_CASE(2) AS_CASE(3) AS_CASE(4)
    }
#undef AS_CASE
    if (a.splits > 1) attn_sweep_join_kernel<<<dim3(grid.x, grid.y), 256, 0, st>>>(a, hf, tq, hb);
    return jl_check_launch("attn_sweep_kernel");
}
