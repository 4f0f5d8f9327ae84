// gl3_hy_plain_kernels.h — kernels of layer-list designs with ONE plain residual stream (gl3_model_desc.streams == 0): the residual
// update with everything that can ride on it (sum of K-split parts, gated shared expert, routed experts' rows, unit-RMS side input,
// weighted average over earlier layers' results, the next sublayer's norm), the per-layer token input's activation, and the mixture of
// experts' router, grouping and input scaling.  Every mechanism takes its sizes and constants as arguments.
#pragma once
#include "gl3_hy_kernels.h"

// ---- residual update ----------------------------------------------------------------------------------------------------------------
// One workgroup per token.  In this order, every part optional (null pointer = absent):
//   d  = ya_mul * ga * sum_z ya[z]              ya: a sublayer's output (or several sublayers' outputs), possibly as K-split parts; ga = sigmoid(gate_z[t * gate_ld]) or 1
//   d += sum_k ew[t top + k] eo[pair_row[t top + k]]   the routed experts' down projections of this token (ew: a weight per pair, null = 1)
//   x += d, or with post_w: x += d / sqrt(mean(d^2) + eps) * post_w    (the sublayer's output passes a norm of its own before it joins the residual)
//   x += yc / sqrt(mean(yc^2) + eps) * cw       a unit-RMS normed input with a plain weight
//   hist_out[t] = x;  x = sum_j mix[j] hist[j][t], j < n_mix, where hist[n_mix - 1] is hist_out (what the layer leaves is an average over
//                                               the embedding output and every layer's result so far)
//   x is written back; xt = x in the matrix type (operand of a following product); tap = x
//   h = x / sqrt(mean(x^2) + eps) * norm_w in the matrix type (the next sublayer's input; norm_w already holds any offset)
struct HyResid {
    float* x; int W;
    const float* ya; int ya_parts; size_t ya_stride; const float* gate_z; int gate_ld; float ya_mul;
    const float* eo; const int* pair_row; int top; const float* ew;
    const float* post_w;
    const float* yc; const float* cw;
    float* hist; size_t hist_stride; int n_mix; const float* mix;      // hist_out = hist + (n_mix - 1) hist_stride
    float* tap;
    const float* norm_w; float eps;
};
// V = 4: rows are read and written 16 bytes at a time (W a multiple of 4); every load of a chunk is issued before the first use, so one
// round trip to memory covers them all.  The first HY_RC chunks of a thread stay in registers for the norm's second pass.
template <int V> __device__ __forceinline__ void hy_ldv(const float* __restrict__ p, float* v) {
    if constexpr (V == 4) { const float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
    else v[0] = *p;
}
template <int V> __device__ __forceinline__ void hy_stv(float* __restrict__ p, const float* v) {
    if constexpr (V == 4) *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    else *p = v[0];
}
template <int V> __device__ __forceinline__ void hy_stv(bf16_t* __restrict__ p, const float* v) {
    if constexpr (V == 4) {
        uint2 t;
        t.x = (uint32_t)hy_f2bf(v[0]) | ((uint32_t)hy_f2bf(v[1]) << 16);
        t.y = (uint32_t)hy_f2bf(v[2]) | ((uint32_t)hy_f2bf(v[3]) << 16);
        *reinterpret_cast<uint2*>(p) = t;
    } else *p = hy_f2bf(v[0]);
}
constexpr int HY_RC = 2, HY_MAX_PARTS = 4, HY_MIX_UNROLL = 4;
template <typename TO, int NT, int V>
static __global__ __launch_bounds__(NT) void hy_resid_kernel(HyResid a, TO* __restrict__ xt, TO* __restrict__ h_out) {
    __shared__ float red[NT / 64];
    const int t = blockIdx.x, W = a.W;
    const size_t row = (size_t)t * W;
    float cr = 0.f;
    if (a.yc) {
        float ss = 0.f;
        for (int w = threadIdx.x * V; w < W; w += NT * V) {
            float v[V];
            hy_ldv<V>(a.yc + row + w, v);
#pragma unroll
            for (int i = 0; i < V; ++i) ss += v[i] * v[i];
        }
        ss = hy_block_sum<NT>(ss, red);
        cr = 1.f / sqrtf(ss / (float)W + a.eps);
    }
    const float ga = (a.gate_z ? hy_sigmoid(a.gate_z[(size_t)t * a.gate_ld]) : 1.f) * a.ya_mul;
    float pr = 0.f;          // post_w: 1 / rms of the sublayer's whole output (the same sums as below, once more)
    if (a.post_w) {
        float sd = 0.f;
        for (int w = threadIdx.x * V; w < W; w += NT * V) {
            float y[V], e[V];
#pragma unroll
            for (int i = 0; i < V; ++i) y[i] = e[i] = 0.f;
            if (a.ya)
                for (int z = 0; z < a.ya_parts; ++z) {
                    float q[V];
                    hy_ldv<V>(a.ya + z * a.ya_stride + row + w, q);
#pragma unroll
                    for (int i = 0; i < V; ++i) y[i] += q[i];
                }
            if (a.eo)
                for (int k = 0; k < a.top; ++k) {
                    float q[V];
                    hy_ldv<V>(a.eo + (size_t)a.pair_row[t * a.top + k] * W + w, q);
                    const float wk = a.ew ? a.ew[t * a.top + k] : 1.f;
#pragma unroll
                    for (int i = 0; i < V; ++i) e[i] = fmaf(wk, q[i], e[i]);
                }
#pragma unroll
            for (int i = 0; i < V; ++i) { const float d = ga * y[i] + e[i]; sd += d * d; }
        }
        sd = hy_block_sum<NT>(sd, red);
        pr = 1.f / sqrtf(sd / (float)W + a.eps);
    }
    float ss = 0.f, keep[HY_RC][V];
    int it = 0;
    for (int w = threadIdx.x * V; w < W; w += NT * V, ++it) {
        float x[V], y[V], e[V], c[V], cw[V];
        hy_ldv<V>(a.x + row + w, x);
#pragma unroll
        for (int i = 0; i < V; ++i) y[i] = e[i] = c[i] = 0.f;
        if (a.ya) {
            float p[HY_MAX_PARTS][V];
#pragma unroll
            for (int z = 0; z < HY_MAX_PARTS; ++z)
                if (z < a.ya_parts) hy_ldv<V>(a.ya + z * a.ya_stride + row + w, p[z]);
#pragma unroll
            for (int z = 0; z < HY_MAX_PARTS; ++z)
                if (z < a.ya_parts)
#pragma unroll
                    for (int i = 0; i < V; ++i) y[i] += p[z][i];
            for (int z = HY_MAX_PARTS; z < a.ya_parts; ++z) {
                float q[V];
                hy_ldv<V>(a.ya + z * a.ya_stride + row + w, q);
#pragma unroll
                for (int i = 0; i < V; ++i) y[i] += q[i];
            }
        }
        if (a.eo)
            for (int k = 0; k < a.top; ++k) {
                float q[V];
                hy_ldv<V>(a.eo + (size_t)a.pair_row[t * a.top + k] * W + w, q);
                const float wk = a.ew ? a.ew[t * a.top + k] : 1.f;
#pragma unroll
                for (int i = 0; i < V; ++i) e[i] = fmaf(wk, q[i], e[i]);
            }
        if (a.yc) { hy_ldv<V>(a.yc + row + w, c); hy_ldv<V>(a.cw + w, cw); }
        if (a.post_w) {
            float pw[V];
            hy_ldv<V>(a.post_w + w, pw);
#pragma unroll
            for (int i = 0; i < V; ++i) x[i] += (ga * y[i] + e[i]) * pr * pw[i];
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                x[i] += ga * y[i];
                x[i] += e[i];
            }
        }
#pragma unroll
        for (int i = 0; i < V; ++i)
            if (a.yc) x[i] += c[i] * cr * cw[i];
        if (a.hist) {
            hy_stv<V>(a.hist + (size_t)(a.n_mix - 1) * a.hist_stride + row + w, x);
            float m[V];
#pragma unroll
            for (int i = 0; i < V; ++i) m[i] = a.mix[a.n_mix - 1] * x[i];
            int j = 0;
            for (; j + HY_MIX_UNROLL <= a.n_mix - 1; j += HY_MIX_UNROLL) {          // earlier results, a few loads in flight at a time
                float q[HY_MIX_UNROLL][V];
#pragma unroll
                for (int u = 0; u < HY_MIX_UNROLL; ++u) hy_ldv<V>(a.hist + (size_t)(j + u) * a.hist_stride + row + w, q[u]);
#pragma unroll
                for (int u = 0; u < HY_MIX_UNROLL; ++u)
#pragma unroll
                    for (int i = 0; i < V; ++i) m[i] = fmaf(a.mix[j + u], q[u][i], m[i]);
            }
            for (; j < a.n_mix - 1; ++j) {
                float q[V];
                hy_ldv<V>(a.hist + (size_t)j * a.hist_stride + row + w, q);
#pragma unroll
                for (int i = 0; i < V; ++i) m[i] = fmaf(a.mix[j], q[i], m[i]);
            }
#pragma unroll
            for (int i = 0; i < V; ++i) x[i] = m[i];
        }
        hy_stv<V>(a.x + row + w, x);
        if (xt) hy_stv<V>(xt + row + w, x);
        if (a.tap) hy_stv<V>(a.tap + row + w, x);
#pragma unroll
        for (int i = 0; i < V; ++i) ss += x[i] * x[i];
#pragma unroll
        for (int q = 0; q < HY_RC; ++q)
            if (q == it)
#pragma unroll
                for (int i = 0; i < V; ++i) keep[q][i] = x[i];
    }
    if (!a.norm_w) return;
    ss = hy_block_sum<NT>(ss, red);
    const float r = 1.f / sqrtf(ss / (float)W + a.eps);
    it = 0;
    for (int w = threadIdx.x * V; w < W; w += NT * V, ++it) {
        float x[V], nw[V];
        if (it < HY_RC) {
#pragma unroll
            for (int q = 0; q < HY_RC; ++q)
                if (q == it)
#pragma unroll
                    for (int i = 0; i < V; ++i) x[i] = keep[q][i];
        } else hy_ldv<V>(a.x + row + w, x);          // a thread re-reads what it wrote
        hy_ldv<V>(a.norm_w + w, nw);
#pragma unroll
        for (int i = 0; i < V; ++i) x[i] = x[i] * r * nw[i];
        hy_stv<V>(h_out + row + w, x);
    }
}

// ---- per-layer token input, portions of many tokens: g[t][d] = gelu_tanh(z[t][d]) * table[token t][col0 + d] as the projection's operand
// (row stride ldg); z arrives as `parts` K-split partial products, pstride apart ----
template <typename T>
static __global__ __launch_bounds__(256) void hy_side_act_kernel(const float* __restrict__ z, int D, int parts, size_t pstride, const int* __restrict__ tokens,
                                                                 const T* __restrict__ table, int table_ld, int col0, T* __restrict__ g, int ldg) {
    const int t = blockIdx.x;
    const T* e = table + (size_t)tokens[t] * table_ld + col0;
    for (int d = threadIdx.x; d < D; d += 256) {
        float v = 0.f;
        for (int p = 0; p < parts; ++p) v += z[p * pstride + (size_t)t * D + d];
        hy_st(g + (size_t)t * ldg + d, hy_gelu_tanh(v) * hy_ld(e + d));
    }
}

// ---- mixture of experts ---------------------------------------------------------------------------------------------------------------
// Router: one wavefront per token.  z[t][0 .. E) are the router's float32 products (the sum of `parts` K-split partial products,
// pstride apart); score = sigmoid(z), or softmax(z) over all E experts (HyRoute.softmax); the `top` largest of score (+ bias[e], where
// bias != null: it decides the choice only) are taken in descending order (the lowest index wins a tie): sel[t top + k], wgt[t top + k] =
// the chosen expert's score (without the bias), divided by the chosen scores' sum + 1e-20 (renorm), times mul.  E <= 64 * HY_RT_PER, top <= 64.
// pair_row != null (a few tokens): the pairs keep their own order, pair_row[p] = p.  extra_out != null: column E of z (the shared
// expert's gate logit) is summed into extra_out[t].
constexpr int HY_RT_PER = 16;
struct HyRoute { int softmax; const float* bias; int renorm; float mul; };
static __global__ __launch_bounds__(64) void hy_route_kernel(const float* __restrict__ z, int ldz, int parts, size_t pstride, int E, int top, int* __restrict__ sel,
                                                             float* __restrict__ wgt, int* __restrict__ pair_row, float* __restrict__ extra_out,
                                                             HyRoute rt = HyRoute{0, nullptr, 0, 1.f}) {
    const int t = blockIdx.x, lane = threadIdx.x;
    constexpr float GONE = -3.0e38f;
    float s[HY_RT_PER], c[HY_RT_PER];          // score; what the choice goes by
    float zmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < HY_RT_PER; ++i) {
        const int e = lane + 64 * i;
        float v = 0.f;
        if (e < E + (extra_out ? 1 : 0))
            for (int p = 0; p < parts; ++p) v += z[p * pstride + (size_t)t * ldz + e];
        if (extra_out && e == E) extra_out[t] = v;
        s[i] = v;
        if (e < E) zmax = fmaxf(zmax, v);
    }
    if (rt.softmax) {
        zmax = hy_wave_max(zmax);
        float den = 0.f;
#pragma unroll
        for (int i = 0; i < HY_RT_PER; ++i) { s[i] = lane + 64 * i < E ? expf(s[i] - zmax) : 0.f; den += s[i]; }
        den = hy_wave_sum(den);
#pragma unroll
        for (int i = 0; i < HY_RT_PER; ++i) s[i] = s[i] / den;
    } else {
#pragma unroll
        for (int i = 0; i < HY_RT_PER; ++i) s[i] = hy_sigmoid(s[i]);
    }
#pragma unroll
    for (int i = 0; i < HY_RT_PER; ++i) {
        const int e = lane + 64 * i;
        c[i] = e < E ? s[i] + (rt.bias ? rt.bias[e] : 0.f) : GONE;
    }
    float wsum = 0.f, myw = 0.f;          // lane k keeps the weight of choice k (top <= 64) until the sum is known
    int mysel = 0;
    for (int k = 0; k < top; ++k) {
        float best = GONE, bs = 0.f;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < HY_RT_PER; ++i)
            if (c[i] > best) { best = c[i]; bs = s[i]; bi = lane + 64 * i; }        // ascending index within a lane: strict > keeps the lowest
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64), os = __shfl_xor(bs, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ob > best || (ob == best && oi < bi)) { best = ob; bs = os; bi = oi; }
        }
        wsum += bs;
        if (lane == k) { myw = bs; mysel = bi; }
#pragma unroll
        for (int i = 0; i < HY_RT_PER; ++i)
            if (lane + 64 * i == bi) c[i] = GONE;
    }
    if (lane < top) {
        sel[t * top + lane] = mysel;
        wgt[t * top + lane] = (rt.renorm || rt.mul != 1.f) ? myw * (rt.mul / (rt.renorm ? wsum + 1e-20f : 1.f)) : myw;
        if (pair_row) pair_row[t * top + lane] = t * top + lane;
    }
}

// Grouping for portions of many tokens: the P = n top (token, choice) pairs are ordered by expert.  pair_row[p] = the pair's row in that
// order; tiles = {first row, rows (<= BM), expert} per BM rows of an expert, ntiles[0] their count (<= P / BM + min(E, P)).  One
// workgroup; the order inside an expert's rows is arbitrary (a row's result does not depend on its place).  LDS: 2 E ints.
static __global__ __launch_bounds__(256) void hy_moe_group_kernel(const int* __restrict__ sel, int P, int E, int BM, int* __restrict__ pair_row, int* __restrict__ tiles,
                                                                  int* __restrict__ ntiles) {
    extern __shared__ int gsm[];
    int* cnt = gsm;          // [E] rows per expert, then the next free row of the expert
    int* off = gsm + E;      // [E] first row of the expert
    for (int e = threadIdx.x; e < E; e += 256) cnt[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += 256) atomicAdd(&cnt[sel[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int row = 0, nt = 0;
        for (int e = 0; e < E; ++e) {
            const int c = cnt[e];
            off[e] = row;
            for (int r = 0; r < c; r += BM) { tiles[3 * nt] = row + r; tiles[3 * nt + 1] = min(BM, c - r); tiles[3 * nt + 2] = e; ++nt; }
            row += c;
        }
        ntiles[0] = nt;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += 256) cnt[e] = off[e];
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += 256) pair_row[p] = atomicAdd(&cnt[sel[p]], 1);
}
// The experts' operand: row pair_row[p] = wgt[p] * h[token of p] (a score scales its expert's INPUT; wgt = null: the plain row), in the matrix type.
template <typename T>
static __global__ __launch_bounds__(256) void hy_moe_scale_kernel(const T* __restrict__ h, int W, int top, const float* __restrict__ wgt, const int* __restrict__ pair_row,
                                                                  T* __restrict__ out) {
    const int p = blockIdx.x, t = p / top;
    const float s = wgt ? wgt[p] : 1.f;
    T* dst = out + (size_t)pair_row[p] * W;
    for (int w = threadIdx.x; w < W; w += 256) hy_st(dst + w, s * hy_ld(h + (size_t)t * W + w));
}
