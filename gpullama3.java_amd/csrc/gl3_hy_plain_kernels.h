// gl3_hy_plain_kernels.h — kernels of layer-list designs with ONE plain residual stream (gl3_model_desc.streams == 0): the residual
// update with everything that can ride on it (sum of K-split parts, gated shared expert, routed experts' rows, unit-RMS side input,
// weighted average over earlier layers' results, the next sublayer's norm), the per-layer token input's activation, and the mixture of
// experts' router, grouping and input scaling.  Every mechanism takes its sizes and constants as arguments.
#pragma once
#include "gl3_hy_kernels.h"

__device__ __forceinline__ float hy_gelu_tanh(float z) { return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

// ---- residual update ----------------------------------------------------------------------------------------------------------------
// One workgroup per token.  In this order, every part optional (null pointer = absent):
//   x += ga * sum_z ya[z]                       ya: a sublayer's output, possibly as K-split parts; ga = sigmoid(gate_z[t * gate_ld]) or 1
//   x += sum_k eo[pair_row[t top + k]]          the routed experts' down projections of this token
//   x += yc / sqrt(mean(yc^2) + eps) * cw       a unit-RMS normed input with a plain weight
//   hist_out[t] = x;  x = sum_j mix[j] hist[j][t], j < n_mix, where hist[n_mix - 1] is hist_out (what the layer leaves is an average over
//                                               the embedding output and every layer's result so far)
//   x is written back; xt = x in the matrix type (operand of a following product); tap = x
//   h = x / sqrt(mean(x^2) + eps) * norm_w in the matrix type (the next sublayer's input; norm_w already holds any offset)
struct HyResid {
    float* x; int W;
    const float* ya; int ya_parts; size_t ya_stride; const float* gate_z; int gate_ld;
    const float* eo; const int* pair_row; int top;
    const float* yc; const float* cw;
    float* hist; size_t hist_stride; int n_mix; const float* mix;      // hist_out = hist + (n_mix - 1) hist_stride
    float* tap;
    const float* norm_w; float eps;
};
template <typename TO, int NT>
static __global__ __launch_bounds__(NT) void hy_resid_kernel(HyResid a, TO* __restrict__ xt, TO* __restrict__ h_out) {
    __shared__ float red[NT / 64];
    const int t = blockIdx.x, W = a.W;
    const size_t row = (size_t)t * W;
    float cr = 0.f;
    if (a.yc) {
        float ss = 0.f;
        for (int w = threadIdx.x; w < W; w += NT) { const float v = a.yc[row + w]; ss += v * v; }
        ss = hy_block_sum<NT>(ss, red);
        cr = 1.f / sqrtf(ss / (float)W + a.eps);
    }
    const float ga = a.gate_z ? hy_sigmoid(a.gate_z[(size_t)t * a.gate_ld]) : 1.f;
    float ss = 0.f;
    for (int w = threadIdx.x; w < W; w += NT) {
        float x = a.x[row + w];
        if (a.ya) {
            float y = a.ya[row + w];
            for (int z = 1; z < a.ya_parts; ++z) y += a.ya[z * a.ya_stride + row + w];
            x += ga * y;
        }
        if (a.eo)
            for (int k = 0; k < a.top; ++k) x += a.eo[(size_t)a.pair_row[t * a.top + k] * W + w];
        if (a.yc) x += a.yc[row + w] * cr * a.cw[w];
        if (a.hist) {
            a.hist[(size_t)(a.n_mix - 1) * a.hist_stride + row + w] = x;
            float m = a.mix[a.n_mix - 1] * x;
            for (int j = 0; j < a.n_mix - 1; ++j) m = fmaf(a.mix[j], a.hist[(size_t)j * a.hist_stride + row + w], m);
            x = m;
        }
        a.x[row + w] = x;
        if (xt) hy_st(xt + row + w, x);
        if (a.tap) a.tap[row + w] = x;
        ss += x * x;
    }
    if (!a.norm_w) return;
    ss = hy_block_sum<NT>(ss, red);
    const float r = 1.f / sqrtf(ss / (float)W + a.eps);
    for (int w = threadIdx.x; w < W; w += NT) hy_st(h_out + row + w, a.x[row + w] * r * a.norm_w[w]);        // a thread re-reads what it wrote
}

// ---- per-layer token input: g[t][d] = gelu_tanh(z[t][d]) * side_embed[token t][col0 + d] as the projection's operand (row stride ldg, zero beyond D) ----
template <typename T>
static __global__ __launch_bounds__(256) void hy_side_act_kernel(const float* __restrict__ z, int D, const int* __restrict__ tokens, const T* __restrict__ table,
                                                                 int table_ld, int col0, T* __restrict__ g, int ldg) {
    const int t = blockIdx.x;
    const T* e = table + (size_t)tokens[t] * table_ld + col0;
    for (int d = threadIdx.x; d < ldg; d += 256) hy_st(g + (size_t)t * ldg + d, d < D ? hy_gelu_tanh(z[(size_t)t * D + d]) * hy_ld(e + d) : 0.f);
}

// ---- mixture of experts ---------------------------------------------------------------------------------------------------------------
// Router: one wavefront per token.  z[t][0 .. E) are the router's float32 products; score = sigmoid(z); the `top` largest scores are
// taken in descending order (the lowest index wins a tie): sel[t top + k], wgt[t top + k] = score.  E <= 64 * HY_RT_PER.
constexpr int HY_RT_PER = 16;
static __global__ __launch_bounds__(64) void hy_route_kernel(const float* __restrict__ z, int ldz, int E, int top, int* __restrict__ sel, float* __restrict__ wgt) {
    const int t = blockIdx.x, lane = threadIdx.x;
    float s[HY_RT_PER];
#pragma unroll
    for (int i = 0; i < HY_RT_PER; ++i) {
        const int e = lane + 64 * i;
        s[i] = e < E ? hy_sigmoid(z[(size_t)t * ldz + e]) : -1.f;
    }
    for (int k = 0; k < top; ++k) {
        float best = -2.f;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < HY_RT_PER; ++i)
            if (s[i] > best) { best = s[i]; bi = lane + 64 * i; }        // ascending index within a lane: strict > keeps the lowest
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
        }
        if (lane == 0) { sel[t * top + k] = bi; wgt[t * top + k] = best; }
#pragma unroll
        for (int i = 0; i < HY_RT_PER; ++i)
            if (lane + 64 * i == bi) s[i] = -1.f;
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
// a few tokens (decode): pairs keep their own order
static __global__ __launch_bounds__(256) void hy_iota_kernel(int* __restrict__ out, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = i;
}

// The experts' operand: row pair_row[p] = wgt[p] * h[token of p] (a score scales its expert's INPUT), in the matrix type.
template <typename T>
static __global__ __launch_bounds__(256) void hy_moe_scale_kernel(const T* __restrict__ h, int W, int top, const float* __restrict__ wgt, const int* __restrict__ pair_row,
                                                                  T* __restrict__ out) {
    const int p = blockIdx.x, t = p / top;
    const float s = wgt[p];
    T* dst = out + (size_t)pair_row[p] * W;
    for (int w = threadIdx.x; w < W; w += 256) hy_st(dst + w, s * hy_ld(h + (size_t)t * W + w));
}
