// moe.hip -- the routing side of a mixture of experts: router scores and the choice (F32), the stable grouping of (token, slot) pairs by expert that
// the grouped product (dense.hip) consumes, the clipped gated activation between an expert's two products, and the weighted sum back into the
// residual stream.  The experts' products themselves are ntk_dense calls over the stacked expert matrices.
//
// A token's result never depends on the other tokens of the launch: the grouping only decides WHERE a pair's row sits, each row is computed on its
// own, and the sum over a token's slots runs in slot order.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

constexpr int kMaxExperts = 256;

// one wave per token: lanes stride the row, one reduction per expert; lane 0 then does the softmax and the `top` picks
__global__ __launch_bounds__(256) void moe_route_kernel(int* ids, float* wts, float* sgate, const float* h, int ldh, const float* wr, const float* wsg, int T,
                                                        int n, int E, int top) {
    __shared__ float zs[4][kMaxExperts];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= T) return;
    const float* x = h + (long long)t * ldh;
    for (int e = 0; e < E; ++e) {
        const float* w = wr + (long long)e * n;
        float s = 0.0f;
        for (int k = lane; k < n; k += 64) s = fmaf(w[k], x[k], s);
        s = wave_sum(s);
        if (lane == 0) zs[wave][e] = s;
    }
    if (wsg && sgate) {
        float s = 0.0f;
        for (int k = lane; k < n; k += 64) s = fmaf(wsg[k], x[k], s);
        s = wave_sum(s);
        if (lane == 0) sgate[t] = 1.0f / (1.0f + expf(-s));
    }
    if (lane != 0) return;
    float* z = zs[wave];
    float m = z[0];
    for (int e = 1; e < E; ++e) m = fmaxf(m, z[e]);
    float den = 0.0f;
    for (int e = 0; e < E; ++e) { z[e] = expf(z[e] - m); den += z[e]; }
    float chosen = 0.0f;
    for (int s = 0; s < top; ++s) {
        int best = -1;
        float bv = -1.0f;
        for (int e = 0; e < E; ++e)
            if (z[e] > bv) { bv = z[e]; best = e; }
        ids[(long long)t * top + s] = best;
        const float sc = bv / den;
        wts[(long long)t * top + s] = sc;
        chosen += sc;
        z[best] = -2.0f;
    }
    const float inv = 1.0f / (chosen + 1e-20f);
    for (int s = 0; s < top; ++s) wts[(long long)t * top + s] *= inv;
}

// stable counting sort of the pairs by expert, one workgroup: thread e counts, thread 0 scans, thread e places
__global__ __launch_bounds__(256) void moe_group_kernel(int* offsets, int* order, int* where, const int* ids, int n_pairs, int E) {
    __shared__ int start[kMaxExperts + 1];
    const int e = threadIdx.x;
    int c = 0;
    if (e < E)
        for (int i = 0; i < n_pairs; ++i) c += ids[i] == e;
    if (e < E) start[e + 1] = c;
    if (e == 0) start[0] = 0;
    __syncthreads();
    if (e == 0)
        for (int i = 0; i < E; ++i) start[i + 1] += start[i];
    __syncthreads();
    if (e <= E) offsets[e] = start[e];
    if (e < E) {
        int at = start[e];
        for (int i = 0; i < n_pairs; ++i)
            if (ids[i] == e) { order[at] = i; where[i] = at; ++at; }
    }
}

__global__ void clipped_glu_kernel(float* a, const float* gu, int ff, float limit, float alpha) {
    const long long r = blockIdx.y;
    const int f = blockIdx.x * blockDim.x + threadIdx.x;
    if (f >= ff) return;
    const float g = fminf(gu[r * 2 * ff + f], limit);
    const float u = fminf(fmaxf(gu[r * 2 * ff + ff + f], -limit), limit);
    a[r * ff + f] = g * (1.0f / (1.0f + expf(-alpha * g))) * (u + 1.0f);
}

__global__ void moe_combine_kernel(float* x, const float* mix, const float* d, const int* where, const float* wts, const float* shared, const float* sgate,
                                   int top, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = 0.0f;
    for (int k = 0; k < top; ++k) s = fmaf(wts[t * top + k], d[(long long)where[t * top + k] * n + i], s);
    if (shared) s = fmaf(sgate[t], shared[t * n + i], s);
    if (mix) s += mix[t * n + i];
    x[t * n + i] += s;
}

}  // namespace ntk

using namespace ntk;

int ntk_moe_route(int* ids, float* wts, float* sgate, const float* h, int ldh, const float* w_router, const float* shared_gate_w, int T, int n, int E, int top,
                  void* stream) {
    if (!ids || !wts || !h || !w_router) return NTK_E_NULL;
    if (T < 0 || n <= 0 || E <= 0 || E > kMaxExperts || top <= 0 || top > E || ldh < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(moe_route_kernel, dim3((T + 3) / 4), dim3(256), 0, resolve_stream(stream), ids, wts, sgate, h, ldh, w_router, shared_gate_w, T, n, E, top);
    return last_launch_status();
}

int ntk_moe_group(int* offsets, int* order, int* where, const int* ids, int T, int top, int E, void* stream) {
    if (!offsets || !order || !where || !ids) return NTK_E_NULL;
    if (T < 0 || top <= 0 || E <= 0 || E >= 256) return NTK_E_SHAPE;
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(256), 0, resolve_stream(stream), offsets, order, where, ids, T * top, E);
    return last_launch_status();
}

int ntk_clipped_glu(float* a, const float* gu, int rows, int ff, float limit, float alpha, void* stream) {
    if (!a || !gu) return NTK_E_NULL;
    if (rows < 0 || ff <= 0) return NTK_E_SHAPE;
    if (rows == 0) return NTK_OK;
    hipLaunchKernelGGL(clipped_glu_kernel, dim3((ff + 255) / 256, rows), dim3(256), 0, resolve_stream(stream), a, gu, ff, limit, alpha);
    return last_launch_status();
}

int ntk_moe_combine(float* x, const float* mix, const float* d, const int* where, const float* wts, const float* shared, const float* sgate, int T, int top,
                    int n, void* stream) {
    if (!x || !d || !where || !wts || (shared && !sgate)) return NTK_E_NULL;
    if (T < 0 || top <= 0 || n <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), x, mix, d, where, wts, shared, sgate, top, n);
    return last_launch_status();
}
