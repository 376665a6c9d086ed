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

// one workgroup per token: its 16 waves share the experts (wave w: experts w, w + 16, ...), a lane requests its whole part of the router row before
// it uses any of it; thread 0 then does the softmax and the `top` picks over the scores in LDS
constexpr int kRouteThreads = 1024;
__global__ __launch_bounds__(kRouteThreads) void moe_route_kernel(int* ids, float* wts, float* sgate, const float* h, int ldh, const float* wr, const float* wsg,
                                                                 int n, int E, int top) {
    __shared__ float z[kMaxExperts];
    extern __shared__ __attribute__((aligned(16))) float xs[];   // the token's row
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = kRouteThreads / 64;
    const long long t = blockIdx.x;
    const float* x = h + t * ldh;
    for (int k = threadIdx.x; k < n; k += kRouteThreads) xs[k] = x[k];
    __syncthreads();
    const bool vec = (n % 4 == 0) && !((uintptr_t)wr & 15) && !(wsg && ((uintptr_t)wsg & 15));
    for (int e = wave; e < E + (wsg ? 1 : 0); e += nw) {
        const float* w = e < E ? wr + (long long)e * n : wsg;
        float s = 0.0f;
        if (vec) {
#pragma unroll 4
            for (int k = lane * 4; k < n; k += 256) {
                const float4 a4 = *reinterpret_cast<const float4*>(w + k), x4 = *reinterpret_cast<const float4*>(xs + k);
                s = fmaf(a4.x, x4.x, s); s = fmaf(a4.y, x4.y, s); s = fmaf(a4.z, x4.z, s); s = fmaf(a4.w, x4.w, s);
            }
        } else {
            for (int k = lane; k < n; k += 64) s = fmaf(w[k], xs[k], s);
        }
        s = wave_sum(s);
        if (lane == 0) {
            if (e < E) z[e] = s;
            else if (sgate) sgate[t] = 1.0f / (1.0f + expf(-s));
        }
    }
    __syncthreads();
    if (wave != 0) return;
    // softmax and the picks by one wave: lane l holds experts l, l + 64, l + 128, l + 192
    float v[4];
    float m = -INFINITY;
#pragma unroll
    for (int c = 0; c < 4; ++c) { v[c] = lane + 64 * c < E ? z[lane + 64 * c] : -INFINITY; m = fmaxf(m, v[c]); }
    m = wave_max(m);
    float den = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) { v[c] = lane + 64 * c < E ? expf(v[c] - m) : -1.0f; den += fmaxf(v[c], 0.0f); }
    den = wave_sum(den);
    __shared__ int pick_id[kMaxExperts];
    __shared__ float pick_sc[kMaxExperts];
    float chosen = 0.0f;
    for (int s = 0; s < top; ++s) {
        float bv = v[0];
        int bi = lane;
#pragma unroll
        for (int c = 1; c < 4; ++c)
            if (v[c] > bv) { bv = v[c]; bi = lane + 64 * c; }      // (equal values: the lower index stays)
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) {
            const float ov = __shfl_xor(bv, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        const float sc = bv / den;
        chosen += sc;
        if (lane == 0) { pick_id[s] = bi; pick_sc[s] = sc; }
        if ((bi & 63) == lane) v[bi >> 6] = -2.0f;
    }
    const float inv = 1.0f / (chosen + 1e-20f);
    for (int s = lane; s < top; s += 64) { ids[t * top + s] = pick_id[s]; wts[t * top + s] = pick_sc[s] * inv; }   // (same wave wrote them: in order)
}

// Stable counting sort of the pairs by expert, one workgroup of 1024: the pairs are cut into S = 1024 / E' contiguous segments (E' = E rounded up to a
// power of two), thread (segment, expert) counts its expert in its segment, one scan in (expert, segment) order gives every thread the place of its
// first row, and it walks its segment once more to place them.  The ids sit in LDS when they fit.
constexpr int kGroupThreads = 1024, kGroupLdsIds = 24 * 1024;
__global__ __launch_bounds__(kGroupThreads) void moe_group_kernel(int* offsets, int* order, int* where, const int* ids_g, int n_pairs, int E, int Ep) {
    __shared__ int cnt[kGroupThreads + 1];
    __shared__ int ids_s[kGroupLdsIds];
    const int* ids = ids_g;
    if (n_pairs <= kGroupLdsIds) {
        for (int i = threadIdx.x; i < n_pairs; i += kGroupThreads) ids_s[i] = ids_g[i];
        ids = ids_s;
    }
    const int S = kGroupThreads / Ep;
    const int e = threadIdx.x % Ep, seg = threadIdx.x / Ep;
    const int per = (n_pairs + S - 1) / S;
    const int i0 = min(seg * per, n_pairs), i1 = min(i0 + per, n_pairs);
    __syncthreads();
    int c = 0;
    if (e < E && seg < S)
        for (int i = i0; i < i1; ++i) c += ids[i] == e;
    // place of thread (e, seg) in (expert, segment) order
    const int slot = e * S + seg;
    cnt[slot] = e < E ? c : 0;             // Ep * S = 1024: every thread has a slot
    __syncthreads();
    {   // exclusive scan of the Ep * S (= 1024) counts: inside each wave by shuffles, the 16 wave totals by the first lanes
        __shared__ int wave_total[kGroupThreads / 64];
        const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
        const int mine = cnt[threadIdx.x];
        int inc = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(inc, o, 64);
            if (lane >= o) inc += up;
        }
        if (lane == 63) wave_total[wv] = inc;
        __syncthreads();
        int before = 0;
        for (int k = 0; k < wv; ++k) before += wave_total[k];
        cnt[threadIdx.x] = before + inc - mine;
        if (threadIdx.x == kGroupThreads - 1) cnt[kGroupThreads] = before + inc;
    }
    __syncthreads();
    if (threadIdx.x <= E) offsets[threadIdx.x] = threadIdx.x < E ? cnt[threadIdx.x * S] : cnt[kGroupThreads];
    if (e < E && seg < S) {
        int at = cnt[slot];
        for (int i = i0; i < i1; ++i)
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
    if ((size_t)n * 4 > 128 * 1024) return NTK_E_SHAPE;
    hipLaunchKernelGGL(moe_route_kernel, dim3(T), dim3(kRouteThreads), (size_t)n * 4, resolve_stream(stream), ids, wts, sgate, h, ldh, w_router, shared_gate_w, n, E, top);
    return last_launch_status();
}

int ntk_moe_group(int* offsets, int* order, int* where, const int* ids, int T, int top, int E, void* stream) {
    if (!offsets || !order || !where || !ids) return NTK_E_NULL;
    if (T < 0 || top <= 0 || E <= 0 || E >= 256) return NTK_E_SHAPE;
    int Ep = 1;
    while (Ep < E) Ep *= 2;
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(kGroupThreads), 0, resolve_stream(stream), offsets, order, where, ids, T * top, E, Ep);
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
