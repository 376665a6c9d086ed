// lightning_attention.hip -- linear attention with a per-head decay, S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, in F32.
//
// A portion is walked in chunks of C tokens.  With S the state before a chunk, i and j token indices inside it and L = ln(decay):
//     o_i   = sum_{j <= i} exp((i - j) L) (q_i . k_j) v_j  +  exp((i + 1) L) S^T q_i
//     S_new = exp(n L) S + sum_j exp((n - 1 - j) L) k_j v_j^T                  (n = tokens of the chunk)
// -- only non-negative powers of the decay occur, so nothing overflows however small it is.  A workgroup owns one head and a slab of 64 value columns and
// keeps its [dn][64] slice of the state in LDS across the chunks; the state is read from memory at the start (zeros when the sequence starts here) and written
// back at the end.  One token (decoding) is a chunk of one: the state slice is read, updated and written once.
// Thread tiles are 4 x 4 (scores: tokens x tokens; outputs: tokens x columns) and (dn / 16) x 4 (state rows x columns); q, k and v pass through silu on
// their way into LDS when the caller asks for it.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

constexpr int LV = 64;     // value columns per workgroup

struct LightArgs {
    float* out; int ldo;
    const float* q; int ldq;
    const float* k; int ldk;
    const float* v; int ldv;
    const float* log_decay;
    float* state;
    int H, dn, dv, silu, pos0, T;
};

__device__ __forceinline__ float decay_pow(float L, int n) { return n == 0 ? 1.0f : expf((float)n * L); }
__device__ __forceinline__ float maybe_silu(float x, int on) { return on ? x / (1.0f + expf(-x)) : x; }

template <int C>
__global__ __launch_bounds__(256) void lightning_attention_kernel(const LightArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int DP = (a.dn + 15) & ~15;              // state rows, padded (the padding stays zero)
    const int LQ = DP + 1;                         // row length of the q / k chunks
    float* Qs = lds;                               // [C][LQ]
    float* Ks = Qs + C * LQ;                       // [C][LQ]
    float* Vs = Ks + C * LQ;                       // [C][LV]
    float* Ss = Vs + C * LV;                       // [DP][LV]
    float* Ps = Ss + DP * LV;                      // [C][C + 1]
    float* Ws = Ps + C * (C + 1);                  // [C] the weight of token j in the new state
    const int h = blockIdx.x, v0 = blockIdx.y * LV, nv = min(LV, a.dv - v0);
    const int tid = threadIdx.x;
    const float L = a.log_decay[h];
    float* sg = a.state + ((long long)h * a.dn) * a.dv + v0;
    for (int e = tid; e < DP * LV; e += 256) {
        const int d = e / LV, c = e % LV;
        Ss[e] = (a.pos0 > 0 && d < a.dn && c < nv) ? sg[(long long)d * a.dv + c] : 0.0f;
    }
    const int ti = tid / 16, tj = tid % 16;        // 16 x 16 thread grid
    constexpr int RI = C / 16;                     // token rows per thread (C = 64: 4, C = 32: 2)
    for (int t0 = 0; t0 < a.T; t0 += C) {
        const int n = min(C, a.T - t0);
        const int nr = min(C, (n + RI - 1) / RI * RI);   // rows a thread tile may touch: the chunk's tokens rounded up to whole tiles
        __syncthreads();                           // the last chunk's readers are done (and the state slice is in place)
        if (tid < C) Ws[tid] = tid < n ? decay_pow(L, n - 1 - tid) : 0.0f;
        for (int e = tid; e < nr * DP; e += 256) {
            const int i = e / DP, d = e % DP;
            float qv = 0.0f, kv = 0.0f;
            if (i < n && d < a.dn) {
                qv = maybe_silu(a.q[(long long)(t0 + i) * a.ldq + h * a.dn + d], a.silu);
                kv = maybe_silu(a.k[(long long)(t0 + i) * a.ldk + h * a.dn + d], a.silu);
            }
            Qs[i * LQ + d] = qv;
            Ks[i * LQ + d] = kv;
        }
        for (int e = tid; e < nr * LV; e += 256) {
            const int i = e / LV, c = e % LV;
            Vs[e] = (i < n && c < nv) ? maybe_silu(a.v[(long long)(t0 + i) * a.ldv + h * a.dv + v0 + c], a.silu) : 0.0f;
        }
        __syncthreads();
        // ---- decayed scores inside the chunk: thread (ti, tj) owns tokens i = ti * RI + r against j = tj * RI + c
        if (ti * RI < n && tj <= ti) {
            float s[RI][RI];
#pragma unroll
            for (int r = 0; r < RI; ++r)
#pragma unroll
                for (int c = 0; c < RI; ++c) s[r][c] = 0.0f;
            for (int d = 0; d < a.dn; ++d) {
                float qv[RI], kv[RI];
#pragma unroll
                for (int r = 0; r < RI; ++r) { qv[r] = Qs[(ti * RI + r) * LQ + d]; kv[r] = Ks[(tj * RI + r) * LQ + d]; }
#pragma unroll
                for (int r = 0; r < RI; ++r)
#pragma unroll
                    for (int c = 0; c < RI; ++c) s[r][c] = fmaf(qv[r], kv[c], s[r][c]);
            }
#pragma unroll
            for (int r = 0; r < RI; ++r)
#pragma unroll
                for (int c = 0; c < RI; ++c) {
                    const int i = ti * RI + r, j = tj * RI + c;
                    Ps[i * (C + 1) + j] = j <= i ? s[r][c] * decay_pow(L, i - j) : 0.0f;
                }
        } else if (ti * RI < n) {
#pragma unroll
            for (int r = 0; r < RI; ++r)
#pragma unroll
                for (int c = 0; c < RI; ++c) Ps[(ti * RI + r) * (C + 1) + tj * RI + c] = 0.0f;
        }
        __syncthreads();
        // ---- outputs: thread (ti, tj) owns tokens ti * RI + r and columns tj * 4 + c
        if (ti * RI < n) {
            float o[RI][4], u[RI][4];
#pragma unroll
            for (int r = 0; r < RI; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) { o[r][c] = 0.0f; u[r][c] = 0.0f; }
            const int jn = min(n, (ti + 1) * RI);
            for (int j = 0; j < jn; ++j) {
                const float4 v4 = *reinterpret_cast<const float4*>(Vs + j * LV + tj * 4);
#pragma unroll
                for (int r = 0; r < RI; ++r) {
                    const float p = Ps[(ti * RI + r) * (C + 1) + j];
                    o[r][0] = fmaf(p, v4.x, o[r][0]); o[r][1] = fmaf(p, v4.y, o[r][1]); o[r][2] = fmaf(p, v4.z, o[r][2]); o[r][3] = fmaf(p, v4.w, o[r][3]);
                }
            }
            for (int d = 0; d < a.dn; ++d) {
                const float4 s4 = *reinterpret_cast<const float4*>(Ss + d * LV + tj * 4);
#pragma unroll
                for (int r = 0; r < RI; ++r) {
                    const float qv = Qs[(ti * RI + r) * LQ + d];
                    u[r][0] = fmaf(qv, s4.x, u[r][0]); u[r][1] = fmaf(qv, s4.y, u[r][1]); u[r][2] = fmaf(qv, s4.z, u[r][2]); u[r][3] = fmaf(qv, s4.w, u[r][3]);
                }
            }
#pragma unroll
            for (int r = 0; r < RI; ++r) {
                const int i = ti * RI + r;
                if (i >= n) continue;
                const float w = decay_pow(L, i + 1);
                float* op = a.out + (long long)(t0 + i) * a.ldo + h * a.dv + v0 + tj * 4;
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    if (tj * 4 + c < nv) op[c] = fmaf(w, u[r][c], o[r][c]);
            }
        }
        __syncthreads();                           // every reader of the old state slice is done
        // ---- the state: thread (ti, tj) owns rows d = ti + 16 r and columns tj * 4 + c; every token's value row is read once for all of them
        {
            const float wn = decay_pow(L, n);
            const int nd = DP / 16;
            float acc[16][4];
#pragma unroll
            for (int r = 0; r < 16; ++r) { acc[r][0] = 0.0f; acc[r][1] = 0.0f; acc[r][2] = 0.0f; acc[r][3] = 0.0f; }
            for (int j = 0; j < n; ++j) {
                const float w = Ws[j];
                const float4 v4 = *reinterpret_cast<const float4*>(Vs + j * LV + tj * 4);
                const float* kr = Ks + j * LQ + ti;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (r < nd) {
                        const float kw = kr[16 * r] * w;
                        acc[r][0] = fmaf(kw, v4.x, acc[r][0]); acc[r][1] = fmaf(kw, v4.y, acc[r][1]); acc[r][2] = fmaf(kw, v4.z, acc[r][2]); acc[r][3] = fmaf(kw, v4.w, acc[r][3]);
                    }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (r < nd) {
                    float4 s4 = *reinterpret_cast<const float4*>(Ss + (ti + 16 * r) * LV + tj * 4);
                    s4.x = fmaf(wn, s4.x, acc[r][0]); s4.y = fmaf(wn, s4.y, acc[r][1]); s4.z = fmaf(wn, s4.z, acc[r][2]); s4.w = fmaf(wn, s4.w, acc[r][3]);
                    *reinterpret_cast<float4*>(Ss + (ti + 16 * r) * LV + tj * 4) = s4;
                }
        }
    }
    __syncthreads();
    for (int e = tid; e < DP * LV; e += 256) {
        const int d = e / LV, c = e % LV;
        if (d < a.dn && c < nv) sg[(long long)d * a.dv + c] = Ss[e];
    }
}

}  // namespace ntk

using namespace ntk;

int ntk_lightning_attention(float* out, int ldo, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* log_decay, float* state,
                            int H, int dn, int dv, int silu, int pos0, int T, void* stream) {
    if (!out || !q || !k || !v || !log_decay || !state) return NTK_E_NULL;
    if (T < 0 || H <= 0 || dn <= 0 || dn > 256 || dv <= 0 || pos0 < 0) return NTK_E_SHAPE;
    if (ldo < H * dv || ldq < H * dn || ldk < H * dn || ldv < H * dv) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    LightArgs a{out, ldo, q, ldq, k, ldk, v, ldv, log_decay, state, H, dn, dv, silu, pos0, T};
    const int DP = (dn + 15) & ~15;
    const int C = dn > 128 ? 32 : 64;          // chunk length: the LDS of two [C][dn] chunks, the value slab, the state slice and the scores
    const size_t lds = ((size_t)2 * C * (DP + 1) + (size_t)C * LV + (size_t)DP * LV + (size_t)C * (C + 1) + C) * sizeof(float);
    if (lds > 156 * 1024) return NTK_E_SHAPE;
    static bool raised = false;   // (idempotent: a race sets the same attribute twice)
    if (!raised) {
        NTK_HIP_TRY(hipFuncSetAttribute((const void*)lightning_attention_kernel<64>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
        NTK_HIP_TRY(hipFuncSetAttribute((const void*)lightning_attention_kernel<32>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
        raised = true;
    }
    const dim3 grid(H, (dv + LV - 1) / LV);
    if (C == 64) hipLaunchKernelGGL(lightning_attention_kernel<64>, grid, dim3(256), lds, resolve_stream(stream), a);
    else hipLaunchKernelGGL(lightning_attention_kernel<32>, grid, dim3(256), lds, resolve_stream(stream), a);
    return last_launch_status();
}
