// lightning_attention.hip -- linear attention with a per-head decay, S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, in F32.
//
// A portion is walked in chunks of C tokens.  With S the state before a chunk, i and j token indices inside it and L = ln(decay):
//     o_i   = sum_{j <= i} exp((i - j) L) (q_i . k_j) v_j  +  exp((i + 1) L) S^T q_i
//     S_new = exp(n L) S + sum_j exp((n - 1 - j) L) k_j v_j^T                  (n = tokens of the chunk)
// -- only non-negative powers of the decay occur, so nothing overflows however small it is.  A workgroup owns one head and a slab of 64 value columns and
// keeps its [dn][64] slice of the state in LDS across the chunks; the state is read from memory at the start (zeros when the sequence starts here) and written
// back at the end.  Thread tiles are 4 x 4 (scores: tokens x tokens; outputs: tokens x columns) and (dn / 16) x 4 (state rows x columns); q, k and v pass
// through silu on their way into LDS when the caller asks for it.
// Three forms of the same sums:
//   * few tokens (decoding, up to kStepRows): lightning_step_kernel keeps its state slice in REGISTERS (thread = (rows d = part + 4 r, one value column)), walks the
//     tokens one by one -- S = decay S + k v^T, o = S^T q with the four row parts added through LDS -- and writes the slice back: state bytes once in, once out;
//   * one chunk or no scratch: lightning_chunk_kernel<C, kWhole>, the walk described above by one workgroup per (head, value slab);
//   * long portions with scratch: the chunks run side by side.  kLocal: every (chunk, head, slab) forms its own sum_j exp((n - 1 - j) L) k_j v_j^T;
//     lightning_scan_kernel then walks the chunks per state element (S_c = exp(n L) S_(c-1) + local_c, leaving S_(c-1) where local_c was) and writes the final
//     state; kOutputs: every (chunk, head, slab) forms its outputs from its chunk's scores and the state before it.
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
    float* scratch;
};

__device__ __forceinline__ float decay_pow(float L, int n) { return n == 0 ? 1.0f : expf((float)n * L); }
__device__ __forceinline__ float maybe_silu(float x, int on) { return on ? x / (1.0f + expf(-x)) : x; }

enum ChunkMode { kWhole = 0, kLocal = 1, kOutputs = 2 };

template <int C, int MODE>
__global__ __launch_bounds__(256) void lightning_chunk_kernel(const LightArgs a) {
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
    // kWhole: the sequence's state; kLocal / kOutputs: this chunk's slot of the scratch [chunks][H][dn][dv] (written / read)
    float* sg = (MODE == kWhole ? a.state : a.scratch + (long long)blockIdx.z * a.H * a.dn * a.dv) + ((long long)h * a.dn) * a.dv + v0;
    // (every staging loop below asks for eight of a thread's entries before it uses the first: a workgroup fills the LDS of its CU, so nobody else hides its latency)
    const bool have = MODE == kOutputs || (MODE == kWhole && a.pos0 > 0);
    for (int e0 = tid; e0 < DP * LV; e0 += 256 * 8) {
        float x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int e = e0 + 256 * u, d = e / LV, c = e % LV;
            x[u] = (have && e < DP * LV && d < a.dn && c < nv) ? sg[(long long)d * a.dv + c] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (e0 + 256 * u < DP * LV) Ss[e0 + 256 * u] = x[u];
    }
    const int ti = tid / 16, tj = tid % 16;        // 16 x 16 thread grid
    constexpr int RI = C / 16;                     // token rows per thread (C = 64: 4, C = 32: 2)
    const int t_first = MODE == kWhole ? 0 : (int)blockIdx.z * C, t_last = MODE == kWhole ? a.T : min(a.T, t_first + C);
    for (int t0 = t_first; t0 < t_last; t0 += C) {
        const int n = min(C, a.T - t0);
        const int nr = min(C, (n + RI - 1) / RI * RI);   // rows a thread tile may touch: the chunk's tokens rounded up to whole tiles
        __syncthreads();                           // the last chunk's readers are done (and the state slice is in place)
        if (tid < C) Ws[tid] = tid < n ? decay_pow(L, n - 1 - tid) : 0.0f;
        for (int e0 = tid; e0 < nr * DP; e0 += 256 * 8) {
            float qv[8], kv[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int e = e0 + 256 * u, i = e / DP, d = e % DP;
                const bool in = e < nr * DP && i < n && d < a.dn;
                qv[u] = in && MODE != kLocal ? a.q[(long long)(t0 + i) * a.ldq + h * a.dn + d] : 0.0f;     // (the local sums need no queries)
                kv[u] = in ? a.k[(long long)(t0 + i) * a.ldk + h * a.dn + d] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int e = e0 + 256 * u, i = e / DP, d = e % DP;
                if (e < nr * DP) { Qs[i * LQ + d] = maybe_silu(qv[u], a.silu); Ks[i * LQ + d] = maybe_silu(kv[u], a.silu); }
            }
        }
        for (int e0 = tid; e0 < nr * LV; e0 += 256 * 8) {
            float x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int e = e0 + 256 * u, i = e / LV, c = e % LV;
                x[u] = (e < nr * LV && i < n && c < nv) ? a.v[(long long)(t0 + i) * a.ldv + h * a.dv + v0 + c] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (e0 + 256 * u < nr * LV) Vs[e0 + 256 * u] = maybe_silu(x[u], a.silu);
        }
        __syncthreads();
        // ---- decayed scores inside the chunk: thread (ti, tj) owns tokens i = ti * RI + r against j = tj * RI + c
        if (MODE != kLocal && ti * RI < n && tj <= ti) {
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
        }
        __syncthreads();
        // ---- outputs: thread (ti, tj) owns tokens ti * RI + r and columns tj * 4 + c (the scores above the diagonal tiles are never read)
        if (MODE != kLocal && ti * RI < n) {
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
        if (MODE == kOutputs) break;
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
    if (MODE == kOutputs) return;
    __syncthreads();
    for (int e = tid; e < DP * LV; e += 256) {
        const int d = e / LV, c = e % LV;
        if (d < a.dn && c < nv) sg[(long long)d * a.dv + c] = Ss[e];
    }
}

// one thread per state element: the chunks' local sums become the states BEFORE their chunks, the sequence's state moves on by the whole portion
template <int C>
__global__ __launch_bounds__(256) void lightning_scan_kernel(const LightArgs a) {
    const long long per = (long long)a.H * a.dn * a.dv;
    const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
    if (e >= per) return;
    const float L = a.log_decay[e / ((long long)a.dn * a.dv)];
    float S = a.pos0 > 0 ? a.state[e] : 0.0f;
    const int chunks = (a.T + C - 1) / C;
    const float wfull = decay_pow(L, C);
    for (int c = 0; c < chunks; ++c) {
        const float local = a.scratch[c * per + e];
        a.scratch[c * per + e] = S;
        const int n = min(C, a.T - c * C);
        S = fmaf(n == C ? wfull : decay_pow(L, n), S, local);
    }
    a.state[e] = S;
}

// few tokens: the state slice of (head, 64 value columns) in registers, rows d = part + 4 r of wave `part`; tokens one by one
constexpr int kStepRows = 8;
template <int NR>
__global__ __launch_bounds__(256) void lightning_step_kernel(const LightArgs a) {
    __shared__ float qs[256], ks[256], red[4][LV];
    const int h = blockIdx.x, v0 = blockIdx.y * LV, col = threadIdx.x & 63, part = threadIdx.x >> 6;
    const bool live = v0 + col < a.dv;
    const float lam = decay_pow(a.log_decay[h], 1);
    float* sg = a.state + ((long long)h * a.dn) * a.dv + v0 + col;
    float S[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const int d = part + 4 * r;
        S[r] = (a.pos0 > 0 && live && d < a.dn) ? sg[(long long)d * a.dv] : 0.0f;
    }
    for (int t = 0; t < a.T; ++t) {
        __syncthreads();                           // the last token's readers are done
        if ((int)threadIdx.x < a.dn) {
            qs[threadIdx.x] = maybe_silu(a.q[(long long)t * a.ldq + h * a.dn + threadIdx.x], a.silu);
            ks[threadIdx.x] = maybe_silu(a.k[(long long)t * a.ldk + h * a.dn + threadIdx.x], a.silu);
        }
        const float vv = live ? maybe_silu(a.v[(long long)t * a.ldv + h * a.dv + v0 + col], a.silu) : 0.0f;
        __syncthreads();
        float o = 0.0f;
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int d = part + 4 * r;
            if (d < a.dn) {
                S[r] = fmaf(lam, S[r], ks[d] * vv);
                o = fmaf(S[r], qs[d], o);
            }
        }
        red[part][col] = o;
        __syncthreads();
        if (part == 0 && live) a.out[(long long)t * a.ldo + h * a.dv + v0 + col] = (red[0][col] + red[1][col]) + (red[2][col] + red[3][col]);
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const int d = part + 4 * r;
        if (live && d < a.dn) sg[(long long)d * a.dv] = S[r];
    }
}

}  // namespace ntk

using namespace ntk;

static int light_chunk(int dn) { return dn > 128 ? 32 : 64; }   // chunk length: the LDS of two [C][dn] chunks, the value slab, the state slice and the scores
// side by side the chunks are 32 tokens long: half the LDS per workgroup (two of them share a CU and hide each other's round trips), twice the workgroups
static int light_chunk_parallel(int) { return 32; }

size_t ntk_lightning_attention_scratch(int T, int H, int dn, int dv) {
    if (T <= 0 || H <= 0 || dn <= 0 || dv <= 0) return 0;
    const int C = light_chunk_parallel(dn);
    return T > light_chunk(dn) ? (size_t)((T + C - 1) / C) * H * dn * dv : 0;
}

int ntk_lightning_attention(float* out, int ldo, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* log_decay, float* state,
                            int H, int dn, int dv, int silu, int pos0, int T, float* scratch, void* stream) {
    if (!out || !q || !k || !v || !log_decay || !state) return NTK_E_NULL;
    if (T < 0 || H <= 0 || dn <= 0 || dn > 256 || dv <= 0 || pos0 < 0) return NTK_E_SHAPE;
    if (ldo < H * dv || ldq < H * dn || ldk < H * dn || ldv < H * dv) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    LightArgs a{out, ldo, q, ldq, k, ldk, v, ldv, log_decay, state, H, dn, dv, silu, pos0, T, scratch};
    hipStream_t s = resolve_stream(stream);
    const int slabs = (dv + LV - 1) / LV;
    if (T <= kStepRows) {
        const dim3 grid(H, slabs);
        if (dn <= 64) hipLaunchKernelGGL(lightning_step_kernel<16>, grid, dim3(256), 0, s, a);
        else if (dn <= 128) hipLaunchKernelGGL(lightning_step_kernel<32>, grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL(lightning_step_kernel<64>, grid, dim3(256), 0, s, a);
        return last_launch_status();
    }
    const int DP = (dn + 15) & ~15;
    const bool side = scratch && T > light_chunk(dn);
    const int C = side ? light_chunk_parallel(dn) : light_chunk(dn);
    const size_t lds = ((size_t)2 * C * (DP + 1) + (size_t)C * LV + (size_t)DP * LV + (size_t)C * (C + 1) + C) * sizeof(float);
    if (lds > 156 * 1024) return NTK_E_SHAPE;
    static bool raised = false;   // (idempotent: a race sets the same attribute twice)
    if (!raised) {
        NTK_HIP_TRY(hipFuncSetAttribute((const void*)lightning_chunk_kernel<64, kWhole>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
        NTK_HIP_TRY(hipFuncSetAttribute((const void*)lightning_chunk_kernel<64, kLocal>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
        NTK_HIP_TRY(hipFuncSetAttribute((const void*)lightning_chunk_kernel<64, kOutputs>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
        NTK_HIP_TRY(hipFuncSetAttribute((const void*)lightning_chunk_kernel<32, kWhole>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
        NTK_HIP_TRY(hipFuncSetAttribute((const void*)lightning_chunk_kernel<32, kLocal>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
        NTK_HIP_TRY(hipFuncSetAttribute((const void*)lightning_chunk_kernel<32, kOutputs>, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
        raised = true;
    }
    if (!side) {
        const dim3 grid(H, slabs);
        if (C == 64) hipLaunchKernelGGL((lightning_chunk_kernel<64, kWhole>), grid, dim3(256), lds, s, a);
        else hipLaunchKernelGGL((lightning_chunk_kernel<32, kWhole>), grid, dim3(256), lds, s, a);
        return last_launch_status();
    }
    const dim3 grid(H, slabs, (T + C - 1) / C);
    const unsigned scan_blocks = (unsigned)(((long long)H * dn * dv + 255) / 256);
    if (C == 64) {
        hipLaunchKernelGGL((lightning_chunk_kernel<64, kLocal>), grid, dim3(256), lds, s, a);
        hipLaunchKernelGGL(lightning_scan_kernel<64>, dim3(scan_blocks), dim3(256), 0, s, a);
        hipLaunchKernelGGL((lightning_chunk_kernel<64, kOutputs>), grid, dim3(256), lds, s, a);
    } else {
        hipLaunchKernelGGL((lightning_chunk_kernel<32, kLocal>), grid, dim3(256), lds, s, a);
        hipLaunchKernelGGL(lightning_scan_kernel<32>, dim3(scan_blocks), dim3(256), 0, s, a);
        hipLaunchKernelGGL((lightning_chunk_kernel<32, kOutputs>), grid, dim3(256), lds, s, a);
    }
    return last_launch_status();
}
