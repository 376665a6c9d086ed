// latent_attention.hip -- attention over a cache of one normed latent and one rotated key part per position.
//
// What is cached per position and layer run is [latent c (kv_rank) | rotated key part (rot_dim)], F32.  Two ways to the same sums:
//   * expanded (prompt portions): the caller up-projects the cached latents of the visible range into per-head keys and values (two products over
//     the cache rows) and the kernel runs ordinary multi-head attention on them, reading the shared rotated part from the cache rows;
//   * shared (few query tokens, decoding): the query's unrotated part is folded through the key up-projection first (ntk_latent_fold_query), so every
//     head scores against the cache rows themselves, [c | rotated] . [folded q | rotated q]; the weighted sum is taken over c and the value
//     up-projection is applied once afterwards (ntk_latent_unfold_value).  Nothing per head is ever materialised for the cached positions.
// Both are one kernel: a workgroup owns 16 query rows (tokens of one head / (token, head) pairs) and walks the visible keys in chunks of 64:
// lane = key for the scores (key slab of 64 dims at a time in LDS), online softmax per row in F32, lane = value column for the weighted sum.
// With splits > 1 the chunks go round the splits and a second launch merges the partial (max, sum, vector) states.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

// ------------------------------------------------------------------------------------------------------------------- cache rows and rotation
// one workgroup per token: latent / rms * w and the rotated key part into the cache row, the rotated part of every query head in place.
// Angles in double (position times frequency, then cos / sin), applied in F32.
__global__ __launch_bounds__(256) void latent_prepare_kernel(float* cache, int row, const float* kv, int ldkv, const float* norm_w, float eps, int R, int dr,
                                                             float* q, int ldq, int H, int qd, const double* freq, float mag, int dims, int pos0) {
    __shared__ float red[16];
    extern __shared__ float cs[];   // [dims / 2] cos, [dims / 2] sin
    const int t = blockIdx.x, pos = pos0 + t;
    const float* src = kv + (long long)t * ldkv;
    float* dst = cache + (long long)pos * row;
    const int half = dims / 2;   // dims <= dr: what lies behind the rotated entries passes unchanged
    for (int i = threadIdx.x; i < half; i += 256) {
        const double a = (double)pos * freq[i];
        cs[i] = (float)(cos(a) * (double)mag);
        cs[half + i] = (float)(sin(a) * (double)mag);
    }
    float ss = 0.0f;
    for (int i = threadIdx.x; i < R; i += 256) ss = fmaf(src[i], src[i], ss);
    ss = block_sum(ss, red);   // (its barriers also publish cs)
    const float inv = 1.0f / sqrtf(ss / (float)R + eps);
    for (int i = threadIdx.x; i < R; i += 256) dst[i] = src[i] * inv * norm_w[i];
    for (int i = threadIdx.x; i < half; i += 256) {
        float ra, rb;
        rope_rotate(src[R + 2 * i], src[R + 2 * i + 1], cs[i], cs[half + i], ra, rb);
        dst[R + 2 * i] = ra;
        dst[R + 2 * i + 1] = rb;
    }
    for (int i = dims + threadIdx.x; i < dr; i += 256) dst[R + i] = src[R + i];
    if (q) {
        float* qt = q + (long long)t * ldq;
        for (int j = threadIdx.x; j < H * half; j += 256) {
            const int h = j / half, i = j % half;
            float* p = qt + h * qd + (qd - dr) + 2 * i;
            float ra, rb;
            rope_rotate(p[0], p[1], cs[i], cs[half + i], ra, rb);
            p[0] = ra;
            p[1] = rb;
        }
    }
}

// ------------------------------------------------------------------------------------------------------------------- the attention kernel
struct AttnArgs {
    float* out; int ldo;              // per token
    const float* q; int ldq;          // per token; head h at h * DK
    const float* kA; long long ldA; int nA; int hA;   // first part of a key: kA + (j - keyA0) * ldA + h * hA, nA entries
    const float* kB; long long ldB; int nB;           // second part: kB + j * ldB, nB entries (the rotated part inside the cache row)
    const float* v; long long ldV; int nV; int hV;    // value: v + (j - keyA0) * ldV + h * hV
    int keyA0;
    int H, shared, pos0, T, window;
    float scale;
    int splits; float* scratch;       // splits > 1: partial states [row][split][2 + nV]
};

constexpr int QROWS = 16, QPW = 4, KCH = 64, SLAB = 64;

__global__ __launch_bounds__(256) void latent_attention_kernel(const AttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int DK = a.nA + a.nB;
    const int DKP = (DK + 3) & ~3;
    float* Qs = lds;                               // [QROWS][DKP]
    float* Sl = Qs + QROWS * DKP;                  // [KCH][SLAB + 1] key slab / [KCH][SLAB] value slab
    float* Ps = Sl + KCH * (SLAB + 1);             // [QROWS][KCH]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // rows of this workgroup
    int head, n_rows_total;
    if (a.shared) { head = 0; n_rows_total = a.T * a.H; } else { head = blockIdx.y; n_rows_total = a.T; }
    const int row0 = blockIdx.x * QROWS;
    auto row_token = [&](int i) { const int r = row0 + i; return a.shared ? r / a.H : r; };
    auto row_head = [&](int i) { const int r = row0 + i; return a.shared ? r % a.H : head; };
    const int last_row = min(row0 + QROWS, n_rows_total) - 1;
    const int pmin = a.pos0 + (a.shared ? row0 / a.H : row0);
    const int pmax = a.pos0 + (a.shared ? last_row / a.H : last_row);
    const int jlo = a.window > 0 ? max(0, pmin - a.window + 1) : 0;
    const int jhi = pmax;   // inclusive
    // queries into LDS
    for (int idx = threadIdx.x; idx < QROWS * DKP; idx += 256) {
        const int i = idx / DKP, d = idx % DKP;
        float v = 0.0f;
        if (row0 + i < n_rows_total && d < DK) v = a.q[(long long)row_token(i) * a.ldq + (long long)row_head(i) * DK + d];
        Qs[idx] = v;
    }
    float m[QPW], l[QPW], acc[QPW][8];
    int rpos[QPW];
#pragma unroll
    for (int i = 0; i < QPW; ++i) {
        m[i] = -INFINITY; l[i] = 0.0f;
        const int ri = wave * QPW + i;
        rpos[i] = row0 + ri < n_rows_total ? a.pos0 + row_token(ri) : -1;
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[i][c] = 0.0f;
    }
    const int hk = a.shared ? 0 : head;
    int chunk = 0;
    for (int j0 = jlo; j0 <= jhi; j0 += KCH, ++chunk) {
        if (a.splits > 1 && chunk % a.splits != (int)blockIdx.z) continue;
        const int nk = min(KCH, jhi + 1 - j0);
        float s[QPW];
#pragma unroll
        for (int i = 0; i < QPW; ++i) s[i] = 0.0f;
        // ---- scores: slabs of SLAB key entries
        for (int d0 = 0; d0 < DK; d0 += SLAB) {
            const int nd = min(SLAB, DK - d0);
            __syncthreads();
            for (int idx = threadIdx.x; idx < KCH * SLAB; idx += 256) {
                const int k = idx / SLAB, d = idx % SLAB;
                float v = 0.0f;
                if (k < nk && d < nd) {
                    const int dd = d0 + d, j = j0 + k;
                    v = dd < a.nA ? a.kA[(long long)(j - a.keyA0) * a.ldA + (long long)hk * a.hA + dd] : a.kB[(long long)j * a.ldB + (dd - a.nA)];
                }
                Sl[k * (SLAB + 1) + d] = v;
            }
            __syncthreads();
            const float* kr = Sl + lane * (SLAB + 1);
            for (int d = 0; d < nd; ++d) {
                const float kvv = kr[d];
#pragma unroll
                for (int i = 0; i < QPW; ++i) s[i] = fmaf(Qs[(wave * QPW + i) * DKP + d0 + d], kvv, s[i]);
            }
        }
        // ---- online softmax, weights to LDS
        const int j = j0 + lane;
#pragma unroll
        for (int i = 0; i < QPW; ++i) {
            const bool vis = lane < nk && rpos[i] >= 0 && j <= rpos[i] && (a.window <= 0 || rpos[i] - j < a.window);
            const float sv = vis ? s[i] * a.scale : -INFINITY;
            const float mn = fmaxf(m[i], wave_max(sv));
            const float ms = mn == -INFINITY ? 0.0f : mn;
            const float p = vis ? expf(sv - ms) : 0.0f;
            const float corr = m[i] == -INFINITY ? 0.0f : expf(m[i] - ms);
            l[i] = l[i] * corr + wave_sum(p);
            m[i] = mn;
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[i][c] *= corr;
            Ps[(wave * QPW + i) * KCH + lane] = p;
        }
        // ---- weighted sum: slabs of SLAB value columns, lane = column
        const int hv = a.shared ? 0 : head;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int v0 = c * SLAB;
            if (v0 < a.nV) {
                const int nvv = min(SLAB, a.nV - v0);
                __syncthreads();
                for (int idx = threadIdx.x; idx < KCH * SLAB; idx += 256) {
                    const int k = idx / SLAB, d = idx % SLAB;
                    float v = 0.0f;
                    if (k < nk && d < nvv) v = a.v[(long long)(j0 + k - a.keyA0) * a.ldV + (long long)hv * a.hV + v0 + d];
                    Sl[k * SLAB + d] = v;
                }
                __syncthreads();
                for (int k = 0; k < nk; ++k) {
                    const float vv = Sl[k * SLAB + lane];
#pragma unroll
                    for (int i = 0; i < QPW; ++i) acc[i][c] = fmaf(Ps[(wave * QPW + i) * KCH + k], vv, acc[i][c]);
                }
            }
        }
    }
    // ---- results
#pragma unroll
    for (int i = 0; i < QPW; ++i) {
        const int ri = wave * QPW + i;
        if (row0 + ri >= n_rows_total) continue;
        const int t = row_token(ri), h = row_head(ri);
        if (a.splits > 1) {
            float* st = a.scratch + ((long long)(row0 + ri) * a.splits + blockIdx.z) * (2 + a.nV);   // (splits only in the shared form: row = t * H + h)
            if (lane == 0) { st[0] = m[i]; st[1] = l[i]; }
#pragma unroll
            for (int c = 0; c < 8; ++c)
                if (c * SLAB + lane < a.nV) st[2 + c * SLAB + lane] = acc[i][c];
        } else {
            const float inv = l[i] > 0.0f ? 1.0f / l[i] : 0.0f;
            float* o = a.out + (long long)t * a.ldo + (long long)h * a.nV;
#pragma unroll
            for (int c = 0; c < 8; ++c)
                if (c * SLAB + lane < a.nV) o[c * SLAB + lane] = acc[i][c] * inv;
        }
    }
}

// merge of the partial states of one (token, head): grid (rows), state index = row as the attention kernel numbered it
__global__ __launch_bounds__(64) void latent_attention_merge_kernel(float* out, int ldo, const float* scratch, int splits, int nV, int H) {
    const int r = blockIdx.x;   // shared numbering: r = t * H + h
    const float* st = scratch + (long long)r * splits * (2 + nV);
    float mx = -INFINITY;
    for (int s = 0; s < splits; ++s) mx = fmaxf(mx, st[(long long)s * (2 + nV)]);
    float den = 0.0f;
    for (int s = 0; s < splits; ++s) {
        const float ms = st[(long long)s * (2 + nV)];
        if (ms != -INFINITY) den += st[(long long)s * (2 + nV) + 1] * expf(ms - mx);
    }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    float* o = out + (long long)(r / H) * ldo + (long long)(r % H) * nV;
    for (int v = threadIdx.x; v < nV; v += 64) {
        float s2 = 0.0f;
        for (int s = 0; s < splits; ++s) {
            const float ms = st[(long long)s * (2 + nV)];
            if (ms != -INFINITY) s2 = fmaf(st[(long long)s * (2 + nV) + 2 + v], expf(ms - mx), s2);
        }
        o[v] = s2 * inv;
    }
}

// ------------------------------------------------------------------------------------------------------------------- fold / unfold
// qf[t][h][r] = sum_d q[t][h][d] W_uk[h * dn + d][r]; rotated part copied behind.  grid (H, T)
template <typename WT>
__global__ __launch_bounds__(256) void latent_fold_query_kernel(float* qf, const float* q, int ldq, const WT* w, int H, int dn, int dr, int R) {
    extern __shared__ float qs[];
    const int h = blockIdx.x, t = blockIdx.y;
    const float* qh = q + (long long)t * ldq + (long long)h * (dn + dr);
    float* o = qf + ((long long)t * H + h) * (R + dr);
    for (int d = threadIdx.x; d < dn + dr; d += 256) qs[d] = qh[d];
    __syncthreads();
    const WT* wh = w + (long long)h * dn * R;
    for (int r = threadIdx.x; r < R; r += 256) {
        float s = 0.0f;
        for (int d = 0; d < dn; ++d) {
            float wv;
            if constexpr (sizeof(WT) == 2) wv = __uint_as_float((uint32_t)wh[(long long)d * R + r] << 16); else wv = wh[(long long)d * R + r];
            s = fmaf(qs[d], wv, s);
        }
        o[r] = s;
    }
    for (int d = threadIdx.x; d < dr; d += 256) o[R + d] = qs[dn + d];
}

// out[t][h * dv + v] = W_uv[h * dv + v][:] . lat[t][h][:] (* sigmoid(gate));  grid (H, T), one wave per output
template <typename WT>
__global__ __launch_bounds__(256) void latent_unfold_value_kernel(float* out, int ldo, const float* lat, const WT* w, const float* gate, int ldg, int H, int dv,
                                                                 int R) {
    extern __shared__ float ls[];
    const int h = blockIdx.x, t = blockIdx.y;
    const float* lh = lat + ((long long)t * H + h) * R;
    for (int r = threadIdx.x; r < R; r += 256) ls[r] = lh[r];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int v = wave; v < dv; v += 4) {
        const WT* wr = w + ((long long)h * dv + v) * R;
        float s = 0.0f;
        for (int r = lane; r < R; r += 64) {
            float wv;
            if constexpr (sizeof(WT) == 2) wv = __uint_as_float((uint32_t)wr[r] << 16); else wv = wr[r];
            s = fmaf(wv, ls[r], s);
        }
        s = wave_sum_lane63(s);
        if (lane == 63) {
            if (gate) s *= 1.0f / (1.0f + expf(-gate[(long long)t * ldg + h * dv + v]));
            out[(long long)t * ldo + h * dv + v] = s;
        }
    }
}

static int attention_splits(int rows, int nkeys) {
    const int blocks = (rows + QROWS - 1) / QROWS, chunks = (nkeys + KCH - 1) / KCH;
    if (blocks >= 128 || chunks < 4) return 1;
    int s = chunks / 2;
    if (s > 32) s = 32;
    while (s > 1 && blocks * s > 1024) --s;
    return s < 1 ? 1 : s;
}

}  // namespace ntk

using namespace ntk;

int ntk_latent_prepare(float* cache, int row, const float* kv, int ldkv, const float* norm_w, float eps, int kv_rank, int rot_dim, float* q, int ldq, int H, int qd,
                       const ntk_rotary* rot, int pos0, int T, void* stream) {
    if (!cache || !kv || !norm_w || !rot || !rot->freq) return NTK_E_NULL;
    if (T < 0 || kv_rank <= 0 || rot_dim < 0 || rot->dims < 0 || (rot->dims & 1) || rot->dims > rot_dim || row < kv_rank + rot_dim || ldkv < kv_rank + rot_dim || pos0 < 0) return NTK_E_SHAPE;
    if (q && (H <= 0 || qd < rot_dim || ldq < H * qd)) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(latent_prepare_kernel, dim3(T), dim3(256), (size_t)(rot_dim + 2) * sizeof(float), resolve_stream(stream), cache, row, kv, ldkv, norm_w,
                       eps, kv_rank, rot_dim, q, ldq, H, qd, rot->freq, rot->mag, rot->dims, pos0);
    return last_launch_status();
}

size_t ntk_latent_attention_scratch(int T, int H, int vdim_or_rank, int nkeys) {
    const int s = attention_splits(T * H, nkeys);
    return s > 1 ? (size_t)T * H * s * (2 + vdim_or_rank) : 0;
}

int ntk_latent_attention(float* out, int ldo, const float* q, int ldq, const float* K, int ldk, const float* V, int ldv, const float* cache, int row,
                         int kv_rank, int rot_dim, int H, int dn, int dv, int shared, int pos0, int T, int key0, int window, float scale, float* scratch,
                         void* stream) {
    if (!out || !q || !cache) return NTK_E_NULL;
    if (!shared && (!K || !V)) return NTK_E_NULL;
    if (T < 0 || H <= 0 || kv_rank <= 0 || rot_dim < 0 || pos0 < 0 || key0 < 0 || row < kv_rank + rot_dim) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    AttnArgs a{};
    a.out = out; a.ldo = ldo; a.q = q; a.ldq = ldq;
    a.kB = cache + kv_rank; a.ldB = row; a.nB = rot_dim;
    a.H = H; a.shared = shared; a.pos0 = pos0; a.T = T; a.window = window; a.scale = scale;
    int rows, nkeys;
    if (shared) {
        a.kA = cache; a.ldA = row; a.nA = kv_rank; a.hA = 0;
        a.v = cache; a.ldV = row; a.nV = kv_rank; a.hV = 0;
        a.keyA0 = 0;
        rows = T * H;
        nkeys = window > 0 ? (window + T < pos0 + T ? window + T : pos0 + T) : pos0 + T;
        a.splits = attention_splits(rows, nkeys);
        if (a.splits > 1 && !scratch) return NTK_E_NULL;
        a.scratch = scratch;
    } else {
        if (dn <= 0 || dv <= 0) return NTK_E_SHAPE;
        a.kA = K; a.ldA = ldk; a.nA = dn; a.hA = dn;
        a.v = V; a.ldV = ldv; a.nV = dv; a.hV = dv;
        a.keyA0 = key0;
        rows = T;
        a.splits = 1;
        a.scratch = nullptr;
    }
    if (a.nV > 8 * SLAB) return NTK_E_SHAPE;
    const int DKP = (a.nA + a.nB + 3) & ~3;
    const size_t lds = ((size_t)QROWS * DKP + KCH * (SLAB + 1) + QROWS * KCH) * sizeof(float);
    if (lds > 150 * 1024) return NTK_E_SHAPE;
    hipStream_t s = resolve_stream(stream);
    const dim3 grid((rows + QROWS - 1) / QROWS, shared ? 1 : H, a.splits);
    if (lds > 48 * 1024) {
        static bool raised = false;   // (idempotent: a race sets the same attribute twice)
        if (!raised) { NTK_HIP_TRY(hipFuncSetAttribute((const void*)latent_attention_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024)); raised = true; }
    }
    hipLaunchKernelGGL(latent_attention_kernel, grid, dim3(256), lds, s, a);
    int st = last_launch_status();
    if (st != NTK_OK) return st;
    if (a.splits > 1) {
        hipLaunchKernelGGL(latent_attention_merge_kernel, dim3(rows), dim3(64), 0, s, out, ldo, (const float*)scratch, a.splits, a.nV, H);
        st = last_launch_status();
    }
    return st;
}

int ntk_latent_fold_query(float* qf, const float* q, int ldq, const void* w_uk, int wdtype, int T, int H, int dn, int dr, int R, void* stream) {
    if (!qf || !q || !w_uk) return NTK_E_NULL;
    if (T < 0 || H <= 0 || dn <= 0 || dr < 0 || R <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    const size_t lds = (size_t)(dn + dr) * sizeof(float);
    if (wdtype == NTK_DT_BF16) hipLaunchKernelGGL(latent_fold_query_kernel<uint16_t>, dim3(H, T), dim3(256), lds, resolve_stream(stream), qf, q, ldq, (const uint16_t*)w_uk, H, dn, dr, R);
    else if (wdtype == NTK_DT_F32) hipLaunchKernelGGL(latent_fold_query_kernel<float>, dim3(H, T), dim3(256), lds, resolve_stream(stream), qf, q, ldq, (const float*)w_uk, H, dn, dr, R);
    else return NTK_E_DTYPE;
    return last_launch_status();
}

int ntk_latent_unfold_value(float* out, int ldo, const float* lat, const void* w_uv, int wdtype, const float* gate, int ldg, int T, int H, int dv, int R,
                            void* stream) {
    if (!out || !lat || !w_uv) return NTK_E_NULL;
    if (T < 0 || H <= 0 || dv <= 0 || R <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    const size_t lds = (size_t)R * sizeof(float);
    if (wdtype == NTK_DT_BF16) hipLaunchKernelGGL(latent_unfold_value_kernel<uint16_t>, dim3(H, T), dim3(256), lds, resolve_stream(stream), out, ldo, lat, (const uint16_t*)w_uv, gate, ldg, H, dv, R);
    else if (wdtype == NTK_DT_F32) hipLaunchKernelGGL(latent_unfold_value_kernel<float>, dim3(H, T), dim3(256), lds, resolve_stream(stream), out, ldo, lat, (const float*)w_uv, gate, ldg, H, dv, R);
    else return NTK_E_DTYPE;
    return last_launch_status();
}
