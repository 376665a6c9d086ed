// dense.hip -- products with dense weight matrices (bfloat16 or float32, row-major [out][in]) for the layer-list model families.
//
// One entry point (ntk_dense) and three kernel forms behind it:
//   * dense_mfma_kernel   bf16 weights, more than kGemvRows rows: 64 x 64 output tiles on v_mfma_f32_16x16x32_bf16; the F32 activations are rounded
//                         to bfloat16 (nearest even) on their way into LDS, sums stay F32 in the accumulators;
//   * dense_fma_kernel    float32 weights, more than kGemvRows rows: the same tiling with plain F32 FMAs, k ascending (true 32-bit);
//   * dense_gemv_kernel   up to kGemvRows rows (decoding): one wave per output row streams the weight row once, 16 bytes per lane, the activation
//                         row sits in LDS; bf16 weights are widened exactly and multiplied in F32.
// Rows can be grouped (a mixture of experts: sorted rows of group g take matrix g) and gathered (row r reads activation row rows[r] / row_div).
// Group sizes live on the device, so the grid covers the worst case and workgroups outside their group's range leave at once.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint16_t f2bf(float f) {   // round to nearest even; NaN stays NaN
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float bf2f(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

struct DenseArgs {
    float* Y; int ldy;
    const float* X; int ldx;
    const void* W; long long wstride;
    const int* offsets;
    const int* rows; int row_div;
    int T, N, K, accumulate, G, vec;
};

__device__ __forceinline__ bool group_range(const DenseArgs& a, int g, int& r0, int& r1) {
    if (a.offsets) { r0 = a.offsets[g]; r1 = a.offsets[g + 1]; } else { r0 = 0; r1 = a.T; }
    return r1 > r0;
}

// ---------------------------------------------------------------------------------------------------------------- bf16, matrix cores
constexpr int TM = 64, TN = 64, BK = 32, LDSK = BK + 8;   // LDS rows of 40 bf16 = 80 bytes: 16-byte aligned operand reads

template <bool VEC>
__global__ __launch_bounds__(256) void dense_mfma_kernel(const DenseArgs a) {
    int r0, r1;
    if (!group_range(a, blockIdx.z, r0, r1)) return;
    const int row_base = r0 + blockIdx.y * TM;
    if (row_base >= r1) return;
    const int n_base = blockIdx.x * TN;
    const uint16_t* W = (const uint16_t*)a.W + (long long)blockIdx.z * a.wstride;
    __shared__ __attribute__((aligned(16))) uint16_t Xs[TM][LDSK];
    __shared__ __attribute__((aligned(16))) uint16_t Ws[TN][LDSK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    // loader: thread -> (row tid / 4, eight k from (tid & 3) * 8)
    const int lr = tid >> 2, lk = (tid & 3) * 8;
    const int xr = row_base + lr;
    const bool x_ok = xr < r1;
    const float* xrow = nullptr;
    if (x_ok) xrow = a.X + (long long)(a.rows ? a.rows[xr] / a.row_div : xr) * a.ldx;
    const int wr = n_base + lr;
    const bool w_ok = wr < a.N;
    const uint16_t* wrow = W + (long long)wr * a.K;
    floatx4_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < a.K; k0 += BK) {
        uint16_t xb[8], wb[8];
        const int k = k0 + lk;
        if (VEC) {
            if (x_ok && k < a.K) {
                const float4 v0 = *reinterpret_cast<const float4*>(xrow + k), v1 = *reinterpret_cast<const float4*>(xrow + k + 4);
                xb[0] = f2bf(v0.x); xb[1] = f2bf(v0.y); xb[2] = f2bf(v0.z); xb[3] = f2bf(v0.w);
                xb[4] = f2bf(v1.x); xb[5] = f2bf(v1.y); xb[6] = f2bf(v1.z); xb[7] = f2bf(v1.w);
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) xb[j] = 0;
            }
            if (w_ok && k < a.K) *reinterpret_cast<uint4*>(wb) = *reinterpret_cast<const uint4*>(wrow + k);
            else *reinterpret_cast<uint4*>(wb) = uint4{0u, 0u, 0u, 0u};
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                xb[j] = (x_ok && k + j < a.K) ? f2bf(xrow[k + j]) : (uint16_t)0;
                wb[j] = (w_ok && k + j < a.K) ? wrow[k + j] : (uint16_t)0;
            }
        }
        __syncthreads();   // the previous chunk's operand reads are done
        *reinterpret_cast<uint4*>(&Xs[lr][lk]) = *reinterpret_cast<const uint4*>(xb);
        *reinterpret_cast<uint4*>(&Ws[lr][lk]) = *reinterpret_cast<const uint4*>(wb);
        __syncthreads();
        bf16x8_t af[2], bfr[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            af[i] = *reinterpret_cast<const bf16x8_t*>(&Xs[wm * 32 + i * 16 + (lane & 15)][(lane >> 4) * 8]);
            bfr[i] = *reinterpret_cast<const bf16x8_t*>(&Ws[wn * 32 + i * 16 + (lane & 15)][(lane >> 4) * 8]);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    // accumulator lane map: row 4 * (lane / 16) + r, column lane % 16
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = row_base + wm * 32 + i * 16 + (lane >> 4) * 4 + r, col = n_base + wn * 32 + j * 16 + (lane & 15);
                if (row < r1 && col < a.N) {
                    float* y = a.Y + (long long)row * a.ldy + col;
                    *y = a.accumulate ? *y + acc[i][j][r] : acc[i][j][r];
                }
            }
}

// ---------------------------------------------------------------------------------------------------------------- float32, vector FMA
constexpr int FK = 16;
__global__ __launch_bounds__(256) void dense_fma_kernel(const DenseArgs a) {
    int r0, r1;
    if (!group_range(a, blockIdx.z, r0, r1)) return;
    const int row_base = r0 + blockIdx.y * TM;
    if (row_base >= r1) return;
    const int n_base = blockIdx.x * TN;
    const float* W = (const float*)a.W + (long long)blockIdx.z * a.wstride;
    __shared__ __attribute__((aligned(16))) float Xs[FK][TM + 4];
    __shared__ __attribute__((aligned(16))) float Ws[FK][TN + 4];
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    const int lr = tid >> 2, lk = (tid & 3) * 4;
    const int xr = row_base + lr;
    const bool x_ok = xr < r1;
    const float* xrow = nullptr;
    if (x_ok) xrow = a.X + (long long)(a.rows ? a.rows[xr] / a.row_div : xr) * a.ldx;
    const int wr = n_base + lr;
    const bool w_ok = wr < a.N;
    const float* wrow = W + (long long)wr * a.K;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < a.K; k0 += FK) {
        float xv[4], wv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            xv[j] = (x_ok && k < a.K) ? xrow[k] : 0.0f;
            wv[j] = (w_ok && k < a.K) ? wrow[k] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) { Xs[lk + j][lr] = xv[j]; Ws[lk + j][lr] = wv[j]; }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < FK; ++k) {
            const float4 xa = *reinterpret_cast<const float4*>(&Xs[k][ty * 4]);
            const float4 wa = *reinterpret_cast<const float4*>(&Ws[k][tx * 4]);
            const float xs[4] = {xa.x, xa.y, xa.z, xa.w}, ws[4] = {wa.x, wa.y, wa.z, wa.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(xs[i], ws[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = row_base + ty * 4 + i, col = n_base + tx * 4 + j;
            if (row < r1 && col < a.N) {
                float* y = a.Y + (long long)row * a.ldy + col;
                *y = a.accumulate ? *y + acc[i][j] : acc[i][j];
            }
        }
}

// ---------------------------------------------------------------------------------------------------------------- few rows: one wave per output
constexpr int kGemvRows = 8;       // up to this many rows take the GEMV form
constexpr int kGemvOut = 16;       // outputs per workgroup (4 waves x 4)
template <typename WT>
__global__ __launch_bounds__(256) void dense_gemv_kernel(const DenseArgs a) {
    extern __shared__ __attribute__((aligned(16))) float xs[];   // the activation row
    const int r = blockIdx.y;
    int g = 0;
    if (a.offsets) {
        if (r >= a.offsets[a.G]) return;
        while (r >= a.offsets[g + 1]) ++g;
    }
    const float* xrow = a.X + (long long)(a.rows ? a.rows[r] / a.row_div : r) * a.ldx;
    for (int k = threadIdx.x; k < a.K; k += 256) xs[k] = xrow[k];
    __syncthreads();
    const WT* W = (const WT*)a.W + (long long)g * a.wstride;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const bool vec = a.vec != 0;
    for (int o = 0; o < kGemvOut / 4; ++o) {
        const int n = blockIdx.x * kGemvOut + wave * (kGemvOut / 4) + o;
        if (n >= a.N) break;                             // uniform per wave
        const WT* w = W + (long long)n * a.K;
        float s = 0.0f;
        if (vec) {
            for (int k = lane * 8; k < a.K; k += 64 * 8) {
                float wv[8];
                if constexpr (sizeof(WT) == 2) {
                    const uint4 u = *reinterpret_cast<const uint4*>(w + k);
                    const uint32_t uu[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) { wv[2 * j] = __uint_as_float(uu[j] << 16); wv[2 * j + 1] = __uint_as_float(uu[j] & 0xffff0000u); }
                } else {
                    const float4 u0 = *reinterpret_cast<const float4*>(w + k), u1 = *reinterpret_cast<const float4*>(w + k + 4);
                    wv[0] = u0.x; wv[1] = u0.y; wv[2] = u0.z; wv[3] = u0.w; wv[4] = u1.x; wv[5] = u1.y; wv[6] = u1.z; wv[7] = u1.w;
                }
                const float4 x0 = *reinterpret_cast<const float4*>(xs + k), x1 = *reinterpret_cast<const float4*>(xs + k + 4);
                s = fmaf(wv[0], x0.x, s); s = fmaf(wv[1], x0.y, s); s = fmaf(wv[2], x0.z, s); s = fmaf(wv[3], x0.w, s);
                s = fmaf(wv[4], x1.x, s); s = fmaf(wv[5], x1.y, s); s = fmaf(wv[6], x1.z, s); s = fmaf(wv[7], x1.w, s);
            }
        } else {
            for (int k = lane; k < a.K; k += 64) {
                float wv;
                if constexpr (sizeof(WT) == 2) wv = bf2f(((const uint16_t*)w)[k]); else wv = ((const float*)w)[k];
                s = fmaf(wv, xs[k], s);
            }
        }
        s = wave_sum_lane63(s);
        if (lane == 63) {
            float* y = a.Y + (long long)r * a.ldy + n;
            *y = a.accumulate ? *y + s : s;
        }
    }
}

}  // namespace ntk

using namespace ntk;

int ntk_dense(const ntk_dense_desc* d, void* stream) {
    if (!d || !d->Y || !d->X || !d->W) return NTK_E_NULL;
    if (d->wdtype != NTK_DT_BF16 && d->wdtype != NTK_DT_F32) return NTK_E_DTYPE;
    if (d->T < 0 || d->N <= 0 || d->K <= 0 || d->ldx < d->K || d->ldy < d->N) return NTK_E_SHAPE;
    if (d->offsets && d->G <= 0) return NTK_E_SHAPE;
    if (d->rows && d->row_div <= 0) return NTK_E_SHAPE;
    if (d->T == 0) return NTK_OK;
    const int G = d->offsets ? d->G : 1;
    DenseArgs a{d->Y, d->ldy, d->X, d->ldx, d->W, d->wstride, d->offsets, d->rows, d->rows ? d->row_div : 1, d->T, d->N, d->K, d->accumulate, G, 0};
    hipStream_t s = resolve_stream(stream);
    if (d->T <= kGemvRows) {
        if ((size_t)d->K * 4 > 160 * 1024 - 1024) return NTK_E_SHAPE;
        a.vec = (d->K % 8 == 0) && !((uintptr_t)d->W & 15) && !((d->wstride * (d->wdtype == NTK_DT_BF16 ? 2 : 4)) & 15);
        const dim3 grid((d->N + kGemvOut - 1) / kGemvOut, d->T, 1);
        const size_t lds = ((size_t)d->K * 4 + 15) & ~(size_t)15;
        if (d->wdtype == NTK_DT_BF16) hipLaunchKernelGGL(dense_gemv_kernel<uint16_t>, grid, dim3(256), lds, s, a);
        else hipLaunchKernelGGL(dense_gemv_kernel<float>, grid, dim3(256), lds, s, a);
        return last_launch_status();
    }
    const dim3 grid((d->N + TN - 1) / TN, (d->T + TM - 1) / TM, G);
    if (d->wdtype == NTK_DT_BF16) {
        const bool vec = (d->K % 8 == 0) && (d->ldx % 4 == 0) && !((uintptr_t)d->X & 15) && !((uintptr_t)d->W & 15) && (d->wstride % 8 == 0);
        if (vec) hipLaunchKernelGGL(dense_mfma_kernel<true>, grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL(dense_mfma_kernel<false>, grid, dim3(256), 0, s, a);
    } else {
        hipLaunchKernelGGL(dense_fma_kernel, grid, dim3(256), 0, s, a);
    }
    return last_launch_status();
}

int ntk_dense_linear(float* Y, int ldy, const float* X, int ldx, const void* W, int wdtype, int T, int N, int K, int accumulate, void* stream) {
    ntk_dense_desc d{};
    d.Y = Y; d.ldy = ldy; d.X = X; d.ldx = ldx; d.W = W; d.wstride = 0; d.wdtype = wdtype; d.offsets = nullptr; d.G = 1; d.rows = nullptr; d.row_div = 1;
    d.T = T; d.N = N; d.K = K; d.accumulate = accumulate;
    return ntk_dense(&d, stream);
}
