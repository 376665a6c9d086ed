// layer_ops.hip -- the small F32 operators around the products of the layer-list families: dense embedding rows, RMS norms whose weight is stored
// plain or around zero (two outputs from one pass over x: the two norms of a parallel layer read the same residual row), layer norms with weight and
// bias (also added onto the stream), the short causal convolution that is added to a sublayer's input (with its carried inputs), the polynomial
// activation with unit-norm terms, the gated RMS norm, row concatenation, sigmoid gates, the residual sum.  Everything is F32; one workgroup per row
// where a row is reduced.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

template <typename TT>
__global__ __launch_bounds__(256) void embed_dense_kernel(float* out, const TT* table, const int* tokens, int vocab, int width, float scale) {
    const int t = blockIdx.x, tok = tokens[t];
    float* o = out + (long long)t * width;
    const bool ok = tok >= 0 && tok < vocab;
    const TT* row = table + (long long)(ok ? tok : 0) * width;
    for (int i = threadIdx.x; i < width; i += 256) {
        float v = 0.0f;
        if (ok) {
            if constexpr (sizeof(TT) == 2) v = __uint_as_float((uint32_t)row[i] << 16); else v = row[i];
        }
        o[i] = v * scale;
    }
}

__global__ __launch_bounds__(256) void rmsnorm_offset_kernel(float* y1, const float* w1, float* y2, const float* w2, int ldy, const float* x, int ldx, int n,
                                                             float eps, float offset) {
    __shared__ float red[16];
    const float* xr = x + (long long)blockIdx.x * ldx;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) ss = fmaf(xr[i], xr[i], ss);
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    float* o1 = y1 + (long long)blockIdx.x * ldy;
    float* o2 = y2 ? y2 + (long long)blockIdx.x * ldy : nullptr;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float u = xr[i] * inv;
        o1[i] = u * (offset + w1[i]);
        if (o2) o2[i] = u * (offset + w2[i]);
    }
}

__global__ void concat_rows_kernel(float* out, const float* a, const float* b, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= 2 * n) return;
    out[t * 2 * n + i] = i < n ? a[t * n + i] : b[t * n + (i - n)];
}

__global__ void sigmoid_gate_kernel(float* y, int ldy, const float* g, int ldg, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    y[t * ldy + i] *= 1.0f / (1.0f + expf(-g[t * ldg + i]));
}

__global__ void rows_copy_kernel(float* dst, const float* src, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

__global__ void residual_add_kernel(float* x, const float* a, const float* b, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = a[i];
    if (b) s += b[i];
    x[i] += s;
}

__global__ void scale_kernel(float* x, long long n, float s) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] *= s;
}

// mean first, then the mean of the squared deviations (the row is read again: it sits in the cache), then the outputs
__device__ __forceinline__ void layernorm_row(float* y, const float* xr, const float* w, const float* b, int n, float eps, bool accumulate, float* red) {
    float s = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) s += xr[i];
    const float mean = block_sum(s, red) / (float)n;
    float v = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) { const float d = xr[i] - mean; v = fmaf(d, d, v); }
    const float inv = 1.0f / sqrtf(block_sum(v, red) / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += 256) {
        float o = (xr[i] - mean) * inv * w[i];
        if (b) o += b[i];
        y[i] = accumulate ? y[i] + o : o;
    }
}

__global__ __launch_bounds__(256) void layernorm_kernel(float* y, int ldy, const float* x, int ldx, const float* w, const float* b, int n, float eps, int accumulate) {
    __shared__ float red[16];
    layernorm_row(y + (long long)blockIdx.x * ldy, x + (long long)blockIdx.x * ldx, w, b, n, eps, accumulate != 0, red);
}

// rows 0 .. taps-2: the carried inputs (zeros before the sequence's start); rows taps-1 ..: the layer norm of the portion's tokens
__global__ __launch_bounds__(256) void layernorm_history_kernel(float* hist, const float* x, int ldx, const float* w, const float* b, const float* state, int taps,
                                                                int pos0, int n, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    float* o = hist + (long long)r * n;
    if (r < taps - 1) {
        const bool before = pos0 - (taps - 1) + r < 0;
        for (int i = threadIdx.x; i < n; i += 256) o[i] = before ? 0.0f : state[(long long)r * n + i];
        return;
    }
    layernorm_row(o, x + (long long)(r - (taps - 1)) * ldx, w, b, n, eps, false, red);
}

// blocks y < T: out[y] = hist[taps-1+y] + sum_j w[:, j] * hist[y+j] (j ascending); blocks y >= T: the carried rows for the next portion
__global__ void causal_conv_mix_kernel(float* out, int ldo, const float* hist, const float* w, float* state, int taps, int T, int n) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, y = blockIdx.y;
    if (c >= n) return;
    if (y >= T) { state[(long long)(y - T) * n + c] = hist[(long long)y * n + c]; return; }
    float s = 0.0f;
    for (int j = 0; j < taps; ++j) s = fmaf(w[(long long)c * taps + j], hist[(long long)(y + j) * n + c], s);
    out[(long long)y * ldo + c] = hist[(long long)(y + taps - 1) * n + c] + s;
}

__global__ __launch_bounds__(256) void polynorm_kernel(float* y, int ldy, const float* z, int ldz, const float* coef, int n, float eps) {
    __shared__ float red[16];
    const float* zr = z + (long long)blockIdx.x * ldz;
    float s2 = 0.0f, s4 = 0.0f, s6 = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float v = zr[i], v2 = v * v, v3 = v2 * v;
        s2 += v2; s4 = fmaf(v2, v2, s4); s6 = fmaf(v3, v3, s6);
    }
    s2 = block_sum(s2, red); s4 = block_sum(s4, red); s6 = block_sum(s6, red);
    const float i1 = coef[0] / sqrtf(s2 / (float)n + eps), i2 = coef[1] / sqrtf(s4 / (float)n + eps), i3 = coef[2] / sqrtf(s6 / (float)n + eps), e = coef[3];
    float* o = y + (long long)blockIdx.x * ldy;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float v = zr[i], v2 = v * v, v3 = v2 * v;
        o[i] = i1 * v + i2 * v2 + i3 * v3 + e;
    }
}

__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(float* y, int ldy, const float* x, int ldx, const float* w, const float* g, int ldg, int n, float eps) {
    __shared__ float red[16];
    const float* xr = x + (long long)blockIdx.x * ldx;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) ss = fmaf(xr[i], xr[i], ss);
    const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)n + eps);
    float* o = y + (long long)blockIdx.x * ldy;
    for (int i = threadIdx.x; i < n; i += 256) {
        float v = xr[i] * inv * w[i];
        if (g) v *= 1.0f / (1.0f + expf(-g[(long long)blockIdx.x * ldg + i]));
        o[i] = v;
    }
}

}  // namespace ntk

using namespace ntk;

int ntk_embed_dense(float* out, const void* table, int tdtype, const int* tokens, int T, int vocab, int width, void* stream) {
    return ntk_embed_dense_scaled(out, table, tdtype, tokens, T, vocab, width, 1.0f, stream);
}

int ntk_embed_dense_scaled(float* out, const void* table, int tdtype, const int* tokens, int T, int vocab, int width, float scale, void* stream) {
    if (!out || !table || !tokens) return NTK_E_NULL;
    if (T < 0 || vocab <= 0 || width <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    if (tdtype == NTK_DT_BF16) hipLaunchKernelGGL(embed_dense_kernel<uint16_t>, dim3(T), dim3(256), 0, resolve_stream(stream), out, (const uint16_t*)table, tokens, vocab, width, scale);
    else if (tdtype == NTK_DT_F32) hipLaunchKernelGGL(embed_dense_kernel<float>, dim3(T), dim3(256), 0, resolve_stream(stream), out, (const float*)table, tokens, vocab, width, scale);
    else return NTK_E_DTYPE;
    return last_launch_status();
}

int ntk_rmsnorm_offset(float* y1, const float* w1, float* y2, const float* w2, int ldy, const float* x, int ldx, int T, int n, float eps, float offset,
                       void* stream) {
    if (!y1 || !w1 || !x || (y2 && !w2)) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldx < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(rmsnorm_offset_kernel, dim3(T), dim3(256), 0, resolve_stream(stream), y1, w1, y2, w2, ldy, x, ldx, n, eps, offset);
    return last_launch_status();
}

int ntk_concat_rows(float* out, const float* a, const float* b, int T, int n, void* stream) {
    if (!out || !a || !b) return NTK_E_NULL;
    if (T < 0 || n <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(concat_rows_kernel, dim3((2 * n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), out, a, b, n);
    return last_launch_status();
}

int ntk_sigmoid_gate(float* y, int ldy, const float* g, int ldg, int T, int n, void* stream) {
    if (!y || !g) return NTK_E_NULL;
    if (T < 0 || n <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(sigmoid_gate_kernel, dim3((n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), y, ldy, g, ldg, n);
    return last_launch_status();
}

int ntk_rows_copy(float* dst, const float* src, long long n, void* stream) {
    if (!dst || !src) return NTK_E_NULL;
    if (n < 0 || n > (1ll << 38)) return NTK_E_SHAPE;
    if (n == 0) return NTK_OK;
    hipLaunchKernelGGL(rows_copy_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, resolve_stream(stream), dst, src, n);
    return last_launch_status();
}

int ntk_residual_add(float* x, const float* a, const float* b, int n, void* stream) {
    if (!x || !a) return NTK_E_NULL;
    if (n < 0) return NTK_E_SHAPE;
    if (n == 0) return NTK_OK;
    hipLaunchKernelGGL(residual_add_kernel, dim3((n + 255) / 256), dim3(256), 0, resolve_stream(stream), x, a, b, n);
    return last_launch_status();
}

int ntk_scale(float* x, long long n, float s, void* stream) {
    if (!x) return NTK_E_NULL;
    if (n < 0 || n > (1ll << 38)) return NTK_E_SHAPE;
    if (n == 0) return NTK_OK;
    hipLaunchKernelGGL(scale_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, resolve_stream(stream), x, n, s);
    return last_launch_status();
}

int ntk_layernorm(float* y, int ldy, const float* x, int ldx, const float* w, const float* b, int T, int n, float eps, int accumulate, void* stream) {
    if (!y || !x || !w) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldx < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(layernorm_kernel, dim3(T), dim3(256), 0, resolve_stream(stream), y, ldy, x, ldx, w, b, n, eps, accumulate);
    return last_launch_status();
}

int ntk_layernorm_history(float* hist, const float* x, int ldx, const float* w, const float* b, const float* state, int taps, int pos0, int T, int n, float eps,
                          void* stream) {
    if (!hist || !x || !w || (taps > 1 && !state)) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldx < n || taps < 1 || pos0 < 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(layernorm_history_kernel, dim3(T + taps - 1), dim3(256), 0, resolve_stream(stream), hist, x, ldx, w, b, state, taps, pos0, n, eps);
    return last_launch_status();
}

int ntk_causal_conv_mix(float* out, int ldo, const float* hist, const float* w, float* state, int taps, int T, int n, void* stream) {
    if (!out || !hist || !w || (taps > 1 && !state)) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldo < n || taps < 1) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(causal_conv_mix_kernel, dim3((n + 255) / 256, T + taps - 1), dim3(256), 0, resolve_stream(stream), out, ldo, hist, w, state, taps, T, n);
    return last_launch_status();
}

int ntk_polynorm(float* y, int ldy, const float* z, int ldz, const float* coef, int T, int n, float eps, void* stream) {
    if (!y || !z || !coef) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldz < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(polynorm_kernel, dim3(T), dim3(256), 0, resolve_stream(stream), y, ldy, z, ldz, coef, n, eps);
    return last_launch_status();
}

int ntk_gated_rmsnorm(float* y, int ldy, const float* x, int ldx, const float* w, const float* g, int ldg, int T, int n, float eps, void* stream) {
    if (!y || !x || !w) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldx < n || (g && ldg < n)) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(gated_rmsnorm_kernel, dim3(T), dim3(256), 0, resolve_stream(stream), y, ldy, x, ldx, w, g, ldg, n, eps);
    return last_launch_status();
}
