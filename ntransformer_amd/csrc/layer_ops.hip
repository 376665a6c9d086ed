// layer_ops.hip -- the small F32 operators around the products of the layer-list families: dense embedding rows, RMS norms whose weight is stored
// plain or around zero (two outputs from one pass over x: the two norms of a parallel layer read the same residual row), row concatenation, sigmoid
// gates, the residual sum.  Everything is F32; one workgroup per row where a row is reduced.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

template <typename TT>
__global__ __launch_bounds__(256) void embed_dense_kernel(float* out, const TT* table, const int* tokens, int vocab, int width) {
    const int t = blockIdx.x, tok = tokens[t];
    float* o = out + (long long)t * width;
    const bool ok = tok >= 0 && tok < vocab;
    const TT* row = table + (long long)(ok ? tok : 0) * width;
    for (int i = threadIdx.x; i < width; i += 256) {
        float v = 0.0f;
        if (ok) {
            if constexpr (sizeof(TT) == 2) v = __uint_as_float((uint32_t)row[i] << 16); else v = row[i];
        }
        o[i] = v;
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

}  // namespace ntk

using namespace ntk;

int ntk_embed_dense(float* out, const void* table, int tdtype, const int* tokens, int T, int vocab, int width, void* stream) {
    if (!out || !table || !tokens) return NTK_E_NULL;
    if (T < 0 || vocab <= 0 || width <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    if (tdtype == NTK_DT_BF16) hipLaunchKernelGGL(embed_dense_kernel<uint16_t>, dim3(T), dim3(256), 0, resolve_stream(stream), out, (const uint16_t*)table, tokens, vocab, width);
    else if (tdtype == NTK_DT_F32) hipLaunchKernelGGL(embed_dense_kernel<float>, dim3(T), dim3(256), 0, resolve_stream(stream), out, (const float*)table, tokens, vocab, width);
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
