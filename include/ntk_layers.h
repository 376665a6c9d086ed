/* include/ntk_layers.h -- operators of the layer-list model families (csrc/dense.hip, csrc/latent_attention.hip, csrc/moe.hip,
 * csrc/layer_ops.hip): dense bfloat16 / float32 weights, F32 activations and residual stream.
 *
 * Same conventions as ntk.h: plain pointers and sizes, stream ordered, no allocation, NTK_OK or a negative NTK_E_* code.  Nothing here knows a
 * model: every size and constant is a parameter.  Two precisions of one operator set:
 *   weights NTK_DT_BF16 : matrix products on the bf16 matrix cores (activations rounded to bfloat16 at the product's input, F32 accumulation);
 *   weights NTK_DT_F32  : every product in true F32 (FMA on the vector units).
 * Norms, rotary angles, attention scores and weights, routers and the residual sum are F32 in both.
 */
#ifndef NTK_LAYERS_H
#define NTK_LAYERS_H

#include "ntk.h"

#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif
#ifdef __cplusplus
extern "C" {
#endif

/* Y[r][0..N) (+)= X[src(r)][0..K) . W_g[N][K]^T for every row r of every group g.
 *   W        : G matrices [N][K], `wstride` elements apart, dtype NTK_DT_BF16 or NTK_DT_F32
 *   offsets  : device int [G + 1], rows [offsets[g], offsets[g+1]) belong to group g; NULL: one group of T rows
 *   rows     : device int [T], src(r) = rows[r] / row_div; NULL: src(r) = r
 *   T        : number of rows (all groups together); Y rows are `ldy` floats apart, X rows `ldx`
 *   accumulate != 0 : Y += instead of Y =
 * A row's result depends on that row alone (not on T, the group sizes or the row's place) up to the kernel form picked by T. */
typedef struct ntk_dense_desc {
    float* Y; int ldy;
    const float* X; int ldx;
    const void* W; long long wstride; int wdtype;
    const int* offsets; int G;
    const int* rows; int row_div;
    int T, N, K;
    int accumulate;
    /* glu_ff > 0 (only with T <= ntk_dense_few_rows(), N == 2 * glu_ff, no accumulate): W holds glu_ff gate rows then glu_ff up rows and
     * Y[r][f] = g' * sigmoid(glu_alpha * g') * (u' + 1), g' = min(gate, glu_limit), u' = clamp(up, -glu_limit, glu_limit) -- the product and ntk_clipped_glu in one launch */
    int glu_ff; float glu_limit, glu_alpha;
    /* norm_w != NULL (only with T <= ntk_dense_few_rows()): every activation row is first divided by sqrt(mean(x^2) + norm_eps) and multiplied by
     * (norm_offset + norm_w[k]), norm_w F32 [K] -- ntk_rmsnorm_offset and the product in one launch */
    const float* norm_w; float norm_eps, norm_offset;
} ntk_dense_desc;
int ntk_dense_few_rows(void);   /* up to this many rows a product takes the row-streaming form */
int ntk_dense(const ntk_dense_desc* d, void* stream);
/* the plain case: Y[T][N] = X[T][K] . W[N][K]^T */
int ntk_dense_linear(float* Y, int ldy, const float* X, int ldx, const void* W, int wdtype, int T, int N, int K, int accumulate, void* stream);

/* ---- layer_ops.hip ---------------------------------------------------------------------------------------------------------------- */
/* out[t][:] = table[tokens[t]][:] (table NTK_DT_BF16 or NTK_DT_F32 [vocab][width]); a token outside [0, vocab) gives a row of zeros */
int ntk_embed_dense(float* out, const void* table, int tdtype, const int* tokens, int T, int vocab, int width, void* stream);
/* y[t][:] = x[t][:] / sqrt(mean(x[t]^2) + eps) * (offset + w[:]) for up to two (w, y) pairs sharing x (w F32 [n]; y2 / w2 may be NULL).
 * offset 1: the weight is stored around zero; offset 0: plain.  x rows ldx floats apart, y rows ldy. */
int ntk_rmsnorm_offset(float* y1, const float* w1, float* y2, const float* w2, int ldy, const float* x, int ldx, int T, int n, float eps, float offset,
                       void* stream);
/* out[t] = [a[t] ; b[t]] (two rows of n floats side by side) */
int ntk_concat_rows(float* out, const float* a, const float* b, int T, int n, void* stream);
/* y[i] *= 1 / (1 + exp(-g[i])) over T rows of n (y rows ldy apart, g rows ldg) */
int ntk_sigmoid_gate(float* y, int ldy, const float* g, int ldg, int T, int n, void* stream);
/* dst[0..n) = src[0..n) */
int ntk_rows_copy(float* dst, const float* src, long long n, void* stream);
/* x[i] += a[i] (+ b[i] if b) */
int ntk_residual_add(float* x, const float* a, const float* b, int n, void* stream);

/* ---- latent_attention.hip ---------------------------------------------------------------------------------------------------------
 * Attention whose keys and values are up-projections of one cached latent per position plus one rotated key part shared by the heads.
 * The cache of a layer run holds rows of `row` = kv_rank + rot_dim floats: [latent (normed) | rotated key part].                       */
typedef struct ntk_rotary {       /* angle of pair i at position p: p * freq[i]; cos and sin times mag */
    const double* freq;           /* device F64 [dims / 2] (after any frequency scaling): angles are formed in double, applied in F32 */
    float mag;
    int dims;                     /* rotated entries at the head of the vector, neighbours (2i, 2i+1) paired */
} ntk_rotary;
/* For T tokens at positions pos0 ...: kv [T][ldkv] = [kv_rank raw latent | rot_dim raw key part] -> cache rows pos0 .. pos0+T-1:
 * latent / rms * norm_w, key part rotated (its first rot->dims entries; the rest copied).  q [T][H][qd], ldq floats between tokens: the rot_dim entries at the
 * end of every head rotated in place the same way. */
int ntk_latent_prepare(float* cache, int row, const float* kv, int ldkv, const float* norm_w, float eps, int kv_rank, int rot_dim, float* q, int ldq, int H, int qd,
                       const ntk_rotary* rot, int pos0, int T, void* stream);
/* Softmax attention of query rows over cached positions.  Two forms of one kernel:
 *  expanded (shared == 0): K [nkeys][H][dn] and V [nkeys][H][dv] hold the up-projected keys / values of positions key0 .. key0+nkeys-1
 *           (ldk / ldv floats between positions), q [T][H][dn+dr]; the rotated part of the score reads the cache rows (offset kv_rank).
 *  shared   (shared != 0): q [T][H][R+dr] = [query folded through the key up-projection | rotated part]; keys AND values are the cache rows
 *           themselves (K = [latent | rotated], V = latent): out [T][H][R].  K / V arguments are unused.
 * Query t (position pos0 + t) sees position j iff j <= pos0 + t and (window <= 0 or pos0 + t - j < window).  scale multiplies the whole score.
 * out rows [T][H][dv] (expanded) / [T][H][R] (shared), ldo floats between tokens.  scratch: F32 [>= ntk_latent_attention_scratch(...)] . */
size_t ntk_latent_attention_scratch(int T, int H, int vdim_or_rank, int nkeys);
int ntk_latent_attention(float* out, int ldo, const float* q, int ldq, const float* K, int ldk, const float* V, int ldv, const float* cache, int row,
                         int kv_rank, int rot_dim, int H, int dn, int dv, int shared, int pos0, int T, int key0, int window, float scale, float* scratch,
                         void* stream);
/* fold the unrotated query part through the key up-projection: qf[t][h][0..R) = sum_d q[t][h][d] * W_uk[h*dn + d][0..R), and copy the rotated part behind it
 * (qf [T][H][R+dr]; q rows ldq floats apart); W_uk NTK_DT_BF16 / F32 [H*dn][R] */
int ntk_latent_fold_query(float* qf, const float* q, int ldq, const void* w_uk, int wdtype, int T, int H, int dn, int dr, int R, void* stream);
/* out[t][h*dv + v] = sum_r W_uv[h*dv + v][r] * lat[t][h][r]  (the value up-projection applied after the weighted sum), times sigmoid(gate[t][h*dv+v]) if gate */
int ntk_latent_unfold_value(float* out, int ldo, const float* lat, const void* w_uv, int wdtype, const float* gate, int ldg, int T, int H, int dv, int R,
                            void* stream);

/* ---- moe.hip ---------------------------------------------------------------------------------------------------------------------- */
/* Router of a mixture of experts, one launch: z = W_r h (F32 weights [E][n]), s = softmax(z); the `top` largest (ties: the lower index), weights
 * s / (sum of the chosen + 1e-20) -> ids [T][top], wts [T][top].  shared_gate_w (F32 [n], may be NULL) -> sgate[t] = sigmoid(w . h[t]).  E <= 256. */
int ntk_moe_route(int* ids, float* wts, float* sgate, const float* h, int ldh, const float* w_router, const float* shared_gate_w, int T, int n, int E, int top,
                  void* stream);
/* Stable grouping of the T*top (token, slot) pairs by expert: offsets [E+1], order [T*top] (pair index t*top+slot of every sorted row),
 * where [T*top] (sorted row of every pair). */
int ntk_moe_group(int* offsets, int* order, int* where, const int* ids, int T, int top, int E, void* stream);
/* a[r][f] = g' * sigmoid(alpha * g') * (u' + 1), g' = min(gu[r][f], limit), u' = clamp(gu[r][ff + f], -limit, limit); gu rows of 2*ff, a rows of ff */
int ntk_clipped_glu(float* a, const float* gu, int rows, int ff, float limit, float alpha, void* stream);
/* x[t][:] += mix[t][:] (if mix) + sum_s wts[t][s] * d[where[t*top+s]][:] + sgate[t] * shared[t][:] (if shared) -- slots in order, one rounding sequence per token */
int ntk_moe_combine(float* x, const float* mix, const float* d, const int* where, const float* wts, const float* shared, const float* sgate, int T, int top,
                    int n, void* stream);

#ifdef __cplusplus
}
#endif
#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#endif /* NTK_LAYERS_H */
