// engine/layer_stack.h -- model families described by a LIST of layers in config.json (type of mixer, its sizes, its feed-forward), with dense
// bfloat16 weights in a safetensors file: a residual stream in F32, parallel layers (mixer and feed-forward read two norms of the same input), an
// optional repeated span of layers (each pass with its own cache, entered through a projection of [stream ; embedding]), and an output norm + head.
//
// Mechanisms are parsed into parameter structs and run by the operators of include/ntk_layers.h, so another family can list them in another order
// or with other constants:
//   mixers        "latent_attention" (query through a normed latent, causal, optional frequency-scaled rotation) and "latent_attention_2" (query from
//                 one matrix, sliding window): one LatentMixer each -- which of the options a layer has is read from its config keys;
//   feed-forward  kind "moe": routed clipped-GLU experts + an optional gated shared expert.
// Registered for the architecture "Fabolorn".
#pragma once
#include <string>
#include <vector>
#include "safetensors.h"
#include "sequence_model.h"
#include "../../../include/ntk_layers.h"

namespace nt {

struct DenseW {                 // a matrix (or a stack of equal matrices) in the model's product dtype, row-major [out][in]
    void* ptr = nullptr;
    int dtype = 0;
    int64_t out_f = 0, in_f = 0;
    int count = 1;
    long long stride() const { return (long long)out_f * in_f; }
};

struct LatentMixer {
    int heads = 0, dim = 0, rot_dim = 0, vdim = 0, kv_rank = 0, q_rank = 0;   // q_rank 0: the query comes from one matrix
    int window = 0;                                                             // 0: causal over everything
    float scale = 1.0f;
    int rot_dims = 0;
    float rot_mag = 1.0f;
    double* rot_freq = nullptr;       // device [rot_dims / 2]
    DenseW in;                        // rows [query or query latent | kv_rank + rot_dim | gate] of one product over the normed input
    int q_off = 0, kv_off = 0, g_off = 0;
    DenseW uq, uk, uv, o;
    float* q_norm = nullptr;          // F32 [q_rank]
    float* kv_norm = nullptr;         // F32 [kv_rank]
    int qd() const { return dim + rot_dim; }
    int row() const { return kv_rank + rot_dim; }
};

struct ClippedExperts {               // `count` experts of the same shape, stacked: gate rows then up rows, and the down matrices
    int ff = 0;
    float limit = 0.0f;
    DenseW gate_up, down;
};

struct MoeFeedForward {
    int experts = 0, top = 0;
    float* router = nullptr;          // F32 [experts][width]
    ClippedExperts routed;
    bool has_shared = false;
    ClippedExperts shared;
    float* shared_gate = nullptr;     // F32 [width]
};

struct StackLayer {
    std::string type;
    float* norm1 = nullptr;
    float* norm2 = nullptr;
    LatentMixer mix;
    bool has_mlp = false;
    MoeFeedForward mlp;
};

class LayerStackModel : public SequenceModel {
public:
    LayerStackModel() = default;
    ~LayerStackModel() override;
    int load(const std::string& dir, const SeqLoadOptions& opt) override;
    const SeqModelInfo& info() const override { return info_; }
    const std::string& error() const override { return err_; }
    uint64_t weight_bytes() const override { return weight_bytes_; }
    int acquire_slot() override;
    int release_slot(int slot) override;
    int slot_length(int slot) const override { return slots_.length(slot); }
    int truncate_slot(int slot, int length) override;
    float* forward(int slot, const int* tokens, int n, const int* want, int n_want) override;
    int copy_logits(float* host, int rows) override;
    int set_capture(bool on) override { capture_ = on; return 0; }
    int copy_capture(float* host) override;
    int sync() override;
    void* stream() const override { return stream_; }
    static constexpr int kSharedRows = 8;     // up to this many tokens per portion take the decode form of the mixer (and the GEMV form of the products)

private:
    struct Run { int layer; bool enters; float* cache; };
    int fail(int st, const std::string& why) { err_ = why; return st; }
    int parse(const ModelFolder& f);
    int parse_mixer(const Json& L, const std::string& type, LatentMixer& m);
    int upload_layer(const ModelFolder& f, int i, StackLayer& L);
    int upload_vector(const ModelFolder& f, const std::string& name, int64_t n, float** out);
    int upload_matrix(const ModelFolder& f, const std::vector<std::string>& names, int64_t in_f, DenseW& out, int count = 1);
    int alloc_buffers();
    void* dev_alloc(size_t bytes);
    int portion(int slot, const int* tokens_dev, int T, int pos0, const int* want_dev, int n_want, float* logits_out);
    int run_mixer(const StackLayer& L, float* cache, int T, int pos0);
    int run_moe(const StackLayer& L, int T);
    int run_experts(const ClippedExperts& ex, const float* h, float* gu, float* act, float* out, int rows, const int* offsets, const int* order, int top);

    SeqModelInfo info_;
    std::string err_;
    SeqLoadOptions opt_;
    int wdtype_ = NTK_DT_BF16;
    float eps_ = 1e-6f;
    std::vector<StackLayer> layers_;
    std::vector<Run> runs_;
    bool has_loop_ = false;
    DenseW embed_, head_, loop_in_;
    float* final_norm_ = nullptr;
    uint64_t weight_bytes_ = 0;
    std::vector<void*> allocs_;
    SlotTable slots_;
    void* stream_ = nullptr;
    int chunk_ = 0;                   // tokens per internal portion
    // maxima over the layers (buffer sizes)
    int max_in_ = 0, max_qrank_ = 0, max_hqd_ = 0, max_hdv_ = 0, max_hdn_ = 0, max_fold_ = 0, max_hr_ = 0, max_top_ = 0, max_e_ = 0, max_ff2_ = 0, max_sff2_ = 0;
    // activations
    float *x_ = nullptr, *x0_ = nullptr, *cat_ = nullptr, *h1_ = nullptr, *h2_ = nullptr, *a_ = nullptr, *cq_ = nullptr, *q_ = nullptr, *qf_ = nullptr, *lat_ = nullptr,
          *att_ = nullptr, *kx_ = nullptr, *vx_ = nullptr, *mix_ = nullptr, *wts_ = nullptr, *sg_ = nullptr, *gu_ = nullptr, *act_ = nullptr, *dn_ = nullptr,
          *sgu_ = nullptr, *sact_ = nullptr, *sdn_ = nullptr, *scratch_ = nullptr, *xw_ = nullptr, *hn_ = nullptr;
    int *ids_ = nullptr, *offsets_ = nullptr, *order_ = nullptr, *where_ = nullptr, *tokens_dev_ = nullptr, *want_dev_ = nullptr;
    int* h_stage_ = nullptr;          // pinned: tokens and wanted places of the pass being launched
    float* logits_ = nullptr;
    size_t logits_rows_ = 0;
    int last_rows_ = 0;
    bool capture_ = false;
    float* capture_buf_ = nullptr;
    size_t capture_floats_ = 0;
    int capture_T_ = 0;
};

}  // namespace nt
