// engine/layer_stack.cpp -- see layer_stack.h
#include "layer_stack.h"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace nt {

#define LS_TRY(expr)                          \
    do {                                      \
        const int st__ = (expr);              \
        if (st__ != NTK_OK) return st__;      \
    } while (0)

static constexpr float kGluAlpha = 1.702f;   // the design fixes the slope of the experts' gate activation
static FamilyRegistrar reg_fabolorn("Fabolorn", [] { return std::unique_ptr<SequenceModel>(new LayerStackModel()); });

LayerStackModel::~LayerStackModel() {
    if (stream_) ntk_stream_synchronize(stream_);
    for (void* p : allocs_) nt_hip_free(p);
    if (logits_) nt_hip_free(logits_);
    if (capture_buf_) nt_hip_free(capture_buf_);
    if (h_stage_) nt_hip_free_host(h_stage_);
}

void* LayerStackModel::dev_alloc(size_t bytes) {
    void* p = nt_hip_malloc(bytes ? bytes : 16);
    if (p) allocs_.push_back(p);
    return p;
}

// ------------------------------------------------------------------------------------------------------------------------ configuration
static bool need_int(const Json& o, const char* key, int& out, std::string& err, const std::string& where) {
    if (!o.at(key).is_number()) { err = where + ": '" + key + "' is missing"; return false; }
    out = (int)o.at(key).integer();
    if (out <= 0) { err = where + ": '" + key + "' must be positive"; return false; }
    return true;
}

int LayerStackModel::parse_mixer(const Json& L, const std::string& type, LatentMixer& m) {
    const Json& mx = L.at("mixer");
    const std::string where = "mixer '" + type + "'";
    if (!mx.is_object()) return fail(NTK_E_FORMAT, where + ": no 'mixer' object");
    if (!need_int(mx, "heads", m.heads, err_, where) || !need_int(mx, "dim", m.dim, err_, where) || !need_int(mx, "rot_dim", m.rot_dim, err_, where) ||
        !need_int(mx, "vdim", m.vdim, err_, where) || !need_int(mx, "kv_rank", m.kv_rank, err_, where))
        return NTK_E_FORMAT;
    if (type == "latent_attention") {
        if (!need_int(mx, "q_rank", m.q_rank, err_, where)) return NTK_E_FORMAT;
    } else {
        m.q_rank = 0;
    }
    if (!mx.at("scale").is_number()) return fail(NTK_E_FORMAT, where + ": 'scale' is missing");
    m.scale = (float)mx.at("scale").number();
    m.window = 0;
    if (mx.has("mask")) {
        if (!need_int(mx.at("mask"), "size", m.window, err_, where + " mask")) return NTK_E_FORMAT;
    } else if (type == "latent_attention_2") {
        return fail(NTK_E_FORMAT, where + ": 'mask' is missing");
    }
    const Json& rot = mx.at("rot");
    if (!rot.is_object() || !rot.at("base").is_number()) return fail(NTK_E_FORMAT, where + ": 'rot' is missing");
    m.rot_dims = rot.has("dims") ? (int)rot.at("dims").integer() : m.rot_dim;
    if (m.rot_dims < 0 || (m.rot_dims & 1) || m.rot_dims > m.rot_dim) return fail(NTK_E_FORMAT, where + ": rot.dims must be even and at most rot_dim");
    const double base = rot.at("base").number();
    const int half = m.rot_dims / 2;
    std::vector<double> f((size_t)std::max(half, 1));
    for (int i = 0; i < half; ++i) f[(size_t)i] = std::pow(base, -2.0 * i / m.rot_dims);
    m.rot_mag = 1.0f;
    if (rot.has("scaling")) {
        const Json& sc = rot.at("scaling");
        const double factor = sc.at("factor").number(1.0), orig = sc.at("original").number(1.0), fast = sc.at("fast").number(1.0), slow = sc.at("slow").number(1.0);
        auto where_dim = [&](double turns) { return m.rot_dims * std::log(orig / (2.0 * M_PI * turns)) / (2.0 * std::log(base)); };
        const double lo = std::max(std::floor(where_dim(fast)), 0.0), hi = std::min(std::ceil(where_dim(slow)), (double)m.rot_dims - 1.0);
        for (int i = 0; i < half; ++i) {
            const double ramp = std::min(std::max((i - lo) / std::max(hi - lo, 0.001), 0.0), 1.0);
            f[(size_t)i] = f[(size_t)i] / factor * ramp + f[(size_t)i] * (1.0 - ramp);
        }
        m.rot_mag = (float)(0.1 * std::log(factor) + 1.0);
    }
    m.rot_freq = (double*)dev_alloc(f.size() * sizeof(double));
    if (!m.rot_freq) return fail(NTK_E_NOMEM, "out of device memory");
    nt_hip_memcpy_h2d(m.rot_freq, f.data(), f.size() * sizeof(double));
    return NTK_OK;
}

int LayerStackModel::parse(const ModelFolder& f) {
    const Json& c = f.config();
    info_.architecture = c.at("architecture").str;
    if (!need_int(c, "vocab", info_.vocab, err_, "config") || !need_int(c, "width", info_.width, err_, "config")) return NTK_E_FORMAT;
    eps_ = (float)c.at("norm").at("eps").number(1e-6);
    if (c.at("bos").is_number()) info_.bos = (int)c.at("bos").integer();
    if (c.at("eos").is_number()) info_.eos = (int)c.at("eos").integer();
    const Json& ls = c.at("layers");
    if (!ls.is_array() || ls.arr.empty()) return fail(NTK_E_FORMAT, "config: 'layers' is missing");
    layers_.resize(ls.arr.size());
    for (size_t i = 0; i < ls.arr.size(); ++i) {
        const Json& L = ls.arr[i];
        StackLayer& S = layers_[i];
        S.type = L.at("type").str;
        if (S.type != "latent_attention" && S.type != "latent_attention_2") return fail(NTK_E_FORMAT, "layer " + std::to_string(i) + ": unknown mixer type '" + S.type + "'");
        LS_TRY(parse_mixer(L, S.type, S.mix));
        S.has_mlp = L.has("mlp");
        if (S.has_mlp) {
            const Json& ml = L.at("mlp");
            const std::string where = "layer " + std::to_string(i) + " mlp";
            if (ml.at("kind").is_string() && ml.at("kind").str != "moe") return fail(NTK_E_FORMAT, where + ": unknown kind '" + ml.at("kind").str + "'");
            MoeFeedForward& M = S.mlp;
            if (!need_int(ml.at("router"), "experts", M.experts, err_, where) || !need_int(ml.at("router"), "top", M.top, err_, where) ||
                !need_int(ml.at("expert"), "ff", M.routed.ff, err_, where))
                return NTK_E_FORMAT;
            if (M.top > M.experts || M.experts > 255) return fail(NTK_E_FORMAT, where + ": top <= experts <= 255 is required");
            M.routed.limit = (float)ml.at("expert").at("limit").number();
            M.has_shared = ml.has("shared");
            if (M.has_shared) {
                if (!need_int(ml.at("shared"), "ff", M.shared.ff, err_, where + " shared")) return NTK_E_FORMAT;
                M.shared.limit = (float)ml.at("shared").at("limit").number();
            }
        }
    }
    // the order of layer runs
    const int n = (int)layers_.size();
    runs_.clear();
    has_loop_ = c.has("loop");
    if (has_loop_) {
        const Json& lp = c.at("loop");
        const int a = (int)lp.at("start").integer(), b = (int)lp.at("stop").integer(), times = (int)lp.at("times").integer(1);
        if (a < 0 || b <= a || b > n || times < 1) return fail(NTK_E_FORMAT, "config: loop needs 0 <= start < stop <= layers and times >= 1");
        for (int i = 0; i < a; ++i) runs_.push_back({i, false, nullptr});
        for (int t = 0; t < times; ++t)
            for (int i = a; i < b; ++i) runs_.push_back({i, i == a, nullptr});
        for (int i = b; i < n; ++i) runs_.push_back({i, false, nullptr});
    } else {
        for (int i = 0; i < n; ++i) runs_.push_back({i, false, nullptr});
    }
    info_.n_layers = n;
    info_.n_layer_runs = (int)runs_.size();
    return NTK_OK;
}

// ------------------------------------------------------------------------------------------------------------------------ weights
static inline float bf16_to_f32(uint16_t b) { uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static bool tensor_to_f32(const StTensor& t, float* dst) {
    const int64_t n = t.numel();
    if (t.dtype == "BF16") { const uint16_t* s = (const uint16_t*)t.data; for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(s[i]); return true; }
    if (t.dtype == "F32") { memcpy(dst, t.data, (size_t)n * 4); return true; }
    return false;
}

int LayerStackModel::upload_vector(const ModelFolder& f, const std::string& name, int64_t n, float** out) {
    const StTensor* t = f.tensor(name);
    if (!t) return fail(NTK_E_FORMAT, "tensor '" + name + "' is missing");
    if (t->numel() != n) return fail(NTK_E_SHAPE, "tensor '" + name + "' has " + std::to_string(t->numel()) + " elements, expected " + std::to_string(n));
    std::vector<float> h((size_t)n);
    if (!tensor_to_f32(*t, h.data())) return fail(NTK_E_DTYPE, "tensor '" + name + "': dtype " + t->dtype + " is not supported");
    *out = (float*)dev_alloc((size_t)n * 4);
    if (!*out) return fail(NTK_E_NOMEM, "out of device memory");
    nt_hip_memcpy_h2d(*out, h.data(), (size_t)n * 4);
    weight_bytes_ += t->nbytes;
    return NTK_OK;
}

// `names` one below the other as ONE matrix (count == 1), or `count` groups of names.size() / count tensors: a stack of equal matrices
int LayerStackModel::upload_matrix(const ModelFolder& f, const std::vector<std::string>& names, int64_t in_f, DenseW& out, int count) {
    int64_t rows = 0;
    for (const auto& nm : names) {
        const StTensor* t = f.tensor(nm);
        if (!t) return fail(NTK_E_FORMAT, "tensor '" + nm + "' is missing");
        if (t->shape.size() != 2 || t->shape[1] != in_f) return fail(NTK_E_SHAPE, "tensor '" + nm + "': expected [*, " + std::to_string(in_f) + "]");
        rows += t->shape[0];
    }
    if (rows % count) return fail(NTK_E_SHAPE, "stacked tensors of unequal shape around '" + names[0] + "'");
    const size_t es = wdtype_ == NTK_DT_BF16 ? 2 : 4;
    std::vector<uint8_t> h((size_t)rows * in_f * es);
    size_t at = 0;
    for (const auto& nm : names) {
        const StTensor* t = f.tensor(nm);
        const int64_t n = t->numel();
        if (wdtype_ == NTK_DT_BF16) {
            uint16_t* d = (uint16_t*)(h.data() + at);
            if (t->dtype == "BF16") memcpy(d, t->data, (size_t)n * 2);
            else if (t->dtype == "F32") { const float* s = (const float*)t->data; for (int64_t i = 0; i < n; ++i) d[i] = f32_to_bf16(s[i]); }
            else return fail(NTK_E_DTYPE, "tensor '" + nm + "': dtype " + t->dtype + " is not supported");
        } else {
            if (!tensor_to_f32(*t, (float*)(h.data() + at))) return fail(NTK_E_DTYPE, "tensor '" + nm + "': dtype " + t->dtype + " is not supported");
        }
        at += (size_t)n * es;
        weight_bytes_ += t->nbytes;
    }
    out.ptr = dev_alloc(h.size() + 256);
    if (!out.ptr) return fail(NTK_E_NOMEM, "out of device memory");
    nt_hip_memcpy_h2d(out.ptr, h.data(), h.size());
    out.dtype = wdtype_;
    out.in_f = in_f;
    out.out_f = rows / count;
    out.count = count;
    return NTK_OK;
}

int LayerStackModel::upload_layer(const ModelFolder& f, int i, StackLayer& L) {
    const std::string p = "l" + std::to_string(i) + ".";
    const int W = info_.width;
    LatentMixer& m = L.mix;
    LS_TRY(upload_vector(f, p + "norm1", W, &L.norm1));
    const int hq = m.heads * m.qd(), hv = m.heads * m.vdim;
    const std::string first = m.q_rank ? p + "mix.dq" : p + "mix.q";
    LS_TRY(upload_matrix(f, {first, p + "mix.dkv", p + "mix.g"}, W, m.in));
    m.q_off = 0;
    m.kv_off = m.q_rank ? m.q_rank : hq;
    m.g_off = m.kv_off + m.row();
    if (m.in.out_f != m.g_off + hv) return fail(NTK_E_SHAPE, "layer " + std::to_string(i) + ": the mixer's input projections do not have the configured sizes");
    if (m.q_rank) {
        LS_TRY(upload_vector(f, p + "mix.dq.norm", m.q_rank, &m.q_norm));
        LS_TRY(upload_matrix(f, {p + "mix.uq"}, m.q_rank, m.uq));
        if (m.uq.out_f != hq) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.uq' does not have heads * (dim + rot_dim) rows");
    }
    LS_TRY(upload_vector(f, p + "mix.dkv.norm", m.kv_rank, &m.kv_norm));
    LS_TRY(upload_matrix(f, {p + "mix.uk"}, m.kv_rank, m.uk));
    LS_TRY(upload_matrix(f, {p + "mix.uv"}, m.kv_rank, m.uv));
    LS_TRY(upload_matrix(f, {p + "mix.o"}, hv, m.o));
    if (m.uk.out_f != m.heads * m.dim || m.uv.out_f != hv || m.o.out_f != W) return fail(NTK_E_SHAPE, "layer " + std::to_string(i) + ": up-projections do not have the configured sizes");
    if (L.has_mlp) {
        MoeFeedForward& M = L.mlp;
        LS_TRY(upload_vector(f, p + "norm2", W, &L.norm2));
        LS_TRY(upload_vector(f, p + "mlp.router", (int64_t)M.experts * W, &M.router));
        std::vector<std::string> gu, dn;
        for (int e = 0; e < M.experts; ++e) {
            const std::string q = p + "mlp.e" + std::to_string(e) + ".";
            gu.push_back(q + "gate"); gu.push_back(q + "up"); dn.push_back(q + "down");
        }
        LS_TRY(upload_matrix(f, gu, W, M.routed.gate_up, M.experts));
        LS_TRY(upload_matrix(f, dn, M.routed.ff, M.routed.down, M.experts));
        if (M.routed.gate_up.out_f != 2 * M.routed.ff || M.routed.down.out_f != W) return fail(NTK_E_SHAPE, "layer " + std::to_string(i) + ": expert matrices do not have the configured sizes");
        if (M.has_shared) {
            LS_TRY(upload_matrix(f, {p + "mlp.shared.gate", p + "mlp.shared.up"}, W, M.shared.gate_up));
            LS_TRY(upload_matrix(f, {p + "mlp.shared.down"}, M.shared.ff, M.shared.down));
            if (M.shared.gate_up.out_f != 2 * M.shared.ff || M.shared.down.out_f != W) return fail(NTK_E_SHAPE, "layer " + std::to_string(i) + ": shared expert matrices do not have the configured sizes");
            LS_TRY(upload_vector(f, p + "mlp.shared.sg", W, &M.shared_gate));
        }
    }
    return NTK_OK;
}

int LayerStackModel::load(const std::string& dir, const SeqLoadOptions& opt) {
    opt_ = opt;
    if (opt_.max_context < 1 || opt_.slots < 1) return fail(NTK_E_SHAPE, "max_context and slots must be positive");
    wdtype_ = opt.float32 ? NTK_DT_F32 : NTK_DT_BF16;
    if (ntk_device_count() <= 0) return fail(NTK_E_NODEVICE, "no GPU");
    stream_ = ntk_stream(0);
    if (!stream_) return fail(NTK_E_NODEVICE, "the HIP runtime did not start");
    ModelFolder f;
    const int st = f.open(dir);
    if (st != NTK_OK) return fail(st, f.error());
    LS_TRY(parse(f));
    const int W = info_.width;
    LS_TRY(upload_matrix(f, {"embed"}, W, embed_));
    LS_TRY(upload_matrix(f, {"head"}, W, head_));
    if (embed_.out_f != info_.vocab || head_.out_f != info_.vocab) return fail(NTK_E_SHAPE, "embed / head do not have 'vocab' rows");
    LS_TRY(upload_vector(f, "final.norm", W, &final_norm_));
    if (has_loop_) {
        LS_TRY(upload_matrix(f, {"loop.in"}, 2 * W, loop_in_));
        if (loop_in_.out_f != W) return fail(NTK_E_SHAPE, "tensor 'loop.in' is not [width, 2 width]");
    }
    for (size_t i = 0; i < layers_.size(); ++i) LS_TRY(upload_layer(f, (int)i, layers_[i]));
    info_.max_context = opt_.max_context;
    slots_.reset(opt_.slots, opt_.max_context);
    return alloc_buffers();
}

int LayerStackModel::alloc_buffers() {
    const int W = info_.width;
    chunk_ = std::min(opt_.max_context, 1024);
    for (const auto& L : layers_) {
        const LatentMixer& m = L.mix;
        max_in_ = std::max<int>(max_in_, (int)m.in.out_f);
        max_qrank_ = std::max(max_qrank_, m.q_rank);
        max_hqd_ = std::max(max_hqd_, m.heads * m.qd());
        max_hdv_ = std::max(max_hdv_, m.heads * m.vdim);
        max_hdn_ = std::max(max_hdn_, m.heads * m.dim);
        max_fold_ = std::max(max_fold_, m.heads * m.row());
        max_hr_ = std::max(max_hr_, m.heads * m.kv_rank);
        if (m.kv_rank > 512 || m.vdim > 512) return fail(NTK_E_SHAPE, "kv_rank and vdim up to 512 are supported");
        if (L.has_mlp) {
            max_top_ = std::max(max_top_, L.mlp.top);
            max_e_ = std::max(max_e_, L.mlp.experts);
            max_ff2_ = std::max(max_ff2_, 2 * L.mlp.routed.ff);
            if (L.mlp.has_shared) max_sff2_ = std::max(max_sff2_, 2 * L.mlp.shared.ff);
        }
    }
    const size_t C = (size_t)chunk_, ctx = (size_t)opt_.max_context;
    auto fl = [&](float** p, size_t n) { *p = (float*)dev_alloc(n * sizeof(float)); return *p != nullptr; };
    auto in = [&](int** p, size_t n) { *p = (int*)dev_alloc(n * sizeof(int)); return *p != nullptr; };
    bool ok = fl(&x_, C * W) && fl(&x0_, C * W) && fl(&cat_, C * 2 * W) && fl(&h1_, C * W) && fl(&h2_, C * W) && fl(&a_, C * max_in_) &&
              fl(&cq_, C * std::max(max_qrank_, 1)) && fl(&q_, C * max_hqd_) && fl(&qf_, (size_t)kSharedRows * max_fold_) && fl(&lat_, (size_t)kSharedRows * max_hr_) &&
              fl(&att_, C * max_hdv_) && fl(&kx_, ctx * max_hdn_) && fl(&vx_, ctx * max_hdv_) && fl(&mix_, C * W) && fl(&xw_, C * W) && fl(&hn_, C * W) &&
              in(&tokens_dev_, 2 * C);
    want_dev_ = tokens_dev_ ? tokens_dev_ + C : nullptr;   // one staging area: [tokens of a pass | wanted places], filled by ONE stream-ordered copy from pinned memory
    h_stage_ = (int*)nt_hip_malloc_host(2 * C * sizeof(int));
    ok = ok && h_stage_ != nullptr;
    size_t sc = 0;
    for (const auto& L : layers_) sc = std::max(sc, ntk_latent_attention_scratch(kSharedRows, L.mix.heads, L.mix.kv_rank, opt_.max_context));
    ok = ok && fl(&scratch_, sc);
    if (max_top_ > 0) {
        const size_t P = C * max_top_;
        ok = ok && in(&ids_, P) && fl(&wts_, P) && fl(&sg_, C) && in(&offsets_, (size_t)max_e_ + 1) && in(&order_, P) && in(&where_, P) && fl(&gu_, P * max_ff2_) &&
             fl(&act_, P * (max_ff2_ / 2)) && fl(&dn_, P * W);
        if (max_sff2_ > 0) ok = ok && fl(&sgu_, C * max_sff2_) && fl(&sact_, C * (max_sff2_ / 2)) && fl(&sdn_, C * W);
    }
    if (!ok) return fail(NTK_E_NOMEM, "out of device memory (activation buffers)");
    for (auto& r : runs_) {
        const size_t row = (size_t)layers_[(size_t)r.layer].mix.row();
        r.cache = (float*)dev_alloc((size_t)opt_.slots * ctx * row * sizeof(float));
        if (!r.cache) return fail(NTK_E_NOMEM, "out of device memory (cache)");
    }
    return NTK_OK;
}

// ------------------------------------------------------------------------------------------------------------------------ slots
int LayerStackModel::acquire_slot() { const int s = slots_.acquire(); return s < 0 ? NTK_E_NOMEM : s; }
int LayerStackModel::release_slot(int slot) { return slots_.release(slot) ? NTK_OK : NTK_E_SHAPE; }
int LayerStackModel::truncate_slot(int slot, int length) {
    if (!slots_.live(slot) || length < 0 || length > slots_.length(slot)) return NTK_E_SHAPE;
    slots_.set_length(slot, length);
    return NTK_OK;
}

// ------------------------------------------------------------------------------------------------------------------------ the step
int LayerStackModel::run_mixer(const StackLayer& L, float* cache, int T, int pos0) {
    const LatentMixer& m = L.mix;
    const int W = info_.width, H = m.heads, qd = m.qd(), row = m.row(), hv = H * m.vdim, na = (int)m.in.out_f;
    // one product for [query (latent) | latent + key part | gate]; decoding: the layer's first norm and the query latent's norm run inside the products
    const bool few = T <= ntk_dense_few_rows();
    ntk_dense_desc d{};
    d.Y = a_; d.ldy = na; d.X = few ? x_ : h1_; d.ldx = W; d.W = m.in.ptr; d.wdtype = m.in.dtype; d.G = 1; d.row_div = 1; d.T = T; d.N = na; d.K = W;
    if (few) { d.norm_w = L.norm1; d.norm_eps = eps_; d.norm_offset = 1.0f; }
    LS_TRY(ntk_dense(&d, stream_));
    float* q = a_;
    int ldq = na;
    if (m.q_rank) {
        d.Y = q_; d.ldy = H * qd; d.X = few ? a_ : cq_; d.ldx = few ? na : m.q_rank; d.W = m.uq.ptr; d.wdtype = m.uq.dtype; d.N = H * qd; d.K = m.q_rank;
        if (few) { d.norm_w = m.q_norm; d.norm_offset = 0.0f; }
        else LS_TRY(ntk_rmsnorm_offset(cq_, m.q_norm, nullptr, nullptr, m.q_rank, a_, na, T, m.q_rank, eps_, 0.0f, stream_));
        LS_TRY(ntk_dense(&d, stream_));
        q = q_;
        ldq = H * qd;
    }
    ntk_rotary rot{m.rot_freq, m.rot_mag, m.rot_dims};
    LS_TRY(ntk_latent_prepare(cache, row, a_ + m.kv_off, na, m.kv_norm, eps_, m.kv_rank, m.rot_dim, q, ldq, H, qd, &rot, pos0, T, stream_));
    if (T <= kSharedRows) {
        LS_TRY(ntk_latent_fold_query(qf_, q, ldq, m.uk.ptr, m.uk.dtype, T, H, m.dim, m.rot_dim, m.kv_rank, stream_));
        LS_TRY(ntk_latent_attention(lat_, H * m.kv_rank, qf_, H * row, nullptr, 0, nullptr, 0, cache, row, m.kv_rank, m.rot_dim, H, m.dim, m.vdim, 1, pos0, T, 0,
                                    m.window, m.scale, scratch_, stream_));
        LS_TRY(ntk_latent_unfold_value(att_, hv, lat_, m.uv.ptr, m.uv.dtype, a_ + m.g_off, na, T, H, m.vdim, m.kv_rank, stream_));
    } else {
        const int key0 = m.window > 0 ? std::max(0, pos0 - m.window + 1) : 0;
        const int nkeys = pos0 + T - key0;
        LS_TRY(ntk_dense_linear(kx_, H * m.dim, cache + (size_t)key0 * row, row, m.uk.ptr, m.uk.dtype, nkeys, H * m.dim, m.kv_rank, 0, stream_));
        LS_TRY(ntk_dense_linear(vx_, hv, cache + (size_t)key0 * row, row, m.uv.ptr, m.uv.dtype, nkeys, hv, m.kv_rank, 0, stream_));
        LS_TRY(ntk_latent_attention(att_, hv, q, ldq, kx_, H * m.dim, vx_, hv, cache, row, m.kv_rank, m.rot_dim, H, m.dim, m.vdim, 0, pos0, T, key0, m.window, m.scale,
                                    nullptr, stream_));
        LS_TRY(ntk_sigmoid_gate(att_, hv, a_ + m.g_off, na, T, hv, stream_));
    }
    return ntk_dense_linear(mix_, W, att_, hv, m.o.ptr, m.o.dtype, T, W, hv, 0, stream_);
}

int LayerStackModel::run_experts(const ClippedExperts& ex, const float* h, float* gu, float* act, float* out, int rows, const int* offsets, const int* order, int top) {
    const int W = info_.width;
    ntk_dense_desc d{};
    d.Y = gu; d.ldy = 2 * ex.ff; d.X = h; d.ldx = W; d.W = ex.gate_up.ptr; d.wstride = ex.gate_up.stride(); d.wdtype = ex.gate_up.dtype;
    d.offsets = offsets; d.G = ex.gate_up.count; d.rows = order; d.row_div = top; d.T = rows; d.N = 2 * ex.ff; d.K = W; d.accumulate = 0;
    if (rows <= ntk_dense_few_rows()) {   // decoding: the activation inside the product's launch
        d.Y = act; d.ldy = ex.ff; d.glu_ff = ex.ff; d.glu_limit = ex.limit; d.glu_alpha = kGluAlpha;
        LS_TRY(ntk_dense(&d, stream_));
        d.glu_ff = 0;
    } else {
        LS_TRY(ntk_dense(&d, stream_));
        LS_TRY(ntk_clipped_glu(act, gu, rows, ex.ff, ex.limit, kGluAlpha, stream_));
    }
    d.Y = out; d.ldy = W; d.X = act; d.ldx = ex.ff; d.W = ex.down.ptr; d.wstride = ex.down.stride(); d.wdtype = ex.down.dtype;
    d.rows = nullptr; d.row_div = 1; d.N = W; d.K = ex.ff;
    return ntk_dense(&d, stream_);
}

int LayerStackModel::run_moe(const StackLayer& L, int T) {
    const MoeFeedForward& M = L.mlp;
    const int W = info_.width;
    LS_TRY(ntk_moe_route(ids_, wts_, M.has_shared ? sg_ : nullptr, h2_, W, M.router, M.has_shared ? M.shared_gate : nullptr, T, W, M.experts, M.top, stream_));
    LS_TRY(ntk_moe_group(offsets_, order_, where_, ids_, T, M.top, M.experts, stream_));
    LS_TRY(run_experts(M.routed, h2_, gu_, act_, dn_, T * M.top, offsets_, order_, M.top));
    if (M.has_shared) LS_TRY(run_experts(M.shared, h2_, sgu_, sact_, sdn_, T, nullptr, nullptr, 1));
    // stream += mixer + sum of the chosen experts + gated shared expert
    return ntk_moe_combine(x_, mix_, dn_, where_, wts_, M.has_shared ? sdn_ : nullptr, M.has_shared ? sg_ : nullptr, T, M.top, W, stream_);
}

int LayerStackModel::portion(int slot, const int* tokens_dev, int T, int pos0, const int* want_dev, int n_want, float* logits_out) {
    const int W = info_.width;
    LS_TRY(ntk_embed_dense(x0_, embed_.ptr, embed_.dtype, tokens_dev, T, info_.vocab, W, stream_));
    bool x_is_x0 = true;   // until the first layer run writes x_
    for (size_t r = 0; r < runs_.size(); ++r) {
        const Run& run = runs_[r];
        const StackLayer& L = layers_[(size_t)run.layer];
        if (x_is_x0 && !run.enters) { LS_TRY(ntk_rows_copy(x_, x0_, (long long)T * W, stream_)); x_is_x0 = false; }
        if (run.enters) {
            LS_TRY(ntk_concat_rows(cat_, x_is_x0 ? x0_ : x_, x0_, T, W, stream_));
            LS_TRY(ntk_dense_linear(x_, W, cat_, 2 * W, loop_in_.ptr, loop_in_.dtype, T, W, 2 * W, 0, stream_));
            x_is_x0 = false;
        }
        if (T > ntk_dense_few_rows()) {
            LS_TRY(ntk_rmsnorm_offset(h1_, L.norm1, L.has_mlp ? h2_ : nullptr, L.has_mlp ? L.norm2 : nullptr, W, x_, W, T, W, eps_, 1.0f, stream_));
        } else if (L.has_mlp) {   // decoding: the mixer's norm runs inside its first product (run_mixer); the feed-forward's input has three readers
            LS_TRY(ntk_rmsnorm_offset(h2_, L.norm2, nullptr, nullptr, W, x_, W, T, W, eps_, 1.0f, stream_));
        }
        float* cache = run.cache + (size_t)slot * opt_.max_context * L.mix.row();
        LS_TRY(run_mixer(L, cache, T, pos0));
        if (L.has_mlp) LS_TRY(run_moe(L, T));
        else LS_TRY(ntk_residual_add(x_, mix_, nullptr, T * W, stream_));
        if (capture_ && capture_buf_) LS_TRY(ntk_rows_copy(capture_buf_ + r * (size_t)T * W, x_, (long long)T * W, stream_));
    }
    if (n_want > 0) {
        // the wanted rows only: gather, norm, head
        const float* xs = x_is_x0 ? x0_ : x_;
        const float* rows = xs;                       // a single decoded token is its own gather
        if (!(T == 1 && n_want == 1)) { LS_TRY(ntk_embed_dense(xw_, xs, NTK_DT_F32, want_dev, n_want, T, W, stream_)); rows = xw_; }
        ntk_dense_desc d{};
        d.Y = logits_out; d.ldy = info_.vocab; d.X = rows; d.ldx = W; d.W = head_.ptr; d.wdtype = head_.dtype; d.G = 1; d.row_div = 1; d.T = n_want;
        d.N = info_.vocab; d.K = W;
        if (n_want <= ntk_dense_few_rows()) { d.norm_w = final_norm_; d.norm_eps = eps_; d.norm_offset = 1.0f; }   // the output norm inside the head's launch
        else { LS_TRY(ntk_rmsnorm_offset(hn_, final_norm_, nullptr, nullptr, W, rows, W, n_want, W, eps_, 1.0f, stream_)); d.X = hn_; }
        LS_TRY(ntk_dense(&d, stream_));
    }
    return NTK_OK;
}

float* LayerStackModel::forward(int slot, const int* tokens, int n, const int* want, int n_want) {
    if (!slots_.live(slot)) { err_ = "forward: the slot is not live"; return nullptr; }
    if (n <= 0 || !tokens || n_want < 0 || (n_want && !want)) { err_ = "forward: no tokens"; return nullptr; }
    const int pos0 = slots_.length(slot);
    if (pos0 + n > opt_.max_context) { err_ = "forward: the slot's " + std::to_string(opt_.max_context) + " positions are used up"; return nullptr; }
    for (int i = 0; i < n_want; ++i)
        if (want[i] < 0 || want[i] >= n || (i && want[i] < want[i - 1])) { err_ = "forward: wanted places must be ascending and inside the portion"; return nullptr; }
    const size_t need = (size_t)std::max(n_want, 1);
    if (need > logits_rows_) {
        if (ntk_stream_synchronize(stream_) != NTK_OK) return nullptr;
        if (logits_) nt_hip_free(logits_);
        logits_rows_ = need;
        logits_ = (float*)nt_hip_malloc(logits_rows_ * (size_t)info_.vocab * sizeof(float));
        if (!logits_) { logits_rows_ = 0; err_ = "out of device memory (logits)"; return nullptr; }
    }
    if (capture_) {
        const size_t cf = runs_.size() * (size_t)n * info_.width;
        if (n > chunk_) { err_ = "capture: the portion must fit one internal pass"; return nullptr; }
        if (cf > capture_floats_) {
            ntk_stream_synchronize(stream_);
            if (capture_buf_) nt_hip_free(capture_buf_);
            capture_buf_ = (float*)nt_hip_malloc(cf * sizeof(float));
            capture_floats_ = capture_buf_ ? cf : 0;
            if (!capture_buf_) { err_ = "out of device memory (capture)"; return nullptr; }
        }
        capture_T_ = n;
    }
    int done_want = 0;
    for (int at = 0; at < n; at += chunk_) {
        const int T = std::min(chunk_, n - at);
        int w1 = done_want;
        while (w1 < n_want && want[w1] < at + T) ++w1;
        std::vector<int> rel((size_t)std::max(w1 - done_want, 1));
        for (int i = done_want; i < w1; ++i) rel[(size_t)(i - done_want)] = want[i] - at;
        // the pinned staging area is free once the previous pass's copy has run: wait for the stream (idle already after a copy_logits), then one
        // stream-ordered copy brings the tokens and the wanted places
        if (ntk_stream_synchronize(stream_) != NTK_OK) { err_ = "forward: the stream failed"; return nullptr; }
        memcpy(h_stage_, tokens + at, (size_t)T * sizeof(int));
        const int nw = w1 - done_want;
        if (nw > 0) memcpy(h_stage_ + chunk_, rel.data(), (size_t)nw * sizeof(int));
        if (ntk_memcpy_h2d_async(tokens_dev_, h_stage_, (size_t)(nw > 0 ? chunk_ + nw : T) * sizeof(int), stream_) != NTK_OK) { err_ = "forward: the copy of the tokens failed"; return nullptr; }
        const int st = portion(slot, tokens_dev_, T, pos0 + at, want_dev_, w1 - done_want, logits_ + (size_t)done_want * info_.vocab);
        if (st != NTK_OK) { if (err_.empty()) err_ = std::string("forward: ") + ntk_status_string(st); return nullptr; }
        done_want = w1;
    }
    slots_.set_length(slot, pos0 + n);
    last_rows_ = n_want;
    return logits_;
}

int LayerStackModel::copy_logits(float* host, int rows) {
    if (!host || rows < 0 || rows > last_rows_) return NTK_E_SHAPE;
    LS_TRY(ntk_stream_synchronize(stream_));
    if (rows) nt_hip_memcpy_d2h(host, logits_, (size_t)rows * info_.vocab * sizeof(float));
    return NTK_OK;
}

int LayerStackModel::copy_capture(float* host) {
    if (!capture_buf_ || !capture_T_) return NTK_E_NULL;
    LS_TRY(ntk_stream_synchronize(stream_));
    nt_hip_memcpy_d2h(host, capture_buf_, runs_.size() * (size_t)capture_T_ * info_.width * sizeof(float));
    return NTK_OK;
}

int LayerStackModel::sync() { return ntk_stream_synchronize(stream_); }

}  // namespace nt
