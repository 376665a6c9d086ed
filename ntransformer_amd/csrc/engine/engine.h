// engine/engine.h -- text generation loop and its statistics.
// Replaces reference src/inference/engine.{h,cpp}: Engine::load / generate / chat / benchmark / print_stats.
// The speculative and self-speculative variants (engine.cpp:150-540) depend on the tiered streaming mode
// and are out of scope.
#pragma once
#include <functional>
#include <string>
#include <vector>
#include "model.h"
#include "sampler.h"
#include "sequence_model.h"
#include "tokenizer.h"

namespace nt {

struct GenerateConfig {   // reference engine.h:17-26, same defaults
    int max_tokens = 256;
    float temperature = 0.7f;
    int top_k = 40;
    float top_p = 0.9f;
    float repeat_penalty = 1.1f;
    int repeat_window = 64;
    uint64_t seed = 42;
    bool verbose = true;
};

struct Stats {            // reference engine.h:76-84
    int prompt_tokens = 0;
    int gen_tokens = 0;
    float prefill_ms = 0;
    float decode_ms = 0;
    float prefill_tok_s() const { return prefill_ms > 0 ? prompt_tokens / (prefill_ms / 1000.0f) : 0.0f; }
    float decode_tok_s() const { return decode_ms > 0 ? gen_tokens / (decode_ms / 1000.0f) : 0.0f; }
};

using TokenCallback = std::function<bool(const std::string& piece, int token_id)>;

struct EngineOptions {
    bool fused = true;            // fused 5-launch/layer decode path (false: the reference's 15-launch sequence)
    bool graph = true;            // replay the fused token from a hipGraph
    bool batched_prefill = true;  // prompts: one pass over each weight matrix per 16 tokens (false: per-token GEMV loops)
    bool device_sampling = true;  // greedy argmax on the device when temperature <= 0 and repeat_penalty <= 1
    bool persistent = false;      // short contexts: the whole token in one persistent launch (decode_persistent.hip)
    int synth_threads = 0;        // 0 = hardware concurrency
    // model folders (config.json + model.safetensors, engine/sequence_model.h); read by load()
    bool float32 = false;         // every product in true F32 instead of bf16 products with F32 sums
    int slots = 1;                // sequences the cache holds at once (generate uses one; the nt_engine_seq_* calls may hold the others)
};

class Engine {
public:
    int load(const std::string& path, int max_context = 4096);
    int load_synthetic(const SynthSpec& spec, int max_context = 4096);
    // a second sequence over the weights `src` holds resident (Model::share_weights): own caches, buffers and stream; `src` must outlive this engine
    int load_shared(Engine& src, int max_context = 4096);
    std::string generate(const std::string& prompt, const GenerateConfig& cfg, TokenCallback cb = nullptr);
    // the generate loop on token ids (no tokenizer, no printing): used by bench.py and the parity tests
    int generate_tokens(const std::vector<int>& prompt, const GenerateConfig& cfg, std::vector<int>& out, bool stop_at_eos);
    // n greedy decode steps continuing from (token, pos): the timed inner loop of run(), nothing else.
    int decode_greedy_steps(int token, int pos, int n, int* out);
    void chat(const GenerateConfig& cfg);
    void benchmark(const std::string& prompt, int n_tokens);
    void print_stats(const Stats& st) const;

    // A model FOLDER loads through the family registry (engine/sequence_model.h) instead of nt::Model; generation then runs on token ids
    // (a folder holds no tokenizer), through the same sampler, one slot of the family's cache per generation.
    bool is_sequence_model() const { return seq_ != nullptr; }
    SequenceModel* sequence_model() { return seq_.get(); }
    int vocab_size() const { return seq_ ? seq_->info().vocab : model_.config().vocab_size; }
    int n_layers() const { return seq_ ? seq_->info().n_layers : model_.config().n_layers; }
    int hidden_size() const { return seq_ ? seq_->info().width : model_.config().hidden_size; }
    int max_context() const { return seq_ ? seq_->info().max_context : model_.config().max_seq_len; }

    Model& model() { return model_; }
    const Tokenizer& tokenizer() const { return tok_; }
    const Stats& last_stats() const { return stats_; }
    EngineOptions& options() { return opt_; }
    const std::string& error() const { return err_; }
    bool loaded() const { return loaded_; }

private:
    int run(std::vector<int>& tokens, const GenerateConfig& cfg, std::string* text, TokenCallback cb, bool print, bool stop_at_eos);
    int run_sequence(std::vector<int>& tokens, const GenerateConfig& cfg, TokenCallback cb, bool stop_at_eos);
    std::unique_ptr<SequenceModel> seq_;
    Model model_;
    Tokenizer tok_;
    Stats stats_;
    EngineOptions opt_;
    std::string err_;
    bool loaded_ = false;
};

}  // namespace nt
