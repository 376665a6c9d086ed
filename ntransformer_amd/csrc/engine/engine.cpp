// engine/engine.cpp -- see engine.h
#include "engine.h"
#include "safetensors.h"
#include "../../../include/ntk_engine.h"

#include <chrono>
#include <cstdio>
#include <iostream>
#include <thread>

namespace nt {

using Clock = std::chrono::high_resolution_clock;
static float ms_since(Clock::time_point t0) { return std::chrono::duration<float, std::milli>(Clock::now() - t0).count(); }

int Engine::load(const std::string& path, int max_context) {
    loaded_ = false;
    seq_.reset();
    if (ModelFolder::looks_like(path)) {
        SeqLoadOptions o;
        o.max_context = max_context;
        o.slots = opt_.slots > 0 ? opt_.slots : 1;
        o.float32 = opt_.float32;
        seq_ = open_model(path, o, &err_);
        if (!seq_) return NTK_E_FORMAT;
        loaded_ = true;
        return NTK_OK;
    }
    const int st = model_.load(path, max_context);
    if (st != NTK_OK) { err_ = model_.error(); return st; }
    tok_.init(model_.vocab(), model_.config().bos_token_id, model_.config().eos_token_id);   // engine.cpp:21
    loaded_ = true;
    return NTK_OK;
}

int Engine::load_synthetic(const SynthSpec& spec, int max_context) {
    loaded_ = false;
    seq_.reset();
    int nt = opt_.synth_threads > 0 ? opt_.synth_threads : (int)std::thread::hardware_concurrency();
    const int st = model_.load_synthetic(spec, max_context, nt > 0 ? nt : 8);
    if (st != NTK_OK) { err_ = model_.error(); return st; }
    tok_.init(model_.vocab(), model_.config().bos_token_id, model_.config().eos_token_id);
    loaded_ = true;
    return NTK_OK;
}

int Engine::load_shared(Engine& src, int max_context) {
    loaded_ = false;
    if (!src.loaded_) { err_ = "load_shared: the source engine is not loaded"; return NTK_E_NULL; }
    if (src.seq_) { err_ = "load_shared: a model folder serves several sequences from the slots of ONE engine (option \"slots\")"; return NTK_E_SHAPE; }
    seq_.reset();
    const int st = model_.share_weights(src.model_, max_context);
    if (st != NTK_OK) { err_ = model_.error(); return st; }
    tok_.init(model_.vocab(), model_.config().bos_token_id, model_.config().eos_token_id);
    loaded_ = true;
    return NTK_OK;
}

// One generation, reference engine.cpp:40-145 step for step:
//   prefill (timed) -> logits -> repeat penalty -> sample first token -> decode loop (timed as a whole;
//   gen_tokens counts loop iterations, so the first sampled token is not counted) -> stop at EOS.
// `tokens` holds the prompt on entry and prompt + generated ids on return.
int Engine::run(std::vector<int>& tokens, const GenerateConfig& cfg, std::string* text, TokenCallback cb, bool print, bool stop_at_eos) {
    stats_ = Stats();
    if (!loaded_) { err_ = "model not loaded"; return NTK_E_NULL; }
    if (tokens.empty()) { err_ = "empty prompt"; return NTK_E_SHAPE; }
    if (seq_) return run_sequence(tokens, cfg, cb, stop_at_eos);
    Sampler sampler;
    SamplerConfig sc;
    sc.temperature = cfg.temperature; sc.top_k = cfg.top_k; sc.top_p = cfg.top_p;
    sc.repeat_penalty = cfg.repeat_penalty; sc.repeat_window = cfg.repeat_window; sc.seed = cfg.seed;
    sampler.init(sc);
    const int V = model_.config().vocab_size;
    const int eos = tok_.eos_id();
    const bool dev_greedy = opt_.fused && opt_.device_sampling && sampler.is_pure_greedy();
    // temperature / top-k / top-p / repeat penalty on the device too (ntk_sample_top_k): the host only draws the uniform number
    const bool dev_sample = opt_.fused && opt_.device_sampling && !dev_greedy &&
                            Model::device_sampler_supports(cfg.temperature, cfg.top_k, V);
    stats_.prompt_tokens = (int)tokens.size();
    if (cfg.verbose) fprintf(stderr, "Prompt tokens: %d\n", stats_.prompt_tokens);

    auto t0 = Clock::now();
    model_.set_batched_prefill(opt_.batched_prefill);
    float* logits = model_.forward(tokens.data(), (int)tokens.size(), 0);
    stats_.prefill_ms = ms_since(t0);
    if (!logits) { err_ = model_.error(); return NTK_E_LAUNCH; }

    std::vector<float> host(V);
    if (model_.copy_logits(host.data()) != NTK_OK) return NTK_E_LAUNCH;
    sampler.apply_repeat_penalty(host.data(), V, tokens);
    int next = sampler.sample(host.data(), V);
    tokens.push_back(next);
    auto emit = [&](int id) -> bool {
        const std::string piece = tok_.decode_token(id);
        if (text) *text += piece;
        if (cb) return cb(piece, id);
        if (print) { fputs(piece.c_str(), stdout); fflush(stdout); }
        return true;
    };
    if (!emit(next)) return NTK_OK;

    int pos = stats_.prompt_tokens;
    const int max_pos = model_.config().max_seq_len;
    int rc = NTK_OK;
    auto d0 = Clock::now();
    if (opt_.fused) {
        model_.set_device_pos(pos);
        model_.set_device_token(next);
    }
    // Greedy decoding on the device keeps ONE step queued ahead of the token the host is waiting for: the token id feeds the next step
    // on the device, so the next step's launches need nothing from the host, and the host's per-token work (poll, EOS check, detokenise,
    // graph launch) overlaps the GPU's.  A step queued behind what turns out to be EOS is discarded (one KV row past the end, harmless).
    int queued = 0;   // greedy steps launched and not yet consumed
    for (int i = 1; i < cfg.max_tokens; ++i) {
        if (stop_at_eos && next == eos) break;              // engine.cpp:106
        if (pos >= max_pos) { fprintf(stderr, "\n[context of %d tokens exhausted]\n", max_pos); break; }
        if (opt_.fused) {
            if (dev_greedy) {
                if (queued == 0) { if ((rc = model_.decode_step_fused(true, opt_.graph)) != NTK_OK) break; ++queued; }
                if (i + 1 < cfg.max_tokens && pos + 1 < max_pos) {   // the step after this one, before this one's token is known
                    if ((rc = model_.decode_step_fused(true, opt_.graph)) != NTK_OK) break;
                    ++queued;
                }
                if ((rc = model_.wait_token(pos, &next)) != NTK_OK) break;   // first max, same as Sampler::argmax
                --queued;
            } else {
            rc = model_.decode_step_fused(false, opt_.graph);
            if (rc != NTK_OK) break;
            if (dev_sample) {
                const int have = (int)tokens.size(), win = std::min(have, cfg.repeat_window);   // sampler.cpp:34
                const float r = cfg.temperature > 0.0f ? sampler.draw() : 0.0f;                  // greedy takes no draw
                rc = model_.sample_on_device(tokens.data() + have - win, win, cfg.repeat_penalty, cfg.temperature, cfg.top_k,
                                             cfg.top_p, r);
                if (rc == NTK_OK) rc = model_.sync();
                if (rc != NTK_OK) break;
                next = model_.host_token();
            } else {
                if ((rc = model_.copy_logits(host.data())) != NTK_OK) break;
                sampler.apply_repeat_penalty(host.data(), V, tokens);
                next = sampler.sample(host.data(), V);
                model_.set_device_token(next);
            }
            }
        } else {
            logits = model_.forward(&next, 1, pos);          // engine.cpp:109
            if (!logits) { rc = NTK_E_LAUNCH; break; }
            if ((rc = model_.copy_logits(host.data())) != NTK_OK) break;
            sampler.apply_repeat_penalty(host.data(), V, tokens);
            next = sampler.sample(host.data(), V);
        }
        ++pos;
        tokens.push_back(next);
        ++stats_.gen_tokens;
        if (!emit(next)) break;
    }
    // the loop's wall time, as the reference counts it (engine.cpp:102-134): up to the last token the host saw.  A run-ahead step queued
    // behind what turned out to be the end (EOS, the callback, the token budget) is drained AFTER the clock stops: it decoded no counted
    // token.  (After run() the device position and the KV cache may therefore be one step past the returned tokens; every run re-bases
    // both -- set_device_pos -- before it decodes.)
    stats_.decode_ms = ms_since(d0);
    if (opt_.fused) { const int sr = model_.sync(); if (rc == NTK_OK) rc = sr; }
    if (rc == NTK_OK && opt_.fused) rc = model_.check_persistent();
    if (rc != NTK_OK) err_ = std::string("decode failed: ") + ntk_status_string(rc);
    return rc;
}

// The generation loop of a model folder: one slot of the family's cache, the prompt in one forward (the family cuts it into its own passes), then
// one token per forward; the reference's sampler and repeat penalty on the host (engine.cpp:66-134).  Tokens are ids: a folder has no tokenizer, so the
// callback gets an empty piece and the id.
int Engine::run_sequence(std::vector<int>& tokens, const GenerateConfig& cfg, TokenCallback cb, bool stop_at_eos) {
    Sampler sampler;
    SamplerConfig sc;
    sc.temperature = cfg.temperature; sc.top_k = cfg.top_k; sc.top_p = cfg.top_p;
    sc.repeat_penalty = cfg.repeat_penalty; sc.repeat_window = cfg.repeat_window; sc.seed = cfg.seed;
    sampler.init(sc);
    const int V = seq_->info().vocab, eos = seq_->info().eos;
    stats_.prompt_tokens = (int)tokens.size();
    const int slot = seq_->acquire_slot();
    if (slot < 0) { err_ = "every slot of the cache is taken"; return NTK_E_NOMEM; }
    int rc = NTK_OK;
    std::vector<float> host((size_t)V);
    auto step = [&](const int* t, int n) -> int {
        const int last = n - 1;
        if (!seq_->forward(slot, t, n, &last, 1)) { err_ = seq_->error(); return NTK_E_LAUNCH; }
        return seq_->copy_logits(host.data(), 1);
    };
    auto t0 = Clock::now();
    rc = step(tokens.data(), (int)tokens.size());
    stats_.prefill_ms = ms_since(t0);
    if (rc == NTK_OK) {
        sampler.apply_repeat_penalty(host.data(), V, tokens);
        int next = sampler.sample(host.data(), V);
        tokens.push_back(next);
        bool go = !cb || cb(std::string(), next);
        auto d0 = Clock::now();
        for (int i = 1; go && i < cfg.max_tokens; ++i) {
            if (stop_at_eos && eos >= 0 && next == eos) break;
            if (seq_->slot_length(slot) >= seq_->info().max_context) break;
            if ((rc = step(&next, 1)) != NTK_OK) break;
            sampler.apply_repeat_penalty(host.data(), V, tokens);
            next = sampler.sample(host.data(), V);
            tokens.push_back(next);
            ++stats_.gen_tokens;
            if (cb && !cb(std::string(), next)) break;
        }
        stats_.decode_ms = ms_since(d0);
    }
    seq_->release_slot(slot);
    if (rc != NTK_OK && err_.empty()) err_ = std::string("decode failed: ") + ntk_status_string(rc);
    return rc;
}

int Engine::decode_greedy_steps(int token, int pos, int n, int* out) {
    if (!loaded_) return NTK_E_NULL;
    if (seq_) { err_ = "decode_greedy_steps: a model folder decodes through generate_tokens / the nt_engine_seq_* calls"; return NTK_E_SHAPE; }
    if (pos < 0 || pos + n > model_.config().max_seq_len) return NTK_E_SHAPE;
    int next = token;
    if (opt_.fused) {
        model_.set_device_pos(pos);
        model_.set_device_token(next);
        // exactly n steps, one always queued ahead of the token the host is waiting for (see Engine::run); the host still sees every
        // token, in order, as Engine::generate does
        int launched = 0;
        for (int i = 0; i < n; ++i) {
            while (launched < n && launched <= i + 1) {
                const int rc = model_.decode_step_fused(true, opt_.graph);
                if (rc != NTK_OK) return rc;
                ++launched;
            }
            const int rc = model_.wait_token(pos + i, &next);
            if (rc != NTK_OK) return rc;
            if (out) out[i] = next;
        }
        { const int rc = model_.sync(); if (rc != NTK_OK) return rc; }
        return model_.check_persistent();   // a bounded in-kernel wait that gave up invalidates the run (and disables the path)
    }
    std::vector<float> host(model_.config().vocab_size);
    for (int i = 0; i < n; ++i) {
        if (!model_.forward(&next, 1, pos + i)) return NTK_E_LAUNCH;
        if (model_.copy_logits(host.data()) != NTK_OK) return NTK_E_LAUNCH;
        next = Sampler::argmax(host.data(), (int)host.size());
        if (out) out[i] = next;
    }
    return NTK_OK;
}

std::string Engine::generate(const std::string& prompt, const GenerateConfig& cfg, TokenCallback cb) {
    if (seq_) { err_ = "a model folder has no tokenizer: generate on token ids (generate_tokens, --tokens)"; return std::string(); }
    std::vector<int> tokens = tok_.encode(prompt, true);
    std::string out;
    run(tokens, cfg, &out, cb, cfg.verbose, true);
    if (cfg.verbose) { fprintf(stdout, "\n"); print_stats(stats_); }
    return out;
}

int Engine::generate_tokens(const std::vector<int>& prompt, const GenerateConfig& cfg, std::vector<int>& out, bool stop_at_eos) {
    std::vector<int> tokens = prompt;
    GenerateConfig c = cfg;
    c.verbose = false;
    const int rc = run(tokens, c, nullptr, nullptr, false, stop_at_eos);
    out.assign(tokens.begin() + (long)prompt.size(), tokens.end());
    return rc;
}

void Engine::chat(const GenerateConfig& cfg) {   // engine.cpp:545-570: stateless turns
    if (seq_) { fprintf(stderr, "chat needs a tokenizer; a model folder has none (use --tokens)\n"); return; }
    fprintf(stdout, "NTransformer Chat (type 'quit' to exit)\nModel: %s (%d params)\n---\n", model_.config().model_name.c_str(),
            model_.config().n_layers);
    std::string line;
    for (;;) {
        fprintf(stdout, "> ");
        fflush(stdout);
        if (!std::getline(std::cin, line)) break;
        if (line == "quit" || line == "exit") break;
        if (line.empty()) continue;
        generate(line, cfg);
        fprintf(stdout, "\n");
    }
}

void Engine::benchmark(const std::string& prompt, int n_tokens) {   // engine.cpp:572-593
    GenerateConfig c;
    c.max_tokens = n_tokens;
    c.temperature = 0.0f;
    c.verbose = false;
    fprintf(stderr, "=== Benchmark ===\nPrompt: \"%s\"\nMax tokens: %d\n", prompt.c_str(), n_tokens);
    auto t0 = Clock::now();
    const std::string out = generate(prompt, c);
    fprintf(stderr, "Total time: %.1f ms\nOutput length: %zu chars\n", ms_since(t0), out.size());
    print_stats(stats_);   // the reference prints nothing here because verbose is false; the numbers are the point of a benchmark
}

void Engine::print_stats(const Stats& st) const {   // engine.cpp:595-607
    fprintf(stderr, "\n--- Stats ---\n");
    fprintf(stderr, "Prompt: %d tokens, %.1f ms (%.1f tok/s)\n", st.prompt_tokens, st.prefill_ms, st.prefill_tok_s());
    fprintf(stderr, "Decode: %d tokens, %.1f ms (%.1f tok/s)\n", st.gen_tokens, st.decode_ms, st.decode_tok_s());
    size_t fr = 0, tot = 0;
    ntk_device_mem_info(&fr, &tot);
    fprintf(stderr, "VRAM: %.1f / %.1f GB\n", (tot - fr) / 1073741824.0, tot / 1073741824.0);
}

}  // namespace nt
