/* include/ntransformer.h -- public C API of the MI355X-native engine.
 *
 * The first block is the reference's public header (reference include/ntransformer.h:12-38), name for name
 * and signature for signature, so an embedder of the reference re-links without source changes.  The
 * reference DECLARES this API but never implements it (no definition exists under reference src/); the
 * semantics below are the ones its header comments promise.  The second block are extensions.
 * No C++ exception crosses this boundary; every function tolerates a NULL engine.
 */
#ifndef NTRANSFORMER_H
#define NTRANSFORMER_H

#include <stddef.h>
#include <stdint.h>

/* the library is built with -fvisibility=hidden: exactly what this header declares is exported */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif
#ifdef __cplusplus
extern "C" {
#endif

typedef void* nt_engine_t;                       /* opaque handle */

nt_engine_t nt_engine_create(void);              /* never loads anything; NULL only on out-of-memory */
void        nt_engine_destroy(nt_engine_t engine);
int         nt_engine_load(nt_engine_t engine, const char* model_path);   /* 0 = ok (context capped at 4096 like the CLI default) */
/* Returns a malloc'd NUL-terminated UTF-8 string (free with nt_free), NULL on failure.
 * repeat_penalty / seed keep the reference's GenerateConfig defaults (1.1 / 42). */
char*       nt_engine_generate(nt_engine_t engine, const char* prompt, int max_tokens, float temperature,
                               int top_k, float top_p);
void        nt_free(char* ptr);
int         nt_engine_vocab_size(nt_engine_t engine);    /* -1 when no model is loaded */
int         nt_engine_n_layers(nt_engine_t engine);
int         nt_engine_hidden_size(nt_engine_t engine);

/* ------------------------------------------------------------------ extensions ------------------- */
typedef struct nt_gen_params {
    int      max_tokens;
    float    temperature;
    int      top_k;
    float    top_p;
    float    repeat_penalty;
    int      repeat_window;
    uint64_t seed;
    int      stop_at_eos;
} nt_gen_params;

typedef struct nt_stats {      /* Engine::Stats of the reference (engine.h:76-84) */
    int   prompt_tokens;
    int   gen_tokens;
    float prefill_ms;
    float decode_ms;
    float decode_tok_s;
} nt_stats;

typedef struct nt_synth_spec { /* seeded synthetic Llama-shaped model (no checkpoint exists offline) */
    int hidden, inter, layers, heads, kv_heads, vocab, ctx;
    float eps, theta;
    int bos, eos;
    const char* mix;           /* "Q8_0" "Q4_0" "Q4_K" "Q5_K" "Q6_K" "F16" "F32" "Q4_K_M" */
    uint64_t seed;
} nt_synth_spec;

int  nt_engine_load_ex(nt_engine_t e, const char* model_path, int max_context);
int  nt_engine_load_synthetic(nt_engine_t e, const nt_synth_spec* spec, int max_context);
/* A second SEQUENCE over the weights `src` already holds resident (the path shards across requests; sequences share nothing but the
 * read-only weights): `e` gets src's tensors (nothing is copied or owned), its own KV caches, activation buffers and HIP stream, so two host threads
 * can decode two requests on one GPU at once (bench.py: 8b_q8_0_x2_per_gpu).  `src` must outlive `e` and must not be re-loaded or change its
 * "repack" level meanwhile; a tensor-parallel source is refused (NTK_E_SHAPE). */
int  nt_engine_load_shared(nt_engine_t e, nt_engine_t src, int max_context);
/* "fused" / "graph" / "device_sampling" / "batched_prefill" / "f16_prefill" (alias "bf16_prefill") = "0" | "1"; "persistent" / "fuse_attention" are accepted
 * everywhere and take effect only in builds of experiments/ (experiments/ntk_experiments.h); "repack" = "0" raw-GGUF decode GEMVs | "1" load-time repack with the GGUF
 * bytes kept resident (K-quant weights twice in HBM) | "2" one resident copy: the GGUF bytes of a repacked matrix are freed and unpacked into a scratch
 * for the launches that read raw blocks (prompt GEMM, 1:1 sequence; a fixed cost per prompt pass) | "3" (default) "2" when both copies would leave less than
 * a fifth of the device's memory free, else "1"; "attention_merge" = "1" split-KV decode attention as one launch | "0" (default) with the separate merge
 * launch (identical results; the one-launch form measured slower) */
int  nt_engine_set_option(nt_engine_t e, const char* key, const char* value);
const char* nt_engine_last_error(nt_engine_t e);
void nt_gen_params_default(nt_gen_params* p);
/* The generate loop on token ids; writes up to out_cap generated ids, returns their count or a negative NTK_E_* */
int  nt_engine_generate_tokens(nt_engine_t e, const int* prompt, int n_prompt, const nt_gen_params* p, int* out, int out_cap);
int  nt_engine_last_stats(nt_engine_t e, nt_stats* out);
/* Transformer::forward: tokens [n] at start_pos -> logits of the last position copied to host (vocab floats) */
int  nt_engine_forward(nt_engine_t e, const int* tokens, int n, int start_pos, float* logits_out);
/* one fused decode step for `token` at position `pos` (device-resident state), logits copied to host */
int  nt_engine_decode_fused(nt_engine_t e, int token, int pos, int use_graph, float* logits_out);
/* n greedy decode steps from (token, pos): exactly the timed inner loop of generate (device argmax, one host
 * sync per token); generated ids to out[n] (may be NULL) */
int  nt_engine_decode_greedy_steps(nt_engine_t e, int token, int pos, int n, int* out);
/* one fused token launched eagerly and timed with HIP events on the compute stream:
 * ms4/calls4[0] quantised GEMV launches, [1] attention, [2] embedding + argmax + position; calls4[3] = timed intervals.
 * coarse = 0: an event pair around every launch; coarse = 1: one event per change of launch class (a run of GEMV
 * launches is timed as a whole: event cost paid once per run, the boundaries inside a run included) */
int  nt_engine_profile_token(nt_engine_t e, int token, int pos, int coarse, float* ms4, int* calls4);
int  nt_engine_tokenize(nt_engine_t e, const char* text, int add_bos, int* out, int out_cap);   /* returns count */
int  nt_engine_detokenize(nt_engine_t e, const int* ids, int n, char* out, int out_cap);       /* returns bytes */
uint64_t nt_engine_bytes_per_token(nt_engine_t e, int pos);   /* algorithmic HBM bytes of one decode token */
uint64_t nt_engine_weight_bytes(nt_engine_t e);            /* the model's tensors in their GGUF encoding */
uint64_t nt_engine_resident_weight_bytes(nt_engine_t e);   /* what they occupy in HBM now: GGUF bytes still resident + the decode repack + the unpack scratch */
uint64_t nt_engine_repacked_bytes(nt_engine_t e);          /* of which the decode repack (tensors that did not fit stay on the raw path and are not counted) */
int  nt_engine_max_context(nt_engine_t e);
/* ---- model folders -----------------------------------------------------------------------------------------------------------------
 * nt_engine_load(_ex) also takes a FOLDER with config.json + model.safetensors (dense bfloat16 weights); the model class is picked by the
 * config's "architecture" from the families built into the library.  Options, before the load: "dtype" = "bfloat16" (default: bf16 matrix
 * products with F32 sums; norms, rotations, attention scores and weights, routers and the residual stream in F32) | "float32" (everything in
 * true F32); "slots" = sequences the cache holds at once.  A folder holds no tokenizer: nt_engine_generate_tokens and nt_engine_forward work
 * on ids (nt_engine_forward uses slot 0, re-based at start_pos); nt_engine_generate and the GGUF path's other entry points return an error.
 * A sequence owns one slot of the cache from acquire to release (a released slot is handed out again as it is); nt_engine_seq_forward appends
 * n tokens to it -- a whole prompt, a portion of any size, one decoded token -- and copies the logits of the places want[0..n_want) (ascending
 * indices into these n tokens) to logits_out [n_want][vocab].  Logits of a position do not depend on how its sequence was cut into calls, beyond
 * rounding.  nt_engine_seq_capture(1): the next forwards keep the residual stream after every layer run, nt_engine_seq_copy_capture copies the
 * last call's [nt_engine_layer_runs][n][hidden] (parity instrumentation). */
int  nt_engine_is_sequence_model(nt_engine_t e);
int  nt_engine_layer_runs(nt_engine_t e);
int  nt_engine_seq_acquire(nt_engine_t e);                     /* slot id >= 0, or negative */
int  nt_engine_seq_release(nt_engine_t e, int slot);
int  nt_engine_seq_length(nt_engine_t e, int slot);
int  nt_engine_seq_truncate(nt_engine_t e, int slot, int length);
int  nt_engine_seq_forward(nt_engine_t e, int slot, const int* tokens, int n, const int* want, int n_want, float* logits_out);
int  nt_engine_seq_capture(nt_engine_t e, int on);
int  nt_engine_seq_copy_capture(nt_engine_t e, float* out);
/* which form the fused decode step takes at the current position: "fused (5 launches/layer)", or (EXPERIMENTS=1 builds with the
 * "persistent" option on) "persistent (...)" */
const char* nt_engine_decode_path(nt_engine_t e);
void* nt_engine_persistent_plan(nt_engine_t e);   /* plan handle for ntk_persistent_debug / ntk_layer_engine_debug; NULL outside EXPERIMENTS=1 builds */
int   nt_engine_persistent_kind(nt_engine_t e);   /* 0 none, 1 decode_persistent.hip, 2 layer_engine.hip ("persistent" = "2") */
/* Tensor-parallel decoding over `world` GPUs, one engine (normally one process) per rank -- SURVEY 8(f) rank 4, no reference
 * counterpart.  nt_engine_tp_configure BEFORE load: the engine then keeps rows [rank/world) of Wq/Wk/Wv/gate/up (whole heads) and
 * the matching columns of Wo/down; n_heads, n_kv_heads and the FFN width must divide by `world`, column slices must be whole
 * quantisation blocks.  After load: nt_engine_tp_export gives this rank's communication buffer as a 64-byte hipIpc handle
 * (other processes) and as a raw device pointer (ranks sharing a process); every rank then calls nt_engine_tp_connect with
 * world x 64 bytes of handles OR world raw pointers, in rank order.  Every rank must then run the same calls with the same
 * tokens: after Wo and after down the ranks' partial vectors are added in rank order by one kernel that reads the peers'
 * buffers over xGMI (ntk_tp_allreduce_add), so hidden states, logits and sampled tokens are bit-identical on all ranks.
 * nt_engine_tp_error after a call: 0, or non-zero if a bounded wait for a peer gave up. */
int  nt_engine_tp_configure(nt_engine_t e, int rank, int world);
int  nt_engine_tp_export(nt_engine_t e, void* handle64, void** raw_ptr);
int  nt_engine_tp_connect(nt_engine_t e, const void* handles, void* const* raw_ptrs);
unsigned nt_engine_tp_error(nt_engine_t e);
/* host only: columns [rank * in/world, (rank + 1) * in/world) of every row of a GGUF matrix, re-packed row-major into dst */
int  nt_tp_slice_columns(void* dst, const void* src, int dtype, int64_t out_features, int64_t in_features, int rank, int world);
/* ---- parity instrumentation (tests/test_parity_depth.py; never used by generate) --------------------------------------------
 * nt_engine_debug_run_layers: layers [first, first + count) of the loaded model on CALLER-SUPPLIED hidden states -- hidden_in
 * [n_tokens][hidden] (host) in, hidden_out [n_tokens][hidden] (host) out -- for tokens at positions start_pos...: layer-wise teacher
 * forcing against a checker (no error amplification through depth).  mode 0: the reference's 1:1 launcher sequence (prompt
 * projections batched or per token, as "batched_prefill" says); mode 1: the fused single-token launches (n_tokens == 1); mode 2: the
 * same captured into a hipGraph and replayed.  The layers write the KV-cache rows of these positions as in a normal forward.
 * nt_engine_debug_kv_read / _write: rows [pos0, pos0 + n) of one layer's K and V cache, [n][n_kv_heads * head_dim] IEEE halves. */
int  nt_engine_debug_run_layers(nt_engine_t e, const float* hidden_in, int n_tokens, int start_pos, int first_layer, int n_layers,
                                int mode, float* hidden_out);
int  nt_engine_debug_kv_read(nt_engine_t e, int layer, int pos0, int n, uint16_t* k_out, uint16_t* v_out);
int  nt_engine_debug_kv_write(nt_engine_t e, int layer, int pos0, int n, const uint16_t* k, const uint16_t* v);
/* write a synthetic GGUF v3 file with the same generator (0 = ok) */
int  nt_synth_write_gguf(const char* path, const nt_synth_spec* spec, int nthreads);
/* fill one tensor of the synthetic plan into host memory (for CPU baselines); returns bytes or negative */
int64_t nt_synth_tensor(const nt_synth_spec* spec, const char* name, void* dst, size_t dst_cap, int nthreads);


/* ------------------------------------------------------------------ host-only entry points ---------
 * GGUF parsing, tokenisation and sampling never touch the GPU; these let tools (and the CPU test-suite)
 * use them without a device. */
/* JSON description of a GGUF file: config, tensor table, vocab size. Returns bytes needed (excl. NUL) or negative. */
int   nt_gguf_describe(const char* path, char* json_out, int cap);
/* JSON description of a model FOLDER (config.json + model.safetensors): architecture, whether a family for it is built in, the families that are,
 * the tensor table (name, dtype, shape, bytes).  Returns bytes needed (excl. NUL) or a negative NTK_E_* (unreadable, malformed header, offsets that
 * do not fit a tensor's shape or the file). */
int   nt_model_folder_describe(const char* path, char* json_out, int cap);
typedef void* nt_tokenizer_t;
nt_tokenizer_t nt_tokenizer_open(const char* gguf_path);       /* NULL on failure */
void  nt_tokenizer_close(nt_tokenizer_t t);
int   nt_tokenizer_encode(nt_tokenizer_t t, const char* text, int text_len, int add_bos, int* out, int cap);
int   nt_tokenizer_decode(nt_tokenizer_t t, const int* ids, int n, char* out, int cap);
int   nt_tokenizer_is_gpt2(nt_tokenizer_t t);
/* n_draws successive Sampler::sample calls on the same logits (penalty applied once per draw over `recent`) */
int   nt_sampler_draw(const float* logits, int n, const nt_gen_params* p, const int* recent, int n_recent,
                      int n_draws, int* out);
/* the first n uniform draws a sampler seeded with `seed` consumes (one per sampled token) */
int   nt_sampler_uniforms(uint64_t seed, int n, float* out);

#ifdef __cplusplus
}
#endif
#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#endif /* NTRANSFORMER_H */
