/*
 * gradhip — MI355X (gfx950) implementation of grad.cpp's KV-cached token loop.
 *
 * Plain C ABI: opaque handles, plain pointers and sizes, status codes.  Each
 * entry point names the grad.cpp interface it stands in for (paths relative to
 * the grad.cpp source tree).  All arithmetic is fp32; token ids are int32.
 *
 * Threading: a model handle is immutable after creation and may be shared by
 * sessions on different host threads.  A session owns one HIP stream; calls on
 * one session must be serialised by the caller (grad.cpp's InferenceSession
 * and TextGen are not thread-safe either).  Sessions on the one-launch engine
 * (batch 1, the shapes it is built for) take turns inside the library: its
 * kernel needs the whole GPU, so a call that launches it holds a process-wide
 * lock until the launch has finished; results do not depend on the order.
 *
 * There is no CPU fallback: every compute entry point fails with
 * GH_ERR_DEVICE when no gfx950 device is usable.
 */
#ifndef GRADHIP_H
#define GRADHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct gh_model gh_model;
typedef struct gh_session gh_session;

/* Status codes.  1..3 name the C++ exception type grad.cpp throws at the same
 * point (std::runtime_error, std::out_of_range, std::invalid_argument); the
 * C++ adapter in gradhip.hpp rethrows exactly those. */
typedef enum gh_status {
    GH_OK = 0,
    GH_ERR_RUNTIME = 1,
    GH_ERR_OUT_OF_RANGE = 2,
    GH_ERR_INVALID_ARGUMENT = 3,
    GH_ERR_DEVICE = 4 /* HIP failure or no usable GPU; surfaces as runtime_error */
} gh_status;

/* Message of the last failure on the calling thread (never NULL). */
const char* gh_last_error(void);

enum { GH_ARCH_GPT2 = 0, GH_ARCH_MODERN = 1 }; /* GPTArch, gpt_model.h:31 */

/* Hyper-parameters of a checkpoint: the header of GPTModel::save
 * (gpt_model.cpp:302-314) plus the derived FFN width (feedforward.h:24-28) and
 * the optional tokenizer fingerprint trailer (gpt_model.cpp:357-363). */
typedef struct gh_config {
    int32_t arch;
    int32_t vocab;
    int32_t d_model;
    int32_t layers;
    int32_t heads;
    int32_t max_len;
    int32_t d_ff;
    float dropout;
    int32_t has_fingerprint;
    uint32_t tokenizer_kind; /* 1 = v1 whitespace BPE, 2 = byte-level BPE */
    uint64_t tokenizer_hash;
} gh_config;

/* ------------------------------------------------------------------ model */

/* GPTModel::load (gpt_model.cpp:383-525): reads a "GPTM" v1/v2 file with the
 * same validation order and the same error texts, then uploads the weights.
 * Unlike the reference it prints nothing on success. */
gh_status gh_model_load(const char* path, gh_model** out);

/* Builds a model from host tensors in checkpoint order (gpt_model.cpp:318-355):
 * E; P (GPT-2 only); per layer W_q W_k W_v W_o b_q b_k b_v b_o, then gate up
 * down (Modern) or W1 b1 W2 b2 (GPT-2), then norm1 gamma beta, norm2 gamma
 * beta; final gamma beta.  Matrices are (in, out) row-major as grad.cpp stores
 * them.  cfg->d_ff is ignored (derived).  Stands in for constructing a
 * GPTModel and assigning its parameters. */
gh_status gh_model_from_host(const gh_config* cfg, const float* const* tensors, int32_t n_tensors,
                             gh_model** out);

/* Number of tensors a checkpoint of this shape holds, and the shape of each. */
int32_t gh_config_num_tensors(const gh_config* cfg);
gh_status gh_config_tensor_shape(const gh_config* cfg, int32_t index, int32_t* rows, int32_t* cols);

/* GPTModel::save (gpt_model.cpp:292-381): writes a v2 file, bitwise equal to
 * the file the model was loaded from (weights are read back from the GPU). */
gh_status gh_model_save(const gh_model* m, const char* path);

void gh_model_free(gh_model* m);
gh_status gh_model_get_config(const gh_model* m, gh_config* out);

/* ---------------------------------------------------------------- session */

typedef enum gh_engine {
    GH_ENGINE_AUTO = 0,
    GH_ENGINE_GRAPH = 1,     /* one kernel per fused op, whole step replayed as a hipGraph */
    GH_ENGINE_EAGER = 2,     /* same kernels launched one by one (debugging, profiling) */
    GH_ENGINE_PERSISTENT = 3 /* one cooperative kernel per step; batch 1 only */
} gh_engine;

typedef struct gh_session_opts {
    int32_t batch;       /* independent sequences decoded in lock step (>= 1) */
    int32_t engine;      /* gh_engine */
    int32_t page_tokens; /* KV-cache page size in positions; 0 = default (64) */
    int32_t shuffle_pages; /* non-zero: hand out physical pages in a scrambled order */
    int32_t flags;         /* GH_FLAG_* */
} gh_session_opts;

/* Keep the sampler's working row in global memory even when it would fit in
 * LDS (the path vocabularies above ~38k entries take); for testing that path. */
enum { GH_FLAG_PICK_GLOBAL_SCRATCH = 1 };

/* Feed prompts token by token (one step() each, as text_gen.cpp:44-46 does)
 * instead of pushing all prompt tokens through each layer at once. */
enum { GH_FLAG_STEPWISE_PROMPT = 2 };

/* Split every (sequence, head) of the decode attention into runs of 16 cache
 * positions, each on a workgroup of its own, instead of the 256 or 512 the
 * session would choose; for testing the merge of partial results at short
 * contexts. */
enum { GH_FLAG_SMALL_ATTENTION_CHUNKS = 4 };

/* The persistent engine has two kernels for the Llama block at d_model 768: one in
 * which every phase of a layer is exchanged among all 256 workgroups (and a head's
 * context beyond 512 positions is shared among idle workgroups), and one that splits a
 * layer over the eight XCDs and streams the weights through LDS.  The first is the
 * faster at every context and the default; GH_FLAG_XCD_PERSISTENT selects the second
 * for every launch of the session (for comparing the kernels and for tests), and
 * GH_FLAG_CLASSIC_PERSISTENT names the default explicitly.  The two exclude each other. */
enum { GH_FLAG_CLASSIC_PERSISTENT = 8 };
enum { GH_FLAG_XCD_PERSISTENT = 16 };

/* In the all-to-all persistent kernel a greedy pick, and a pick with 0 < top_k <= 64,
 * that follows a step of the same launch is made by every workgroup at once from a
 * few candidates per workgroup; every other pick by one workgroup from the whole row
 * of logits.  This flag leaves every pick to the one workgroup, for comparing the two
 * and for tests. */
enum { GH_FLAG_ROW_PICKS = 32 };

/* InferenceSession::InferenceSession (inference.cpp:121-148): allocates the
 * paged KV cache (2 * layers * max_len * d_model floats per sequence) and the
 * per-step scratch, and records the step graph. */
gh_status gh_session_create(const gh_model* m, const gh_session_opts* opts, gh_session** out);
void gh_session_free(gh_session* s);

/* Forgets the context: position 0, empty token history. */
gh_status gh_session_reset(gh_session* s);

/* InferenceSession::step (inference.cpp:150-258) for every sequence of the
 * batch: appends ids[b] to sequence b and computes the next-token logits.
 * logits_host, when non-NULL, receives batch * vocab floats.  Errors as the
 * reference: GH_ERR_RUNTIME "InferenceSession: context exceeds max_len",
 * GH_ERR_OUT_OF_RANGE "InferenceSession: token id out of vocab range". */
gh_status gh_session_step(gh_session* s, const int32_t* ids, float* logits_host);

/* Logits of the last step in session-owned pinned host memory, valid until the
 * next call on the session (the "valid until the next step() call" rule of
 * inference.h:20-22).  batch * vocab floats. */
gh_status gh_session_logits(gh_session* s, const float** logits);

/* Feeds `len` tokens per sequence (ids is batch x len, row-major) in one call;
 * equivalent to `len` step() calls (text_gen.cpp:44-46) whose logits are
 * dropped except the last.  Prompts of 8 tokens and more go through each layer
 * in one pass (matrix-core projections over all tokens, causal attention over
 * the cache they fill).  last_logits_host may be NULL. */
gh_status gh_session_prefill(gh_session* s, const int32_t* ids, int32_t len,
                             float* last_logits_host);

int32_t gh_session_position(const gh_session* s); /* inference.h:27 */
int32_t gh_session_capacity(const gh_session* s); /* inference.h:28 */
int32_t gh_session_vocab(const gh_session* s);    /* inference.h:29 */
int32_t gh_session_batch(const gh_session* s);

/* Copies K (kv = 0, after RoPE) or V (kv = 1) row `pos` of `layer` for sequence
 * `seq` out of the paged cache: d_model floats in the reference's row layout
 * (inference.cpp:195-196). */
gh_status gh_session_read_kv(gh_session* s, int32_t seq, int32_t layer, int32_t kv, int32_t pos,
                             float* out_host);

/* --------------------------------------------------------------- sampling */

/* SamplingOptions (src/cli/common.h:140-147) as TextGen takes them
 * (text_gen.h:23-37).  greedy != 0 selects generate_greedy's arg-max. */
typedef struct gh_sampling {
    float temperature;
    int32_t top_k; /* 0 = off */
    float top_p;   /* 1 = off */
    float repetition_penalty;
    int32_t greedy;
} gh_sampling;

/* One pick from the current logits of every sequence, on the GPU:
 * logits_with_penalty (text_gen.cpp:14-33) over the session's token history,
 * then arg-max (text_gen.cpp:52-60) or sample_from_logits (text_gen.cpp:135-209).
 * uniforms: one float per sequence, or NULL to draw Philox4x32-10(seed,
 * sequence, pick index).  The picked ids are written to out_ids (batch int32)
 * but not stepped: the history the penalty looks at is the tokens stepped so
 * far, so pass the pick (or another id) to gh_session_step next. */
gh_status gh_session_pick(gh_session* s, const gh_sampling* opt, const float* uniforms,
                          uint64_t seed, int32_t* out_ids);

/* The decode loop of TextGen::generate_* (text_gen.cpp:48-64, :80-89) continued
 * from the session's current context: up to max_tokens rounds of pick, push,
 * stop at capacity, else step.  out_ids (batch x max_tokens, row stride
 * max_tokens) receives the picks, *out_count how many were made per sequence.
 * uniforms is batch x max_tokens or NULL (on-device Philox; the draw index
 * continues across calls).  This is what a chat turn that keeps its cache
 * calls after gh_session_prefill. */
gh_status gh_session_decode(gh_session* s, int32_t max_tokens, const gh_sampling* opt,
                            const float* uniforms, uint64_t seed, int32_t* out_ids,
                            int32_t* out_count);

/* Receives the picks of one round (ids[b] for sequence b; index counts rounds
 * from 0) as soon as they exist.  A nonzero return asks for the run to end. */
typedef int32_t (*gh_token_callback)(void* user, const int32_t* ids, int32_t index);

/* TextGen::generate_stream's loop (text_gen.cpp:107-118) continued from the
 * session's current context: gh_session_decode with every round's picks handed
 * to on_tokens as they are made, plus two ways to end before max_tokens, which
 * the reference lacks (its loop always runs to max_tokens or capacity):
 *   stop_token >= 0: the run ends once every sequence has picked that id (an
 *     end-of-text id); the round that picked it is completed (pushed and stepped);
 *   on_tokens returns nonzero: the run ends as soon as the device learns of it.
 * With one sequence on the persistent engine the whole loop is ONE kernel launch
 * that writes each pick to pinned host memory while it goes on computing, and the
 * calling thread runs on_tokens beside it: a request to stop takes effect a round
 * or two later, and those rounds' picks are still delivered.  Every round that is
 * delivered is complete, so *out_count rounds later the session is exactly where
 * gh_session_decode with max_tokens = *out_count would have left it, and a later
 * call continues the same stream of picks.  on_tokens must not call into this
 * session.  out_ids (batch x max_tokens, may be NULL), uniforms and seed as in
 * gh_session_decode. */
gh_status gh_session_decode_stream(gh_session* s, int32_t max_tokens, const gh_sampling* opt,
                                   const float* uniforms, uint64_t seed, int32_t stop_token,
                                   gh_token_callback on_tokens, void* user, int32_t* out_ids,
                                   int32_t* out_count);

/* TextGen::generate_greedy / generate_sample (text_gen.cpp:37-91) for `batch`
 * prompts of equal length, with the token loop kept on the GPU.  prompts is
 * batch x prompt_len; out_tokens is batch x (prompt_len + max_tokens) and
 * receives prompt + generated ids; *out_len their count per sequence.
 * uniforms is batch x max_tokens (draw i of sequence b at [b * max_tokens + i])
 * or NULL for the on-device Philox stream.  The session is reset first.
 * step_logits_host, when non-NULL, receives the logits of every step() call
 * (steps x batch x vocab) and *n_steps their count. */
gh_status gh_session_generate(gh_session* s, const int32_t* prompts, int32_t prompt_len,
                              int32_t max_tokens, const gh_sampling* opt, const float* uniforms,
                              uint64_t seed, int32_t* out_tokens, int32_t* out_len,
                              float* step_logits_host, int32_t* n_steps);

/* -------------------------------------------------------------- tokenizer */

/* Host-side text <-> ids for the two ends of the token loop.  Runs on the CPU
 * (as in grad.cpp); nothing here touches the GPU. */
typedef struct gh_tokenizer gh_tokenizer;

typedef struct gh_tokenizer_info {
    uint32_t kind;        /* TokenizerKind, fingerprint.h:15-18: 1 = v1 whitespace BPE, 2 = byte-level BPE */
    int32_t vocab_size;   /* Tokenizer::vocab_size */
    int32_t eos_id;       /* Tokenizer::eos_id ("<|endoftext|>"; "<eos>" for v1), -1 when absent */
    int32_t n_merges;
    int32_t n_specials;
    uint64_t fingerprint; /* Tokenizer::fingerprint; what a checkpoint's TKFP trailer records */
} gh_tokenizer_info;

/* load_tokenizer (tokenizer.h:52, tokenizer.cpp:119-124): a file that starts
 * with "GTOK" is a v2 file (ByteBpe::load, byte_bpe.cpp:676-744), anything else
 * is taken for a v1 cache (BPETokenizer::load, bpe_tokenizer.cpp:373-417, with
 * 64-bit size_t and 32-bit int fields); same validation and messages. */
gh_status gh_tokenizer_load(const char* path, gh_tokenizer** out);
/* ByteBpe(merges, specials) (byte_bpe.h:50-53): merges is n_merges x 2 ids;
 * specials[i] has special_lens[i] bytes.  GH_ERR_INVALID_ARGUMENT with the
 * constructor's messages. */
gh_status gh_tokenizer_from_merges(const int32_t* merges, int32_t n_merges, const char* const* specials,
                                   const int32_t* special_lens, int32_t n_specials, gh_tokenizer** out);
/* Tokenizer::save (byte_bpe.cpp:655-674): writes a file grad.cpp loads. */
gh_status gh_tokenizer_save(const gh_tokenizer* t, const char* path);
void gh_tokenizer_free(gh_tokenizer* t);
gh_status gh_tokenizer_get_info(const gh_tokenizer* t, gh_tokenizer_info* out);
/* Tokenizer::special_id (tokenizer.h:33): *id = -1 when token is not special. */
gh_status gh_tokenizer_special_id(const gh_tokenizer* t, const char* token, size_t len, int32_t* id);
/* Tokenizer::encode (with_specials != 0) / ByteBpe::encode_ordinary (== 0),
 * byte_bpe.cpp:555-591; a v1 tokenizer has one encoding (bpe_tokenizer.cpp:175-270).  *n receives the number of ids of the whole text; at
 * most cap of them are written to ids (call with cap = 0 to size a buffer). */
gh_status gh_tokenizer_encode(const gh_tokenizer* t, const char* text, size_t len, int32_t with_specials,
                              int32_t* ids, size_t cap, size_t* n);
/* Tokenizer::decode (byte_bpe.cpp:649-653): bytes of the ids, concatenated;
 * *len receives their total, at most cap are written (no terminator).
 * GH_ERR_OUT_OF_RANGE for an id outside the vocabulary. */
gh_status gh_tokenizer_decode(const gh_tokenizer* t, const int32_t* ids, size_t n, char* out, size_t cap,
                              size_t* len);
/* pretok::split (pretokenize.h:44, pretokenize.cpp:159-167): the end offset of
 * every piece of text under GPT-2's pattern; *n receives the number of pieces,
 * at most cap offsets are written. */
gh_status gh_pretokenize(const char* text, size_t len, size_t* ends, size_t cap, size_t* n);
/* pretok::classify (pretokenize.h:36): 0 other, 1 letter, 2 number, 3 white space. */
int32_t gh_codepoint_class(uint32_t codepoint);

/* ------------------------------------------------------------------ scoring */

/* What `grad eval` computes per window (training::mean_loss, src/training/trainer.cpp:319-340:
 * GPTModel::forward, gpt_model.cpp:74-142, then Variable::cross_entropy,
 * variable.cpp:589-592), before the mean: nll_host[b * len + t] = -log
 * softmax(logits at position t of sequence b)[targets[b * len + t]], all
 * positions in one pass over the weights.  ids and targets are batch x len.
 * The pass fills the KV cache and advances the position like gh_session_prefill
 * (call gh_session_reset between windows); same errors as gh_session_prefill. */
gh_status gh_session_score(gh_session* s, const int32_t* ids, const int32_t* targets, int32_t len,
                           float* nll_host);

/* No counterpart in grad.cpp: gh_session_pick for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  Every pointer except opt is DEVICE memory owned by the caller:
 * logits is batch x vocab, history is batch x history_stride token ids of which the
 * first n_history of each row are read (the repetition penalty's window; may be NULL
 * when n_history is 0), uniforms is one draw per sequence or NULL for the on-device
 * Philox4x32-10(seed, sequence, pick_index), out_ids receives batch ids.  The kernel
 * is enqueued on hip_stream (a hipStream_t, NULL for the default stream) and the call
 * returns without waiting.  The sampler's working rows live in a 4 MiB array that is
 * part of the library's code object (1,048,576 floats per GPU, held until the
 * process ends): batch x (vocab + 1024, rounded up to 4) floats must fit, otherwise
 * GH_ERR_INVALID_ARGUMENT.  The call makes no allocation of any kind after its first
 * use on a device (which looks the array's address up; gh_device_info does the same
 * look-up ahead of time).  All calls on one GPU share the array: calls that overlap
 * in time on one GPU race; serialise them on one stream. */
gh_status gh_pick_noalloc(const float* logits, int32_t batch, int32_t vocab, const int32_t* history,
                          int32_t history_stride, int32_t n_history, const gh_sampling* opt,
                          const float* uniforms, uint64_t seed, int32_t pick_index, int32_t* out_ids,
                          void* hip_stream);

/* ------------------------------------------------------------ measurement */

/* GPU time of the last gh_session_generate call, from HIP events recorded on
 * the session's stream: the prompt steps and the decode steps separately. */
typedef struct gh_timing {
    float prompt_ms;
    float decode_ms;
    int32_t prompt_steps;
    int32_t decode_steps;
    int32_t launches_per_step; /* kernel launches (or graph nodes) in one step */
    /* Persistent engine, since the session was created: picks that one workgroup made from
     * the whole row of logits.  The others (greedy, or 0 < top_k <= 64, after a step of the
     * same launch) were made by every workgroup at once from a few candidates per workgroup. */
    int32_t row_picks;
} gh_timing;
gh_status gh_session_last_timing(const gh_session* s, gh_timing* out);

/* Device facts for reports: name, compute units, and whether it is gfx950. */
gh_status gh_device_info(char* name, size_t name_len, int32_t* compute_units, int32_t* is_gfx950);

/* Measurement aid with no counterpart in grad.cpp: the rate (GB/s) at which a
 * plain streaming kernel reads `bytes` of device memory, best of `repeats`
 * passes.  It says how much of the published HBM peak a bandwidth-bound kernel
 * can reach on this device, which is what roofline fractions are read against. */
gh_status gh_device_read_bandwidth(size_t bytes, int32_t repeats, double* gb_per_s);

/* Measurement aid with no counterpart in grad.cpp: the same streaming kernel launched
 * `passes` times back to back over one buffer of `bytes` (after two warm-up
 * launches), timed as one span, launch gaps included.  A buffer that fits the memory-side cache is then
 * served from it; the rate over a range of sizes shows where that stops. */
gh_status gh_device_reread_bandwidth(size_t bytes, int32_t passes, double* gb_per_s);

/* Measurement aid with no counterpart in grad.cpp: what handing a word from one
 * workgroup to another costs.  Workgroup 0 and workgroup `peer` (1..15; workgroups go
 * round-robin over the XCDs, so 8 shares workgroup 0's XCD and 1 does not) bounce a
 * counter 1000 times; *us_per_round_trip is the time per round trip (two hand-offs).
 * load_policy: 0 ordinary, 1 non-temporal (served by the L2, never kept in the vector
 * cache), 2 device scope.  device_scope_store: write-through store, or an ordinary
 * one.  busy: 240 more workgroups stream from HBM meanwhile.  *xcd_a / *xcd_b (may be
 * NULL) receive the XCDs the two workgroups ran on. */
gh_status gh_device_handoff_latency(int32_t load_policy, int32_t device_scope_store, int32_t peer, int32_t busy,
                                    double* us_per_round_trip, int32_t* xcd_a, int32_t* xcd_b);

/* Measurement aid with no counterpart in grad.cpp: does anything else issue on a SIMD while
 * an fp32 matrix product (v_mfma_f32_32x32x2_f32, 64 cycles) runs there?  256 workgroups of
 * eight wavefronts, two per SIMD.  mode 1: wavefronts 0-3 run a dependent chain of products;
 * mode 2: wavefronts 4-7 run slots of valu_per_slot (8, 16 or 24) independent multiply-adds;
 * mode 3: both at once, on the same SIMDs; mode 4: wavefronts 0-3 alone, one slot of
 * multiply-adds after each of their own products; mode 6: 4 and 2 together.
 * *clk_per_product: shader-clock cycles per product of wavefronts 0-3 (per product + slot in
 * modes 4 and 6); *clk_per_valu_slot: cycles per slot of wavefronts 4-7; *shader_mhz: the
 * shader clock the busy wavefronts saw.  If ordinary arithmetic could run beside a product,
 * mode 3 would cost wavefronts 4-7 what mode 2 does; on gfx950 it costs them mode 1 + mode 2. */
gh_status gh_device_mfma_issue(int32_t mode, int32_t valu_per_slot, double* clk_per_product, double* clk_per_valu_slot,
                               double* shader_mhz);

#ifdef __cplusplus
}
#endif
#endif
