/*
 * gradref — CPU restatement of grad.cpp's KV-cached token loop.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It exists to check the HIP
 * path and to be timed as the CPU baseline.  Only the test suite, the smoke
 * check and the benchmark's cpu_baseline leg may load it; the shipped library
 * never links, loads or calls anything in this directory.
 *
 * Every function names the reference file:line it restates (paths relative to
 * the grad.cpp source tree).
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   gr_model_load / gr_model_save  : the byte offsets, sizes and exact error
 *       strings asserted by tests/unit/test_core_regressions.cpp:426-541.
 *   gr_session_step                : the reference's own invariant
 *       "step(i) == row i of the full-sequence forward"
 *       (tests/integration/sanity_tests.cpp:293-333) against an independent
 *       float64 restatement of GPTModel::forward, plus closed forms
 *       (ctx = 1, zero input => b_o, RoPE at position 0, norm moments,
 *       relative-position invariance of rotated dot products).
 *   gr_logits_with_penalty, gr_argmax_first, gr_sample_from_logits,
 *   gr_generate_greedy, gr_generate_sample : the reference has no test and no
 *       stored vector for them; they are pinned by hand-derived cases and by
 *       brute force on tiny vocabularies.  The real reference could not be
 *       compiled here (it needs <cblas.h>, which this image lacks), so the
 *       exact token streams of the reference binary are "parity unpinned".
 */
#ifndef GRADREF_H
#define GRADREF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct gr_model gr_model;
typedef struct gr_session gr_session;

enum { GR_ARCH_GPT2 = 0, GR_ARCH_MODERN = 1 };

/* Error handling: functions return 0 on success.  Non-zero codes say which
 * C++ exception type the reference throws at that point. */
enum {
    GR_OK = 0,
    GR_RUNTIME_ERROR = 1,    /* std::runtime_error */
    GR_OUT_OF_RANGE = 2,     /* std::out_of_range */
    GR_INVALID_ARGUMENT = 3  /* std::invalid_argument */
};
const char* gr_last_error(void);

/* ---- model container + checkpoint format (gpt_model.cpp:187-525) ---- */
gr_model* gr_model_new(int arch, int vocab, int d_model, int layers, int heads, int max_len,
                       float dropout);
void gr_model_free(gr_model* m);
int gr_model_load(const char* path, gr_model** out);
int gr_model_save(const gr_model* m, const char* path);
/* Tensors in checkpoint order (gpt_model.cpp:318-355). */
int gr_model_num_tensors(const gr_model* m);
float* gr_model_tensor(gr_model* m, int index, int* rows, int* cols);
void gr_model_dims(const gr_model* m, int* arch, int* vocab, int* d_model, int* layers, int* heads,
                   int* max_len, int* d_ff, float* dropout);
void gr_model_set_fingerprint(gr_model* m, uint32_t kind, uint64_t hash);
int gr_model_get_fingerprint(const gr_model* m, uint32_t* kind, uint64_t* hash); /* 1 if set */

/* ---- InferenceSession (inference.cpp:121-258) ---- */
gr_session* gr_session_new(const gr_model* m);
void gr_session_free(gr_session* s);
int gr_session_step(gr_session* s, int token_id, const float** logits);
int gr_session_position(const gr_session* s);
int gr_session_capacity(const gr_session* s);
int gr_session_vocab(const gr_session* s);
/* Read access to the caches for cache-content checks: row `pos` of layer `l`. */
const float* gr_session_k_row(const gr_session* s, int layer, int pos);
const float* gr_session_v_row(const gr_session* s, int layer, int pos);

/* ---- TextGen (text_gen.cpp:14-209) ---- */
void gr_logits_with_penalty(const float* logits, int vocab, const int* tokens, size_t n_tokens,
                            float penalty, float* out);
int gr_argmax_first(const float* data, int vocab);
/* sample_from_logits with the uniform draw supplied by the caller.  When
 * probs_out is non-NULL it receives the final (post top-p) probabilities. */
int gr_sample_from_logits(const float* logits, int vocab, float temperature, int top_k,
                          float top_p, float u, float* probs_out);
/* Generate loops.  out_tokens receives prompt + generated ids (capacity
 * n_prompt + max_tokens); *out_n their count.  If step_logits is non-NULL it
 * receives the raw logits of every step() call in order (vocab floats each,
 * n_prompt + max_tokens rows at most); *n_steps their count. */
int gr_generate_greedy(const gr_model* m, const int* prompt, size_t n_prompt, int max_tokens,
                       float penalty, int* out_tokens, size_t* out_n, float* step_logits,
                       size_t* n_steps);
int gr_generate_sample(const gr_model* m, const int* prompt, size_t n_prompt, float temperature,
                       int max_tokens, float penalty, int top_k, float top_p,
                       const float* uniforms, int* out_tokens, size_t* out_n, float* step_logits,
                       size_t* n_steps);

/* ---- BLAS provider for the projections (blas_wrapper.h:67-83) ---- */
/* Tries libopenblas, the OpenBLAS inside numpy/scipy wheels, then MKL; falls
 * back to plain loops.  `hint` may name a library file to try first.  Returns
 * a description string ("loops" when nothing was found). */
const char* gr_blas_init(const char* hint);
void gr_blas_set_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
