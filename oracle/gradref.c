/*
 * gradref.c — CPU restatement of grad.cpp's KV-cached token loop.
 * Test infrastructure only; see gradref.h for the rules and the pinning table.
 *
 * Single-threaded, fp32, same operation order as the reference: one M=1 sgemm
 * per projection, one sdot / saxpy of length head_size per cached position,
 * scalar expf / tanhf.
 */
#define _GNU_SOURCE
#include "gradref.h"

#include <dlfcn.h>
#include <glob.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ errors */

static __thread char g_err[1024];

const char* gr_last_error(void) { return g_err; }

static int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

/* ------------------------------------------------------------ BLAS provider */
/* blas_wrapper.h:67-83 routes every projection through cblas_sgemm, and
 * :130-137 routes the attention dot/axpy through cblas_sdot / cblas_saxpy.
 * The provider is looked up at run time; plain loops are the fallback. */

typedef void (*sgemm_fn)(int order, int ta, int tb, int m, int n, int k, float alpha,
                         const float* a, int lda, const float* b, int ldb, float beta, float* c,
                         int ldc);
typedef float (*sdot_fn)(int n, const float* x, int incx, const float* y, int incy);
typedef void (*saxpy_fn)(int n, float alpha, const float* x, int incx, float* y, int incy);
typedef void (*setthreads_fn)(int n);

static sgemm_fn p_sgemm;
static sdot_fn p_sdot;
static saxpy_fn p_saxpy;
static setthreads_fn p_setthreads;
static char g_blas_desc[512] = "loops";

static int try_provider(const char* file, const char* prefix) {
    void* h = dlopen(file, RTLD_NOW | RTLD_LOCAL);
    if (!h) return 0;
    char name[128];
    snprintf(name, sizeof name, "%scblas_sgemm", prefix);
    sgemm_fn g = (sgemm_fn)dlsym(h, name);
    snprintf(name, sizeof name, "%scblas_sdot", prefix);
    sdot_fn d = (sdot_fn)dlsym(h, name);
    snprintf(name, sizeof name, "%scblas_saxpy", prefix);
    saxpy_fn a = (saxpy_fn)dlsym(h, name);
    if (!g || !d || !a) {
        dlclose(h);
        return 0;
    }
    p_sgemm = g;
    p_sdot = d;
    p_saxpy = a;
    snprintf(name, sizeof name, "%sopenblas_set_num_threads", prefix);
    p_setthreads = (setthreads_fn)dlsym(h, name);
    if (!p_setthreads) p_setthreads = (setthreads_fn)dlsym(h, "MKL_Set_Num_Threads");
    const char* cfg = "";
    snprintf(name, sizeof name, "%sopenblas_get_config", prefix);
    const char* (*getcfg)(void) = (const char* (*)(void))dlsym(h, name);
    if (getcfg) cfg = getcfg();
    snprintf(g_blas_desc, sizeof g_blas_desc, "%s [%s]", file, cfg);
    return 1;
}

static int try_glob(const char* pattern, const char* prefix) {
    glob_t gl;
    int ok = 0;
    if (glob(pattern, 0, NULL, &gl) == 0) {
        for (size_t i = 0; i < gl.gl_pathc && !ok; i++) ok = try_provider(gl.gl_pathv[i], prefix);
    }
    globfree(&gl);
    return ok;
}

const char* gr_blas_init(const char* hint) {
    if (p_sgemm) return g_blas_desc;
    if (hint && *hint && (try_provider(hint, "") || try_provider(hint, "scipy_"))) return g_blas_desc;
    if (try_provider("libopenblas.so.0", "")) return g_blas_desc;
    if (try_provider("libopenblas.so", "")) return g_blas_desc;
    /* LP64 OpenBLAS shipped inside the scipy wheel (symbols carry a scipy_ prefix). */
    if (try_glob("/usr/local/lib/python3*/dist-packages/scipy.libs/libscipy_openblas-*.so", "scipy_"))
        return g_blas_desc;
    if (try_glob("/usr/lib/python3*/site-packages/scipy.libs/libscipy_openblas-*.so", "scipy_"))
        return g_blas_desc;
    if (try_provider("libmkl_rt.so", "")) return g_blas_desc;
    if (try_provider("/opt/conda/lib/libmkl_rt.so", "")) return g_blas_desc;
    return g_blas_desc;
}

void gr_blas_set_threads(int n) {
    if (p_setthreads) p_setthreads(n);
}

/* C(1,n) = alpha * x(1,k) @ op(B) + beta * C — the only sgemm shape on the path. */
static void sgemm_m1(const float* x, const float* B, float* y, size_t n, size_t k, int transB,
                     float beta) {
    if (p_sgemm) {
        p_sgemm(101, 111, transB ? 112 : 111, 1, (int)n, (int)k, 1.0f, x, (int)k, B,
                transB ? (int)k : (int)n, beta, y, (int)n);
        return;
    }
    if (beta == 0.0f) memset(y, 0, n * sizeof(float));
    if (!transB) {
        for (size_t i = 0; i < k; i++) {
            const float xi = x[i];
            const float* row = B + i * n;
            for (size_t j = 0; j < n; j++) y[j] += xi * row[j];
        }
    } else {
        for (size_t j = 0; j < n; j++) {
            const float* row = B + j * k;
            float acc = 0.0f;
            for (size_t i = 0; i < k; i++) acc += x[i] * row[i];
            y[j] += acc;
        }
    }
}

static float vec_dot(const float* x, const float* y, size_t n) {
    if (p_sdot) return p_sdot((int)n, x, 1, y, 1);
    float s = 0.0f;
    for (size_t i = 0; i < n; i++) s += x[i] * y[i];
    return s;
}

static void vec_axpy(float alpha, const float* x, float* y, size_t n) {
    if (p_saxpy) {
        p_saxpy((int)n, alpha, x, 1, y, 1);
        return;
    }
    for (size_t i = 0; i < n; i++) y[i] += alpha * x[i];
}

/* blas_wrapper.h:139-149 (Linux branch): index-order scalar sum. */
static float vec_sum(const float* x, size_t n) {
    float s = 0.0f;
    for (size_t i = 0; i < n; i++) s += x[i];
    return s;
}

/* ---------------------------------------------------------- model container */

typedef struct {
    int rows, cols;
    float* data;
    char name[40];
} tensor_t;

struct gr_model {
    int arch, vocab, d_model, layers, heads, max_len, d_ff;
    float dropout;
    int n_tensors;
    tensor_t* t;
    int has_fp;
    uint32_t fp_kind;
    uint64_t fp_hash;
};

/* feedforward.h:24-28 */
static int ffn_width(int d_model, int modern) {
    if (!modern) return 4 * d_model;
    return ((8 * d_model / 3) + 63) / 64 * 64;
}

/* Tensor slots per layer, in file order (gpt_model.cpp:323-352). */
enum { L_WQ, L_WK, L_WV, L_WO, L_BQ, L_BK, L_BV, L_BO, L_FFN0 };

static int per_layer(int modern) { return 8 + (modern ? 3 : 4) + 4; }
static int layer_base(const gr_model* m, int l) {
    return (m->arch == GR_ARCH_MODERN ? 1 : 2) + l * per_layer(m->arch == GR_ARCH_MODERN);
}

static void set_tensor(tensor_t* t, int rows, int cols, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t->name, sizeof t->name, fmt, ap);
    va_end(ap);
    t->rows = rows;
    t->cols = cols;
    t->data = (float*)calloc((size_t)rows * (size_t)cols, sizeof(float));
}

gr_model* gr_model_new(int arch, int vocab, int d, int layers, int heads, int max_len,
                       float dropout) {
    const int modern = arch == GR_ARCH_MODERN;
    gr_model* m = (gr_model*)calloc(1, sizeof *m);
    m->arch = arch;
    m->vocab = vocab;
    m->d_model = d;
    m->layers = layers;
    m->heads = heads;
    m->max_len = max_len;
    m->dropout = dropout;
    m->d_ff = ffn_width(d, modern);
    const int F = m->d_ff;
    m->n_tensors = (modern ? 1 : 2) + layers * per_layer(modern) + 2;
    m->t = (tensor_t*)calloc((size_t)m->n_tensors, sizeof(tensor_t));
    int k = 0;
    set_tensor(&m->t[k++], vocab, d, "token embedding");
    if (!modern) set_tensor(&m->t[k++], max_len, d, "position embedding");
    for (int l = 0; l < layers; l++) {
        static const char* const attn[] = {"W_q", "W_k", "W_v", "W_o", "b_q", "b_k", "b_v", "b_o"};
        for (int p = 0; p < 8; p++)
            set_tensor(&m->t[k++], p < 4 ? d : 1, d, "layer %d %s", l, attn[p]);
        if (modern) {
            set_tensor(&m->t[k++], d, F, "layer %d FFN gate", l);
            set_tensor(&m->t[k++], d, F, "layer %d FFN up", l);
            set_tensor(&m->t[k++], F, d, "layer %d FFN down", l);
        } else {
            set_tensor(&m->t[k++], d, F, "layer %d FFN W1", l);
            set_tensor(&m->t[k++], 1, F, "layer %d FFN b1", l);
            set_tensor(&m->t[k++], F, d, "layer %d FFN W2", l);
            set_tensor(&m->t[k++], 1, d, "layer %d FFN b2", l);
        }
        set_tensor(&m->t[k++], 1, d, "layer %d norm1 gamma", l);
        set_tensor(&m->t[k++], 1, d, "layer %d norm1 beta", l);
        set_tensor(&m->t[k++], 1, d, "layer %d norm2 gamma", l);
        set_tensor(&m->t[k++], 1, d, "layer %d norm2 beta", l);
    }
    set_tensor(&m->t[k++], 1, d, "final norm gamma");
    set_tensor(&m->t[k++], 1, d, "final norm beta");
    return m;
}

void gr_model_free(gr_model* m) {
    if (!m) return;
    for (int i = 0; i < m->n_tensors; i++) free(m->t[i].data);
    free(m->t);
    free(m);
}

int gr_model_num_tensors(const gr_model* m) { return m->n_tensors; }

float* gr_model_tensor(gr_model* m, int index, int* rows, int* cols) {
    if (index < 0 || index >= m->n_tensors) return NULL;
    if (rows) *rows = m->t[index].rows;
    if (cols) *cols = m->t[index].cols;
    return m->t[index].data;
}

void gr_model_dims(const gr_model* m, int* arch, int* vocab, int* d_model, int* layers, int* heads,
                   int* max_len, int* d_ff, float* dropout) {
    if (arch) *arch = m->arch;
    if (vocab) *vocab = m->vocab;
    if (d_model) *d_model = m->d_model;
    if (layers) *layers = m->layers;
    if (heads) *heads = m->heads;
    if (max_len) *max_len = m->max_len;
    if (d_ff) *d_ff = m->d_ff;
    if (dropout) *dropout = m->dropout;
}

void gr_model_set_fingerprint(gr_model* m, uint32_t kind, uint64_t hash) {
    m->has_fp = 1;
    m->fp_kind = kind;
    m->fp_hash = hash;
}

int gr_model_get_fingerprint(const gr_model* m, uint32_t* kind, uint64_t* hash) {
    if (!m->has_fp) return 0;
    if (kind) *kind = m->fp_kind;
    if (hash) *hash = m->fp_hash;
    return 1;
}

/* ------------------------------------------------------- checkpoint format */
/* gpt_model.cpp:187-193: "GPTM", trailer tag "TKFP" with a 12-byte payload,
 * trailer payloads capped at 1 MiB. */
#define CK_MAGIC 0x4750544Du
#define CK_TRAILER_PAYLOAD 12u
#define CK_MAX_TRAILER (1u << 20)

/* gpt_model.cpp:292-381 */
int gr_model_save(const gr_model* m, const char* path) {
    FILE* f = fopen(path, "wb");
    if (!f) return fail(GR_RUNTIME_ERROR, "Error: Could not open file for writing: %s", path);
    const uint32_t magic = CK_MAGIC, version = 2, arch = (uint32_t)m->arch;
    int ok = 1;
    ok &= fwrite(&magic, 4, 1, f) == 1;
    ok &= fwrite(&version, 4, 1, f) == 1;
    ok &= fwrite(&arch, 4, 1, f) == 1;
    const int32_t hdr[5] = {m->vocab, m->d_model, m->layers, m->heads, m->max_len};
    ok &= fwrite(hdr, 4, 5, f) == 5;
    ok &= fwrite(&m->dropout, 4, 1, f) == 1;
    for (int i = 0; i < m->n_tensors && ok; i++) {
        const tensor_t* t = &m->t[i];
        const int32_t rc[2] = {t->rows, t->cols};
        const size_t n = (size_t)t->rows * (size_t)t->cols;
        ok &= fwrite(rc, 4, 2, f) == 2;
        ok &= fwrite(t->data, 4, n, f) == n;
    }
    if (ok && m->has_fp) {
        unsigned char tr[20];
        memcpy(tr, "TKFP", 4);
        for (int i = 0; i < 4; i++) tr[4 + i] = (unsigned char)((CK_TRAILER_PAYLOAD >> (8 * i)) & 0xFF);
        for (int i = 0; i < 4; i++) tr[8 + i] = (unsigned char)((m->fp_kind >> (8 * i)) & 0xFF);
        for (int i = 0; i < 8; i++) tr[12 + i] = (unsigned char)((m->fp_hash >> (8 * i)) & 0xFF);
        ok &= fwrite(tr, 1, 20, f) == 20;
    }
    if (fclose(f) != 0) ok = 0;
    if (!ok) return fail(GR_RUNTIME_ERROR, "Error: writing checkpoint failed: %s", path);
    return GR_OK;
}

typedef struct {
    FILE* f;
    char msg[512];
} reader_t;

/* CheckpointReader::scalar, gpt_model.cpp:235-241 */
static int rd_scalar(reader_t* r, void* out, const char* what) {
    if (fread(out, 4, 1, r->f) != 1) {
        snprintf(r->msg, sizeof r->msg, "file ends while reading %s", what);
        return 0;
    }
    return 1;
}

/* check_range, gpt_model.cpp:283-288 */
static int rd_range(reader_t* r, const char* name, int v, int lo, int hi) {
    if (v < lo || v > hi) {
        snprintf(r->msg, sizeof r->msg, "header field %s = %d is outside [%d, %d]", name, v, lo, hi);
        return 0;
    }
    return 1;
}

/* CheckpointReader::tensor_like, gpt_model.cpp:246-260 */
static int rd_tensor(reader_t* r, tensor_t* t) {
    int32_t rows, cols;
    if (!rd_scalar(r, &rows, t->name) || !rd_scalar(r, &cols, t->name)) return 0;
    if (rows <= 0 || cols <= 0 || rows != t->rows || cols != t->cols) {
        snprintf(r->msg, sizeof r->msg, "%s is %dx%d, model expects %dx%d", t->name, rows, cols,
                 t->rows, t->cols);
        return 0;
    }
    const size_t n = (size_t)rows * (size_t)cols;
    if (fread(t->data, 4, n, r->f) != n) {
        snprintf(r->msg, sizeof r->msg, "file ends inside %s", t->name);
        return 0;
    }
    return 1;
}

static uint64_t get_le(const unsigned char* p, int bytes) {
    uint64_t v = 0;
    for (int i = 0; i < bytes; i++) v |= (uint64_t)p[i] << (8 * i);
    return v;
}

/* GPTModel::load, gpt_model.cpp:383-525 */
int gr_model_load(const char* path, gr_model** out) {
    *out = NULL;
    FILE* f = fopen(path, "rb");
    if (!f) return fail(GR_RUNTIME_ERROR, "Could not open checkpoint for reading: %s", path);
    reader_t r = {f, {0}};
    gr_model* m = NULL;
    int code = GR_RUNTIME_ERROR;

    uint32_t magic, version, arch_tag = 0;
    if (!rd_scalar(&r, &magic, "magic number")) goto bad;
    if (magic != CK_MAGIC) {
        snprintf(r.msg, sizeof r.msg, "not a grad.cpp checkpoint (wrong magic number)");
        goto bad;
    }
    if (!rd_scalar(&r, &version, "format version")) goto bad;
    if (version != 1 && version != 2) {
        snprintf(r.msg, sizeof r.msg, "unsupported format version %u", version);
        goto bad;
    }
    if (version == 2) {
        if (!rd_scalar(&r, &arch_tag, "architecture tag")) goto bad;
        if (arch_tag != 0 && arch_tag != 1) {
            snprintf(r.msg, sizeof r.msg, "unknown architecture tag %u", arch_tag);
            goto bad;
        }
    }
    int32_t vocab, d, layers, heads, max_len;
    float dropout;
    if (!rd_scalar(&r, &vocab, "vocab_size") || !rd_scalar(&r, &d, "d_model")
        || !rd_scalar(&r, &layers, "num_layers") || !rd_scalar(&r, &heads, "num_heads")
        || !rd_scalar(&r, &max_len, "max_len") || !rd_scalar(&r, &dropout, "dropout_rate"))
        goto bad;
    if (!rd_range(&r, "vocab_size", vocab, 1, 1 << 24) || !rd_range(&r, "d_model", d, 1, 1 << 16)
        || !rd_range(&r, "num_layers", layers, 1, 1 << 12)
        || !rd_range(&r, "num_heads", heads, 1, d) || !rd_range(&r, "max_len", max_len, 1, 1 << 20))
        goto bad;
    if (d % heads != 0) {
        snprintf(r.msg, sizeof r.msg, "d_model %d is not divisible by num_heads %d", d, heads);
        goto bad;
    }
    if (!(dropout >= 0.0f && dropout < 1.0f)) {
        snprintf(r.msg, sizeof r.msg, "dropout_rate %f is outside [0, 1)", (double)dropout);
        goto bad;
    }
    /* The model is constructed next; MultiHeadAttention's constructor rejects
     * an odd head size under RoPE (multihead_attention.cpp:333-335). */
    if (arch_tag == 1 && (d / heads) % 2 != 0) {
        snprintf(r.msg, sizeof r.msg, "RoPE requires an even head size");
        goto bad;
    }
    m = gr_model_new((int)arch_tag, vocab, d, layers, heads, max_len, dropout);
    for (int i = 0; i < m->n_tensors; i++)
        if (!rd_tensor(&r, &m->t[i])) goto bad;

    /* Trailer sections, gpt_model.cpp:489-515. */
    for (;;) {
        int c = fgetc(f);
        if (c == EOF) break;
        ungetc(c, f);
        unsigned char hdr[8];
        if (fread(hdr, 1, 8, f) != 8) {
            snprintf(r.msg, sizeof r.msg, "file ends while reading trailer section header");
            goto bad;
        }
        const uint32_t len = (uint32_t)get_le(hdr + 4, 4);
        if (len > CK_MAX_TRAILER) {
            snprintf(r.msg, sizeof r.msg, "trailer section has an implausible length (%u bytes)", len);
            goto bad;
        }
        if (memcmp(hdr, "TKFP", 4) != 0) {
            unsigned char sink[4096];
            uint32_t left = len;
            while (left) {
                size_t want = left < sizeof sink ? left : sizeof sink;
                if (fread(sink, 1, want, f) != want) {
                    snprintf(r.msg, sizeof r.msg, "file ends inside trailer section");
                    goto bad;
                }
                left -= (uint32_t)want;
            }
            continue;
        }
        if (len != CK_TRAILER_PAYLOAD) {
            snprintf(r.msg, sizeof r.msg, "tokenizer trailer has length %u, expected %u", len,
                     CK_TRAILER_PAYLOAD);
            goto bad;
        }
        unsigned char pl[12];
        if (fread(pl, 1, 12, f) != 12) {
            snprintf(r.msg, sizeof r.msg, "file ends while reading tokenizer trailer");
            goto bad;
        }
        const uint32_t kind = (uint32_t)get_le(pl, 4);
        if (kind != 1 && kind != 2) {
            snprintf(r.msg, sizeof r.msg, "unknown tokenizer kind %u", kind);
            goto bad;
        }
        gr_model_set_fingerprint(m, kind, get_le(pl + 4, 8));
    }
    fclose(f);
    *out = m;
    return GR_OK;

bad:
    fclose(f);
    gr_model_free(m);
    return fail(code, "Failed to load model from %s: %s", path, r.msg);
}

/* -------------------------------------------------------- InferenceSession */

struct gr_session {
    const gr_model* m;
    size_t d, L, H, hs, F, C, V, pos;
    float **k_cache, **v_cache;
    float *x, *h, *q, *attn, *scores, *ffn_hidden, *ffn_gate, *rope_cos, *rope_sin, *logits;
    float *tmp; /* the heap temporaries of gelu_row / silu_row (inference.cpp:72, :83) */
};

static float* zalloc(size_t n) { return (float*)calloc(n ? n : 1, sizeof(float)); }

/* inference.cpp:121-148 */
gr_session* gr_session_new(const gr_model* m) {
    gr_session* s = (gr_session*)calloc(1, sizeof *s);
    s->m = m;
    s->d = (size_t)m->d_model;
    s->L = (size_t)m->layers;
    s->H = (size_t)m->heads;
    s->hs = s->d / s->H;
    s->F = (size_t)m->d_ff;
    s->C = (size_t)m->max_len;
    s->V = (size_t)m->vocab;
    s->k_cache = (float**)calloc(s->L, sizeof(float*));
    s->v_cache = (float**)calloc(s->L, sizeof(float*));
    for (size_t l = 0; l < s->L; l++) {
        s->k_cache[l] = zalloc(s->C * s->d);
        s->v_cache[l] = zalloc(s->C * s->d);
    }
    s->x = zalloc(s->d);
    s->h = zalloc(s->d);
    s->q = zalloc(s->d);
    s->attn = zalloc(s->d);
    s->scores = zalloc(s->C);
    s->ffn_hidden = zalloc(s->F);
    s->ffn_gate = zalloc(s->F);
    s->tmp = zalloc(s->F);
    s->rope_cos = zalloc(s->hs / 2);
    s->rope_sin = zalloc(s->hs / 2);
    s->logits = zalloc(s->V);
    return s;
}

void gr_session_free(gr_session* s) {
    if (!s) return;
    for (size_t l = 0; l < s->L; l++) {
        free(s->k_cache[l]);
        free(s->v_cache[l]);
    }
    free(s->k_cache);
    free(s->v_cache);
    free(s->x);
    free(s->h);
    free(s->q);
    free(s->attn);
    free(s->scores);
    free(s->ffn_hidden);
    free(s->ffn_gate);
    free(s->tmp);
    free(s->rope_cos);
    free(s->rope_sin);
    free(s->logits);
    free(s);
}

int gr_session_position(const gr_session* s) { return (int)s->pos; }
int gr_session_capacity(const gr_session* s) { return (int)s->C; }
int gr_session_vocab(const gr_session* s) { return (int)s->V; }
const float* gr_session_k_row(const gr_session* s, int l, int pos) {
    return s->k_cache[l] + (size_t)pos * s->d;
}
const float* gr_session_v_row(const gr_session* s, int l, int pos) {
    return s->v_cache[l] + (size_t)pos * s->d;
}

/* inference.cpp:14-19 — y = b + x @ W, W is (in,out) row-major. */
static void matvec(const float* x, const tensor_t* W, const tensor_t* b, float* y) {
    memcpy(y, b->data, (size_t)W->cols * sizeof(float));
    sgemm_m1(x, W->data, y, (size_t)W->cols, (size_t)W->rows, 0, 1.0f);
}

/* inference.cpp:22-28 — y += b + x @ W. */
static void matvec_add(const float* x, const tensor_t* W, const tensor_t* b, float* y) {
    for (int j = 0; j < W->cols; j++) y[j] += b->data[j];
    sgemm_m1(x, W->data, y, (size_t)W->cols, (size_t)W->rows, 0, 1.0f);
}

/* inference.cpp:94-96 */
static void matvec_nobias(const float* x, const tensor_t* W, float* y) {
    sgemm_m1(x, W->data, y, (size_t)W->cols, (size_t)W->rows, 0, 0.0f);
}

/* inference.cpp:30-58; eps = 1e-5 (layer_norm.h:18) */
static void layer_norm_row(const float* x, const float* g, const float* beta, int rms, size_t d,
                           float* out) {
    const float eps = 1e-5f;
    if (rms) {
        float ms = 0.0f;
        for (size_t j = 0; j < d; j++) ms += x[j] * x[j];
        const float r = 1.0f / sqrtf(ms / (float)d + eps);
        for (size_t j = 0; j < d; j++) out[j] = g[j] * x[j] * r;
        return;
    }
    const float mean = vec_sum(x, d) / (float)d;
    float variance = 0.0f;
    for (size_t j = 0; j < d; j++) {
        const float diff = x[j] - mean;
        variance += diff * diff;
    }
    variance /= (float)d;
    const float inv_std = 1.0f / sqrtf(variance + eps);
    for (size_t j = 0; j < d; j++) out[j] = g[j] * (x[j] - mean) * inv_std + beta[j];
}

/* inference.cpp:60-67 */
static void softmax_row(float* s, size_t n) {
    float max_val = s[0];
    for (size_t t = 1; t < n; t++) max_val = s[t] > max_val ? s[t] : max_val;
    for (size_t t = 0; t < n; t++) s[t] -= max_val;
    for (size_t t = 0; t < n; t++) s[t] = expf(s[t]);
    const float inv_sum = 1.0f / vec_sum(s, n);
    for (size_t t = 0; t < n; t++) s[t] *= inv_sum;
}

/* inference.cpp:69-80 */
static void gelu_row(float* x, float* t, size_t n) {
    const float k = 0.79788456f;
    const float a = 0.044715f;
    for (size_t i = 0; i < n; i++) t[i] = k * (x[i] + a * x[i] * x[i] * x[i]);
    for (size_t i = 0; i < n; i++) t[i] = tanhf(t[i]);
    for (size_t i = 0; i < n; i++) x[i] = 0.5f * x[i] * (1.0f + t[i]);
}

/* inference.cpp:82-91 */
static void silu_row(float* x, float* e, size_t n) {
    for (size_t i = 0; i < n; i++) e[i] = -x[i];
    for (size_t i = 0; i < n; i++) e[i] = expf(e[i]);
    for (size_t i = 0; i < n; i++) x[i] = x[i] / (1.0f + e[i]);
}

/* inference.cpp:101-115 — pairs (2j, 2j+1) within each head. */
static void rope_row(float* row, size_t H, size_t hs, const float* cos_p, const float* sin_p) {
    const size_t half = hs / 2;
    for (size_t h = 0; h < H; h++) {
        float* head = row + h * hs;
        for (size_t j = 0; j < half; j++) {
            const float c = cos_p[j], s = sin_p[j];
            const float a = head[2 * j], b = head[2 * j + 1];
            head[2 * j] = a * c - b * s;
            head[2 * j + 1] = a * s + b * c;
        }
    }
}

/* inference.cpp:150-258 */
int gr_session_step(gr_session* s, int token_id, const float** logits_out) {
    const gr_model* m = s->m;
    if (s->pos >= s->C) return fail(GR_RUNTIME_ERROR, "InferenceSession: context exceeds max_len");
    if (token_id < 0 || (size_t)token_id >= s->V)
        return fail(GR_OUT_OF_RANGE, "InferenceSession: token id out of vocab range");

    const int modern = m->arch == GR_ARCH_MODERN;
    const size_t d = s->d;
    const tensor_t* E = &m->t[0];
    const float emb_scale = 1.0f; /* token_embedding.h:12 */
    const float* e_row = E->data + (size_t)token_id * d;

    if (modern) {
        for (size_t j = 0; j < d; j++) s->x[j] = e_row[j] * emb_scale;
        const size_t half = s->hs / 2;
        for (size_t j = 0; j < half; j++) {
            const float theta = powf(10000.0f, -2.0f * (float)j / (float)s->hs);
            s->rope_cos[j] = cosf((float)s->pos * theta);
            s->rope_sin[j] = sinf((float)s->pos * theta);
        }
    } else {
        const float* p_row = m->t[1].data + s->pos * d;
        for (size_t j = 0; j < d; j++) s->x[j] = e_row[j] * emb_scale + p_row[j];
    }

    const float inv_sqrt_hs = 1.0f / sqrtf((float)s->hs);
    const size_t ctx = s->pos + 1;

    for (size_t l = 0; l < s->L; l++) {
        const tensor_t* T = &m->t[layer_base(m, (int)l)];
        const tensor_t* N = T + L_FFN0 + (modern ? 3 : 4); /* norm1 gamma, beta, norm2 gamma, beta */

        layer_norm_row(s->x, N[0].data, N[1].data, modern, d, s->h);

        float* k_row = s->k_cache[l] + s->pos * d;
        float* v_row = s->v_cache[l] + s->pos * d;
        matvec(s->h, &T[L_WQ], &T[L_BQ], s->q);
        matvec(s->h, &T[L_WK], &T[L_BK], k_row);
        matvec(s->h, &T[L_WV], &T[L_BV], v_row);

        if (modern) {
            rope_row(s->q, s->H, s->hs, s->rope_cos, s->rope_sin);
            rope_row(k_row, s->H, s->hs, s->rope_cos, s->rope_sin);
        }

        const float* K = s->k_cache[l];
        const float* V = s->v_cache[l];
        for (size_t hd = 0; hd < s->H; hd++) {
            const size_t off = hd * s->hs;
            const float* qh = s->q + off;
            for (size_t t = 0; t < ctx; t++)
                s->scores[t] = vec_dot(qh, K + t * d + off, s->hs) * inv_sqrt_hs;
            softmax_row(s->scores, ctx);
            float* out_h = s->attn + off;
            memset(out_h, 0, s->hs * sizeof(float));
            for (size_t t = 0; t < ctx; t++) vec_axpy(s->scores[t], V + t * d + off, out_h, s->hs);
        }

        matvec_add(s->attn, &T[L_WO], &T[L_BO], s->x);

        layer_norm_row(s->x, N[2].data, N[3].data, modern, d, s->h);
        const tensor_t* Fp = T + L_FFN0;
        if (modern) {
            /* gate, up, down (inference.cpp:232-241) */
            matvec_nobias(s->h, &Fp[0], s->ffn_gate);
            silu_row(s->ffn_gate, s->tmp, s->F);
            matvec_nobias(s->h, &Fp[1], s->ffn_hidden);
            for (size_t j = 0; j < s->F; j++) s->ffn_hidden[j] *= s->ffn_gate[j];
            sgemm_m1(s->ffn_hidden, Fp[2].data, s->x, d, s->F, 0, 1.0f);
        } else {
            /* W1, b1, W2, b2 (inference.cpp:242-248) */
            matvec(s->h, &Fp[0], &Fp[1], s->ffn_hidden);
            gelu_row(s->ffn_hidden, s->tmp, s->F);
            matvec_add(s->ffn_hidden, &Fp[2], &Fp[3], s->x);
        }
    }

    const tensor_t* FN = &m->t[m->n_tensors - 2];
    layer_norm_row(s->x, FN[0].data, FN[1].data, modern, d, s->h);
    /* logits = h @ E^T (inference.cpp:254) */
    sgemm_m1(s->h, E->data, s->logits, s->V, d, 1, 0.0f);

    s->pos++;
    if (logits_out) *logits_out = s->logits;
    return GR_OK;
}

/* ------------------------------------------------------------------ TextGen */

/* text_gen.cpp:14-33 — each of the last min(50, n) tokens is penalised once
 * per occurrence, in order. */
void gr_logits_with_penalty(const float* logits, int vocab, const int* tokens, size_t n_tokens,
                            float penalty, float* out) {
    memcpy(out, logits, (size_t)vocab * sizeof(float));
    if (penalty != 1.0f) {
        const size_t window = n_tokens < 50 ? n_tokens : 50;
        for (size_t k = n_tokens - window; k < n_tokens; k++) {
            const int id = tokens[k];
            if (out[id] > 0)
                out[id] /= penalty;
            else
                out[id] *= penalty;
        }
    }
}

/* text_gen.cpp:52-60 — strict '>' keeps the lowest index among equal maxima. */
int gr_argmax_first(const float* data, int vocab) {
    int next = 0;
    float best = data[0];
    for (int j = 1; j < vocab; j++) {
        if (data[j] > best) {
            best = data[j];
            next = j;
        }
    }
    return next;
}

static int cmp_desc(const void* a, const void* b) {
    const float x = *(const float*)a, y = *(const float*)b;
    return (x < y) - (x > y);
}

/* text_gen.cpp:135-209 with the draw `u` supplied by the caller.  The
 * reference sorts (value, index) pairs by value only; just the sorted values
 * matter (k-th value; cumulative sums of equal values are order-free). */
int gr_sample_from_logits(const float* logits, int vocab, float temperature, int top_k,
                          float top_p, float u, float* probs_out) {
    const size_t n = (size_t)vocab;
    float* p = (float*)malloc(n * sizeof(float));
    float* sorted = (float*)malloc(n * sizeof(float));

    /* Tensor::scale(1/T), tensor.cpp:459-464 */
    const float inv_t = 1.0f / temperature;
    for (size_t i = 0; i < n; i++) p[i] = logits[i] * inv_t;

    if (top_k > 0 && top_k < vocab) {
        memcpy(sorted, p, n * sizeof(float));
        qsort(sorted, n, sizeof(float), cmp_desc);
        const float min_logit = sorted[top_k - 1];
        for (size_t i = 0; i < n; i++)
            if (p[i] < min_logit) p[i] = -1e10f;
    }

    /* Tensor::softmax, tensor.cpp:421-452 */
    float max_val = p[0];
    for (size_t j = 1; j < n; j++) max_val = p[j] > max_val ? p[j] : max_val;
    for (size_t j = 0; j < n; j++) p[j] = p[j] - max_val;
    for (size_t j = 0; j < n; j++) p[j] = expf(p[j]);
    const float inv_sum = 1.0f / vec_sum(p, n);
    for (size_t j = 0; j < n; j++) p[j] *= inv_sum;

    if (top_p < 1.0f) {
        memcpy(sorted, p, n * sizeof(float));
        qsort(sorted, n, sizeof(float), cmp_desc);
        float cumulative = 0.0f;
        size_t cutoff_idx = 0;
        for (size_t i = 0; i < n; i++) {
            cumulative += sorted[i];
            if (cumulative >= top_p) {
                cutoff_idx = i;
                break;
            }
        }
        const float cutoff_prob = sorted[cutoff_idx];
        float total_kept = 0.0f;
        for (size_t i = 0; i < n; i++) {
            if (p[i] < cutoff_prob)
                p[i] = 0.0f;
            else
                total_kept += p[i];
        }
        if (total_kept > 0.0f)
            for (size_t i = 0; i < n; i++) p[i] = p[i] / total_kept;
    }

    if (probs_out) memcpy(probs_out, p, n * sizeof(float));

    int chosen = vocab - 1;
    float cumulative = 0.0f;
    for (size_t i = 0; i < n; i++) {
        cumulative += p[i];
        if (u <= cumulative) {
            chosen = (int)i;
            break;
        }
    }
    free(p);
    free(sorted);
    return chosen;
}

/* text_gen.cpp:37-91: the greedy and sampled loops differ only in the pick. */
static int generate(const gr_model* m, const int* prompt, size_t n_prompt, int greedy,
                    float temperature, int max_tokens, float penalty, int top_k, float top_p,
                    const float* uniforms, int* out_tokens, size_t* out_n, float* step_logits,
                    size_t* n_steps) {
    *out_n = 0;
    if (n_steps) *n_steps = 0;
    if (n_prompt == 0) return GR_OK; /* text_gen.cpp:40 */
    memcpy(out_tokens, prompt, n_prompt * sizeof(int));
    size_t n = n_prompt, steps = 0;

    gr_session* s = gr_session_new(m);
    const int V = gr_session_vocab(s);
    const float* logits = NULL;
    float* work = (float*)malloc((size_t)V * sizeof(float));
    int rc = GR_OK;
    for (size_t i = 0; i < n_prompt; i++) {
        if ((rc = gr_session_step(s, prompt[i], &logits)) != GR_OK) goto done;
        if (step_logits) memcpy(step_logits + steps * (size_t)V, logits, (size_t)V * sizeof(float));
        steps++;
    }
    for (int i = 0; i < max_tokens; i++) {
        gr_logits_with_penalty(logits, V, out_tokens, n, penalty, work);
        const int next = greedy ? gr_argmax_first(work, V)
                                : gr_sample_from_logits(work, V, temperature, top_k, top_p,
                                                        uniforms[i], NULL);
        out_tokens[n++] = next;
        if (gr_session_position(s) >= gr_session_capacity(s)) break;
        if ((rc = gr_session_step(s, next, &logits)) != GR_OK) goto done;
        if (step_logits) memcpy(step_logits + steps * (size_t)V, logits, (size_t)V * sizeof(float));
        steps++;
    }
done:
    free(work);
    gr_session_free(s);
    *out_n = n;
    if (n_steps) *n_steps = steps;
    return rc;
}

int gr_generate_greedy(const gr_model* m, const int* prompt, size_t n_prompt, int max_tokens,
                       float penalty, int* out_tokens, size_t* out_n, float* step_logits,
                       size_t* n_steps) {
    return generate(m, prompt, n_prompt, 1, 1.0f, max_tokens, penalty, 0, 1.0f, NULL, out_tokens,
                    out_n, step_logits, n_steps);
}

int gr_generate_sample(const gr_model* m, const int* prompt, size_t n_prompt, float temperature,
                       int max_tokens, float penalty, int top_k, float top_p,
                       const float* uniforms, int* out_tokens, size_t* out_n, float* step_logits,
                       size_t* n_steps) {
    return generate(m, prompt, n_prompt, 0, temperature, max_tokens, penalty, top_k, top_p,
                    uniforms, out_tokens, out_n, step_logits, n_steps);
}
