"""ctypes binding of oracle/libgradref.so (the CPU checker).  Test-side only."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_LIB_PATH = os.path.join(ROOT, "oracle", "libgradref.so")

GR_OK, GR_RUNTIME_ERROR, GR_OUT_OF_RANGE, GR_INVALID_ARGUMENT = 0, 1, 2, 3
_EXC = {GR_RUNTIME_ERROR: RuntimeError, GR_OUT_OF_RANGE: IndexError, GR_INVALID_ARGUMENT: ValueError}

_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int)


def _load():
    if not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    lib = C.CDLL(_LIB_PATH)
    lib.gr_last_error.restype = C.c_char_p
    lib.gr_model_new.restype = C.c_void_p
    lib.gr_model_new.argtypes = [C.c_int] * 6 + [C.c_float]
    lib.gr_model_free.argtypes = [C.c_void_p]
    lib.gr_model_load.argtypes = [C.c_char_p, C.POINTER(C.c_void_p)]
    lib.gr_model_save.argtypes = [C.c_void_p, C.c_char_p]
    lib.gr_model_num_tensors.argtypes = [C.c_void_p]
    lib.gr_model_tensor.restype = _f32p
    lib.gr_model_tensor.argtypes = [C.c_void_p, C.c_int, _i32p, _i32p]
    lib.gr_model_dims.argtypes = [C.c_void_p] + [_i32p] * 7 + [_f32p]
    lib.gr_model_set_fingerprint.argtypes = [C.c_void_p, C.c_uint32, C.c_uint64]
    lib.gr_model_get_fingerprint.argtypes = [C.c_void_p, C.POINTER(C.c_uint32), C.POINTER(C.c_uint64)]
    lib.gr_session_new.restype = C.c_void_p
    lib.gr_session_new.argtypes = [C.c_void_p]
    lib.gr_session_free.argtypes = [C.c_void_p]
    lib.gr_session_step.argtypes = [C.c_void_p, C.c_int, C.POINTER(_f32p)]
    for n in ("position", "capacity", "vocab"):
        getattr(lib, "gr_session_" + n).argtypes = [C.c_void_p]
    for n in ("k_row", "v_row"):
        fn = getattr(lib, "gr_session_" + n)
        fn.restype = _f32p
        fn.argtypes = [C.c_void_p, C.c_int, C.c_int]
    lib.gr_logits_with_penalty.restype = None
    lib.gr_logits_with_penalty.argtypes = [_f32p, C.c_int, _i32p, C.c_size_t, C.c_float, _f32p]
    lib.gr_argmax_first.argtypes = [_f32p, C.c_int]
    lib.gr_sample_from_logits.argtypes = [_f32p, C.c_int, C.c_float, C.c_int, C.c_float, C.c_float, _f32p]
    lib.gr_generate_greedy.argtypes = [C.c_void_p, _i32p, C.c_size_t, C.c_int, C.c_float, _i32p,
                                       C.POINTER(C.c_size_t), _f32p, C.POINTER(C.c_size_t)]
    lib.gr_generate_sample.argtypes = [C.c_void_p, _i32p, C.c_size_t, C.c_float, C.c_int, C.c_float,
                                       C.c_int, C.c_float, _f32p, _i32p, C.POINTER(C.c_size_t),
                                       _f32p, C.POINTER(C.c_size_t)]
    lib.gr_blas_init.restype = C.c_char_p
    lib.gr_blas_init.argtypes = [C.c_char_p]
    lib.gr_blas_set_threads.argtypes = [C.c_int]
    return lib


lib = _load()


def _check(rc):
    if rc != GR_OK:
        raise _EXC.get(rc, RuntimeError)(lib.gr_last_error().decode())


def _fp(a):
    return a.ctypes.data_as(_f32p)


def _ip(a):
    return a.ctypes.data_as(_i32p)


def blas_init(hint: str | None = None) -> str:
    return lib.gr_blas_init(hint.encode() if hint else None).decode()


def blas_set_threads(n: int) -> None:
    lib.gr_blas_set_threads(n)


class Model:
    def __init__(self, handle):
        self.h = handle

    @classmethod
    def new(cls, arch, vocab, d_model, layers, heads, max_len, dropout=0.0):
        return cls(lib.gr_model_new(arch, vocab, d_model, layers, heads, max_len, dropout))

    @classmethod
    def load(cls, path):
        h = C.c_void_p()
        _check(lib.gr_model_load(os.fsencode(path), C.byref(h)))
        return cls(h.value)

    @classmethod
    def from_tensors(cls, cfg, tensors):
        m = cls.new(cfg.arch, cfg.vocab, cfg.d_model, cfg.layers, cfg.heads, cfg.max_len, cfg.dropout)
        assert m.num_tensors == len(tensors)
        for i, t in enumerate(tensors):
            m.tensor(i)[...] = t
        return m

    def save(self, path):
        _check(lib.gr_model_save(self.h, os.fsencode(path)))

    @property
    def num_tensors(self):
        return lib.gr_model_num_tensors(self.h)

    def tensor(self, i):
        r, c = C.c_int(), C.c_int()
        p = lib.gr_model_tensor(self.h, i, C.byref(r), C.byref(c))
        return np.ctypeslib.as_array(p, shape=(r.value, c.value))

    def dims(self):
        v = [C.c_int() for _ in range(7)]
        dr = C.c_float()
        lib.gr_model_dims(self.h, *[C.byref(x) for x in v], C.byref(dr))
        keys = ("arch", "vocab", "d_model", "layers", "heads", "max_len", "d_ff")
        out = {k: x.value for k, x in zip(keys, v)}
        out["dropout"] = dr.value
        return out

    def set_fingerprint(self, kind, h):
        lib.gr_model_set_fingerprint(self.h, kind, h)

    def fingerprint(self):
        k, h = C.c_uint32(), C.c_uint64()
        if not lib.gr_model_get_fingerprint(self.h, C.byref(k), C.byref(h)):
            return None
        return (k.value, h.value)

    def __del__(self):
        if getattr(self, "h", None):
            lib.gr_model_free(self.h)
            self.h = None


class Session:
    def __init__(self, model: Model):
        self.model = model
        self.h = lib.gr_session_new(model.h)
        self.vocab = lib.gr_session_vocab(self.h)
        self.d = model.dims()["d_model"]

    def step(self, token: int) -> np.ndarray:
        p = _f32p()
        _check(lib.gr_session_step(self.h, int(token), C.byref(p)))
        return np.ctypeslib.as_array(p, shape=(self.vocab,)).copy()

    @property
    def position(self):
        return lib.gr_session_position(self.h)

    @property
    def capacity(self):
        return lib.gr_session_capacity(self.h)

    def k_row(self, layer, pos):
        return np.ctypeslib.as_array(lib.gr_session_k_row(self.h, layer, pos), shape=(self.d,)).copy()

    def v_row(self, layer, pos):
        return np.ctypeslib.as_array(lib.gr_session_v_row(self.h, layer, pos), shape=(self.d,)).copy()

    def __del__(self):
        if getattr(self, "h", None):
            lib.gr_session_free(self.h)
            self.h = None


def logits_with_penalty(logits, tokens, penalty):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    tokens = np.ascontiguousarray(tokens, dtype=np.int32)
    out = np.empty_like(logits)
    lib.gr_logits_with_penalty(_fp(logits), len(logits), _ip(tokens), len(tokens), penalty, _fp(out))
    return out


def argmax_first(data):
    data = np.ascontiguousarray(data, dtype=np.float32)
    return lib.gr_argmax_first(_fp(data), len(data))


def sample_from_logits(logits, temperature=1.0, top_k=0, top_p=1.0, u=0.5, want_probs=False):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    probs = np.empty_like(logits)
    tok = lib.gr_sample_from_logits(_fp(logits), len(logits), temperature, top_k, top_p, u, _fp(probs))
    return (tok, probs) if want_probs else tok


def _generate(fn, model, prompt, max_tokens, want_logits, *mid):
    prompt = np.ascontiguousarray(prompt, dtype=np.int32)
    cap = len(prompt) + max(max_tokens, 0)
    out = np.zeros(max(cap, 1), dtype=np.int32)
    n, ns = C.c_size_t(), C.c_size_t()
    V = model.dims()["vocab"]
    sl = np.zeros((cap, V), dtype=np.float32) if want_logits else None
    _check(fn(model.h, _ip(prompt), len(prompt), *mid, _ip(out), C.byref(n),
              _fp(sl) if want_logits else None, C.byref(ns)))
    toks = out[:n.value].copy()
    return (toks, sl[:ns.value]) if want_logits else toks


def generate_greedy(model, prompt, max_tokens=50, penalty=1.2, want_logits=False):
    return _generate(lib.gr_generate_greedy, model, prompt, max_tokens, want_logits,
                     C.c_int(max_tokens), C.c_float(penalty))


def generate_sample(model, prompt, uniforms, temperature=1.0, max_tokens=50, penalty=1.2, top_k=0,
                    top_p=1.0, want_logits=False):
    u = np.ascontiguousarray(uniforms, dtype=np.float32)
    assert len(u) >= max_tokens
    prompt = np.ascontiguousarray(prompt, dtype=np.int32)
    cap = len(prompt) + max(max_tokens, 0)
    out = np.zeros(max(cap, 1), dtype=np.int32)
    n, ns = C.c_size_t(), C.c_size_t()
    V = model.dims()["vocab"]
    sl = np.zeros((cap, V), dtype=np.float32) if want_logits else None
    _check(lib.gr_generate_sample(model.h, _ip(prompt), len(prompt), temperature, max_tokens, penalty,
                                  top_k, top_p, _fp(u), _ip(out), C.byref(n),
                                  _fp(sl) if want_logits else None, C.byref(ns)))
    toks = out[:n.value].copy()
    return (toks, sl[:ns.value]) if want_logits else toks


def nll_rows(logits, targets):
    """Negative log-likelihood of targets[i] under softmax(logits[i]), in float64:
    Variable::cross_entropy's log_softmax + nll_loss (variable.cpp:589-592) before the mean
    over rows.  Pinned by closed forms in tests/test_oracle_textgen.py."""
    x = np.asarray(logits, dtype=np.float64)
    m = x.max(axis=-1, keepdims=True)
    lse = np.log(np.exp(x - m).sum(axis=-1)) + m[..., 0]
    return lse - np.take_along_axis(x, np.asarray(targets)[..., None], axis=-1)[..., 0]


def score(model, ids, targets):
    """Per-position NLL of one sequence, logits from step() (what `grad eval` averages,
    training/trainer.cpp:319-340, with the full-sequence forward replaced by the token loop,
    which the reference's own parity tests tie together, sanity_tests.cpp:293-333)."""
    s = Session(model)
    return np.array([nll_rows(s.step(int(t)), int(g)) for t, g in zip(ids, targets)])
