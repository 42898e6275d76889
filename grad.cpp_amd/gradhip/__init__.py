"""ctypes binding of libgradhip.so — the C ABI declared in include/gradhip.h.

This module is a thin host-side mirror used by the tests and the benchmark; it
holds no compute of its own and has no fallback: loading fails loudly when the
library has not been built, and every compute call fails when no GPU is usable.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import synth  # noqa: F401  (re-exported)

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(PKG, "lib", "libgradhip.so")

GH_OK, GH_ERR_RUNTIME, GH_ERR_OUT_OF_RANGE, GH_ERR_INVALID_ARGUMENT, GH_ERR_DEVICE = range(5)
ENGINE_AUTO, ENGINE_GRAPH, ENGINE_EAGER, ENGINE_PERSISTENT = range(4)
FLAG_PICK_GLOBAL_SCRATCH = 1
FLAG_STEPWISE_PROMPT = 2
FLAG_SMALL_ATTENTION_CHUNKS = 4
FLAG_CLASSIC_PERSISTENT = 8
FLAG_XCD_PERSISTENT = 16
FLAG_ROW_PICKS = 32


class DeviceError(RuntimeError):
    pass


_EXC = {GH_ERR_RUNTIME: RuntimeError, GH_ERR_OUT_OF_RANGE: IndexError,
        GH_ERR_INVALID_ARGUMENT: ValueError, GH_ERR_DEVICE: DeviceError}


class GhConfig(C.Structure):
    _fields_ = [("arch", C.c_int32), ("vocab", C.c_int32), ("d_model", C.c_int32),
                ("layers", C.c_int32), ("heads", C.c_int32), ("max_len", C.c_int32),
                ("d_ff", C.c_int32), ("dropout", C.c_float), ("has_fingerprint", C.c_int32),
                ("tokenizer_kind", C.c_uint32), ("tokenizer_hash", C.c_uint64)]


class GhSessionOpts(C.Structure):
    _fields_ = [("batch", C.c_int32), ("engine", C.c_int32), ("page_tokens", C.c_int32),
                ("shuffle_pages", C.c_int32), ("flags", C.c_int32)]


class GhSampling(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_int32), ("top_p", C.c_float),
                ("repetition_penalty", C.c_float), ("greedy", C.c_int32)]


class GhTiming(C.Structure):
    _fields_ = [("prompt_ms", C.c_float), ("decode_ms", C.c_float), ("prompt_steps", C.c_int32),
                ("decode_steps", C.c_int32), ("launches_per_step", C.c_int32), ("row_picks", C.c_int32)]


class GhTokenizerInfo(C.Structure):
    _fields_ = [("kind", C.c_uint32), ("vocab_size", C.c_int32), ("eos_id", C.c_int32),
                ("n_merges", C.c_int32), ("n_specials", C.c_int32), ("fingerprint", C.c_uint64)]


# Every symbol include/gradhip.h declares: name -> (restype, argtypes)
_f32p, _i32p, _vp = C.POINTER(C.c_float), C.POINTER(C.c_int32), C.c_void_p
TokenCallback = C.CFUNCTYPE(C.c_int32, C.c_void_p, C.POINTER(C.c_int32), C.c_int32)  # gh_token_callback
SYMBOLS = {
    "gh_last_error": (C.c_char_p, []),
    "gh_model_load": (C.c_int, [C.c_char_p, C.POINTER(_vp)]),
    "gh_model_from_host": (C.c_int, [C.POINTER(GhConfig), C.POINTER(_f32p), C.c_int32, C.POINTER(_vp)]),
    "gh_config_num_tensors": (C.c_int32, [C.POINTER(GhConfig)]),
    "gh_config_tensor_shape": (C.c_int, [C.POINTER(GhConfig), C.c_int32, _i32p, _i32p]),
    "gh_model_save": (C.c_int, [_vp, C.c_char_p]),
    "gh_model_free": (None, [_vp]),
    "gh_model_get_config": (C.c_int, [_vp, C.POINTER(GhConfig)]),
    "gh_session_create": (C.c_int, [_vp, C.POINTER(GhSessionOpts), C.POINTER(_vp)]),
    "gh_session_free": (None, [_vp]),
    "gh_session_reset": (C.c_int, [_vp]),
    "gh_session_step": (C.c_int, [_vp, _i32p, _f32p]),
    "gh_session_logits": (C.c_int, [_vp, C.POINTER(_f32p)]),
    "gh_session_prefill": (C.c_int, [_vp, _i32p, C.c_int32, _f32p]),
    "gh_session_score": (C.c_int, [_vp, _i32p, _i32p, C.c_int32, _f32p]),
    "gh_session_position": (C.c_int32, [_vp]),
    "gh_session_capacity": (C.c_int32, [_vp]),
    "gh_session_vocab": (C.c_int32, [_vp]),
    "gh_session_batch": (C.c_int32, [_vp]),
    "gh_session_read_kv": (C.c_int, [_vp, C.c_int32, C.c_int32, C.c_int32, C.c_int32, _f32p]),
    "gh_session_pick": (C.c_int, [_vp, C.POINTER(GhSampling), _f32p, C.c_uint64, _i32p]),
    "gh_session_decode": (C.c_int, [_vp, C.c_int32, C.POINTER(GhSampling), _f32p, C.c_uint64, _i32p, _i32p]),
    "gh_session_decode_stream": (C.c_int, [_vp, C.c_int32, C.POINTER(GhSampling), _f32p, C.c_uint64, C.c_int32,
                                           TokenCallback, _vp, _i32p, _i32p]),
    "gh_session_generate": (C.c_int, [_vp, _i32p, C.c_int32, C.c_int32, C.POINTER(GhSampling), _f32p,
                                      C.c_uint64, _i32p, _i32p, _f32p, _i32p]),
    "gh_pick_noalloc": (C.c_int, [_vp, C.c_int32, C.c_int32, _vp, C.c_int32, C.c_int32, C.POINTER(GhSampling), _vp,
                                  C.c_uint64, C.c_int32, _vp, _vp]),
    "gh_session_last_timing": (C.c_int, [_vp, C.POINTER(GhTiming)]),
    "gh_tokenizer_load": (C.c_int, [C.c_char_p, C.POINTER(_vp)]),
    "gh_tokenizer_from_merges": (C.c_int, [_i32p, C.c_int32, C.POINTER(C.c_char_p), _i32p, C.c_int32,
                                           C.POINTER(_vp)]),
    "gh_tokenizer_save": (C.c_int, [_vp, C.c_char_p]),
    "gh_tokenizer_free": (None, [_vp]),
    "gh_tokenizer_get_info": (C.c_int, [_vp, C.POINTER(GhTokenizerInfo)]),
    "gh_tokenizer_special_id": (C.c_int, [_vp, C.c_char_p, C.c_size_t, _i32p]),
    "gh_tokenizer_encode": (C.c_int, [_vp, C.c_char_p, C.c_size_t, C.c_int32, _i32p, C.c_size_t,
                                      C.POINTER(C.c_size_t)]),
    "gh_tokenizer_decode": (C.c_int, [_vp, _i32p, C.c_size_t, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]),
    "gh_pretokenize": (C.c_int, [C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t), C.c_size_t,
                                 C.POINTER(C.c_size_t)]),
    "gh_codepoint_class": (C.c_int32, [C.c_uint32]),
    "gh_device_info": (C.c_int, [C.c_char_p, C.c_size_t, _i32p, _i32p]),
    "gh_device_read_bandwidth": (C.c_int, [C.c_size_t, C.c_int32, C.POINTER(C.c_double)]),
    "gh_device_reread_bandwidth": (C.c_int, [C.c_size_t, C.c_int32, C.POINTER(C.c_double)]),
    "gh_device_handoff_latency": (C.c_int, [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_double),
                                            C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "gh_device_mfma_issue": (C.c_int, [C.c_int32, C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_double),
                                       C.POINTER(C.c_double)]),
}

_lib = None


def load_library(path: str | None = None):
    """Loads libgradhip.so and binds every declared symbol (AttributeError if one
    is missing).  Needs no GPU."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise FileNotFoundError(
            f"{p} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
    lib = C.CDLL(p)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


def _check(rc):
    if rc != GH_OK:
        raise _EXC.get(rc, RuntimeError)(load_library().gh_last_error().decode())


def device_info():
    lib = load_library()
    name = C.create_string_buffer(256)
    cu, ok = C.c_int32(), C.c_int32()
    _check(lib.gh_device_info(name, 256, C.byref(cu), C.byref(ok)))
    return {"name": name.value.decode(), "compute_units": cu.value, "is_gfx950": bool(ok.value)}


def read_bandwidth(nbytes: int = 2 << 30, repeats: int = 5) -> float:
    """GB/s of a plain streaming read of `nbytes` of device memory (best of `repeats`)."""
    out = C.c_double()
    _check(load_library().gh_device_read_bandwidth(nbytes, repeats, C.byref(out)))
    return out.value


def reread_bandwidth(nbytes: int, passes: int = 20) -> float:
    """GB/s of `passes` back-to-back streaming reads of one buffer of `nbytes` (one timed span)."""
    out = C.c_double(0.0)
    _check(load_library().gh_device_reread_bandwidth(nbytes, passes, C.byref(out)))
    return out.value


def handoff_latency(load_policy: int, device_scope_store: bool, peer: int, busy: bool):
    """(us per round trip, XCD of workgroup 0, XCD of workgroup `peer`) of a two-workgroup ping-pong."""
    out, xa, xb = C.c_double(0.0), C.c_int32(-1), C.c_int32(-1)
    _check(load_library().gh_device_handoff_latency(load_policy, 1 if device_scope_store else 0, peer,
                                                    1 if busy else 0, C.byref(out), C.byref(xa), C.byref(xb)))
    return out.value, xa.value, xb.value


def mfma_issue(mode: int, valu_per_slot: int = 8):
    """(cycles per fp32 matrix product of wavefronts 0-3, cycles per slot of multiply-adds of
    wavefronts 4-7, shader MHz); the modes are gh_device_mfma_issue's."""
    a, b, c = C.c_double(0.0), C.c_double(0.0), C.c_double(0.0)
    _check(load_library().gh_device_mfma_issue(mode, valu_per_slot, C.byref(a), C.byref(b), C.byref(c)))
    return a.value, b.value, c.value


def pick_noalloc(logits_ptr: int, batch: int, vocab: int, history_ptr: int, history_stride: int, n_history: int,
                 opt: GhSampling, out_ids_ptr: int, uniforms_ptr: int = 0, seed: int = 0, pick_index: int = 0,
                 stream: int = 0) -> None:
    """gh_pick_noalloc: every *_ptr is a DEVICE address (an int); enqueues the pick on
    `stream` (a hipStream_t as an int, 0 = default stream) and returns without waiting."""
    _check(load_library().gh_pick_noalloc(logits_ptr, batch, vocab, history_ptr or None, history_stride, n_history,
                                          C.byref(opt), uniforms_ptr or None, seed, pick_index, out_ids_ptr,
                                          stream or None))


def _cfg_struct(cfg: synth.Config, fingerprint=None) -> GhConfig:
    c = GhConfig(cfg.arch, cfg.vocab, cfg.d_model, cfg.layers, cfg.heads, cfg.max_len, 0, cfg.dropout,
                 0, 0, 0)
    if fingerprint is not None:
        c.has_fingerprint, c.tokenizer_kind, c.tokenizer_hash = 1, fingerprint[0], fingerprint[1]
    return c


class Model:
    """Device-resident weights of one checkpoint (stands in for grad::GPTModel)."""

    def __init__(self, handle):
        self._h = handle

    @classmethod
    def load(cls, path) -> "Model":
        h = _vp()
        _check(load_library().gh_model_load(os.fsencode(path), C.byref(h)))
        return cls(h.value)

    @classmethod
    def from_tensors(cls, cfg: synth.Config, tensors, fingerprint=None) -> "Model":
        lib = load_library()
        keep = [np.ascontiguousarray(t, dtype=np.float32) for t in tensors]
        arr = (_f32p * len(keep))(*[t.ctypes.data_as(_f32p) for t in keep])
        h = _vp()
        c = _cfg_struct(cfg, fingerprint)
        _check(lib.gh_model_from_host(C.byref(c), arr, len(keep), C.byref(h)))
        return cls(h.value)

    def save(self, path) -> None:
        _check(load_library().gh_model_save(self._h, os.fsencode(path)))

    @property
    def config(self) -> GhConfig:
        c = GhConfig()
        _check(load_library().gh_model_get_config(self._h, C.byref(c)))
        return c

    def close(self):
        if self._h:
            load_library().gh_model_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def pretokenize(text: bytes) -> list:
    """Pieces of `text` under GPT-2's pattern (stands in for grad::pretok::split)."""
    lib = load_library()
    n = C.c_size_t()
    _check(lib.gh_pretokenize(text, len(text), None, 0, C.byref(n)))
    ends = (C.c_size_t * max(n.value, 1))()
    _check(lib.gh_pretokenize(text, len(text), ends, n.value, C.byref(n)))
    out, pos = [], 0
    for e in ends[:n.value]:
        out.append(text[pos:e])
        pos = e
    return out


def codepoint_class(cp: int) -> int:
    """0 other, 1 letter, 2 number, 3 white space (grad::pretok::classify)."""
    return load_library().gh_codepoint_class(cp)


class Tokenizer:
    """Byte-level BPE over a GTOK v2 file (stands in for grad::ByteBpe behind grad::Tokenizer).
    Text goes in and out as bytes: decode(encode(b)) == b for every byte string."""

    def __init__(self, handle):
        self._h = handle

    @classmethod
    def load(cls, path) -> "Tokenizer":
        h = _vp()
        _check(load_library().gh_tokenizer_load(os.fsencode(path), C.byref(h)))
        return cls(h.value)

    @classmethod
    def from_merges(cls, merges, specials=(b"<|endoftext|>",)) -> "Tokenizer":
        m = np.ascontiguousarray(np.asarray(merges, dtype=np.int32).reshape(-1, 2))
        sp = [bytes(x) for x in specials]
        arr = (C.c_char_p * max(len(sp), 1))(*sp)
        lens = (C.c_int32 * max(len(sp), 1))(*[len(x) for x in sp])
        h = _vp()
        _check(load_library().gh_tokenizer_from_merges(m.ctypes.data_as(_i32p), len(m), arr, lens, len(sp),
                                                       C.byref(h)))
        return cls(h.value)

    def save(self, path) -> None:
        _check(load_library().gh_tokenizer_save(self._h, os.fsencode(path)))

    @property
    def info(self) -> GhTokenizerInfo:
        out = GhTokenizerInfo()
        _check(load_library().gh_tokenizer_get_info(self._h, C.byref(out)))
        return out

    def special_id(self, token: bytes):
        out = C.c_int32()
        _check(load_library().gh_tokenizer_special_id(self._h, token, len(token), C.byref(out)))
        return None if out.value < 0 else out.value

    def encode(self, text: bytes, with_specials=True) -> np.ndarray:
        lib = load_library()
        n = C.c_size_t()
        cap = max(len(text), 1)  # never more ids than bytes
        ids = np.empty(cap, np.int32)
        _check(lib.gh_tokenizer_encode(self._h, text, len(text), 1 if with_specials else 0,
                                       ids.ctypes.data_as(_i32p), cap, C.byref(n)))
        return ids[:n.value].copy()

    def decode(self, ids) -> bytes:
        lib = load_library()
        a = np.ascontiguousarray(ids, dtype=np.int32)
        n = C.c_size_t()
        _check(lib.gh_tokenizer_decode(self._h, a.ctypes.data_as(_i32p), len(a), None, 0, C.byref(n)))
        buf = C.create_string_buffer(max(n.value, 1))
        _check(lib.gh_tokenizer_decode(self._h, a.ctypes.data_as(_i32p), len(a), buf, n.value, C.byref(n)))
        return buf.raw[:n.value]

    def close(self):
        if self._h:
            load_library().gh_tokenizer_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def sampling(temperature=1.0, top_k=0, top_p=1.0, repetition_penalty=1.2, greedy=False) -> GhSampling:
    return GhSampling(temperature, top_k, top_p, repetition_penalty, 1 if greedy else 0)


class Session:
    """KV-cached decoder state for `batch` sequences (stands in for grad::InferenceSession)."""

    def __init__(self, model: Model, batch=1, engine=ENGINE_AUTO, page_tokens=0, shuffle_pages=False,
                 flags=0):
        self.model = model
        opts = GhSessionOpts(batch, engine, page_tokens, 1 if shuffle_pages else 0, flags)
        h = _vp()
        _check(load_library().gh_session_create(model._h, C.byref(opts), C.byref(h)))
        self._h = h.value
        self.batch = batch
        self.vocab = load_library().gh_session_vocab(self._h)

    def close(self):
        if self._h:
            load_library().gh_session_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def position(self):
        return load_library().gh_session_position(self._h)

    @property
    def capacity(self):
        return load_library().gh_session_capacity(self._h)

    def reset(self):
        _check(load_library().gh_session_reset(self._h))

    def step(self, ids) -> np.ndarray:
        ids = np.ascontiguousarray(np.atleast_1d(ids), dtype=np.int32)
        assert ids.shape == (self.batch,)
        out = np.empty((self.batch, self.vocab), dtype=np.float32)
        _check(load_library().gh_session_step(self._h, ids.ctypes.data_as(_i32p),
                                              out.ctypes.data_as(_f32p)))
        return out

    def prefill(self, ids) -> np.ndarray:
        ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(self.batch, -1)
        out = np.empty((self.batch, self.vocab), dtype=np.float32)
        _check(load_library().gh_session_prefill(self._h, ids.ctypes.data_as(_i32p), ids.shape[1],
                                                 out.ctypes.data_as(_f32p)))
        return out

    def score(self, ids, targets) -> np.ndarray:
        """Negative log-likelihood of targets[b, t] at every position (what `grad eval` averages)."""
        ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(self.batch, -1)
        targets = np.ascontiguousarray(targets, dtype=np.int32).reshape(self.batch, -1)
        assert ids.shape == targets.shape
        out = np.empty(ids.shape, dtype=np.float32)
        _check(load_library().gh_session_score(self._h, ids.ctypes.data_as(_i32p), targets.ctypes.data_as(_i32p),
                                               ids.shape[1], out.ctypes.data_as(_f32p)))
        return out

    def read_kv(self, seq, layer, kv, pos) -> np.ndarray:
        d = self.model.config.d_model
        out = np.empty(d, dtype=np.float32)
        _check(load_library().gh_session_read_kv(self._h, seq, layer, kv, pos, out.ctypes.data_as(_f32p)))
        return out

    def pick(self, opt: GhSampling, uniforms=None, seed=0) -> np.ndarray:
        out = np.empty(self.batch, dtype=np.int32)
        u = None
        if uniforms is not None:
            u = np.ascontiguousarray(np.atleast_1d(uniforms), dtype=np.float32)
            assert u.shape == (self.batch,)
        _check(load_library().gh_session_pick(self._h, C.byref(opt),
                                              u.ctypes.data_as(_f32p) if u is not None else None,
                                              seed, out.ctypes.data_as(_i32p)))
        return out

    def decode(self, max_tokens, opt: GhSampling, uniforms=None, seed=0) -> np.ndarray:
        """Continues from the current context; returns the picks (batch, n)."""
        out = np.zeros((self.batch, max(max_tokens, 1)), dtype=np.int32)
        n = C.c_int32()
        u = None
        if uniforms is not None:
            u = np.ascontiguousarray(uniforms, dtype=np.float32).reshape(self.batch, -1)
            u = np.ascontiguousarray(u[:, :max_tokens])
            assert u.shape[1] == max_tokens
        _check(load_library().gh_session_decode(
            self._h, max_tokens, C.byref(opt), u.ctypes.data_as(_f32p) if u is not None else None, seed,
            out.ctypes.data_as(_i32p), C.byref(n)))
        return out[:, :n.value].copy()

    def decode_stream(self, max_tokens, opt: GhSampling, on_tokens, stop_token=-1, uniforms=None, seed=0):
        """decode() with every round's picks handed to on_tokens(ids, index) as they are made; a
        true return value asks for the run to end, stop_token ends it after the round that picks
        it.  Returns the picks (batch, n)."""
        out = np.zeros((self.batch, max(max_tokens, 1)), dtype=np.int32)
        n = C.c_int32()
        u = None
        if uniforms is not None:
            u = np.ascontiguousarray(uniforms, dtype=np.float32).reshape(self.batch, max_tokens)
        failure = []

        def relay(_user, ids, index):
            if failure:
                return 1
            try:
                return 1 if on_tokens([ids[b] for b in range(self.batch)], index) else 0
            except BaseException as e:  # raised again once the run has ended
                failure.append(e)
                return 1

        _check(load_library().gh_session_decode_stream(
            self._h, max_tokens, C.byref(opt), u.ctypes.data_as(_f32p) if u is not None else None, seed,
            stop_token, TokenCallback(relay), None, out.ctypes.data_as(_i32p), C.byref(n)))
        if failure:
            raise failure[0]
        return out[:, :n.value].copy()

    def generate(self, prompts, max_tokens, opt: GhSampling, uniforms=None, seed=0, want_logits=False):
        """Returns tokens (batch, n) and, when asked, step logits (steps, batch, vocab)."""
        prompts = np.ascontiguousarray(prompts, dtype=np.int32).reshape(self.batch, -1)
        plen = prompts.shape[1]
        out = np.zeros((self.batch, plen + max(max_tokens, 0)), dtype=np.int32)
        n, ns = C.c_int32(), C.c_int32()
        u = None
        if uniforms is not None:
            u = np.ascontiguousarray(uniforms, dtype=np.float32).reshape(self.batch, -1)
            assert u.shape[1] >= max_tokens
            u = np.ascontiguousarray(u[:, :max_tokens])
        sl = np.zeros((plen + max(max_tokens, 0), self.batch, self.vocab), dtype=np.float32) \
            if want_logits else None
        _check(load_library().gh_session_generate(
            self._h, prompts.ctypes.data_as(_i32p), plen, max_tokens, C.byref(opt),
            u.ctypes.data_as(_f32p) if u is not None else None, seed, out.ctypes.data_as(_i32p),
            C.byref(n), sl.ctypes.data_as(_f32p) if want_logits else None, C.byref(ns)))
        toks = out[:, :n.value].copy()
        return (toks, sl[:ns.value]) if want_logits else toks

    def last_timing(self) -> dict:
        t = GhTiming()
        _check(load_library().gh_session_last_timing(self._h, C.byref(t)))
        return {k: getattr(t, k) for k, _ in GhTiming._fields_}
