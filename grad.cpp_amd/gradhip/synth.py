"""Seeded synthetic inputs: Philox4x32-10 -> Box-Muller weights, prompts, uniforms,
and a writer for grad.cpp's "GPTM" v2 checkpoint files.

Everything here is fully specified integer/float64 arithmetic, so the same seed
gives the same bytes on every host.  The checkpoint layout follows
src/transformer/gpt_model.cpp:292-381 of grad.cpp (header, tensor records in
getAllParameters order, optional "TKFP" trailer).
"""
from __future__ import annotations

import struct
from dataclasses import dataclass

import numpy as np

ARCH_GPT2 = 0
ARCH_MODERN = 1

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_W0 = 0x9E3779B9
_W1 = 0xBB67AE85
_MASK = np.uint64(0xFFFFFFFF)
_SH32 = np.uint64(32)


def philox4x32(counter: np.ndarray, key: tuple[int, int], rounds: int = 10) -> np.ndarray:
    """Philox4x32 on an (n, 4) uint32 counter array with one (k0, k1) key."""
    c = [counter[:, i].astype(np.uint64) for i in range(4)]
    k0, k1 = key[0] & 0xFFFFFFFF, key[1] & 0xFFFFFFFF
    for _ in range(rounds):
        p0 = _M0 * c[0]
        p1 = _M1 * c[2]
        hi0, lo0 = p0 >> _SH32, p0 & _MASK
        hi1, lo1 = p1 >> _SH32, p1 & _MASK
        c = [hi1 ^ c[1] ^ np.uint64(k0), lo1, hi0 ^ c[3] ^ np.uint64(k1), lo0]
        k0 = (k0 + _W0) & 0xFFFFFFFF
        k1 = (k1 + _W1) & 0xFFFFFFFF
    return np.stack(c, axis=1).astype(np.uint32)


def _blocks(n_blocks: int, start: int = 0) -> np.ndarray:
    idx = np.arange(start, start + n_blocks, dtype=np.uint64)
    ctr = np.zeros((n_blocks, 4), dtype=np.uint32)
    ctr[:, 0] = (idx & _MASK).astype(np.uint32)
    ctr[:, 1] = (idx >> _SH32).astype(np.uint32)
    return ctr


def random_u32(n: int, seed: int, stream: int) -> np.ndarray:
    """n uint32 words of stream (seed, stream); word i is lane i%4 of block i//4."""
    out = np.empty(((n + 3) // 4) * 4, dtype=np.uint32)
    chunk = 1 << 20
    nb = (n + 3) // 4
    for b in range(0, nb, chunk):
        m = min(chunk, nb - b)
        out[4 * b:4 * (b + m)] = philox4x32(_blocks(m, b), (seed, stream)).reshape(-1)
    return out[:n]


def normal(n: int, seed: int, stream: int, std: float) -> np.ndarray:
    """n float32 draws of N(0, std): Box-Muller in float64 on 32-bit uniforms."""
    words = random_u32(2 * ((n + 1) // 2), seed, stream).astype(np.float64)
    u1 = (words[0::2] + 0.5) / 4294967296.0
    u2 = (words[1::2] + 0.5) / 4294967296.0
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.empty(2 * len(u1), dtype=np.float64)
    z[0::2] = r * np.cos(2.0 * np.pi * u2)
    z[1::2] = r * np.sin(2.0 * np.pi * u2)
    return (z[:n] * std).astype(np.float32)


def uniform_tokens(n: int, vocab: int, seed: int, stream: int = 0) -> np.ndarray:
    """n token ids uniform on [0, vocab) (multiply-shift on 32-bit words)."""
    w = random_u32(n, seed, stream).astype(np.uint64)
    return ((w * np.uint64(vocab)) >> _SH32).astype(np.int32)


def uniforms(n: int, seed: int, stream: int = 0) -> np.ndarray:
    """n float32 uniforms on [0, 1): the top 24 bits of each 32-bit word."""
    w = random_u32(n, seed, stream)
    return ((w >> np.uint32(8)).astype(np.float32) * np.float32(1.0 / 16777216.0)).astype(np.float32)


@dataclass(frozen=True)
class Config:
    arch: int
    vocab: int
    d_model: int
    layers: int
    heads: int
    max_len: int
    dropout: float = 0.0

    @property
    def modern(self) -> bool:
        return self.arch == ARCH_MODERN

    @property
    def head_size(self) -> int:
        return self.d_model // self.heads

    @property
    def d_ff(self) -> int:
        # include/grad/transformer/feedforward.h:24-28
        if not self.modern:
            return 4 * self.d_model
        return ((8 * self.d_model // 3) + 63) // 64 * 64


# The shapes of the benchmark configurations (src/cli/presets.cpp:40-120 of grad.cpp).
PRESETS = {
    "c0": Config(ARCH_GPT2, 5000, 512, 6, 8, 96),
    "c1": Config(ARCH_GPT2, 16000, 768, 8, 12, 256),
    "c2": Config(ARCH_MODERN, 16000, 768, 8, 12, 256),
    "c4": Config(ARCH_MODERN, 16000, 768, 8, 12, 2048),
}


def tensor_specs(cfg: Config) -> list[tuple[str, int, int, str]]:
    """(name, rows, cols, kind) in checkpoint order; kind in matrix|bias|gamma|beta."""
    d, F = cfg.d_model, cfg.d_ff
    specs = [("token embedding", cfg.vocab, d, "matrix")]
    if not cfg.modern:
        specs.append(("position embedding", cfg.max_len, d, "matrix"))
    for l in range(cfg.layers):
        p = f"layer {l} "
        for n in ("W_q", "W_k", "W_v", "W_o"):
            specs.append((p + n, d, d, "matrix"))
        for n in ("b_q", "b_k", "b_v", "b_o"):
            specs.append((p + n, 1, d, "bias"))
        if cfg.modern:
            specs += [(p + "FFN gate", d, F, "matrix"), (p + "FFN up", d, F, "matrix"),
                      (p + "FFN down", F, d, "matrix")]
        else:
            specs += [(p + "FFN W1", d, F, "matrix"), (p + "FFN b1", 1, F, "bias"),
                      (p + "FFN W2", F, d, "matrix"), (p + "FFN b2", 1, d, "bias")]
        specs += [(p + "norm1 gamma", 1, d, "gamma"), (p + "norm1 beta", 1, d, "beta"),
                  (p + "norm2 gamma", 1, d, "gamma"), (p + "norm2 beta", 1, d, "beta")]
    specs += [("final norm gamma", 1, d, "gamma"), ("final norm beta", 1, d, "beta")]
    return specs


def make_weights(cfg: Config, seed: int, std: float = 0.02, norm_noise: float = 0.0):
    """Seeded tensors in checkpoint order.  Matrices and linear biases ~ N(0, std);
    norm gamma = 1 and beta = 0 (plus N(0, norm_noise) when asked, for tests that
    need the gain/shift paths to matter).  Tensor i draws from stream i."""
    out = []
    for i, (_, rows, cols, kind) in enumerate(tensor_specs(cfg)):
        n = rows * cols
        if kind in ("matrix", "bias"):
            t = normal(n, seed, i, std)
        elif kind == "gamma":
            t = np.ones(n, dtype=np.float32)
            if norm_noise:
                t = t + normal(n, seed, i, norm_noise)
        else:
            t = np.zeros(n, dtype=np.float32)
            if norm_noise:
                t = t + normal(n, seed, i, norm_noise)
        out.append(t.reshape(rows, cols))
    return out


def write_checkpoint(path, cfg: Config, tensors, fingerprint: tuple[int, int] | None = None,
                     version: int = 2) -> None:
    """GPTM file: u32 magic, u32 version, [u32 arch], 5 x i32 dims, f32 dropout,
    then (i32 rows, i32 cols, rows*cols f32) records, then an optional trailer."""
    with open(path, "wb") as f:
        f.write(struct.pack("<II", 0x4750544D, version))
        if version == 2:
            f.write(struct.pack("<I", cfg.arch))
        f.write(struct.pack("<5if", cfg.vocab, cfg.d_model, cfg.layers, cfg.heads, cfg.max_len,
                            cfg.dropout))
        for t in tensors:
            t = np.ascontiguousarray(t, dtype="<f4")
            f.write(struct.pack("<2i", t.shape[0], t.shape[1]))
            f.write(t.tobytes())
        if fingerprint is not None:
            f.write(b"TKFP" + struct.pack("<IIQ", 12, fingerprint[0], fingerprint[1]))
