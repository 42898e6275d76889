"""Float64 restatement of grad.cpp's FULL-SEQUENCE forward (the training/eval path),
used as the independent second oracle for the token-at-a-time decoder.

It follows a different part of the reference than the decoder does:
  GPTModel::forward            src/transformer/gpt_model.cpp:74-110
  TransformerBlock::forward    src/transformer/transformer_block.cpp:17-26
  MultiHeadAttention::forward  src/transformer/multihead_attention.cpp:414-522
      (all positions at once, additive causal mask of -1e9, softmax over rows)
  build_rope_tables/rope_apply src/transformer/multihead_attention.cpp:40-77
  LayerNorm::forward           src/transformer/layer_norm.cpp:99-135
  FeedForward::forward         src/transformer/feedforward.cpp:19-34
The reference's own test requires row i of this forward to equal the i-th
InferenceSession::step (tests/integration/sanity_tests.cpp:293-333).
"""
from __future__ import annotations

import numpy as np


def _norm(x, gamma, beta, rms, eps=1e-5):
    if rms:
        r = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
        return gamma * x * r
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    return gamma * ((x - mean) / np.sqrt(var + eps)) + beta


def rope_tables(S, head_size):
    """cos/sin(i * theta_j); the angle is formed in float32 as the reference does
    (it is part of the function's definition), the trig is exact."""
    half = head_size // 2
    j = np.arange(half, dtype=np.float32)
    theta = np.power(np.float32(10000.0), np.float32(-2.0) * j / np.float32(head_size)).astype(np.float32)
    ang = (np.arange(S, dtype=np.float32)[:, None] * theta[None, :]).astype(np.float32).astype(np.float64)
    return np.cos(ang), np.sin(ang)


def _rope(x, H, hs, cos_t, sin_t):
    S = x.shape[0]
    v = x.reshape(S, H, hs // 2, 2)
    a, b = v[..., 0], v[..., 1]
    c, s = cos_t[:, None, :], sin_t[:, None, :]
    out = np.stack([a * c - b * s, a * s + b * c], axis=-1)
    return out.reshape(S, H * hs)


def forward(cfg, tensors, tokens, return_kv=False):
    """Logits (S, vocab) in float64 for one sequence; optionally the per-layer
    (K after RoPE, V) projections the decoder's cache must hold."""
    T = [np.asarray(t, dtype=np.float64) for t in tensors]
    modern = cfg.modern
    d, H, hs = cfg.d_model, cfg.heads, cfg.head_size
    S = len(tokens)
    it = iter(T)
    E = next(it)
    x = E[np.asarray(tokens)]
    if not modern:
        P = next(it)
        x = x + P[:S]
    if modern:
        cos_t, sin_t = rope_tables(S, hs)
    mask = np.triu(np.full((S, S), -1e9), k=1)
    scale = 1.0 / np.sqrt(np.float64(hs))
    kv = []
    for _ in range(cfg.layers):
        Wq, Wk, Wv, Wo, bq, bk, bv, bo = (next(it) for _ in range(8))
        if modern:
            Wg, Wu, Wd = (next(it) for _ in range(3))
        else:
            W1, b1, W2, b2 = (next(it) for _ in range(4))
        g1, be1, g2, be2 = (next(it) for _ in range(4))

        h = _norm(x, g1, be1, modern)
        Q, K, V = h @ Wq + bq, h @ Wk + bk, h @ Wv + bv
        if modern:
            Q, K = _rope(Q, H, hs, cos_t, sin_t), _rope(K, H, hs, cos_t, sin_t)
        kv.append((K, V))
        concat = np.empty_like(Q)
        for hd in range(H):
            sl = slice(hd * hs, (hd + 1) * hs)
            sc = Q[:, sl] @ K[:, sl].T * scale + mask
            sc = np.exp(sc - sc.max(axis=-1, keepdims=True))
            sc = sc / sc.sum(axis=-1, keepdims=True)
            concat[:, sl] = sc @ V[:, sl]
        x = x + (concat @ Wo + bo)

        h = _norm(x, g2, be2, modern)
        if modern:
            g = h @ Wg
            ffn = ((g / (1.0 + np.exp(-g))) * (h @ Wu)) @ Wd
        else:
            a = h @ W1 + b1
            a = 0.5 * a * (1.0 + np.tanh(0.79788456 * (a + 0.044715 * a ** 3)))
            ffn = a @ W2 + b2
        x = x + ffn
    gf, bf = next(it), next(it)
    logits = _norm(x, gf, bf, modern) @ E.T
    return (logits, kv) if return_kv else logits
