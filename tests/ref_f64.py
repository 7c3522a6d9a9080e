"""Independent float64 textbook implementation of a Llama decoder (numpy only).

Written from the standard formulas (RMSNorm, rotary embedding as complex multiplication on
interleaved pairs, grouped-query softmax attention, SwiGLU), NOT from the oracle's C file, so
that a dropped term, a wrong index or a transposed operand in the oracle shows up as a
difference far above rounding noise.
"""
import numpy as np


def dequant(state, prefix, shape):
    w = state[prefix + ".weight"]
    if w.dtype == np.int8:
        return w.astype(np.float64) * state[prefix + ".scale"].astype(np.float64)[:, None]
    if w.dtype == np.uint8:
        code = np.array([-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635, -0.18477343022823334,
                         -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
                         0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0]).astype(np.float16).astype(np.float64)
        nib = np.stack([w >> 4, w & 15], -1).reshape(-1)
        return (code[nib].reshape(-1, 64) * state[prefix + ".scale"].astype(np.float64).reshape(-1, 1)).reshape(shape)
    return w.astype(np.float64)


def rmsnorm(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def rope(x, pos, theta):
    """x [S, n_heads, hd]; rotate pairs (2i, 2i+1) by angle pos * theta^(-2i/hd)."""
    S, nh, hd = x.shape
    freqs = 1.0 / theta ** (np.arange(0, hd, 2, dtype=np.float64) / hd)
    ang = pos[:, None] * freqs[None, :]
    z = (x[..., 0::2] + 1j * x[..., 1::2]) * np.exp(1j * ang)[:, None, :]
    out = np.empty_like(x)
    out[..., 0::2], out[..., 1::2] = z.real, z.imag
    return out


def forward_full(cfg, state, tokens):
    """Causal forward over the whole token sequence from position 0; returns logits [S, vocab]."""
    d, H, KV, L = cfg["dim"], cfg["n_heads"], cfg["n_kv_heads"], cfg["n_layers"]
    hd, F, V = d // H, cfg["hidden_dim"], cfg["vocab_size"]
    S = len(tokens)
    emb = dequant(state, "tok_embeddings", (V, d))
    h = emb[np.asarray(tokens)]
    pos = np.arange(S, dtype=np.float64)
    mask = np.triu(np.full((S, S), -np.inf), 1)
    for l in range(L):
        p = f"layers.{l}."
        xn = rmsnorm(h, state[p + "attention_norm.weight"].astype(np.float64), cfg["norm_eps"])
        q = (xn @ dequant(state, p + "attention.wq", (H * hd, d)).T).reshape(S, H, hd)
        k = (xn @ dequant(state, p + "attention.wk", (KV * hd, d)).T).reshape(S, KV, hd)
        v = (xn @ dequant(state, p + "attention.wv", (KV * hd, d)).T).reshape(S, KV, hd)
        q, k = rope(q, pos, cfg["rope_theta"]), rope(k, pos, cfg["rope_theta"])
        out = np.empty((S, H, hd))
        for hh in range(H):
            g = hh // (H // KV)
            sc = q[:, hh, :] @ k[:, g, :].T / np.sqrt(hd) + mask
            sc = np.exp(sc - sc.max(-1, keepdims=True))
            out[:, hh, :] = (sc / sc.sum(-1, keepdims=True)) @ v[:, g, :]
        h = h + out.reshape(S, H * hd) @ dequant(state, p + "attention.wo", (d, H * hd)).T
        xn = rmsnorm(h, state[p + "ffn_norm.weight"].astype(np.float64), cfg["norm_eps"])
        a = xn @ dequant(state, p + "feed_forward.w1", (F, d)).T
        u = xn @ dequant(state, p + "feed_forward.w3", (F, d)).T
        h = h + (a / (1.0 + np.exp(-a)) * u) @ dequant(state, p + "feed_forward.w2", (d, F)).T
    return rmsnorm(h, state["norm.weight"].astype(np.float64), cfg["norm_eps"]) @ dequant(state, "output", (V, d)).T
