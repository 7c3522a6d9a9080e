"""Synthetic Llama-3-shaped configurations and seeded random-init weights (numpy only).

The shapes are the ones `Transformer(dim, hidden_dim, n_heads, n_layers, norm_eps, vocab_size,
linear, embedding, n_kv_heads, rope_theta, max_context)` takes in the reference
(/root/reference/jsgrad/models/llama.ts:193) and the 1B/8B rows of MODEL_PARAMS
(/root/reference/jsgrad/models/llama3.ts:119-132).  Weights are N(0, 0.02) from
`numpy.random.default_rng(seed)`; RMSNorm weights are ones as RMSNorm initialises them
(/root/reference/jsgrad/nn/index.ts:583).  Keys are the Meta-style names
`get_state_dict(Transformer)` yields.
"""
from __future__ import annotations

import numpy as np

CONFIGS: dict[str, dict] = {
    # tiny decoder the reference can run on its CPU backend
    "tiny": dict(dim=256, hidden_dim=768, n_heads=4, n_kv_heads=2, n_layers=2, vocab_size=1024, norm_eps=1e-5,
                 rope_theta=500000.0, max_context=64, act_dtype="float32", quantize=None, tied=False),
    "tiny16": dict(dim=256, hidden_dim=768, n_heads=4, n_kv_heads=2, n_layers=2, vocab_size=1024, norm_eps=1e-5,
                   rope_theta=500000.0, max_context=64, act_dtype="float16", quantize="float16", tied=False),
    "1B": dict(dim=2048, hidden_dim=8192, n_heads=32, n_kv_heads=8, n_layers=16, vocab_size=128256, norm_eps=1e-5,
               rope_theta=500000.0, max_context=1024, act_dtype="float16", quantize="float16", tied=True),
    "3B-int8": dict(dim=3072, hidden_dim=8192, n_heads=24, n_kv_heads=8, n_layers=28, vocab_size=128256, norm_eps=1e-5,
                    rope_theta=500000.0, max_context=1536, act_dtype="float16", quantize="int8", tied=True),
    "8B-nf4": dict(dim=4096, hidden_dim=14336, n_heads=32, n_kv_heads=8, n_layers=32, vocab_size=128256, norm_eps=1e-5,
                   rope_theta=500000.0, max_context=4352, act_dtype="float16", quantize="nf4", tied=False),
    "8B-int8": dict(dim=4096, hidden_dim=14336, n_heads=32, n_kv_heads=8, n_layers=32, vocab_size=128256, norm_eps=1e-5,
                    rope_theta=500000.0, max_context=2304, act_dtype="float16", quantize="int8", tied=True),
}


def config(name: str, **override) -> dict:
    cfg = dict(CONFIGS[name])
    cfg.update(override)
    cfg["name"] = name
    return cfg


def linear_shapes(cfg: dict) -> dict[str, tuple[int, int]]:
    """[out, in] of every Linear of one block plus the lm_head (models/llama.ts:56-59,103-105,196)."""
    d, H, KV, F = cfg["dim"], cfg["n_heads"], cfg["n_kv_heads"], cfg["hidden_dim"]
    hd = d // H
    return {"attention.wq": (H * hd, d), "attention.wk": (KV * hd, d), "attention.wv": (KV * hd, d), "attention.wo": (d, H * hd),
            "feed_forward.w1": (F, d), "feed_forward.w2": (d, F), "feed_forward.w3": (F, d)}


def random_state_dict(cfg: dict, seed: int = 0, std: float = 0.02) -> dict[str, np.ndarray]:
    """Unquantised weights in the model's weight dtype (float32 for act float32, float16 otherwise)."""
    rng = np.random.default_rng(seed)
    wdt = np.float32 if cfg["act_dtype"] == "float32" else np.float16
    sd: dict[str, np.ndarray] = {}

    def randn(shape):
        return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(wdt)

    sd["tok_embeddings.weight"] = randn((cfg["vocab_size"], cfg["dim"]))
    for l in range(cfg["n_layers"]):
        for name, shp in linear_shapes(cfg).items():
            sd[f"layers.{l}.{name}.weight"] = randn(shp)
        sd[f"layers.{l}.attention_norm.weight"] = np.ones(cfg["dim"], wdt)
        sd[f"layers.{l}.ffn_norm.weight"] = np.ones(cfg["dim"], wdt)
    sd["norm.weight"] = np.ones(cfg["dim"], wdt)
    sd["output.weight"] = sd["tok_embeddings.weight"] if cfg.get("tied") else randn((cfg["vocab_size"], cfg["dim"]))
    return sd


def random_prompt(cfg: dict, n: int, seed: int = 0) -> np.ndarray:
    """Uniform random token ids in [0, vocab)."""
    return np.random.default_rng(seed + 1000003).integers(0, cfg["vocab_size"], size=n, dtype=np.int32)


def weight_bytes_per_token(cfg: dict) -> int:
    """Algorithmic HBM bytes one decoded token must read besides the KV cache: every linear
    weight (+ quantisation scales) once, every norm weight, the lm_head, one embedding row."""
    d, V, L = cfg["dim"], cfg["vocab_size"], cfg["n_layers"]
    q = cfg["quantize"]
    elems = sum(o * i for o, i in linear_shapes(cfg).values())
    rows = sum(o for o, _ in linear_shapes(cfg).values())
    act = 4 if cfg["act_dtype"] == "float32" else 2
    if q == "int8":
        per_layer = elems + rows * 2
        head = V * d + V * 2
    elif q == "nf4":
        per_layer = elems // 2 + (elems // 64) * 2
        head = V * d * 2
    else:
        per_layer = elems * act
        head = V * d * act
    norms = (2 * L + 1) * d * act
    return L * per_layer + head + norms


def kv_bytes_per_position(cfg: dict) -> int:
    act = 4 if cfg["act_dtype"] == "float32" else 2
    hd = cfg["dim"] // cfg["n_heads"]
    return 2 * cfg["n_layers"] * cfg["n_kv_heads"] * hd * act
