"""Checkpoint formats on the way into the model, restated in numpy (test infrastructure, not product code).

What the reference does between a checkpoint file and `load_state_dict`:
  * `ggml_data_to_tensor` (/root/reference/jsgrad/nn/state.ts:192-223): GGML blocks -> float32 values for the quantised
    types Q4_0 (2), Q4_1 (3), Q8_0 (8), Q6_K (14) and the native types f32 (0), f16 (1), i8 (16), i16 (17), i32 (18);
  * `convert_from_huggingface` (/root/reference/jsgrad/models/llama.ts:224-253): the key map and the row permutation of
    q_proj / k_proj that turns the rotate-half layout into interleaved pairs;
  * `fix_bf16` (llama.ts:272-279): bfloat16 -> float32 -> float16.

`ggml_dequant` follows the reference's tensor expressions step by step (the reshape / expand / idiv / transpose / flatten
chain of `q_to_uint8`), NOT the loops of ggml itself: the tests pin it against those published loops
(ggml `dequantize_row_q4_0/q4_1/q8_0/q6_K`), which is what says the reference's reshapes address the right bits.
Arithmetic: every product is float32 in the order the reference writes it (`d.mul(q).mul(scales)`, `q.mul(d).add(m)`).
"""
from __future__ import annotations

import numpy as np

GGML_BLOCK = {2: (32, 18), 3: (32, 20), 8: (32, 34), 14: (256, 210)}   # type -> (elements, bytes) per block, state.ts:207
GGML_NATIVE = {0: np.float32, 1: np.float16, 16: np.int8, 17: np.int16, 18: np.int32}   # state.ts:194


def _q_to_uint8(t: np.ndarray, b: int) -> np.ndarray:
    """state.ts:199-203: split every byte into 8/b fields of b bits, low field first, and lay the fields of one kind
    next to each other: [..., n] -> [..., (8/b) * n] with out[..., i*n + j] = (t[..., j] >> (i*b)) & mask."""
    nf = 8 // b
    shift = (2 ** (np.arange(nf) * b)).astype(np.uint8)
    mask = 0xFF >> (8 - b)
    x = np.broadcast_to(t[..., None], t.shape + (nf,))         # unsqueeze(-1).expand
    x = (x // shift) & mask                                     # idiv(shift_tensor).bitwise_and(bitmask)
    x = np.swapaxes(x, -1, -2)                                  # transpose(-1, -2)
    return np.ascontiguousarray(x).reshape(t.shape[:-1] + (nf * t.shape[-1],)).astype(np.uint8)   # flatten(-2)


def _f16(b: np.ndarray) -> np.ndarray:
    """two bytes per row -> the float16 they hold, as float32 (bitcast(float16).cast(float32))"""
    return np.ascontiguousarray(b).view(np.float16).astype(np.float32)


def ggml_dequant(raw, n: int, ggml_type: int) -> np.ndarray:
    """state.ts:192-223.  raw: bytes / uint8 array holding at least the blocks of n elements.  Returns n values:
    float32 for the quantised types, the native dtype otherwise."""
    raw = np.frombuffer(raw, np.uint8) if isinstance(raw, (bytes, bytearray, memoryview)) else np.asarray(raw, np.uint8)
    if ggml_type in GGML_NATIVE:
        dt = np.dtype(GGML_NATIVE[ggml_type])
        return raw[: dt.itemsize * n].view(dt).copy()
    if ggml_type not in GGML_BLOCK:
        raise ValueError(f"GGML type '{ggml_type}' is not supported!")
    ne, nb = GGML_BLOCK[ggml_type]
    blocks = raw[: (n // ne) * nb].reshape(-1, nb)
    with np.errstate(over="ignore", invalid="ignore"):
        if ggml_type == 2:
            q = _q_to_uint8(blocks[:, 2:], 4).view(np.int8) - np.int8(8)
            out = q.astype(np.float32) * _f16(blocks[:, :2])
        elif ggml_type == 3:
            d, m = _f16(blocks[:, 0:2]), _f16(blocks[:, 2:4])
            out = _q_to_uint8(blocks[:, 4:], 4).view(np.int8).astype(np.float32) * d + m
        elif ggml_type == 8:
            out = _f16(blocks[:, :2]) * blocks[:, 2:].view(np.int8).astype(np.float32)
        else:
            xl = _q_to_uint8(blocks[:, :128].reshape(-1, 2, 64), 4)
            xh = (_q_to_uint8(blocks[:, 128:192].reshape(-1, 2, 32), 2) << 4).astype(np.uint8)
            scales = np.repeat(blocks[:, 192:208].view(np.int8), 16, axis=1).astype(np.float32)   # unsqueeze(-1).expand(-1,16,16).reshape(-1,256)
            d = _f16(blocks[:, -2:])
            q = ((xl | xh).view(np.int8) - np.int8(32)).reshape(-1, 256).astype(np.float32)
            out = (d * q).astype(np.float32) * scales
    return out.astype(np.float32).reshape(-1)


def hf_permute(v: np.ndarray, n_heads: int) -> np.ndarray:
    """llama.ts:225-227: v[n_heads * hd, in] -> reshape(n_heads, 2, hd/2, in).transpose(1, 2).reshape(same)."""
    out_f, in_f = v.shape
    return v.reshape(n_heads, 2, out_f // n_heads // 2, in_f).swapaxes(1, 2).reshape(out_f, in_f)


def hf_keymap(n_layers: int) -> dict[str, str]:
    """llama.ts:229-239.  Three template strings there lack the `$` of the interpolation (the bias keys and
    `model.layers.{l}.post_attention_layernorm.weight`), so as written they map the literal text `{l}` and a real
    checkpoint's ffn_norm weights end up under the key `undefined`.  This is the mapping the lines are meant to spell
    (every other entry, and the function they were translated from, use the layer number); biases do not occur in
    Llama-3 checkpoints and are left out."""
    km = {"model.embed_tokens.weight": "tok_embeddings.weight", "model.norm.weight": "norm.weight", "lm_head.weight": "output.weight"}
    for l in range(n_layers):
        km[f"model.layers.{l}.input_layernorm.weight"] = f"layers.{l}.attention_norm.weight"
        km[f"model.layers.{l}.post_attention_layernorm.weight"] = f"layers.{l}.ffn_norm.weight"
        for x in "qkvo":
            km[f"model.layers.{l}.self_attn.{x}_proj.weight"] = f"layers.{l}.attention.w{x}.weight"
        for x, y in (("gate", "1"), ("down", "2"), ("up", "3")):
            km[f"model.layers.{l}.mlp.{x}_proj.weight"] = f"layers.{l}.feed_forward.w{y}.weight"
    return km


def bf16_to_f16(bits: np.ndarray) -> np.ndarray:
    """llama.ts:275: bfloat16 -> float32 (exact) -> float16 (round to nearest even).  bits: uint16 array."""
    f32 = (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)
    with np.errstate(over="ignore"):
        return f32.astype(np.float16)
