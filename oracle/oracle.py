"""ctypes front end of oracle/jsgrad_oracle.c (test infrastructure, not product code).

The C file restates jsgrad's CLANG arithmetic for the Llama-3 path; this module only
marshals numpy arrays into it.  State-dict keys are the ones `get_state_dict(Transformer)`
yields in the reference (/root/reference/jsgrad/nn/state.ts:112-117 with
/root/reference/jsgrad/models/llama.ts:187-199): `tok_embeddings.weight`,
`layers.N.attention.{wq,wk,wv,wo}.weight`, `layers.N.feed_forward.{w1,w2,w3}.weight`,
`layers.N.{attention_norm,ffn_norm}.weight`, `norm.weight`, `output.weight`, and `.scale`
next to every quantised `.weight` (/root/reference/jsgrad/models/llama3.ts:45-46,107).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

W_F32, W_F16, W_I8, W_NF4 = 0, 1, 2, 3
_WHICH = {"attention.wq": 0, "attention.wk": 1, "attention.wv": 2, "attention.wo": 3,
          "feed_forward.w1": 4, "feed_forward.w2": 5, "feed_forward.w3": 6}


def build(force: bool = False) -> str:
    """Compile liboracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        vp, i32, f32, i64 = C.c_void_p, C.c_int, C.c_float, C.c_long
        sig = {
            "or_f2h_soft": ([f32], C.c_uint16), "or_h2f_soft": ([C.c_uint16], f32),
            "or_f32_to_f16": ([vp, vp, i64], None), "or_f16_to_f32": ([vp, vp, i64], None),
            "or_xexp2f_vec": ([vp, vp, i64], None), "or_xexp2h_vec": ([vp, vp, i64], None),
            "or_xsinf_vec": ([vp, vp, i64], None), "or_silu_vec": ([vp, vp, i64, i32], None),
            "or_round_vec": ([vp, vp, i64], None),
            "or_freqs_cis": ([i32, i32, f32, vp], None),
            "or_int8_quantize": ([vp, i32, i32, vp, vp], None), "or_int8_dequant": ([vp, vp, i32, i32, vp], None),
            "or_nf4_code": ([vp], None),
            "or_nf4_quantize": ([vp, i64, vp, vp], None), "or_nf4_dequant": ([vp, vp, i64, vp], None),
            "or_linear_call": ([i32, i32, i32, vp, vp, vp, i32, vp, i32], None),
            "or_linear_call_rowwise": ([i32, i32, i32, vp, vp, vp, i32, vp, i32], None),
            "or_set_threads": ([i32], None),
            "or_set_sum_order": ([i32], None),
            "or_rmsnorm": ([vp, vp, i32, f32, i32, vp], None),
            "or_rope": ([vp, i32, i32, vp, i32], None),
            "or_argmax": ([vp, i32], i32),
            "or_model_new": ([i32, i32, i32, i32, i32, i32, i32, f32, f32, i32], vp),
            "or_model_free": ([vp], None), "or_model_reset_cache": ([vp], None), "or_model_set_batched": ([vp, C.c_int], None),
            "or_model_set_linear": ([vp, i32, i32, i32, i32, i32, vp, vp], None),
            "or_model_set_norm": ([vp, i32, i32, vp], None),
            "or_model_set_embedding": ([vp, i32, vp, vp], None),
            "or_model_freqs": ([vp], vp), "or_model_cache_k": ([vp], vp), "or_model_cache_v": ([vp], vp),
            "or_embed": ([vp, i32, vp], None),
            "or_model_forward": ([vp, vp, i32, i32, vp], i32),
            "or_model_generate": ([vp, vp, i32, i32, i32, vp], i32),
        }
        for name, (args, res) in sig.items():
            fn = getattr(L, name)
            fn.argtypes, fn.restype = args, res
        _lib = L
    return _lib


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


# ---------------------------------------------------------------- scalar / vector helpers

def f32_to_f16_bits(x) -> np.ndarray:
    x = _f32(x)
    out = np.empty(x.shape, np.uint16)
    lib().or_f32_to_f16(_p(x), _p(out), x.size)
    return out


def f16_bits_to_f32(h) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().or_f16_to_f32(_p(h), _p(out), h.size)
    return out


def _vec(fn_name, x, *extra):
    x = _f32(x)
    y = np.empty_like(x)
    getattr(lib(), fn_name)(_p(x), _p(y), x.size, *extra)
    return y


def xexp2f(x): return _vec("or_xexp2f_vec", x)
def xexp2h(x): return _vec("or_xexp2h_vec", x)
def xsinf(x): return _vec("or_xsinf_vec", x)
def silu(x, act16: bool): return _vec("or_silu_vec", x, int(act16))
def round_half_even(x): return _vec("or_round_vec", x)


def freqs_cis(dim: int, end: int, theta: float) -> np.ndarray:
    """precompute_freqs_cis -> float32 [end, dim//2, 2] (cos, sin)."""
    out = np.empty((end, dim // 2, 2), np.float32)
    lib().or_freqs_cis(dim, end, theta, _p(out))
    return out


def nf4_code() -> np.ndarray:
    out = np.empty(16, np.float32)
    lib().or_nf4_code(_p(out))
    return out


def int8_quantize(w) -> tuple[np.ndarray, np.ndarray]:
    """Int8Linear.quantize for one [out,in] float matrix -> (int8 codes, fp16 scale bits as float16)."""
    w = _f32(w)
    q = np.empty(w.shape, np.int8)
    s = np.empty(w.shape[0], np.uint16)
    lib().or_int8_quantize(_p(w), w.shape[0], w.shape[1], _p(q), _p(s))
    return q, s.view(np.float16)


def int8_dequant(q, scale) -> np.ndarray:
    q = np.ascontiguousarray(q, np.int8)
    s = np.ascontiguousarray(scale, np.float16)
    out = np.empty(q.shape, np.uint16)
    lib().or_int8_dequant(_p(q), _p(s), q.shape[0], q.shape[1], _p(out))
    return out.view(np.float16)


def nf4_quantize(w) -> tuple[np.ndarray, np.ndarray]:
    """NF4Linear(64).quantize for a flat/2-D float array -> (uint8 [n/2], float16 scale [n/64, 1])."""
    w = _f32(w).reshape(-1)
    assert w.size % 64 == 0
    packed = np.empty(w.size // 2, np.uint8)
    s = np.empty(w.size // 64, np.uint16)
    lib().or_nf4_quantize(_p(w), w.size, _p(packed), _p(s))
    return packed, s.view(np.float16).reshape(-1, 1)


def nf4_dequant(packed, scale) -> np.ndarray:
    packed = np.ascontiguousarray(packed, np.uint8)
    s = np.ascontiguousarray(scale, np.float16).reshape(-1)
    out = np.empty(packed.size * 2, np.uint16)
    lib().or_nf4_dequant(_p(packed), _p(s), packed.size * 2, _p(out))
    return out.view(np.float16)


def _kind_of(w: np.ndarray, scale) -> int:
    if w.dtype == np.float32: return W_F32
    if w.dtype == np.float16: return W_F16
    if w.dtype == np.int8: return W_I8
    if w.dtype == np.uint8: return W_NF4
    raise TypeError(f"unsupported weight dtype {w.dtype}")


def set_threads(n: int) -> None:
    """Threads for loops over independent outputs (1 = single-threaded like the reference's CLANG device, the default).
    Results do not depend on it."""
    lib().or_set_threads(int(n))


def set_sum_order(mode: int) -> None:
    """0: the restatement's order of a one-row Linear's sum (one accumulator, sequential); 1: the same products in
    eight interleaved accumulators added pairwise.  A yardstick for tests (how far two float summation orders drift
    apart through a deep model), never the reference arithmetic."""
    lib().or_set_sum_order(int(mode))


def linear(w, scale, x, out_f: int, in_f: int, act16: bool, rowwise: bool = False) -> np.ndarray:
    """y = x . W^T for n rows of x (float32 values already representable in the activation dtype).
    rowwise: evaluate row by row with the one-row routine (same results; the tests compare the two)."""
    w = np.ascontiguousarray(w)
    s = None if scale is None else np.ascontiguousarray(scale, np.float16)
    x = _f32(x).reshape(-1, in_f)
    y = np.empty((x.shape[0], out_f), np.float32)
    fn = lib().or_linear_call_rowwise if rowwise else lib().or_linear_call
    fn(_kind_of(w, s), out_f, in_f, _p(w), _p(s), _p(x), x.shape[0], _p(y), int(act16))
    return y


def rmsnorm(x, w, eps: float, act16: bool) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    y = np.empty_like(x)
    lib().or_rmsnorm(_p(x), _p(w), x.size, eps, int(act16), _p(y))
    return y


def rope(x, n_heads: int, hd: int, fc_row, act16: bool) -> np.ndarray:
    """Rotate [n_heads*hd] in interleaved pairs with table row fc_row [hd/2,2] (already in the activation dtype)."""
    x = _f32(x).copy()
    fc = _f32(fc_row)
    lib().or_rope(_p(x), n_heads, hd, _p(fc), int(act16))
    return x


def argmax(x) -> int:
    x = _f32(x)
    return lib().or_argmax(_p(x), x.size)


# ---------------------------------------------------------------- model

class OracleModel:
    """Transformer (models/llama.ts:186-221) driven at temperature 0 on one sequence."""

    def __init__(self, cfg: dict, state: dict[str, np.ndarray]):
        L = lib()
        self.cfg = cfg
        self.act16 = cfg["act_dtype"] == "float16"
        self.vocab = cfg["vocab_size"]
        self._keep: list[np.ndarray] = []
        self._m = L.or_model_new(cfg["dim"], cfg["hidden_dim"], cfg["n_heads"], cfg["n_kv_heads"], cfg["n_layers"],
                                 cfg["vocab_size"], cfg["max_context"], cfg["norm_eps"], cfg["rope_theta"], int(self.act16))

        def hold(a):
            a = np.ascontiguousarray(a)
            self._keep.append(a)
            return a

        def set_linear(layer, which, prefix):
            w = hold(state[prefix + ".weight"])
            s = hold(state[prefix + ".scale"]) if prefix + ".scale" in state else None
            kind = _kind_of(w, s)
            if kind == W_NF4:
                out_f, in_f = self._shape_of(prefix)
            else:
                out_f, in_f = w.shape
            L.or_model_set_linear(self._m, layer, which, kind, out_f, in_f, _p(w), _p(s))

        for l in range(cfg["n_layers"]):
            for name, which in _WHICH.items():
                set_linear(l, which, f"layers.{l}.{name}")
            L.or_model_set_norm(self._m, l, 0, _p(hold(_f32(state[f"layers.{l}.attention_norm.weight"]))))
            L.or_model_set_norm(self._m, l, 1, _p(hold(_f32(state[f"layers.{l}.ffn_norm.weight"]))))
        L.or_model_set_norm(self._m, -1, 0, _p(hold(_f32(state["norm.weight"]))))
        emb = hold(state["tok_embeddings.weight"])
        es = hold(state["tok_embeddings.scale"]) if "tok_embeddings.scale" in state else None
        L.or_model_set_embedding(self._m, _kind_of(emb, es), _p(emb), _p(es))
        set_linear(-1, 0, "output")

    def _shape_of(self, prefix: str) -> tuple[int, int]:
        c = self.cfg
        hd = c["dim"] // c["n_heads"]
        table = {"wq": (c["n_heads"] * hd, c["dim"]), "wk": (c["n_kv_heads"] * hd, c["dim"]), "wv": (c["n_kv_heads"] * hd, c["dim"]),
                 "wo": (c["dim"], c["n_heads"] * hd), "w1": (c["hidden_dim"], c["dim"]), "w3": (c["hidden_dim"], c["dim"]),
                 "w2": (c["dim"], c["hidden_dim"]), "output": (c["vocab_size"], c["dim"])}
        return table[prefix.split(".")[-1]]

    def __del__(self):
        if getattr(self, "_m", None):
            lib().or_model_free(self._m)
            self._m = None

    def reset(self):
        lib().or_model_reset_cache(self._m)

    def set_batched(self, batched: bool) -> None:
        """Treat every forward as one sequence of a batch of several (weights expanded over rows even for S == 1)."""
        lib().or_model_set_batched(self._m, int(batched))

    def forward(self, tokens, start_pos: int, want_logits: bool = True):
        """Transformer.forward on tokens [S] at start_pos -> (greedy token, float32 logits of the last position)."""
        t = np.ascontiguousarray(tokens, np.int32).reshape(-1)
        lg = np.empty(self.vocab, np.float32) if want_logits else None
        tok = lib().or_model_forward(self._m, _p(t), t.size, start_pos, _p(lg))
        return tok, lg

    def generate(self, prompt, n_new: int, start_pos: int = 0) -> np.ndarray:
        """Token-serial prefill then greedy decode (models/llama3.ts:284-312)."""
        p = np.ascontiguousarray(prompt, np.int32).reshape(-1)
        out = np.empty(n_new, np.int32)
        lib().or_model_generate(self._m, _p(p), p.size, start_pos, n_new, _p(out))
        return out

    def embed(self, tok: int) -> np.ndarray:
        h = np.empty(self.cfg["dim"], np.float32)
        lib().or_embed(self._m, tok, _p(h))
        return h

    def _cache(self, fn):
        c = self.cfg
        hd = c["dim"] // c["n_heads"]
        shape = (c["n_layers"], c["max_context"], c["n_kv_heads"], hd)
        ptr = fn(self._m)
        n = int(np.prod(shape))
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_float)), shape=(n,)).reshape(shape)

    @property
    def cache_k(self): return self._cache(lib().or_model_cache_k)
    @property
    def cache_v(self): return self._cache(lib().or_model_cache_v)

    @property
    def freqs(self) -> np.ndarray:
        c = self.cfg
        hd = c["dim"] // c["n_heads"]
        n = 2 * c["max_context"] * hd
        return np.ctypeslib.as_array(C.cast(lib().or_model_freqs(self._m), C.POINTER(C.c_float)), shape=(n,)).reshape(2 * c["max_context"], hd // 2, 2)
