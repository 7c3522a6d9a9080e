"""Layers of the Llama path: Linear, RMSNorm, Embedding (/root/reference/jsgrad/nn/index.ts:403-412,580-620).

Each `call` queues one kernel of libjsgrad_hip.so on a single activation row.  The fused entry points the
Transformer uses (norm + projection + epilogue in one launch) live in llama.py; the classes here are the
unfused building blocks with the reference's names and argument order.
"""
from __future__ import annotations

from . import ffi
from .device import DTYPES
from .ffi import check
from .tensor import Tensor

_KIND = {"float32": ffi.W_F32, "float16": ffi.W_F16, "int8": ffi.W_I8, "uint8": ffi.W_NF4}


def act_code(dtype: str) -> int:
    code = DTYPES[dtype][1]
    if code is None:
        raise TypeError(f"{dtype} is not an activation dtype")
    return code


class Linear:
    """y = x . W^T (bias-free on the Llama path; the reference's Llama never constructs a bias)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False):
        if bias:
            raise NotImplementedError("bias is not used by the Llama path")
        self.in_features, self.out_features = in_features, out_features
        self.weight: Tensor | None = None   # [out_features, in_features], float32 or float16
        self.scale: Tensor | None = None

    @property
    def kind(self) -> int:
        return _KIND[self.weight.dtype]

    def call(self, x: Tensor, out: Tensor | None = None, residual: Tensor | None = None, norm: "RMSNorm | None" = None) -> Tensor:
        out = out if out is not None else Tensor.empty((self.out_features,), x.dtype, x.device)
        check(ffi.load().jsgrad_hip_linear(self.kind, self.weight.ptr, self.scale.ptr if self.scale is not None else None, self.out_features, self.in_features,
                                           x.ptr, out.ptr, norm.weight.ptr if norm is not None else None, norm.eps if norm is not None else 0.0,
                                           residual.ptr if residual is not None else None, act_code(x.dtype)))
        return out


class RMSNorm:
    def __init__(self, dim: int, eps: float = 1e-6):
        self.dim, self.eps = dim, eps
        self.weight: Tensor | None = None

    def call(self, x: Tensor, out: Tensor | None = None) -> Tensor:
        out = out if out is not None else Tensor.empty((self.dim,), x.dtype, x.device)
        check(ffi.load().jsgrad_hip_rmsnorm(x.ptr, self.weight.ptr, out.ptr, self.dim, self.eps, act_code(x.dtype)))
        return out


class Embedding:
    """Row gather of the token held in the device `state` word (see Transformer)."""

    def __init__(self, vocab_size: int, embed_size: int):
        self.vocab_size, self.embed_size = vocab_size, embed_size
        self.weight: Tensor | None = None
        self.scale: Tensor | None = None

    @property
    def out_dtype(self) -> str:
        return "float32" if self.weight.dtype == "float32" else "float16"

    def call(self, state: Tensor, out: Tensor | None = None) -> Tensor:
        out = out if out is not None else Tensor.empty((self.embed_size,), self.out_dtype, state.device)
        check(ffi.load().jsgrad_hip_embed(_KIND[self.weight.dtype], self.weight.ptr, self.scale.ptr if self.scale is not None else None, state.ptr, out.ptr,
                                          self.embed_size, self.vocab_size, act_code(out.dtype)))
        return out
