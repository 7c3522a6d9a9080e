"""A deliberately small Tensor: a shaped, typed handle on a device Buffer.

The reference's Tensor is a lazy graph builder (/root/reference/jsgrad/tensor.ts); on this backend the
Llama path does not go through a graph, so the only things kept are the ones the model classes and
their callers touch: construction from host data, `numpy()`, `item()` (the per-token device->host
read of /root/reference/jsgrad/models/llama3.ts:336), shape/dtype, and device-side random / constant
initialisers.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import ffi
from .device import DTYPES, Buffer, Device
from .ffi import check


def _np_name(dt) -> str:
    name = np.dtype(dt).name
    if name not in DTYPES:
        raise TypeError(f"unsupported dtype {name}")
    return name


class Tensor:
    def __init__(self, data=None, dtype: str | None = None, device: str = "HIP", shape=None, buffer: Buffer | None = None):
        self.device = Device.canonicalize(device)
        if buffer is not None:
            self.lazydata, self.shape, self.dtype = buffer, tuple(shape), dtype or buffer.dtype
            return
        arr = np.asarray(data)
        if dtype == "bfloat16":
            if arr.dtype != np.uint16:
                raise TypeError("bfloat16 data is passed as its 16-bit patterns (uint16)")
            self.dtype, self.shape = "bfloat16", tuple(arr.shape)
            self.lazydata = Buffer(self.device, max(1, arr.size), "bfloat16")
            self.lazydata.allocate()
            if arr.size:
                self.lazydata.copyin(np.ascontiguousarray(arr))
            return
        if dtype is not None:
            arr = arr.astype(DTYPES[dtype][0])
        elif arr.dtype == np.float64:
            arr = arr.astype(np.float32)
        elif arr.dtype == np.int64:
            arr = arr.astype(np.int32)
        self.dtype = _np_name(arr.dtype)
        self.shape = tuple(arr.shape)
        self.lazydata = Buffer(self.device, max(1, arr.size), self.dtype)
        self.lazydata.allocate()
        if arr.size:
            self.lazydata.copyin(arr)

    # ---- constructors
    @staticmethod
    def empty(shape, dtype: str = "float32", device: str = "HIP") -> "Tensor":
        shape = tuple(int(s) for s in shape)
        buf = Buffer(Device.canonicalize(device), max(1, int(np.prod(shape))), dtype).allocate()
        return Tensor(buffer=buf, shape=shape, dtype=dtype, device=device)

    @staticmethod
    def zeros(shape, dtype: str = "float32", device: str = "HIP") -> "Tensor":
        t = Tensor.empty(shape, dtype, device)
        check(ffi.load().jsgrad_hip_memset(t.ptr, 0, t.nbytes))
        return t

    @staticmethod
    def full(shape, value: float, dtype: str = "float32", device: str = "HIP") -> "Tensor":
        t = Tensor.empty(shape, dtype, device)
        check(ffi.load().jsgrad_hip_fill(t.ptr, t.numel, DTYPES[dtype][1], float(value)))
        return t

    @staticmethod
    def ones(shape, dtype: str = "float32", device: str = "HIP") -> "Tensor":
        return Tensor.full(shape, 1.0, dtype, device)

    @staticmethod
    def randn(shape, dtype: str = "float32", seed: int = 0, std: float = 1.0, device: str = "HIP") -> "Tensor":
        t = Tensor.empty(shape, dtype, device)
        check(ffi.load().jsgrad_hip_randn(t.ptr, t.numel, DTYPES[dtype][1], seed, std))
        return t

    # ---- properties
    @property
    def ptr(self) -> int:
        return self.lazydata.ptr

    @property
    def numel(self) -> int:
        return int(np.prod(self.shape)) if self.shape else 1

    @property
    def nbytes(self) -> int:
        return self.numel * np.dtype(DTYPES[self.dtype][0]).itemsize

    @property
    def ndim(self) -> int:
        return len(self.shape)

    # ---- host access
    def numpy(self) -> np.ndarray:
        out = np.empty(self.numel, DTYPES[self.dtype][0])
        ptr = self.ptr                      # allocates a not-yet-allocated view, which also binds its allocator
        self.lazydata.allocator._copyout(out, ptr)
        return out.reshape(self.shape)

    def item(self):
        if self.numel != 1:
            raise ValueError(f"must have one element for item. shape={self.shape}")
        return self.numpy().reshape(-1)[0].item()

    def realize(self) -> "Tensor":
        return self

    def reshape(self, shape) -> "Tensor":
        shape = tuple(int(s) for s in shape)
        if -1 in shape:
            known = -int(np.prod(shape))
            shape = tuple(self.numel // known if s == -1 else s for s in shape)
        if int(np.prod(shape)) != self.numel:
            raise ValueError(f"size mismatch, can't reshape {self.shape} -> {shape}")
        return Tensor(buffer=self.lazydata, shape=shape, dtype=self.dtype, device=self.device)

    def cast(self, dtype: str) -> "Tensor":
        """Tensor.cast (tensor.ts:4141-4148) between float32 / float16, and from bfloat16 (through float32, which is what
        fix_bf16 spells out, models/llama.ts:275).  Same dtype: the tensor itself."""
        if dtype == self.dtype:
            return self
        if self.dtype not in ("float32", "float16", "bfloat16") or dtype not in ("float32", "float16"):
            raise NotImplementedError(f"cast {self.dtype} -> {dtype} is not built on this device")
        out = Tensor.empty(self.shape, dtype, self.device)
        check(ffi.load().jsgrad_hip_cast(self.ptr, DTYPES[self.dtype][1], out.ptr, DTYPES[dtype][1], self.numel))
        return out

    def __repr__(self) -> str:
        return f"<Tensor {self.shape} {self.dtype} on {self.device}>"
