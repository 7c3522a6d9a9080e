"""State-dict plumbing: get_state_dict / load_state_dict / safe_load / safe_save
(/root/reference/jsgrad/nn/state.ts:62-96,105-179) for the model classes of this package."""
from __future__ import annotations

import numpy as np

from .tensor import Tensor


def get_state_dict(obj, prefix: str = "") -> dict[str, Tensor]:
    """Walk attributes and lists the way nn/state.ts:105-117 does; `layers.N.attention.wq.weight` style keys."""
    out: dict[str, Tensor] = {}
    if isinstance(obj, Tensor):
        return {prefix.strip("."): obj}
    if isinstance(obj, (list, tuple)):
        for i, x in enumerate(obj):
            out.update(get_state_dict(x, f"{prefix}{i}."))
        return out
    if hasattr(obj, "__dict__"):
        for k, v in vars(obj).items():
            if k.startswith("_") or k in ("state", "tokens_out", "freqs_cis", "cache_kv", "forward_jit", "alpha_counter"):
                continue
            if isinstance(v, (Tensor, list, tuple)) or (hasattr(v, "__dict__") and not callable(v)):
                out.update(get_state_dict(v, f"{prefix}{k}."))
    return out


def _slots(obj, prefix: str = ""):
    """(key, owner, attribute) for every tensor slot, including the still-empty ones."""
    if isinstance(obj, (list, tuple)):
        for i, x in enumerate(obj):
            yield from _slots(x, f"{prefix}{i}.")
        return
    for k, v in vars(obj).items():
        if k in ("weight", "scale"):
            yield f"{prefix}{k}", obj, k
        elif k.startswith("_"):
            continue
        elif isinstance(v, (list, tuple)) or (hasattr(v, "__dict__") and not isinstance(v, Tensor) and not callable(v) and not k.startswith("_") and k not in ("forward_jit",)):
            yield from _slots(v, f"{prefix}{k}.")


def load_state_dict(model, state_dict: dict, strict: bool = True, verbose: bool = False, consume: bool = False) -> None:
    """nn/state.ts:159-179: place every tensor of `state_dict` (numpy arrays or Tensors) into the model by key.
    A `.scale` slot that the dict does not mention stays empty (unquantised layer)."""
    seen = set()
    for key, owner, attr in _slots(model):
        if key not in state_dict:
            if attr == "scale":
                continue
            if strict:
                raise KeyError(f"{key} missing from the state dict")
            continue
        v = state_dict[key]
        t = v if isinstance(v, Tensor) else Tensor(np.ascontiguousarray(v), device=model.device if hasattr(model, "device") else "HIP")
        setattr(owner, attr, t)
        seen.add(key)
        if consume and not isinstance(v, Tensor):
            state_dict[key] = None
    if strict:
        unused = [k for k in state_dict if k not in seen and state_dict[k] is not None]
        if unused:
            raise KeyError(f"unused weights in state_dict: {sorted(unused)[:8]}")


_SAFE_DTYPES = {"F32": np.float32, "F16": np.float16, "I8": np.int8, "U8": np.uint8, "I32": np.int32, "I16": np.int16, "I64": np.int64, "BOOL": np.bool_, "F64": np.float64}
BF16 = np.dtype(np.uint16, metadata={"bfloat16": True})   # host stand-in: the 16-bit patterns, tagged


def is_bf16(a) -> bool:
    return isinstance(a, np.ndarray) and a.dtype == np.uint16 and bool((a.dtype.metadata or {}).get("bfloat16"))


def safe_load(fn: str) -> dict[str, np.ndarray]:
    """safetensors file -> host arrays that alias a read-only memory map of it (nn/state.ts:62-71: an 8-byte little-endian
    header length, the JSON header, then the tensor bytes at `data_offsets`).  bfloat16 tensors, which numpy cannot
    name, come back as their bit patterns with dtype `BF16` (see is_bf16); `to_device` / `fix_bf16` know what to do with them."""
    import json
    mm = np.memmap(fn, np.uint8, "r")
    n = int(mm[:8].view("<u8")[0])
    header = json.loads(bytes(mm[8:8 + n]))
    out = {}
    for k, v in header.items():
        if k == "__metadata__":
            continue
        a, b = v["data_offsets"]
        raw = mm[8 + n + a:8 + n + b]
        if v["dtype"] == "BF16":
            arr = raw.view(np.uint16).view(BF16)
        elif v["dtype"] in _SAFE_DTYPES:
            arr = raw.view(_SAFE_DTYPES[v["dtype"]])
        else:
            raise TypeError(f"{k}: safetensors dtype {v['dtype']} is not supported")
        out[k] = arr.reshape(v["shape"])
    return out


def to_device(a, device: str = "HIP") -> Tensor:
    """A host array (or Tensor) as a device Tensor; bfloat16 bit patterns keep their dtype."""
    if isinstance(a, Tensor):
        return a
    if is_bf16(a):
        return Tensor(np.ascontiguousarray(a).view(np.uint16), dtype="bfloat16", device=device)
    return Tensor(np.ascontiguousarray(a), device=device)


def safe_save(tensors: dict, fn: str) -> None:
    """nn/state.ts:79-96."""
    from safetensors.numpy import save_file
    save_file({k: (v.numpy() if isinstance(v, Tensor) else np.ascontiguousarray(v)) for k, v in tensors.items()}, fn)


# ---------------------------------------------------------------- GGUF (nn/state.ts:185-290)
GGML_QUANT = {2: (32, 18), 3: (32, 20), 8: (32, 34), 14: (256, 210)}      # type -> (elements, bytes) per block (state.ts:207)
GGML_NATIVE = {0: "float32", 1: "float16", 16: "int8", 17: "int16", 18: "int32"}   # state.ts:194


def ggml_data_to_tensor(t: np.ndarray, n: int, ggml_type: int, device: str = "HIP") -> Tensor:
    """nn/state.ts:192-223: the first n elements of GGML data `t` (uint8) as a device tensor: native types as they are,
    Q4_0 / Q4_1 / Q8_0 / Q6_K dequantised to float32 on the device (jsgrad_hip_ggml_dequant)."""
    from . import ffi
    from .ffi import check
    t = np.asarray(t, np.uint8).reshape(-1)
    if ggml_type in GGML_NATIVE:
        dt = np.dtype(DTYPES_NP[GGML_NATIVE[ggml_type]])
        return Tensor(np.ascontiguousarray(t[:dt.itemsize * n]).view(dt), device=device)
    if ggml_type not in GGML_QUANT:
        raise ValueError(f"GGML type '{ggml_type}' is not supported!")
    ne, nb = GGML_QUANT[ggml_type]
    if n % ne or t.size < n // ne * nb:
        raise ValueError(f"{n} elements of GGML type {ggml_type} need whole blocks of {ne} and {n // ne * nb} bytes, got {t.size} bytes")
    blocks = Tensor(np.ascontiguousarray(t[:(n // ne) * nb]), device=device)
    out = Tensor.empty((n // ne * ne,), "float32", device)
    check(ffi.load().jsgrad_hip_ggml_dequant(ggml_type, blocks.ptr, out.numel, out.ptr))
    return out


DTYPES_NP = {"float32": np.float32, "float16": np.float16, "int8": np.int8, "int16": np.int16, "int32": np.int32}
_GGUF_SCALARS = {0: "<u1", 1: "<i1", 2: "<u2", 3: "<i2", 4: "<u4", 5: "<i4", 6: "<f4", 7: "?", 10: "<u8", 11: "<i8", 12: "<f8"}   # state.ts:225


def gguf_load(data, device: str = "HIP") -> tuple[dict, dict[str, Tensor]]:
    """nn/state.ts:236-290: parse a GGUF file (a path, bytes, or a uint8 array; versions 2 and 3) into its key/value
    metadata and a state dict of device tensors shaped as the reversed GGUF dims."""
    buf = np.memmap(data, np.uint8, "r") if isinstance(data, str) else np.frombuffer(data, np.uint8) if isinstance(data, (bytes, bytearray, memoryview)) else np.asarray(data, np.uint8)
    pos = 0

    def read(n: int) -> np.ndarray:
        nonlocal pos
        if pos + n > buf.size:
            raise ValueError("GGUF data ends inside a field")
        out = buf[pos:pos + n]
        pos += n
        return out

    def scalar(typ: int):
        dt = np.dtype(_GGUF_SCALARS[typ])
        return np.frombuffer(bytes(read(dt.itemsize)), dt)[0].item()

    def string() -> str:
        return bytes(read(scalar(10))).decode("utf-8")

    def value(typ: int):
        if typ == 8:
            return string()
        if typ == 9:
            et, n = scalar(5), scalar(10)
            return [value(et) for _ in range(n)]
        if typ not in _GGUF_SCALARS:
            raise ValueError(f"GGUF value type {typ} is not supported")
        return scalar(typ)

    magic, version, n_tensors, n_kv = bytes(read(4)), scalar(5), scalar(11), scalar(11)
    if magic != b"GGUF" or version not in (2, 3):
        raise ValueError(f"Invalid GGUF format, magic= {magic!r}")
    kv_data = {}
    for _ in range(n_kv):
        k, typ = string(), scalar(5)
        kv_data[k] = value(typ)
    infos = []
    for _ in range(n_tensors):
        name = string()
        dims = [scalar(10) for _ in range(scalar(4))]
        infos.append((name, dims, scalar(5), scalar(10)))
    align = int(kv_data.get("general.alignment") or 32)
    data_start = (pos + align - 1) // align * align
    state_dict = {}
    for name, dims, typ, off in infos:
        n = int(np.prod(dims)) if dims else 1
        state_dict[name] = ggml_data_to_tensor(buf[data_start + off:], n, typ, device).reshape(tuple(reversed(dims)))
    return kv_data, state_dict
