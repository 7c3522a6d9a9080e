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
            if k.startswith("_") or k in ("state", "tokens_out", "freqs_cis", "cache_kv", "forward_jit"):
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


def safe_load(fn: str) -> dict[str, np.ndarray]:
    """safetensors file -> host arrays (nn/state.ts:62-71)."""
    from safetensors.numpy import load_file
    return load_file(fn)


def safe_save(tensors: dict, fn: str) -> None:
    """nn/state.ts:79-96."""
    from safetensors.numpy import save_file
    save_file({k: (v.numpy() if isinstance(v, Tensor) else np.ascontiguousarray(v)) for k, v in tensors.items()}, fn)
