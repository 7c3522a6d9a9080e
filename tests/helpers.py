"""Shared test helpers: oracle-side quantisation of a synthetic state dict."""
import numpy as np

import oracle as orc


def quantize_state(cfg, sd):
    """Int8Linear.quantize / NF4Linear.quantize key selection (/root/reference/jsgrad/models/llama3.ts:40,55-58,101)
    applied with the oracle's quantisers; the result is what both the CPU and the GPU path load."""
    q = cfg["quantize"]
    if q not in ("int8", "nf4"):
        return dict(sd)
    out = {}
    for k, v in sd.items():
        is_lin = "feed_forward" in k or "attention.w" in k
        if q == "int8" and (is_lin or k == "tok_embeddings.weight"):
            w, s = orc.int8_quantize(v.astype(np.float32))
            out[k], out[k.replace("weight", "scale")] = w, s
        elif q == "nf4" and is_lin:
            w, s = orc.nf4_quantize(v.astype(np.float32))
            out[k], out[k.replace(".weight", ".scale")] = w, s
        elif k.startswith("output.") and q == "int8":
            continue
        else:
            out[k] = v
    if q == "int8":
        out["output.weight"], out["output.scale"] = out["tok_embeddings.weight"], out["tok_embeddings.scale"]
    return out
