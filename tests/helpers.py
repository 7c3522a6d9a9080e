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


def assert_close(got, ref, act16, what="", composed=False):
    """Two layers: the north-star tolerance (1e-2 of the output scale for fp16 activations, 1e-4 for float32), and the
    much tighter statement that the two paths differ only by float summation order: at most 2 ulp of the activation
    dtype (plus float summation noise at the output scale, which matters for results that cancel) and mostly identical values."""
    got, ref = np.asarray(got, np.float32), np.asarray(ref, np.float32)
    scale = max(1.0, float(np.abs(ref).max()))
    assert np.max(np.abs(got - ref)) <= (1e-2 if act16 else 1e-4) * scale, what
    if act16:
        ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float32)
        if composed:   # a fused RMSNorm in front: a few inputs differ by one fp16 ulp, which moves every output a little
            assert np.all(np.abs(got - ref) <= 4 * ulp + scale * 2.0 ** -11), what
            assert np.mean(got == ref) > 0.5, what
        else:
            assert np.all(np.abs(got - ref) <= 2 * ulp + scale * 2.0 ** -18), what    # + float-sum noise for results that cancel to ~0
            assert np.mean(got == ref) > 0.9, what
    else:
        assert np.all(np.abs(got - ref) <= scale * 2.0 ** (-15 if composed else -18)), what
