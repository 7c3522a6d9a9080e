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


def assert_close(got, ref, act16, what="", composed=False, ulp_at=None):
    """Two layers: the north-star tolerance (1e-2 of the output scale for fp16 activations, 1e-4 for float32), and the
    much tighter statement that the two paths differ only by float summation order: at most 2 ulp of the activation
    dtype (plus float summation noise at the output scale, which matters for results that cancel) and mostly identical values.
    ulp_at: magnitudes at which the ulp is taken where they exceed |ref| (a rounded intermediate that a residual cancels)."""
    got, ref = np.asarray(got, np.float32), np.asarray(ref, np.float32)
    scale = max(1.0, float(np.abs(ref).max()))
    assert np.max(np.abs(got - ref)) <= (1e-2 if act16 else 1e-4) * scale, what
    if act16:
        mag = np.abs(ref) if ulp_at is None else np.maximum(np.abs(ref), np.abs(np.asarray(ulp_at, np.float32)))
        ulp = np.spacing(mag.astype(np.float16)).astype(np.float32)
        if composed:   # a fused RMSNorm in front: a few inputs differ by one fp16 ulp, which moves every output a little
            assert np.all(np.abs(got - ref) <= 4 * ulp + scale * 2.0 ** -11), what
            assert np.mean(got == ref) > 0.5, what
        else:
            assert np.all(np.abs(got - ref) <= 2 * ulp + scale * 2.0 ** -18), what    # + float-sum noise for results that cancel to ~0
            assert np.mean(got == ref) > 0.9, what
    else:
        assert np.all(np.abs(got - ref) <= scale * 2.0 ** (-15 if composed else -18)), what


# ---------------------------------------------------------------- GGML / GGUF writers for tests
# Simple quantisers that produce VALID blocks from real values (not ggml's own rounding choices): what is under test is
# the way back, and `dequant(quant(x))` staying within a block's step of x is a check that does not share any bit
# twiddling with the code that dequantises (a wrong nibble or scale order scrambles the values).
def _f16b(x):
    return np.asarray(x, np.float16).reshape(-1, 1).view(np.uint8)


def ggml_quantize(x, ggml_type: int) -> np.ndarray:
    x = np.asarray(x, np.float32).reshape(-1)
    if ggml_type == 8:      # Q8_0: d = amax / 127, int8 codes
        b = x.reshape(-1, 32)
        d = (np.abs(b).max(1) / 127.0).astype(np.float16)
        q = np.rint(b / np.where(d == 0, 1, d).astype(np.float32)[:, None]).clip(-127, 127).astype(np.int8)
        return np.concatenate([_f16b(d), q.view(np.uint8)], 1).reshape(-1)
    if ggml_type in (2, 3):  # Q4_0: symmetric codes 0..15 around 8; Q4_1: min + step
        b = x.reshape(-1, 32)
        if ggml_type == 2:
            d = (np.abs(b).max(1) / 7.0).astype(np.float16)
            q = (np.rint(b / np.where(d == 0, 1, d).astype(np.float32)[:, None]) + 8).clip(0, 15).astype(np.uint8)
            head = _f16b(d)
        else:
            m = b.min(1).astype(np.float16)
            d = ((b.max(1) - m.astype(np.float32)) / 15.0).astype(np.float16)
            q = np.rint((b - m.astype(np.float32)[:, None]) / np.where(d == 0, 1, d).astype(np.float32)[:, None]).clip(0, 15).astype(np.uint8)
            head = np.concatenate([_f16b(d), _f16b(m)], 1)
        packed = (q[:, :16] | (q[:, 16:] << 4)).astype(np.uint8)   # element e < 16 in the low half of byte e
        return np.concatenate([head, packed], 1).reshape(-1)
    if ggml_type == 14:     # Q6_K: 16 groups of 16 with an int8 scale each, 6-bit codes around 32, one f16 super scale
        b = x.reshape(-1, 256)
        g = b.reshape(-1, 16, 16)
        gs = np.abs(g).max(2) / 31.0                                   # ideal float scale per group
        d = (gs.max(1) / 127.0).astype(np.float16)
        df = np.where(d == 0, 1, d).astype(np.float32)
        sc = np.rint(gs / df[:, None]).clip(1, 127).astype(np.int8)
        step = df[:, None] * sc.astype(np.float32)
        q = (np.rint(g / step[:, :, None]) + 32).clip(0, 63).astype(np.uint8).reshape(-1, 256)
        ql = np.zeros((b.shape[0], 128), np.uint8)
        qh = np.zeros((b.shape[0], 64), np.uint8)
        for h in range(2):      # ggml's layout (dequantize_row_q6_K), written out
            for l in range(32):
                e = [h * 128 + l, h * 128 + l + 32, h * 128 + l + 64, h * 128 + l + 96]
                ql[:, h * 64 + l] = (q[:, e[0]] & 15) | ((q[:, e[2]] & 15) << 4)
                ql[:, h * 64 + l + 32] = (q[:, e[1]] & 15) | ((q[:, e[3]] & 15) << 4)
                qh[:, h * 32 + l] = (q[:, e[0]] >> 4) | ((q[:, e[1]] >> 4) << 2) | ((q[:, e[2]] >> 4) << 4) | ((q[:, e[3]] >> 4) << 6)
        return np.concatenate([ql, qh, sc.view(np.uint8), _f16b(d)], 1).reshape(-1)
    raise ValueError(ggml_type)


def gguf_write(kv: dict, tensors: dict, alignment: int | None = None, version: int = 3) -> bytes:
    """A GGUF file image: kv values may be str, bool, int (int32 / uint64 by size), float (float32), or lists of one of
    those; `tensors` maps name -> (array, ggml_type), quantised types taken from ggml_quantize of the array."""
    import struct
    out = bytearray()
    wstr = lambda s: out.extend(struct.pack("<Q", len(s.encode())) + s.encode())

    def wval(v, with_type=True):
        if isinstance(v, str):
            if with_type: out.extend(struct.pack("<i", 8))
            wstr(v)
        elif isinstance(v, bool):
            if with_type: out.extend(struct.pack("<i", 7))
            out.extend(struct.pack("<?", v))
        elif isinstance(v, int):
            big = not (-2 ** 31 <= v < 2 ** 31)
            if with_type: out.extend(struct.pack("<i", 10 if big else 5))
            out.extend(struct.pack("<Q" if big else "<i", v))
        elif isinstance(v, float):
            if with_type: out.extend(struct.pack("<i", 6))
            out.extend(struct.pack("<f", v))
        elif isinstance(v, list):
            et = 8 if isinstance(v[0], str) else 7 if isinstance(v[0], bool) else 5 if isinstance(v[0], int) else 6
            out.extend(struct.pack("<i", 9) + struct.pack("<i", et) + struct.pack("<Q", len(v)))
            for x in v: wval(x, False)
        else:
            raise TypeError(type(v))

    kv = dict(kv)
    if alignment is not None:
        kv["general.alignment"] = alignment
    out.extend(b"GGUF" + struct.pack("<i", version) + struct.pack("<q", len(tensors)) + struct.pack("<q", len(kv)))
    for k, v in kv.items():
        wstr(k)
        wval(v)
    blobs, off = [], 0
    align = alignment or 32
    native = {0: np.float32, 1: np.float16, 16: np.int8, 17: np.int16, 18: np.int32}
    for name, (arr, typ) in tensors.items():
        arr = np.asarray(arr)
        data = arr.astype(native[typ]).tobytes() if typ in native else ggml_quantize(arr, typ).tobytes()
        wstr(name)
        out.extend(struct.pack("<I", arr.ndim))
        for dim in reversed(arr.shape):     # GGUF lists dims fastest-first
            out.extend(struct.pack("<Q", dim))
        out.extend(struct.pack("<i", typ) + struct.pack("<Q", off))
        blobs.append((off, data))
        off = (off + len(data) + align - 1) // align * align
    out.extend(b"\0" * ((len(out) + align - 1) // align * align - len(out)))
    start = len(out)
    for o, data in blobs:
        out.extend(b"\0" * (start + o - len(out)))
        out.extend(data)
    return bytes(out)
