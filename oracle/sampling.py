"""The sampler and its random numbers, restated in numpy (test infrastructure, not product code).

  * `sample` (/root/reference/jsgrad/models/llama.ts:131-185): alpha penalties, NaN -> -inf, softmax of logits / temp,
    then either `multinomial` over the whole vocabulary (top_k == 0) or the k largest by repeated argmax, the
    "approximate top p" mask over them, and `multinomial` over those k;
  * `Tensor.multinomial` (/root/reference/jsgrad/tensor.ts:1164-1172): cdf = cumsum(w) / cumsum(w)[-1], one uniform u,
    index = number of cdf entries that u is >= of;
  * `Tensor.rand` (tensor.ts:798-843) for one float32: Threefry-2x32-20 (ops.ts:1874-1890) of the 64-bit counter
    (counter + 1) << 32 | counter under the key seed << 32 | sha256(device number), the low word's top 23 bits as the
    mantissa of a float in [1, 2), minus 1.

Float arithmetic: float32 throughout, `a / b` as `a * (1 / b)` (tensor.ts:3576-3579), exp as the reference's polynomial
exp2 (oracle.xexp2f).  ORDER OF THE SUMS: `cumsum` is the reference's two-level scheme (tensor.ts:2629-2641): the vector
padded on the left to a multiple of 256, sequential running sums inside chunks of 256, plus the sequential running sum of
the chunk totals before the chunk.  The plain sums (softmax denominator, the mass left after top-k) are taken the same
way - sequential inside chunks of 256 (padded on the left), then sequential over the chunk sums; that order is this
build's choice, shared with the device kernels.  The order the reference's generated C takes for a sum over the whole
vocabulary was not observed, so a token decided by the last bit of a cdf entry (u within a few 1e-8 of a boundary) is
unpinned against the reference; everything else below is pinned by the tests in tests/test_sampling.py.
"""
from __future__ import annotations

import hashlib

import numpy as np

from . import oracle as orc

SPLIT = 256


# ---------------------------------------------------------------- random numbers
def threefry2x32(x0, x1, k0, k1):
    """ops.ts:1874-1890 (Threefry-2x32, 20 rounds): counter words (x0, x1), key words (k0, k1) -> two uint32 words."""
    x0, x1 = np.asarray(x0, np.uint32).copy(), np.asarray(x1, np.uint32).copy()
    k0, k1 = np.uint32(k0), np.uint32(k1)
    ks = [k1, k0 ^ k1 ^ np.uint32(0x1BD11BDA), k0]
    rot = [[13, 15, 26, 6], [17, 29, 16, 24]]
    with np.errstate(over="ignore"):
        x0, x1 = x0 + ks[2], x1 + ks[0]
        for i in range(5):
            for r in rot[i % 2]:
                x0 = x0 + x1
                x1 = x0 ^ ((x1 << np.uint32(r)) | (x1 >> np.uint32(32 - r)))
            x0, x1 = x0 + ks[i % 3], x1 + ks[(i + 1) % 3] + np.uint32(i + 1)
    return x0, x1


def device_key0(n_devices_seen: int = 0) -> int:
    """tensor.ts:814: sha256 of the 4-byte big-endian count of devices seeded so far, as a big-endian integer mod 2^32"""
    return int.from_bytes(hashlib.sha256(int(n_devices_seen).to_bytes(4, "big")).digest(), "big") % 2 ** 32


def rand_f32(seed: int, counter: int, key0: int | None = None) -> np.float32:
    """The float32 that `Tensor.rand([1, 1, 1])` returns when the device's counter stands at `counter` (the first call
    after manual_seed has 0, every later call of one number adds 1 before it draws, tensor.ts:818-819)."""
    key0 = device_key0(0) if key0 is None else key0
    c0 = np.uint32(counter & 0xFFFFFFFF)
    c1 = np.uint32((counter + 1) & 0xFFFFFFFF)            # counts1 = counts0 + ceildiv(num, 2), num = 1
    y0, _ = threefry2x32(c0, c1, key0, seed & 0xFFFFFFFF)  # bits = cat(low words, high words)[:1] = the low word
    bits = (np.uint32(y0) >> np.uint32(9)) | np.uint32(0x3F800000)
    return np.float32(np.array([bits], np.uint32).view(np.float32)[0] - np.float32(1.0))


# ---------------------------------------------------------------- sums in a fixed order
def _chunks(x: np.ndarray) -> np.ndarray:
    """x padded with zeros on the LEFT to a multiple of 256, as [chunks, 256] (tensor.ts:2637)"""
    pad = (-x.size) % SPLIT
    return np.concatenate([np.zeros(pad, np.float32), x.astype(np.float32)]).reshape(-1, SPLIT)


def seq_sum(x: np.ndarray) -> np.float32:
    """sequential inside chunks of 256, then sequential over the chunk sums"""
    if x.size == 0:
        return np.float32(0)
    c = np.cumsum(_chunks(x), axis=1, dtype=np.float32)[:, -1]
    return np.float32(np.cumsum(c, dtype=np.float32)[-1])


def cumsum(x: np.ndarray) -> np.ndarray:
    """tensor.ts:2622-2641 for a 1-D float32 vector: one level up to 512 elements, two levels beyond."""
    x = x.astype(np.float32)
    if x.size <= 2 * SPLIT:
        return np.cumsum(x, dtype=np.float32)
    within = np.cumsum(_chunks(x), axis=1, dtype=np.float32)
    totals = within[:, -1]
    base = np.concatenate([np.zeros(1, np.float32), np.cumsum(totals, dtype=np.float32)[:-1]])     # _cumalu(..., include_initial)
    return (within + base[:, None]).astype(np.float32).reshape(-1)[-x.size:]


def multinomial(w: np.ndarray, u: np.float32) -> int:
    """tensor.ts:1164-1172 for a 1-D weight vector and one uniform number."""
    cw = cumsum(w)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        cdf = cw * (np.float32(1.0) / cw[-1])
    return int(np.sum(np.float32(u) >= cdf))


# ---------------------------------------------------------------- the sampler
def exp_f32(x: np.ndarray) -> np.ndarray:
    """Tensor.exp on float32 (tensor.ts:147-154): exp2(x * 1/ln2) with the polynomial exp2"""
    return orc.xexp2f((x.astype(np.float32) * np.float32(1.4426950408889634)).astype(np.float32))


def softmax_t(logits: np.ndarray, temp: float) -> np.ndarray:
    """(logits / temp).softmax() in float32 (llama.ts:155, tensor.ts:2186-2214)"""
    y = (logits.astype(np.float32) * np.float32(1.0 / temp)).astype(np.float32)
    m = (y - np.max(y)).astype(np.float32)
    e = exp_f32(m)
    with np.errstate(divide="ignore", invalid="ignore"):
        return (e * (np.float32(1.0) / seq_sum(e))).astype(np.float32)


def sample(logits, temp: float, k: int, p: float, af: float, ap: float, u: np.float32, alpha_counter: np.ndarray | None = None) -> int:
    """llama.ts:131-185 with the uniform number handed in.  alpha_counter (int32[V]) is updated in place when af or ap is set."""
    logits = np.asarray(logits, np.float32)
    n = logits.size
    if not 0 <= p <= 1:
        raise ValueError("p must be between 0 and 1")
    if not 0 <= k <= n:
        raise ValueError("k must be between 0 and numel")
    if temp < 1e-6:
        return orc.argmax(logits)
    if af or ap:
        if alpha_counter is None:
            raise ValueError("alpha sampling needs the counter")
        pen = (alpha_counter.astype(np.float32) * np.float32(af)).astype(np.float32) + ((alpha_counter >= 0).astype(np.float32) * np.float32(ap)).astype(np.float32)
        logits = (logits - pen.astype(np.float32)).astype(np.float32)
    logits = np.where(logits != logits, np.float32(-np.inf), logits)
    t = softmax_t(logits, temp)
    if k:
        out, idx = np.zeros(k, np.float32), np.zeros(k, np.int32)
        for i in range(k):
            t_max = np.max(t)
            j = int(np.argmax(t == t_max))             # the lowest index among the maxima (llama.ts:166)
            out[i], idx[i] = t_max, j
            t = t.copy()
            t[j] = 0
        rest = seq_sum(t)
        rev = cumsum(out[::-1])[::-1]                               # output.flip().cumsum().flip()
        keep = (rev + rest).astype(np.float32) >= np.float32(1 - p)
        out, idx = keep * out, keep * idx
        i = multinomial(out.astype(np.float32), u)
        token = int(idx[i]) if i < k else 0                         # an index past the end gathers nothing (tensor.ts:1495-1519)
    else:
        token = multinomial(t, u)
    if (af or ap) and token < n:
        alpha_counter[token] += 1
    return token
