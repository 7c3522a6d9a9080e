"""Pins the scalar / per-op functions of the CPU oracle against closed forms, brute force
and independent float64 arithmetic (the reference's own tests hold no stored vectors for
this path: every expectation in /root/reference/test is produced at run time by an
un-vendored tinygrad checkout, /root/reference/test/helpers.ts:255-336)."""
import numpy as np
import pytest

import oracle as orc

RNG = np.random.default_rng(7)
ULP32 = np.float32(2.0 ** -23)


# ------------------------------------------------------------------ fp16 conversion
def test_f16_roundtrip_all_halves():
    bits = np.arange(65536, dtype=np.uint16)
    f = orc.f16_bits_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(f[~nan], ref[~nan]) and np.all(np.isnan(f[nan]))
    back = orc.f32_to_f16_bits(f)
    assert np.array_equal(back[~nan], bits[~nan])
    soft = np.array([orc.lib().or_h2f_soft(int(b)) for b in bits[::7]], np.float32)
    assert np.array_equal(soft[~np.isnan(soft)], ref[::7][~np.isnan(ref[::7])])


def test_f32_to_f16_matches_numpy_and_soft():
    x = np.concatenate([RNG.standard_normal(20000).astype(np.float32) * s for s in (1e-8, 1e-5, 1e-3, 1.0, 300.0, 70000.0)])
    # exact ties between two halves must go to even
    h = np.arange(0x0400, 0x7bff, 37, dtype=np.uint16).view(np.float16).astype(np.float32)
    ties = (h + np.nextafter(h.astype(np.float16), np.float16(np.inf)).astype(np.float32)) / 2
    x = np.concatenate([x, ties, -ties, np.float32([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e30, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, np.inf, -np.inf])])
    hw = orc.f32_to_f16_bits(x)
    with np.errstate(over="ignore"):
        assert np.array_equal(hw, x.astype(np.float16).view(np.uint16))
    soft = np.array([orc.lib().or_f2h_soft(float(v)) for v in x[::5]], np.uint16)
    assert np.array_equal(soft, hw[::5])


# ------------------------------------------------------------------ exp2 / sin
def test_xexp2f_accuracy_and_specials():
    x = np.concatenate([RNG.uniform(-126, 127, 200000), RNG.uniform(-2, 2, 50000)]).astype(np.float32)
    y = orc.xexp2f(x)
    ref = np.exp2(x.astype(np.float64))
    assert np.max(np.abs(y - ref) / ref) < 2.5 * ULP32          # "1.0 ULP approximation" (ops.ts:1646)
    ints = np.arange(-126, 128, dtype=np.float32)
    assert np.array_equal(orc.xexp2f(ints), np.exp2(ints.astype(np.float64)).astype(np.float32))  # s == 0 -> exactly 2^q
    sp = orc.xexp2f(np.float32([np.inf, -np.inf, np.nan, 128.0, 127.99, -150.5, -149.0, 0.0]))
    assert sp[0] == np.inf and sp[1] == 0.0 and np.isnan(sp[2]) and sp[3] == np.inf and np.isfinite(sp[4]) and sp[5] == 0.0 and sp[6] > 0 and sp[7] == 1.0


def test_xexp2h_accuracy_and_bounds():
    x = RNG.uniform(-22, 23, 100000).astype(np.float16).astype(np.float32)
    x = x[(x >= -22) & (x < 23)]
    y = orc.xexp2h(x)
    ref = np.exp2(x.astype(np.float64))
    # coefficients are rounded to fp16 (2^-11 relative each); the polynomial then differs from 2^x by < 1e-3
    assert np.max(np.abs(y - ref) / ref) < 1e-3
    assert np.max(np.abs(y - ref) / ref) > 1e-5, "fp16-rounded coefficients must be visible; a float32 table would be ~1e-7"
    b = orc.xexp2h(np.float32([23.0, 22.984375, -22.0, -22.015625, 0.0, np.nan]))
    assert b[0] == np.inf and np.isfinite(b[1]) and b[2] > 0 and b[3] == 0.0 and b[4] == 1.0 and np.isnan(b[5])


def test_xsinf_small_and_large_arguments():
    x = np.concatenate([RNG.uniform(-30, 30, 200000), RNG.uniform(-1e-3, 1e-3, 1000)]).astype(np.float32)
    err = np.abs(orc.xsinf(x) - np.sin(x.astype(np.float64)))
    assert err.max() < 4e-7
    # Payne-Hanek branch (|x| >= 30), up to well past 2*max_context positions times freq 1.0
    xl = np.concatenate([RNG.uniform(30, 40000, 200000), np.arange(30, 20000, dtype=np.float64), -RNG.uniform(30, 1e6, 20000)]).astype(np.float32)
    errl = np.abs(orc.xsinf(xl) - np.sin(xl.astype(np.float64)))
    assert errl.max() < 1e-6
    sp = orc.xsinf(np.float32([0.0, np.inf, -np.inf, np.nan, np.pi / 2, -np.pi / 2]))
    assert sp[0] == 0.0 and np.all(np.isnan(sp[1:4])) and abs(sp[4] - 1) < 1e-7 and abs(sp[5] + 1) < 1e-7


def test_silu_against_float64():
    x32 = RNG.uniform(-20, 20, 50000).astype(np.float32)
    ref = x32.astype(np.float64) / (1 + np.exp(-x32.astype(np.float64)))
    assert np.max(np.abs(orc.silu(x32, False) - ref)) < 2e-6
    x16 = x32.astype(np.float16).astype(np.float32)
    ref16 = x16.astype(np.float64) / (1 + np.exp(-x16.astype(np.float64)))
    y16 = orc.silu(x16, True)
    assert np.max(np.abs(y16 - ref16) / (np.abs(ref16) + 1e-3)) < 5e-3      # fp16 constants: well inside 1e-2
    assert orc.silu(np.float32([-17.0]), True)[0] == 0.0                    # exp2 saturates to +inf above 23 -> sigmoid 0
    assert orc.silu(np.float32([16.0]), True)[0] == 16.0                    # exp2 flushes to 0 below -22 -> sigmoid 1


# ------------------------------------------------------------------ RoPE table
def test_freqs_cis_reference_test_case():
    """Same arguments as the reference's own test (test/models/llama.test.ts:8-21), its tolerance (4 decimals)."""
    t = orc.freqs_cis(4, 164, 500.0)
    pos = np.arange(164, dtype=np.float64)[:, None]
    ang = pos / 500.0 ** (np.arange(0, 4, 2) / 4.0)[None, :]
    assert t.shape == (164, 2, 2)
    assert np.max(np.abs(t[..., 0] - np.cos(ang))) < 1e-4 and np.max(np.abs(t[..., 1] - np.sin(ang))) < 1e-4


def test_freqs_cis_llama3_shapes():
    for hd in (64, 128):
        end = 2 * 4352
        t = orc.freqs_cis(hd, end, 500000.0)
        f64 = 1.0 / 500000.0 ** (np.arange(0, hd, 2, dtype=np.float64) / hd)
        # float32 rounding of freqs_i, of pos*freqs_i and (for cos) of pi/2 - angle gives an error that grows with
        # the angle: a few 2^-24 relative.  The scaled bound is ~1e-6 at small angles, which is what catches
        # quadrant / sign / index slips (those are O(1) at any angle).
        ang = np.arange(end, dtype=np.float64)[:, None] * f64[None, :]
        bound = 1e-6 + 1.5e-6 * ang   # freqs_i = 1/exp(t*ln theta) carries ~1e-6 relative error in float32
        assert np.all(np.abs(t[..., 0] - np.cos(ang)) < bound) and np.all(np.abs(t[..., 1] - np.sin(ang)) < bound)
        assert np.allclose(t[..., 0] ** 2 + t[..., 1] ** 2, 1.0, atol=1e-3)   # cos is sin(fl(pi/2 - a)): the float32 subtraction moves the angle by up to ulp(a)/2
        assert np.array_equal(t[0, :, 0], np.ones(hd // 2, np.float32)) and np.array_equal(t[0, :, 1], np.zeros(hd // 2, np.float32))


# ------------------------------------------------------------------ rounding and quantisers
def test_round_half_even():
    x = np.concatenate([RNG.uniform(-130, 130, 20000), np.arange(-128.5, 129, 1.0), np.arange(-128, 129, 0.25)]).astype(np.float32)
    assert np.array_equal(orc.round_half_even(x), np.round(x))      # numpy rounds half to even


def test_int8_dequant_closed_form_all_codes():
    codes = np.arange(-128, 128, dtype=np.int8)
    scales = np.concatenate([np.abs(RNG.standard_normal(300)) * 1e-3, [0.0, 6.1e-5, 5.96e-8, 1.0, 0.00787353515625]]).astype(np.float16)
    q = np.tile(codes, (scales.size, 1))
    got = orc.int8_dequant(q, scales)
    exact = q.astype(np.float64) * scales.astype(np.float64)[:, None]     # exact in float64
    assert np.array_equal(got.view(np.uint16), exact.astype(np.float16).view(np.uint16))


def test_int8_quantize_invariants():
    w = (RNG.standard_normal((64, 512)) * 0.02).astype(np.float16).astype(np.float32)
    w[3] = 0.0
    w[5, 7] = 0.5
    q, s = orc.int8_quantize(w)
    sf = s.astype(np.float64)
    amax = np.abs(w).max(1).astype(np.float64)
    c127 = np.float64(np.float16(1 / 127.0))
    assert np.array_equal(s.view(np.uint16), (amax * c127).astype(np.float16).view(np.uint16))   # closed form of the scale
    assert q.dtype == np.int8 and np.all(np.abs(q.astype(np.int32)) <= 127)
    nz = amax > 0
    assert np.all(np.abs(q[nz].astype(np.int32)).max(1) == 127) and np.all(q[~nz] == 0)
    # dequantisation error <= scale/2 (+ one fp16 ulp of the scaled value, which is rounded before round())
    err = np.abs(q[nz].astype(np.float64) * sf[nz, None] - w[nz])
    assert np.all(err <= sf[nz, None] * (0.5 + 0.0625))
    # codes equal round-half-even of the fp16-rounded ratio
    t = (w[nz].astype(np.float32) * (np.float32(1) / s[nz].astype(np.float32))[:, None]).astype(np.float16).astype(np.float64)
    assert np.array_equal(q[nz].astype(np.float64), np.round(t))


def test_nf4_codebook_dequant_and_layout():
    code = orc.nf4_code()
    lit = np.array([-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635, -0.18477343022823334,
                    -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
                    0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0])        # literal at models/llama3.ts:80
    assert np.array_equal(code, lit.astype(np.float16).astype(np.float32)) and np.all(np.diff(code) > 0)
    # all 256 bytes x many scales: high nibble is the even element (llama3.ts:92-94,105)
    scales = np.concatenate([np.abs(RNG.standard_normal(62)) * 0.05, [1.0, 0.0]]).astype(np.float16)
    packed = np.tile(np.arange(256, dtype=np.uint8), 8)[: 64 * 32]
    packed = packed.reshape(64, 32)
    got = orc.nf4_dequant(packed.reshape(-1), scales.reshape(-1, 1)).reshape(64, 64)
    hi, lo = packed >> 4, packed & 15
    exact = np.empty((64, 64))
    exact[:, 0::2] = code.astype(np.float64)[hi] * scales.astype(np.float64)[:, None]
    exact[:, 1::2] = code.astype(np.float64)[lo] * scales.astype(np.float64)[:, None]
    assert np.array_equal(got.view(np.uint16), exact.astype(np.float16).view(np.uint16))


def test_nf4_quantize_is_nearest_code():
    w = (RNG.standard_normal((8, 256)) * 0.02).astype(np.float16).astype(np.float32)
    packed, s = orc.nf4_quantize(w)
    assert packed.shape == (8 * 256 // 2,) and s.shape == (8 * 256 // 64, 1)
    g = w.reshape(-1, 64)
    amax = np.abs(g).max(1)
    assert np.array_equal(s.reshape(-1), amax.astype(np.float16))
    code = orc.nf4_code().astype(np.float64)
    ratio = (g * (np.float32(1) / amax)[:, None]).astype(np.float64)
    best = np.abs(ratio[..., None] - code).argmin(-1)               # first index on ties, like argmin
    nib = np.stack([packed >> 4, packed & 15], -1).reshape(-1, 64)
    assert np.array_equal(nib, best)
    # idempotent on code points: quantising a dequantised block returns the same codes
    deq = orc.nf4_dequant(packed, s).astype(np.float32)
    p2, s2 = orc.nf4_quantize(deq)
    full = np.abs(nib).max(1) >= 0   # every block holds +-1 by construction (absmax element)
    assert np.array_equal(p2.reshape(-1, 32)[full], packed.reshape(-1, 32)[full]) and np.array_equal(s2, s)


# ------------------------------------------------------------------ per-op layers
@pytest.mark.parametrize("kind", ["f32", "f16", "i8", "nf4"])
def test_linear_against_float64(kind):
    out_f, in_f = 48, 256
    w = (RNG.standard_normal((out_f, in_f)) * 0.05).astype(np.float32)
    act16 = kind != "f32"
    x = RNG.standard_normal((3, in_f)).astype(np.float32)
    scale = None
    if kind == "f32": wq, wd = w, w.astype(np.float64)
    elif kind == "f16": wq = w.astype(np.float16); wd = wq.astype(np.float64)
    elif kind == "i8": wq, scale = orc.int8_quantize(w); wd = wq.astype(np.float64) * scale.astype(np.float64)[:, None]
    else:
        wq, scale = orc.nf4_quantize(w.astype(np.float16).astype(np.float32))
        nib = np.stack([wq >> 4, wq & 15], -1).reshape(-1, 64)
        wd = (orc.nf4_code().astype(np.float64)[nib] * scale.astype(np.float64)).reshape(out_f, in_f)
    if act16: x = x.astype(np.float16).astype(np.float32)
    for rows in (x[:1], x):       # one row: fused dequant; several rows: fp16-materialised dequant
        y = orc.linear(wq, scale, rows, out_f, in_f, act16)
        ref = rows.astype(np.float64) @ wd.T
        tol = (2e-3 if act16 else 1e-5) * np.abs(ref).max() + (2e-3 if (act16 and len(rows) > 1 and kind in ("i8", "nf4")) else 0)
        assert np.max(np.abs(y - ref)) < tol
        if act16: assert np.array_equal(y, y.astype(np.float16).astype(np.float32))
    # structure: a one-hot x selects a column (catches a transposed operand); identity weight is a copy
    e = np.zeros((1, in_f), np.float32); e[0, 5] = 1.0
    col = orc.linear(wq, scale, e, out_f, in_f, act16)[0]
    assert np.allclose(col, wd[:, 5], rtol=2e-3 if act16 else 1e-6, atol=1e-7)
    eye = np.eye(64, dtype=np.float32)
    v = RNG.standard_normal(64).astype(np.float16).astype(np.float32)
    assert np.array_equal(orc.linear(eye, None, v[None], 64, 64, False)[0], v)


def test_rmsnorm_against_float64_and_rounding_points():
    d = 256
    x = RNG.standard_normal(d).astype(np.float32) * 3
    w = (1 + 0.1 * RNG.standard_normal(d)).astype(np.float32)
    ref = x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5) * w
    assert np.max(np.abs(orc.rmsnorm(x, w, 1e-5, False) - ref)) < 2e-6 * np.abs(ref).max()
    x16, w16 = x.astype(np.float16).astype(np.float32), w.astype(np.float16).astype(np.float32)
    y16 = orc.rmsnorm(x16, w16, 1e-5, True)
    ref16 = x16.astype(np.float64) / np.sqrt(np.mean(x16.astype(np.float64) ** 2) + 1e-5)
    # the normalised value is cast to fp16 BEFORE the weight multiply (nn/index.ts:588)
    two_step = (ref16.astype(np.float16).astype(np.float64) * w16).astype(np.float16).astype(np.float32)
    assert np.mean(y16 == two_step) > 0.98 and np.max(np.abs(y16 - two_step)) <= np.max(np.abs(two_step)) * 2.0 ** -10
    # eps matters: an all-zero row maps to zero, not NaN
    assert np.array_equal(orc.rmsnorm(np.zeros(d, np.float32), w, 1e-5, False), np.zeros(d, np.float32))


def test_rope_is_complex_rotation_on_interleaved_pairs():
    nh, hd, pos = 3, 64, 37
    table = orc.freqs_cis(hd, 64, 500000.0)
    x = RNG.standard_normal(nh * hd).astype(np.float32)
    y = orc.rope(x, nh, hd, table[pos], False)
    z = (x.reshape(nh, hd // 2, 2)[..., 0] + 1j * x.reshape(nh, hd // 2, 2)[..., 1]).astype(np.complex128)
    ang = pos / 500000.0 ** (np.arange(0, hd, 2) / hd)
    zr = z * np.exp(1j * ang)[None, :]
    ref = np.stack([zr.real, zr.imag], -1).reshape(-1)
    assert np.max(np.abs(y - ref)) < 1e-5
    assert np.allclose(np.linalg.norm(y.reshape(nh, hd), axis=1), np.linalg.norm(x.reshape(nh, hd), axis=1), rtol=1e-6)
    assert np.array_equal(orc.rope(x, nh, hd, table[0], False), x)        # position 0 is the identity
    # the half-split ("rotate_half") layout must NOT match: pins the interleaved reshape of models/llama.ts:25-26
    xs = x.reshape(nh, hd)
    half = np.concatenate([xs[:, : hd // 2] * np.cos(ang) - xs[:, hd // 2:] * np.sin(ang), xs[:, : hd // 2] * np.sin(ang) + xs[:, hd // 2:] * np.cos(ang)], 1).reshape(-1)
    assert np.max(np.abs(y - half)) > 0.1


def test_argmax_lowest_index_on_ties():
    assert orc.argmax([1, 5, 5, 2]) == 1
    assert orc.argmax([3, 3, 3]) == 0
    assert orc.argmax([-np.inf, -1, -1]) == 1
    x = RNG.standard_normal(128256).astype(np.float16).astype(np.float32)
    assert orc.argmax(x) == int(np.argmax(x))
    for n in (1, 2, 7):
        for perm in range(20):
            v = RNG.integers(0, 3, n).astype(np.float32)
            assert orc.argmax(v) == int(np.flatnonzero(v == v.max())[0])


# ---------------------------------------------------------------- the several-row organisation and threads change nothing
@pytest.mark.parametrize("kind", ["f32", "f16", "i8", "nf4"])
def test_linear_rows_path_is_bit_identical_to_row_by_row(kind):
    """or_linear_rows (tiles of input rows side by side, weight row converted once, outputs split over threads) must give
    exactly the sums of the one-row routine evaluated row by row."""
    rng = np.random.default_rng(11)
    out_f, in_f = 70, 192
    w = (rng.standard_normal((out_f, in_f)) * 0.05).astype(np.float32)
    for n_rows in (2, 31, 32, 33, 67):
        x = rng.standard_normal((n_rows, in_f)).astype(np.float16).astype(np.float32)
        if kind == "f32":
            args = (w, None)
        elif kind == "f16":
            args = (w.astype(np.float16), None)
        elif kind == "i8":
            args = orc.int8_quantize(w)
        else:
            args = orc.nf4_quantize(w)
        act16 = kind != "f32"
        ref = orc.linear(*args, x, out_f, in_f, act16, rowwise=True)
        for threads in (1, 3):
            orc.set_threads(threads)
            try:
                got = orc.linear(*args, x, out_f, in_f, act16)
            finally:
                orc.set_threads(1)
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (kind, n_rows, threads)


def test_model_forward_does_not_depend_on_threads():
    from denograd_amd import synthetic
    from tests.helpers import quantize_state
    cfg = dict(synthetic.config("tiny16"), quantize="int8", tied=True)
    sd = quantize_state(cfg, synthetic.random_state_dict(cfg, seed=3))
    toks = synthetic.random_prompt(cfg, 9, seed=3)
    outs = []
    for threads in (1, 4):
        orc.set_threads(threads)
        try:
            m = orc.OracleModel(cfg, sd)
            t1, lg1 = m.forward(toks[:6], 0)           # several rows
            t2, lg2 = m.forward([int(toks[6])], 6)     # one row on top of the cache
            outs.append((t1, lg1.copy(), t2, lg2.copy()))
        finally:
            orc.set_threads(1)
    assert outs[0][0] == outs[1][0] and outs[0][2] == outs[1][2]
    assert np.array_equal(outs[0][1].view(np.uint32), outs[1][1].view(np.uint32))
    assert np.array_equal(outs[0][3].view(np.uint32), outs[1][3].view(np.uint32))
