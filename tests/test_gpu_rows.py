"""Per-kernel parity of the several-row kernels (batched prefill / batched decode) through the C ABI.

Linear layers on the matrix cores are checked against the oracle's several-row Linear (quantised weights realised in
fp16 first, float accumulation): same products, different float summation order, so results agree to an fp16 ulp or two
and mostly bit for bit.  Causal attention is checked against a float64 restatement of the textbook formula (the kernel
rescales running sums where the reference normalises once, so the bar there is the north-star tolerance of 1e-2).
Gathers, norms and argmax are bit-exact."""
import numpy as np
import pytest

import oracle as orc
from denograd_amd import ffi
from denograd_amd.ffi import check
from denograd_amd.tensor import Tensor
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(23)
KINDS = {"float16": ffi.W_F16, "int8": ffi.W_I8, "nf4": ffi.W_NF4}


def make_weight(kind, out_f, in_f, std=0.05):
    w = (RNG.standard_normal((out_f, in_f)) * std).astype(np.float32)
    if kind == "float16":
        return w.astype(np.float16), None
    if kind == "int8":
        return orc.int8_quantize(w)
    return orc.nf4_quantize(w)


def dev(w, s):
    return Tensor(w), (Tensor(s) if s is not None else None)


def sp(t):
    return t.ptr if t is not None else None


@pytest.mark.parametrize("kind", ["float16", "int8", "nf4"])
@pytest.mark.parametrize("rows,out_f,in_f", [(2, 128, 64), (16, 256, 512), (33, 384, 256), (64, 128, 1024), (65, 256, 128), (300, 384, 192), (512, 512, 512),
                                             # at most 32 rows and K in whole chunks: the weight-streaming kernel (2, 3, 4 and 5 chunks; 16- and 32-row blocks)
                                             (2, 128, 2048), (5, 256, 2048), (16, 256, 3072), (17, 128, 4096), (32, 384, 5120), (16, 128, 1536), (31, 128, 1024)])
def test_gemm_matches_several_row_linear(hip, kind, rows, out_f, in_f):
    w, s = make_weight(kind, out_f, in_f)
    x = RNG.standard_normal((rows, in_f)).astype(np.float16)
    res = RNG.standard_normal((rows, out_f)).astype(np.float16)
    tw, ts = dev(w, s)
    tx, tr, ty = Tensor(x), Tensor(res), Tensor.empty((rows, out_f), "float16")
    check(hip.jsgrad_hip_gemm(KINDS[kind], tw.ptr, sp(ts), out_f, in_f, tx.ptr, rows, ty.ptr, None))
    ref = orc.linear(w, s, x, out_f, in_f, True)
    assert_close(ty.numpy().astype(np.float32), ref, True, f"gemm {kind} {rows}x{out_f}x{in_f}")
    check(hip.jsgrad_hip_gemm(KINDS[kind], tw.ptr, sp(ts), out_f, in_f, tx.ptr, rows, ty.ptr, tr.ptr))
    ref_r = (res.astype(np.float32) + ref).astype(np.float16).astype(np.float32)
    # a one-ulp difference in the product, then a sum that may cancel: compare at the scale of the operands
    assert_close(ty.numpy().astype(np.float32), ref_r, True, f"gemm+residual {kind} {rows}x{out_f}x{in_f}", composed=True)


def test_gemm_special_inputs(hip):
    """Identity weight returns the input; one-hot rows pick weight columns exactly (no summation involved)."""
    n = 256
    w = np.eye(n, dtype=np.float16)
    x = RNG.standard_normal((40, n)).astype(np.float16)
    tw, tx, ty = Tensor(w), Tensor(x), Tensor.empty((40, n), "float16")
    check(hip.jsgrad_hip_gemm(ffi.W_F16, tw.ptr, None, n, n, tx.ptr, 40, ty.ptr, None))
    assert np.array_equal(ty.numpy().view(np.uint16), x.view(np.uint16))
    w2 = RNG.standard_normal((n, n)).astype(np.float16)
    onehot = np.zeros((n, n), np.float16)
    onehot[np.arange(n), RNG.permutation(n)] = 1
    tw2, to = Tensor(w2), Tensor(onehot)
    ty2 = Tensor.empty((n, n), "float16")
    check(hip.jsgrad_hip_gemm(ffi.W_F16, tw2.ptr, None, n, n, to.ptr, n, ty2.ptr, None))
    assert np.array_equal(ty2.numpy().view(np.uint16), (onehot.astype(np.float32) @ w2.astype(np.float32).T).astype(np.float16).view(np.uint16))


def test_gemm_dequantised_tile_is_the_realised_weight(hip):
    """x = one-hot rows: the output is the dequantised weight itself, which must be bit-exact RN16(code * scale)."""
    out_f, in_f = 128, 128
    for kind in ("int8", "nf4"):
        w, s = make_weight(kind, out_f, in_f, std=0.3)
        tw, ts = dev(w, s)
        eye = np.eye(in_f, dtype=np.float16)
        tx, ty = Tensor(eye), Tensor.empty((in_f, out_f), "float16")
        check(hip.jsgrad_hip_gemm(KINDS[kind], tw.ptr, sp(ts), out_f, in_f, tx.ptr, in_f, ty.ptr, None))
        deq = orc.int8_dequant(w, s) if kind == "int8" else orc.nf4_dequant(w, s).reshape(out_f, in_f)
        assert np.array_equal(ty.numpy().view(np.uint16), np.ascontiguousarray(deq.T).view(np.uint16)), kind


def test_gemm_rejects_bad_shapes(hip):
    t = Tensor.zeros((128 * 128,), "float16")
    with pytest.raises(ffi.HipError, match="multiple of 128"):
        check(hip.jsgrad_hip_gemm(ffi.W_F16, t.ptr, None, 96, 64, t.ptr, 4, t.ptr, None))
    with pytest.raises(ffi.HipError, match="multiple of 64"):
        check(hip.jsgrad_hip_gemm(ffi.W_F16, t.ptr, None, 128, 96, t.ptr, 4, t.ptr, None))
    with pytest.raises(ffi.HipError, match="not built for several rows"):
        check(hip.jsgrad_hip_gemm(ffi.W_F32, t.ptr, None, 128, 64, t.ptr, 4, t.ptr, None))
    with pytest.raises(ffi.HipError, match="scales"):
        check(hip.jsgrad_hip_gemm(ffi.W_I8, t.ptr, None, 128, 64, t.ptr, 4, t.ptr, None))
    with pytest.raises(ffi.HipError, match="16-byte aligned"):
        check(hip.jsgrad_hip_gemm(ffi.W_F16, t.ptr, None, 128, 64, t.ptr + 2, 4, t.ptr, None))
    with pytest.raises(ffi.HipError, match="16-byte aligned"):
        check(hip.jsgrad_hip_gemm(ffi.W_F16, t.ptr, None, 128, 64, t.ptr, 4, t.ptr, t.ptr + 8))


def test_few_rows_streaming_kernel_equals_tiled_kernel(hip, monkeypatch):
    """The several-row kernels compute the same products; their float sums differ in order only.  The weight-streaming
    kernel with one and with two tiles of 16 weight rows per block against the tiled kernel."""
    out_f, in_f = 256, 4096
    monkeypatch.setenv("JSG_GEMM_NO_STREAM", "1")      # int8 with at most 16 rows would go to the LDS-streamed kernel
    for kind in ("float16", "int8", "nf4"):
        for rows in (16, 29):
            w, s = make_weight(kind, out_f, in_f)
            x = RNG.standard_normal((rows, in_f)).astype(np.float16)
            tw, ts = dev(w, s)
            tx = Tensor(x)
            got = {}
            for shape in ("1", "2", "tiled"):
                monkeypatch.setenv("JSG_GEMM_NO_SKINNY", "1") if shape == "tiled" else monkeypatch.setenv("JSG_GEMM_SKINNY_TILES", shape)
                y = Tensor.empty((rows, out_f), "float16")
                check(hip.jsgrad_hip_gemm(KINDS[kind], tw.ptr, sp(ts), out_f, in_f, tx.ptr, rows, y.ptr, None))
                got[shape] = y.numpy().astype(np.float32)
                monkeypatch.delenv("JSG_GEMM_NO_SKINNY", raising=False)
                monkeypatch.delenv("JSG_GEMM_SKINNY_TILES", raising=False)
            ref = orc.linear(w, s, x, out_f, in_f, True)
            for shape, y in got.items():
                assert_close(y, ref, True, f"{shape} {kind} {rows} rows")
            assert np.array_equal(got["1"], got["2"])     # same order of summation
            assert (got["1"] == got["tiled"]).mean() > 0.97


@pytest.mark.parametrize("kind", ["float16", "int8", "nf4"])
def test_tile_shapes_of_the_tiled_kernel_agree_bit_for_bit(hip, monkeypatch, kind):
    """Every block shape of the tiled kernel (256x256 out of two LDS buffers, 256x256 and 256x128 out of one, 128x128)
    walks K in the same order, so the outputs are identical; 1, 3 and 4 K tiles, a ragged last row tile, with a residual."""
    for rows, out_f, in_f in ((300, 512, 192), (257, 256, 256), (130, 256, 64)):
        w, s = make_weight(kind, out_f, in_f)
        x = RNG.standard_normal((rows, in_f)).astype(np.float16)
        res = RNG.standard_normal((rows, out_f)).astype(np.float16)
        tw, ts = dev(w, s)
        tx, tr = Tensor(x), Tensor(res)
        got = {}
        for shape in ("db", "wide", "tall", "small"):
            monkeypatch.setenv("JSG_GEMM_TILE", shape)
            y = Tensor.empty((rows, out_f), "float16")
            check(hip.jsgrad_hip_gemm(KINDS[kind], tw.ptr, sp(ts), out_f, in_f, tx.ptr, rows, y.ptr, tr.ptr))
            got[shape] = y.numpy().view(np.uint16)
        monkeypatch.delenv("JSG_GEMM_TILE")
        ref = (res.astype(np.float32) + orc.linear(w, s, x, out_f, in_f, True)).astype(np.float16).astype(np.float32)
        assert_close(got["db"].view(np.float16).astype(np.float32), ref, True, f"{kind} {rows}x{out_f}x{in_f}", composed=True)
        for shape in ("wide", "tall", "small"):
            assert np.array_equal(got["db"], got[shape]), f"{kind} {shape} {rows}x{out_f}x{in_f}"


@pytest.mark.parametrize("shape", ["db", "wide", "tall", "small"])
def test_tile_shapes_fused_epilogues(hip, monkeypatch, shape):
    """SwiGLU and rotary / cache epilogues of the tiled kernel under every block shape."""
    monkeypatch.setenv("JSG_GEMM_TILE", shape)
    test_gemm_ffn_gate(hip, "int8", 130, 256, 384)
    test_gemm_ffn_gate(hip, "nf4", 70, 128, 256)
    test_gemm_qkv_rope_writes_queries_and_cache(hip, "float16", 64, 3, 40, 256)
    test_gemm_qkv_rope_writes_queries_and_cache(hip, "int8", 128, 2, 50, 192)


@pytest.mark.parametrize("tpw", ["1", "2"])
@pytest.mark.parametrize("rows", [16, 5])
def test_lds_streamed_kernel_against_oracle_and_the_tiled_kernel(hip, monkeypatch, tpw, rows):
    """int8 weights, at most 16 rows: whole stretches of weight rows through LDS, K split over blocks for narrow outputs.
    Every admissible number of K parts gives a valid result; a given number gives the same bits on every run (the parts
    are added in K order by whoever arrives last)."""
    monkeypatch.setenv("JSG_SG_TPW", tpw)
    for out_f, in_f in ((256, 4096), (1024, 1536), (128, 14336)):
        w, s = make_weight("int8", out_f, in_f)
        x = RNG.standard_normal((rows, in_f)).astype(np.float16)
        res = RNG.standard_normal((rows, out_f)).astype(np.float16)
        tw, ts = dev(w, s)
        tx, tr = Tensor(x), Tensor(res)
        lin = orc.linear(w, s, x, out_f, in_f, True)
        ref = (res.astype(np.float32) + lin).astype(np.float16).astype(np.float32)
        monkeypatch.setenv("JSG_GEMM_NO_SKINNY", "1")
        monkeypatch.setenv("JSG_GEMM_NO_STREAM", "1")
        y = Tensor.empty((rows, out_f), "float16")
        check(hip.jsgrad_hip_gemm(ffi.W_I8, tw.ptr, sp(ts), out_f, in_f, tx.ptr, rows, y.ptr, tr.ptr))
        tiled = y.numpy().astype(np.float32)
        monkeypatch.delenv("JSG_GEMM_NO_SKINNY")
        monkeypatch.delenv("JSG_GEMM_NO_STREAM")
        nchunks = in_f // 512
        for parts in ["", "1", "2", "3", "4", "7", "8"]:
            if parts and (nchunks % int(parts) or (nchunks // int(parts)) * int(tpw) < 2):
                continue
            monkeypatch.setenv("JSG_SG_SPLITK", parts) if parts else monkeypatch.delenv("JSG_SG_SPLITK", raising=False)
            runs = []
            for _ in range(2):
                y = Tensor.full((rows, out_f), 7.0, "float16")
                check(hip.jsgrad_hip_gemm(ffi.W_I8, tw.ptr, sp(ts), out_f, in_f, tx.ptr, rows, y.ptr, tr.ptr))
                runs.append(y.numpy())
            assert np.array_equal(runs[0].view(np.uint16), runs[1].view(np.uint16)), (out_f, in_f, parts)
            got = runs[0].astype(np.float32)
            assert_close(got, ref, True, f"{out_f}x{in_f} parts={parts or 'auto'}", ulp_at=lin)
            assert (got == tiled).mean() > 0.97, (out_f, in_f, parts)
        monkeypatch.delenv("JSG_SG_SPLITK", raising=False)


@pytest.mark.parametrize("tpw", ["1", "2"])
def test_lds_streamed_kernel_fused_epilogues(hip, monkeypatch, tpw):
    """SwiGLU and rotary / cache epilogues of the LDS-streamed kernel, with and without K parts."""
    monkeypatch.setenv("JSG_SG_TPW", tpw)
    for parts in ("", "2"):
        monkeypatch.setenv("JSG_SG_SPLITK", parts) if parts else monkeypatch.delenv("JSG_SG_SPLITK", raising=False)
        test_gemm_ffn_gate(hip, "int8", 16, 2048, 256)
        test_gemm_ffn_gate(hip, "int8", 3, 1024, 384)
        test_gemm_qkv_rope_writes_queries_and_cache(hip, "int8", 128, 16, 1, 2048)
        test_gemm_qkv_rope_writes_queries_and_cache(hip, "int8", 128, 3, 2, 1024)


@pytest.mark.parametrize("tiles", ["1", "2"])
def test_few_rows_fused_epilogues_with_one_and_two_tiles_per_block(hip, monkeypatch, tiles):
    """SwiGLU and rotary / cache epilogues of the weight-streaming kernel, tiles per block pinned."""
    monkeypatch.setenv("JSG_GEMM_SKINNY_TILES", tiles)
    monkeypatch.setenv("JSG_GEMM_NO_STREAM", "1")
    test_gemm_ffn_gate(hip, "int8", 16, 2048, 256)
    test_gemm_ffn_gate(hip, "float16", 20, 1024, 128)
    test_gemm_qkv_rope_writes_queries_and_cache(hip, "int8", 128, 16, 1, 2048)
    test_gemm_qkv_rope_writes_queries_and_cache(hip, "float16", 64, 3, 9, 2048)
    test_gemm_ffn_gate(hip, "nf4", 16, 2048, 256)
    test_gemm_ffn_gate(hip, "nf4", 20, 1024, 128)
    test_gemm_qkv_rope_writes_queries_and_cache(hip, "nf4", 64, 16, 1, 2048)


@pytest.mark.parametrize("kind", ["float16", "int8", "nf4"])
@pytest.mark.parametrize("rows,dim,hidden", [(3, 256, 384), (16, 256, 384), (130, 256, 384), (16, 2048, 256), (20, 3072, 128)])
def test_gemm_ffn_gate(hip, kind, rows, dim, hidden):
    w1, s1 = make_weight(kind, hidden, dim)
    w3, s3 = make_weight(kind, hidden, dim)
    x = RNG.standard_normal((rows, dim)).astype(np.float16)
    t1, ts1 = dev(w1, s1)
    t3, ts3 = dev(w3, s3)
    tx, tg = Tensor(x), Tensor.empty((rows, hidden), "float16")
    check(hip.jsgrad_hip_gemm_ffn_gate(KINDS[kind], t1.ptr, sp(ts1), t3.ptr, sp(ts3), tx.ptr, rows, tg.ptr, dim, hidden))
    a = orc.linear(w1, s1, x, hidden, dim, True)
    u = orc.linear(w3, s3, x, hidden, dim, True)
    ref = (orc.silu(a.reshape(-1), True).reshape(a.shape) * u).astype(np.float16).astype(np.float32)
    assert_close(tg.numpy().astype(np.float32), ref, True, f"ffn_gate {kind} {rows}", composed=True)


def test_swiglu_epilogue_silu_bit_exact_for_every_fp16_input(hip):
    """One-hot input rows pick single weights, so the gate GEMM output is each fp16 value itself (no summation) and the
    epilogue's silu(g) * 1 can be compared with the oracle's on every finite fp16 bit pattern (weight rows that hold an infinity
    or a NaN are left out: 0 * inf in the other rows' sums makes the whole row NaN)."""
    hidden, dim = 1024, 64
    w1 = np.arange(65536, dtype=np.uint16).view(np.float16).reshape(hidden, dim)
    w3 = np.ones((hidden, dim), np.float16)
    x = np.eye(dim, dtype=np.float16)
    t1, t3, tx, tg = Tensor(w1), Tensor(w3), Tensor(x), Tensor.empty((dim, hidden), "float16")
    check(hip.jsgrad_hip_gemm_ffn_gate(ffi.W_F16, t1.ptr, None, t3.ptr, None, tx.ptr, dim, tg.ptr, dim, hidden))
    got = tg.numpy().T.reshape(-1)                                   # got[n * dim + r] = silu(w1[n][r])
    vals = w1.reshape(-1).astype(np.float32)
    with np.errstate(all="ignore"):
        ref = orc.silu(vals, True).astype(np.float16)
    finite_in = np.isfinite(vals)
    nan_rows = ~np.isfinite(w1.astype(np.float32)).reshape(hidden, dim)
    clean = np.repeat(~nan_rows.any(axis=1), dim)
    sel = finite_in & clean
    sel[0x8000] = False      # -0.0 leaves the GEMM as +0.0 (a sum that starts from +0.0), so silu sees another input
    assert sel.sum() > 60000
    assert np.array_equal(got[sel].view(np.uint16), ref[sel].view(np.uint16))


@pytest.mark.parametrize("B,S,dim", [(2, 37, 256), (16, 1, 2048), (3, 9, 2048)])   # prefill rows; batched decode and few rows on the streaming kernel
@pytest.mark.parametrize("kind,hd", [("float16", 64), ("int8", 128), ("nf4", 64)])
def test_gemm_qkv_rope_writes_queries_and_cache(hip, kind, hd, B, S, dim):
    start, ctx = 5, 64
    H, KV = (4, 2) if hd == 64 else (2, 1)
    wq, sq = make_weight(kind, H * hd, dim)
    wk, sk = make_weight(kind, KV * hd, dim)
    wv, sv = make_weight(kind, KV * hd, dim)
    x = RNG.standard_normal((B * S, dim)).astype(np.float16)
    table = Tensor.empty((2 * ctx, hd // 2, 2), "float16")
    check(hip.jsgrad_hip_rope_table(table.ptr, hd, 2 * ctx, 500000.0, ffi.F16))
    fc = table.numpy().astype(np.float32)
    tq, tsq = dev(wq, sq); tk, tsk = dev(wk, sk); tv, tsv = dev(wv, sv)
    tx = Tensor(x)
    q_out = Tensor.empty((B * S, H * hd), "float16")
    ck, cv = Tensor.zeros((B, ctx, KV, hd), "float16"), Tensor.zeros((B, ctx, KV, hd), "float16")
    check(hip.jsgrad_hip_gemm_qkv_rope(KINDS[kind], tq.ptr, sp(tsq), tk.ptr, sp(tsk), tv.ptr, sp(tsv), tx.ptr, B * S, S, start, table.ptr,
                                       q_out.ptr, ck.ptr, cv.ptr, dim, H, KV, hd, ctx))
    q = orc.linear(wq, sq, x, H * hd, dim, True)
    k = orc.linear(wk, sk, x, KV * hd, dim, True)
    v = orc.linear(wv, sv, x, KV * hd, dim, True)
    q_ref, ck_ref, cv_ref = np.zeros_like(q), np.zeros((B, ctx, KV * hd), np.float32), np.zeros((B, ctx, KV * hd), np.float32)
    for m in range(B * S):
        b, pos = m // S, start + m % S
        q_ref[m] = orc.rope(q[m], H, hd, fc[pos], True)
        ck_ref[b, pos] = orc.rope(k[m], KV, hd, fc[pos], True)
        cv_ref[b, pos] = v[m]
    assert_close(q_out.numpy().astype(np.float32), q_ref, True, "q", composed=True)
    got_k, got_v = ck.numpy().astype(np.float32).reshape(B, ctx, -1), cv.numpy().astype(np.float32).reshape(B, ctx, -1)
    assert_close(got_k, ck_ref, True, "cache_k", composed=True)
    assert_close(got_v, cv_ref, True, "cache_v")
    untouched = np.ones(ctx, bool); untouched[start:start + S] = False
    assert not got_k[:, untouched].any() and not got_v[:, untouched].any()


def attention_ref(q, ck, cv, B, S, start, H, KV, hd):
    """float64 causal GQA attention; probabilities rounded to fp16 as the reference does (tensor.ts:3933)."""
    out = np.zeros((B * S, H * hd))
    n_rep = H // KV
    for b in range(B):
        for s in range(S):
            T = start + s + 1
            for h in range(H):
                g = h // n_rep
                qv = q[b * S + s, h * hd:(h + 1) * hd].astype(np.float64)
                sc = ck[b, :T, g].astype(np.float64) @ qv / np.sqrt(hd)
                p = np.exp(sc - sc.max()); p /= p.sum()
                p = p.astype(np.float16).astype(np.float64)
                out[b * S + s, h * hd:(h + 1) * hd] = p @ cv[b, :T, g].astype(np.float64)
    return out


@pytest.mark.parametrize("hd,H,KV", [(64, 4, 2), (128, 4, 1), (128, 2, 2)])
@pytest.mark.parametrize("B,S,start", [(1, 1, 0), (1, 5, 0), (2, 70, 3), (1, 200, 61), (1, 129, 127)])
def test_attn_prefill_matches_float64_reference(hip, hd, H, KV, B, S, start):
    ctx = start + S + 3
    q = RNG.standard_normal((B * S, H * hd)).astype(np.float16)
    ck = RNG.standard_normal((B, ctx, KV, hd)).astype(np.float16)
    cv = RNG.standard_normal((B, ctx, KV, hd)).astype(np.float16)
    tq, tk, tv, to = Tensor(q), Tensor(ck), Tensor(cv), Tensor.empty((B * S, H * hd), "float16")
    check(hip.jsgrad_hip_attn_prefill(tq.ptr, tk.ptr, tv.ptr, to.ptr, B, S, start, H, KV, hd, ctx))
    ref = attention_ref(q, ck, cv, B, S, start, H, KV, hd)
    got = to.numpy().astype(np.float64)
    assert np.allclose(got, ref, rtol=1e-2, atol=1e-2)
    assert np.max(np.abs(got - ref)) < 4e-3     # in practice: an fp16 ulp of the output plus the fp16 rounding of p


def test_attn_prefill_one_position_equals_decode_attention(hip):
    """S = 1 through the several-position kernel against the decode kernel on the same cache."""
    H, KV, hd, ctx, pos = 8, 2, 128, 300, 211
    q = RNG.standard_normal((1, H * hd)).astype(np.float16)
    ck = RNG.standard_normal((1, ctx, KV, hd)).astype(np.float16)
    cv = RNG.standard_normal((1, ctx, KV, hd)).astype(np.float16)
    tq, tk, tv = Tensor(q), Tensor(ck), Tensor(cv)
    o1, o2 = Tensor.empty((1, H * hd), "float16"), Tensor.empty((1, H * hd), "float16")
    check(hip.jsgrad_hip_attn_prefill(tq.ptr, tk.ptr, tv.ptr, o1.ptr, 1, 1, pos, H, KV, hd, ctx))
    st = Tensor(np.array([0, pos], np.int32))
    ws = Tensor.zeros((hip.jsgrad_hip_attn_workspace_bytes(H, KV, hd),), "uint8")
    check(hip.jsgrad_hip_attn_decode(tq.ptr, tk.ptr, tv.ptr, st.ptr, o2.ptr, ws.ptr, H, KV, hd, ctx, ffi.F16))
    assert np.allclose(o1.numpy().astype(np.float32), o2.numpy().astype(np.float32), atol=2e-3)


def test_attn_decode_batch_equals_per_sequence(hip):
    B, H, KV, hd, ctx, pos = 5, 8, 2, 128, 700, 533
    q = RNG.standard_normal((B, H * hd)).astype(np.float16)
    ck = RNG.standard_normal((B, ctx, KV, hd)).astype(np.float16)
    cv = RNG.standard_normal((B, ctx, KV, hd)).astype(np.float16)
    tq, tk, tv = Tensor(q), Tensor(ck), Tensor(cv)
    st = Tensor(np.array([0, pos], np.int32))
    ob = Tensor.empty((B, H * hd), "float16")
    wsb = Tensor.zeros((hip.jsgrad_hip_attn_batch_workspace_bytes(B, H, KV, hd),), "uint8")
    for _ in range(2):   # twice: the workspace counters must come back to zero
        check(hip.jsgrad_hip_attn_decode_batch(tq.ptr, tk.ptr, tv.ptr, st.ptr, ob.ptr, wsb.ptr, B, H, KV, hd, ctx))
    ws = Tensor.zeros((hip.jsgrad_hip_attn_workspace_bytes(H, KV, hd),), "uint8")
    row = ctx * KV * hd * 2
    for b in range(B):
        o = Tensor.empty((H * hd,), "float16")
        check(hip.jsgrad_hip_attn_decode(tq.ptr + b * H * hd * 2, tk.ptr + b * row, tv.ptr + b * row, st.ptr, o.ptr, ws.ptr, H, KV, hd, ctx, ffi.F16))
        # the two launches cut the positions into chunks of different lengths (several sequences: shorter chunks, smaller
        # blocks), so the float sums differ in their last bits: the same values to an fp16 ulp, and mostly the same bits
        got, one = ob.numpy()[b].astype(np.float32), o.numpy().astype(np.float32)
        assert np.all(np.abs(got - one) <= np.spacing(np.abs(one).astype(np.float16)).astype(np.float32)), b
        assert np.mean(got == one) > 0.9, b
    ref = attention_ref(q, ck, cv, B, 1, pos, H, KV, hd)
    assert np.allclose(ob.numpy().astype(np.float64), ref, rtol=1e-2, atol=1e-2) and np.max(np.abs(ob.numpy().astype(np.float64) - ref)) < 4e-3


def test_row_companions_bit_exact(hip):
    rows, dim, vocab = 19, 320, 1000
    table = RNG.standard_normal((vocab, dim)).astype(np.float16)
    toks = RNG.integers(0, vocab, rows).astype(np.int32)
    tt, tk, out = Tensor(table), Tensor(toks), Tensor.empty((rows, dim), "float16")
    check(hip.jsgrad_hip_embed_rows(ffi.W_F16, tt.ptr, None, tk.ptr, rows, out.ptr, dim, vocab))
    assert np.array_equal(out.numpy().view(np.uint16), table[toks].view(np.uint16))
    codes, scale = orc.int8_quantize(table.astype(np.float32))
    tc, ts = Tensor(codes), Tensor(scale)
    check(hip.jsgrad_hip_embed_rows(ffi.W_I8, tc.ptr, ts.ptr, tk.ptr, rows, out.ptr, dim, vocab))
    assert np.array_equal(out.numpy().view(np.uint16), orc.int8_dequant(codes, scale)[toks].view(np.uint16))
    # RMSNorm rows: the sum of squares is reduced in a different order, so a few last bits may move
    x = RNG.standard_normal((rows, dim)).astype(np.float16)
    w = (1 + 0.1 * RNG.standard_normal(dim)).astype(np.float16)
    tx, tw, ty = Tensor(x), Tensor(w), Tensor.empty((rows, dim), "float16")
    check(hip.jsgrad_hip_rmsnorm_rows(tx.ptr, tw.ptr, ty.ptr, rows, dim, 1e-5))
    ref = np.stack([orc.rmsnorm(x[r], w, 1e-5, True) for r in range(rows)])
    assert_close(ty.numpy().astype(np.float32), ref, True, "rmsnorm rows")
    # argmax rows with ties: lowest index wins
    lg = RNG.standard_normal((rows, vocab)).astype(np.float16)
    lg[3, 500] = lg[3, 17] = 9.0
    lg[4, :] = 1.0
    tl, ti = Tensor(lg), Tensor.empty((rows,), "int32")
    check(hip.jsgrad_hip_argmax_rows(tl.ptr, rows, vocab, ti.ptr))
    assert np.array_equal(ti.numpy(), np.array([orc.argmax(lg[r]) for r in range(rows)], np.int32))
    assert ti.numpy()[3] == 17 and ti.numpy()[4] == 0
