"""Per-kernel parity of the HIP path against the CPU oracle, through the C ABI.  Integer / byte results
(quantiser codes, scales, dequantised weights, argmax indices, gathered rows) must be bit-exact; floating
point results must agree within the tolerance written in each test (north star: rtol/atol 1e-2 for fp16)."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from denograd_amd import ffi
from denograd_amd.ffi import check
from denograd_amd.tensor import Tensor
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(11)
NPDT = {"float32": np.float32, "float16": np.float16}


def act_code(dt): return ffi.F16 if dt == "float16" else ffi.F32
def f32(t): return t.numpy().astype(np.float32)


def test_device_is_gfx950(hip):
    buf = C.create_string_buffer(256)
    check(hip.jsgrad_hip_device_name(buf, 256))
    assert b"gfx950" in buf.value
    n = C.c_int()
    check(hip.jsgrad_hip_cu_count(C.byref(n)))
    assert n.value >= 64


def test_copy_roundtrip_and_memset(hip):
    x = RNG.integers(0, 255, 100003, dtype=np.uint8)
    t = Tensor(x)
    assert np.array_equal(t.numpy(), x)
    check(hip.jsgrad_hip_memset(t.ptr, 0x5A, 100003))
    assert np.all(t.numpy() == 0x5A)
    z = Tensor.zeros((4096,), "float32")
    assert np.all(z.numpy() == 0)
    with pytest.raises(ffi.HipError, match="positive"):
        p = C.c_void_p()
        check(hip.jsgrad_hip_malloc(0, C.byref(p)))


def test_freed_blocks_are_reused_by_size_class_without_a_wait(hip):
    """LRUAllocator (allocator.ts:53-77) behind jsgrad_hip_malloc/free: a freed block is handed to the next request of its
    class, frees never return memory to the driver by themselves, free_cache does, and a foreign or repeated free is an error."""
    def mem():
        live, idle = C.c_size_t(), C.c_size_t()
        check(hip.jsgrad_hip_mem_info(C.byref(live), C.byref(idle)))
        return live.value, idle.value
    check(hip.jsgrad_hip_free_cache())
    live0, idle0 = mem()
    assert idle0 == 0
    a, b, c = C.c_void_p(), C.c_void_p(), C.c_void_p()
    check(hip.jsgrad_hip_malloc(1000003, C.byref(a)))
    live1, _ = mem()
    assert 1000003 <= live1 - live0 <= 1000003 * 1.02          # rounded up to its class, under 2 %
    # a kernel still queued on the block when it is freed: the next owner's work queues behind it
    x = np.random.default_rng(5).integers(0, 255, 1000003, dtype=np.uint8)
    check(hip.jsgrad_hip_copyin(a, x.ctypes.data_as(C.c_void_p), x.nbytes))
    check(hip.jsgrad_hip_memset(a, 7, 1000003))
    check(hip.jsgrad_hip_free(a))
    assert mem() == (live0, live1 - live0)
    check(hip.jsgrad_hip_malloc(1000100, C.byref(b)))          # same class
    assert b.value == a.value and mem() == (live1, 0)
    got = np.empty(1000003, np.uint8)
    check(hip.jsgrad_hip_copyout(got.ctypes.data_as(C.c_void_p), b, got.nbytes))
    assert np.all(got == 7)
    check(hip.jsgrad_hip_malloc(5000, C.byref(c)))             # another class: a new block
    assert c.value != b.value
    check(hip.jsgrad_hip_free(b))
    with pytest.raises(ffi.HipError, match="freed already"):
        check(hip.jsgrad_hip_free(b))
    with pytest.raises(ffi.HipError, match="not handed out"):
        check(hip.jsgrad_hip_free(C.c_void_p(c.value + 256)))
    check(hip.jsgrad_hip_free(c))
    assert mem()[1] > 0
    check(hip.jsgrad_hip_free_cache())
    assert mem() == (live0, 0)


def test_generic_program_launch(hip):
    """The reference's device smoke test (cli/devices.ts:4-24): [1,2,3]*2 == [2,4,6] through Compiler + Program."""
    from denograd_amd.device import Device
    dev = Device.get("HIP").init()
    src = 'extern "C" __global__ void E_3(float* data0, const float* data1, const int n) { int i = blockIdx.x*blockDim.x+threadIdx.x; if (i < n) data0[i] = data1[i]*2.0f; }'
    prg = dev.runtime("E_3", dev.compiler.compile_cached(src))
    a = Tensor(np.float32([1, 2, 3]))
    out = Tensor.empty((3,), "float32")
    secs = prg.call([out.ptr, a.ptr], global_size=(1, 1, 1), local_size=(64, 1, 1), vals=(3,), wait=True)
    assert np.array_equal(out.numpy(), np.float32([2, 4, 6])) and secs is not None and 0 <= secs < 1.0


@pytest.mark.parametrize("dt", ["float32", "float16"])
def test_rope_table_bit_exact(hip, dt):
    for hd, end in ((64, 2 * 1024), (128, 2 * 300), (4, 164)):
        t = Tensor.empty((end, hd // 2, 2), dt)
        check(hip.jsgrad_hip_rope_table(t.ptr, hd, end, 500000.0, act_code(dt)))
        ref = orc.freqs_cis(hd, end, 500000.0).astype(NPDT[dt])
        assert np.array_equal(t.numpy().view(np.uint16 if dt == "float16" else np.uint32), ref.view(np.uint16 if dt == "float16" else np.uint32))


def test_int8_quantize_dequant_bit_exact(hip):
    for dt in ("float16", "float32"):
        w = (RNG.standard_normal((96, 512)) * 0.02).astype(NPDT[dt])
        w[7] = 0
        codes, scale, tw = Tensor.empty(w.shape, "int8"), Tensor.empty((96,), "float16"), Tensor(w)
        check(hip.jsgrad_hip_int8_quantize(tw.ptr, 96, 512, codes.ptr, scale.ptr, act_code(dt)))
        q_ref, s_ref = orc.int8_quantize(w.astype(np.float32))
        assert np.array_equal(codes.numpy(), q_ref) and np.array_equal(scale.numpy().view(np.uint16), s_ref.view(np.uint16))
    # dequantisation over every code value and awkward scales
    q = np.tile(np.arange(-128, 128, dtype=np.int8), (64, 2))
    s = np.concatenate([np.abs(RNG.standard_normal(60)) * 1e-3, [0.0, 6.1e-5, 5.96e-8, 1.0]]).astype(np.float16)
    out, tq, ts = Tensor.empty(q.shape, "float16"), Tensor(q), Tensor(s)
    check(hip.jsgrad_hip_int8_dequant(tq.ptr, ts.ptr, 64, 512, out.ptr))
    assert np.array_equal(out.numpy().view(np.uint16), orc.int8_dequant(q, s).view(np.uint16))


def test_nf4_quantize_dequant_bit_exact(hip):
    for dt in ("float16", "float32"):
        w = (RNG.standard_normal((32, 256)) * 0.02).astype(NPDT[dt])
        packed, scale, tw = Tensor.empty((w.size // 2,), "uint8"), Tensor.empty((w.size // 64, 1), "float16"), Tensor(w)
        check(hip.jsgrad_hip_nf4_quantize(tw.ptr, w.size, packed.ptr, scale.ptr, act_code(dt)))
        p_ref, s_ref = orc.nf4_quantize(w.astype(np.float32))
        assert np.array_equal(packed.numpy(), p_ref) and np.array_equal(scale.numpy().view(np.uint16), s_ref.view(np.uint16))
    allb = np.tile(np.arange(256, dtype=np.uint8), 8)
    s = np.concatenate([np.abs(RNG.standard_normal(62)) * 0.05, [1.0, 0.0]]).astype(np.float16).reshape(-1, 1)
    out, tb, ts = Tensor.empty((allb.size * 2,), "float16"), Tensor(allb), Tensor(s)
    check(hip.jsgrad_hip_nf4_dequant(tb.ptr, ts.ptr, allb.size * 2, out.ptr))
    assert np.array_equal(out.numpy().view(np.uint16), orc.nf4_dequant(allb, s).view(np.uint16))


def make_weight(kind, out_f, in_f, dt):
    w = (RNG.standard_normal((out_f, in_f)) * 0.05).astype(np.float32)
    if kind == "f32": return w, None, ffi.W_F32
    if kind == "f16": return w.astype(np.float16), None, ffi.W_F16
    if kind == "i8":
        q, s = orc.int8_quantize(w)
        return q, s, ffi.W_I8
    q, s = orc.nf4_quantize(w.astype(np.float16).astype(np.float32))
    return q, s, ffi.W_NF4


LINEAR_CASES = [("f32", "float32", 40, 256), ("f32", "float32", 1024, 768), ("f16", "float16", 72, 512), ("f16", "float16", 2048, 2048), ("f16", "float32", 64, 512),
                ("i8", "float16", 100, 1024), ("i8", "float16", 4096, 4096), ("i8", "float16", 96, 14336), ("i8", "float32", 64, 256),
                ("nf4", "float16", 64, 2048), ("nf4", "float16", 130, 4096), ("nf4", "float16", 48, 64),
                # the three ways a launch requests its items (by the items a wavefront walks): two batches of one row pair,
                # three row pairs per wavefront of a full grid with a ragged end, and (above: 96 x 14336) four batches
                ("f16", "float16", 256, 4096), ("f16", "float16", 20000, 512)]


@pytest.mark.parametrize("kind,dt,out_f,in_f", LINEAR_CASES)
def test_linear_against_oracle(hip, kind, dt, out_f, in_f):
    """y = x.W^T (+ fused RMSNorm, + residual).  Tolerance: 1e-2 relative to the output scale for fp16 activations
    (north star), 1e-4 for float32; in practice the two differ only in float summation order."""
    w, s, code = make_weight(kind, out_f, in_f, dt)
    act16 = dt == "float16"
    x = RNG.standard_normal(in_f).astype(NPDT[dt])
    res = RNG.standard_normal(out_f).astype(NPDT[dt])
    nw = (1 + 0.1 * RNG.standard_normal(in_f)).astype(NPDT[dt])
    tw, ts, tx, tr, tn = Tensor(w), (Tensor(s) if s is not None else None), Tensor(x), Tensor(res), Tensor(nw)
    y = Tensor.empty((out_f,), dt)
    tol = 1e-2 if act16 else 1e-4
    for use_norm in (False, True):
        if use_norm and in_f > 8192:          # the fused norm is for in_features = model dim; larger rows are rejected
            with pytest.raises(ffi.HipError, match="fused RMSNorm handles at most"):
                check(hip.jsgrad_hip_linear(code, tw.ptr, ts.ptr if ts else None, out_f, in_f, tx.ptr, y.ptr, tn.ptr, 1e-5, None, act_code(dt)))
            continue
        for use_res in (False, True):
            check(hip.jsgrad_hip_linear(code, tw.ptr, ts.ptr if ts else None, out_f, in_f, tx.ptr, y.ptr, tn.ptr if use_norm else None, 1e-5, tr.ptr if use_res else None, act_code(dt)))
            xin = x.astype(np.float32)
            if use_norm: xin = orc.rmsnorm(xin, nw.astype(np.float32), 1e-5, act16)
            lin = ref = orc.linear(w, s, xin, out_f, in_f, act16)[0]
            if use_res:
                ref = ref + res.astype(np.float32)
                if act16: ref = ref.astype(np.float16).astype(np.float32)
            # the product is rounded to the activation type before the residual is added: where the two cancel, one ulp of
            # the product is many ulps of the sum
            assert_close(f32(y), ref, act16, (use_norm, use_res), composed=use_norm, ulp_at=lin if use_res else None)


def test_linear_rejects_bad_shapes(hip):
    x, y, w = Tensor.zeros((100,), "float16"), Tensor.zeros((8,), "float16"), Tensor.zeros((8, 100), "int8")
    with pytest.raises(ffi.HipError, match="multiple of 16"):
        check(hip.jsgrad_hip_linear(ffi.W_I8, w.ptr, y.ptr, 8, 100, x.ptr, y.ptr, None, 0.0, None, ffi.F16))
    with pytest.raises(ffi.HipError, match="needs a scale"):
        check(hip.jsgrad_hip_linear(ffi.W_I8, w.ptr, None, 8, 96, x.ptr, y.ptr, None, 0.0, None, ffi.F16))
    # the weights are read through 32-bit byte offsets: a matrix of 4 GiB or more is refused before anything is launched
    with pytest.raises(ffi.HipError, match="4 GiB"):
        check(hip.jsgrad_hip_linear(ffi.W_F32, w.ptr, None, 70000, 16384, x.ptr, y.ptr, None, 0.0, None, ffi.F32))


@pytest.mark.parametrize("dt", ["float32", "float16"])
def test_rmsnorm_against_oracle(hip, dt):
    for d in (256, 2048, 3072, 4096):
        x = (RNG.standard_normal(d) * 2).astype(NPDT[dt])
        w = (1 + 0.1 * RNG.standard_normal(d)).astype(NPDT[dt])
        y, tx, tw = Tensor.empty((d,), dt), Tensor(x), Tensor(w)
        check(hip.jsgrad_hip_rmsnorm(tx.ptr, tw.ptr, y.ptr, d, 1e-5, act_code(dt)))
        ref = orc.rmsnorm(x.astype(np.float32), w.astype(np.float32), 1e-5, dt == "float16")
        tol = 1e-2 if dt == "float16" else 1e-5
        assert np.max(np.abs(f32(y) - ref)) <= tol * np.abs(ref).max()
        if dt == "float16": assert np.mean(f32(y) == ref) > 0.99


@pytest.mark.parametrize("kind", ["f32", "f16", "i8"])
def test_embedding_gather_bit_exact(hip, kind):
    V, d = 1000, 256
    dt = "float32" if kind == "f32" else "float16"
    w, s, code = make_weight(kind, V, d, dt)
    tw, ts = Tensor(w), (Tensor(s) if s is not None else None)
    out = Tensor.empty((d,), dt)
    for tok in (0, 17, V - 1):
        st = Tensor(np.int32([tok, 3]))
        check(hip.jsgrad_hip_embed(code, tw.ptr, ts.ptr if ts else None, st.ptr, out.ptr, d, V, act_code(dt)))
        if kind == "i8": ref = (w[tok].astype(np.float64) * float(s[tok])).astype(np.float16)
        else: ref = w[tok]
        assert np.array_equal(out.numpy().view(np.uint16 if dt == "float16" else np.uint32), ref.view(np.uint16 if dt == "float16" else np.uint32))


@pytest.mark.parametrize("dt", ["float32", "float16"])
def test_argmax_lowest_index_and_state_update(hip, dt):
    toks = Tensor.zeros((64,), "int32")
    for n, vals in ((5, [1, 5, 5, 2, 5]), (3, [3, 3, 3]), (3, [-np.inf, -1, -1])):
        st = Tensor(np.int32([0, 7]))
        tv = Tensor(np.array(vals, NPDT[dt]))
        check(hip.jsgrad_hip_argmax(tv.ptr, n, st.ptr, toks.ptr, 64, 1, act_code(dt)))
        assert list(st.numpy()) == [orc.argmax(vals), 8] and toks.numpy()[7] == orc.argmax(vals)
    x = RNG.standard_normal(128256).astype(np.float16).astype(NPDT[dt])
    x[[100000, 2000, 77777]] = x.max() + 1            # three-way tie, lowest index wins
    st, tx = Tensor(np.int32([0, 0])), Tensor(x)
    check(hip.jsgrad_hip_argmax(tx.ptr, x.size, st.ptr, None, 0, 0, act_code(dt)))
    assert list(st.numpy()) == [2000, 0]


QKV_CASES = [("f32", "float32", 256, 4, 2, 64), ("f16", "float16", 2048, 32, 8, 64), ("i8", "float16", 1024, 8, 2, 128), ("nf4", "float16", 1024, 8, 8, 128),
             ("i8", "float16", 768, 6, 2, 128)]


@pytest.mark.parametrize("kind,dt,dim,H,KV,hd", QKV_CASES)
def test_qkv_rope_cache_write(hip, kind, dt, dim, H, KV, hd):
    """attention_norm + wq/wk/wv + rotary + cache assign (models/llama.ts:61-87) at a non-zero position."""
    act16, ctx, pos = dt == "float16", 48, 37
    (wq, sq, code), (wk, sk, _), (wv, sv, _) = make_weight(kind, H * hd, dim, dt), make_weight(kind, KV * hd, dim, dt), make_weight(kind, KV * hd, dim, dt)
    x = RNG.standard_normal(dim).astype(NPDT[dt])
    nw = (1 + 0.1 * RNG.standard_normal(dim)).astype(NPDT[dt])
    table = Tensor.empty((2 * ctx, hd // 2, 2), dt)
    check(hip.jsgrad_hip_rope_table(table.ptr, hd, 2 * ctx, 500000.0, act_code(dt)))
    ck, cv = Tensor.zeros((ctx, KV, hd), dt), Tensor.zeros((ctx, KV, hd), dt)
    q = Tensor.empty((H * hd,), dt)
    T = lambda a: Tensor(a) if a is not None else None
    tq, tk, tv, tsq, tsk, tsv = T(wq), T(wk), T(wv), T(sq), T(sk), T(sv)
    p = lambda t: t.ptr if t is not None else None
    st, tx, tnw = Tensor(np.int32([0, pos])), Tensor(x), Tensor(nw)
    check(hip.jsgrad_hip_qkv_rope(code, tq.ptr, p(tsq), tk.ptr, p(tsk), tv.ptr, p(tsv), tx.ptr, tnw.ptr, 1e-5, table.ptr, st.ptr,
                                  q.ptr, ck.ptr, cv.ptr, dim, H, KV, hd, ctx, act_code(dt)))
    xn = orc.rmsnorm(x.astype(np.float32), nw.astype(np.float32), 1e-5, act16)
    fc = orc.freqs_cis(hd, 2 * ctx, 500000.0)[pos].astype(NPDT[dt]).astype(np.float32)
    q_ref = orc.rope(orc.linear(wq, sq, xn, H * hd, dim, act16)[0], H, hd, fc, act16)
    k_ref = orc.rope(orc.linear(wk, sk, xn, KV * hd, dim, act16)[0], KV, hd, fc, act16)
    v_ref = orc.linear(wv, sv, xn, KV * hd, dim, act16)[0]
    for got, ref in ((f32(q), q_ref), (f32(ck)[pos].reshape(-1), k_ref), (f32(cv)[pos].reshape(-1), v_ref)):
        assert_close(got, ref, act16, composed=True)
    rows = np.arange(ctx) != pos
    assert np.all(f32(ck)[rows] == 0) and np.all(f32(cv)[rows] == 0)      # only row `pos` is written
    # a position outside the cache must not write anything (and must not fault)
    st2 = Tensor(np.int32([0, ctx]))
    before = ck.numpy().copy()
    check(hip.jsgrad_hip_qkv_rope(code, tq.ptr, p(tsq), tk.ptr, p(tsk), tv.ptr, p(tsv), tx.ptr, tnw.ptr, 1e-5, table.ptr, st2.ptr,
                                  q.ptr, ck.ptr, cv.ptr, dim, H, KV, hd, ctx, act_code(dt)))
    assert np.array_equal(ck.numpy(), before)


@pytest.mark.parametrize("kind,dt,dim,F", [("f32", "float32", 256, 768), ("f16", "float16", 2048, 8192), ("i8", "float16", 1024, 2816), ("nf4", "float16", 1024, 1000)])
def test_ffn_gate_swiglu(hip, kind, dt, dim, F):
    act16 = dt == "float16"
    (w1, s1, code), (w3, s3, _) = make_weight(kind, F, dim, dt), make_weight(kind, F, dim, dt)
    x = (RNG.standard_normal(dim) * 3).astype(NPDT[dt])
    nw = (1 + 0.1 * RNG.standard_normal(dim)).astype(NPDT[dt])
    T = lambda a: Tensor(a) if a is not None else None
    t1, t3, ts1, ts3 = T(w1), T(w3), T(s1), T(s3)
    p = lambda t: t.ptr if t is not None else None
    g, tx, tnw = Tensor.empty((F,), dt), Tensor(x), Tensor(nw)
    check(hip.jsgrad_hip_ffn_gate(code, t1.ptr, p(ts1), t3.ptr, p(ts3), tx.ptr, tnw.ptr, 1e-5, g.ptr, dim, F, act_code(dt)))
    xn = orc.rmsnorm(x.astype(np.float32), nw.astype(np.float32), 1e-5, act16)
    a, u = orc.linear(w1, s1, xn, F, dim, act16)[0], orc.linear(w3, s3, xn, F, dim, act16)[0]
    ref = orc.silu(a, act16) * u
    if act16: ref = ref.astype(np.float16).astype(np.float32)
    assert_close(f32(g), ref, act16, composed=True)


def attn_oracle(q, K, V, H, KV, hd, T, act16, round_p=True):
    """scores -> softmax -> P.V with the oracle's exp and rounding points, written with numpy around orc.xexp2f.
    round_p=False leaves the probabilities in float32 (what the kernels do: see test_attention_decode_unrounded_probabilities)."""
    out = np.empty(H * hd, np.float32)
    scale = np.float32(1.0 / np.sqrt(hd))
    for h in range(H):
        g = h // (H // KV)
        s = np.array([np.float32(np.dot(q[h * hd:(h + 1) * hd].astype(np.float64), K[t, g].astype(np.float64))) for t in range(T)], np.float32) * scale
        e = orc.xexp2f(((s - s.max()) * np.float32(1.4426950408889634)).astype(np.float32))
        p = (e * (np.float32(1) / e.astype(np.float32).sum(dtype=np.float32))).astype(np.float32)
        if act16 and round_p: p = p.astype(np.float16).astype(np.float32)
        o = (p[:, None].astype(np.float64) * V[:T, g].astype(np.float64)).sum(0).astype(np.float32)
        out[h * hd:(h + 1) * hd] = o.astype(np.float16).astype(np.float32) if act16 else o
    return out


@pytest.mark.parametrize("dt,H,KV,hd,ctx", [("float32", 4, 2, 64, 64), ("float16", 32, 8, 64, 1024), ("float16", 24, 8, 128, 600), ("float16", 8, 8, 128, 300),
                                             ("float16", 8, 1, 64, 2100), ("float32", 6, 2, 128, 96),
                                             ("float16", 8, 2, 128, 4096),
                                             ("float16", 4, 2, 64, 17000)])   # beyond 16384 positions: the 16-wavefront blocks with 256-row chunks
def test_attention_decode(hip, dt, H, KV, hd, ctx):
    """GQA decode attention over the cache for several T, including T=1, chunk boundaries and the full cache;
    repeated launches share one workspace (the merging block must leave the counters at zero)."""
    act16 = dt == "float16"
    K = (RNG.standard_normal((ctx, KV, hd)) * 0.7).astype(NPDT[dt])
    V = RNG.standard_normal((ctx, KV, hd)).astype(NPDT[dt])
    q = (RNG.standard_normal(H * hd) * 0.7).astype(NPDT[dt])
    tK, tV, tq = Tensor(K), Tensor(V), Tensor(q)
    out = Tensor.empty((H * hd,), dt)
    ws = Tensor.zeros((hip.jsgrad_hip_attn_workspace_bytes(H, KV, hd),), "uint8")
    for T in sorted(t for t in {1, 2, 31, 32, 33, 65, ctx // 2 + 1, ctx - 1, ctx} if t <= ctx):
        st = Tensor(np.int32([0, T - 1]))
        check(hip.jsgrad_hip_attn_decode(tq.ptr, tK.ptr, tV.ptr, st.ptr, out.ptr, ws.ptr, H, KV, hd, ctx, act_code(dt)))
        ref = attn_oracle(q.astype(np.float32), K.astype(np.float32), V.astype(np.float32), H, KV, hd, T, act16)
        tol = 1e-2 if act16 else 1e-4
        assert np.max(np.abs(f32(out) - ref)) <= tol * max(1.0, np.abs(ref).max()), f"T={T}"
        assert np.mean(np.abs(f32(out) - ref) <= np.abs(ref) * (2.0 ** -8 if act16 else 2.0 ** -16) + 2e-4) > 0.99, f"T={T}"
    assert np.all(ws.numpy() == 0)   # a launch leaves the workspace as it found it: zero words mean `not written yet`


@pytest.mark.parametrize("H,KV,hd,ctx", [(32, 8, 128, 1500), (8, 2, 64, 700)])
def test_attention_decode_unrounded_probabilities(hip, H, KV, hd, ctx):
    """The one place where the decode attention leaves the oracle's rounding points: the oracle rounds every probability
    to fp16 before P.V (tensor.ts:3931-3933 on fp16 tensors), the kernels multiply V by the float32 probability (the
    normalisation 1/sum is only known after the last chunk).  This pins the size of that difference: against the same
    arithmetic WITHOUT the rounding the kernel is within one fp16 unit of the result everywhere, and the two references
    differ by at most 2^-11 * sum_t p_t |v_t| <= 2^-11 * max|V| (each probability moves by at most half an fp16 unit of itself)."""
    rng = np.random.default_rng(H * 1000 + ctx)
    K = (rng.standard_normal((ctx, KV, hd)) * 0.7).astype(np.float16)
    V = rng.standard_normal((ctx, KV, hd)).astype(np.float16)
    q = (rng.standard_normal(H * hd) * 0.7).astype(np.float16)
    tK, tV, tq = Tensor(K), Tensor(V), Tensor(q)
    out = Tensor.empty((H * hd,), "float16")
    ws = Tensor.zeros((hip.jsgrad_hip_attn_workspace_bytes(H, KV, hd),), "uint8")
    for T in (ctx, ctx // 3):
        check(hip.jsgrad_hip_attn_decode(tq.ptr, tK.ptr, tV.ptr, Tensor(np.int32([0, T - 1])).ptr, out.ptr, ws.ptr, H, KV, hd, ctx, act_code("float16")))
        got = f32(out)
        args = (q.astype(np.float32), K.astype(np.float32), V.astype(np.float32), H, KV, hd, T, True)
        rounded, unrounded = attn_oracle(*args), attn_oracle(*args, round_p=False)
        ulp = np.maximum(np.abs(unrounded), 2.0 ** -14) * 2.0 ** -10          # one unit in the last place of an fp16 of that size
        assert np.all(np.abs(got - unrounded) <= ulp), f"T={T}: {np.max(np.abs(got - unrounded) / ulp):.2f} units"
        bound = 2.0 ** -11 * float(np.abs(V[:T].astype(np.float32)).max())
        assert np.max(np.abs(rounded - unrounded)) <= bound + float(ulp.max()), f"T={T}"
        assert np.max(np.abs(got - rounded)) <= bound + 2 * float(ulp.max()), f"T={T}"


@pytest.mark.parametrize("kind,H,KV,hd,ctx", [("f16", 32, 8, 64, 1024), ("i8", 8, 2, 128, 4096), ("f16", 4, 4, 64, 96), ("i8", 24, 8, 128, 640), ("f16", 8, 2, 64, 8192),
                                              ("nf4", 32, 8, 128, 640), ("nf4", 8, 2, 64, 4160)])
def test_attention_and_wo_in_one_launch(hip, kind, H, KV, hd, ctx):
    """jsgrad_hip_attn_wo == jsgrad_hip_attn_decode followed by jsgrad_hip_linear(wo, residual), bit for bit, for several T,
    two layers sharing one workspace (the version tag tells their rows apart), and no bounded wait ever running out."""
    dim, qdim = 256, H * hd
    K = (RNG.standard_normal((ctx, KV, hd)) * 0.7).astype(np.float16)
    V = RNG.standard_normal((ctx, KV, hd)).astype(np.float16)
    q = (RNG.standard_normal(qdim) * 0.7).astype(np.float16)
    res = RNG.standard_normal(dim).astype(np.float16)
    w = (RNG.standard_normal((dim, qdim)) * 0.05).astype(np.float32)
    if kind == "i8":
        wq, sc = orc.int8_quantize(w)
        tw, ts, code = Tensor(wq), Tensor(sc), ffi.W_I8
    elif kind == "nf4":
        wq, sc = orc.nf4_quantize(w)
        tw, ts, code = Tensor(wq), Tensor(sc), ffi.W_NF4
    else:
        tw, ts, code = Tensor(w.astype(np.float16)), None, ffi.W_F16
    tK, tV, tq, tres = Tensor(K), Tensor(V), Tensor(q), Tensor(res)
    attn, y_two, y_one = Tensor.empty((qdim,), "float16"), Tensor.empty((dim,), "float16"), Tensor.empty((dim,), "float16")
    ws2 = Tensor.zeros((hip.jsgrad_hip_attn_workspace_bytes(H, KV, hd),), "uint8")
    ws1 = Tensor.zeros((hip.jsgrad_hip_attn_wo_workspace_bytes(H, KV, hd),), "uint8")
    sp_ = ts.ptr if ts is not None else None
    for T in sorted(t for t in {1, 2, 33, 65, ctx // 2 + 1, ctx} if t <= ctx):
        st = Tensor(np.int32([0, T - 1]))
        check(hip.jsgrad_hip_attn_decode(tq.ptr, tK.ptr, tV.ptr, st.ptr, attn.ptr, ws2.ptr, H, KV, hd, ctx, ffi.F16))
        check(hip.jsgrad_hip_linear(code, tw.ptr, sp_, dim, qdim, attn.ptr, y_two.ptr, None, 0.0, tres.ptr, ffi.F16))
        for layer in (0, 1):
            check(hip.jsgrad_hip_memset(y_one.ptr, 0, y_one.nbytes))
            check(hip.jsgrad_hip_attn_wo(tq.ptr, tK.ptr, tV.ptr, st.ptr, ws1.ptr, H, KV, hd, ctx, code, tw.ptr, sp_, dim, tres.ptr, y_one.ptr, layer))
            assert np.array_equal(y_one.numpy(), y_two.numpy()), f"T={T} layer={layer}"
    # without a residual (T is the last one of the loop; layer 0 again, another position would do as well)
    st = Tensor(np.int32([0, max(ctx // 4, 1) - 1]))
    check(hip.jsgrad_hip_attn_decode(tq.ptr, tK.ptr, tV.ptr, st.ptr, attn.ptr, ws2.ptr, H, KV, hd, ctx, ffi.F16))
    check(hip.jsgrad_hip_linear(code, tw.ptr, sp_, dim, qdim, attn.ptr, y_two.ptr, None, 0.0, None, ffi.F16))
    check(hip.jsgrad_hip_attn_wo(tq.ptr, tK.ptr, tV.ptr, st.ptr, ws1.ptr, H, KV, hd, ctx, code, tw.ptr, sp_, dim, None, y_one.ptr, 0))
    assert np.array_equal(y_one.numpy(), y_two.numpy()), "no residual"
    e = C.c_int(0)
    check(hip.jsgrad_hip_attn_wo_status(ws1.ptr, C.byref(e)))
    assert e.value == 0
    assert np.all(ws1.numpy()[:256] == 0)      # the chunk counters are left at zero
