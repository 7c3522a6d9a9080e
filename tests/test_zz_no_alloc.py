"""The entry point that allocates nothing (jsgrad_hip_attn_decode_static: decode attention with the library's built-in
workspace) against jsgrad_hip_attn_decode with a caller-owned workspace: bit-identical outputs, on two calls in a row, the
second with a smaller input (fewer heads, a shorter context, another head_dim), then the first shape again."""
import numpy as np
import pytest

from denograd_amd import ffi
from denograd_amd.ffi import check
from denograd_amd.tensor import Tensor

pytestmark = pytest.mark.gpu


def run_both(hip, rng, H, KV, hd, ctx, pos, act="float16"):
    dt = np.float16 if act == "float16" else np.float32
    code = ffi.F16 if act == "float16" else ffi.F32
    q = rng.standard_normal((H * hd,)).astype(dt)
    ck = rng.standard_normal((ctx, KV, hd)).astype(dt)
    cv = rng.standard_normal((ctx, KV, hd)).astype(dt)
    tq, tk, tv = Tensor(q), Tensor(ck), Tensor(cv)
    st = Tensor(np.array([0, pos], np.int32))
    want, got = Tensor.zeros((H * hd,), act), Tensor.zeros((H * hd,), act)
    ws = Tensor.zeros((hip.jsgrad_hip_attn_workspace_bytes(H, KV, hd),), "uint8")
    check(hip.jsgrad_hip_attn_decode(tq.ptr, tk.ptr, tv.ptr, st.ptr, want.ptr, ws.ptr, H, KV, hd, ctx, code))
    check(hip.jsgrad_hip_attn_decode_static(tq.ptr, tk.ptr, tv.ptr, st.ptr, got.ptr, H, KV, hd, ctx, code))
    a, b = want.numpy(), got.numpy()
    assert np.any(a != 0)
    assert np.array_equal(a.view(np.uint16 if act == "float16" else np.uint32), b.view(np.uint16 if act == "float16" else np.uint32)), (H, KV, hd, ctx, pos)


def test_static_workspace_attention_equals_the_workspace_version(hip):
    rng = np.random.default_rng(5)
    run_both(hip, rng, 32, 8, 128, 4352, 4200)        # the 8B shape at a long context: many chunks per kv head
    run_both(hip, rng, 8, 2, 64, 300, 37)             # smaller: fewer heads, fewer chunks, other head_dim (stale partials behind it)
    run_both(hip, rng, 32, 8, 128, 4352, 4200)        # and the large shape again
    run_both(hip, rng, 4, 4, 64, 64, 0, act="float32")  # one visible position, float32 activations


def test_static_workspace_attention_refuses_what_does_not_fit(hip):
    t = Tensor.zeros((64,), "float16")
    st = Tensor(np.array([0, 0], np.int32))
    assert hip.jsgrad_hip_attn_decode_static_max_bytes() == 8 << 20
    with pytest.raises(ffi.HipError, match="built-in one holds"):
        check(hip.jsgrad_hip_attn_decode_static(t.ptr, t.ptr, t.ptr, st.ptr, t.ptr, 128, 64, 128, 65536, ffi.F16))
    with pytest.raises(ffi.HipError, match="null pointer"):
        check(hip.jsgrad_hip_attn_decode_static(None, t.ptr, t.ptr, st.ptr, t.ptr, 8, 2, 64, 128, ffi.F16))


def test_static_workspace_attention_captured_in_a_graph_allocates_nothing(hip):
    """The call only launches kernels (the built-in workspace's address was resolved by jsgrad_hip_init), so it may be
    recorded into a graph: every replay equals the eager result bit for bit, with the library's eager work and waits
    between the replays, and the allocator's books (live and parked bytes) do not move around the call or the replays."""
    import ctypes as C
    rng = np.random.default_rng(9)
    H, KV, hd, ctx = 32, 8, 128, 1024
    q = rng.standard_normal((H * hd,)).astype(np.float16)
    ck = rng.standard_normal((ctx, KV, hd)).astype(np.float16)
    cv = rng.standard_normal((ctx, KV, hd)).astype(np.float16)
    tq, tk, tv = Tensor(q), Tensor(ck), Tensor(cv)
    st = Tensor(np.array([0, 700], np.int32))
    want, got = Tensor.zeros((H * hd,), "float16"), Tensor.zeros((H * hd,), "float16")
    ws = Tensor.zeros((hip.jsgrad_hip_attn_workspace_bytes(H, KV, hd),), "uint8")

    def mem():
        live, idle = C.c_size_t(), C.c_size_t()
        check(hip.jsgrad_hip_mem_info(C.byref(live), C.byref(idle)))
        return live.value, idle.value
    before = mem()
    check(hip.jsgrad_hip_attn_decode_static(tq.ptr, tk.ptr, tv.ptr, st.ptr, got.ptr, H, KV, hd, ctx, ffi.F16))     # eager
    graph = C.c_void_p()
    check(hip.jsgrad_hip_graph_begin())
    try:
        check(hip.jsgrad_hip_attn_decode_static(tq.ptr, tk.ptr, tv.ptr, st.ptr, got.ptr, H, KV, hd, ctx, ffi.F16))
    finally:
        check(hip.jsgrad_hip_graph_end(C.byref(graph)))
    assert mem() == before
    for pos in (700, 5, 1023, 64):
        check(hip.jsgrad_hip_copyin(st.ptr, np.array([0, pos], np.int32).ctypes.data, 8))
        check(hip.jsgrad_hip_attn_decode(tq.ptr, tk.ptr, tv.ptr, st.ptr, want.ptr, ws.ptr, H, KV, hd, ctx, ffi.F16))   # eager work between replays
        check(hip.jsgrad_hip_memset(got.ptr, 0, got.nbytes))
        check(hip.jsgrad_hip_graph_launch(graph))
        check(hip.jsgrad_hip_sync())
        assert np.array_equal(want.numpy().view(np.uint16), got.numpy().view(np.uint16)), pos
        assert mem() == before
    check(hip.jsgrad_hip_graph_destroy(graph))
    e = C.c_int(7)
    check(hip.jsgrad_hip_attn_decode_static_status(C.byref(e)))
    assert e.value == 0
    check(hip.jsgrad_hip_attn_decode_status(ws.ptr, H, KV, hd, C.byref(e)))
    assert e.value == 0


def test_attention_status_reports_and_clears_a_spoilt_workspace(hip):
    """What jsgrad_hip_attn_decode_status does after a wait ran out, forced from the host: the error word is set and stale
    partial results sit in the workspace (as a merging block that gave up leaves them).  The call reports the error once,
    clears the whole workspace, and the next launch on it is correct again."""
    import ctypes as C
    rng = np.random.default_rng(10)
    H, KV, hd, ctx, pos = 8, 2, 64, 512, 400
    q = rng.standard_normal((H * hd,)).astype(np.float16)
    ck = rng.standard_normal((ctx, KV, hd)).astype(np.float16)
    cv = rng.standard_normal((ctx, KV, hd)).astype(np.float16)
    tq, tk, tv = Tensor(q), Tensor(ck), Tensor(cv)
    st = Tensor(np.array([0, pos], np.int32))
    want, got = Tensor.zeros((H * hd,), "float16"), Tensor.zeros((H * hd,), "float16")
    n = hip.jsgrad_hip_attn_workspace_bytes(H, KV, hd)
    ws, spoilt = Tensor.zeros((n,), "uint8"), Tensor.zeros((n,), "uint8")
    check(hip.jsgrad_hip_attn_decode(tq.ptr, tk.ptr, tv.ptr, st.ptr, want.ptr, ws.ptr, H, KV, hd, ctx, ffi.F16))
    junk = rng.integers(1, 255, n, dtype=np.uint8)
    junk[:4] = (1, 0, 0, 0)                                  # the error word
    check(hip.jsgrad_hip_copyin(spoilt.ptr, junk.ctypes.data, n))
    e = C.c_int(0)
    check(hip.jsgrad_hip_attn_decode_status(spoilt.ptr, H, KV, hd, C.byref(e)))
    assert e.value == 1
    assert not spoilt.numpy().any()
    check(hip.jsgrad_hip_attn_decode_status(spoilt.ptr, H, KV, hd, C.byref(e)))
    assert e.value == 0
    check(hip.jsgrad_hip_attn_decode(tq.ptr, tk.ptr, tv.ptr, st.ptr, got.ptr, spoilt.ptr, H, KV, hd, ctx, ffi.F16))
    assert np.array_equal(want.numpy().view(np.uint16), got.numpy().view(np.uint16))
