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
