"""Llama decoder on the HIP device: the classes of /root/reference/jsgrad/models/llama.ts with the same
names, constructor arguments and call order, executing hand-written gfx950 kernels instead of a lazy graph.

Decode (one token, one sequence) is five launches per layer:
  attention_norm + wq/wk/wv + rotary + KV-cache write | GQA attention over the cache | wo + residual |
  ffn_norm + w1/w3 + SwiGLU | w2 + residual
plus the embedding gather, final norm + lm_head, and the greedy argmax.  The token id and start_pos live
in a device int32[2] (`state`) that the kernels read, so the whole step is position-independent and can
be captured once as a HIP graph (the role TinyJit's symbolic `start_pos` plays at llama.ts:214-220).
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import ffi
from .ffi import check
from .nn import Embedding, Linear, RMSNorm, act_code
from .tensor import Tensor


def precompute_freqs_cis(dim: int, end: int, theta: float = 10000.0, dtype: str = "float32", device: str = "HIP") -> Tensor:
    """llama.ts:10-14 -> [1, end, 1, dim//2, 2] (cos, sin); `dtype` applies the cast of llama.ts:205."""
    t = Tensor.empty((1, end, 1, dim // 2, 2), dtype, device)
    check(ffi.load().jsgrad_hip_rope_table(t.ptr, dim, end, float(theta), act_code(dtype)))
    return t


class Attention:
    def __init__(self, dim: int, n_heads: int, n_kv_heads: int | None, max_context: int, linear=Linear):
        self.n_heads = n_heads
        self.n_kv_heads = n_kv_heads if n_kv_heads is not None else n_heads
        self.head_dim = dim // n_heads
        self.n_rep = self.n_heads // self.n_kv_heads
        self.max_context = max_context
        self.dim = dim
        self.wq = linear(dim, self.n_heads * self.head_dim, False)
        self.wk = linear(dim, self.n_kv_heads * self.head_dim, False)
        self.wv = linear(dim, self.n_kv_heads * self.head_dim, False)
        self.wo = linear(self.n_heads * self.head_dim, dim, False)
        self.cache_kv: Tensor | None = None
        self.layer_id: int | None = None   # set by Transformer: which layer of the model this is

    def _ensure_cache(self, dtype: str, device: str, bsz: int = 1) -> None:
        # Tensor.zeros([2, bsz, max_context, n_kv_heads, head_dim]) (llama.ts:78-80); created for the batch size of the
        # first call, as in the reference, and recreated (empty) when a call arrives with another batch size
        if self.cache_kv is None or self.cache_kv.shape[1] != bsz:
            self.cache_kv = Tensor.zeros((2, bsz, self.max_context, self.n_kv_heads, self.head_dim), dtype, device)

    def call_rows(self, xn: Tensor, bsz: int, seqlen: int, start_pos: int, state: Tensor, freqs_cis: Tensor, rows: "_RowScratch", residual: Tensor, out: Tensor) -> Tensor:
        """Several positions and/or sequences: xn [bsz*seqlen, dim] is the normed input; out = residual + wo(attention)."""
        lib = ffi.load()
        half = self.cache_kv.nbytes // 2
        ck, cv = self.cache_kv.ptr, self.cache_kv.ptr + half
        n = bsz * seqlen
        sp = lambda l: l.scale.ptr if l.scale is not None else None
        check(lib.jsgrad_hip_gemm_qkv_rope(self.wq.kind, self.wq.weight.ptr, sp(self.wq), self.wk.weight.ptr, sp(self.wk), self.wv.weight.ptr, sp(self.wv),
                                           xn.ptr, n, seqlen, start_pos, freqs_cis.ptr, rows.q.ptr, ck, cv,
                                           self.dim, self.n_heads, self.n_kv_heads, self.head_dim, self.max_context))
        if seqlen == 1:
            check(lib.jsgrad_hip_attn_decode_batch(rows.q.ptr, ck, cv, state.ptr, rows.attn.ptr, rows.workspace.ptr, bsz,
                                                   self.n_heads, self.n_kv_heads, self.head_dim, self.max_context))
        else:
            check(lib.jsgrad_hip_attn_prefill(rows.q.ptr, ck, cv, rows.attn.ptr, bsz, seqlen, start_pos, self.n_heads, self.n_kv_heads, self.head_dim, self.max_context))
        check(lib.jsgrad_hip_gemm(self.wo.kind, self.wo.weight.ptr, sp(self.wo), self.dim, self.n_heads * self.head_dim, rows.attn.ptr, n, out.ptr, residual.ptr))
        return out

    def call(self, x: Tensor, state: Tensor, freqs_cis: Tensor, norm: RMSNorm, ctx: "_Scratch") -> Tensor:
        """x: the block input row; returns x + wo(attention(norm(x))) in ctx.h2."""
        lib = ffi.load()
        act = act_code(x.dtype)
        self._ensure_cache(x.dtype, x.device)
        half = self.cache_kv.nbytes // 2
        ck, cv = self.cache_kv.ptr, self.cache_kv.ptr + half
        sp = lambda l: l.scale.ptr if l.scale is not None else None
        check(lib.jsgrad_hip_qkv_rope(self.wq.kind, self.wq.weight.ptr, sp(self.wq), self.wk.weight.ptr, sp(self.wk), self.wv.weight.ptr, sp(self.wv),
                                      x.ptr, norm.weight.ptr, norm.eps, freqs_cis.ptr, state.ptr, ctx.q.ptr, ck, cv,
                                      self.dim, self.n_heads, self.n_kv_heads, self.head_dim, self.max_context, act))
        if ctx.fuse_attn_wo and self.layer_id is not None:
            # attention and wo as one launch: the wo weights are on their way while the attention items run
            check(lib.jsgrad_hip_attn_wo(ctx.q.ptr, ck, cv, state.ptr, ctx.attn_wo_ws.ptr, self.n_heads, self.n_kv_heads, self.head_dim, self.max_context,
                                         self.wo.kind, self.wo.weight.ptr, sp(self.wo), self.dim, x.ptr, ctx.h2.ptr, self.layer_id))
            return ctx.h2
        check(lib.jsgrad_hip_attn_decode(ctx.q.ptr, ck, cv, state.ptr, ctx.attn.ptr, ctx.workspace.ptr,
                                         self.n_heads, self.n_kv_heads, self.head_dim, self.max_context, act))
        return self.wo.call(ctx.attn, out=ctx.h2, residual=x)


class FeedForward:
    def __init__(self, dim: int, hidden_dim: int, linear=Linear):
        self.dim, self.hidden_dim = dim, hidden_dim
        self.w1 = linear(dim, hidden_dim, False)
        self.w2 = linear(hidden_dim, dim, False)
        self.w3 = linear(dim, hidden_dim, False)  # the gate in Gated Linear Unit

    def call(self, x: Tensor, norm: RMSNorm, ctx: "_Scratch", out: Tensor) -> Tensor:
        """out = x + w2( silu(w1 n) * (w3 n) ), n = norm(x)  (SwiGLU, llama.ts:108-110 with the residual of :126)."""
        sp = lambda l: l.scale.ptr if l.scale is not None else None
        check(ffi.load().jsgrad_hip_ffn_gate(self.w1.kind, self.w1.weight.ptr, sp(self.w1), self.w3.weight.ptr, sp(self.w3), x.ptr, norm.weight.ptr, norm.eps,
                                             ctx.g.ptr, self.dim, self.hidden_dim, act_code(x.dtype)))
        return self.w2.call(ctx.g, out=out, residual=x)

    def call_rows(self, xn: Tensor, n: int, rows: "_RowScratch", residual: Tensor, out: Tensor) -> Tensor:
        """out = residual + w2( silu(w1 xn) * (w3 xn) ) for n rows of normed input."""
        lib = ffi.load()
        sp = lambda l: l.scale.ptr if l.scale is not None else None
        check(lib.jsgrad_hip_gemm_ffn_gate(self.w1.kind, self.w1.weight.ptr, sp(self.w1), self.w3.weight.ptr, sp(self.w3), xn.ptr, n, rows.g.ptr, self.dim, self.hidden_dim))
        check(lib.jsgrad_hip_gemm(self.w2.kind, self.w2.weight.ptr, sp(self.w2), self.dim, self.hidden_dim, rows.g.ptr, n, out.ptr, residual.ptr))
        return out


class TransformerBlock:
    def __init__(self, dim: int, hidden_dim: int, n_heads: int, n_kv_heads: int | None, norm_eps: float, max_context: int, linear=Linear, feed_forward=FeedForward):
        self.attention = Attention(dim, n_heads, n_kv_heads, max_context, linear)
        self.feed_forward = feed_forward(dim, hidden_dim, linear)
        self.attention_norm = RMSNorm(dim, norm_eps)
        self.ffn_norm = RMSNorm(dim, norm_eps)

    def call(self, x: Tensor, state: Tensor, freqs_cis: Tensor, ctx: "_Scratch") -> Tensor:
        h = self.attention.call(x, state, freqs_cis, self.attention_norm, ctx)     # ctx.h2
        return self.feed_forward.call(h, self.ffn_norm, ctx, out=x)                # back into x

    def call_rows(self, x: Tensor, bsz: int, seqlen: int, start_pos: int, state: Tensor, freqs_cis: Tensor, rows: "_RowScratch") -> Tensor:
        """TransformerBlock.call (llama.ts:124-127) on x [bsz*seqlen, dim]; the result is written back into x."""
        lib, n = ffi.load(), bsz * seqlen
        check(lib.jsgrad_hip_rmsnorm_rows(x.ptr, self.attention_norm.weight.ptr, rows.xn.ptr, n, self.attention.dim, self.attention_norm.eps))
        h = self.attention.call_rows(rows.xn, bsz, seqlen, start_pos, state, freqs_cis, rows, residual=x, out=rows.h2)
        check(lib.jsgrad_hip_rmsnorm_rows(h.ptr, self.ffn_norm.weight.ptr, rows.xn.ptr, n, self.attention.dim, self.ffn_norm.eps))
        return self.feed_forward.call_rows(rows.xn, n, rows, residual=h, out=x)


def attn_wo_fits(n_heads: int, n_kv_heads: int, head_dim: int, max_context: int, kind: int, dim: int, capacity: int | None = None) -> bool:
    """Whether attention and wo of this shape may share a launch: every block that runs an attention item (kv heads x chunks
    of the context) must be on the device at once, because the blocks that are done wait there for the attention row.
    `capacity`: blocks of that kernel the device holds at once (asked of the library when not given)."""
    lib = ffi.load()
    if capacity is None:
        items, cap = C.c_int(0), C.c_int(0)
        check(lib.jsgrad_hip_attn_wo_fits(n_heads, n_kv_heads, head_dim, max_context, kind, dim, C.byref(items), C.byref(cap)))
        return items.value <= cap.value
    return lib.jsgrad_hip_attn_wo_items(n_kv_heads, max_context) <= capacity


class _Scratch:
    """Per-model activation rows and the attention workspace, allocated once (nothing is allocated per token)."""

    def __init__(self, dim: int, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int, vocab: int, dtype: str, device: str):
        self.h = Tensor.empty((dim,), dtype, device)
        self.h2 = Tensor.empty((dim,), dtype, device)
        self.q = Tensor.empty((n_heads * head_dim,), dtype, device)
        self.attn = Tensor.empty((n_heads * head_dim,), dtype, device)
        self.g = Tensor.empty((hidden,), dtype, device)
        self.logits = Tensor.empty((vocab,), dtype, device)
        nbytes = ffi.load().jsgrad_hip_attn_workspace_bytes(n_heads, n_kv_heads, head_dim)
        self.workspace = Tensor.zeros((nbytes,), "uint8", device)
        # attention + wo as one launch (set up by Transformer._prepare when the model qualifies)
        self.fuse_attn_wo = False
        self.attn_wo_ws: Tensor | None = None

    def enable_attn_wo(self, n_heads: int, n_kv_heads: int, head_dim: int, device: str) -> None:
        nbytes = ffi.load().jsgrad_hip_attn_wo_workspace_bytes(n_heads, n_kv_heads, head_dim)
        self.attn_wo_ws = Tensor.zeros((nbytes,), "uint8", device)
        self._tagged_row_bytes = n_heads * head_dim * 4
        self.fuse_attn_wo = True

    def clear_attn_row(self) -> None:
        """Wipe the attention row that the blocks of a fused attention + wo launch hand to each other.  Its words carry a
        16-bit tag made from (position, layer) modulo 65535, unique among CONSECUTIVE launches (each rewrites the whole row);
        after a jump of the position an old row could carry the tag a new launch expects (128 * dpos = dlayer mod 65535), so
        whoever moves the position clears the row: tag 0 matches no launch."""
        if self.attn_wo_ws is not None:
            ws = self.attn_wo_ws
            check(ffi.load().jsgrad_hip_memset(ws.ptr + ws.nbytes - self._tagged_row_bytes, 0, self._tagged_row_bytes))


class _RowScratch:
    """Activations of a several-row call: bsz*seqlen rows (grown on demand, never shrunk)."""

    def __init__(self, bsz: int, seqlen: int, dim: int, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int, vocab: int, device: str):
        n = bsz * seqlen
        self.bsz, self.n = bsz, n
        f16 = "float16"
        self.tokens = Tensor.empty((n,), "int32", device)
        self.h = Tensor.empty((n, dim), f16, device)
        self.h2 = Tensor.empty((n, dim), f16, device)
        self.xn = Tensor.empty((n, dim), f16, device)
        self.q = Tensor.empty((n, n_heads * head_dim), f16, device)
        self.attn = Tensor.empty((n, n_heads * head_dim), f16, device)
        self.g = Tensor.empty((n, hidden), f16, device)
        self.last = Tensor.empty((bsz, dim), f16, device)
        self.logits = Tensor.empty((bsz, vocab), f16, device)
        self.next_tokens = Tensor.empty((bsz,), "int32", device)
        nbytes = ffi.load().jsgrad_hip_attn_batch_workspace_bytes(bsz, n_heads, n_kv_heads, head_dim)
        self.workspace = Tensor.zeros((nbytes,), "uint8", device)

    def fits(self, bsz: int, seqlen: int) -> bool:
        return bsz == self.bsz and bsz * seqlen <= self.n


class _FusedStep:
    """Descriptor of the single-kernel decode step (jsgrad_hip_decode_step): device array of per-layer tensors, the
    activation rows and the workspace.  Built once per model; plays the role of the GraphRunner that replaces a captured
    list of kernels by one device-side program (engine/jit.ts:71)."""

    def __init__(self, model: "Transformer", ctx: "_Scratch", mode: str = "barrier"):
        lib = ffi.load()
        m = model
        self.mode = mode   # "barrier": jsgrad_hip_decode_step; "stream": jsgrad_hip_stream_step
        kinds = {l.kind for blk in m.layers for l in (blk.attention.wq, blk.attention.wk, blk.attention.wv, blk.attention.wo,
                                                      blk.feed_forward.w1, blk.feed_forward.w2, blk.feed_forward.w3)}
        if m.dtype != "float16" or len(kinds) != 1 or next(iter(kinds)) not in (ffi.W_F16, ffi.W_I8) or m.output.kind != next(iter(kinds)):
            raise NotImplementedError("the single-kernel step is built for fp16 activations with fp16 or int8 layers and an lm_head stored the same way")
        hd = m.dim // m.n_heads
        if hd not in (64, 128) or m.n_heads // m.n_kv_heads not in ((1, 2, 4) if mode == "stream" else (1, 2, 3, 4)):
            raise NotImplementedError("the single-kernel step is built for head_dim 64/128 and up to 4 query heads per kv head")
        if mode == "stream" and (m.dim > 4096 or m.max_context > 8192 or len(m.layers) < 1):
            raise NotImplementedError("the streaming step is built for dim <= 4096 and max_context <= 8192")
        arr = (ffi.LayerDesc * len(m.layers))()
        p = lambda t: t.ptr if t is not None else None
        for i, blk in enumerate(m.layers):
            a, f = blk.attention, blk.feed_forward
            half = a.cache_kv.nbytes // 2
            arr[i] = ffi.LayerDesc(a.wq.weight.ptr, a.wk.weight.ptr, a.wv.weight.ptr, a.wo.weight.ptr, f.w1.weight.ptr, f.w2.weight.ptr, f.w3.weight.ptr,
                                   p(a.wq.scale), p(a.wk.scale), p(a.wv.scale), p(a.wo.scale), p(f.w1.scale), p(f.w2.scale), p(f.w3.scale),
                                   blk.attention_norm.weight.ptr, blk.ffn_norm.weight.ptr, a.cache_kv.ptr, a.cache_kv.ptr + half)
        raw = np.frombuffer(bytes(arr), np.uint8) if len(m.layers) else np.zeros(1, np.uint8)
        self.layers = Tensor(raw.copy(), device=m.device)
        nbytes = (lib.jsgrad_hip_stream_workspace_bytes if mode == "stream" else lib.jsgrad_hip_step_workspace_bytes)(m.n_heads, m.n_kv_heads, hd)
        self.workspace = Tensor.zeros((nbytes,), "uint8", m.device)
        emb = m.tok_embeddings
        from .nn import _KIND
        self.desc = ffi.StepDesc(self.layers.ptr, len(m.layers), m.dim, m.hidden_dim, m.n_heads, m.n_kv_heads, hd, m.vocab_size, m.max_context,
                                 m.norm.eps, next(iter(kinds)), m.output.kind, _KIND[emb.weight.dtype], ffi.F16,
                                 emb.weight.ptr, p(emb.scale), m.output.weight.ptr, p(m.output.scale), m.norm.weight.ptr, m.freqs_cis.ptr,
                                 m.state.ptr, m.tokens_out.ptr, m.max_context,
                                 ctx.h.ptr, ctx.h2.ptr, ctx.q.ptr, ctx.attn.ptr, ctx.g.ptr, ctx.logits.ptr, self.workspace.ptr, None)

    def launch(self) -> None:
        lib = ffi.load()
        check((lib.jsgrad_hip_stream_step if self.mode == "stream" else lib.jsgrad_hip_decode_step)(C.byref(self.desc)))

    def error(self) -> int:
        e = C.c_int(0)
        lib = ffi.load()
        check((lib.jsgrad_hip_stream_status if self.mode == "stream" else lib.jsgrad_hip_step_status)(self.workspace.ptr, C.byref(e)))
        return e.value


class TinyJit:
    """Capture-and-replay of one decode step (engine/jit.ts:236-352): call 0 runs eagerly, call 1 runs and is
    captured into a HIP graph, later calls replay the graph."""

    def __init__(self, fxn):
        self.fxn, self.cnt, self.graph = fxn, 0, C.c_void_p()
        self.on_replay = None   # host bookkeeping that the captured function would have done

    def call(self, *args):
        lib = ffi.load()
        if self.cnt == 0:
            ret = self.fxn(*args)
        elif self.cnt == 1:
            check(lib.jsgrad_hip_graph_begin())
            try:
                ret = self.fxn(*args)
            finally:
                check(lib.jsgrad_hip_graph_end(C.byref(self.graph)))
            self._ret = ret
            check(lib.jsgrad_hip_graph_launch(self.graph))   # capture records, it does not execute
        else:
            check(lib.jsgrad_hip_graph_launch(self.graph))
            ret = self._ret
            if self.on_replay is not None:
                self.on_replay()
        self.cnt += 1
        return ret

    def reset(self):
        if self.graph:
            ffi.load().jsgrad_hip_graph_destroy(self.graph)
        self.cnt, self.graph = 0, C.c_void_p()


class Transformer:
    def __init__(self, dim: int, hidden_dim: int, n_heads: int, n_layers: int, norm_eps: float, vocab_size: int, linear=Linear, embedding=Embedding,
                 n_kv_heads: int | None = None, rope_theta: float = 10000, max_context: int = 1024, jit: bool = True, feed_forward=FeedForward, device: str = "HIP",
                 fused_step: bool = False, fuse_attn_wo: bool = True):
        self.dim, self.hidden_dim, self.n_heads, self.vocab_size, self.max_context = dim, hidden_dim, n_heads, vocab_size, max_context
        self.n_kv_heads = n_kv_heads if n_kv_heads is not None else n_heads
        self.rope_theta, self.device = rope_theta, device
        self.layers = [TransformerBlock(dim, hidden_dim, n_heads, n_kv_heads, norm_eps, max_context, linear, feed_forward) for _ in range(n_layers)]
        self.norm = RMSNorm(dim, norm_eps)
        self.tok_embeddings = embedding(vocab_size, dim)
        self.output = Linear(dim, vocab_size, False) if embedding is Embedding else linear(dim, vocab_size, False)
        self.freqs_cis: Tensor | None = None          # built on first use in the activation dtype (llama.ts:198,205)
        self.forward_jit = TinyJit(self._step) if jit else None
        if self.forward_jit is not None:
            self.forward_jit.on_replay = self._advance_host_pos
        self.state = Tensor(np.zeros(2, np.int32), device=device)            # {token, start_pos}
        self.tokens_out = Tensor.zeros((max_context,), "int32", device)      # token produced at each start_pos
        self._ctx: _Scratch | None = None
        self._pos = 0                                                        # host mirror of state[1]
        # False: one launch per fused op (the faster of the two today); True: the whole step as one persistent kernel
        self.fused_step = fused_step
        self.fuse_attn_wo = fuse_attn_wo   # attention and wo of a layer as one launch, where the model qualifies
        self._fused: _FusedStep | None = None
        self._rows: _RowScratch | None = None
        # sampling (llama.ts:131-185): (temperature, top_k, top_p, alpha_f, alpha_p) of the current calls; greedy until told otherwise
        self._sampling = (0.0, 0, 0.0, 0.0, 0.0)
        self.alpha_counter: Tensor | None = None      # llama.ts:130: created on the first call with alpha_f or alpha_p (module-wide in the reference)
        self._sample_ws: Tensor | None = None

    def attn_wo_error(self) -> int:
        """1 if a bounded wait inside a fused attention + wo launch ever ran out (its result is then not to be trusted)."""
        if self._ctx is None or self._ctx.attn_wo_ws is None:
            return 0
        e = C.c_int(0)
        check(ffi.load().jsgrad_hip_attn_wo_status(self._ctx.attn_wo_ws.ptr, C.byref(e)))
        return e.value

    def attn_decode_error(self) -> int:
        """1 if a bounded wait inside a jsgrad_hip_attn_decode launch ran out since the last call (the path of models whose
        attention and wo do not share a launch).  Reading it clears the workspace for further use."""
        if self._ctx is None or self._ctx.fuse_attn_wo:
            return 0
        e = C.c_int(0)
        check(ffi.load().jsgrad_hip_attn_decode_status(self._ctx.workspace.ptr, self.n_heads, self.n_kv_heads, self.dim // self.n_heads, C.byref(e)))
        return e.value

    def check_errors(self) -> None:
        """Raise if a bounded wait inside an attention launch ran out since the model was made (another process holding
        compute units, or a device fault): the tokens after that point are not to be trusted.  Called wherever the host
        waits for the device anyway (the per-token read of Llama3._call, the end of Llama3.generate)."""
        if self.attn_wo_error():
            raise ffi.HipError("a fused attention + wo launch gave up waiting for its attention row; results after that launch are invalid")
        if self.attn_decode_error():
            raise ffi.HipError("an attention launch gave up waiting for its partial results; results after that launch are invalid")


    # ---- plumbing
    @property
    def dtype(self) -> str:
        return self.tok_embeddings.out_dtype

    def _fused_mode(self) -> str:
        return "stream" if self.fused_step == "stream" else "barrier"

    def _prepare(self) -> _Scratch:
        if self._ctx is None:
            hd = self.dim // self.n_heads
            self._ctx = _Scratch(self.dim, self.hidden_dim, self.n_heads, self.n_kv_heads, hd, self.vocab_size, self.dtype, self.device)
            self.freqs_cis = precompute_freqs_cis(hd, self.max_context * 2, self.rope_theta, self.dtype, self.device)
            for i, layer in enumerate(self.layers):
                layer.attention._ensure_cache(self.dtype, self.device)
                layer.attention.layer_id = i
            wo = self.layers[0].attention.wo
            if (self.fuse_attn_wo and self.dtype == "float16" and wo.kind in (ffi.W_F16, ffi.W_I8, ffi.W_NF4) and 2 <= len(self.layers) <= 128 and hd in (64, 128)
                    and self.n_heads // self.n_kv_heads in (1, 2, 3, 4) and self.max_context <= 64 * 128 and self.n_heads * hd * 2 <= 64 * 1024
                    and self.n_kv_heads <= 64 and attn_wo_fits(self.n_heads, self.n_kv_heads, hd, self.max_context, wo.kind, self.dim)):
                self._ctx.enable_attn_wo(self.n_heads, self.n_kv_heads, hd, self.device)
            if self.fused_step:
                self._fused = _FusedStep(self, self._ctx, self._fused_mode())      # raises NotImplementedError for models it was not built for
        return self._ctx

    def _step(self, draw: bool = True) -> Tensor:
        """One decode step for the token / position in `state`; leaves the picked token in state[0] and
        advances state[1].  Pure kernel launches: safe to capture.  draw=False: the token of this position is not wanted
        (an inner position of a several-token call), so nothing is drawn from the random stream; the argmax fills in."""
        ctx = self._prepare()
        if self._pos >= self.max_context:
            raise ValueError(f"KV cache of {self.max_context} positions is full")
        self._pos += 1
        if self._fused is not None:
            self._fused.launch()
            return Tensor(buffer=self.state.lazydata.view(1, "int32", 0), shape=(), dtype="int32", device=self.device)
        h = self.tok_embeddings.call(self.state, out=ctx.h)
        for layer in self.layers:
            h = layer.call(h, self.state, self.freqs_cis, ctx)
        self.output.call(h, out=ctx.logits, norm=self.norm)
        self._pick_token(ctx.logits, draw)
        return Tensor(buffer=self.state.lazydata.view(1, "int32", 0), shape=(), dtype="int32", device=self.device)

    def _pick_token(self, logits: Tensor, draw: bool = True) -> None:
        """`sample(logits.flatten(), ...)` (llama.ts:212): the token goes to state[0], the position advances."""
        lib = ffi.load()
        temp, k, p, af, ap = self._sampling
        if temp < 1e-6 or not draw:
            check(lib.jsgrad_hip_argmax(logits.ptr, self.vocab_size, self.state.ptr, self.tokens_out.ptr, self.max_context, 1, act_code(self.dtype)))
            return
        if self._sample_ws is None:
            self._sample_ws = Tensor.zeros((lib.jsgrad_hip_sample_workspace_bytes(self.vocab_size),), "uint8", self.device)
        if (af or ap) and self.alpha_counter is None:
            self.alpha_counter = Tensor.zeros((self.vocab_size,), "int32", self.device)
        check(lib.jsgrad_hip_sample(logits.ptr, self.vocab_size, act_code(self.dtype), temp, k, p, af, ap,
                                    self.alpha_counter.ptr if self.alpha_counter is not None else None, rng_state(self.device).ptr,
                                    self.state.ptr, self.tokens_out.ptr, self.max_context, 1, self._sample_ws.ptr))

    def _set_sampling(self, temperature: float, top_k: int, top_p: float, alpha_f: float, alpha_p: float) -> None:
        """Argument checks of `sample` (llama.ts:132-134); a change of parameters drops the captured graph, which has them baked in."""
        if temperature >= 1e-6:
            if not 0 <= top_p <= 1:
                raise ValueError("p must be between 0 and 1")
            if not 0 <= top_k <= self.vocab_size:
                raise ValueError("k must be between 0 and numel")
            if self.fused_step:
                raise NotImplementedError("the whole-step kernels end in the greedy argmax; sampling runs on the per-op path")
            new = (float(temperature), int(top_k), float(top_p), float(alpha_f), float(alpha_p))
        else:
            new = (0.0, 0, 0.0, 0.0, 0.0)
        if new != self._sampling:
            self._sampling = new
            if self.forward_jit is not None:
                self.forward_jit.reset()

    def _advance_host_pos(self) -> None:
        self._pos += 1

    def set_state(self, token: int, start_pos: int) -> None:
        if not (0 <= start_pos < self.max_context):
            raise ValueError(f"start_pos {start_pos} outside the KV cache of {self.max_context} positions")
        if not (0 <= token < self.vocab_size):
            raise ValueError(f"token {token} outside the vocabulary of {self.vocab_size}")
        self.state.lazydata.copyin(np.array([token, start_pos], np.int32))
        if start_pos != self._pos and self._ctx is not None:
            self._ctx.clear_attn_row()      # the position jumps: see _Scratch.clear_attn_row
        self._pos = start_pos

    @property
    def logits(self) -> Tensor:
        """lm_head output of the last step, `.float()` of llama.ts:210 left to the caller (`numpy().astype`)."""
        return self._prepare().logits

    # ---- the reference's entry points
    def forward(self, tokens, start_pos: int, temperature: float = 0.0, top_k: int = 0, top_p: float = 0.8, alpha_f: float = 0.0, alpha_p: float = 0.0) -> Tensor:
        """llama.ts:201-213 for one sequence.  Several tokens are fed position by position (the reference's own
        prefill is token-serial, models/llama3.ts:307-311); the returned tensor is the token picked after the last one
        and it is the only draw of the call: the reference samples once, from the logits of the last position
        (llama.ts:210-212), so one call advances the random counter and the alpha counter by one whatever seqlen is.
        Llama3._prefill calls with one token each, so there every position draws, as in the reference)."""
        self._set_sampling(temperature, top_k, top_p, alpha_f, alpha_p)
        toks = np.asarray(tokens.numpy() if isinstance(tokens, Tensor) else tokens, np.int32)
        if toks.ndim != 2 or toks.shape[0] != 1:
            raise ValueError(f"tokens must have shape [1, seqlen], got {toks.shape}; several sequences go through forward_rows")
        ret = None
        n = toks.shape[1]
        for i, t in enumerate(toks[0]):
            self.set_state(int(t), start_pos + i)
            ret = self._step(draw=(i == n - 1))
        return ret

    def forward_rows(self, tokens, start_pos: int, temperature: float = 0.0, top_k: int = 0, top_p: float = 0.8, alpha_f: float = 0.0, alpha_p: float = 0.0) -> Tensor:
        """llama.ts:201-213 for tokens of shape [bsz, seqlen] in ONE pass: every Linear is a matrix-core GEMM over all
        bsz*seqlen rows, attention is causal over cache rows [0, start_pos + s].  Returns the next token of every
        sequence, an int32 tensor [bsz]: for one sequence picked like `forward` does (one draw from the last position's
        logits at temperature > 0), for several the greedy one (the reference flattens the logits of all sequences into
        one sample, llama.ts:212, which is only meaningful for bsz == 1).  fp16 activations; fp16 / int8 / NF4 weights.
        `tokens` may be a device int32 tensor [bsz, seqlen] (e.g. the tensor a previous call returned, reshaped)."""
        lib = ffi.load()
        ctx = self._prepare()
        if self.dtype != "float16":
            raise NotImplementedError("several rows at once are built for fp16 activations; float32 models take one position per call")
        if isinstance(tokens, Tensor):
            if tokens.dtype != "int32" or len(tokens.shape) not in (1, 2):
                raise ValueError(f"tokens must be int32 [bsz, seqlen] (or [bsz] for one position each), got {tokens.dtype} {tokens.shape}")
            bsz, seqlen = tokens.shape if len(tokens.shape) == 2 else (tokens.shape[0], 1)
            tok_dev = tokens
        else:
            toks = np.ascontiguousarray(tokens, np.int32)
            if toks.ndim != 2:
                raise ValueError(f"tokens must have shape [bsz, seqlen], got {toks.shape}")
            if toks.size and (toks.min() < 0 or toks.max() >= self.vocab_size):
                raise ValueError(f"token outside the vocabulary of {self.vocab_size}")
            bsz, seqlen = toks.shape
            tok_dev = None
        if bsz < 1 or seqlen < 1:
            raise ValueError(f"empty token tensor {bsz}x{seqlen}")
        if temperature >= 1e-6 and bsz != 1:
            raise NotImplementedError("sampling is defined for one sequence; several sequences are decoded greedily")
        if not (0 <= start_pos and start_pos + seqlen <= self.max_context):
            raise ValueError(f"positions [{start_pos}, {start_pos + seqlen}) outside the KV cache of {self.max_context} positions")
        hd = self.dim // self.n_heads
        if self._rows is None or not self._rows.fits(bsz, seqlen):
            self._rows = _RowScratch(bsz, seqlen, self.dim, self.hidden_dim, self.n_heads, self.n_kv_heads, hd, self.vocab_size, self.device)
        rows, n = self._rows, bsz * seqlen
        if any(layer.attention.cache_kv.shape[1] != bsz for layer in self.layers):
            for layer in self.layers:
                layer.attention._ensure_cache(self.dtype, self.device, bsz)
            if self.forward_jit is not None:
                self.forward_jit.reset()     # a captured step holds the old cache addresses
            if self._fused is not None:
                self._fused = _FusedStep(self, ctx, self._fused_mode())
        if tok_dev is None:
            rows.tokens.lazydata.view(n, "int32", 0).ensure_allocated().copyin(toks.reshape(-1))
            tok_dev = rows.tokens
        emb = self.tok_embeddings
        from .nn import _KIND
        check(lib.jsgrad_hip_embed_rows(_KIND[emb.weight.dtype], emb.weight.ptr, emb.scale.ptr if emb.scale is not None else None, tok_dev.ptr, n, rows.h.ptr,
                                        self.dim, self.vocab_size))
        # the attention of a one-position call reads the position from the device state word, like the one-row kernels
        self.state.lazydata.ensure_allocated().copyin(np.array([0, start_pos + seqlen - 1], np.int32))
        ctx.clear_attn_row()     # the position moves by more than one: see _Scratch.clear_attn_row
        h = rows.h
        for layer in self.layers:
            h = layer.call_rows(h, bsz, seqlen, start_pos, self.state, self.freqs_cis, rows)
        # logits of the last position of every sequence (llama.ts:210)
        if seqlen == 1:
            last = h
        else:
            for b in range(bsz):
                check(lib.jsgrad_hip_copy(rows.last.ptr + b * self.dim * 2, h.ptr + ((b + 1) * seqlen - 1) * self.dim * 2, self.dim * 2))
            last = rows.last
        out = self.output
        if bsz == 1:
            # one row: the one-row kernels, which also leave {token, start_pos + seqlen} in the state words so that
            # single-position decode continues from here
            if seqlen > 1 and self.vocab_size % 128 == 0 and out.kind != ffi.W_F32:
                # the reference applies the lm_head to all seqlen rows before selecting the last (llama.ts:210), i.e. with
                # the weight expanded over rows: the several-row kernel reproduces that arithmetic for the row that is kept
                check(lib.jsgrad_hip_rmsnorm_rows(last.ptr, self.norm.weight.ptr, rows.xn.ptr, 1, self.dim, self.norm.eps))
                check(lib.jsgrad_hip_gemm(out.kind, out.weight.ptr, out.scale.ptr if out.scale is not None else None, self.vocab_size, self.dim, rows.xn.ptr, 1,
                                          ctx.logits.ptr, None))
            else:
                out.call(Tensor(buffer=last.lazydata.view(self.dim, "float16", 0), shape=(self.dim,), dtype="float16", device=self.device), out=ctx.logits, norm=self.norm)
            self._set_sampling(temperature, top_k, top_p, alpha_f, alpha_p)
            self._pick_token(ctx.logits)
            check(lib.jsgrad_hip_copy(rows.next_tokens.ptr, self.state.ptr, 4))
            self._pos = start_pos + seqlen
        else:
            check(lib.jsgrad_hip_rmsnorm_rows(last.ptr, self.norm.weight.ptr, rows.xn.ptr, bsz, self.dim, self.norm.eps))
            check(lib.jsgrad_hip_gemm(out.kind, out.weight.ptr, out.scale.ptr if out.scale is not None else None, self.vocab_size, self.dim, rows.xn.ptr, bsz,
                                      rows.logits.ptr, None))
            check(lib.jsgrad_hip_argmax_rows(rows.logits.ptr, bsz, self.vocab_size, rows.next_tokens.ptr))
        return Tensor(buffer=rows.next_tokens.lazydata.view(bsz, "int32", 0), shape=(bsz,), dtype="int32", device=self.device)

    def rows_logits(self) -> Tensor:
        """float16 logits [bsz, vocab] of the last forward_rows call (bsz > 1), or the [vocab] row for bsz == 1."""
        return self._rows.logits if self._rows is not None and self._rows.bsz > 1 else self._prepare().logits

    def call(self, tokens, start_pos: int, temperature: float = 0.0, top_k: int = 0, top_p: float = 0.8, alpha_f: float = 0.0, alpha_p: float = 0.0) -> Tensor:
        """llama.ts:214-220: single-token calls past position 0 go through the jit (a captured graph)."""
        toks = np.asarray(tokens.numpy() if isinstance(tokens, Tensor) else tokens, np.int32)
        if toks.shape == (1, 1) and self.forward_jit is not None and start_pos != 0:
            self._set_sampling(temperature, top_k, top_p, alpha_f, alpha_p)
            self.set_state(int(toks[0, 0]), start_pos)
            return self.forward_jit.call()
        return self.forward(toks, start_pos, temperature, top_k, top_p, alpha_f, alpha_p)

    def generate(self, n_steps: int) -> None:
        """Free-running greedy decode: n_steps replays with the token fed back on the device (state[0] -> embedding),
        no host round trip per token.  Tokens land in `tokens_out[start_pos]`."""
        if n_steps <= 0:
            return
        if self.forward_jit is None:
            for _ in range(n_steps):
                self._step()
            return
        if self._pos + n_steps > self.max_context:
            raise ValueError(f"{n_steps} steps from position {self._pos} overrun the KV cache of {self.max_context} positions")
        for _ in range(n_steps):
            self.forward_jit.call()


# *** random numbers of the sampler (tensor.ts:773-843) ***
_SEED = [0]
_RNG: dict[str, Tensor] = {}


def manual_seed(seed: int = 0) -> None:
    """Tensor.manual_seed (tensor.ts:773-775): the seed of the next draws; every device starts over at counter 0."""
    _SEED[0] = int(seed) & 0xFFFFFFFF
    _RNG.clear()


def rng_state(device: str = "HIP") -> Tensor:
    """The device words Tensor.rand works from: {sha256(number of devices seeded before this one) mod 2^32, seed, counter}
    (tensor.ts:813-819), as int32 storage; jsgrad_hip_sample reads them and advances the counter."""
    from .device import Device
    device = Device.canonicalize(device)
    if device not in _RNG:
        import hashlib
        key0 = int.from_bytes(hashlib.sha256(len(_RNG).to_bytes(4, "big")).digest(), "big") % 2 ** 32
        _RNG[device] = Tensor(np.array([key0, _SEED[0], 0], np.uint32).view(np.int32), device=device)
    return _RNG[device]


# *** helpers (llama.ts:222-279) ***

def convert_from_huggingface(weights: dict, n_layers: int, n_heads: int, n_kv_heads: int, permute_layers: bool = True, device: str = "HIP") -> dict[str, Tensor]:
    """models/llama.ts:224-253: Hugging Face key names -> the model's, and q_proj / k_proj rows permuted from the
    rotate-half layout to the interleaved pairs that apply_rotary_emb rotates (on the device, jsgrad_hip_hf_permute).
    `weights`: host arrays (as safe_load returns them) or device Tensors; the result holds device Tensors.

    The reference's key map writes `{l}` instead of `${l}` in the entries for `post_attention_layernorm` and the biases
    (llama.ts:234-235), so there a real checkpoint's ffn_norm weights land under the key `undefined`; here they are mapped
    to `layers.N.ffn_norm.weight`, as every other line of the map (and the function it was translated from) does."""
    from .state import to_device
    lib = ffi.load()
    keymap = {"model.embed_tokens.weight": "tok_embeddings.weight", "model.norm.weight": "norm.weight", "lm_head.weight": "output.weight"}
    for l in range(n_layers):
        keymap[f"model.layers.{l}.input_layernorm.weight"] = f"layers.{l}.attention_norm.weight"
        keymap[f"model.layers.{l}.post_attention_layernorm.weight"] = f"layers.{l}.ffn_norm.weight"
        for x in "qkvo":
            keymap[f"model.layers.{l}.self_attn.{x}_proj.weight"] = f"layers.{l}.attention.w{x}.weight"
            keymap[f"model.layers.{l}.self_attn.{x}_proj.bias"] = f"layers.{l}.attention.w{x}.bias"
        for x, y in (("gate", "1"), ("down", "2"), ("up", "3")):
            keymap[f"model.layers.{l}.mlp.{x}_proj.weight"] = f"layers.{l}.feed_forward.w{y}.weight"
    sd: dict[str, Tensor] = {}
    for k, v in weights.items():
        if ".rotary_emb." in k:
            continue
        if k not in keymap:
            raise KeyError(f"{k} is not a key of a Hugging Face Llama checkpoint with {n_layers} layers")
        t = to_device(v, device)
        if "model.layers" in k and permute_layers and ("q_proj" in k or "k_proj" in k):
            heads = n_heads if "q_proj" in k else n_kv_heads
            if t.ndim != 2:
                raise ValueError(f"{k}: expected a matrix, got shape {t.shape}")
            out = Tensor.empty(t.shape, t.dtype, device)
            check(lib.jsgrad_hip_hf_permute(t.ptr, out.ptr, t.shape[0], t.nbytes // t.shape[0], heads))
            t = out
        sd[keymap[k]] = t
    return sd


def convert_from_gguf(weights: dict[str, Tensor], n_layers: int) -> dict[str, Tensor]:
    """models/llama.ts:255-270: GGUF tensor names -> the model's; the lm_head is the embedding table."""
    keymap = {"token_embd.weight": "tok_embeddings.weight", "output_norm.weight": "norm.weight", "rope_freqs.weight": "rope_freqs.weight"}
    for l in range(n_layers):
        keymap[f"blk.{l}.attn_norm.weight"] = f"layers.{l}.attention_norm.weight"
        keymap[f"blk.{l}.ffn_norm.weight"] = f"layers.{l}.ffn_norm.weight"
        keymap[f"blk.{l}.attn_output.weight"] = f"layers.{l}.attention.wo.weight"
        for x in "qkv":
            keymap[f"blk.{l}.attn_{x}.weight"] = f"layers.{l}.attention.w{x}.weight"
        for x, y in (("gate", "1"), ("down", "2"), ("up", "3")):
            keymap[f"blk.{l}.ffn_{x}.weight"] = f"layers.{l}.feed_forward.w{y}.weight"
    for k in weights:
        if k not in keymap:
            raise KeyError(f"{k} is not a tensor of a GGUF Llama checkpoint with {n_layers} layers")
    sd = {keymap[k]: v for k, v in weights.items()}
    sd["output.weight"] = weights["token_embd.weight"]
    return sd


def fix_bf16(weights: dict[str, Tensor]) -> dict[str, Tensor]:
    """models/llama.ts:272-279: bfloat16 tensors become float16 by way of float32."""
    return {k: (v.cast("float16") if v.dtype == "bfloat16" else v) for k, v in weights.items()}
