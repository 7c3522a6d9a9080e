"""Weight-only-quantised layers and the user-facing Llama3 runner of
/root/reference/jsgrad/models/llama3.ts on the HIP device.

Int8Linear / Int8Embedding / NF4Linear keep the reference's storage (int8 codes + one fp16 scale per output
row; two 4-bit codes per byte + one fp16 scale per 64 elements) and its quantisers; `call` runs the fused
dequantising GEMV.  Llama3 drives a Transformer the way the reference does: token-serial prefill, greedy
decode, per-token `.item()`; `generate` is the free-running variant that keeps the token on the device.
Downloading checkpoints is out of scope here: a model is built from a state dict
(host arrays), a checkpoint file (.safetensors in the model's or in Hugging Face names, a .safetensors.index.json, a
.gguf with F32 / F16 / Q4_0 / Q4_1 / Q8_0 / Q6_K tensors), or seeded random-init weights made on the device.
"""
from __future__ import annotations

import os
import time

import numpy as np

from . import ffi, synthetic
from .device import DTYPES
from .ffi import check
from .llama import Transformer, convert_from_gguf, convert_from_huggingface, fix_bf16
from .nn import Embedding, Linear, act_code
from .state import gguf_load, load_state_dict, safe_load, to_device
from .tensor import Tensor


class Int8Linear(Linear):
    """llama3.ts:27-61."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False):
        if bias is not False:
            raise ValueError("Int8Linear bias has to be false")
        super().__init__(in_features, out_features, False)

    @staticmethod
    def quantize(tensors: dict[str, Tensor], device=None, scale_dtype: str = "float16", quantize_embeds: bool = False) -> dict[str, Tensor]:
        """llama3.ts:37-60: every `feed_forward` / `attention.w` weight (and the embedding table when asked) becomes
        int8 codes + a `.scale`; with quantised embeddings the lm_head shares the table."""
        if scale_dtype != "float16":
            raise NotImplementedError("scales are fp16 on this device")
        lib = ffi.load()
        new_tensors: dict[str, Tensor] = {}
        for name, v in tensors.items():
            if "feed_forward" in name or "attention.w" in name or (quantize_embeds and "tok_embeddings.weight" in name):
                if "weight" not in name:
                    raise ValueError(name)
                out_f, in_f = v.shape
                codes = Tensor.empty((out_f, in_f), "int8", v.device)
                scale = Tensor.empty((out_f,), "float16", v.device)
                check(lib.jsgrad_hip_int8_quantize(v.ptr, out_f, in_f, codes.ptr, scale.ptr, act_code(v.dtype)))
                new_tensors[name] = codes
                new_tensors[name.replace("weight", "scale")] = scale
            else:
                new_tensors[name] = v
        if quantize_embeds:
            new_tensors["output.weight"] = new_tensors["tok_embeddings.weight"]
            new_tensors["output.scale"] = new_tensors["tok_embeddings.scale"]
        return new_tensors


class Int8Embedding(Embedding):
    """llama3.ts:63-78: int8 table + fp16 row scales; `call` gathers RN16(code * scale[row])."""


def NF4Linear(block_size: int):
    """llama3.ts:79-117; only block_size 64 (what Llama3 uses, llama3.ts:198) is built."""
    if block_size != 64:
        raise NotImplementedError("NF4 kernels are built for block_size 64")

    class _NF4Linear(Linear):
        def __init__(self, in_features: int, out_features: int, bias: bool = False):
            if bias:
                raise ValueError("bias not supported")
            super().__init__(in_features, out_features, False)

        @staticmethod
        def quantize(state_dict: dict[str, Tensor], device=None, scale_dtype: str = "float16") -> dict[str, Tensor]:
            if scale_dtype != "float16":
                raise NotImplementedError("scales are fp16 on this device")
            lib = ffi.load()
            new_state_dict: dict[str, Tensor] = {}
            for k, v in state_dict.items():
                if "feed_forward" in k or "attention.w" in k:
                    n = v.numel
                    packed = Tensor.empty((n // 2,), "uint8", v.device)
                    scale = Tensor.empty((n // block_size, 1), "float16", v.device)
                    check(lib.jsgrad_hip_nf4_quantize(v.ptr, n, packed.ptr, scale.ptr, act_code(v.dtype)))
                    new_state_dict[k] = packed
                    new_state_dict[k.replace(".weight", ".scale")] = scale
                else:
                    new_state_dict[k] = v
            return new_state_dict

    return _NF4Linear


MODEL_PARAMS = {
    "1B": {"args": {"dim": 2048, "n_heads": 32, "n_kv_heads": 8, "n_layers": 16, "norm_eps": 1e-5, "rope_theta": 500000, "vocab_size": 128256, "hidden_dim": 8192}, "files": 1},
    "8B": {"args": {"dim": 4096, "n_heads": 32, "n_kv_heads": 8, "n_layers": 32, "norm_eps": 1e-5, "rope_theta": 500000, "vocab_size": 128256, "hidden_dim": 14336}, "files": 1},
    "70B": {"args": {"dim": 8192, "n_heads": 64, "n_kv_heads": 8, "n_layers": 80, "norm_eps": 1e-5, "rope_theta": 500000, "vocab_size": 128256, "hidden_dim": 28672}, "files": 8},
}


def _classes(quantize: str | None):
    """llama3.ts:193-199."""
    if quantize == "int8":
        return Int8Linear, Int8Embedding, True
    if quantize == "nf4":
        return NF4Linear(64), Embedding, False
    return Linear, Embedding, False


class Llama3:
    """llama3.ts:170-338 without the download / tokenizer plumbing: construct from shape parameters (`size` or an
    explicit `args` dict), load a state dict, then `_prefill` / `_call` / `generate` token ids."""

    def __init__(self, size: str | None = None, quantize: str | None = None, device: str = "HIP", max_context: int = 8192, temperature: float = 0.95,
                 top_k: int = 0, top_p: float = 0.0, alpha_f: float = 0.0, alpha_p: float = 0.0, args: dict | None = None, fused_step: bool = False):
        # quantize: None (tensors as loaded), "float16" (every tensor cast to float16, llama3.ts:234), "int8", "nf4"
        self.cast_float16 = quantize == "float16"
        quantize = None if quantize == "float16" else quantize
        self.size, self.quantize, self.device, self.max_context = size, quantize, device, max_context
        self.temperature, self.top_k, self.top_p, self.alpha_f, self.alpha_p = temperature, top_k, top_p, alpha_f, alpha_p
        self.linear, self.embedding, self.quantize_embeds = _classes(quantize)
        params = dict(MODEL_PARAMS[size]["args"]) if args is None else dict(args)
        self.params = params
        self.model = Transformer(params["dim"], params["hidden_dim"], params["n_heads"], params["n_layers"], params["norm_eps"], params["vocab_size"],
                                 self.linear, self.embedding, params.get("n_kv_heads"), params["rope_theta"], self.max_context, True, device=device,
                                 fused_step=fused_step)
        self.start_pos = 0
        self.tokenizer = None                  # set by load_tokenizer
        self.last_seen_toks: list[int] = []
        # False: prompts are fed one token per call, as the reference does (llama3.ts:307-311).  True: the prompt is one
        # several-position call (matrix-core GEMMs + causal attention), the reference's Transformer.forward on [1, S]
        self.batched_prefill = False

    # ---- loading
    @staticmethod
    def from_config(cfg: dict, device: str = "HIP", fused_step: bool = False, temperature: float = 0.0) -> "Llama3":
        """A model of a synthetic configuration (denograd_amd/synthetic.py).  Greedy unless told otherwise: the parity and
        benchmark runs compare argmax tokens; the constructor itself defaults to the reference's temperature 0.95 (llama3.ts:192)."""
        args = {k: cfg[k] for k in ("dim", "hidden_dim", "n_heads", "n_kv_heads", "n_layers", "norm_eps", "rope_theta", "vocab_size")}
        q = cfg["quantize"] if cfg["quantize"] in ("int8", "nf4") else None
        return Llama3(quantize=q, device=device, max_context=cfg["max_context"], temperature=temperature, args=args, fused_step=fused_step)

    def load_weights(self, weights: dict, quantized: bool = False) -> "Llama3":
        """llama3.ts:233-255: `weights` holds unquantised Meta-style tensors (host arrays or device Tensors) unless
        `quantized` says the codes and scales are already there; quantise per self.quantize, then load."""
        dev = {k: (v if isinstance(v, Tensor) else Tensor(np.ascontiguousarray(v), device=self.device)) for k, v in weights.items()}
        if not quantized:
            if self.quantize == "int8":
                dev = Int8Linear.quantize(dev, self.device, "float16", self.quantize_embeds)
            elif self.quantize == "nf4":
                dev = self.linear.quantize(dev, self.device, "float16")
        load_state_dict(self.model, dev, strict=False)
        return self

    def _load(self, fn: str) -> dict:
        """llama3.ts:201-213: a `.safetensors` file, a `.safetensors.index.json` that names several, or a `.gguf` file."""
        if fn.endswith(".index.json"):
            import json
            with open(fn) as f:
                weight_map = json.load(f)["weight_map"]
            base = os.path.dirname(fn)
            parts = {n: self._load(os.path.join(base, n)) for n in sorted(set(weight_map.values()))}
            return {k: parts[n][k] for k, n in weight_map.items()}
        if fn.endswith(".gguf"):
            return gguf_load(fn, self.device)[1]
        if fn.endswith(".safetensors"):
            return safe_load(fn)
        raise ValueError("invalid file")

    def load(self, fn: str) -> "Llama3":
        """llama3.ts:215-255 from the file on: read, rename (Hugging Face or GGUF names, told apart by their embedding
        key), bfloat16 -> float16, then `quantize == float16` casts every tensor to float16 and the quantised modes
        quantise; tensors of a file already in the model's own names and dtype load as they are."""
        p = self.params
        weights = self._load(fn)
        if "model.embed_tokens.weight" in weights:
            weights = convert_from_huggingface(weights, p["n_layers"], p["n_heads"], p.get("n_kv_heads") or p["n_heads"], device=self.device)
        elif "token_embd.weight" in weights:
            weights = convert_from_gguf(weights, p["n_layers"])
            weights.pop("rope_freqs.weight", None)   # carried through by the reference's map, not a tensor of the model
        weights = fix_bf16({k: to_device(v, self.device) for k, v in weights.items()})
        if self.cast_float16 or self.quantize is not None:
            # the quantisers start from float16 (`v.cast(scale_dtype)`, llama3.ts:42,103); the tensors they leave alone (norms,
            # an unquantised embedding) are cast as well, so that the model has one activation dtype on this device
            weights = {k: (v.cast("float16") if v.dtype == "float32" else v) for k, v in weights.items()}
        return self.load_weights(weights)

    def random_init(self, seed: int = 0, std: float = 0.02, tied: bool = True) -> "Llama3":
        """Seeded N(0, std) weights generated on the device in fp16 (fp32 for a float32 model is not offered here),
        quantised on the device; RMSNorm weights are ones.  For shapes too large to ship from the host."""
        p, sd, i = self.params, {}, 0
        cfg = dict(p, quantize=self.quantize, act_dtype="float16")

        def randn(shape):
            nonlocal i
            i += 1
            return Tensor.randn(shape, "float16", seed * 100003 + i, std, self.device)

        def quantise_one(name, t):
            one = {name: t}
            if self.quantize == "int8":
                return Int8Linear.quantize(one, self.device, "float16", "tok_embeddings" in name and self.quantize_embeds)
            if self.quantize == "nf4":
                return self.linear.quantize(one, self.device, "float16")
            return one

        sd.update({k: v for k, v in quantise_one("tok_embeddings.weight", randn((p["vocab_size"], p["dim"]))).items() if k.startswith("tok_embeddings")})
        for l in range(p["n_layers"]):
            for name, shp in synthetic.linear_shapes(cfg).items():
                sd.update(quantise_one(f"layers.{l}.{name}.weight", randn(shp)))   # the fp16 source is freed right after
            sd[f"layers.{l}.attention_norm.weight"] = Tensor.ones((p["dim"],), "float16", self.device)
            sd[f"layers.{l}.ffn_norm.weight"] = Tensor.ones((p["dim"],), "float16", self.device)
        sd["norm.weight"] = Tensor.ones((p["dim"],), "float16", self.device)
        if self.quantize_embeds or tied:
            sd["output.weight"] = sd["tok_embeddings.weight"]
            if "tok_embeddings.scale" in sd:
                sd["output.scale"] = sd["tok_embeddings.scale"]
        else:
            sd["output.weight"] = randn((p["vocab_size"], p["dim"]))
        load_state_dict(self.model, sd, strict=False)
        return self

    # ---- inference (token ids in, token ids out)
    def _call(self, tok: int) -> int:
        """llama3.ts:334-337: one model call and the per-token device->host read."""
        res = self.model.call(np.array([[tok]], np.int32), self.start_pos, self.temperature, self.top_k, self.top_p, self.alpha_f, self.alpha_p)
        tok = int(res.item())
        self.model.check_errors()
        return tok

    def _prefill(self, toks: list[int]) -> None:
        """llama3.ts:297-312: skip the shared prefix of the previous prompt when starting over, then feed tokens one at a time."""
        toks = [int(t) for t in toks]
        if self.start_pos == 0:
            same = all(a == b for a, b in zip(toks, self.last_seen_toks))
            i = min(len(toks), len(self.last_seen_toks)) if same else 0
            self.start_pos += i
            self.last_seen_toks = toks
            toks = toks[i:]
        if self.batched_prefill and len(toks) > 1:
            self.model.forward_rows(np.array([toks], np.int32), self.start_pos, self.temperature, self.top_k, self.top_p, self.alpha_f, self.alpha_p)
            self.start_pos += len(toks)
            return
        for tok in toks:
            self._call(tok)
            self.start_pos += 1

    # ---- text in, text out (llama3.ts:257-296)
    def load_tokenizer(self, path: str) -> "Llama3":
        """llama3.ts:257: the `tokenizer.model` next to the checkpoint."""
        from .tokenizer import Tokenizer
        self.tokenizer = Tokenizer.llama(path)
        return self

    def _system(self, msg: str = "You are an helpful assistant.") -> None:
        """llama3.ts:266-269: begin_of_text and the system message, fed once; a later chat continues from there."""
        self._prefill([self.tokenizer.bos_id, *self.tokenizer.encode_message("system", msg)])

    def chat(self, messages: list[dict], on_token=None, max_new_tokens: int | None = None) -> dict:
        """llama3.ts:270-296: frame the messages, prefill all but the last prompt token, then decode token by token (with the
        sampler settings of this Llama3) until a stop token.  `max_new_tokens` (not in the reference, which only stops at a
        stop token) bounds the loop; it also stops when the KV cache is full.  Returns the reference's response fields."""
        tk = self.tokenizer
        toks = [t for m in messages for t in tk.encode_message(m["role"], m["content"])] + tk.encode_role("assistant")
        st = time.perf_counter()
        self._prefill(toks[:-1])
        ttft = time.perf_counter() - st
        last, content = toks[-1], ""
        usage = {"input_tokens": len(toks) - 1, "time_to_first_token": ttft, "output_tokens": 0, "tokens_per_second": 0.0}
        st = time.perf_counter()
        while True:
            if self.start_pos >= self.max_context or (max_new_tokens is not None and usage["output_tokens"] >= max_new_tokens):
                return {"stop_reason": "max_tokens", "message": {"role": "assistant", "content": content}, "usage": usage}
            tok = self._call(last)
            self.start_pos += 1
            usage["output_tokens"] += 1
            usage["tokens_per_second"] = usage["output_tokens"] / (time.perf_counter() - st)
            last = tok
            if tok in tk.stop_tokens:
                return {"stop_reason": "end_turn", "message": {"role": "assistant", "content": content}, "usage": usage}
            piece = tk.decode([tok])
            content += piece
            if on_token is not None:
                on_token({"message": {"role": "assistant", "content": content}, "usage": usage, "token": piece})

    def chat_tokens(self, toks: list[int], max_new_tokens: int, stop_tokens=()) -> dict:
        """The loop of Llama3.chat (llama3.ts:270-296) on token ids: prefill all but the last prompt token, then decode
        greedily, syncing once per token as the reference does.  Returns tokens and the reference's usage fields."""
        st = time.perf_counter()
        self._prefill(toks[:-1])
        ttft = time.perf_counter() - st
        last, out = int(toks[-1]), []
        st = time.perf_counter()
        while len(out) < max_new_tokens:
            tok = self._call(last)
            self.start_pos += 1
            out.append(tok)
            last = tok
            if tok in stop_tokens:
                break
        dt = time.perf_counter() - st
        return {"tokens": out, "usage": {"input_tokens": len(toks) - 1, "output_tokens": len(out), "time_to_first_token": ttft,
                                          "tokens_per_second": len(out) / dt if dt > 0 else float("inf")}}

    def generate_batch(self, prompts, n_new: int) -> np.ndarray:
        """Several equally long prompts at once, from position 0: one several-position pass over all prompts, then n_new - 1
        batched decode steps with the tokens fed back on the device.  Returns int32 [bsz, n_new]."""
        prompts = np.ascontiguousarray(prompts, np.int32)
        if prompts.ndim != 2:
            raise ValueError(f"prompts must have shape [bsz, seqlen], got {prompts.shape}")
        bsz, seqlen = prompts.shape
        m = self.model
        hist = Tensor.empty((n_new, bsz), "int32", self.device)
        tok = m.forward_rows(prompts, 0)
        pos = seqlen
        for i in range(n_new):
            check(ffi.load().jsgrad_hip_copy(hist.ptr + i * bsz * 4, tok.ptr, bsz * 4))
            if i + 1 < n_new:
                tok = m.forward_rows(tok, pos)
                pos += 1
        self.start_pos = pos
        return hist.numpy().T.copy()

    def generate(self, prompt, n_new: int) -> np.ndarray:
        """Token-serial prefill, then n_new greedy tokens with the token fed back on the device (no per-token host
        sync); one read of the token history at the end."""
        prompt = [int(t) for t in prompt]
        self._prefill(prompt[:-1])
        first_pos = self.start_pos
        first = self._call(prompt[-1])
        self.start_pos += 1
        if n_new > 1:
            self.model.generate(n_new - 1)
            self.start_pos += n_new - 1
        hist = self.model.tokens_out.numpy()
        self.model.check_errors()
        out = hist[first_pos:first_pos + n_new].astype(np.int32)
        assert out[0] == first
        return out
