"""Checkpoint formats on the device against the numpy restatement (oracle/formats.py), bit for bit, through the C ABI;
and whole checkpoints (Hugging Face safetensors, GGUF) loaded through Llama3.load giving the tokens of the same weights
loaded directly."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from denograd_amd import ffi, synthetic
from denograd_amd.ffi import check
from denograd_amd.llama import convert_from_gguf, convert_from_huggingface, fix_bf16
from denograd_amd.llama3 import Llama3
from denograd_amd.state import BF16, ggml_data_to_tensor, gguf_load, safe_load
from denograd_amd.tensor import Tensor
from oracle import formats as F
from tests.helpers import ggml_quantize, gguf_write
from tests.test_formats import _blocks

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(21)


@pytest.mark.parametrize("typ", [2, 3, 8, 14])
@pytest.mark.parametrize("nblocks", [1, 3, 2049])
def test_ggml_dequant_kernel_equals_restatement(hip, typ, nblocks):
    ne, nb = F.GGML_BLOCK[typ]
    raw = _blocks(typ, nblocks, seed=100 + typ)
    if nblocks == 3:     # scales that are not ordinary numbers: inf, nan, zero, subnormal
        raw.reshape(-1, nb)[0, (208 if typ == 14 else 0):(210 if typ == 14 else 2)] = np.array([np.inf], np.float16).view(np.uint8)
        raw.reshape(-1, nb)[1, (208 if typ == 14 else 0):(210 if typ == 14 else 2)] = np.array([6e-8], np.float16).view(np.uint8)
    n = nblocks * ne
    assert hip.jsgrad_hip_ggml_nbytes(typ, n) == raw.size
    src, out = Tensor(raw), Tensor.empty((n,), "float32")
    check(hip.jsgrad_hip_ggml_dequant(typ, src.ptr, n, out.ptr))
    want = F.ggml_dequant(raw, n, typ)
    got = out.numpy()
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.array_equal(np.isnan(got), np.isnan(want))


def test_ggml_dequant_errors_and_empty(hip):
    src, out = Tensor(np.zeros(256, np.uint8)), Tensor.empty((256,), "float32")
    check(hip.jsgrad_hip_ggml_dequant(8, src.ptr, 0, out.ptr))                      # nothing to do
    assert hip.jsgrad_hip_ggml_dequant(12, src.ptr, 32, out.ptr) != 0 and b"not supported" in hip.jsgrad_hip_last_error()
    assert hip.jsgrad_hip_ggml_dequant(14, src.ptr, 32, out.ptr) != 0               # not a whole Q6_K block
    assert hip.jsgrad_hip_ggml_dequant(8, src.ptr + 1, 32, out.ptr) != 0            # odd address
    assert hip.jsgrad_hip_ggml_nbytes(12, 32) == 0
    with pytest.raises(ValueError, match="whole blocks"):
        ggml_data_to_tensor(np.zeros(100, np.uint8), 256, 14)
    with pytest.raises(ValueError, match="not supported"):
        ggml_data_to_tensor(np.zeros(100, np.uint8), 32, 12)


def test_casts(hip):
    torch = pytest.importorskip("torch")
    x = np.concatenate([(RNG.standard_normal(5000) * 10 ** RNG.uniform(-8, 5, 5000)).astype(np.float32), np.float32([0, -0.0, 65504, 65520, 65519.99, 1e-8, 5.96e-8, 2.98e-8, np.inf, -np.inf])])
    t = Tensor(x)
    with np.errstate(over="ignore"):
        assert np.array_equal(t.cast("float16").numpy().view(np.uint16), x.astype(np.float16).view(np.uint16))      # round to nearest even, overflow to inf
    assert t.cast("float32") is t
    with np.errstate(over="ignore"):
        h = x.astype(np.float16)
    assert np.array_equal(Tensor(h).cast("float32").numpy(), h.astype(np.float32))
    bits = np.concatenate([RNG.integers(0, 65536, 4096).astype(np.uint16), np.array([0, 0x8000, 0x7F80, 0xFF80, 0x3F80, 1, 0x477F, 0x4780], np.uint16)])
    tb = Tensor(bits, dtype="bfloat16")
    want = F.bf16_to_f16(bits)
    got = tb.cast("float16").numpy()
    assert np.array_equal(got.view(np.uint16)[~np.isnan(want)], want.view(np.uint16)[~np.isnan(want)]) and np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(tb.cast("float32").numpy().view(np.uint32), bits.astype(np.uint32) << 16)
    assert fix_bf16({"a": tb, "b": t})["a"].dtype == "float16" and fix_bf16({"a": tb, "b": t})["b"] is t
    with pytest.raises(NotImplementedError):
        Tensor(np.arange(4, dtype=np.int32)).cast("float16")


@pytest.mark.parametrize("dtype", ["float16", "float32"])
def test_hf_permute_kernel(hip, dtype):
    H, hd, in_f = 6, 64, 200
    w = RNG.standard_normal((H * hd, in_f)).astype(dtype)
    out = Tensor.empty(w.shape, dtype)
    check(hip.jsgrad_hip_hf_permute(Tensor(w).ptr, out.ptr, H * hd, in_f * w.itemsize, H))
    assert np.array_equal(out.numpy(), F.hf_permute(w, H))
    assert hip.jsgrad_hip_hf_permute(out.ptr, out.ptr, H * hd, in_f * w.itemsize, H) != 0       # in place
    assert hip.jsgrad_hip_hf_permute(Tensor(w).ptr, out.ptr, H * hd, in_f * w.itemsize, 7) != 0   # rows do not divide into heads


# ---- whole checkpoints
CFG = dict(synthetic.config("tiny16"))


def _tokens(llm, n=12):
    prompt = [int(t) for t in synthetic.random_prompt(CFG, 6, seed=3)]
    return llm.chat_tokens(prompt, n)["tokens"]


def _to_hf(sd, cfg):
    """the model's own layout -> Hugging Face names and rotate-half rows (the inverse of what the loader does)"""
    inv = {v: k for k, v in F.hf_keymap(cfg["n_layers"]).items()}
    out = {}
    for k, v in sd.items():
        v = np.asarray(v)
        if ".attention.wq." in k or ".attention.wk." in k:
            heads = cfg["n_heads"] if ".wq." in k else cfg["n_kv_heads"]
            hd = v.shape[0] // heads
            v = v.reshape(heads, hd // 2, 2, v.shape[1]).swapaxes(1, 2).reshape(v.shape)
        out[inv[k]] = v
    return out


@pytest.mark.parametrize("store", ["float16", "bfloat16", "sharded"])
def test_hugging_face_checkpoint_loads_to_the_same_model(tmp_path, store):
    torch = pytest.importorskip("torch")
    st = pytest.importorskip("safetensors.torch")
    sd = synthetic.random_state_dict(CFG, seed=5, std=0.05)
    if store == "bfloat16":   # values a bfloat16 holds exactly, so that both ways of loading see the same numbers
        sd = {k: torch.from_numpy(np.asarray(v, np.float32)).bfloat16().float().numpy().astype(np.float16) for k, v in sd.items()}
    direct = Llama3.from_config(CFG).load_weights(sd)
    hf = {k: torch.from_numpy(np.ascontiguousarray(v)) for k, v in _to_hf(sd, CFG).items()}
    if store == "bfloat16":
        hf = {k: v.float().bfloat16() for k, v in hf.items()}
    hf["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(4)      # present in old checkpoints, skipped by the loader
    if store == "sharded":
        names = sorted(hf)
        parts = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
        for fn, keys in parts.items():
            st.save_file({k: hf[k] for k in keys}, str(tmp_path / fn))
        path = str(tmp_path / "model.safetensors.index.json")
        with open(path, "w") as f:
            json.dump({"weight_map": {k: fn for fn, keys in parts.items() for k in keys}}, f)
    else:
        path = str(tmp_path / "model.safetensors")
        st.save_file(hf, path)
    loaded = Llama3.from_config(CFG).load(path)
    assert loaded.model.dtype == "float16"
    for k in ("layers.1.attention.wq.weight", "layers.0.attention.wk.weight", "layers.1.ffn_norm.weight", "output.weight"):
        from denograd_amd.state import get_state_dict
        assert np.array_equal(get_state_dict(loaded.model)[k].numpy(), get_state_dict(direct.model)[k].numpy()), k
    assert _tokens(loaded) == _tokens(direct)


def test_gguf_checkpoint_loads_to_the_same_model(tmp_path):
    sd = synthetic.random_state_dict(CFG, seed=6, std=0.05)
    inv = {"tok_embeddings.weight": "token_embd.weight", "norm.weight": "output_norm.weight"}
    for l in range(CFG["n_layers"]):
        inv[f"layers.{l}.attention_norm.weight"] = f"blk.{l}.attn_norm.weight"
        inv[f"layers.{l}.ffn_norm.weight"] = f"blk.{l}.ffn_norm.weight"
        inv[f"layers.{l}.attention.wo.weight"] = f"blk.{l}.attn_output.weight"
        for x in "qkv":
            inv[f"layers.{l}.attention.w{x}.weight"] = f"blk.{l}.attn_{x}.weight"
        for x, y in (("gate", "1"), ("down", "2"), ("up", "3")):
            inv[f"layers.{l}.feed_forward.w{y}.weight"] = f"blk.{l}.ffn_{x}.weight"
    types = {"token_embd.weight": 14, "output_norm.weight": 0}
    tensors = {}
    for k, v in sd.items():
        if k == "output.weight":
            continue                                  # GGUF Llama checkpoints tie the lm_head to the embedding table
        name = inv[k]
        typ = types.get(name, 0 if "norm" in name else (14 if "ffn" in name else 8 if "attn_q" in name or "attn_k" in name else 2 if "attn_v" in name else 3))
        tensors[name] = (np.asarray(v, np.float32), typ)
    tensors["rope_freqs.weight"] = (np.ones(CFG["dim"] // CFG["n_heads"] // 2, np.float32), 0)
    path = str(tmp_path / "model.gguf")
    with open(path, "wb") as f:
        f.write(gguf_write({"general.architecture": "llama", "llama.block_count": CFG["n_layers"]}, tensors))
    # what the file holds, dequantised by the numpy restatement, loaded directly
    want = {}
    for name, (arr, typ) in tensors.items():
        raw = arr.astype(F.GGML_NATIVE[typ]).view(np.uint8).reshape(-1) if typ in F.GGML_NATIVE else ggml_quantize(arr, typ)
        want[name] = F.ggml_dequant(raw, arr.size, typ).reshape(arr.shape)
    kv, dev = gguf_load(path)
    assert kv["llama.block_count"] == CFG["n_layers"]
    for name in tensors:
        assert dev[name].shape == tensors[name][0].shape and np.array_equal(dev[name].numpy(), want[name]), name
    direct_sd = {k: want[inv[k]].astype(np.float16) for k in sd if k != "output.weight"}
    direct_sd["output.weight"] = direct_sd["tok_embeddings.weight"]
    direct = Llama3.from_config(CFG).load_weights(direct_sd)
    loaded = Llama3(quantize="float16", temperature=0.0, max_context=CFG["max_context"], args={k: CFG[k] for k in ("dim", "hidden_dim", "n_heads", "n_kv_heads", "n_layers", "norm_eps", "rope_theta", "vocab_size")}).load(path)
    assert loaded.model.dtype == "float16"
    assert _tokens(loaded) == _tokens(direct)
    # and through the int8 quantiser: the same codes as quantising the dequantised values directly
    q_loaded = Llama3(quantize="int8", temperature=0.0, max_context=CFG["max_context"], args=loaded.params).load(path)
    q_direct = Llama3(quantize="int8", temperature=0.0, max_context=CFG["max_context"], args=loaded.params).load_weights(direct_sd)
    assert _tokens(q_loaded) == _tokens(q_direct)
