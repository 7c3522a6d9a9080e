"""CPU tests of the checkpoint formats: the numpy restatement (oracle/formats.py) against what is published about the
formats, and the host-side parsers (safetensors with bfloat16, GGUF) of the package.  No GPU."""
import json
import os
import struct

import numpy as np
import pytest

from oracle import formats as F
from tests.helpers import ggml_quantize, gguf_write

RNG = np.random.default_rng(20)


def _blocks(typ, nblocks, seed=0):
    """random block bytes with finite, moderate f16 scales"""
    rng = np.random.default_rng(seed)
    ne, nb = F.GGML_BLOCK[typ]
    raw = rng.integers(0, 256, (nblocks, nb), dtype=np.uint8)
    f16 = lambda n: (rng.standard_normal(n) * 0.05).astype(np.float16).view(np.uint8).reshape(n, 2)
    if typ in (2, 8): raw[:, 0:2] = f16(nblocks)
    if typ == 3: raw[:, 0:2], raw[:, 2:4] = f16(nblocks), f16(nblocks)
    if typ == 14: raw[:, 208:210] = f16(nblocks)
    return raw.reshape(-1)


# ---- ggml's own dequantisation loops (ggml-quants.c: dequantize_row_q4_0 / q4_1 / q8_0 / q6_K), element by element
def _ggml_loops(raw, typ):
    ne, nb = F.GGML_BLOCK[typ]
    out = []
    f16 = lambda b: np.float32(np.frombuffer(bytes(b), np.float16)[0])
    for blk in raw.reshape(-1, nb):
        y = np.zeros(ne, np.float32)
        if typ == 2:
            d = f16(blk[0:2])
            for j in range(16):
                y[j] = np.float32((int(blk[2 + j]) & 0xF) - 8) * d
                y[j + 16] = np.float32((int(blk[2 + j]) >> 4) - 8) * d
        elif typ == 3:
            d, m = f16(blk[0:2]), f16(blk[2:4])
            for j in range(16):
                y[j] = np.float32(int(blk[4 + j]) & 0xF) * d + m
                y[j + 16] = np.float32(int(blk[4 + j]) >> 4) * d + m
        elif typ == 8:
            d = f16(blk[0:2])
            for j in range(32):
                y[j] = np.float32(np.int8(blk[2 + j])) * d
        else:
            ql, qh, sc, d = blk[:128], blk[128:192], blk[192:208].view(np.int8), f16(blk[208:210])
            for n in range(2):
                for l in range(32):
                    i_s = l // 16
                    q = [np.int8((int(ql[n * 64 + l]) & 0xF) | (((int(qh[n * 32 + l]) >> 0) & 3) << 4)) - 32,
                         np.int8((int(ql[n * 64 + l + 32]) & 0xF) | (((int(qh[n * 32 + l]) >> 2) & 3) << 4)) - 32,
                         np.int8((int(ql[n * 64 + l]) >> 4) | (((int(qh[n * 32 + l]) >> 4) & 3) << 4)) - 32,
                         np.int8((int(ql[n * 64 + l + 32]) >> 4) | (((int(qh[n * 32 + l]) >> 6) & 3) << 4)) - 32]
                    for k in range(4):
                        y[n * 128 + l + 32 * k] = np.float32(d * np.float32(q[k])) * np.float32(sc[n * 8 + i_s + 2 * k])
        out.append(y)
    return np.concatenate(out)


@pytest.mark.parametrize("typ", [2, 3, 8, 14])
def test_ggml_dequant_restatement_addresses_the_bits_ggml_does(typ):
    """The reference's reshape / transpose chain == ggml's loops, value for value (same float32 products)."""
    raw = _blocks(typ, 7, seed=typ)
    n = 7 * F.GGML_BLOCK[typ][0]
    assert np.array_equal(F.ggml_dequant(raw, n, typ), _ggml_loops(raw, typ))


@pytest.mark.parametrize("typ,steps", [(2, 1.0 / 7), (3, 1.0 / 15), (8, 1.0 / 127), (14, 1.0 / 31)])
def test_ggml_dequant_inverts_a_quantiser(typ, steps):
    """dequant(quant(x)) stays within one code step of x (a quantiser written from the format description alone)."""
    ne = F.GGML_BLOCK[typ][0]
    x = (RNG.standard_normal(ne * 12) * 0.02).astype(np.float32)
    y = F.ggml_dequant(ggml_quantize(x, typ), x.size, typ)
    amax = np.abs(x.reshape(-1, ne)).max(1, keepdims=True)
    span = (x.reshape(-1, ne).max(1, keepdims=True) - x.reshape(-1, ne).min(1, keepdims=True)) if typ == 3 else amax
    assert np.all(np.abs(y.reshape(-1, ne) - x.reshape(-1, ne)) <= span * steps * 1.02 + 1e-6)


def test_ggml_dequant_known_blocks():
    """hand-made blocks with values that can be read off"""
    q8 = np.concatenate([np.array([0.5], np.float16).view(np.uint8), np.arange(-16, 16, dtype=np.int8).view(np.uint8)])
    assert np.array_equal(F.ggml_dequant(q8, 32, 8), 0.5 * np.arange(-16, 16, dtype=np.float32))
    q4 = np.concatenate([np.array([2.0], np.float16).view(np.uint8), np.array([(15 - i) << 4 | i for i in range(16)], np.uint8)])
    want = np.concatenate([2.0 * (np.arange(16) - 8), 2.0 * (15 - np.arange(16) - 8)]).astype(np.float32)
    assert np.array_equal(F.ggml_dequant(q4, 32, 2), want)
    q41 = np.concatenate([np.array([0.25, -1.0], np.float16).view(np.uint8), np.array([(15 - i) << 4 | i for i in range(16)], np.uint8)])
    assert np.array_equal(F.ggml_dequant(q41, 32, 3), np.concatenate([0.25 * np.arange(16) - 1, 0.25 * (15 - np.arange(16)) - 1]).astype(np.float32))
    # Q6_K: all codes 33 (= +1 after the offset), scales 1..16, d = 0.5 -> element e is 0.5 * (1 + e // 16)
    ql = np.full(128, 0x11, np.uint8)           # low nibbles 1
    qh = np.full(64, 0b10101010, np.uint8)      # high pairs 2 -> code 0x21 = 33
    blk = np.concatenate([ql, qh, np.arange(1, 17, dtype=np.int8).view(np.uint8), np.array([0.5], np.float16).view(np.uint8)])
    assert np.array_equal(F.ggml_dequant(blk, 256, 14), 0.5 * (1 + np.arange(256) // 16).astype(np.float32))
    for typ, dt in F.GGML_NATIVE.items():
        a = np.arange(-3, 5).astype(dt)
        assert np.array_equal(F.ggml_dequant(a.view(np.uint8), 8, typ), a)
    with pytest.raises(ValueError, match="not supported"):
        F.ggml_dequant(np.zeros(64, np.uint8), 32, 12)


def test_hf_permute_is_the_rotate_half_to_interleaved_map():
    """What the permutation is FOR pins its direction: rotating the rows of the permuted matrix as interleaved pairs
    (models/llama.ts:17-32) gives the same numbers as rotating the original rows the Hugging Face way (first half /
    second half of a head), up to that same permutation of the outputs."""
    H, hd, in_f = 3, 8, 5
    w = RNG.standard_normal((H * hd, in_f))
    x = RNG.standard_normal(in_f)
    ang = RNG.uniform(0, 6.28, hd // 2)
    c, s = np.cos(ang), np.sin(ang)
    q = (w @ x).reshape(H, hd)
    hf = np.concatenate([q[:, :hd // 2] * c - q[:, hd // 2:] * s, q[:, hd // 2:] * c + q[:, :hd // 2] * s], 1)     # rotate_half form
    qp = (F.hf_permute(w, H) @ x).reshape(H, hd // 2, 2)
    inter = np.stack([qp[..., 0] * c - qp[..., 1] * s, qp[..., 0] * s + qp[..., 1] * c], -1).reshape(H, hd)      # interleaved pairs
    assert np.allclose(inter.reshape(H, hd // 2, 2)[..., 0], hf[:, :hd // 2]) and np.allclose(inter.reshape(H, hd // 2, 2)[..., 1], hf[:, hd // 2:])
    # and the index formula the device kernel uses: output row h*hd + 2i + j is input row h*hd + j*hd/2 + i
    rows = np.arange(H * hd)
    src = (rows // hd) * hd + (rows % hd % 2) * (hd // 2) + (rows % hd) // 2
    assert np.array_equal(F.hf_permute(w, H), w[src])


def test_bf16_to_f16_matches_torch():
    torch = pytest.importorskip("torch")
    bits = np.concatenate([RNG.integers(0, 65536, 4096).astype(np.uint16), np.array([0x0000, 0x8000, 0x7F80, 0xFF80, 0x3F80, 0x0001, 0x477F, 0x4780], np.uint16)])
    want = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float().half().numpy()
    got = F.bf16_to_f16(bits)
    assert np.array_equal(got.view(np.uint16)[~np.isnan(want)], want.view(np.uint16)[~np.isnan(want)])
    assert np.array_equal(np.isnan(got), np.isnan(want))


def test_hf_keymap_covers_a_llama_checkpoint():
    km = F.hf_keymap(2)
    assert km["model.layers.1.post_attention_layernorm.weight"] == "layers.1.ffn_norm.weight"
    assert km["model.layers.0.mlp.down_proj.weight"] == "layers.0.feed_forward.w2.weight"
    assert km["model.layers.0.self_attn.o_proj.weight"] == "layers.0.attention.wo.weight"
    assert len(km) == 3 + 2 * 9


# ---- host-side parsers of the package (no device needed)
def test_safe_load_reads_what_safetensors_wrote(tmp_path):
    torch = pytest.importorskip("torch")
    st = pytest.importorskip("safetensors.torch")
    from denograd_amd.state import is_bf16, safe_load
    t = {"a": torch.randn(3, 5), "b": torch.randn(4, 2).half(), "c": torch.randn(2, 6).bfloat16(), "d": torch.arange(7, dtype=torch.int32), "e": torch.zeros(0, 3)}
    fn = str(tmp_path / "x.safetensors")
    st.save_file(t, fn, metadata={"format": "pt"})
    got = safe_load(fn)
    assert set(got) == set(t)
    for k in "abde":
        assert got[k].shape == tuple(t[k].shape) and np.array_equal(got[k], t[k].numpy())
    assert is_bf16(got["c"]) and not is_bf16(got["b"])
    assert np.array_equal(np.asarray(got["c"]).view(np.uint16), t["c"].view(torch.int16).numpy().view(np.uint16))


def test_gguf_parser_reads_metadata_and_tensor_table(monkeypatch):
    """gguf_load's parsing, with the device step replaced by the numpy restatement (the device kernel has its own test)."""
    from denograd_amd import state
    monkeypatch.setattr(state, "ggml_data_to_tensor", lambda t, n, typ, device="HIP": _HostTensor(F.ggml_dequant(np.asarray(t), n, typ)))
    w = (RNG.standard_normal((4, 64)) * 0.02).astype(np.float32)
    kv = {"general.architecture": "llama", "llama.block_count": 2, "llama.rope.freq_base": 500000.0, "flag": True, "big": 2 ** 40,
          "tokenizer.ggml.tokens": ["a", "bc", "def"], "ints": [1, 2, 3]}
    for align in (None, 64):
        img = gguf_write(kv, {"token_embd.weight": (w, 8), "norm": (np.arange(5, dtype=np.float32), 0), "h": (w, 1), "q6": (np.tile(w, (1, 4)), 14)}, alignment=align)
        meta, sd = state.gguf_load(img)
        assert meta["general.architecture"] == "llama" and meta["llama.block_count"] == 2 and meta["flag"] is True and meta["big"] == 2 ** 40
        assert meta["tokenizer.ggml.tokens"] == ["a", "bc", "def"] and meta["ints"] == [1, 2, 3] and abs(meta["llama.rope.freq_base"] - 5e5) < 1
        assert sd["token_embd.weight"].shape == (4, 64) and sd["q6"].shape == (4, 256) and sd["norm"].shape == (5,)
        assert np.array_equal(sd["norm"].a, np.arange(5, dtype=np.float32))
        assert np.array_equal(sd["h"].a, w.astype(np.float16))
        assert np.max(np.abs(sd["token_embd.weight"].a - w)) <= np.abs(w).max() / 127 * 1.02
        assert np.max(np.abs(sd["q6"].a - np.tile(w, (1, 4)))) <= np.abs(w).max() / 31 * 1.05
    with pytest.raises(ValueError, match="Invalid GGUF"):
        state.gguf_load(b"GGML" + img[4:])
    with pytest.raises(ValueError, match="Invalid GGUF"):
        state.gguf_load(img[:4] + struct.pack("<i", 1) + img[8:])
    with pytest.raises(ValueError, match="ends inside"):
        state.gguf_load(img[:40])


class _HostTensor:
    def __init__(self, a): self.a = np.asarray(a)
    def reshape(self, shape): return _HostTensor(self.a.reshape(shape))
    @property
    def shape(self): return self.a.shape
