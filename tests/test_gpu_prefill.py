"""End-to-end parity of the several-position / several-sequence path (Transformer.forward on tokens [B, S] in one pass:
matrix-core GEMMs, causal attention, batched decode) against the CPU oracle's several-row forward, which realises
quantised weights in fp16 first as the reference does when a weight is expanded over rows.

Bars: logits within rtol/atol 1e-2 of the oracle's (north star, fp16); KV cache rows within the same tolerance; greedy
tokens identical unless the oracle's own top-2 logits are within 2 fp16 ulp; decoding on from a batched prefill gives
what decoding on from the token-serial prefill gives."""
import numpy as np
import pytest

import oracle as orc
from denograd_amd import ffi, synthetic
from denograd_amd.llama3 import Llama3
from tests.helpers import quantize_state

pytestmark = pytest.mark.gpu

SMALL = dict(dim=512, hidden_dim=1536, n_heads=8, n_kv_heads=2, n_layers=3, vocab_size=2048, norm_eps=1e-5, rope_theta=500000.0, max_context=320, tied=False)
CASES = {
    "tiny-f16": dict(synthetic.config("tiny16"), max_context=320),
    "small-int8": dict(SMALL, act_dtype="float16", quantize="int8", tied=True, name="small-int8"),
    "small-nf4": dict(SMALL, act_dtype="float16", quantize="nf4", name="small-nf4"),
    "small-f16-hd128": dict(SMALL, n_heads=4, n_kv_heads=4, act_dtype="float16", quantize="float16", name="small-f16-hd128"),
}


def build(name, seed=0):
    cfg = CASES[name]
    sd = quantize_state(cfg, synthetic.random_state_dict(cfg, seed=seed, std=0.02))
    return cfg, sd, Llama3.from_config(cfg).load_weights(sd, quantized=True), orc.OracleModel(cfg, sd)


def check_token(tok_g, tok_c, lg_c, what):
    if tok_g != tok_c:
        gap = lg_c[tok_c] - lg_c[tok_g]
        ulp = float(np.spacing(np.float16(abs(lg_c[tok_c]))))
        assert 0 <= gap <= 2 * ulp, f"{what}: token {tok_g} != {tok_c} with an oracle gap of {gap / ulp:.1f} ulp"


def cache_rows(gpu, layer, b, n):
    c = gpu.model.layers[layer].attention.cache_kv.numpy().astype(np.float32)     # [2, B, ctx, KV, hd]
    return c[0, b, :n], c[1, b, :n]


@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("S", [2, 37, 200])
def test_one_pass_prefill_matches_oracle(name, S):
    cfg, sd, gpu, cpu = build(name)
    prompt = synthetic.random_prompt(cfg, S, seed=S)
    tok_c, lg_c = cpu.forward(prompt, 0)
    tok_g = int(gpu.model.forward_rows(np.array([prompt], np.int32), 0).numpy()[0])
    lg_g = gpu.model.logits.numpy().astype(np.float32)
    assert np.allclose(lg_g, lg_c, rtol=1e-2, atol=1e-2), f"{name} S={S}: max |dlogit| {np.max(np.abs(lg_g - lg_c))}"
    check_token(tok_g, tok_c, lg_c, f"{name} S={S}")
    for layer in (0, cfg["n_layers"] - 1):
        k_g, v_g = cache_rows(gpu, layer, 0, S)
        assert np.allclose(k_g, cpu.cache_k[layer, :S], rtol=1e-2, atol=1e-2) and np.allclose(v_g, cpu.cache_v[layer, :S], rtol=1e-2, atol=1e-2)
    # the state words are left for single-position decode to continue
    assert list(gpu.model.state.numpy()) == [tok_g, S]


@pytest.mark.parametrize("name", ["tiny-f16", "small-int8"])
def test_chunked_prefill_with_a_start_position(name):
    """Two several-position calls, the second starting where the first ended, against the oracle doing the same."""
    cfg, sd, gpu, cpu = build(name)
    prompt = synthetic.random_prompt(cfg, 150, seed=9)
    cpu.forward(prompt[:70], 0)
    tok_c, lg_c = cpu.forward(prompt[70:], 70)
    gpu.model.forward_rows(np.array([prompt[:70]], np.int32), 0)
    tok_g = int(gpu.model.forward_rows(np.array([prompt[70:]], np.int32), 70).numpy()[0])
    lg_g = gpu.model.logits.numpy().astype(np.float32)
    assert np.allclose(lg_g, lg_c, rtol=1e-2, atol=1e-2)
    check_token(tok_g, tok_c, lg_c, name)


@pytest.mark.parametrize("name", ["tiny-f16", "small-int8", "small-nf4"])
def test_decode_after_one_pass_prefill_follows_the_oracle(name):
    """Batched prefill, then 24 single-position decode steps (graph replay), teacher-forced with the oracle's tokens."""
    cfg, sd, gpu, cpu = build(name)
    gpu.batched_prefill = True
    prompt = [int(t) for t in synthetic.random_prompt(cfg, 41, seed=4)]
    cpu.forward(prompt[:-1], 0)
    gpu._prefill(prompt[:-1])
    assert gpu.start_pos == 40
    t, near = prompt[-1], 0
    for pos in range(40, 64):
        tok_c, lg_c = cpu.forward([t], pos)
        tok_g = gpu._call(t); gpu.start_pos += 1
        lg_g = gpu.model.logits.numpy().astype(np.float32)
        assert np.allclose(lg_g, lg_c, rtol=1e-2, atol=1e-2), f"{name}: logits differ at position {pos}"
        check_token(tok_g, tok_c, lg_c, f"{name} pos {pos}")
        near += tok_g != tok_c
        t = tok_c
    assert near <= 2


@pytest.mark.parametrize("name", ["tiny-f16", "small-int8", "small-f16-hd128"])
def test_batched_sequences_match_the_oracle_one_by_one(name):
    """B = 3 sequences: one several-position pass over all prompts, then batched one-position decode steps, teacher-forced
    per sequence with the oracle's tokens.  The oracle runs each sequence on its own with `batched` set."""
    cfg, sd, gpu, _ = build(name)
    B, S, steps = 3, 21, 6
    prompts = np.stack([synthetic.random_prompt(cfg, S, seed=30 + b) for b in range(B)]).astype(np.int32)
    cpus = [orc.OracleModel(cfg, sd) for _ in range(B)]
    for c in cpus:
        c.set_batched(True)
    ref = [c.forward(prompts[b], 0) for b, c in enumerate(cpus)]
    tok = gpu.model.forward_rows(prompts, 0).numpy()
    lg = gpu.model.rows_logits().numpy().astype(np.float32)
    for b in range(B):
        assert np.allclose(lg[b], ref[b][1], rtol=1e-2, atol=1e-2), f"{name}: sequence {b} prefill logits"
        check_token(int(tok[b]), ref[b][0], ref[b][1], f"{name} seq {b}")
    feed = np.array([r[0] for r in ref], np.int32)
    for i in range(steps):
        pos = S + i
        ref = [c.forward([int(feed[b])], pos) for b, c in enumerate(cpus)]
        tok = gpu.model.forward_rows(feed.reshape(B, 1), pos).numpy()
        lg = gpu.model.rows_logits().numpy().astype(np.float32)
        for b in range(B):
            assert np.allclose(lg[b], ref[b][1], rtol=1e-2, atol=1e-2), f"{name}: sequence {b} decode logits at {pos}"
            check_token(int(tok[b]), ref[b][0], ref[b][1], f"{name} seq {b} pos {pos}")
        feed = np.array([r[0] for r in ref], np.int32)
    k_g, v_g = cache_rows(gpu, 1, 2, S + steps)
    assert np.allclose(k_g, cpus[2].cache_k[1, :S + steps], rtol=1e-2, atol=1e-2)


def test_generate_batch_equals_sequences_run_alone():
    """Size-independent property: a sequence decoded inside a batch gives the tokens it gives as a batch of one copy of
    itself (same kernels, same rows arithmetic), and all copies of one prompt in a batch agree."""
    cfg, sd, gpu, _ = build("small-int8")
    p = synthetic.random_prompt(cfg, 33, seed=77).astype(np.int32)
    q = synthetic.random_prompt(cfg, 33, seed=78).astype(np.int32)
    out = gpu.generate_batch(np.stack([p, q, p, p]), 12)
    assert out.shape == (4, 12)
    assert np.array_equal(out[0], out[2]) and np.array_equal(out[0], out[3])
    two = gpu.generate_batch(np.stack([q, p]), 12)
    assert np.array_equal(two[0], out[1]) and np.array_equal(two[1], out[0])


def test_rows_path_rejects_what_it_was_not_built_for():
    cfg = synthetic.config("tiny")      # float32 activations
    sd = synthetic.random_state_dict(cfg, seed=0)
    gpu = Llama3.from_config(cfg).load_weights(sd, quantized=True)
    with pytest.raises(NotImplementedError, match="fp16 activations"):
        gpu.model.forward_rows(np.zeros((1, 4), np.int32), 0)
    cfg, sd, gpu, _ = build("tiny-f16")
    with pytest.raises(ValueError, match="KV cache"):
        gpu.model.forward_rows(np.zeros((1, 8), np.int32), cfg["max_context"] - 4)
    with pytest.raises(ValueError, match="vocabulary"):
        gpu.model.forward_rows(np.full((1, 4), cfg["vocab_size"], np.int32), 0)
