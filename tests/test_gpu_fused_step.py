"""The single-kernel decode steps (jsgrad_hip_decode_step: phase-by-phase blocks; jsgrad_hip_stream_step: role-specialised
wavefronts) against the one-launch-per-op path and the oracle: same arithmetic, so the same tokens and (to summation order
inside attention chunks and k-batches) the same logits."""
import numpy as np
import pytest

import oracle as orc
from denograd_amd import synthetic
from denograd_amd.llama3 import Llama3
from tests.helpers import quantize_state
from tests.test_gpu_model import CASES

pytestmark = pytest.mark.gpu
FUSABLE = ["tiny-f16", "small-int8", "small-f16-hd128"]
MODES = [True, "stream"]      # fused_step=True is the barrier kernel


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("name", FUSABLE)
def test_fused_step_equals_per_op_path_and_oracle(name, mode):
    cfg = CASES[name]
    sd = quantize_state(cfg, synthetic.random_state_dict(cfg, seed=0, std=0.02))
    fused = Llama3.from_config(cfg, fused_step=mode).load_weights(sd, quantized=True)
    plain = Llama3.from_config(cfg, fused_step=False).load_weights(sd, quantized=True)
    cpu = orc.OracleModel(cfg, sd)
    prompt = [int(t) for t in synthetic.random_prompt(cfg, 16, seed=1)]
    a = fused.chat_tokens(prompt, 32)["tokens"]
    b = plain.chat_tokens(prompt, 32)["tokens"]
    assert fused.model._fused is not None and plain.model._fused is None
    assert fused.model._fused.mode == ("stream" if mode == "stream" else "barrier")
    assert fused.model._fused.error() == 0, "a bounded wait inside the step kernel ran out"
    assert a == b
    assert a == list(cpu.generate(prompt, 32))
    la, lb = fused.model.logits.numpy().astype(np.float32), plain.model.logits.numpy().astype(np.float32)
    # attention is cut into different chunks on the two paths, so sums differ in their last bits and a few fp16 roundings flip
    assert np.allclose(la, lb, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("mode", MODES)
def test_fused_step_long_context_many_chunks(mode):
    """Several attention chunks per kv head and more items than blocks per head.  Both paths are fed the same tokens
    (teacher forcing): over a thousand free-running steps on near-flat logits the two would part at the first sub-ulp tie."""
    cfg = dict(CASES["tiny-f16"], max_context=1536, name="tiny-f16-long")
    sd = synthetic.random_state_dict(cfg, seed=3, std=0.05)
    fused = Llama3.from_config(cfg, fused_step=mode).load_weights(sd, quantized=True)
    plain = Llama3.from_config(cfg, fused_step=False).load_weights(sd, quantized=True)
    toks = [int(t) for t in synthetic.random_prompt(cfg, 1300, seed=2)]
    agree = 0
    for pos, t in enumerate(toks):
        ta = fused._call(t); fused.start_pos += 1
        tb = plain._call(t); plain.start_pos += 1
        agree += int(ta == tb)
        if pos in (0, 63, 64, 65, 300, 777, 1299):
            la, lb = fused.model.logits.numpy().astype(np.float32), plain.model.logits.numpy().astype(np.float32)
            # logits of magnitude 1-4 are spaced 1e-3..2e-3 apart in fp16: the paths stay within two spacings of each other at
            # every position (no growth with the position), with a mean difference of a third of a spacing
            assert np.allclose(la, lb, rtol=2e-3, atol=3e-3), f"position {pos}"
            assert np.abs(la - lb).mean() < 1e-3, f"position {pos}"
    assert fused.model._fused.error() == 0
    assert agree >= 0.99 * len(toks)


def test_two_streaming_models_in_one_process_keep_their_own_workspaces():
    """Each model owns its workspace (epoch word, flags, attention partials); steps of the two interleave on one stream."""
    cfg = CASES["tiny-f16"]
    sds = [synthetic.random_state_dict(cfg, seed=s, std=0.02) for s in (0, 5)]
    pairs = [(Llama3.from_config(cfg, fused_step="stream").load_weights(sd, quantized=True),
              Llama3.from_config(cfg, fused_step=False).load_weights(sd, quantized=True)) for sd in sds]
    toks = [int(t) for t in synthetic.random_prompt(cfg, 24, seed=4)]
    for t in toks:
        for fused, plain in pairs:
            ta = fused._call(t); fused.start_pos += 1
            tb = plain._call(t); plain.start_pos += 1
            assert ta == tb
    assert all(f.model._fused.error() == 0 for f, _ in pairs)


@pytest.mark.parametrize("mode", MODES)
def test_fused_step_rejects_what_it_was_not_built_for(mode):
    cfg = CASES["small-nf4"]
    sd = quantize_state(cfg, synthetic.random_state_dict(cfg, seed=0))
    llm = Llama3.from_config(cfg, fused_step=mode).load_weights(sd, quantized=True)
    with pytest.raises(NotImplementedError):
        llm._call(1)
    auto = Llama3.from_config(cfg).load_weights(sd, quantized=True)      # default: falls back to one launch per op
    auto._call(1)
    assert auto.model._fused is None


@pytest.mark.parametrize("name", ["tiny-f16", "small-int8", "small-f16-hd128"])
def test_attention_and_wo_in_one_launch_is_bit_identical_to_two(name):
    """jsgrad_hip_attn_wo runs the same arithmetic in the same order as jsgrad_hip_attn_decode + jsgrad_hip_linear(wo)."""
    cfg = dict(CASES[name], max_context=640)
    sd = quantize_state(cfg, synthetic.random_state_dict(cfg, seed=0, std=0.02))
    one = Llama3.from_config(cfg).load_weights(sd, quantized=True)
    two = Llama3.from_config(cfg).load_weights(sd, quantized=True)
    two.model.fuse_attn_wo = False
    toks = [int(t) for t in synthetic.random_prompt(cfg, 300, seed=6)]
    for pos, t in enumerate(toks):
        ta = one._call(t); one.start_pos += 1
        tb = two._call(t); two.start_pos += 1
        assert ta == tb, f"position {pos}"
        if pos in (0, 1, 31, 32, 33, 255, 256, 299):
            assert np.array_equal(one.model.logits.numpy(), two.model.logits.numpy()), f"position {pos}"
    assert one.model._ctx.fuse_attn_wo and not two.model._ctx.fuse_attn_wo
    assert one.model.attn_wo_error() == 0
    # graph replay of the fused launch: positions advance on the device
    p0 = one.start_pos
    one.model.generate(24)
    two.model.generate(24)
    ta, tb = one.model.tokens_out.numpy()[p0:p0 + 24], two.model.tokens_out.numpy()[p0:p0 + 24]
    assert np.array_equal(ta, tb)
    assert np.array_equal(one.model.logits.numpy(), two.model.logits.numpy())
    assert one.model.attn_wo_error() == 0
