"""The committed vectors under tests/golden/ (frozen results of the CPU oracle, see make_fixtures.py there).

CPU: the oracle of this tree still reproduces them bit for bit (a change to the oracle or to the synthetic weights is
deliberate or it is a regression).  GPU: the HIP path, fed the same prompt, produces the same greedy tokens and logits
within the north-star tolerance of the stored ones."""
import importlib.util
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
mk = importlib.util.module_from_spec(spec)
spec.loader.exec_module(mk)


def load(name):
    with np.load(os.path.join(HERE, "golden", f"decode_{name}.npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("name", list(mk.CASES))
def test_oracle_reproduces_the_committed_vectors(name):
    want, got = load(name), mk.compute(name)
    assert sorted(want) == sorted(got)
    for k in want:
        assert np.array_equal(want[k], got[k]), f"{name}: {k}"


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(mk.CASES))
def test_hip_path_against_the_committed_vectors(name):
    from denograd_amd import synthetic
    from denograd_amd.llama3 import Llama3
    from tests.helpers import quantize_state
    cfg, want = mk.CASES[name], load(name)
    sd = quantize_state(cfg, synthetic.random_state_dict(cfg, seed=0, std=0.05))
    llm = Llama3.from_config(cfg).load_weights(sd, quantized=True)
    tol = 1e-2 if cfg["act_dtype"] == "float16" else 1e-4
    feed, toks = [int(t) for t in want["prompt"]], []
    for pos in range(mk.PROMPT + mk.STEPS):
        tok = llm._call(feed[pos]); llm.start_pos += 1
        if pos in mk.LOGIT_POSITIONS:
            lg, ref = llm.model.logits.numpy().astype(np.float32), want[f"logits_{pos}"]
            assert np.allclose(lg, ref, rtol=tol, atol=tol), f"{name}: logits at position {pos}"
        if pos >= mk.PROMPT - 1:
            toks.append(int(tok))
            if len(feed) <= pos + 1:
                feed.append(int(want["tokens"][len(toks) - 1]))     # teacher forcing with the stored token
    assert toks[:mk.STEPS + 1] == [int(t) for t in want["tokens"]], name
