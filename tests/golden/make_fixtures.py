"""Writes tests/golden/decode_<case>.npz: what the CPU oracle computes for three seeded random-init models.

The reference (jsgrad) holds no stored vectors for this path and cannot run in the build image, so these are not reference
outputs: they are the oracle's own results, frozen so that a change to the oracle, to the synthetic weight generator or to the
HIP path shows up as a difference against a committed file rather than only against a freshly computed oracle run.
Each file holds the prompt, the greedy tokens of 8 decode steps and the float32 logits at three positions.
Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle as orc                                   # noqa: E402
from denograd_amd import synthetic                     # noqa: E402
from tests.helpers import quantize_state               # noqa: E402

SMALL = dict(dim=512, hidden_dim=1536, n_heads=8, n_kv_heads=2, n_layers=3, vocab_size=2048, norm_eps=1e-5, rope_theta=500000.0, max_context=96, tied=False)
CASES = {
    "tiny-f32": synthetic.config("tiny"),
    "tiny-f16": synthetic.config("tiny16"),
    "small-int8": dict(SMALL, act_dtype="float16", quantize="int8", tied=True, name="small-int8"),
}
PROMPT, STEPS, LOGIT_POSITIONS = 12, 8, (0, 11, 19)


def compute(name):
    cfg = CASES[name]
    sd = quantize_state(cfg, synthetic.random_state_dict(cfg, seed=0, std=0.05))
    cpu = orc.OracleModel(cfg, sd)
    prompt = [int(t) for t in synthetic.random_prompt(cfg, PROMPT, seed=1)]
    toks, logits, feed = [], {}, list(prompt)
    for pos in range(PROMPT + STEPS):
        tok, lg = cpu.forward([feed[pos]], pos)
        if pos in LOGIT_POSITIONS:
            logits[pos] = np.asarray(lg, np.float32).copy()
        if pos >= PROMPT - 1:
            toks.append(int(tok))
            if len(feed) <= pos + 1:
                feed.append(int(tok))
    return {"prompt": np.int32(prompt), "tokens": np.int32(toks[:STEPS + 1]), **{f"logits_{p}": v for p, v in logits.items()}}


if __name__ == "__main__":
    for name in CASES:
        out = os.path.join(os.path.dirname(os.path.abspath(__file__)), f"decode_{name}.npz")
        np.savez_compressed(out, **compute(name))
        print("wrote", out, os.path.getsize(out), "bytes")
