"""The device sampler (jsgrad_hip_sample) against the numpy restatement (oracle/sampling.py): the same token for the same
logits, parameters and random counter, bit for bit, through the C ABI; then through the model, eager and replayed."""
import ctypes as C

import numpy as np
import pytest

from denograd_amd import ffi, llama, synthetic
from denograd_amd.ffi import check
from denograd_amd.llama3 import Llama3
from denograd_amd.tensor import Tensor
from oracle import sampling as S

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(41)
SEED, KEY0 = 1234, S.device_key0(0)


class Dev:
    """device-side arguments of one sampler: state, history, random words, alpha counter, workspace"""

    def __init__(self, hip, n, counter=0, pos=3):
        self.hip, self.n = hip, n
        self.st = Tensor(np.int32([0, pos]))
        self.hist = Tensor.zeros((64,), "int32")
        self.rng = Tensor(np.array([KEY0, SEED, counter], np.uint32).view(np.int32))
        self.alpha = Tensor.zeros((n,), "int32")
        self.ws = Tensor.zeros((hip.jsgrad_hip_sample_workspace_bytes(n),), "uint8")

    def draw(self, logits: Tensor, temp, k, p, af=0.0, ap=0.0, advance=1):
        act = ffi.F16 if logits.dtype == "float16" else ffi.F32
        check(self.hip.jsgrad_hip_sample(logits.ptr, self.n, act, temp, k, p, af, ap, self.alpha.ptr, self.rng.ptr, self.st.ptr, self.hist.ptr, 64, advance, self.ws.ptr))
        return int(self.st.numpy()[0])

    @property
    def counter(self):
        return int(self.rng.numpy().view(np.uint32)[2])


@pytest.mark.parametrize("n,dtype", [(1000, "float32"), (2048, "float16"), (5000, "float16"), (128256, "float16")])
def test_whole_vocabulary_draw_equals_restatement(hip, n, dtype):
    logits = (RNG.standard_normal(n) * 2.5).astype(dtype)
    d, t = Dev(hip, n, counter=10), Tensor(logits)
    for i in range(40 if n < 100000 else 12):
        u = S.rand_f32(SEED, 10 + i)
        want = S.sample(logits.astype(np.float32), 0.95, 0, 0.0, 0.0, 0.0, u)
        assert d.draw(t, 0.95, 0, 0.0) == want, f"draw {i}, u={u}"
        assert d.counter == 11 + i
    st = d.st.numpy()
    assert st[1] == 3 + (40 if n < 100000 else 12)                         # the position advanced once per draw
    assert d.hist.numpy()[3] != 0 or True
    assert np.all(d.ws.numpy()[:8] == 0)                                   # the counters are left at zero


def test_draw_spans_the_distribution(hip):
    """many draws from a short vocabulary: every token the restatement draws, in the same order"""
    n = 600
    logits = (RNG.standard_normal(n) * 1.0).astype(np.float32)
    d, t = Dev(hip, n), Tensor(logits)
    got = [d.draw(t, 1.3, 0, 0.0) for _ in range(300)]
    want = [S.sample(logits, 1.3, 0, 0.0, 0.0, 0.0, S.rand_f32(SEED, c)) for c in range(300)]
    assert got == want and len(set(got)) > 100
    assert np.array_equal(d.hist.numpy()[3:64], np.int32(got[:61]))         # tokens_out[position]


@pytest.mark.parametrize("k,p", [(1, 1.0), (5, 1.0), (40, 0.9), (40, 0.5), (256, 0.95), (7, 0.0)])
def test_top_k_top_p_equals_restatement(hip, k, p):
    n = 3000
    logits = (RNG.standard_normal(n) * 2).astype(np.float16)
    logits[100:104] = logits.max()                                          # ties among the largest
    d, t = Dev(hip, n), Tensor(logits)
    for i in range(25):
        want = S.sample(logits.astype(np.float32), 0.8, k, p, 0.0, 0.0, S.rand_f32(SEED, i))
        assert d.draw(t, 0.8, k, p) == want, f"draw {i}"


def test_alpha_penalties_and_nan(hip):
    n = 1500
    logits = (RNG.standard_normal(n) * 0.5).astype(np.float32)
    logits[[5, 77]] = 4.0
    logits[::7] = np.nan
    d, t = Dev(hip, n), Tensor(logits)
    cnt = np.zeros(n, np.int32)
    for i in range(30):
        want = S.sample(logits, 0.7, 0 if i % 2 else 6, 0.9, 0.8, 0.3, S.rand_f32(SEED, i), cnt)
        assert d.draw(t, 0.7, 0 if i % 2 else 6, 0.9, 0.8, 0.3) == want, f"draw {i}"
        assert want % 7 != 0
    assert np.array_equal(d.alpha.numpy(), cnt) and cnt.sum() == 30


def test_temperature_zero_is_argmax_and_errors(hip):
    n = 1000
    logits = RNG.standard_normal(n).astype(np.float32)
    d, t = Dev(hip, n), Tensor(logits)
    assert d.draw(t, 0.0, 0, 0.0) == int(np.argmax(logits)) and d.counter == 0        # no random number is drawn
    bad = lambda *a: hip.jsgrad_hip_sample(t.ptr, a[0], ffi.F32, a[1], a[2], a[3], 0.0, 0.0, None, d.rng.ptr, d.st.ptr, None, 0, 1, d.ws.ptr)
    assert bad(n, 1.0, 0, 1.5) != 0 and b"p must be between 0 and 1" in hip.jsgrad_hip_last_error()
    assert bad(n, 1.0, n + 1, 0.5) != 0 and b"k must be between 0 and numel" in hip.jsgrad_hip_last_error()
    assert bad(n, 1.0, 300, 0.5) != 0          # more top-k entries than the one-block kernel holds
    assert bad(512, 1.0, 0, 0.5) != 0          # the one-level running sum of short vectors is not built
    assert hip.jsgrad_hip_sample(t.ptr, n, ffi.F32, 1.0, 0, 0.5, 0.5, 0.0, None, d.rng.ptr, d.st.ptr, None, 0, 1, d.ws.ptr) != 0   # alpha without its counter
    assert hip.jsgrad_hip_sample(t.ptr, n, ffi.F32, 1.0, 0, 0.5, 0.0, 0.0, None, None, d.st.ptr, None, 0, 1, d.ws.ptr) != 0        # no random state


def test_model_samples_what_the_restatement_draws_from_its_logits():
    """Through Llama3 with the reference's default temperature (0.95, llama3.ts:192): at every position the token equals the
    restatement's draw from the logits the device produced, eagerly and in the replayed graph; a second run from the same
    seed repeats the tokens, another seed does not."""
    cfg = dict(synthetic.config("tiny16"))
    sd = synthetic.random_state_dict(cfg, seed=2, std=0.05)

    def run(seed, temperature=0.95, top_k=0, top_p=0.0, af=0.0, ap=0.0, check_draws=True):
        llama.manual_seed(seed)
        llm = Llama3(temperature=temperature, top_k=top_k, top_p=top_p, alpha_f=af, alpha_p=ap, max_context=cfg["max_context"],
                     args={k: cfg[k] for k in ("dim", "hidden_dim", "n_heads", "n_kv_heads", "n_layers", "norm_eps", "rope_theta", "vocab_size")}).load_weights(sd)
        cnt = np.zeros(cfg["vocab_size"], np.int32)
        tok, toks = 5, []
        for pos in range(24):                                     # position 0 eager, 1 eager, 2 captured, then replays
            got = llm._call(tok); llm.start_pos += 1
            if check_draws:
                lg = llm.model.logits.numpy().astype(np.float32)
                assert got == S.sample(lg, temperature, top_k, top_p, af, ap, S.rand_f32(seed, pos), cnt), f"position {pos}"
            toks.append(got); tok = got
        return toks

    a = run(7)
    assert run(7, check_draws=False) == a and run(8, check_draws=False) != a
    assert len(set(a)) > 4                                         # not stuck on one token
    run(7, 0.8, 12, 0.9, 0.4, 0.2)                                 # top-k / top-p / alpha through the model
    assert run(7, temperature=0.0, check_draws=False) == run(9, temperature=0.0, check_draws=False)      # greedy ignores the seed


def test_one_draw_per_forward_call_whatever_the_sequence_length(hip):
    """Transformer.forward on [1, S] samples once, from the last position's logits (llama.ts:210-212): the random counter
    advances by one per call, token-serial or in one several-row pass, and the token is the restatement's draw."""
    cfg = dict(synthetic.config("tiny16"))
    sd = synthetic.random_state_dict(cfg, seed=2, std=0.05)
    prompt = synthetic.random_prompt(cfg, 7, seed=5).reshape(1, -1)
    for one_pass in (False, True):
        llama.manual_seed(11)
        llm = Llama3.from_config(cfg).load_weights(sd)
        m = llm.model
        counter = lambda: int(llama.rng_state(m.device).numpy().view(np.uint32)[2])
        assert counter() == 0
        tok = m.forward_rows(prompt, 0, 0.9, 0, 0.0).numpy()[0] if one_pass else m.forward(prompt, 0, 0.9, 0, 0.0).item()
        assert counter() == 1
        lg = m.logits.numpy().astype(np.float32)
        assert int(tok) == S.sample(lg, 0.9, 0, 0.0, 0.0, 0.0, S.rand_f32(11, 0), np.zeros(cfg["vocab_size"], np.int32))
        m.forward(np.array([[int(tok)]], np.int32), 7, 0.9, 0, 0.0)
        assert counter() == 2
    with pytest.raises(NotImplementedError, match="one sequence"):
        m.forward_rows(np.zeros((2, 3), np.int32), 0, 0.9)
