"""Llama3.chat end to end on the device with a synthetic tokenizer: the framing the reference feeds the model, the per-token
loop with its stop tokens, the response fields, and the reuse of a prompt prefix that is already in the KV cache."""
import numpy as np
import pytest

from denograd_amd import llama, synthetic
from denograd_amd.llama3 import Llama3
from denograd_amd.tokenizer import Tokenizer
from tests.test_tokenizer import make_ranks

pytestmark = pytest.mark.gpu
CFG = dict(synthetic.config("tiny16"))       # vocabulary 1024 >= 278 ranks + 256 special tokens


def make(temperature=0.0):
    sd = synthetic.random_state_dict(CFG, seed=11, std=0.05)
    llm = Llama3(temperature=temperature, max_context=CFG["max_context"],
                 args={k: CFG[k] for k in ("dim", "hidden_dim", "n_heads", "n_kv_heads", "n_layers", "norm_eps", "rope_theta", "vocab_size")}).load_weights(sd)
    llm.tokenizer = Tokenizer.from_ranks(make_ranks())
    return llm


def test_chat_feeds_the_reference_framing_and_decodes_token_by_token():
    llm = make()
    tk = llm.tokenizer
    llm._system("be brief")
    sys_toks = [tk.bos_id, *tk.encode_message("system", "be brief")]
    assert llm.start_pos == len(sys_toks) and llm.last_seen_toks == sys_toks
    seen = []
    res = llm.chat([{"role": "user", "content": " hello the world "}], on_token=lambda ev: seen.append(ev["token"]), max_new_tokens=10)
    prompt = [*tk.encode_message("user", "hello the world"), *tk.encode_role("assistant")]
    # the same tokens through the token-level loop on a fresh model
    ref = make()
    ref._prefill(sys_toks)
    out = ref.chat_tokens(prompt, 10, stop_tokens=tk.stop_tokens)["tokens"]
    n_out = res["usage"]["output_tokens"]
    assert res["usage"]["input_tokens"] == len(prompt) - 1 and 1 <= n_out <= 10
    assert res["stop_reason"] in ("end_turn", "max_tokens")
    expect = out[:n_out]
    if res["stop_reason"] == "end_turn":
        assert expect[-1] in tk.stop_tokens
        expect = expect[:-1]
    assert res["message"] == {"role": "assistant", "content": tk.decode(expect)}
    assert "".join(seen) == res["message"]["content"]
    assert res["usage"]["tokens_per_second"] > 0 and res["usage"]["time_to_first_token"] > 0


def test_chat_stops_at_a_full_cache_and_samples_with_the_models_settings():
    llama.manual_seed(3)
    llm = make(temperature=0.95)
    res = llm.chat([{"role": "user", "content": "the thing"}])
    assert res["stop_reason"] in ("end_turn", "max_tokens") and llm.start_pos <= CFG["max_context"]
    llama.manual_seed(3)
    again = make(temperature=0.95).chat([{"role": "user", "content": "the thing"}])
    assert again["message"] == res["message"]                    # the same seed draws the same reply


def test_prefill_skips_a_prefix_that_is_already_in_the_cache():
    llm = make()
    tk = llm.tokenizer
    a = [tk.bos_id, *tk.encode_message("system", "the world")]
    llm._prefill(a)
    first = llm.model.logits.numpy().copy()
    llm.start_pos = 0                                              # start over, as a caller that resends the conversation does
    llm._prefill(a + tk.encode_role("user"))
    assert llm.start_pos == len(a) + len(tk.encode_role("user"))
    fresh = make()
    fresh._prefill(a + tk.encode_role("user"))
    assert np.array_equal(llm.model.logits.numpy(), fresh.model.logits.numpy()) and not np.array_equal(first, fresh.model.logits.numpy())
