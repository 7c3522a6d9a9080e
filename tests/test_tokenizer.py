"""The tokenizer (denograd_amd/tokenizer.py, host code) against what tokenizer.ts does: split pattern, lowest-rank merges,
special-token numbering, chat framing, and a round trip through a tiktoken-style file."""
import base64

import pytest

from denograd_amd.tokenizer import SPECIAL_TOKENS, Tokenizer

MERGES = [b"th", b"the", b" t", b" th", b" the", b"in", b"ing", b"er", b"he", b"ll", b"llo", b"hello", b" w", b"or", b"ld", b"world", b"\n\n",
          b"12", b"123", "é".encode(), "日本".encode()[:2], "日".encode()]


def make_ranks():
    ranks = {bytes([b]): b for b in range(256)}
    for m in MERGES:
        ranks[m] = len(ranks)
    return ranks


@pytest.fixture(scope="module")
def tk():
    return Tokenizer.from_ranks(make_ranks())


def test_special_tokens_are_numbered_after_the_ranks_as_the_reference_does(tk):
    n = len(make_ranks())
    assert tk.bos_id == n and tk.stop_tokens == [n + 1, n + 9]
    assert tk.special_tokens["<|start_header_id|>"] == n + 6 and tk.special_tokens["<|end_header_id|>"] == n + 7
    assert len(SPECIAL_TOKENS) == 256
    # tokenizer.ts:21 numbers the reserved tokens of the tail by their position in the mapped range (0, 1, ...), so the names
    # reserved_special_token_0..4 occur twice and keep the later number
    assert tk.special_tokens["<|reserved_special_token_0|>"] == n + 10 and tk.special_tokens["<|reserved_special_token_4|>"] == n + 14
    assert tk.special_tokens["<|reserved_special_token_245|>"] == n + 255
    assert max(tk.special_tokens.values()) == n + 255


def test_pattern_pieces(tk):
    pieces = lambda s: [m.group(0) for m in tk.pat.finditer(s)]
    assert pieces("Hello world") == ["Hello", " world"]
    assert pieces("I'm here, it'S 12345!") == ["I", "'m", " here", ",", " it", "'S", " ", "123", "45", "!"]
    assert pieces("a\n\n b") == ["a", "\n\n", " b"]
    assert pieces("x  y") == ["x", " ", " y"]
    assert pieces("<|eot_id|>") == ["<|", "eot", "_id", "|>"]        # a special token's text never survives as one piece


def test_bpe_takes_the_lowest_rank_pair_first(tk):
    r = make_ranks()
    assert tk.encode("the") == [r[b"the"]]
    assert tk.encode(" the") == [r[b" the"]]
    assert tk.encode("then") == [r[b"the"], ord("n")]
    assert tk.encode("hello world") == [r[b"hello"], r[b" w"], r[b"or"], r[b"ld"]]     # " w" outranks "wo.."; "world" is never formed after it
    assert tk.encode("thing") == [r[b"th"], r[b"ing"]]
    assert tk.encode("12345") == [r[b"123"], ord("4"), ord("5")]                       # the pattern cuts digits in threes first
    assert tk.encode("") == []
    # every occurrence of the chosen pair is merged in the same round
    assert tk.encode("ththth") == [r[b"th"]] * 3


@pytest.mark.parametrize("text", ["Hello, world! It's 2024.", "é日本語 ünïcödé 🙂", "tabs\tand\nnewlines\r\n\r\n  spaces   ", "a" * 100, "the the the\n\nthe"])
def test_round_trip_and_valid_segmentation(tk, text):
    toks = tk.encode(text)
    assert tk.decode(toks) == text
    assert all(t in tk.decode_map for t in toks)


def test_decode_drops_special_tokens_and_replaces_broken_utf8(tk):
    toks = [tk.bos_id, *tk.encode("hi"), tk.special_tokens["<|eot_id|>"]]
    assert tk.decode(toks) == "hi"
    assert tk.decode([0xE6]) == "�"            # a lone lead byte of a 3-byte character


def test_chat_framing(tk):
    r, sp = make_ranks(), tk.special_tokens
    assert tk.encode_role("user") == [sp["<|start_header_id|>"], *tk.encode("user"), sp["<|end_header_id|>"], r[b"\n\n"]]
    msg = tk.encode_message("user", "  hello world \n")
    assert msg == [*tk.encode_role("user"), *tk.encode("hello world"), sp["<|eot_id|>"]]     # content is trimmed


def test_tiktoken_file_round_trip(tmp_path, tk):
    ranks = make_ranks()
    fn = tmp_path / "tokenizer.model"
    fn.write_text("\n".join(f"{base64.b64encode(k).decode()} {v}" for k, v in ranks.items()) + "\n")
    t2 = Tokenizer.llama(str(fn))
    assert t2.mergeable_ranks == ranks and t2.special_tokens == tk.special_tokens
    assert t2.encode("hello the world 123") == tk.encode("hello the world 123")
