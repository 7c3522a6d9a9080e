"""The Llama-3 tokenizer of the reference (/root/reference/jsgrad/models/tokenizer.ts): byte-pair merges over the
pieces a split pattern cuts the text into, the mergeable ranks read from a tiktoken-style file (`base64(token) rank` per
line), 256 special tokens numbered after them, and the chat framing of `encode_role` / `encode_message`.  Host code."""
from __future__ import annotations

import base64

import regex

# tokenizer.ts:26, with the flags 'giu': case-insensitive, unicode classes
PAT = r"'s|'t|'re|'ve|'m|'ll|'d|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}{1,3}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+"
SPECIAL_TOKENS = ["<|begin_of_text|>", "<|end_of_text|>", "<|reserved_special_token_0|>", "<|reserved_special_token_1|>", "<|reserved_special_token_2|>",
                  "<|reserved_special_token_3|>", "<|start_header_id|>", "<|end_header_id|>", "<|reserved_special_token_4|>", "<|eot_id|>",
                  # tokenizer.ts:21 numbers the remaining ones by their index in the mapped range, i.e. from 0 again
                  *[f"<|reserved_special_token_{i}|>" for i in range(256 - 10)]]


class Tokenizer:
    def __init__(self, pat: str, mergeable_ranks: dict[bytes, int], special_tokens: dict[str, int]):
        self.pat = regex.compile(pat, regex.IGNORECASE | regex.UNICODE)
        self.mergeable_ranks, self.special_tokens = mergeable_ranks, special_tokens
        self.decode_map = {i: t for t, i in mergeable_ranks.items()}

    @staticmethod
    def llama(path: str) -> "Tokenizer":
        """tokenizer.ts:6-30: `path` is the tokenizer.model that ships with a Llama-3 checkpoint."""
        with open(path) as f:
            ranks = [line.split(" ") for line in f.read().split("\n") if line]
        return Tokenizer.from_ranks({base64.b64decode(k): int(v) for k, v in ranks})

    @staticmethod
    def from_ranks(mergeable_ranks: dict[bytes, int]) -> "Tokenizer":
        n = len(mergeable_ranks)
        special = {}
        for i, tok in enumerate(SPECIAL_TOKENS):
            special[tok] = n + i     # a name that occurs twice keeps its last number, as Object.fromEntries does
        return Tokenizer(PAT, mergeable_ranks, special)

    @property
    def bos_id(self) -> int:
        return self.special_tokens["<|begin_of_text|>"]

    @property
    def stop_tokens(self) -> list[int]:
        return [self.special_tokens["<|end_of_text|>"], self.special_tokens["<|eot_id|>"]]

    def decode(self, toks) -> str:
        """tokenizer.ts:43-55: special tokens are dropped; bytes that do not form valid UTF-8 become U+FFFD."""
        n = len(self.mergeable_ranks)
        return b"".join(self.decode_map[int(t)] for t in toks if int(t) < n).decode("utf-8", errors="replace")

    def encode(self, text: str, allow_special: bool = False) -> list[int]:
        """tokenizer.ts:57-68.  The pattern cuts a special token's text into several pieces, so `allow_special` only ever
        matches a piece that IS a special token's whole text, which the pattern never produces: as in the reference, special
        tokens enter a prompt through encode_role / encode_message, not through encode."""
        tokens: list[int] = []
        for piece in (m.group(0) for m in self.pat.finditer(text)):
            if allow_special and piece in self.special_tokens:
                tokens.append(self.special_tokens[piece])
            else:
                tokens.extend(self._bpe_encode(piece.encode("utf-8")))
        return tokens

    def _bpe_encode(self, data: bytes) -> list[int]:
        """tokenizer.ts:70-108: repeatedly merge, everywhere it occurs, the adjacent pair with the lowest rank (the first
        one found among equals)."""
        parts = [bytes([b]) for b in data]
        while True:
            best, pair = None, None
            for i in range(len(parts) - 1):
                r = self.mergeable_ranks.get(parts[i] + parts[i + 1])
                if r is not None and (best is None or r < best):
                    best, pair = r, (parts[i], parts[i + 1])
            if pair is None:
                break
            out, i = [], 0
            while i < len(parts):
                if i < len(parts) - 1 and parts[i] == pair[0] and parts[i + 1] == pair[1]:
                    out.append(parts[i] + parts[i + 1])
                    i += 2
                else:
                    out.append(parts[i])
                    i += 1
            parts = out
        return [self.mergeable_ranks[p] for p in parts]

    def encode_role(self, role: str) -> list[int]:
        return [self.special_tokens["<|start_header_id|>"], *self.encode(role), self.special_tokens["<|end_header_id|>"], *self.encode("\n\n")]

    def encode_message(self, role: str, content: str) -> list[int]:
        return [*self.encode_role(role), *self.encode(content.strip()), self.special_tokens["<|eot_id|>"]]
