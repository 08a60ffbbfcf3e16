"""Tokenizer plumbing: a Hugging Face ``tokenizer.json`` when the checkpoint directory
has one (loaded with the ``tokenizers`` library, no model-directory code is ever
executed), else an identity tokenizer for synthetic checkpoints whose "text" is the
decimal token ids."""

from __future__ import annotations

import json
from pathlib import Path


class IdTokenizer:
    def __init__(self, vocab_size: int, eos_token_ids: list[int] | None = None):
        self.vocab_size = vocab_size
        self.eos_token_ids = list(eos_token_ids or [])

    def encode(self, text: str, add_special_tokens: bool = False) -> list[int]:
        return [int(t) % self.vocab_size for t in text.split()]

    def decode(self, ids) -> str:
        return "".join(f"{int(i)} " for i in ids)


class HFTokenizer:
    def __init__(self, tok, eos_token_ids: list[int]):
        self._tok = tok
        self.eos_token_ids = eos_token_ids

    def encode(self, text: str, add_special_tokens: bool = False) -> list[int]:
        return self._tok.encode(text, add_special_tokens=add_special_tokens).ids

    def decode(self, ids) -> str:
        return self._tok.decode(list(ids), skip_special_tokens=False)


def load_tokenizer(model_dir: str | Path, vocab_size: int):
    model_dir = Path(model_dir)
    tj = model_dir / "tokenizer.json"
    if not tj.exists():
        return IdTokenizer(vocab_size)
    from tokenizers import Tokenizer

    eos: list[int] = []
    for name in ("generation_config.json", "config.json"):
        p = model_dir / name
        if p.exists():
            with open(p) as f:
                e = json.load(f).get("eos_token_id")
            if e is not None:
                eos = [e] if isinstance(e, int) else list(e)
                break
    return HFTokenizer(Tokenizer.from_file(str(tj)), eos)
