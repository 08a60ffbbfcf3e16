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


class StreamingDetokenizer:
    """Incremental detokenisation of one sequence - the ``tokenizer.detokenizer`` object of
    mlx_lm the reference keeps per request (src/exo/worker/engines/mlx/generator/
    batch_generate.py:319, :352-356: ``add_token``, ``finalize``, ``last_segment``).

    Ids are decoded in context, not one by one: with a byte-level BPE a character may be split
    over several ids, and each id alone decodes to U+FFFD.  Text is released only once it is
    stable: the window ``ids[prefix:]`` is decoded, and while the result ends in U+FFFD (an
    incomplete character) or has not grown, nothing new is released.  ``last_segment``
    returns the text released since it was last read; ``finalize`` releases the rest."""

    def __init__(self, tokenizer):
        self._tok = tokenizer
        self._ids: list[int] = []
        self._prefix = 0   # start of the decoding window
        self._read = 0     # ids[prefix:read] is already released text
        self.text = ""     # everything released so far
        self._taken = 0    # characters of `text` already handed out by last_segment

    def _window(self) -> tuple[str, str]:
        return self._tok.decode(self._ids[self._prefix : self._read]), self._tok.decode(self._ids[self._prefix :])

    def add_token(self, token: int) -> None:
        self._ids.append(int(token))
        done, now = self._window()
        if len(now) > len(done) and not now.endswith("\ufffd"):
            self.text += now[len(done) :]
            self._prefix, self._read = self._read, len(self._ids)

    def finalize(self) -> None:
        done, now = self._window()
        self.text += now[len(done) :]
        self._prefix = self._read = len(self._ids)

    @property
    def last_segment(self) -> str:
        seg = self.text[self._taken :]
        self._taken = len(self.text)
        return seg


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
