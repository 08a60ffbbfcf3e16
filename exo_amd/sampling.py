"""Device-resident sampling state of the decode step.

The reference builds, per request, a list of logits processors and a sampler
(src/exo/worker/engines/mlx/generator/generate.py:599-619) and applies them inside the
batched decode step (src/exo/worker/engines/mlx/patches/opt_batch_gen.py:67-107).  Here
the same per-request settings live in device arrays indexed by batch row, and ONE C-ABI
call (``exo_sample``) at the end of the captured decode graph does processors, log-
normaliser, filters, the seeded draw and the top-20 log-probabilities for all rows - a
request with temperature 0.7 never leaves the graph.

``SamplerSettings`` is the host-side record of one request; ``DeviceSampler`` owns the
arrays (parameters, history ring of the latest tokens, draw counters, outputs) for
``max_rows`` rows.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from . import native
from .native import check
from .ops import _stream

MAX_CONTEXT = 256   # EXO_SAMPLER_MAX_CONTEXT
MAX_BANNED = 8      # EXO_SAMPLER_MAX_BANNED
TOP_LOGPROBS = 20   # EXO_SAMPLER_TOP_LOGPROBS (opt_batch_gen.py:7)
MODE_EDITS, MODE_DRAW, MODE_TABLE, MODE_TOP = 1, 2, 4, 8

# struct exo_sampler_params (include/exo_mi355x.h), 84 bytes
PARAMS_DTYPE = np.dtype([
    ("temperature", "<f4"), ("top_p", "<f4"), ("min_p", "<f4"), ("top_k", "<i4"),
    ("repetition_penalty", "<f4"), ("repetition_context", "<i4"),
    ("presence_penalty", "<f4"), ("presence_context", "<i4"),
    ("frequency_penalty", "<f4"), ("frequency_context", "<i4"),
    ("seed_lo", "<u4"), ("seed_hi", "<u4"), ("n_banned", "<i4"), ("banned", "<i4", (MAX_BANNED,)),
])
assert PARAMS_DTYPE.itemsize == 84


@dataclass
class SamplerSettings:
    """One request's sampler and processors (defaults = the reference's, generate.py:614-619
    and :599-608)."""

    temperature: float = 0.7
    top_p: float = 1.0
    min_p: float = 0.05
    top_k: int = 0
    repetition_penalty: float | None = None
    repetition_context: int = 20
    presence_penalty: float | None = None
    presence_context: int = 20
    frequency_penalty: float | None = None
    frequency_context: int = 20
    banned: list = field(default_factory=list)
    seed: int = 42

    @staticmethod
    def from_task(task, eos_token_ids=(), zero_seed_is_default=True) -> "SamplerSettings":
        """generate.py:599-619: penalties from the task, EOS banned in bench mode.

        The single-request generator reads the seed as `task.seed or 42` (generate.py:547: seed 0
        becomes 42), the batch generator as `seed if seed is not None else 42`
        (batch_generate.py:182: seed 0 stays 0); `zero_seed_is_default` picks between them."""
        rp = task.repetition_penalty
        if rp is not None and rp < 0:
            raise ValueError("repetition_penalty must be a non-negative float")
        return SamplerSettings(
            temperature=task.temperature if task.temperature is not None else 0.7,
            top_p=task.top_p if task.top_p is not None else 1.0,
            min_p=task.min_p if task.min_p is not None else 0.05,
            top_k=task.top_k if task.top_k is not None else 0,
            repetition_penalty=rp,
            repetition_context=task.repetition_context_size
            if task.repetition_context_size is not None else 20,
            presence_penalty=task.presence_penalty, frequency_penalty=task.frequency_penalty,
            banned=list(eos_token_ids or []) if task.bench else [],
            seed=(task.seed or 42) if zero_seed_is_default
            else (task.seed if task.seed is not None else 42))

    # ---- what the row needs
    @property
    def edits(self) -> bool:
        return bool(self.banned) or self.repetition_penalty not in (None, 0, 0.0, 1, 1.0) or bool(
            self.presence_penalty) or bool(self.frequency_penalty)

    @property
    def draws(self) -> bool:
        return self.temperature != 0

    @property
    def table(self) -> bool:
        return self.draws and (self.top_k > 0 or 0.0 < self.top_p < 1.0)

    def on_device(self) -> bool:
        """False for the few settings the kernels do not take (contexts beyond the history
        ring, more banned ids than the parameter block holds)."""
        ctx = max(self.repetition_context if self.repetition_penalty else 0,
                  self.presence_context if self.presence_penalty else 0,
                  self.frequency_context if self.frequency_penalty else 0)
        return ctx <= MAX_CONTEXT and len(self.banned) <= MAX_BANNED

    def record(self) -> np.ndarray:
        r = np.zeros((), PARAMS_DTYPE)
        r["temperature"], r["top_p"], r["min_p"], r["top_k"] = (
            self.temperature, self.top_p, self.min_p, self.top_k)
        r["repetition_penalty"] = self.repetition_penalty or 0.0
        r["repetition_context"] = self.repetition_context
        r["presence_penalty"] = self.presence_penalty or 0.0
        r["presence_context"] = self.presence_context
        r["frequency_penalty"] = self.frequency_penalty or 0.0
        r["frequency_context"] = self.frequency_context
        r["seed_lo"], r["seed_hi"] = self.seed & 0xFFFFFFFF, (self.seed >> 32) & 0xFFFFFFFF
        r["n_banned"] = len(self.banned)
        b = np.zeros(MAX_BANNED, np.int32)
        b[: len(self.banned)] = self.banned
        r["banned"] = b
        return r


class DeviceSampler:
    """Sampling state for ``max_rows`` batch rows on one device."""

    def __init__(self, max_rows: int, vocab_size: int, device, hist_cap: int = MAX_CONTEXT):
        lib = native.load()
        self.max_rows, self.V, self.hist_cap = max_rows, vocab_size, hist_cap
        self.device = torch.device(device)
        z = dict(device=self.device)
        self.params = torch.zeros(max_rows * PARAMS_DTYPE.itemsize, dtype=torch.uint8, **z)
        self.history = torch.zeros(max_rows, hist_cap, dtype=torch.int32, **z)
        self.hist_len = torch.zeros(max_rows, dtype=torch.int32, **z)
        self.draws = torch.zeros(max_rows, dtype=torch.int32, **z)  # uint32 on the device
        self.token = torch.zeros(max_rows, dtype=torch.int32, **z)
        self.logprob = torch.zeros(max_rows, dtype=torch.float32, **z)
        self.lse = torch.zeros(max_rows, dtype=torch.float32, **z)
        self.top_idx = torch.zeros(max_rows, TOP_LOGPROBS, dtype=torch.int32, **z)
        self.top_val = torch.zeros(max_rows, TOP_LOGPROBS, dtype=torch.float32, **z)
        self.workspace = torch.zeros(lib.exo_sample_workspace(max_rows), dtype=torch.uint8, **z)
        self.settings: list[SamplerSettings | None] = [None] * max_rows

    # ---- rows
    def set_row(self, row: int, settings: SamplerSettings, tokens_so_far, draws: int = 0) -> None:
        """Install a request in ``row``: its parameters, the ring holding the latest of
        the tokens its processors have seen so far, the draw counter."""
        if not settings.on_device():
            raise ValueError("sampler settings outside what the device kernels take")
        n = PARAMS_DTYPE.itemsize
        rec = torch.from_numpy(np.frombuffer(settings.record().tobytes(), np.uint8).copy())
        self.params[row * n : (row + 1) * n].copy_(rec)
        toks = [int(t) for t in tokens_so_far]
        ring = np.zeros(self.hist_cap, np.int32)
        for a in range(max(0, len(toks) - self.hist_cap), len(toks)):
            ring[a % self.hist_cap] = toks[a]  # token at absolute position a sits at a mod cap
        self.history[row].copy_(torch.from_numpy(ring))
        self.hist_len[row : row + 1].copy_(torch.tensor([len(toks)], dtype=torch.int32))
        self.draws[row : row + 1].copy_(torch.tensor([draws], dtype=torch.int32))
        self.settings[row] = settings

    def move_row(self, src: int, dst: int) -> None:
        n = PARAMS_DTYPE.itemsize
        self.params[dst * n : (dst + 1) * n].copy_(self.params[src * n : (src + 1) * n])
        self.history[dst].copy_(self.history[src])
        self.hist_len[dst : dst + 1].copy_(self.hist_len[src : src + 1])
        self.draws[dst : dst + 1].copy_(self.draws[src : src + 1])
        self.settings[dst] = self.settings[src]

    def snapshot(self):
        """The state a launch advances (history ring, its fill count, the draw counters)."""
        return self.history.clone(), self.hist_len.clone(), self.draws.clone()

    def restore(self, snap) -> None:
        self.history.copy_(snap[0])
        self.hist_len.copy_(snap[1])
        self.draws.copy_(snap[2])

    def mode(self, rows: int, want_top: bool = False) -> int:
        s = [x for x in self.settings[:rows] if x is not None]
        m = MODE_TOP if want_top else 0
        if any(x.edits for x in s):
            m |= MODE_EDITS
        if any(x.draws for x in s):
            m |= MODE_DRAW
        if any(x.table for x in s):
            m |= MODE_TABLE
        return m

    # ---- the launch
    def sample(self, logits: torch.Tensor, rows: int, mode: int, feedback: torch.Tensor | None = None,
               pos_inc: torch.Tensor | None = None) -> None:
        """Launch the sampling kernels for the first ``rows`` rows on the current stream:
        results in ``token`` / ``logprob`` / ``lse`` (/ ``top_idx``, ``top_val``)."""
        lib = native.load()
        assert logits.dtype == torch.bfloat16 and logits.is_contiguous()
        if logits.shape[0] < rows or logits.shape[1] != self.V or rows > self.max_rows:
            raise ValueError(f"sample: logits {tuple(logits.shape)} for {rows} rows of V={self.V}")
        p = lambda t: None if t is None else t.data_ptr()  # noqa: E731
        check(lib.exo_sample(
            logits.data_ptr(), self.params.data_ptr(), self.history.data_ptr(),
            self.hist_len.data_ptr(), self.draws.data_ptr(), self.token.data_ptr(),
            self.logprob.data_ptr(), self.lse.data_ptr(), self.top_idx.data_ptr(),
            self.top_val.data_ptr(), p(feedback), p(pos_inc), self.workspace.data_ptr(),
            self.workspace.numel(), rows, self.V, self.hist_cap, mode,
            _stream()), "sample")
