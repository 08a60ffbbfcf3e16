"""Logits processors, sampling filters, the seeded draw and the top-k log-probabilities of
one decode step, restated on the CPU (numpy).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

What the reference does per generated token (src/exo/worker/engines/mlx/patches/
opt_batch_gen.py:57-107): per sequence the logits processors edit the last-position
logits, ``logprobs = logits - logsumexp(logits)``, the sequence's sampler draws a token
from the log-probabilities, and - when a request asked for them - the 20 most likely
tokens are precomputed (``argpartition`` then a sort, :93-107).  Processors and sampler
are built by the reference with mlx_lm's ``make_logits_processors`` / ``make_sampler``
(src/exo/worker/engines/mlx/generator/generate.py:599-619; signatures in
.typings/mlx_lm/sample_utils.pyi:10-72) and ``ban_token_ids`` (generate.py:465-473).

mlx_lm's source is not in the reference tree, so the formulas below are the documented /
commonly stated ones and are "parity unpinned" against mlx_lm itself:
  * repetition: logits of the tokens seen in the last ``context`` positions are divided by
    the penalty when positive, multiplied when negative;
  * presence: the penalty is subtracted once from each token seen in the context;
  * frequency: the penalty is subtracted once per occurrence in the context;
  * every processor works on the logits in their own dtype, so its result is rounded to
    bf16 (the model's logits are bf16);
  * top-p keeps token i iff the probability mass of the tokens not more likely than i
    (itself included) exceeds 1 - top_p; min-p keeps i iff p_i >= min_p * p_max; top-k keeps
    the k most likely (here: every token tied with the k-th as well); the filters compose to
    one value threshold; the draw is from softmax(logprobs / temp) over the kept tokens.
Which tokens the processors see: here, at the step that samples token k, the context is the
last two prompt tokens followed by tokens 0..k-1 - the order of mlx_lm's sequential generator
(and of src/exo/worker/engines/mlx/generator/generate.py).  The reference's batched step
lags by one: it calls the processors with ``self.tokens[e]`` (opt_batch_gen.py:75) and appends
the token being fed only afterwards (:127), so its step k does not yet see token k-1.  The
device path follows the sequential order in both engines, on purpose: one definition for both,
and a token repeated at once is penalised at once.
The random stream is this build's own (Philox-4x32-10 keyed by the request seed, one block
per draw): MLX's generator cannot be reproduced without MLX.  What IS pinned: Philox
against the published known-answer vectors, the filters against independent torch
restatements (sort / cumsum / topk) and against the logits warpers of ``transformers``
(TopP / TopK / MinP: same kept sets), the repetition penalty against
``transformers.RepetitionPenaltyLogitsProcessor``, top-k log-probabilities against
``torch.topk``, the inverse-CDF draw against hand-worked cases.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from .affine import bf16_round

TOP_LOGPROBS = 20  # opt_batch_gen.py:7 (_PRECOMPUTE_TOP_K)
BAN_VALUE = -1e9   # generate.py:471

# ------------------------------------------------------------------------------ Philox

_M0, _M1 = 0xD2511F53, 0xCD9E8D57
_W0, _W1 = 0x9E3779B9, 0xBB67AE85


def philox4x32_10(counter, key):
    """Philox-4x32 with 10 rounds (Salmon et al., "Parallel random numbers: as easy as
    1, 2, 3", SC'11): counter = 4 x uint32, key = 2 x uint32 -> 4 x uint32."""
    c = [int(v) & 0xFFFFFFFF for v in counter]
    k = [int(v) & 0xFFFFFFFF for v in key]
    for _ in range(10):
        p0, p1 = _M0 * c[0], _M1 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xFFFFFFFF, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xFFFFFFFF]
        k = [(k[0] + _W0) & 0xFFFFFFFF, (k[1] + _W1) & 0xFFFFFFFF]
    return c


def uniform(seed: int, draw: int) -> np.float32:
    """The draw-th uniform of a request: 24 bits of the first Philox word of block
    (draw, 0, 0, 0) under key (seed low, seed high), in [0, 1)."""
    r = philox4x32_10((draw, 0, 0, 0), (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    return np.float32((r[0] >> 8) * 2.0 ** -24)


# --------------------------------------------------------------------------- processors


@dataclass
class SamplerParams:
    temperature: float = 0.0
    top_p: float = 1.0
    min_p: float = 0.0
    top_k: int = 0
    repetition_penalty: float = 0.0   # 0 or 1: off
    repetition_context: int = 20
    presence_penalty: float = 0.0
    presence_context: int = 20
    frequency_penalty: float = 0.0
    frequency_context: int = 20
    banned: list = field(default_factory=list)
    seed: int = 42


def _r(v) -> np.float32:
    """One float32 value rounded to bf16."""
    return bf16_round(np.array([v], np.float32))[0]


def apply_processors(logits: np.ndarray, history, p: SamplerParams) -> np.ndarray:
    """logits float32 [V] holding bf16 values; history = every token of the sequence so far
    (prompt and generated).  Order: ban, repetition, presence, frequency (generate.py:599-612)."""
    x = np.array(logits, np.float32, copy=True)
    h = [int(t) for t in history]

    def ctx(n):
        return h[-n:] if n > 0 else []

    if p.banned:
        x[list(p.banned)] = _r(BAN_VALUE)
    if p.repetition_penalty not in (0.0, 1.0):
        for t in set(ctx(p.repetition_context)):
            v = x[t]
            x[t] = _r(v * np.float32(p.repetition_penalty) if v < 0 else v / np.float32(p.repetition_penalty))
    if p.presence_penalty != 0.0:
        for t in set(ctx(p.presence_context)):
            x[t] = _r(x[t] - np.float32(p.presence_penalty))
    if p.frequency_penalty != 0.0:
        c = ctx(p.frequency_context)
        for t in set(c):
            x[t] = _r(x[t] - np.float32(p.frequency_penalty) * np.float32(c.count(t)))
    return x


# ------------------------------------------------------------------------------ sampler


def logsumexp(x: np.ndarray) -> np.float32:
    m = np.float32(x.max())
    return np.float32(m + np.log(np.sum(np.exp((x - m).astype(np.float64)))))


def keep_threshold(x: np.ndarray, p: SamplerParams) -> np.float32:
    """The value t such that exactly the tokens with x >= t survive top-p, min-p and top-k."""
    x = x.astype(np.float32)
    t = np.float32(-np.inf)
    if 0.0 < p.top_p < 1.0:
        prob = np.exp((x - logsumexp(x)).astype(np.float64))
        order = np.argsort(x, kind="stable")
        xs, cs = x[order], np.cumsum(prob[order])
        vals, first = np.unique(xs, return_index=True)        # ascending distinct values
        last = np.r_[first[1:], xs.size] - 1
        below = cs[last]                                      # mass of the tokens with value <= v
        t = max(t, np.float32(vals[np.argmax(below > 1.0 - p.top_p)]))
    if p.min_p > 0.0:
        t = max(t, np.float32(np.float32(x.max()) + np.float32(np.log(np.float32(p.min_p)))))
    if p.top_k > 0:
        k = min(p.top_k, x.size)
        t = max(t, np.float32(np.partition(x, x.size - k)[x.size - k]))
    return np.float32(t)


def sample(x: np.ndarray, p: SamplerParams, u: float, return_interval: bool = False):
    """Token drawn from processed logits x (float32 [V]) with the uniform u in [0,1):
    temperature 0 -> argmax (lowest index on ties); else inverse CDF in vocabulary order over
    the kept tokens, weights exp((x - max) / temperature)."""
    x = x.astype(np.float32)
    if p.temperature == 0:
        return int(np.argmax(x))
    t = keep_threshold(x, p)
    keep = x >= t
    w = np.where(keep, np.exp(((x - x.max()) / np.float32(p.temperature)).astype(np.float64)), 0.0)
    cdf = np.cumsum(w)
    target = float(u) * cdf[-1]
    i = int(np.searchsorted(cdf, target, side="right"))
    kept = np.flatnonzero(keep)
    i = min(i, int(kept[-1]))
    if return_interval:
        return i, (cdf[i] - w[i]) / cdf[-1], cdf[i] / cdf[-1]
    return i


def top_logprobs(x: np.ndarray, k: int = TOP_LOGPROBS):
    """The k most likely tokens, most likely first, ties to the lower id; (ids, logprobs)."""
    x = x.astype(np.float32)
    lp = (x - logsumexp(x)).astype(np.float32)
    order = np.lexsort((np.arange(x.size), -x))[: min(k, x.size)]
    return order.astype(np.int32), lp[order]
