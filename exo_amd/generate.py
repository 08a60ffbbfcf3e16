"""Prefill and sequential generation with the reference's protocol.

Mirrors src/exo/worker/engines/mlx/generator/generate.py:
  ``prefill`` (:282-396)   feeds n tokens so that the cache ends up holding n-1
  ``mlx_generate`` (:532-827) -> ``generate`` here: prefill on prompt[:-1], then the
      last TWO prompt tokens are fed as single-token forwards, then one single-token
      forward per generated token.
Single-token forwards always take the GEMV path (like the reference's M=1 calls), so
token N-2 of the prompt is not folded into the prefill GEMM.
"""

from __future__ import annotations

import time
from collections.abc import Callable, Generator

import torch

from . import ops
from .cache import ShardKVCache, cache_length
from .model import ShardModel
from .types import GenerationResponse, GenerationStats, TextGenerationTaskParams, TopLogprobItem, Usage

MAX_TOKENS = 32168  # src/exo/worker/engines/mlx/constants.py:7
DEFAULT_TOP_LOGPROBS = 5
PREFILL_STEP_SIZE = 4096  # generate.py:334


class PrefillCancelled(BaseException):
    """Raised from a progress callback to abandon a prefill (generate.py:153-154)."""


# ---------------------------------------------------------------------- sampling


def make_sampler(temp: float = 0.0, top_p: float = 1.0, min_p: float = 0.0, top_k: int = 0,
                 generator: torch.Generator | None = None) -> Callable[[torch.Tensor], torch.Tensor]:
    """mlx_lm ``make_sampler`` semantics (.typings/mlx_lm/sample_utils.pyi:10-45) on
    float32 log-probabilities [B,V] -> token ids int64 [B]: temp 0 is argmax; otherwise
    top_p, then min_p, then top_k filters are applied to the log-probabilities and a
    token is drawn from softmax(logprobs / temp)."""
    if temp == 0:
        return lambda lp: torch.argmax(lp, dim=-1)

    def sample(lp: torch.Tensor) -> torch.Tensor:
        lp = lp.float()
        if 0 < top_p < 1.0:
            probs = lp.exp()
            sp, si = torch.sort(probs, dim=-1)  # ascending
            cum = sp.cumsum(-1)
            keep = cum > (1 - top_p)
            masked = torch.where(keep, lp.gather(-1, si), torch.full_like(lp, -float("inf")))
            lp = torch.empty_like(lp).scatter_(-1, si, masked)
        if min_p > 0:
            top = lp.max(-1, keepdim=True).values
            lp = torch.where(lp < top + torch.log(torch.tensor(min_p, device=lp.device)),
                             torch.full_like(lp, -float("inf")), lp)
        if top_k > 0:
            kth = lp.topk(min(top_k, lp.shape[-1]), dim=-1).values[..., -1:]
            lp = torch.where(lp < kth, torch.full_like(lp, -float("inf")), lp)
        p = torch.softmax(lp / temp, dim=-1)
        return torch.multinomial(p, 1, generator=generator).squeeze(-1)

    return sample


def ban_token_ids(token_ids: list[int]) -> Callable[[torch.Tensor, torch.Tensor], torch.Tensor]:
    """generate.py:465-473: set the banned logits to -1e9."""
    ids = list(token_ids)

    def proc(_tokens: torch.Tensor, logits: torch.Tensor) -> torch.Tensor:
        if ids:
            logits = logits.clone()
            logits[..., ids] = -1e9
        return logits

    return proc


def make_logits_processors(repetition_penalty: float | None = None,
                           repetition_context_size: int | None = 20,
                           presence_penalty: float | None = None,
                           presence_context_size: int | None = 20,
                           frequency_penalty: float | None = None,
                           frequency_context_size: int | None = 20,
                           ) -> list[Callable[[torch.Tensor, torch.Tensor], torch.Tensor]]:
    """mlx_lm ``make_logits_processors`` (.typings/mlx_lm/sample_utils.pyi:47-72) as the
    reference calls it (generate.py:599-608): each processor maps (tokens so far,
    logits [1,V]) to logits.  Definitions as commonly stated, the library's source not
    being at hand: repetition divides the positive / multiplies the negative logits of
    the tokens seen in the last ``context`` positions by the penalty; presence subtracts
    the penalty once from each token seen there; frequency subtracts it once per
    occurrence.  A penalty of None or 0 adds no processor."""
    procs: list[Callable[[torch.Tensor, torch.Tensor], torch.Tensor]] = []

    def context(tokens: torch.Tensor, size: int | None, device) -> torch.Tensor:
        t = torch.as_tensor(tokens, dtype=torch.int64).reshape(-1)
        if size is not None:
            t = t[-size:] if size > 0 else t[:0]
        return t.to(device)

    if repetition_penalty is not None and repetition_penalty != 0:
        if repetition_penalty < 0:
            raise ValueError("repetition_penalty must be a non-negative float")

        def repetition(tokens, logits):
            ctx = context(tokens, repetition_context_size, logits.device)
            if ctx.numel() == 0:
                return logits
            logits = logits.clone()
            sel = logits[..., ctx]
            logits[..., ctx] = torch.where(sel < 0, sel * repetition_penalty, sel / repetition_penalty)
            return logits

        procs.append(repetition)
    if presence_penalty:
        def presence(tokens, logits):
            ctx = torch.unique(context(tokens, presence_context_size, logits.device))
            if ctx.numel() == 0:
                return logits
            logits = logits.clone()
            logits[..., ctx] -= presence_penalty
            return logits

        procs.append(presence)
    if frequency_penalty:
        def frequency(tokens, logits):
            ctx = context(tokens, frequency_context_size, logits.device)
            if ctx.numel() == 0:
                return logits
            counts = torch.zeros(logits.shape[-1], dtype=logits.dtype, device=logits.device)
            counts.index_add_(0, ctx, torch.ones(ctx.numel(), dtype=logits.dtype, device=logits.device))
            return logits - frequency_penalty * counts

        procs.append(frequency)
    return procs


def processors_for(task: TextGenerationTaskParams, eos_token_ids) -> list:
    """Processor list of one request: the penalties of its parameters, preceded in bench
    mode by the EOS ban so that exactly max_tokens are produced (generate.py:599-612)."""
    procs = make_logits_processors(
        repetition_penalty=task.repetition_penalty,
        repetition_context_size=task.repetition_context_size
        if task.repetition_context_size is not None else 20,
        presence_penalty=task.presence_penalty, frequency_penalty=task.frequency_penalty)
    eos = list(eos_token_ids or [])
    if task.bench and eos:
        procs = [ban_token_ids(eos)] + procs
    return procs


def extract_top_logprobs(logprobs: torch.Tensor, tokenizer, top_logprobs: int,
                         selected_token: int) -> tuple[float, list[TopLogprobItem]]:
    """generate.py:483-529: the selected token's logprob and the k most likely tokens,
    descending."""
    k = min(top_logprobs, logprobs.shape[-1])
    vals, idx = torch.topk(logprobs.float(), k)
    items = []
    for v, i in zip(vals.tolist(), idx.tolist()):
        text = tokenizer.decode([i]) if tokenizer is not None else str(i)
        items.append(TopLogprobItem(token=text, logprob=float(v), bytes=list(text.encode("utf-8"))))
    return float(logprobs[selected_token]), items


# ---------------------------------------------------------------------- prefill


def prefill(model: ShardModel, prompt_tokens, cache: ShardKVCache,
            on_prefill_progress: Callable[[int, int], None] | None = None,
            step: int = PREFILL_STEP_SIZE, faithful_extra_steps: bool = True,
            row: int = 0, graph_steps: bool = False) -> tuple[float, int]:
    """Fill cache row ``row`` from ``prompt_tokens`` (n ids).  After it the row holds
    n-1 entries (invariant asserted by the reference's test_kv_prefix_cache.py:157).

    Protocol (generate.py:354-387): chunks of at most ``step`` tokens cover the first
    n-1 tokens; token n-1 is then run as a single-token forward whose sample is
    discarded, the generator it came from had already computed one more single-token
    forward, and ``trim(2)`` removes both entries.  ``faithful_extra_steps=False``
    skips those two forwards (same cache contents, less work).  ``graph_steps``: run them as
    replays of the captured single-token step of this cache row instead of launch by launch
    (same kernels; worth it for a cache that serves many requests).
    Returns (tokens_per_sec, n)."""
    n = len(prompt_tokens)
    if n == 0:
        return 0.0, 0
    t0 = time.perf_counter()
    toks = torch.as_tensor(prompt_tokens, dtype=torch.int32).reshape(1, -1)
    rows = slice(row, row + 1)
    done = 0
    while n - done > 1:
        m = min(step, n - done - 1)
        model(toks[:, done : done + m], cache, logits="none", rows=rows)
        done += m
        if on_prefill_progress is not None:
            on_prefill_progress(done, n)
    if faithful_extra_steps:
        if graph_steps and model.is_first and model.is_last:
            # the same two single-token forwards as graph replays (a cache that outlives the
            # call keeps its captured step per row): the second consumes the first's argmax
            bufs = model._buffers(1, 1)
            bufs.tokens.copy_(toks[0, done : done + 1])
            model.decode_step(cache, 1, feedback=True, row0=row)
            model.decode_step(cache, 1, feedback=True, row0=row)
        else:
            lg = model(toks[:, done : done + 1], cache, logits="last", rows=rows)
            nxt = torch.argmax(lg[0, -1].float()).reshape(1, 1)
            model(nxt, cache, logits="last", rows=rows)
        cache.trim(2, rows=range(row, row + 1))
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return (n / dt if dt > 0 else 0.0), n


# ---------------------------------------------------------------------- per-sequence host state


class _NoTokenizer:
    eos_token_ids: list = []

    def decode(self, ids) -> str:
        return ""


class TokenStream:
    """Host-side bookkeeping of one generating sequence, the part of the reference's decode
    loop that runs after a token is known (src/exo/worker/engines/mlx/generator/
    batch_generate.py:337-460, generate.py:735-827): streaming detokenisation, EOS / length /
    stop-sequence finish, log-probability items, statistics and usage at the end."""

    def __init__(self, tokenizer, task: TextGenerationTaskParams, eos_token_ids, max_tokens: int,
                 n_prompt: int, prefill_tps: float, prefix_cache_hit: str, device,
                 prompt_tokens_stat: int | None = None):
        from .tokenizer import StreamingDetokenizer
        self.tokenizer = tokenizer if tokenizer is not None else _NoTokenizer()
        self.task, self.eos, self.max_tokens = task, set(eos_token_ids or []), max_tokens
        self.n_prompt, self.prefill_tps, self.prefix_cache_hit = n_prompt, prefill_tps, prefix_cache_hit
        self.prompt_tokens_stat = n_prompt if prompt_tokens_stat is None else prompt_tokens_stat
        self.device = device
        self.detok = StreamingDetokenizer(self.tokenizer)
        self.stop_sequences = [task.stop] if isinstance(task.stop, str) else list(task.stop or [])
        self.max_stop_len = max((len(s) for s in self.stop_sequences), default=0)
        self.pending_stop_text = ""
        self.n_gen = 0
        self.t_first: float | None = None
        self.t_last: float | None = None

    def top_items(self, ids, values, k: int) -> list[TopLogprobItem]:
        """generate.py:513-529: ids and log-probabilities (most likely first) -> items."""
        items = []
        for i, v in list(zip(ids, values))[:k]:
            if i < 0 or v != v:
                continue
            text = self.tokenizer.decode([int(i)]) if not isinstance(self.tokenizer, _NoTokenizer) else str(int(i))
            items.append(TopLogprobItem(token=text, logprob=float(v), bytes=list(text.encode("utf-8"))))
        return items

    def push(self, tok: int, now: float, logprob: float | None = None,
             top_logprobs: list[TopLogprobItem] | None = None) -> GenerationResponse:
        self.n_gen += 1
        if self.t_first is None:
            self.t_first = now
        self.t_last = now
        finish = None
        if tok in self.eos and not self.task.bench:
            finish = "stop"
        elif self.n_gen >= self.max_tokens:
            finish = "length"
        if finish != "stop":
            self.detok.add_token(tok)
        if finish is not None:
            self.detok.finalize()
        text = self.detok.last_segment
        self.pending_stop_text += text
        for s in self.stop_sequences:
            if s and s in self.pending_stop_text:
                cut = self.pending_stop_text.find(s)
                chunk_start = len(self.pending_stop_text) - len(text)
                text = self.pending_stop_text[:cut][chunk_start:]
                finish = "stop"
                break
        stats = usage = None
        if finish is not None:
            # generation_tps = (n-1)/(t_last - t_first)  (batch_generate.py:418-426)
            dt = (self.t_last - self.t_first) if self.n_gen > 1 else 0.0
            stats = GenerationStats(
                prompt_tps=float(self.prefill_tps),
                generation_tps=float((self.n_gen - 1) / dt) if dt > 0 else 0.0,
                prompt_tokens=int(self.prompt_tokens_stat), generation_tokens=self.n_gen,
                peak_memory_usage=int(torch.cuda.max_memory_allocated(self.device)),
                prefix_cache_hit=self.prefix_cache_hit)
            usage = Usage(self.n_prompt, self.n_gen, self.n_prompt + self.n_gen)
        elif self.max_stop_len and len(self.pending_stop_text) > self.max_stop_len:
            self.pending_stop_text = self.pending_stop_text[-self.max_stop_len:]
        return GenerationResponse(text=text, token=tok, logprob=logprob, top_logprobs=top_logprobs,
                                  finish_reason=finish, stats=stats, usage=usage)


# ---------------------------------------------------------------------- generate


class GenerateState:
    """A KV cache row and the sampling arrays that serve one request after another: the HIP
    graphs ``generate()`` captures are bound to them, so a caller that keeps the state (the
    sequential engine) captures once instead of once per request."""

    def __init__(self, model: ShardModel, max_seq: int):
        from .sampling import DeviceSampler
        self.max_seq = max_seq
        self.cache = model.make_cache(1, max_seq)
        self.sampler = DeviceSampler(1, model.cfg.vocab_size, model.device)


def generate(model: ShardModel, tokenizer, task: TextGenerationTaskParams, prompt_tokens: list[int],
             on_prefill_progress: Callable[[int, int], None] | None = None,
             on_generation_token: Callable[[], None] | None = None,
             max_seq: int | None = None, eos_token_ids: list[int] | None = None,
             kv_prefix_cache=None, state: GenerateState | None = None,
             ) -> Generator[GenerationResponse, None, None]:
    """Sequential (batch 1) generation for a full-model shard: yields one
    GenerationResponse per token; the last carries finish_reason, stats and usage.
    ``kv_prefix_cache`` (a KVPrefixCache) is consulted and updated the way the reference's
    mlx_generate does (generate.py:577-706): bench requests only with use_prefix_cache.

    Every step is one graph replay that ends in the device sampling kernels; the host only
    reads the sampled token (and log-probabilities when asked for).  Settings the kernels do
    not take (penalty contexts beyond 256 tokens, more than 8 banned ids) run the processors
    and the sampler on the host with torch instead."""
    from .sampling import DeviceSampler, SamplerSettings
    if not (model.is_first and model.is_last):
        raise ValueError("generate() needs a shard that holds the whole model")
    max_tokens = task.max_output_tokens or MAX_TOKENS
    n_prompt = len(prompt_tokens)
    if n_prompt == 0:
        raise ValueError("empty prompt")
    if state is not None:
        cache = state.cache
        cache.reset()
        if n_prompt + 2 > cache.max_seq:
            raise ValueError(f"prompt of {n_prompt} tokens exceeds the cache ({cache.max_seq})")
        max_tokens = min(max_tokens, cache.max_seq - n_prompt - 2)
    else:
        cache = model.make_cache(1, max_seq or (n_prompt + max_tokens + 8))
    torch.cuda.reset_peak_memory_stats(model.device)

    eos = list(eos_token_ids or [])
    settings = SamplerSettings.from_task(task, eos)

    if task.bench and not task.use_prefix_cache:
        kv_prefix_cache = None
    remaining, matched_index, is_exact_hit = list(prompt_tokens), None, False
    if kv_prefix_cache is not None:
        _, remaining, matched_index, is_exact_hit = kv_prefix_cache.get_kv_cache(cache, prompt_tokens)
    prefix_hit_length = n_prompt - len(remaining)
    prefill_tps, prefill_tokens = prefill(model, remaining[:-1], cache, on_prefill_progress,
                                          graph_steps=state is not None)
    assert cache_length(cache) == max(n_prompt - 2, prefix_hit_length)
    prefix_cache_hit = "none"
    if matched_index is not None and prefix_hit_length > 0:
        prefix_cache_hit = "exact" if is_exact_hit else "partial"
        if is_exact_hit:
            prefill_tps = kv_prefix_cache.prefill_tps[matched_index]
    if kv_prefix_cache is not None:
        from .prefix_cache import save_prefix_cache
        save_prefix_cache(kv_prefix_cache, prompt_tokens, cache, 0, prefix_hit_length,
                          matched_index, prefill_tps=prefill_tps)

    # the last two prompt tokens, one forward each (generate.py:710-733); they are also all
    # the logits processors see of the prompt (stream_generate is handed prompt[-2:])
    if len(remaining) >= 2:
        if state is not None:  # the captured step of this cache (its sample is not used)
            model._buffers(1, 1).tokens[0] = int(remaining[-2])
            model.decode_step(cache, 1)
        else:
            model(torch.tensor([[remaining[-2]]], dtype=torch.int32), cache, logits="none")
    tok = int(prompt_tokens[-1])
    history = [int(t) for t in prompt_tokens[-2:]]
    stream = TokenStream(tokenizer, task, eos, max_tokens, n_prompt, prefill_tps, prefix_cache_hit,
                         model.device, prompt_tokens_stat=prefill_tokens + min(n_prompt, 2))
    want_top = bool(task.logprobs)
    k_top = task.top_logprobs or DEFAULT_TOP_LOGPROBS
    on_device = settings.on_device() and k_top <= 20
    if on_device:
        ds = state.sampler if state is not None else DeviceSampler(1, model.cfg.vocab_size, model.device)
        ds.set_row(0, settings, history)
        mode = ds.mode(1, want_top)
    else:
        gen = torch.Generator(device=model.device)
        gen.manual_seed(settings.seed)
        processors = processors_for(task, eos)
        sampler = make_sampler(settings.temperature, settings.top_p, settings.min_p, settings.top_k, gen)
    bufs = model._buffers(1, 1)
    bufs.tokens[0] = tok
    for _ in range(max_tokens):
        logprob = top = None
        if on_device:
            model.decode_step(cache, 1, feedback=True, sampler=ds, mode=mode)
            tok = int(ds.token[0])  # synchronises
            if want_top:
                logprob = float(ds.logprob[0])
                top = stream.top_items(ds.top_idx[0].tolist(), ds.top_val[0].tolist(), k_top)
        else:
            bufs.tokens[0] = tok
            bufs = model.decode_step(cache, 1)
            logits = bufs.logits[0:1].float()
            for p in processors:
                logits = p(torch.tensor(history), logits)
            logprobs = logits - torch.logsumexp(logits, dim=-1, keepdim=True)
            tok = int(sampler(logprobs)[0])
            history.append(tok)
            if want_top:
                logprob, top = extract_top_logprobs(logprobs[0], tokenizer, k_top, tok)
        resp = stream.push(tok, time.perf_counter(), logprob, top)
        if on_generation_token is not None:
            on_generation_token()
        yield resp
        if resp.finish_reason is not None:
            break
