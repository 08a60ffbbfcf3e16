"""The drop-in boundary: ``Builder`` / ``Engine`` for one MI355X.

Mirrors the reference's plugin interface (src/exo/worker/engines/base.py:16-60) and
its MLX implementations:
  Mi355xBuilder        <-> MlxBuilder        (src/exo/worker/engines/mlx/builder.py:33-113)
  BatchGenerator       <-> BatchGenerator    (src/exo/worker/runner/llm_inference/batch_generator.py:320-572)
  ShardBatchGenerator  <-> ExoBatchGenerator (src/exo/worker/engines/mlx/generator/batch_generate.py:93-536)
Same method names, argument meaning and error behaviour: ``step`` emits an ErrorChunk
through ``event_sender`` before re-raising; a cancelled prefill raises
PrefillCancelled; every method runs on the caller's (the runner's main) thread.
``event_sender`` needs ``send(obj)``, ``cancel_receiver`` needs ``collect() -> list``;
exo's MpSender / MpReceiver satisfy both.
"""

from __future__ import annotations

import logging
import os
import time
import uuid
from abc import ABC, abstractmethod
from collections import deque
from collections.abc import Callable, Generator, Iterable
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any

import torch

from .cache import ShardKVCache
from .config import ModelConfig
from .generate import (
    DEFAULT_TOP_LOGPROBS, MAX_TOKENS, PrefillCancelled, TokenStream, extract_top_logprobs,
    GenerateState, generate, make_sampler, prefill, processors_for,
)
from .loader import load_shard_weights
from .model import ShardModel
from .prefix_cache import KVPrefixCache, save_prefix_cache
from .sampling import TOP_LOGPROBS, DeviceSampler, SamplerSettings
from .tokenizer import load_tokenizer
logger = logging.getLogger("exo_amd")

from .types import (
    BoundInstance, CancelledResponse, ErrorChunk, FinishedResponse, GenerationResponse,
    GenerationStats, GenerationTask, ModelLoadingResponse, PrefillProgressChunk,
    TextGenerationTaskParams, TokenChunk, Usage,
)

EXO_MAX_CONCURRENT_REQUESTS = int(os.environ.get("EXO_MAX_CONCURRENT_REQUESTS", "8"))
REMOTE_PREFILL_MIN_TOKENS = 1000  # src/exo/worker/engines/mlx/generator/batch_generate.py:62
CANCEL_ALL_TASKS = "CANCEL_ALL_TASKS"


# ----------------------------------------------------------------------- ABCs


class Engine(ABC):
    _cancelled_tasks: set

    def should_cancel(self, task_id) -> bool:
        return task_id in self._cancelled_tasks or CANCEL_ALL_TASKS in self._cancelled_tasks

    @abstractmethod
    def warmup(self) -> None: ...

    @abstractmethod
    def submit(self, task: GenerationTask) -> None: ...

    @abstractmethod
    def step(self) -> Iterable[tuple[Any, Any]]: ...

    @abstractmethod
    def close(self) -> None: ...

    @abstractmethod
    def serve_prefill(self, request, wfile) -> None: ...


class Builder(ABC):
    @abstractmethod
    def connect(self, bound_instance: BoundInstance) -> None: ...

    @abstractmethod
    def load(self, bound_instance: BoundInstance) -> Generator[ModelLoadingResponse, None, None]: ...

    @abstractmethod
    def build(self) -> Engine: ...

    @abstractmethod
    def close(self) -> None: ...


# ------------------------------------------------------- inner batch generator


@dataclass
class _Seq:
    uid: int
    params: TextGenerationTaskParams
    prompt_tokens: list[int]
    settings: SamplerSettings
    stream: TokenStream
    on_generation_token: Callable[[], None] | None
    want_top: bool
    k_top: int
    # host-side sampling, only for settings the device kernels do not take
    sampler: Callable | None = None
    processors: list | None = None
    tokens: list[int] = field(default_factory=list)  # what the logits processors see

    @property
    def on_device(self) -> bool:
        return self.sampler is None


@dataclass
class _Flight:
    """One launched decode step whose results the host has not read yet."""

    rows: list            # the sequences of the step, by batch row at launch time
    slot: int             # which pinned host buffer set its outputs are copied into
    event: Any
    want_top: bool


class ShardBatchGenerator:
    """Continuous batching over one KV pool of ``max_batch`` rows.  ``submit`` prefills
    the request into the next free row (batch-1 path) and feeds the last-but-one
    prompt token as a single-token forward; ``step`` returns one token per active row.
    Active rows are kept compact at the front of the pool.

    A step is ONE graph replay: the single-token forward of all active rows followed by the
    device sampling kernels (processors, filters, draw, top-20 log-probabilities), with the
    chosen tokens written back as the next step's input.  Like the reference's patched step
    (src/exo/worker/engines/mlx/patches/opt_batch_gen.py:108-124: ``async_eval`` of step n+1
    before step n is read), ``step`` launches the NEXT replay before it waits for the results
    of the one it returns, so the device never idles on the host's detokenising and
    bookkeeping; the results travel through pinned host buffers guarded by an event.  When
    the set of rows changes (a request finishes, is cancelled or joins), the chain restarts
    from the host's tokens after the step in flight has been read."""

    def __init__(self, model: ShardModel, tokenizer, max_batch: int = EXO_MAX_CONCURRENT_REQUESTS,
                 max_seq: int = 8192, kv_prefix_cache: KVPrefixCache | None = None):
        if not (model.is_first and model.is_last):
            raise ValueError("the batch generator needs a shard that holds the whole model")
        self.model, self.tokenizer = model, tokenizer
        self.max_batch, self.max_seq = max_batch, max_seq
        self.cache: ShardKVCache = model.make_cache(max_batch, max_seq)
        self.kv_prefix_cache = kv_prefix_cache
        self.rows: list[_Seq] = []
        self._next_uid = 0
        self._pending_input: list[int] = []  # latest token per active row, as the host knows it
        self.sampler = DeviceSampler(max_batch, model.cfg.vocab_size, model.device)
        self._flight: _Flight | None = None
        pin = dict(pin_memory=True)
        self._host = [dict(token=torch.zeros(max_batch, dtype=torch.int32, **pin),
                           logprob=torch.zeros(max_batch, dtype=torch.float32, **pin),
                           top_idx=torch.zeros(max_batch, TOP_LOGPROBS, dtype=torch.int32, **pin),
                           top_val=torch.zeros(max_batch, TOP_LOGPROBS, dtype=torch.float32, **pin))
                      for _ in range(2)]
        self._slot = 0
        self._sampler_stale = False

    @property
    def has_work(self) -> bool:
        return bool(self.rows)

    def _eos(self) -> list[int]:
        return list(getattr(self.tokenizer, "eos_token_ids", []) or [])

    def submit(self, task_params: TextGenerationTaskParams, prompt,
               on_prefill_progress: Callable[[int, int], None] | None = None,
               distributed_prompt_progress_callback: Callable[[], None] | None = None,
               on_generation_token: Callable[[], None] | None = None) -> int:
        if len(self.rows) >= self.max_batch:
            raise RuntimeError("no free batch row")
        toks = prompt if not isinstance(prompt, str) else self.tokenizer.encode(prompt)
        toks = [int(t) for t in toks]
        if not toks:
            raise ValueError("empty prompt")
        max_tokens = task_params.max_output_tokens or MAX_TOKENS
        if len(toks) + max_tokens + 2 > self.max_seq:
            max_tokens = self.max_seq - len(toks) - 2
            if max_tokens <= 0:
                raise ValueError(f"prompt of {len(toks)} tokens exceeds the cache ({self.max_seq})")
        settings = SamplerSettings.from_task(task_params, self._eos(), zero_seed_is_default=False)
        row = len(self.rows)
        # prefix cache lookup (batch_generate.py:164-181): bench requests opt in
        use_prefix = self.kv_prefix_cache is not None and (
            not task_params.bench or task_params.use_prefix_cache)
        matched_index, is_exact_hit, remaining = None, False, toks
        if use_prefix:
            _, remaining, matched_index, is_exact_hit = self.kv_prefix_cache.get_kv_cache(
                self.cache, toks, row=row)
        else:
            self.cache.reset(rows=range(row, row + 1))
        prefix_hit_length = len(toks) - len(remaining)

        def progress(done: int, total: int) -> None:
            if distributed_prompt_progress_callback is not None:
                distributed_prompt_progress_callback()  # may raise PrefillCancelled
            if on_prefill_progress is not None:
                on_prefill_progress(done, total)

        try:
            tps, n = self._prefill_row(task_params, toks, remaining, prefix_hit_length, row, progress,
                                       on_prefill_progress)
        except PrefillCancelled:
            self.cache.reset(rows=range(row, row + 1))
            raise
        prefix_cache_hit = "none"
        if matched_index is not None and prefix_hit_length > 0:
            prefix_cache_hit = "exact" if is_exact_hit else "partial"
            if is_exact_hit:
                tps = self.kv_prefix_cache.prefill_tps[matched_index]
        if use_prefix:
            try:
                save_prefix_cache(self.kv_prefix_cache, toks, self.cache, row, prefix_hit_length,
                                  matched_index, prefill_tps=tps)
            except Exception:  # a failed save never fails the request (batch_generate.py:534)
                logger.warning("failed to save prefix cache", exc_info=True)
        if len(remaining) >= 2:
            self.model(torch.tensor([[remaining[-2]]], dtype=torch.int32), self.cache,
                       logits="none", rows=slice(row, row + 1))
        k_top = task_params.top_logprobs or DEFAULT_TOP_LOGPROBS
        seq = _Seq(
            uid=self._next_uid, params=task_params, prompt_tokens=toks, settings=settings,
            stream=TokenStream(self.tokenizer, task_params, self._eos(), max_tokens, len(toks), tps,
                               prefix_cache_hit, self.model.device),
            on_generation_token=on_generation_token, want_top=bool(task_params.logprobs), k_top=k_top,
            # the generator is handed the last two prompt tokens (batch_generate.py:282,301):
            # they are all the logits processors see of the prompt
            tokens=list(toks[-2:]))
        if settings.on_device() and k_top <= TOP_LOGPROBS:
            self.sampler.set_row(row, settings, seq.tokens)
        else:
            gen = torch.Generator(device=self.model.device)
            gen.manual_seed(settings.seed)
            seq.processors = processors_for(task_params, self._eos())
            seq.sampler = make_sampler(settings.temperature, settings.top_p, settings.min_p,
                                       settings.top_k, gen)
        self._next_uid += 1
        self.rows.append(seq)
        self._pending_input.append(toks[-1])
        return seq.uid

    def _prefill_row(self, task_params, toks, remaining, prefix_hit_length, row, progress,
                     on_prefill_progress) -> tuple[float, int]:
        """Fill row ``row`` up to the last-but-one prompt position: locally, or - for a long
        uncached remainder when the task names a prefill server - by fetching the KV over the
        wire (batch_generate.py:205-246; a failed fetch falls back to the local path).

        Two departures from the reference's call, both where it contradicts its own server
        (disaggregated/serve.py:43-58): the whole prompt is sent, not only the uncached
        remainder, because the server prefills ``token_ids`` as a complete prompt and
        ``start_pos`` only says which positions to ship; and whatever positions the reply
        leaves short of N-2 (the server stops a few positions early) are computed here, so
        the cache is complete whichever way it was filled."""
        use_remote = (len(remaining) > REMOTE_PREFILL_MIN_TOKENS
                      and task_params.prefill_endpoint is not None)
        if use_remote:
            from .disaggregated import remote_prefill
            t0 = time.perf_counter()
            try:
                remote_prefill(toks[:-1], self.cache, on_prefill_progress,
                               endpoint=task_params.prefill_endpoint, request_id=str(uuid.uuid4()),
                               model_id=str(task_params.model), start_pos=prefix_hit_length, row=row)
                have, need = self.cache.offsets[row], len(toks) - 2
                if have > need:
                    self.cache.trim(have - need, rows=range(row, row + 1))
                elif have < need:
                    self.model(torch.tensor([toks[have:need]], dtype=torch.int32), self.cache,
                               logits="none", rows=slice(row, row + 1))
                torch.cuda.synchronize()
                n = len(remaining) - 1
                return n / max(time.perf_counter() - t0, 1e-3), n
            except PrefillCancelled:
                raise
            except Exception:
                logger.warning("remote prefill failed, falling back to local prefill", exc_info=True)
                self.cache.offsets[row] = prefix_hit_length
                self.cache.sync_pos()
        return prefill(self.model, remaining[:-1], self.cache, progress, row=row, graph_steps=True)

    # ------------------------------------------------------------------ the step
    def _launch(self, from_host: bool) -> _Flight:
        """Enqueue one decode step for the current rows and the copy of its results into
        a pinned host buffer set.  ``from_host``: the input tokens are uploaded; otherwise
        they are where the previous replay of the same rows left them."""
        B = len(self.rows)
        bufs = self.model._buffers(B, 1)
        if from_host:
            bufs.tokens.copy_(torch.tensor(self._pending_input, dtype=torch.int32))
        want_top = any(s.want_top for s in self.rows)
        self.model.decode_step(self.cache, B, feedback=True, sampler=self.sampler,
                               mode=self.sampler.mode(B, want_top))
        slot, self._slot = self._slot, self._slot ^ 1
        h, d = self._host[slot], self.sampler
        h["token"][:B].copy_(d.token[:B], non_blocking=True)
        h["logprob"][:B].copy_(d.logprob[:B], non_blocking=True)
        if want_top:
            h["top_idx"][:B].copy_(d.top_idx[:B], non_blocking=True)
            h["top_val"][:B].copy_(d.top_val[:B], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        return _Flight(rows=list(self.rows), slot=slot, event=ev, want_top=want_top)

    def step(self) -> list[tuple[int, GenerationResponse]]:
        if not self.rows:
            self._flight = None
            return []
        if not all(s.on_device for s in self.rows):
            if self._flight is not None:  # drain the device-side chain first
                cur, self._flight = self._flight, None
                return self._collect(cur)
            return self._step_host()
        if self._flight is None:
            if self._sampler_stale:  # steps were taken on the host meanwhile
                for r, q in enumerate(self.rows):
                    self.sampler.set_row(r, q.settings, q.tokens, draws=q.stream.n_gen)
                self._sampler_stale = False
            self._flight = self._launch(from_host=True)
        cur = self._flight
        # the next replay goes out before this one is read, if the same rows will still be
        # there: nothing joined or left since the launch and nobody reaches its token limit
        same = len(cur.rows) == len(self.rows) and all(a is b for a, b in zip(cur.rows, self.rows))
        go_on = same and all(s.stream.n_gen + 2 <= s.stream.max_tokens for s in cur.rows)
        self._flight = self._launch(from_host=False) if go_on else None
        return self._collect(cur)

    def _collect(self, fl: _Flight) -> list[tuple[int, GenerationResponse]]:
        """Wait for a launched step and turn its tokens into responses."""
        fl.event.synchronize()
        h = self._host[fl.slot]
        B = len(fl.rows)
        toks = h["token"][:B].tolist()
        lps = h["logprob"][:B].tolist()
        now = time.perf_counter()
        out: list[tuple[int, GenerationResponse]] = []
        finished: list[_Seq] = []
        for r, seq in enumerate(fl.rows):
            cur_row = next((i for i, s in enumerate(self.rows) if s is seq), None)
            if cur_row is None:
                continue  # finished or cancelled while this step was in flight
            tok = int(toks[r])
            logprob = top = None
            if seq.want_top:
                logprob = float(lps[r])
                top = seq.stream.top_items(h["top_idx"][r].tolist(), h["top_val"][r].tolist(), seq.k_top)
            seq.tokens.append(tok)
            self._pending_input[cur_row] = tok
            resp = seq.stream.push(tok, now, logprob, top)
            if seq.on_generation_token is not None:
                seq.on_generation_token()
            out.append((seq.uid, resp))
            if resp.finish_reason is not None:
                finished.append(seq)
        self._drop_rows([i for i, s in enumerate(self.rows) if any(s is f for f in finished)])
        if not self.rows:
            self._flight = None
        return out

    def _step_host(self) -> list[tuple[int, GenerationResponse]]:
        """A step with the processors and samplers of every row run on the host with torch:
        taken only while a row's settings are outside what the sampling kernels accept."""
        B = len(self.rows)
        self._sampler_stale = True
        bufs = self.model._buffers(B, 1)
        bufs.tokens.copy_(torch.tensor(self._pending_input, dtype=torch.int32))
        bufs = self.model.decode_step(self.cache, B)
        greedy_tokens = bufs.next_token.tolist()  # synchronises
        now = time.perf_counter()
        out: list[tuple[int, GenerationResponse]] = []
        finished: list[int] = []
        for r, seq in enumerate(self.rows):
            logits = bufs.logits[r : r + 1].float()
            if seq.on_device:  # its settings on the host all the same, for this step
                procs = processors_for(seq.params, self._eos())
                if seq.settings.temperature == 0 and not procs:
                    tok, logprobs = int(greedy_tokens[r]), None
                else:
                    for p in procs:
                        logits = p(torch.tensor(seq.tokens), logits)
                    logprobs = logits - torch.logsumexp(logits, dim=-1, keepdim=True)
                    gen = torch.Generator(device=self.model.device)
                    gen.manual_seed(seq.settings.seed + seq.stream.n_gen)
                    tok = int(make_sampler(seq.settings.temperature, seq.settings.top_p,
                                           seq.settings.min_p, seq.settings.top_k, gen)(logprobs)[0])
            else:
                for p in seq.processors:
                    logits = p(torch.tensor(seq.tokens), logits)
                logprobs = logits - torch.logsumexp(logits, dim=-1, keepdim=True)
                tok = int(seq.sampler(logprobs)[0])
            logprob = top = None
            if seq.want_top:
                if logprobs is None:
                    logprobs = logits - torch.logsumexp(logits, dim=-1, keepdim=True)
                logprob, top = extract_top_logprobs(logprobs[0], self.tokenizer, seq.k_top, tok)
            seq.tokens.append(tok)
            self._pending_input[r] = tok
            resp = seq.stream.push(tok, now, logprob, top)
            if seq.on_generation_token is not None:
                seq.on_generation_token()
            out.append((seq.uid, resp))
            if resp.finish_reason is not None:
                finished.append(r)
        self._drop_rows(finished)
        return out

    def _drop_rows(self, rows: list[int]) -> None:
        for r in sorted(rows, reverse=True):
            last = len(self.rows) - 1
            if r != last:  # keep active rows compact: move the last row into the hole
                self.cache.copy_row(last, r)
                if self.rows[last].on_device:
                    self.sampler.move_row(last, r)
                self.rows[r] = self.rows[last]
                self._pending_input[r] = self._pending_input[last]
            self.rows.pop()
            self._pending_input.pop()

    def cancel(self, uids: list[int]) -> None:
        self._drop_rows([r for r, s in enumerate(self.rows) if s.uid in set(uids)])
        if not self.rows:
            self._flight = None

    def close(self) -> None:
        self.rows.clear()
        self._pending_input.clear()
        self._flight = None
        self.cache = None  # type: ignore[assignment]


# ----------------------------------------------------------------------- Engine


def map_responses_to_chunks(r: GenerationResponse, model_id: str) -> TokenChunk:
    return TokenChunk(model=model_id, text=r.text, token_id=r.token, usage=r.usage,
                      finish_reason=r.finish_reason, stats=r.stats, logprob=r.logprob,
                      top_logprobs=r.top_logprobs, is_thinking=r.is_thinking)


def _prompt_of(tokenizer, params: TextGenerationTaskParams):
    """The reference renders ``params.input`` through the tokenizer's chat template
    (apply_chat_template, utils_mlx.py:413-510).  Here: a list of ints is taken as token
    ids; strings / message dicts are joined and encoded as plain text."""
    inp = params.input
    if inp and all(isinstance(t, int) for t in inp):
        return list(inp)
    parts = []
    for m in inp:
        parts.append(m if isinstance(m, str) else str(m.get("content", "")) if isinstance(m, dict)
                     else str(getattr(m, "content", m)))
    return "\n".join(parts)


@dataclass(eq=False)
class BatchGenerator(Engine):
    model: ShardModel
    tokenizer: Any
    model_id: str
    device_rank: int = 0
    cancel_receiver: Any = None
    event_sender: Any = None
    check_for_cancel_every: int = 50
    max_seq: int = 8192
    kv_prefix_cache: KVPrefixCache | None = None
    gen_factory: Any = None  # tests inject a fake inner generator (like the reference's FakeExoBatchGenerator)
    _cancelled_tasks: set = field(default_factory=set, init=False)
    _all_tasks: dict = field(default_factory=dict, init=False)
    _queue: deque = field(default_factory=deque, init=False)
    _active_tasks: dict = field(default_factory=dict, init=False)
    _prefill_cache: Any = field(default=None, init=False)

    def __post_init__(self) -> None:
        if self.gen_factory is not None:
            self._gen = self.gen_factory()
        else:
            self._gen = ShardBatchGenerator(self.model, self.tokenizer, EXO_MAX_CONCURRENT_REQUESTS,
                                            self.max_seq, self.kv_prefix_cache)

    def warmup(self) -> None:
        """generate.py:399-462: a short greedy generation on a fixed prompt; sets how
        often a running generation checks for cancellation (about once per second)."""
        params = TextGenerationTaskParams(model=self.model_id, max_output_tokens=50, temperature=0.0,
                                          bench=True)
        prompt = [1 % self.model.cfg.vocab_size] * 16
        uid = self._gen.submit(params, prompt)
        t0 = time.perf_counter()
        n = 0
        while self._gen.has_work:
            self._gen.step()
            n += 1
        dt = time.perf_counter() - t0
        del uid
        self.check_for_cancel_every = max(1, min(100, int(n / dt))) if dt > 0 else 50

    def submit(self, task: GenerationTask) -> None:
        self._cancelled_tasks.discard(CANCEL_ALL_TASKS)
        self._all_tasks[task.task_id] = task
        self._queue.append(task)

    def agree_on_cancellations(self) -> None:
        if self.cancel_receiver is None:
            return
        for task_id in self.cancel_receiver.collect():
            if task_id == CANCEL_ALL_TASKS:
                self._cancelled_tasks.add(CANCEL_ALL_TASKS)
            elif task_id in self._all_tasks:
                self._cancelled_tasks.add(task_id)

    def step(self):
        while self._queue and len(self._active_tasks) < EXO_MAX_CONCURRENT_REQUESTS:
            task = self._queue.popleft()
            try:
                uid = self._start_task(task)
            except PrefillCancelled:
                continue
            except Exception as e:
                self._send_error(task, e)
                raise
            self._active_tasks[uid] = task
        if not self._gen.has_work:
            return list(self._apply_cancellations())
        try:
            results = self._gen.step()
        except Exception as e:
            for task in self._active_tasks.values():
                self._send_error(task, e)
            raise
        output: list[tuple[Any, Any]] = []
        for uid, response in results:
            task = self._active_tasks.get(uid)
            if task is None:
                continue
            if self.device_rank == 0:
                output.append((task.task_id, map_responses_to_chunks(response, self.model_id)))
            if response.finish_reason is not None:
                output.append((task.task_id, FinishedResponse()))
                del self._active_tasks[uid]
        output.extend(self._apply_cancellations())
        return output

    def _apply_cancellations(self):
        if not self._cancelled_tasks:
            return []
        cancel_all = CANCEL_ALL_TASKS in self._cancelled_tasks
        uids, results = [], []
        for uid, task in list(self._active_tasks.items()):
            if task.task_id in self._cancelled_tasks or cancel_all:
                uids.append(uid)
                results.append((task.task_id, CancelledResponse()))
                del self._active_tasks[uid]
        if uids:
            self._gen.cancel(uids)
        done = {tid for tid, _ in results}
        for tid in self._cancelled_tasks:
            if tid != CANCEL_ALL_TASKS and tid not in done:
                results.append((tid, CancelledResponse()))
        self._cancelled_tasks.clear()
        return results

    def _send_error(self, task: GenerationTask, e: Exception) -> None:
        if self.device_rank == 0 and self.event_sender is not None:
            self.event_sender.send(
                (task.command_id, ErrorChunk(model=self.model_id, error_message=str(e))))

    def _start_task(self, task: GenerationTask) -> int:
        prompt = _prompt_of(self.tokenizer, task.task_params)

        def on_prefill_progress(processed: int, total: int) -> None:
            if self.device_rank == 0 and self.event_sender is not None:
                self.event_sender.send(
                    (task.command_id, PrefillProgressChunk(self.model_id, processed, total)))

        def distributed_prompt_progress_callback() -> None:
            self.agree_on_cancellations()
            if self.should_cancel(task.task_id):
                raise PrefillCancelled()

        since = self.check_for_cancel_every

        def on_generation_token() -> None:
            nonlocal since
            since += 1
            if since >= self.check_for_cancel_every:
                since = 0
                self.agree_on_cancellations()

        return self._gen.submit(task.task_params, prompt, on_prefill_progress,
                                distributed_prompt_progress_callback, on_generation_token)

    def close(self) -> None:
        self._gen.close()
        self.model = None  # type: ignore[assignment]
        self.tokenizer = None

    def serve_prefill(self, request, wfile) -> None:
        """Prefill ``request.token_ids`` and stream the KV to ``wfile`` in the reference's
        wire format (batch_generator.py:558-572).  Runs on the engine's thread in a KV row
        of its own, so running generations are not disturbed."""
        from .disaggregated import run_prefill_for_request, write_cache_to_wire
        n = len(request.token_ids)
        if n > self.max_seq:
            raise ValueError(f"prefill request of {n} tokens exceeds the cache ({self.max_seq})")
        if self._prefill_cache is None:
            self._prefill_cache = self.model.make_cache(1, self.max_seq)
        cache = run_prefill_for_request(model=self.model, kv_prefix_cache=self.kv_prefix_cache,
                                        request=request, cache=self._prefill_cache, row=0)
        write_cache_to_wire(wfile, cache, row=0, request_id=request.request_id,
                            model_id=request.model_id, start_pos=request.start_pos)


@dataclass(eq=False)
class SequentialGenerator(Engine):
    """One request at a time through ``generate()``: the reference's SequentialGenerator
    (src/exo/worker/runner/llm_inference/batch_generator.py:90-318), which its builder picks
    when EXO_NO_BATCH is set (src/exo/worker/engines/mlx/builder.py:86-99).  A step yields the
    next token of the running request; the step after its last token yields
    FinishedResponse and starts the next queued request.  Cancellation is looked at every
    ``check_for_cancel_every`` tokens and between prefill chunks."""

    model: ShardModel
    tokenizer: Any
    model_id: str
    device_rank: int = 0
    cancel_receiver: Any = None
    event_sender: Any = None
    check_for_cancel_every: int = 50
    max_seq: int = 8192
    kv_prefix_cache: KVPrefixCache | None = None
    _cancelled_tasks: set = field(default_factory=set, init=False)
    _all_tasks: dict = field(default_factory=dict, init=False)
    _queue: deque = field(default_factory=deque, init=False)
    _active: Any = field(default=None, init=False)  # (task, generator)
    _prefill_cache: Any = field(default=None, init=False)
    _state: Any = field(default=None, init=False)   # GenerateState

    def _eos(self) -> list[int]:
        return list(getattr(self.tokenizer, "eos_token_ids", None) or [])

    def warmup(self) -> None:
        params = TextGenerationTaskParams(model=self.model_id, max_output_tokens=50, temperature=0.0,
                                          bench=True)
        prompt = [1 % self.model.cfg.vocab_size] * 16
        t0 = time.perf_counter()
        if self._state is None:
            self._state = GenerateState(self.model, self.max_seq)
        n = sum(1 for _ in generate(self.model, self.tokenizer, params, prompt,
                                    eos_token_ids=self._eos(), state=self._state))
        dt = time.perf_counter() - t0
        self.check_for_cancel_every = max(1, min(100, int(n / dt))) if dt > 0 else 50

    def submit(self, task: GenerationTask) -> None:
        self._cancelled_tasks.discard(CANCEL_ALL_TASKS)
        self._all_tasks[task.task_id] = task
        self._queue.append(task)

    def agree_on_cancellations(self) -> None:
        if self.cancel_receiver is None:
            return
        for task_id in self.cancel_receiver.collect():
            if task_id == CANCEL_ALL_TASKS:
                self._cancelled_tasks.add(CANCEL_ALL_TASKS)
            elif task_id in self._all_tasks:
                self._cancelled_tasks.add(task_id)

    def _cancelled(self):
        out = [(tid, CancelledResponse()) for tid in self._cancelled_tasks if tid != CANCEL_ALL_TASKS]
        self._cancelled_tasks.clear()
        return out

    def step(self):
        if self._active is None:
            if not self._queue:
                self.agree_on_cancellations()
                return self._cancelled()
            self._start_next()
        task, gen = self._active
        output: list[tuple[Any, Any]] = []
        try:
            response = next(gen)
            if self.device_rank == 0:
                output.append((task.task_id, map_responses_to_chunks(response, self.model_id)))
        except (StopIteration, PrefillCancelled):
            output.append((task.task_id, FinishedResponse()))
            self._active = None
            self._all_tasks.pop(task.task_id, None)
            if self._queue:
                self._start_next()
        except Exception as e:
            self._send_error(task, e)
            self._active = None
            raise
        return output + self._cancelled()

    def _start_next(self) -> None:
        task = self._queue.popleft()
        try:
            self._active = (task, self._build_generator(task))
        except Exception as e:
            self._send_error(task, e)
            raise

    def _send_error(self, task: GenerationTask, e: Exception) -> None:
        if self.device_rank == 0 and self.event_sender is not None:
            self.event_sender.send(
                (task.command_id, ErrorChunk(model=self.model_id, error_message=str(e))))

    def _build_generator(self, task: GenerationTask):
        prompt = _prompt_of(self.tokenizer, task.task_params)
        if isinstance(prompt, str):
            prompt = self.tokenizer.encode(prompt)

        def check_cancel() -> None:
            self.agree_on_cancellations()
            if self.should_cancel(task.task_id):
                raise PrefillCancelled()

        def on_prefill_progress(processed: int, total: int) -> None:
            if self.device_rank == 0 and self.event_sender is not None:
                self.event_sender.send(
                    (task.command_id, PrefillProgressChunk(self.model_id, processed, total)))
            check_cancel()

        since = self.check_for_cancel_every

        def on_generation_token() -> None:
            nonlocal since
            since += 1
            if since >= self.check_for_cancel_every:
                since = 0
                check_cancel()

        if self._state is None:  # one cache row and sampler for all requests: graphs stay valid
            self._state = GenerateState(self.model, self.max_seq)
        return generate(self.model, self.tokenizer, task.task_params, list(prompt), on_prefill_progress,
                        on_generation_token, eos_token_ids=self._eos(),
                        kv_prefix_cache=self.kv_prefix_cache, state=self._state)

    def close(self) -> None:
        self._active = None
        self._state = None
        self.model = None  # type: ignore[assignment]
        self.tokenizer = None

    def serve_prefill(self, request, wfile) -> None:
        BatchGenerator.serve_prefill(self, request, wfile)  # the same KV row of its own


# ----------------------------------------------------------------------- Builder


def build_model_path(model_id: str) -> Path:
    """src/exo/download/download_utils.py:152-178: first directory that holds the model
    among EXO_MODELS_READ_ONLY_DIRS, EXO_MODELS_DIRS, else EXO_DEFAULT_MODELS_DIR."""
    name = model_id.replace("/", "--")
    cands = []
    for var in ("EXO_MODELS_READ_ONLY_DIRS", "EXO_MODELS_DIRS"):
        cands += [Path(p) / name for p in os.environ.get(var, "").split(":") if p]
    default = Path(os.environ.get("EXO_DEFAULT_MODELS_DIR", str(Path.home() / ".exo" / "models")))
    cands.append(default / name)
    for c in cands:
        if (c / "config.json").exists():
            return c
    return cands[-1]


@dataclass
class Mi355xBuilder(Builder):
    model_id: str
    event_sender: Any = None
    cancel_receiver: Any = None
    device: str = "cuda:0"
    max_seq: int = 8192
    inference_model: ShardModel | None = None
    tokenizer: Any = None

    def connect(self, bound_instance: BoundInstance) -> None:
        if bound_instance.bound_shard.world_size != 1:
            raise NotImplementedError(
                "this engine serves single-device instances; multi-device groups are not wired")

    def load(self, bound_instance: BoundInstance) -> Generator[ModelLoadingResponse, None, None]:
        shard = bound_instance.bound_shard
        if shard.immediate_exception:
            raise RuntimeError("immediate_exception requested by shard metadata")
        path = Path(bound_instance.model_path) if bound_instance.model_path else build_model_path(
            shard.model_id)
        cfg = ModelConfig.from_path(path)
        if shard.n_layers != cfg.num_hidden_layers:
            raise ValueError(f"shard says {shard.n_layers} layers, checkpoint has {cfg.num_hidden_layers}")
        it = load_shard_weights(path, cfg, shard.start_layer, shard.end_layer, self.device)
        try:
            while True:
                done, total = next(it)
                yield ModelLoadingResponse(layers_loaded=done, total=total)
        except StopIteration as stop:
            weights = stop.value
        self.inference_model = ShardModel(cfg, weights, shard.start_layer, shard.end_layer, self.device)
        self.tokenizer = load_tokenizer(path, cfg.vocab_size)

    def build(self) -> Engine:
        assert self.inference_model is not None
        if os.environ.get("EXO_NO_BATCH"):  # builder.py:86-99
            return SequentialGenerator(model=self.inference_model, tokenizer=self.tokenizer,
                                       model_id=self.model_id, device_rank=0,
                                       cancel_receiver=self.cancel_receiver,
                                       event_sender=self.event_sender, max_seq=self.max_seq,
                                       kv_prefix_cache=KVPrefixCache(None, self.device))
        return BatchGenerator(model=self.inference_model, tokenizer=self.tokenizer,
                              model_id=self.model_id, device_rank=0,
                              cancel_receiver=self.cancel_receiver, event_sender=self.event_sender,
                              max_seq=self.max_seq,
                              kv_prefix_cache=KVPrefixCache(None, self.device))  # builder.py:83

    def close(self) -> None:
        self.inference_model = None
        self.tokenizer = None
