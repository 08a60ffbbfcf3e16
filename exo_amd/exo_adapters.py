"""The two adapters between this engine's plain dataclasses and exo's pydantic events.

exo's runner sends ``ChunkGenerated(command_id, chunk)`` events whose ``chunk`` is one of
the pydantic models of ``src/exo/shared/types/chunks.py:19-95`` and builds its engine from
a pydantic ``BoundInstance`` (``src/exo/worker/runner/bootstrap.py:67-86``).  The engine in
this package emits ``(command_id, chunk)`` tuples of the dataclasses in ``exo_amd.types``
(same field names) and takes ``exo_amd.types.BoundInstance``.  The functions here convert
between the two.  They never import exo: the caller passes exo's modules (or any namespace
with classes of the same names and fields), so this module loads - and is tested - where
exo itself is not installed.

    from exo.shared.types import chunks, events
    from exo.shared.types.memory import Memory
    sender = ExoEventSender(event_sender, events, chunks, memory_cls=Memory)
    builder = Mi355xBuilder(model_id, sender, cancel_receiver)
"""
from __future__ import annotations

import dataclasses
from typing import Any

from . import types as T


def _usage_fields(u: T.Usage) -> dict[str, Any]:
    """exo nests the two detail counters (``src/exo/api/types/api.py:118-135``)."""
    return {
        "prompt_tokens": u.prompt_tokens,
        "completion_tokens": u.completion_tokens,
        "total_tokens": u.total_tokens,
        "prompt_tokens_details": {"cached_tokens": u.cached_tokens},
        "completion_tokens_details": {"reasoning_tokens": u.reasoning_tokens},
    }


def _stats_fields(s: T.GenerationStats, memory_cls) -> dict[str, Any]:
    """``peak_memory_usage`` is a ``Memory`` model over there (``shared/types/memory.py:7-13``),
    a byte count here."""
    d = dataclasses.asdict(s)
    d["peak_memory_usage"] = (memory_cls.from_bytes(s.peak_memory_usage) if memory_cls is not None
                              else {"in_bytes": s.peak_memory_usage})
    return d


def to_exo_chunk(chunk, chunks_mod, memory_cls=None):
    """A ``TokenChunk`` / ``ErrorChunk`` / ``PrefillProgressChunk`` of ``exo_amd.types`` as the
    class of the same name in ``chunks_mod`` (``src/exo/shared/types/chunks.py:23-95``)."""
    name = type(chunk).__name__
    if name not in ("TokenChunk", "ErrorChunk", "PrefillProgressChunk"):
        raise TypeError(f"not a chunk of this engine: {type(chunk)!r}")
    cls = getattr(chunks_mod, name)
    fields: dict[str, Any] = {}
    for f in dataclasses.fields(chunk):
        v = getattr(chunk, f.name)
        if isinstance(v, T.Usage):
            v = _usage_fields(v)
        elif isinstance(v, T.GenerationStats):
            v = _stats_fields(v, memory_cls)
        elif f.name == "top_logprobs" and v is not None:
            v = [dataclasses.asdict(t) for t in v]
        fields[f.name] = v
    return cls(**fields)


class ExoEventSender:
    """Wraps exo's ``event_sender`` for ``Mi355xBuilder``: ``send((command_id, chunk))``
    becomes ``event_sender.send(ChunkGenerated(command_id=..., chunk=...))``
    (``src/exo/shared/types/events.py:93-95``, what ``runner.py:388-394`` sends).  Anything
    that is not such a tuple is passed through unchanged."""

    def __init__(self, event_sender, events_mod, chunks_mod, memory_cls=None):
        self._sender = event_sender
        self._events = events_mod
        self._chunks = chunks_mod
        self._memory = memory_cls

    def send(self, item) -> None:
        if (isinstance(item, tuple) and len(item) == 2 and dataclasses.is_dataclass(item[1])
                and type(item[1]).__name__ in ("TokenChunk", "ErrorChunk", "PrefillProgressChunk")):
            command_id, chunk = item
            item = self._events.ChunkGenerated(
                command_id=command_id, chunk=to_exo_chunk(chunk, self._chunks, self._memory))
        self._sender.send(item)


def to_amd_bound_instance(bound_instance, model_path: str) -> T.BoundInstance:
    """exo's pydantic ``BoundInstance`` (``bound_shard`` with the pipeline shard's layer range,
    ``src/exo/shared/types/worker/shards.py``) as ``exo_amd.types.BoundInstance`` plus the
    resolved checkpoint directory."""
    sh = bound_instance.bound_shard
    model_id = getattr(getattr(sh, "model_card", None), "model_id", None) or getattr(sh, "model_id")
    return T.BoundInstance(
        T.ShardMetadata(str(model_id), sh.start_layer, sh.end_layer, sh.n_layers,
                        getattr(sh, "device_rank", 0), getattr(sh, "world_size", 1),
                        getattr(sh, "immediate_exception", False), getattr(sh, "should_timeout", None)),
        model_path=str(model_path))
