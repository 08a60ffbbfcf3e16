"""The exo-side adapters (exo_amd/exo_adapters.py) against pydantic stand-ins that declare the
fields of exo's own models: chunks (src/exo/shared/types/chunks.py:19-95), the nested API types
(src/exo/api/types/api.py:101-170), ChunkGenerated (shared/types/events.py:93-95) and Memory
(shared/types/memory.py:7-13).  exo itself needs Python 3.13 and is not importable here; the
stand-ins forbid unknown fields, so a renamed or missing field fails validation."""
import types as pytypes
from typing import Literal

import pytest
from pydantic import BaseModel, ConfigDict, ValidationError

from exo_amd import types as T
from exo_amd.exo_adapters import ExoEventSender, to_amd_bound_instance, to_exo_chunk


class _Strict(BaseModel):
    model_config = ConfigDict(extra="forbid")


class Memory(_Strict):
    in_bytes: int = 0

    @classmethod
    def from_bytes(cls, val):
        return cls(in_bytes=val)


class TopLogprobItem(_Strict):
    token: str
    logprob: float
    bytes: list[int] | None = None


class PromptTokensDetails(_Strict):
    cached_tokens: int = 0
    audio_tokens: int = 0


class CompletionTokensDetails(_Strict):
    reasoning_tokens: int = 0
    audio_tokens: int = 0
    accepted_prediction_tokens: int = 0
    rejected_prediction_tokens: int = 0


class Usage(_Strict):
    prompt_tokens: int
    completion_tokens: int
    total_tokens: int
    prompt_tokens_details: PromptTokensDetails
    completion_tokens_details: CompletionTokensDetails


class GenerationStats(_Strict):
    prompt_tps: float
    generation_tps: float
    prompt_tokens: int
    generation_tokens: int
    peak_memory_usage: Memory
    prefix_cache_hit: Literal["none", "partial", "exact"] = "none"


class TokenChunk(_Strict):
    model: str
    text: str
    token_id: int
    usage: Usage | None
    finish_reason: Literal["stop", "length", "content_filter"] | None = None
    stats: GenerationStats | None = None
    logprob: float | None = None
    top_logprobs: list[TopLogprobItem] | None = None
    is_thinking: bool = False


class ErrorChunk(_Strict):
    model: str
    error_message: str
    finish_reason: Literal["error"] = "error"


class PrefillProgressChunk(_Strict):
    model: str
    processed_tokens: int
    total_tokens: int


class ChunkGenerated(_Strict):
    command_id: str
    chunk: TokenChunk | ErrorChunk | PrefillProgressChunk


CHUNKS = pytypes.SimpleNamespace(TokenChunk=TokenChunk, ErrorChunk=ErrorChunk,
                                 PrefillProgressChunk=PrefillProgressChunk)
EVENTS = pytypes.SimpleNamespace(ChunkGenerated=ChunkGenerated)


def test_token_chunk_with_every_field():
    c = T.TokenChunk(
        model="m", text="hi", token_id=7,
        usage=T.Usage(prompt_tokens=10, completion_tokens=3, total_tokens=13, cached_tokens=4, reasoning_tokens=1),
        finish_reason="length",
        stats=T.GenerationStats(prompt_tps=100.0, generation_tps=50.0, prompt_tokens=10, generation_tokens=3,
                                peak_memory_usage=123456, prefix_cache_hit="partial"),
        logprob=-0.5, top_logprobs=[T.TopLogprobItem("a", -0.5, [97]), T.TopLogprobItem("b", -1.5)],
        is_thinking=False)
    for mem in (Memory, None):
        e = to_exo_chunk(c, CHUNKS, memory_cls=mem)
        assert isinstance(e, TokenChunk)
        assert (e.model, e.text, e.token_id, e.finish_reason, e.logprob) == ("m", "hi", 7, "length", -0.5)
        assert e.usage.total_tokens == 13 and e.usage.prompt_tokens_details.cached_tokens == 4
        assert e.usage.completion_tokens_details.reasoning_tokens == 1
        assert e.stats.peak_memory_usage.in_bytes == 123456 and e.stats.prefix_cache_hit == "partial"
        assert [(t.token, t.logprob, t.bytes) for t in e.top_logprobs] == [("a", -0.5, [97]), ("b", -1.5, None)]


def test_plain_token_error_and_progress_chunks():
    e = to_exo_chunk(T.TokenChunk(model="m", text="x", token_id=1), CHUNKS)
    assert e.usage is None and e.stats is None and e.finish_reason is None and e.top_logprobs is None
    e = to_exo_chunk(T.ErrorChunk(model="m", error_message="boom"), CHUNKS)
    assert isinstance(e, ErrorChunk) and e.error_message == "boom" and e.finish_reason == "error"
    e = to_exo_chunk(T.PrefillProgressChunk(model="m", processed_tokens=5, total_tokens=9), CHUNKS)
    assert isinstance(e, PrefillProgressChunk) and (e.processed_tokens, e.total_tokens) == (5, 9)
    with pytest.raises(TypeError):
        to_exo_chunk(T.Usage(1, 1, 2), CHUNKS)
    with pytest.raises(ValidationError):  # a finish reason exo does not know is refused by exo's model
        to_exo_chunk(T.TokenChunk(model="m", text="x", token_id=1, finish_reason="weird"), CHUNKS)


def test_event_sender_wraps_chunks_and_passes_the_rest():
    sent = []
    s = ExoEventSender(pytypes.SimpleNamespace(send=sent.append), EVENTS, CHUNKS, memory_cls=Memory)
    s.send(("cmd-1", T.TokenChunk(model="m", text="x", token_id=1)))
    s.send(("cmd-1", T.PrefillProgressChunk(model="m", processed_tokens=1, total_tokens=2)))
    other = object()
    s.send(other)
    assert isinstance(sent[0], ChunkGenerated) and sent[0].command_id == "cmd-1" and sent[0].chunk.token_id == 1
    assert isinstance(sent[1].chunk, PrefillProgressChunk)
    assert sent[2] is other


def test_bound_instance():
    card = pytypes.SimpleNamespace(model_id="org/model-4bit")
    shard = pytypes.SimpleNamespace(model_card=card, start_layer=12, end_layer=24, n_layers=48, device_rank=1,
                                    world_size=4, immediate_exception=False, should_timeout=None)
    b = to_amd_bound_instance(pytypes.SimpleNamespace(bound_shard=shard), "/models/x")
    assert isinstance(b, T.BoundInstance) and b.model_path == "/models/x"
    sm = b.bound_shard
    assert (sm.model_id, sm.start_layer, sm.end_layer, sm.n_layers, sm.device_rank, sm.world_size) == (
        "org/model-4bit", 12, 24, 48, 1, 4)
    assert not sm.is_first_layer
