"""Boundary data types of the engine, field-for-field subsets of the reference's
pydantic models (plain dataclasses here; exo's own objects duck-type onto them):

  GenerationResponse / FinishedResponse / CancelledResponse / ModelLoadingResponse
      src/exo/shared/types/worker/runner_response.py:19-81
  GenerationStats, Usage              src/exo/api/types/api.py:130-169
  TextGenerationTaskParams            src/exo/shared/types/text_generation.py:102-136
  ShardMetadata                       src/exo/shared/types/worker/shards.py:15-62
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass
class GenerationStats:
    prompt_tps: float
    generation_tps: float
    prompt_tokens: int
    generation_tokens: int
    peak_memory_usage: int  # bytes
    prefix_cache_hit: str = "none"


@dataclass
class Usage:
    prompt_tokens: int
    completion_tokens: int
    total_tokens: int
    cached_tokens: int = 0
    reasoning_tokens: int = 0


@dataclass
class TopLogprobItem:
    token: str
    logprob: float
    bytes: list[int] | None = None


@dataclass
class GenerationResponse:
    text: str
    token: int
    logprob: float | None = None
    top_logprobs: list[TopLogprobItem] | None = None
    finish_reason: str | None = None  # "stop" | "length" | ...
    stats: GenerationStats | None = None
    usage: Usage | None = None
    is_thinking: bool = False


@dataclass
class FinishedResponse:
    pass


@dataclass
class CancelledResponse:
    pass


@dataclass
class ModelLoadingResponse:
    layers_loaded: int
    total: int


@dataclass
class PrefillProgressResponse:
    processed_tokens: int
    total_tokens: int


@dataclass
class TokenChunk:
    """src/exo/shared/types/chunks.py:23-95 (text generation subset)."""

    model: str
    text: str
    token_id: int
    usage: Usage | None = None
    finish_reason: str | None = None
    stats: GenerationStats | None = None
    logprob: float | None = None
    top_logprobs: list[TopLogprobItem] | None = None
    is_thinking: bool = False


@dataclass
class ErrorChunk:
    model: str
    error_message: str
    finish_reason: str = "error"


@dataclass
class PrefillProgressChunk:
    model: str
    processed_tokens: int
    total_tokens: int


@dataclass(frozen=True)
class TextGenerationTaskParams:
    model: str
    input: list[Any] = field(default_factory=list)
    max_output_tokens: int | None = None
    temperature: float | None = None
    top_p: float | None = None
    bench: bool = False
    use_prefix_cache: bool = False
    top_k: int | None = None
    stop: str | list[str] | None = None
    seed: int | None = None
    logprobs: bool = False
    top_logprobs: int | None = None
    min_p: float | None = None
    repetition_penalty: float | None = None
    repetition_context_size: int | None = None
    presence_penalty: float | None = None
    frequency_penalty: float | None = None
    prefill_endpoint: str | None = None  # "host:port" of a disaggregated-prefill server


@dataclass
class GenerationTask:
    """A TextGeneration task as the runner hands it to Engine.submit
    (src/exo/shared/types/tasks.py): id + params."""

    task_id: str
    command_id: str
    task_params: TextGenerationTaskParams


@dataclass
class ShardMetadata:
    """Half-open layer range [start_layer, end_layer) of n_layers."""

    model_id: str
    start_layer: int
    end_layer: int
    n_layers: int
    device_rank: int = 0
    world_size: int = 1
    immediate_exception: bool = False
    should_timeout: float | None = None

    @property
    def is_first_layer(self) -> bool:
        return self.start_layer == 0

    @property
    def is_last_layer(self) -> bool:
        return self.end_layer == self.n_layers


@dataclass
class BoundInstance:
    """src/exo/shared/types/worker/instances.py:42-51: the shard this runner owns."""

    bound_shard: ShardMetadata
    model_path: str | None = None  # resolved checkpoint directory

    @property
    def is_pipeline_or_single(self) -> bool:
        return True
