"""Model configuration parsed from an MLX checkpoint's ``config.json``.

Field names follow the Hugging Face / mlx_lm config keys the reference's model cards
and loaders rely on (resources/inference_model_cards/*.toml; mlx_lm ``ModelArgs``
reached through src/exo/worker/engines/mlx/utils_mlx.py:163-229).
"""

from __future__ import annotations

import json
from dataclasses import asdict, dataclass
from pathlib import Path

SUPPORTED_MODEL_TYPES = ("llama", "qwen3_moe")


@dataclass
class ModelConfig:
    model_type: str
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: dict | None = None
    tie_word_embeddings: bool = False
    group_size: int = 64
    bits: int = 4
    num_experts: int = 0
    num_experts_per_tok: int = 0
    moe_intermediate_size: int = 0
    norm_topk_prob: bool = True
    # per-module-path entries of config.json's "quantization" map (mlx_lm writes one for
    # every module converted at another width than the default, e.g. a MoE router kept
    # at 8 bits): path -> {"group_size", "bits"}.  The engine itself takes each tensor's
    # width from its shapes; this map only drives weight synthesis and round-trips.
    quant_overrides: dict | None = None

    def __post_init__(self):
        if self.model_type not in SUPPORTED_MODEL_TYPES:
            raise ValueError(
                f"model_type {self.model_type!r} not supported (have {SUPPORTED_MODEL_TYPES})"
            )
        if self.group_size != 64 or self.bits not in (4, 8):
            raise ValueError(
                f"only affine group_size=64 bits in (4,8) supported, got "
                f"group_size={self.group_size} bits={self.bits}"
            )

    @property
    def is_moe(self) -> bool:
        return self.model_type == "qwen3_moe"

    def bits_for(self, path: str) -> int:
        """Bit width of the module at ``path`` (e.g. ``model.layers.3.mlp.gate``)."""
        o = (self.quant_overrides or {}).get(path)
        return int(o["bits"]) if o else self.bits

    @staticmethod
    def from_dict(d: dict) -> "ModelConfig":
        q = d.get("quantization") or d.get("quantization_config") or {}
        hd = d.get("head_dim") or d["hidden_size"] // d["num_attention_heads"]
        return ModelConfig(
            model_type=d["model_type"],
            hidden_size=d["hidden_size"],
            num_hidden_layers=d["num_hidden_layers"],
            num_attention_heads=d["num_attention_heads"],
            num_key_value_heads=d.get("num_key_value_heads", d["num_attention_heads"]),
            head_dim=hd,
            intermediate_size=d.get("intermediate_size", 0),
            vocab_size=d["vocab_size"],
            rms_norm_eps=d.get("rms_norm_eps", 1e-5),
            rope_theta=d.get("rope_theta", 10000.0),
            rope_scaling=d.get("rope_scaling"),
            tie_word_embeddings=d.get("tie_word_embeddings", False),
            group_size=q.get("group_size", 64),
            bits=q.get("bits", 4),
            num_experts=d.get("num_experts", 0),
            num_experts_per_tok=d.get("num_experts_per_tok", 0),
            moe_intermediate_size=d.get("moe_intermediate_size", 0),
            norm_topk_prob=d.get("norm_topk_prob", True),
            quant_overrides={k: v for k, v in q.items() if isinstance(v, dict)} or None,
        )

    @staticmethod
    def from_path(model_dir: str | Path) -> "ModelConfig":
        with open(Path(model_dir) / "config.json") as f:
            return ModelConfig.from_dict(json.load(f))

    def to_dict(self) -> dict:
        d = asdict(self)
        d["quantization"] = {"group_size": d.pop("group_size"), "bits": d.pop("bits"),
                             **(d.pop("quant_overrides") or {})}
        return d


LLAMA3_SCALING = {
    "rope_type": "llama3",
    "low_freq_factor": 1.0,
    "high_freq_factor": 4.0,
    "original_max_position_embeddings": 8192,
}


def named_config(name: str) -> ModelConfig:
    """Architectures of the benchmark configurations (random-weight stand-ins)."""
    if name == "llama-3.2-1b":
        return ModelConfig("llama", 2048, 16, 32, 8, 64, 8192, 128256, 1e-5, 5e5,
                           dict(LLAMA3_SCALING, factor=32.0), True, 64, 4)
    if name == "llama-3.1-8b":
        return ModelConfig("llama", 4096, 32, 32, 8, 128, 14336, 128256, 1e-5, 5e5,
                           dict(LLAMA3_SCALING, factor=8.0), False, 64, 4)
    if name == "qwen3-30b-a3b":
        return ModelConfig("qwen3_moe", 2048, 48, 32, 4, 128, 6144, 151936, 1e-6, 1e6, None,
                           False, 64, 4, 128, 8, 768, True)
    if name == "qwen3-235b-a22b":
        return ModelConfig("qwen3_moe", 4096, 94, 64, 4, 128, 12288, 151936, 1e-6, 5e6, None,
                           False, 64, 8, 128, 8, 1536, True)
    raise KeyError(name)
