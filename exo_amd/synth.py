"""Random-weight checkpoints in the MLX layout, for benchmarks and tests.

Every matrix is drawn N(0, 0.02) in float32 from a per-tensor seeded generator, cast
to bf16 and affine-quantised (group 64); norm weights are 1.  Tensor names are the
mlx_lm module paths the reference touches (src/exo/worker/engines/mlx/
auto_parallel.py:209-243,638-648,792-800,1249-1259).  Random streams differ between
CPU and GPU generators; a checkpoint written to disk is the portable artefact.
"""

from __future__ import annotations

import json
import zlib
from pathlib import Path

import torch

from .config import ModelConfig
from .quantize import quantize


def _seed(base: int, name: str) -> int:
    return (zlib.crc32(name.encode()) ^ (base * 0x9E3779B1)) & 0x7FFFFFFF


def _qlinear(out: dict, name: str, n: int, k: int, cfg: ModelConfig, base_seed: int, device,
             experts: int = 0, std: float = 0.02) -> None:
    gen = torch.Generator(device=device)
    gen.manual_seed(_seed(base_seed, name))
    rows = n * max(experts, 1)
    w = torch.empty(rows, k, dtype=torch.float32, device=device)
    # drawn in slabs to bound the float32 transient
    slab = max(1, (1 << 28) // k)
    for r0 in range(0, rows, slab):
        w[r0 : r0 + slab].normal_(0.0, std, generator=gen)
    wq, s, b = quantize(w.bfloat16().float(), cfg.group_size, cfg.bits_for(name))
    del w
    if experts:
        wq = wq.reshape(experts, n, -1)
        s = s.reshape(experts, n, -1)
        b = b.reshape(experts, n, -1)
    out[name + ".weight"] = wq
    out[name + ".scales"] = s
    out[name + ".biases"] = b


def synth_weights(cfg: ModelConfig, start_layer: int = 0, end_layer: int | None = None,
                  seed: int = 0, device="cpu") -> dict[str, torch.Tensor]:
    """Weights of the shard [start_layer, end_layer) plus the layer-independent tensors
    that shard needs (embedding on the first, final norm + lm_head on the last)."""
    end_layer = cfg.num_hidden_layers if end_layer is None else end_layer
    H, D = cfg.hidden_size, cfg.head_dim
    out: dict[str, torch.Tensor] = {}
    ones = lambda n: torch.ones(n, dtype=torch.bfloat16, device=device)  # noqa: E731
    first, last = start_layer == 0, end_layer == cfg.num_hidden_layers
    if first or (last and cfg.tie_word_embeddings):
        _qlinear(out, "model.embed_tokens", cfg.vocab_size, H, cfg, seed, device)
    for i in range(start_layer, end_layer):
        p = f"model.layers.{i}."
        out[p + "input_layernorm.weight"] = ones(H)
        out[p + "post_attention_layernorm.weight"] = ones(H)
        _qlinear(out, p + "self_attn.q_proj", cfg.num_attention_heads * D, H, cfg, seed, device)
        _qlinear(out, p + "self_attn.k_proj", cfg.num_key_value_heads * D, H, cfg, seed, device)
        _qlinear(out, p + "self_attn.v_proj", cfg.num_key_value_heads * D, H, cfg, seed, device)
        _qlinear(out, p + "self_attn.o_proj", H, cfg.num_attention_heads * D, cfg, seed, device)
        if cfg.is_moe:
            out[p + "self_attn.q_norm.weight"] = ones(D)
            out[p + "self_attn.k_norm.weight"] = ones(D)
            E, Ie = cfg.num_experts, cfg.moe_intermediate_size
            _qlinear(out, p + "mlp.gate", E, H, cfg, seed, device)
            _qlinear(out, p + "mlp.switch_mlp.gate_proj", Ie, H, cfg, seed, device, experts=E)
            _qlinear(out, p + "mlp.switch_mlp.up_proj", Ie, H, cfg, seed, device, experts=E)
            _qlinear(out, p + "mlp.switch_mlp.down_proj", H, Ie, cfg, seed, device, experts=E)
        else:
            I = cfg.intermediate_size
            _qlinear(out, p + "mlp.gate_proj", I, H, cfg, seed, device)
            _qlinear(out, p + "mlp.up_proj", I, H, cfg, seed, device)
            _qlinear(out, p + "mlp.down_proj", H, I, cfg, seed, device)
    if last:
        out["model.norm.weight"] = ones(H)
        if not cfg.tie_word_embeddings:
            _qlinear(out, "lm_head", cfg.vocab_size, H, cfg, seed, device)
    return out


def write_checkpoint(path: str | Path, cfg: ModelConfig, seed: int = 0, device="cpu") -> Path:
    """Write ``config.json`` + ``model.safetensors`` (packed words as U32, like MLX)."""
    from safetensors.torch import save_file

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    w = synth_weights(cfg, seed=seed, device=device)
    tensors = {}
    for k, v in w.items():
        v = v.cpu().contiguous()
        tensors[k] = v.view(torch.uint32) if v.dtype == torch.int32 else v
    save_file(tensors, str(path / "model.safetensors"), metadata={"format": "mlx"})
    with open(path / "config.json", "w") as f:
        json.dump(cfg.to_dict(), f, indent=1)
    return path
