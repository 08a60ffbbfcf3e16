"""Load the tensors of one layer range from an MLX safetensors checkpoint directory.

Mirrors the reference's load step (src/exo/worker/engines/mlx/utils_mlx.py:163-286:
``load_model(path, lazy=True)`` then per-layer materialisation with progress), and
its rule for which tensors a shard needs (src/exo/download/huggingface_utils.py:
91-97,154-168): a key whose first all-digit dotted component lies in
[start_layer, end_layer) belongs to the shard; keys with no numeric component
(embedding, final norm, lm_head) are needed by every shard - of those this loader
keeps only what the shard's position uses.  Tensors go file -> (mmap) -> HBM one at
a time; there is never a full host copy of the checkpoint.
"""

from __future__ import annotations

import json
from collections.abc import Generator
from pathlib import Path

import torch

from .config import ModelConfig


def layer_index_of(key: str) -> int | None:
    for part in key.split("."):
        if part.isdigit():
            return int(part)
    return None


def _checkpoint_files(model_dir: Path) -> dict[str, Path]:
    """tensor name -> file, from the index if there is one."""
    idx = model_dir / "model.safetensors.index.json"
    if idx.exists():
        with open(idx) as f:
            wm = json.load(f)["weight_map"]
        return {k: model_dir / v for k, v in wm.items()}
    from safetensors import safe_open

    out: dict[str, Path] = {}
    files = sorted(model_dir.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors files under {model_dir}")
    for fp in files:
        with safe_open(str(fp), "pt") as f:
            for k in f.keys():
                out[k] = fp
    return out


def wanted(key: str, cfg: ModelConfig, start_layer: int, end_layer: int) -> bool:
    li = layer_index_of(key)
    if li is not None:
        return start_layer <= li < end_layer
    first, last = start_layer == 0, end_layer == cfg.num_hidden_layers
    if key.startswith("model.embed_tokens."):
        return first or (last and cfg.tie_word_embeddings)
    if key.startswith("model.norm.") or key.startswith("lm_head."):
        return last
    return False


def load_shard_weights(
    model_dir: str | Path, cfg: ModelConfig, start_layer: int, end_layer: int, device
) -> Generator[tuple[int, int], None, dict[str, torch.Tensor]]:
    """Generator: yields (layers_loaded, total_layers) after each local layer is
    resident (the reference's ModelLoadingResponse cadence, runner.py:263-269) and
    returns the name -> device tensor dict.  Packed words come back as int32."""
    from safetensors import safe_open

    model_dir = Path(model_dir)
    files = _checkpoint_files(model_dir)
    keys = [k for k in files if wanted(k, cfg, start_layer, end_layer)]
    if not keys:
        raise ValueError(f"checkpoint at {model_dir} holds no tensor of layers "
                         f"[{start_layer},{end_layer})")

    def order(k: str):
        li = layer_index_of(k)
        return (0, 0, k) if li is None else (1, li, k)

    keys.sort(key=order)
    out: dict[str, torch.Tensor] = {}
    handles: dict[Path, object] = {}
    total = end_layer - start_layer
    done_layer = None
    try:
        for k in keys:
            li = layer_index_of(k)
            if li is not None and done_layer is not None and li != done_layer:
                yield (done_layer - start_layer + 1, total)
            if li is not None:
                done_layer = li
            fp = files[k]
            if fp not in handles:
                handles[fp] = safe_open(str(fp), "pt")
            t = handles[fp].get_tensor(k)
            if t.dtype == torch.uint32:
                t = t.view(torch.int32)
            elif t.dtype in (torch.float16, torch.float32):
                t = t.to(torch.bfloat16)
            out[k] = t.to(device, non_blocking=False).contiguous()
        if done_layer is not None:
            yield (done_layer - start_layer + 1, total)
    finally:
        handles.clear()
    return out
