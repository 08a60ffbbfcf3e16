"""KV cache for one shard: one plain bf16 cache per LOCAL layer.

Mirrors what the reference builds with ``make_kv_cache`` (src/exo/worker/engines/mlx/
cache.py:560-581: ``[KVCache() for _ in model.layers]``) and the parts of mlx_lm's
``KVCache`` the engine touches (``offset``, ``trim``, ``is_trimmable``;
.typings/mlx_lm/models/cache.pyi:150-169).

HBM layout: per layer two tensors ``[B, Hkv, S_max, D]`` bf16, preallocated (no
growth steps, no reallocation while decoding, so a captured HIP graph stays valid).
The per-sequence fill level lives twice: ``pos`` int32 ``[B]`` on the device (read by
the RoPE/append and attention kernels, advanced on the device) and ``offsets`` on the
host (what ``offset`` / ``cache_length`` report).
"""

from __future__ import annotations

import torch


class LayerKV:
    """The per-layer entry of the cache list."""

    def __init__(self, owner: "ShardKVCache", index: int):
        self._owner = owner
        self.index = index

    @property
    def keys(self) -> torch.Tensor:
        return self._owner.k[self.index]

    @property
    def values(self) -> torch.Tensor:
        return self._owner.v[self.index]

    @property
    def offset(self) -> int:
        return max(self._owner.offsets, default=0)

    def is_trimmable(self) -> bool:
        return True

    def trim(self, n: int) -> int:
        """Entries are trimmed together (every layer holds the same tokens); the call on
        layer 0 performs it and the other layers report the same count, so the
        reference's ``for c in cache: c.trim(2)`` loop trims by 2, not 2*L."""
        if self.index == 0:
            self._owner._last_trim = self._owner.trim(n)
        return self._owner._last_trim


class ShardKVCache(list):
    """list[LayerKV] plus the shared storage."""

    def __init__(self, n_layers: int, batch: int, n_kv_heads: int, head_dim: int,
                 max_seq: int, device):
        super().__init__(LayerKV(self, i) for i in range(n_layers))
        self.batch, self.max_seq = batch, max_seq
        shape = (batch, n_kv_heads, max_seq, head_dim)
        self.k = [torch.zeros(shape, dtype=torch.bfloat16, device=device) for _ in range(n_layers)]
        self.v = [torch.zeros(shape, dtype=torch.bfloat16, device=device) for _ in range(n_layers)]
        self.pos = torch.zeros(batch, dtype=torch.int32, device=device)
        self.offsets = [0] * batch
        self._last_trim = 0

    # -- fill level
    def advance_host(self, t: int, rows=None) -> None:
        for r in (range(self.batch) if rows is None else rows):
            self.offsets[r] += t

    def sync_pos(self) -> None:
        """Push the host offsets to the device copy."""
        self.pos.copy_(torch.tensor(self.offsets, dtype=torch.int32), non_blocking=False)

    def trim(self, n: int, rows=None) -> int:
        rows = range(self.batch) if rows is None else rows
        n = min([n] + [self.offsets[r] for r in rows])
        for r in rows:
            self.offsets[r] -= n
        self.sync_pos()
        return n

    def reset(self, rows=None) -> None:
        for r in (range(self.batch) if rows is None else rows):
            self.offsets[r] = 0
        self.sync_pos()

    def nbytes(self) -> int:
        return sum(t.numel() * 2 for t in self.k) * 2

    def copy_row(self, src: int, dst: int) -> None:
        """Move one sequence's cache to another batch row (slot compaction)."""
        n = self.offsets[src]
        for k, v in zip(self.k, self.v):
            k[dst, :, :n].copy_(k[src, :, :n])
            v[dst, :, :n].copy_(v[src, :, :n])
        self.offsets[dst] = n
        self.sync_pos()


def cache_length(cache) -> int:
    """src/exo/worker/engines/mlx/cache.py:533-535."""
    return max((c.offset for c in cache), default=0)
