"""KV prefix cache: keep the K/V of finished prefills in HBM and start a later request
from the longest stored prompt prefix.

Host-side mirror of ``KVPrefixCache`` (src/exo/worker/engines/mlx/cache.py:232-471) for
the plain-KV model families of this engine (every layer is a trimmable ``KVCache``, so
the reference's snapshot machinery for SSM / rotating caches has no counterpart here):

* ``add_kv_cache`` / ``update_kv_cache`` store a detached copy of one pool row
  (cache.py:255-302: ``deepcopy(cache)``);
* ``get_kv_cache`` picks the entry with the longest common token prefix; a match of the
  whole prompt (``>= len-1`` tokens) is an *exact* hit and is cut back to ``len-1`` so
  that at least one token remains to be fed (cache.py:321-393);
* entries are evicted least-recently-used first while memory use is above
  ``EXO_MEMORY_THRESHOLD`` (cache.py:433-456).  The reference watches host RAM because
  the Mac's memory is unified; here the KV lives in HBM, so the pressure signal is the
  device's used fraction.

Stored layout: per layer one bf16 tensor ``[2, Hkv, n, D]`` (keys, values) holding just
the ``n`` valid positions, contiguous, so an entry costs exactly its tokens and a restore
is ``2 * L`` strided device copies into the pool row.
"""

from __future__ import annotations

import gc
import os
from dataclasses import dataclass

import numpy as np
import torch

from .cache import ShardKVCache


def _default_memory_threshold(total_bytes: int) -> float:
    """cache.py:36-44, applied to the device's memory size."""
    total_gb = total_bytes / 1e9
    if total_gb >= 128:
        return 0.85
    if total_gb >= 64:
        return 0.80
    if total_gb >= 32:
        return 0.75
    return 0.70


def memory_threshold(device=None) -> float:
    env = os.environ.get("EXO_MEMORY_THRESHOLD")
    if env is not None:
        return float(env)
    if torch.cuda.is_available():
        return _default_memory_threshold(torch.cuda.mem_get_info(device)[1])
    return 0.85


def get_memory_used_percentage(device=None) -> float:
    """Used fraction (0..1) of the device's memory (cache.py:554-557 reads host RAM)."""
    free, total = torch.cuda.mem_get_info(device)
    return 1.0 - free / total


def get_prefix_length(prompt, cached_prompt) -> int:
    """Length of the common prefix of two token sequences (cache.py:538-546)."""
    a = np.asarray(prompt, dtype=np.int64).reshape(-1)
    b = np.asarray(cached_prompt, dtype=np.int64).reshape(-1)
    n = min(a.shape[0], b.shape[0])
    if n == 0:
        return 0
    neq = np.nonzero(a[:n] != b[:n])[0]
    return int(neq[0]) if neq.size else n


@dataclass
class StoredKV:
    """One entry: the first ``length`` positions of every local layer."""

    layers: list[torch.Tensor]  # per layer [2, Hkv, length, D] bf16
    length: int

    @property
    def offset(self) -> int:
        return self.length

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.layers)


def snapshot_row(cache: ShardKVCache, row: int) -> StoredKV:
    n = cache.offsets[row]
    layers = [torch.stack((k[row, :, :n], v[row, :, :n])) for k, v in zip(cache.k, cache.v)]
    return StoredKV(layers, n)


def restore_row(stored: StoredKV, cache: ShardKVCache, row: int, length: int) -> None:
    """Write the first ``length`` stored positions into pool row ``row`` and set its fill
    level (the reference deep-copies the entry and trims the copy, cache.py:377-387)."""
    if length > stored.length:
        raise ValueError(f"restore of {length} positions from an entry of {stored.length}")
    if length > cache.max_seq:
        raise ValueError(f"restore of {length} positions into a cache of {cache.max_seq}")
    if len(stored.layers) != len(cache.k):
        raise ValueError("stored entry and cache differ in layer count")
    for kv, k, v in zip(stored.layers, cache.k, cache.v):
        k[row, :, :length].copy_(kv[0, :, :length])
        v[row, :, :length].copy_(kv[1, :, :length])
    cache.offsets[row] = length
    cache.sync_pos()


def cache_length(entry) -> int:
    """cache.py:533-535 for a stored entry or a live cache."""
    if isinstance(entry, StoredKV):
        return entry.length
    return max((c.offset for c in entry), default=0)


class KVPrefixCache:
    def __init__(self, group=None, device=None):
        if group is not None:
            raise ValueError("one GPU: no process group")
        self.prompts: list[np.ndarray] = []
        self.caches: list[StoredKV] = []
        self._last_used: list[float] = []
        self.prefill_tps: list[float] = []
        self._access_counter = 0
        self._device = device

    def clear(self) -> None:
        self.prompts.clear()
        self.caches.clear()
        self._last_used.clear()
        self.prefill_tps.clear()

    # ------------------------------------------------------------------ store
    def add_kv_cache(self, prompt_tokens, cache: ShardKVCache, row: int = 0,
                     prefill_tps: float = 0.0) -> None:
        """Add a new entry; evicts LRU entries first if memory is high (cache.py:255-272)."""
        self._evict_if_needed()
        self.prompts.append(np.asarray(prompt_tokens, dtype=np.int64).reshape(-1).copy())
        self.caches.append(snapshot_row(cache, row))
        self.prefill_tps.append(prefill_tps)
        self._access_counter += 1
        self._last_used.append(self._access_counter)

    def update_kv_cache(self, index: int, prompt_tokens, cache: ShardKVCache, row: int = 0,
                        restore_pos: int = 0, prefill_tps: float = 0.0) -> None:
        """Replace entry ``index`` in place (cache.py:274-302; ``restore_pos`` only selects
        snapshots there, and plain KV has none)."""
        self.prompts[index] = np.asarray(prompt_tokens, dtype=np.int64).reshape(-1).copy()
        self.caches[index] = snapshot_row(cache, row)
        self.prefill_tps[index] = prefill_tps
        self._access_counter += 1
        self._last_used[index] = self._access_counter

    # ------------------------------------------------------------------ fetch
    def get_kv_cache(self, cache: ShardKVCache, prompt_tokens, row: int = 0,
                     ) -> tuple[ShardKVCache, list[int], int | None, bool]:
        """Prepare pool row ``row`` for ``prompt_tokens``: restore the best stored prefix
        (or reset the row) and return ``(cache, remaining_tokens, matched_index,
        is_exact)`` as cache.py:321-393 does."""
        toks = np.asarray(prompt_tokens, dtype=np.int64).reshape(-1)
        max_length = int(toks.shape[0])
        best_index: int | None = None
        best_length = 0
        is_exact = False
        for i, cached_prompt in enumerate(self.prompts):
            length = get_prefix_length(toks, cached_prompt)
            if length >= max_length - 1 and length > 0:
                best_index, best_length, is_exact = i, length, True
                break
            if length > best_length:
                best_index, best_length = i, length
        if best_index is None:
            cache.reset(rows=range(row, row + 1))
            return cache, toks.tolist(), None, False
        stored = self.caches[best_index]
        desired = (max_length - 1) if is_exact else best_length
        restore_pos = min(stored.length, desired)
        restore_row(stored, cache, row, restore_pos)
        self._access_counter += 1
        self._last_used[best_index] = self._access_counter
        return cache, toks[restore_pos:].tolist(), best_index, is_exact

    # --------------------------------------------------------------- eviction
    def _evict_if_needed(self) -> None:
        if not self.caches:
            return
        evicted = False
        threshold = memory_threshold(self._device)
        while self.caches and self.get_memory_used_percentage() > threshold:
            lru = self._last_used.index(min(self._last_used))
            for lst in (self.prompts, self.caches, self._last_used, self.prefill_tps):
                lst.pop(lru)
            evicted = True
        if evicted:
            gc.collect()
            if torch.cuda.is_available():
                torch.cuda.empty_cache()  # hand the freed blocks back (mx.clear_cache there)

    def get_memory_used_percentage(self) -> float:
        return get_memory_used_percentage(self._device)

    def nbytes(self) -> int:
        return sum(c.nbytes() for c in self.caches)


MIN_PREFIX_HIT_RATIO_TO_UPDATE = 0.5  # generator/batch_generate.py:61
MIN_PREFIX_HIT_LENGTH = 1000          # generator/batch_generate.py:268-270


def save_prefix_cache(kv_prefix_cache: KVPrefixCache | None, all_prompt_tokens,
                      cache: ShardKVCache, row: int, prefix_hit_length: int,
                      matched_index: int | None,
                      min_prefix_hit_length: int = MIN_PREFIX_HIT_LENGTH,
                      prefill_tps: float = 0.0) -> None:
    """Store the freshly prefilled row: update the matched entry in place when the hit
    was long (>= min length and >= half the prompt), else add a new entry
    (generator/batch_generate.py:493-535)."""
    if kv_prefix_cache is None:
        return
    n = len(all_prompt_tokens)
    hit_ratio = prefix_hit_length / n if n > 0 else 0.0
    if matched_index is not None and prefix_hit_length >= min_prefix_hit_length \
            and hit_ratio >= MIN_PREFIX_HIT_RATIO_TO_UPDATE:
        kv_prefix_cache.update_kv_cache(matched_index, all_prompt_tokens, cache, row,
                                        restore_pos=prefix_hit_length, prefill_tps=prefill_tps)
    else:
        kv_prefix_cache.add_kv_cache(all_prompt_tokens, cache, row, prefill_tps=prefill_tps)
