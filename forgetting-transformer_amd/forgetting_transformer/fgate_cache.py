"""Key / value / forget-gate cache of the FoX layer for decoding, grown in place.

Mirrors ``FgateDynamicCache`` of the reference
(``src/forgetting_transformer/model/forgetting_transformer/fgate_cache.py:5-203``): the same
attributes and methods, called by the layer as ``past_key_values.update(k, v, log_fgate, layer_idx)``
(``modeling_forgetting_transformer.py:356-357``), ``get_seq_length`` (``:329-330``) and
``key_shift_cache`` / ``value_shift_cache`` (``:298-299``, ``:715-719``).

The reference appends with ``torch.cat`` (``fgate_cache.py:107-116``), which copies the whole cache
of a layer at every step: at 32768 cached tokens of 16 heads x 128 and batch 16 that is 8 GiB of
traffic per layer per token, more than twice what the attention itself reads.  Here every layer owns
buffers with spare capacity along the sequence axis, ``(batch, heads, capacity, head_dim)`` and
``(batch, heads, capacity)``; ``update`` copies only the new tokens behind the cached ones and hands
back views of the filled part.  The views have the reference's shapes; their (batch, head) slices
are ``capacity`` rows apart instead of ``seq_len``, which ``forgetting_attention`` takes as it takes
any strided input.  When a layer runs out of capacity its buffers are reallocated ``growth`` times
larger (amortised constant cost per token); with ``max_length`` given they are allocated once at that
size and never move.  Depends on nothing but torch.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch

__all__ = ["FgateDynamicCache"]


def _round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


class FgateDynamicCache:
    """Per-layer key, value and log-forget-gate states ``[batch, heads, seq_len, head_dim]`` /
    ``[batch, heads, seq_len]``, plus the token-shift states of the key and value projections."""

    def __init__(self, max_length: Optional[int] = None, growth: float = 2.0, min_capacity: int = 256) -> None:
        assert growth > 1.0, "growth must be above 1"
        assert max_length is None or max_length > 0
        self.max_length = max_length
        self.growth = float(growth)
        self.min_capacity = int(min_capacity)
        # the filled parts, as views of the buffers below (same names and meaning as in the reference)
        self.key_cache: List[torch.Tensor] = []
        self.value_cache: List[torch.Tensor] = []
        self.log_fgate_cache: List[torch.Tensor] = []
        self.key_shift_cache: List[torch.Tensor] = []
        self.value_shift_cache: List[torch.Tensor] = []
        self._key_buf: List[torch.Tensor] = []
        self._value_buf: List[torch.Tensor] = []
        self._log_fgate_buf: List[torch.Tensor] = []
        self._seen_tokens = 0   # what generate() has pushed through layer 0 so far

    # ------------------------------------------------------------------ the reference's interface
    def update_shift_cache(self, key_shift_state: torch.Tensor, value_shift_state: torch.Tensor, layer_idx):
        assert layer_idx == len(self.key_shift_cache) == len(self.value_shift_cache)
        self.key_shift_cache.append(key_shift_state)
        self.value_shift_cache.append(value_shift_state)

    def __getitem__(self, layer_idx: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        if layer_idx < len(self):
            return (self.key_cache[layer_idx], self.value_cache[layer_idx], self.log_fgate_cache[layer_idx])
        raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer_idx}")

    def __iter__(self):
        for layer_idx in range(len(self)):
            yield (self.key_cache[layer_idx], self.value_cache[layer_idx], self.log_fgate_cache[layer_idx])

    def __len__(self):
        return len(self.key_cache)

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, log_fgate_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """Append the new tokens of layer ``layer_idx`` and return that layer's keys, values and log forget gates,
        cached and new (``fgate_cache.py:78-118``)."""
        assert log_fgate_states.ndim == 3, f"log_fgate must be (B, H, T), but get {log_fgate_states.size()}"
        assert key_states.ndim == 4 and key_states.shape == value_states.shape
        assert log_fgate_states.shape == key_states.shape[:3], "log_fgate must be (B, H, T) like the keys"
        assert layer_idx <= len(self), "layers must be added in order"
        new = key_states.shape[-2]
        if layer_idx == 0:
            self._seen_tokens += new
        old = self.get_seq_length(layer_idx)
        self._reserve(layer_idx, old + new, key_states, value_states, log_fgate_states)
        self._key_buf[layer_idx][:, :, old:old + new].copy_(key_states)
        self._value_buf[layer_idx][:, :, old:old + new].copy_(value_states)
        self._log_fgate_buf[layer_idx][:, :, old:old + new].copy_(log_fgate_states)
        self._set_length(layer_idx, old + new)
        return self.key_cache[layer_idx], self.value_cache[layer_idx], self.log_fgate_cache[layer_idx]

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        if len(self.key_cache) <= layer_idx:
            return 0
        return self.key_cache[layer_idx].shape[-2]

    def get_max_length(self) -> Optional[int]:
        """None unless the cache was built with ``max_length`` (the reference's cache has no maximum)."""
        return self.max_length

    def to_legacy_cache(self) -> Tuple[Tuple[torch.Tensor, torch.Tensor, torch.Tensor], ...]:
        return tuple((self.key_cache[i], self.value_cache[i], self.log_fgate_cache[i]) for i in range(len(self)))

    @classmethod
    def from_legacy_cache(cls, past_key_values=None, num_layers: Optional[int] = None) -> "FgateDynamicCache":
        raise NotImplementedError   # as in the reference (fgate_cache.py:137-141)

    def crop(self, max_length: int):
        """Keep the first ``max_length`` tokens (a negative value removes that many from the end); the buffers stay."""
        if max_length < 0:
            max_length = self.get_seq_length() - abs(max_length)
        if self.get_seq_length() <= max_length:
            return
        self._seen_tokens = max_length
        for idx in range(len(self)):
            self._set_length(idx, max_length)

    def batch_split(self, full_batch_size: int, split_size: int) -> List["FgateDynamicCache"]:
        out = []
        for i in range(0, full_batch_size, split_size):
            part = FgateDynamicCache(self.max_length, self.growth, self.min_capacity)
            part._seen_tokens = self._seen_tokens
            for idx in range(len(self)):
                n = self.get_seq_length(idx)
                # views of the filled part only: a split has no spare capacity of the parent's to write into, so its
                # first update moves it to a buffer of its own and neither cache sees the other's later tokens
                part._adopt(self._key_buf[idx][i:i + split_size, :, :n], self._value_buf[idx][i:i + split_size, :, :n],
                            self._log_fgate_buf[idx][i:i + split_size, :, :n], n)
            out.append(part)
        return out

    @classmethod
    def from_batch_splits(cls, splits: List["FgateDynamicCache"]) -> "FgateDynamicCache":
        cache = cls(splits[0].max_length, splits[0].growth, splits[0].min_capacity)
        for idx in range(len(splits[0])):
            cache.update(torch.cat([s.key_cache[idx] for s in splits], dim=0),
                         torch.cat([s.value_cache[idx] for s in splits], dim=0),
                         torch.cat([s.log_fgate_cache[idx] for s in splits], dim=0), idx)
        return cache

    def batch_repeat_interleave(self, repeats: int):
        for idx in range(len(self)):
            n = self.get_seq_length(idx)
            self._replace(idx, *(b.repeat_interleave(repeats, dim=0) for b in self._buffers(idx)), n)

    def batch_select_indices(self, indices: torch.Tensor):
        for idx in range(len(self)):
            n = self.get_seq_length(idx)
            self._replace(idx, *(b[indices, ...] for b in self._buffers(idx)), n)

    # ------------------------------------------------------------------ capacity
    def capacity(self, layer_idx: int = 0) -> int:
        """Tokens layer ``layer_idx`` can hold before its buffers are reallocated."""
        return self._key_buf[layer_idx].shape[-2] if layer_idx < len(self._key_buf) else 0

    def reserve(self, length: int) -> None:
        """Make room for ``length`` tokens in every layer the cache already holds."""
        for idx in range(len(self)):
            self._reserve(idx, length, *self._buffers(idx))

    def _buffers(self, idx):
        return self._key_buf[idx], self._value_buf[idx], self._log_fgate_buf[idx]

    def _set_length(self, idx: int, n: int) -> None:
        views = (self._key_buf[idx][:, :, :n], self._value_buf[idx][:, :, :n], self._log_fgate_buf[idx][:, :, :n])
        for store, view in zip((self.key_cache, self.value_cache, self.log_fgate_cache), views):
            if idx < len(store):
                store[idx] = view
            else:
                store.append(view)

    def _adopt(self, k, v, g, n: int) -> None:
        self._key_buf.append(k)
        self._value_buf.append(v)
        self._log_fgate_buf.append(g)
        self._set_length(len(self._key_buf) - 1, n)

    def _replace(self, idx: int, k, v, g, n: int) -> None:
        self._key_buf[idx], self._value_buf[idx], self._log_fgate_buf[idx] = k, v, g
        self._set_length(idx, n)

    def _reserve(self, idx: int, need: int, k_like, v_like, g_like) -> None:
        if self.max_length is not None and need > self.max_length:
            raise ValueError(f"the cache was built for {self.max_length} tokens, {need} were requested")
        have = self.capacity(idx)
        if idx < len(self._key_buf) and need <= have:
            return
        if self.max_length is not None:
            cap = self.max_length
        else:   # rows in multiples of 64: whole key tiles of the attention kernels
            cap = _round_up(max(need, int(have * self.growth), self.min_capacity), 64)
        B, H, _, D = k_like.shape
        k = torch.empty((B, H, cap, D), dtype=k_like.dtype, device=k_like.device)
        v = torch.empty((B, H, cap, D), dtype=v_like.dtype, device=v_like.device)
        g = torch.empty((B, H, cap), dtype=g_like.dtype, device=g_like.device)
        if idx < len(self._key_buf):
            n = self.get_seq_length(idx)
            k[:, :, :n].copy_(self.key_cache[idx])
            v[:, :, :n].copy_(self.value_cache[idx])
            g[:, :, :n].copy_(self.log_fgate_cache[idx])
            self._replace(idx, k, v, g, n)
        else:
            self._adopt(k, v, g, 0)
