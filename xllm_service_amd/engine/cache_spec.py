"""What each layer of a model keeps between steps.

A model may expose `cache_specs()` returning one spec per layer; the model
runner allocates the tensors and hands layer i its entry of `kv_caches`:

  PagedKV          (k_cache, v_cache), [blocks, n_kv, block, head_dim] (the
                   value cache has v_dim in place of head_dim when given;
                   with values_are_keys there is one tensor, handed out as
                   both members of the pair)
  PagedLatent      one tensor [blocks, block, width] (a shared row per token)
  RecurrentState   one fp32 tensor [state_slots, heads, dim, vdim]; a
                   sequence owns one slot for its whole life
  ConvState        one tensor [state_slots, taps - 1, channels] in the model
                   dtype: the last inputs of a short causal convolution
  SharedCache      the very tensor of an earlier layer (read-only user)
  CacheGroup       a tuple of the above for a layer that keeps several things
                   (its entry of `kv_caches` is the tuple of their tensors)

Models without `cache_specs()` get PagedKV for every layer.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Tuple


@dataclass(frozen=True)
class PagedKV:
    n_kv: int
    head_dim: int
    v_dim: Optional[int] = None          # None: values as wide as keys
    values_are_keys: bool = False        # the layer reads its keys as values

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_dim is None else self.v_dim

    def block_bytes(self, block_size: int, dtype_bytes: int) -> int:
        per_token = self.head_dim + (0 if self.values_are_keys
                                     else self.value_dim)
        return self.n_kv * block_size * per_token * dtype_bytes


@dataclass(frozen=True)
class PagedLatent:
    width: int

    def block_bytes(self, block_size: int, dtype_bytes: int) -> int:
        return block_size * self.width * dtype_bytes


@dataclass(frozen=True)
class RecurrentState:
    heads: int
    dim: int
    vdim: int

    def block_bytes(self, block_size: int, dtype_bytes: int) -> int:
        return 0

    def slot_bytes(self) -> int:
        return 4 * self.heads * self.dim * self.vdim


@dataclass(frozen=True)
class ConvState:
    channels: int
    taps: int

    def block_bytes(self, block_size: int, dtype_bytes: int) -> int:
        return 0

    def slot_bytes(self, dtype_bytes: int = 4) -> int:
        return dtype_bytes * self.channels * max(self.taps - 1, 0)


@dataclass(frozen=True)
class CacheGroup:
    parts: Tuple

    def block_bytes(self, block_size: int, dtype_bytes: int) -> int:
        return sum(p.block_bytes(block_size, dtype_bytes) for p in self.parts)

    def slot_bytes(self) -> int:
        return sum(p.slot_bytes() for p in self.parts
                   if hasattr(p, "slot_bytes"))


@dataclass(frozen=True)
class SharedCache:
    source: int

    def block_bytes(self, block_size: int, dtype_bytes: int) -> int:
        return 0


def default_specs(cfg, n_kv_local: int) -> List[PagedKV]:
    return [PagedKV(n_kv_local, cfg.head_dim) for _ in range(cfg.num_layers)]


def flat_specs(specs):
    """Every leaf spec, groups opened."""
    for s in specs:
        if isinstance(s, CacheGroup):
            yield from flat_specs(s.parts)
        else:
            yield s


def needs_state_slots(specs) -> bool:
    return any(isinstance(s, (RecurrentState, ConvState))
               for s in flat_specs(specs))
