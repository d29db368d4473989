"""What each layer of a model keeps between steps.

A model may expose `cache_specs()` returning one spec per layer; the model
runner allocates the tensors and hands layer i its entry of `kv_caches`:

  PagedKV          (k_cache, v_cache), each [blocks, n_kv, block, head_dim]
  PagedLatent      one tensor [blocks, block, width] (a shared row per token)
  RecurrentState   one fp32 tensor [state_slots, heads, dim, vdim]; a
                   sequence owns one slot for its whole life
  SharedCache      the very tensor of an earlier layer (read-only user)

Models without `cache_specs()` get PagedKV for every layer.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List


@dataclass(frozen=True)
class PagedKV:
    n_kv: int
    head_dim: int

    def block_bytes(self, block_size: int, dtype_bytes: int) -> int:
        return 2 * self.n_kv * block_size * self.head_dim * dtype_bytes


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
class SharedCache:
    source: int

    def block_bytes(self, block_size: int, dtype_bytes: int) -> int:
        return 0


def default_specs(cfg, n_kv_local: int) -> List[PagedKV]:
    return [PagedKV(n_kv_local, cfg.head_dim) for _ in range(cfg.num_layers)]


def needs_state_slots(specs) -> bool:
    return any(isinstance(s, RecurrentState) for s in specs)
