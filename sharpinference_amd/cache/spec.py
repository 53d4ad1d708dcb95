"""What a mixer asks of the cache manager.

Two kinds of per-request memory exist.  ``KVSpec``: keys and values that grow with the
sequence, kept in pages; a window tells which of them a later query can still see, so that
pages behind it go back to the pool.  ``StateSpec``: a block of fixed size per request (a
recurrent state, a convolution tail), kept in a slot
(reference: src/SharpInference.Engine/GdnStateCache.cs:7-33 for the fixed-size kind,
src/SharpInference.Engine/PagedKvCache.cs:20-110 for the paged kind).  A mixer that needs both
(attention behind short convolutions; attention beside a recurrent mixer) asks with a
``MixedSpec``: at most one ``KVSpec`` and any number of ``StateSpec``, which it finds again in
the order it gave them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

WINDOW_NONE, WINDOW_CHUNK, WINDOW_SLIDING = 0, 1, 2


@dataclass(frozen=True)
class KVSpec:
    """Paged keys and values of one layer.  ``head_dim`` is the width of a key; ``v_head_dim`` the
    width of a value where it differs (0: the same).  Keys are kept [page, kv head, position,
    head_dim], values transposed inside the page, [page, kv head, v_head_dim, position]."""

    num_kv_heads: int
    head_dim: int
    window_kind: int = WINDOW_NONE
    window: int = 0
    v_head_dim: int = 0
    values_in_keys: bool = False     # the values are a leading part of the key rows: no value tensor is kept

    @property
    def value_dim(self) -> int:
        return self.v_head_dim or self.head_dim

    @property
    def elements_per_token(self) -> int:
        """Cache elements one token takes in one layer of this kind."""
        return self.num_kv_heads * (self.head_dim + (0 if self.values_in_keys else self.value_dim))

    def first_visible(self, pos: int) -> int:
        """The earliest key position a query at `pos` can see."""
        if self.window_kind == WINDOW_CHUNK:
            return (pos // self.window) * self.window
        if self.window_kind == WINDOW_SLIDING:
            return max(0, pos - self.window + 1)
        return 0

    def group_key(self):
        # layers whose pages live and die together share a block table
        return ("kv", self.window_kind, self.window)


@dataclass(frozen=True)
class StateSpec:
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def group_key(self):
        return ("state",)


@dataclass(frozen=True)
class MixedSpec:
    """Paged keys and values and fixed-size states of one layer together."""

    kv: Optional[KVSpec]
    states: Tuple[StateSpec, ...] = ()

    def group_key(self):
        return self.kv.group_key() if self.kv is not None else ("state",)


def kv_of(spec) -> Optional[KVSpec]:
    """The paged part of what a layer asks for, if it has one."""
    if isinstance(spec, KVSpec):
        return spec
    return spec.kv if isinstance(spec, MixedSpec) else None


def states_of(spec) -> Tuple[StateSpec, ...]:
    """The fixed-size states a layer asks for, in its order."""
    if isinstance(spec, StateSpec):
        return (spec,)
    return tuple(spec.states) if isinstance(spec, MixedSpec) else ()


def combine_specs(specs) -> object:
    """One request for the memory of several mixers that share a layer: the one paged part among
    them and all their states, in order.  None if none of them keeps anything."""
    kvs = [kv_of(s) for s in specs if kv_of(s) is not None]
    if len(kvs) > 1:
        raise ValueError("a layer can hold the pages of one mixer only")
    states = tuple(st for s in specs for st in states_of(s))
    if not kvs and not states:
        return None
    if not states:
        return kvs[0]
    if not kvs and len(states) == 1:
        return states[0]
    return MixedSpec(kvs[0] if kvs else None, states)
