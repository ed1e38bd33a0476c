"""The kinds of memory a mixer may keep between steps, and what the engine binds to a run
of a layer for each.

A mixer names its need with an object (``KVCacheNeed``, ``StateNeed``, or one of a type
registered here); the type of that object selects a ``CacheKind``, which says how such
memory is sized, allocated, shared between runs and cleared for a new request.  Planning
and allocation (``cache.storage``) and the engine go through this registry only, so another
kind of memory (a latent cache, a ring of recent tokens) is registered, not patched in.

The reference plans its pools from per-class specs in the same spirit
(atom/model_ops/attentions/sub_pool_spec.py:49-246: STATE classes sized by
``max_num_seqs``, one PAGE class taking the rest).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..parts.base import KVCacheNeed, LatentCacheNeed, StateNeed


@dataclass
class KVBinding:
    """The pages of one run of a layer.  ``writes`` is False for a run that reads the
    keys and values another run wrote."""

    group: int
    k_cache: torch.Tensor  # [num_pages, Hkv, page_size, D]
    v_cache: torch.Tensor  # [num_pages, Hkv, D, page_size] (D: the value heads' size where it differs)
    writes: bool = True


@dataclass
class LatentBinding:
    """The pages of one run of a layer that keeps one row per token for all its heads."""

    group: int
    pages: torch.Tensor    # [num_pages, page_size, width]
    writes: bool = True


@dataclass
class StateBinding:
    """The per-request state of one run of a layer: ``state[slot]`` belongs to the request
    that holds ``slot``; it is zero when the request's first tokens arrive."""

    state: torch.Tensor  # [num_slots, *shape]


def _elem_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class CacheKind:
    """How one kind of memory is planned and bound.  ``paged`` kinds live in pages that the cache
    manager hands out per request (runs with the same ``window`` share block tables); the others hold
    a fixed amount per state slot."""

    paged = False

    def is_paged(self, need) -> bool:
        """Whether ``need`` lives in pages (the kind's ``paged`` unless a kind decides per need)."""
        return self.paged

    def window(self, need) -> int | None:
        """Paged kinds: how many of the latest tokens a later query can still see (None: all)."""
        return None

    def chunk(self, need) -> int | None:
        """Paged kinds: a later query sees only what its own run of this many positions (counted from position 0)
        holds (None: no such limit)."""
        return None

    def keeps_every_token(self, need) -> bool:
        """True if everything a request's earlier tokens left is still there later, in pages: only then
        can a new request take over pages that already hold its beginning (the prefix cache)."""
        return False

    def page_bytes(self, need, page_size: int, dtype: torch.dtype) -> int:
        return 0

    def request_bytes(self, need, dtype: torch.dtype) -> int:
        """Bytes held per state slot, whatever the context length."""
        return 0

    def allocate(self, need, *, group: int | None, num_pages: int, page_size: int, num_slots: int, device,
                 dtype: torch.dtype):
        raise NotImplementedError

    def share(self, binding):
        """What a run gets that reads the memory of the run that owns ``binding``."""
        raise ValueError(f"{type(self).__name__}: this kind of memory cannot be read from another run")

    def reset(self, binding, slots: torch.Tensor) -> None:
        """Clears the per-request part of ``binding`` for the state slots in ``slots`` (int64, on the device),
        whose requests start in the coming step."""


class PagedKeysValues(CacheKind):
    paged = True

    def window(self, need):
        return need.window

    def chunk(self, need):
        return need.chunk

    def keeps_every_token(self, need):
        return need.window is None and need.chunk is None

    def page_bytes(self, need, page_size, dtype):
        return need.num_kv_heads * (need.head_dim + (need.value_dim or need.head_dim)) * page_size * _elem_size(dtype)

    def allocate(self, need, *, group, num_pages, page_size, num_slots, device, dtype):
        k = torch.zeros((num_pages, need.num_kv_heads, page_size, need.head_dim), dtype=dtype, device=device)
        v = torch.zeros((num_pages, need.num_kv_heads, need.value_dim or need.head_dim, page_size), dtype=dtype,
                        device=device)
        return KVBinding(group, k, v, writes=True)

    def share(self, binding):
        return KVBinding(binding.group, binding.k_cache, binding.v_cache, writes=False)


class PagedLatents(CacheKind):
    """One row per token in pages, addressed through the same block tables as keys and values."""

    paged = True

    def window(self, need):
        return need.window

    def keeps_every_token(self, need):
        return need.window is None

    def page_bytes(self, need, page_size, dtype):
        return need.width * page_size * _elem_size(dtype)

    def allocate(self, need, *, group, num_pages, page_size, num_slots, device, dtype):
        return LatentBinding(group, torch.zeros((num_pages, page_size, need.width), dtype=dtype, device=device))

    def share(self, binding):
        return LatentBinding(binding.group, binding.pages, writes=False)


class SlotState(CacheKind):
    def request_bytes(self, need, dtype):
        n = 1
        for s in need.shape:
            n *= int(s)
        return n * _elem_size(need.dtype)

    def allocate(self, need, *, group, num_pages, page_size, num_slots, device, dtype):
        return StateBinding(torch.zeros((num_slots, *need.shape), dtype=need.dtype, device=device))

    def reset(self, binding, slots):
        binding.state.index_fill_(0, slots, 0)


@dataclass
class JointBinding:
    """What the branches of a layer whose mixers run side by side are bound to, in the branches' order (None for a
    branch that keeps nothing).  ``group`` is the paged branch's group."""

    parts: list
    group: int | None = None


class JointMemory(CacheKind):
    """The memory of mixers that run side by side (``parts.parallel.JointNeed``): each branch's need is sized,
    allocated, shared and cleared by the kind it names itself.  At most one branch keeps pages."""

    paged = True    # asked per need through ``is_paged``

    def _paged(self, need):
        found = [n for n in need.needs if n is not None and kind_of(n).is_paged(n)]
        if len(found) > 1:
            raise ValueError("mixers side by side: at most one of them may keep pages")
        return found[0] if found else None

    def is_paged(self, need):
        return self._paged(need) is not None

    def window(self, need):
        n = self._paged(need)
        return kind_of(n).window(n) if n is not None else None

    def chunk(self, need):
        n = self._paged(need)
        return kind_of(n).chunk(n) if n is not None else None

    def keeps_every_token(self, need):
        return all(kind_of(n).keeps_every_token(n) for n in need.needs if n is not None)

    def page_bytes(self, need, page_size, dtype):
        return sum(kind_of(n).page_bytes(n, page_size, dtype) for n in need.needs if n is not None)

    def request_bytes(self, need, dtype):
        return sum(kind_of(n).request_bytes(n, dtype) for n in need.needs if n is not None)

    def allocate(self, need, *, group, num_pages, page_size, num_slots, device, dtype):
        parts = []
        for n in need.needs:
            if n is None:
                parts.append(None)
                continue
            kind = kind_of(n)
            paged = kind.is_paged(n)
            parts.append(kind.allocate(n, group=group if paged else None, num_pages=num_pages if paged else 0,
                                       page_size=page_size if paged else 0, num_slots=num_slots, device=device,
                                       dtype=dtype))
        binding = JointBinding(parts, group)
        binding.kinds = [kind_of(n) if n is not None else None for n in need.needs]
        return binding

    def share(self, binding):
        raise ValueError("mixers side by side keep memory that another run cannot read")

    def reset(self, binding, slots):
        for kind, part in zip(binding.kinds, binding.parts):
            if part is not None:
                kind.reset(part, slots)


_KINDS: dict[type, CacheKind] = {}


def register_cache_kind(need_type: type, kind: CacheKind, *, replace: bool = False) -> None:
    if need_type in _KINDS and not replace:
        raise KeyError(f"a cache kind for {need_type.__name__} is already registered")
    _KINDS[need_type] = kind


def unregister_cache_kind(need_type: type) -> None:
    _KINDS.pop(need_type, None)


def kind_of(need) -> CacheKind | None:
    """The kind that handles ``need`` (None for a mixer that keeps nothing)."""
    if need is None:
        return None
    for cls in type(need).__mro__:
        if cls in _KINDS:
            return _KINDS[cls]
    raise KeyError(f"no cache kind is registered for {type(need).__name__}; known: "
                   f"{sorted(t.__name__ for t in _KINDS)}")


register_cache_kind(KVCacheNeed, PagedKeysValues())
register_cache_kind(LatentCacheNeed, PagedLatents())
register_cache_kind(StateNeed, SlotState())


def _register_joint() -> None:
    from ..parts.parallel import JointNeed

    register_cache_kind(JointNeed, JointMemory())


_register_joint()
