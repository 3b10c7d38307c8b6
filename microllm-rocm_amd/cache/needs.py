"""What a run entry can ask of the cache, and how each kind of need is allocated, measured and handed over.

A need is a small frozen description that a mixer returns from ``cache_need()``. The manager never looks inside
one: it asks the need itself whether it lives in pages (a block table per request, pages given back when the
request ends or a window has passed them) or in one slot of fixed size per request, lets it allocate its
storage, and hands the mixer whatever ``bind`` returns. Needs that compare equal share a group: one pool of
pages and one block table per request. A new kind of cache payload (one latent vector a token, keys alone, keys
and values of different widths) is a new subclass, defined wherever its mixer is; nothing here lists kinds.

The kinds this package's own parts use are here: ``PagedKVNeed`` (keys and values in the tile order the MFMA
attention kernels read, see ``cache.layout``), ``PagedKeyValueNeed`` (keys and values of widths of their own in plain
pages), ``StateNeed`` (a tensor per request, zero when it opens) and ``CompositeNeed`` (several of these for one
mixer: one that runs an attention beside a layer with state asks for both).
The reference has one ``[slots, kv_heads, capacity, head_dim]`` tensor per layer and nothing else
(src/inference/kv_cache.cpp:11-64).
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, List, Optional, Tuple

import torch

from .layout import check_sizes, key_page_shape, value_page_shape


def _element_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class CacheNeed:
    """Base of every need. Subclasses are frozen dataclasses (hashable: equal needs share a group).

    A paged need sets ``paged = True``, may carry ``window`` (positions older than that are never read again,
    so their pages go back), and implements ``check_page_size``, ``allocate_pages`` and ``bytes_per_position``.
    A slot need leaves ``paged`` False and implements ``allocate_slots``, ``zero_slot`` and ``bytes_per_request``.
    Both implement ``bind``: what the mixer's ``forward`` receives as ``cache``; it must have ``need``, ``owned``,
    ``tensors()`` and ``shared()`` (the ``Binding`` base gives these)."""
    paged = False
    window: Optional[int] = None

    # ---- paged needs ---------------------------------------------------------------------
    def check_page_size(self, page_size: int) -> None:
        """Raise ``ValueError`` if pages of ``page_size`` positions cannot hold this need's layout."""

    def allocate_pages(self, num_pages: int, page_size: int, dtype: torch.dtype, device: torch.device) -> Any:
        raise NotImplementedError(f"{type(self).__name__} does not live in pages")

    def bytes_per_position(self, dtype: torch.dtype) -> int:
        """Bytes one position of one run entry takes in its pages."""
        raise NotImplementedError(f"{type(self).__name__} does not live in pages")

    # ---- slot needs ----------------------------------------------------------------------
    def allocate_slots(self, max_requests: int, dtype: torch.dtype, device: torch.device) -> Any:
        raise NotImplementedError(f"{type(self).__name__} does not live in request slots")

    def zero_slot(self, storage: Any, slot: int) -> None:
        """A request opens in ``slot``: make the slot what a fresh request must find."""
        raise NotImplementedError(f"{type(self).__name__} does not live in request slots")

    def bytes_per_request(self, dtype: torch.dtype) -> int:
        raise NotImplementedError(f"{type(self).__name__} does not live in request slots")

    # ---- both ----------------------------------------------------------------------------
    def bind(self, group: Optional[int], storage: Any, owned: bool) -> "Binding":
        """What the mixer gets: ``group`` indexes ``ctx.paged`` (None for a slot need), ``storage`` is what the
        allocation returned (None where the manager only keeps books, without a device)."""
        raise NotImplementedError


@dataclass
class Binding:
    """What a mixer's forward receives as ``cache``. ``owned`` is False for a run entry that reads another's."""
    need: CacheNeed
    owned: bool = True

    def tensors(self) -> List[torch.Tensor]:
        """The device tensors behind this binding (for accounting, and for filling a cache with stand-in data)."""
        return []

    def shared(self) -> "Binding":
        """The same storage for a run entry that reads it without owning it."""
        return dataclasses.replace(self, owned=False)


# ---- keys and values in pages ------------------------------------------------------------------
@dataclass(frozen=True)
class PagedKVNeed(CacheNeed):
    """Keys and values in pages; ``window`` is None when every key stays needed."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None
    paged = True

    def check_page_size(self, page_size: int) -> None:
        check_sizes(page_size, self.head_dim)     # pages are tiled by 16 positions

    def allocate_pages(self, num_pages, page_size, dtype, device):
        # Zeroed once: a kernel may read a whole tile whose tail was never written.
        k = torch.zeros(key_page_shape(num_pages, self.kv_heads, page_size, self.head_dim), dtype=dtype, device=device)
        v = torch.zeros(value_page_shape(num_pages, self.kv_heads, page_size, self.head_dim), dtype=dtype, device=device)
        return k, v

    def bytes_per_position(self, dtype):
        return 2 * self.kv_heads * self.head_dim * _element_size(dtype)

    def bind(self, group, storage, owned):
        k, v = storage if storage is not None else (None, None)
        return PagedBinding(self, owned, group, k, v)


@dataclass
class PagedBinding(Binding):
    """What a mixer gets for paged keys and values: its entry's page arrays and its group."""
    group: int = 0
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None

    def tensors(self):
        return [tensor for tensor in (self.k, self.v) if tensor is not None]


# ---- keys and values of different widths, in plain pages ---------------------------------------------------
@dataclass(frozen=True)
class PagedKeyValueNeed(CacheNeed):
    """Keys ``[page, position, kv_head, key_dim]`` and values ``[page, position, kv_head, value_dim]``: the two widths
    are free, and a position's row is contiguous (what the attention with a bias by distance reads)."""
    kv_heads: int
    key_dim: int
    value_dim: int
    window: Optional[int] = None
    paged = True

    def check_page_size(self, page_size: int) -> None:
        if page_size <= 0:
            raise ValueError("page_size must be positive")

    def allocate_pages(self, num_pages, page_size, dtype, device):
        k = torch.zeros((num_pages, page_size, self.kv_heads, self.key_dim), dtype=dtype, device=device)
        v = torch.zeros((num_pages, page_size, self.kv_heads, self.value_dim), dtype=dtype, device=device)
        return k, v

    def bytes_per_position(self, dtype):
        return self.kv_heads * (self.key_dim + self.value_dim) * _element_size(dtype)

    def bind(self, group, storage, owned):
        k, v = storage if storage is not None else (None, None)
        return PagedBinding(self, owned, group, k, v)


# ---- one latent row a position, in plain pages -------------------------------------------------------------------------
@dataclass(frozen=True)
class PagedLatentNeed(CacheNeed):
    """One row of ``width`` elements a position, ``[page, position, width]``: what an attention keeps whose keys and
    values are projections of one cached vector (a latent and whatever rides with it, e.g. a rotated key part)."""
    width: int
    window: Optional[int] = None
    paged = True

    def check_page_size(self, page_size: int) -> None:
        if page_size <= 0:
            raise ValueError("page_size must be positive")

    def allocate_pages(self, num_pages, page_size, dtype, device):
        return torch.zeros((num_pages, page_size, self.width), dtype=dtype, device=device)

    def bytes_per_position(self, dtype):
        return self.width * _element_size(dtype)

    def bind(self, group, storage, owned):
        return LatentBinding(self, owned, group, storage)


@dataclass
class LatentBinding(Binding):
    """What a mixer gets for latent rows in pages: its entry's page array and its group."""
    group: int = 0
    rows: Optional[torch.Tensor] = None

    def tensors(self):
        return [self.rows] if self.rows is not None else []


# ---- per-request state of fixed size -------------------------------------------------------------
@dataclass(frozen=True)
class StateNeed(CacheNeed):
    """Per-request state of fixed size: one slot of ``shape`` and ``dtype`` per live request."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def allocate_slots(self, max_requests, dtype, device):
        return torch.zeros((max_requests, *self.shape), dtype=self.dtype, device=device)

    def zero_slot(self, storage, slot):
        storage[slot].zero_()

    def bytes_per_request(self, dtype):
        count = 1
        for size in self.shape:
            count *= int(size)
        return count * _element_size(self.dtype)

    def bind(self, group, storage, owned):
        return StateBinding(self, owned, storage)


@dataclass
class StateBinding(Binding):
    """What a mixer gets for per-request state: ``state[slot]`` is the request's, zero when it opens."""
    state: Optional[torch.Tensor] = None

    def tensors(self):
        return [self.state] if self.state is not None else []


# ---- several needs of one mixer ----------------------------------------------------------------------------
@dataclass(frozen=True)
class CompositeNeed(CacheNeed):
    """What a mixer made of several mixers keeps: each part's need, in the parts' order (None for a part that keeps
    nothing). The manager gives every part what it would give a run entry with that need alone (paged parts join
    the groups of equal needs, state parts get slots) and hands the mixer a ``CompositeBinding``."""
    parts: Tuple[Optional[CacheNeed], ...]

    def flat(self) -> List[CacheNeed]:
        """Every need that is no composite itself, in order."""
        found: List[CacheNeed] = []
        for part in self.parts:
            if isinstance(part, CompositeNeed):
                found += part.flat()
            elif part is not None:
                found.append(part)
        return found


@dataclass
class CompositeBinding(Binding):
    """``parts[i]`` is the binding of the i-th part's need (None where that part keeps nothing)."""
    parts: Tuple[Optional[Binding], ...] = ()

    def tensors(self):
        return [tensor for part in self.parts if part is not None for tensor in part.tensors()]

    def shared(self):
        return dataclasses.replace(self, owned=False, parts=tuple(part.shared() if part is not None else None for part in self.parts))


def flat_needs(need: Optional[CacheNeed]) -> List[CacheNeed]:
    """The needs behind ``need`` that are no composites: what memory estimates and byte counts add up."""
    if need is None:
        return []
    return need.flat() if isinstance(need, CompositeNeed) else [need]


def flat_bindings(binding: Optional[Binding]) -> List[Binding]:
    """The bindings behind ``binding`` that are no composites."""
    if binding is None:
        return []
    if isinstance(binding, CompositeBinding):
        return [inner for part in binding.parts for inner in flat_bindings(part)]
    return [binding]
