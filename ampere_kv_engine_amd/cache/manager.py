"""The cache manager: page pools for groups of layers with the same needs, one block table per request and
group, and slots for per-request state of fixed size.

The reference keeps one pool and one tensor pair per layer and lets every request hold one table per layer
that all grow in lock-step (ampere_kv/scheduler.py:63-69, ampere_kv/paged_cache.py:10-62).  Here layers whose
mixers ask for the same thing (`PagedKV(kv_heads, head_dim, window, value_dim)`) form a group with ONE pool, ONE
table per request and one tensor `[layers, elements of a layer]` - a layer's keys `[pages, kv_heads, page_size,
head_dim]`, then its values `[pages, kv_heads, value_dim, page_size]` -, so a page id is valid for every layer of
its group.  Within a page, keys lie `[page_size, head_dim]` and values `[value_dim, page_size]`: scores contract
over head_dim and the weighted sum over keys, and each reaches the matrix cores with its contracted axis
contiguous.  Keys and values need not be equally wide, and a mixer may ask for no values at all.  Groups with a window give pages back while the request lives.  Mixers that ask
for `SlotState` get a tensor `[slots, *shape]` per layer, zeroed (or set by the mixer's own `init`) when a request
takes the slot.

Everything here except the tensors is host bookkeeping and runs without a GPU (`allocate_tensors=False`).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..parts.base import PagedKV, SlotState
from .pages import BlockTable, PageAllocator, PagePoolExhausted
from .slots import SlotArrays, SlotTable


@dataclass
class PagedGroup:
    index: int
    need: PagedKV
    layers: list[int]                 # cache-layer ids, in the order of the tensor's first axis
    allocator: PageAllocator
    page_size: int
    pages: torch.Tensor | None = None  # [len(layers), num_pages * kv_heads * page_size * (head_dim + value_dim)]

    def bytes_per_token(self, element_size: int) -> int:
        return len(self.layers) * self.need.kv_heads * (self.need.head_dim + self.need.v_dim) * element_size


@dataclass
class LayerCache:
    """What one cache layer's mixer sees: its group id and its own key and value pages, or its state."""
    group: int | None = None
    k: torch.Tensor | None = None      # [num_pages, kv_heads, page_size, head_dim]
    v: torch.Tensor | None = None      # [num_pages, kv_heads, value_dim, page_size]; None where the mixer keeps none
    state: torch.Tensor | None = None  # [slots, *shape]


@dataclass
class Sequence:
    """A live request's hold on the cache: its slot and one table per paged group."""
    request_id: str
    slot: int
    tables: list[BlockTable]
    length: int = 0
    closed: bool = False


class CacheManager:
    def __init__(self, needs: dict[int, PagedKV | SlotState | None], *, page_size: int, num_pages: int,
                 max_seqs: int, dtype: torch.dtype = torch.bfloat16, device: str | torch.device = "cpu",
                 allocate_tensors: bool = True, max_pages_per_seq: int | None = None):
        """`needs[cache_layer]` is what that layer's mixer asked for.  `max_pages_per_seq` is the width of the block
        tables kept on the device (default: the whole pool)."""
        self.page_size, self.num_pages, self.max_seqs = page_size, num_pages, max_seqs
        self.max_pages_per_seq = max_pages_per_seq if max_pages_per_seq is not None else num_pages
        self.dtype, self.device = dtype, device
        self.slots = SlotTable(max_seqs)
        self.groups: list[PagedGroup] = []
        self.layer_cache: dict[int, LayerCache] = {}
        self._state_tensors: list[tuple[torch.Tensor, SlotState]] = []
        self._live: dict[str, Sequence] = {}
        by_need: dict[PagedKV, PagedGroup] = {}
        for layer in sorted(needs):
            need = needs[layer]
            if isinstance(need, PagedKV):
                if need not in by_need:
                    by_need[need] = PagedGroup(len(self.groups), need, [], PageAllocator(num_pages), page_size)
                    self.groups.append(by_need[need])
                by_need[need].layers.append(layer)
        for group in self.groups:
            heads, k_dim, v_dim = group.need.kv_heads, group.need.head_dim, group.need.v_dim
            k_elements, v_elements = num_pages * heads * page_size * k_dim, num_pages * heads * page_size * v_dim
            if allocate_tensors:
                group.pages = torch.empty((len(group.layers), k_elements + v_elements), dtype=dtype, device=device)
            for row, layer in enumerate(group.layers):
                view = LayerCache(group=group.index)
                if group.pages is not None:
                    view.k = group.pages[row, :k_elements].view(num_pages, heads, page_size, k_dim)
                    if v_dim:
                        view.v = group.pages[row, k_elements:].view(num_pages, heads, v_dim, page_size)
                self.layer_cache[layer] = view
        for layer in sorted(needs):
            need = needs[layer]
            if isinstance(need, SlotState):
                state = (torch.zeros((max_seqs, *need.shape), dtype=need.dtype, device=device)
                         if allocate_tensors else None)
                self.layer_cache[layer] = LayerCache(state=state)
                if state is not None:
                    self._state_tensors.append((state, need))
            elif need is None:
                self.layer_cache[layer] = LayerCache()
        # what every request keeps on the device between steps: its slot's words and its rows of the block tables
        self.arrays = (SlotArrays(max_seqs, len(self.groups), self.max_pages_per_seq, device)
                       if allocate_tensors else None)

    # ---- sizes --------------------------------------------------------------------------------------
    def pages_for(self, num_tokens: int, group: PagedGroup | None = None, chunk: int | None = None) -> int:
        """Most pages a request of `num_tokens` tokens holds at one time in `group` (in any group if None).
        A windowed group never holds more than the window plus the tokens of one step (`chunk`)."""
        def one(g: PagedGroup) -> int:
            full = (num_tokens + self.page_size - 1) // self.page_size
            if g.need.window is None:
                return full
            span = g.need.window + (chunk if chunk is not None else num_tokens)
            return min(full, (span + self.page_size - 1) // self.page_size + 1)
        if group is not None:
            return one(group)
        return max((one(g) for g in self.groups), default=0)

    def bytes_per_token(self) -> int:
        size = torch.empty((), dtype=self.dtype).element_size()
        return sum(g.bytes_per_token(size) for g in self.groups)

    @property
    def num_free_pages(self) -> list[int]:
        return [g.allocator.num_free for g in self.groups]

    # ---- a request's life ---------------------------------------------------------------------------
    def open(self, request_id: str, temperature: float = 0.0, seed: int = 0) -> Sequence:
        """A new request takes a slot.  `temperature` and `seed` are what the sampler will find in the slot."""
        if request_id in self._live:
            raise ValueError(f"request {request_id!r} already holds a sequence")
        if temperature < 0 or not 0 <= seed < 2 ** 63:
            raise ValueError("temperature must not be negative and the seed must fit in 63 bits")
        slot = self.slots.take()
        if self.arrays is not None:
            self.arrays.take(slot, temperature, seed)
        for state, need in self._state_tensors:     # a reused slot starts as a fresh one
            if need.init is not None:
                need.init(state[slot])
            else:
                state[slot].zero_()
        seq = Sequence(request_id, slot,
                       [BlockTable(g.allocator, self.page_size, g.need.window) for g in self.groups])
        self._live[request_id] = seq
        return seq

    def can_reserve(self, seq: Sequence, num_tokens: int) -> bool:
        for table, group in zip(seq.tables, self.groups):
            required = (table.length + num_tokens + self.page_size - 1) // self.page_size
            additional = max(0, required - table.num_pages)
            if additional > group.allocator.num_free + table._passed_pages(table.length):
                return False
        return True

    def reserve(self, seq: Sequence, num_tokens: int) -> int:
        """Register `num_tokens` new tokens in every group (all or nothing); returns their first position."""
        if seq.closed:
            raise ValueError(f"request {seq.request_id!r} was closed")
        if not self.can_reserve(seq, num_tokens):
            raise PagePoolExhausted(f"no pages for {num_tokens} more token(s) of request {seq.request_id!r}; "
                                    "nothing was registered")
        start = seq.length
        for table in seq.tables:
            got = table.append_tokens(num_tokens)
            assert got == start
        seq.length = start + num_tokens
        return start

    def close(self, seq: Sequence) -> None:
        """Give back the request's pages and slot.  Calling it twice is harmless."""
        if seq.closed:
            return
        for table in seq.tables:
            table.release()
        self.slots.give_back(seq.slot)
        if self.arrays is not None:
            self.arrays.give_back(seq.slot)
        seq.closed = True
        self._live.pop(seq.request_id, None)

    def live(self) -> list[Sequence]:
        return list(self._live.values())

    # ---- debugging / tests --------------------------------------------------------------------------
    def gather(self, seq: Sequence, layer: int) -> tuple[torch.Tensor, torch.Tensor]:
        """The request's keys and values of one cache layer in logical order, `[length, kv_heads, head_dim]`
        (positions whose pages were given back are left out).  A copy for checks; kernels read the pages."""
        view = self.layer_cache[layer]
        table = seq.tables[view.group]
        keys, values = [], []
        pages = table.pages
        for position in range(table.length):
            index, offset = divmod(position, self.page_size)
            page = pages[index]
            if page < 0:
                continue
            keys.append(view.k[page, :, offset])
            values.append(view.v[page, :, :, offset])
        return torch.stack(keys), torch.stack(values)
