"""One step's batch: (request, its next tokens) for any mix of prompt portions and single decoded tokens,
flattened to `tokens` rows, plus everything kernels need to find each token's request, position and pages.

The reference builds three different inputs for its three forward functions and uploads block tables once
per layer (ampere_kv/runner.py:205-215, :227-229; ampere_kv/scheduler.py:133-139).  Here one batch layout
serves every step and all of its integer metadata reaches the device in one copy.  Block tables are not part of it:
they live on the device, a row per request slot, and a step brings only the entries that changed - the pages its
requests were handed or gave back - as (offset, value) pairs that a small kernel applies before anything reads them.
A decode step of 64 requests with 32,768 tokens each thus uploads some hundreds of integers instead of 130,000.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Sequence as Seq

import numpy as np
import torch

from ..cache.manager import CacheManager, Sequence


LAST_TOKEN = (-1,)      # as a `StepEntry`'s tokens: the one token that was chosen last for the request (the sampler
                        # left it in the request's slot on the device; the host need not send it back)


@dataclass
class StepEntry:
    """A request's share of a step: its next `tokens` and `want`, the places among them whose logits are
    asked for."""
    seq: Sequence
    tokens: Seq[int]
    want: Seq[int] = ()
    # further integers per token for parts that need more than a position (the axes of a multi-axis position encoding,
    # a segment id): name -> [len(tokens)][width].  Every entry of a step carries the same names and widths; the parts
    # find them on the device as `ctx.extra[name]`, int32 [tokens, width].
    extra: dict | None = None


@dataclass
class PagedMeta:
    """Per cache group: where each new token's key/value goes and where each request's pages are."""
    block_table: torch.Tensor     # int32 [slots, width]: the group's persistent table; RELEASED (-1) or stale entries
                                  # are never read
    slot_map: torch.Tensor        # int32 [tokens]: page * page_size + offset of the token's own slot
    width: int                    # entries of a table row
    window: int | None
    rows: torch.Tensor | None = None   # int32 [seqs]: the table row of each request of the step (its slot); None: row r


class Arena:
    """Bump allocator for a step's activations.  Chunks are kept between steps, so after the first step
    of a given size no device memory is allocated and addresses repeat from step to step."""

    ALIGN = 256
    ELEMENT_BYTES = {torch.float32: 4, torch.bfloat16: 2, torch.int32: 4, torch.int64: 8, torch.uint8: 1,
                     torch.float16: 2}

    def __init__(self, device, chunk_bytes: int = 64 << 20):
        self.device = device
        self.chunk_bytes = chunk_bytes
        self.chunks: list[torch.Tensor] = []
        self.chunk_index = 0
        self.offset = 0
        # Steps ask for the same pieces in the same order again and again: the tensor made for (chunk, offset, shape,
        # dtype) is kept and handed out again instead of slicing and viewing anew (chunks are never replaced).
        self._views: dict[tuple, torch.Tensor] = {}

    def reset(self) -> None:
        self.chunk_index = 0
        self.offset = 0

    def take(self, shape, dtype: torch.dtype) -> torch.Tensor:
        count = 1
        for s in shape:
            count *= int(s)
        size = self.ELEMENT_BYTES.get(dtype) or torch.empty((), dtype=dtype).element_size()
        nbytes = max(count * size, 1)
        nbytes = (nbytes + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        while True:
            if self.chunk_index >= len(self.chunks):
                self.chunks.append(torch.empty(max(nbytes, self.chunk_bytes), dtype=torch.uint8, device=self.device))
            chunk = self.chunks[self.chunk_index]
            if self.offset + nbytes <= chunk.numel():
                key = (self.chunk_index, self.offset, tuple(shape), dtype)
                view = self._views.get(key)
                if view is None:
                    if len(self._views) >= 8192:     # shapes keep changing: do not keep them all
                        self._views.clear()
                    view = self._views[key] = chunk[self.offset:self.offset + count * size].view(dtype).view(*shape)
                self.offset += nbytes
                return view
            self.chunk_index += 1
            self.offset = 0


@dataclass
class StepContext:
    """What every part sees of the step."""
    num_tokens: int
    num_seqs: int
    num_decode_seqs: int           # the first `num_decode_seqs` requests bring exactly one token each
    token_ids: torch.Tensor        # int32 [tokens]
    positions: torch.Tensor        # int32 [tokens], absolute
    seq_of_token: torch.Tensor     # int32 [tokens], row of the step's request list
    q_start: torch.Tensor          # int32 [seqs + 1], first token row of each request
    seq_lens: torch.Tensor         # int32 [seqs], tokens the request holds after this step
    seq_slots: torch.Tensor        # int32 [seqs], per-request state slot
    logit_rows: torch.Tensor       # int32 [wanted], token rows whose logits are asked for
    paged: list[PagedMeta]
    arena: Arena
    # host copies for parts that loop on the host (and for sizing launches without a device read)
    host_q_start: list[int] = field(default_factory=list)
    host_seq_lens: list[int] = field(default_factory=list)
    host_seq_slots: list[int] = field(default_factory=list)
    max_seq_len: int = 0           # longest request of the step, after the step
    max_new_tokens: int = 0        # longest portion of the step
    most_wanted: int = 0           # the most places any one request wants logits at
    arenas: tuple = ()             # two arenas used by alternate layers (a layer's output outlives its own arena's reset)
    stream_buffer: torch.Tensor | None = None   # float32 [max tokens, hidden]: the residual sum
    spare_buffer: torch.Tensor | None = None    # float32 [a few rows, hidden]: where a small step may move it
    stream: torch.Tensor | None = None          # the step's residual sum, wherever it is now
    spare_stream: torch.Tensor | None = None    # the other buffer's rows, or None where the step has too many
    # set by the model's pass and by blocks around every branch: the branch may add its output to the residual sum in
    # its last product and return `StreamSums` (see `parts.base.Part`)
    fold_into_stream: bool = False
    # ... and the weight of the norm that will read what the branch leaves, where that norm has one (`Norm.fold_gain`)
    fold_gain: object = None
    # the device's persistent integer state (slot words, block tables) and what this step changes in it
    table_pages: int = 0                        # bound on the pages of the step's longest request (sizes launches)
    patches: torch.Tensor | None = None         # int32 [2 * patch_room]: (offset into slot_state, value) pairs
    patch_count: torch.Tensor | None = None     # int32 [1]: how many of them this step brings
    patch_room: int = 0
    slot_state: torch.Tensor | None = None      # int32: the whole state
    slot_words: torch.Tensor | None = None      # int32 [slots, SLOT_WORDS]: its first part
    extra: dict = field(default_factory=dict)   # name -> int32 [tokens, width]: what the entries brought per token


class BatchBuilder:
    """Turns entries into a `StepContext`: registers the new tokens with the cache manager (which hands out
    pages), lays the tokens out with single-token requests first, and uploads the metadata in one copy."""

    EXTRA_WORDS_PER_TOKEN = 8       # room for the entries' further integers per token, all names together

    def __init__(self, cache: CacheManager, device, max_batched_tokens: int, max_seqs: int, max_pages_per_seq: int):
        self.cache = cache
        self.device = torch.device(device)
        self.max_tokens, self.max_seqs, self.max_width = max_batched_tokens, max_seqs, max_pages_per_seq
        groups = len(cache.groups)
        if cache.arrays is not None:        # a request cannot outgrow its row of the device's block table
            self.max_width = min(self.max_width, cache.arrays.table_width)
        most_patches = groups * 2 * (self.max_tokens // cache.page_size + 2 * self.max_seqs)
        capacity = (3 * self.max_tokens + 3 * self.max_seqs + 1 + self.max_tokens
                    + groups * self.max_tokens + 1 + 2 * most_patches + self.EXTRA_WORDS_PER_TOKEN * self.max_tokens)
        pin = self.device.type == "cuda"
        # Two pinned staging buffers in turn: the copy of one step may still be in flight while the host
        # lays out the next, so a buffer is written again only after the copy that read it has finished.
        self._hosts = [torch.empty(capacity, dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self._copied = [torch.cuda.Event() if pin else None for _ in range(2)]
        self._turn = 0
        self._device = torch.empty(capacity, dtype=torch.int32, device=self.device)
        self.arenas = (Arena(self.device), Arena(self.device))

    def patch_capacity(self, counts) -> int:
        """The most block-table entries a step can change whose requests bring `counts` tokens: per request and group
        the pages its tokens may open, and as many that a window may close."""
        page = self.cache.page_size
        return len(self.cache.groups) * sum(2 * ((count + page - 1) // page + 1) for count in counts)

    def build(self, entries: list[StepEntry], width_multiple: int = 1) -> tuple[StepContext, list[int]]:
        """Returns the context and, for every entry in the caller's order, the offset of its first wanted
        row in the logits the step returns.  `ctx.table_pages` is the longest request's page count rounded up to
        `width_multiple` pages: a bound that sizes launches and is the same for all steps under it (what a recorded
        graph needs)."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        if len(entries) > self.max_seqs:
            raise ValueError(f"{len(entries)} requests in one step; the engine was built for {self.max_seqs}")
        if len({id(e.seq) for e in entries}) != len(entries):
            raise ValueError("a request appears twice in one step")
        total = sum(len(e.tokens) for e in entries)
        if total > self.max_tokens:
            raise ValueError(f"{total} tokens in one step; the engine was built for {self.max_tokens}")
        for e in entries:
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.seq.request_id!r} brings no tokens")
            for place in e.want:
                if not 0 <= place < len(e.tokens):
                    raise ValueError(f"request {e.seq.request_id!r} wants place {place} of {len(e.tokens)} tokens")
            if e.seq.length + len(e.tokens) > self.max_width * self.cache.page_size:
                raise ValueError(f"request {e.seq.request_id!r} would reach {e.seq.length + len(e.tokens)} tokens; "
                                 f"the engine was built for {self.max_width * self.cache.page_size}")
        order = sorted(range(len(entries)), key=lambda i: (len(entries[i].tokens) != 1, i))
        ordered = [entries[i] for i in order]
        # all-or-nothing over the whole step: check every request before registering any
        self._check_pages(ordered)
        num_decode = sum(1 for e in ordered if len(e.tokens) == 1)
        starts = [self.cache.reserve(e.seq, len(e.tokens)) for e in ordered]

        n, r = total, len(ordered)
        width = max(max((t.num_pages for t in e.seq.tables), default=1) for e in ordered)
        width = max(width, 1)
        width = min((width + width_multiple - 1) // width_multiple * width_multiple, max(self.max_width, width))
        arrays = self.cache.arrays
        patch_room = self.patch_capacity(len(e.tokens) for e in ordered)
        self._turn ^= 1
        if self._copied[self._turn] is not None:
            self._copied[self._turn].synchronize()
        host_tensor = self._hosts[self._turn]
        host = host_tensor.numpy()
        cursor = 0

        def region(count):
            nonlocal cursor
            view = host[cursor:cursor + count]
            span = (cursor, cursor + count)
            cursor += count
            return view, span

        token_ids, s_ids = region(n)
        positions, s_pos = region(n)
        seq_of_token, s_sot = region(n)
        q_start, s_qs = region(r + 1)
        seq_lens, s_sl = region(r)
        seq_slots, s_ss = region(r)
        wanted = sum(len(e.want) for e in entries)
        logit_rows, s_lr = region(wanted)
        group_spans = []
        for g in self.cache.groups:
            slot_map, s_sm = region(n)
            group_spans.append((slot_map, s_sm))
        patch_count, s_pc = region(1)
        patches, s_pa = region(2 * patch_room)
        changed = 0
        extra_spans = self._extra_regions(ordered, n, region)

        row = 0
        first_row_of = [0] * len(entries)
        page_size = self.cache.page_size
        for index, (e, start) in enumerate(zip(ordered, starts)):
            count = len(e.tokens)
            if count == 1:      # a decode token: scalars, no temporary arrays
                token_ids[row] = e.tokens[0]
                positions[row] = start
                seq_of_token[row] = index
            else:
                token_ids[row:row + count] = np.asarray(e.tokens, dtype=np.int64)
                positions[row:row + count] = np.arange(start, start + count)
                seq_of_token[row:row + count] = index
            for name, (view, _, width_of) in extra_spans.items():
                view.reshape(n, width_of)[row:row + count] = np.asarray(e.extra[name], dtype=np.int64).reshape(count, width_of)
            q_start[index] = row
            seq_lens[index] = start + count
            seq_slots[index] = e.seq.slot
            first_row_of[order[index]] = row
            for g, (slot_map, _) in zip(self.cache.groups, group_spans):
                table = e.seq.tables[g.index]
                pages = table.page_array
                if arrays is not None:      # what this step changed in the request's row of the device's table
                    changes = table.take_changes()
                    if len(changes) > 2 * ((count + page_size - 1) // page_size + 1):
                        # (tokens were registered outside a step: the row goes to the device as a whole)
                        arrays.write_row(g.index, e.seq.slot, pages)
                        changes = ()
                    for entry, page in changes:
                        patches[2 * changed] = arrays.table_offset(g.index, e.seq.slot, entry)
                        patches[2 * changed + 1] = page
                        changed += 1
                if count == 1:
                    slot_map[row] = int(pages[start // page_size]) * page_size + start % page_size
                else:
                    pos = np.arange(start, start + count)
                    slot_map[row:row + count] = pages[pos // page_size].astype(np.int64) * page_size + pos % page_size
            row += count
        # wanted rows in the caller's order of entries and places, whatever the layout above
        want_cursor = 0
        first_wanted_of = []
        for e, first_row in zip(entries, first_row_of):
            first_wanted_of.append(want_cursor)
            for place in e.want:
                logit_rows[want_cursor] = first_row + place
                want_cursor += 1
        q_start[r] = row
        assert changed <= patch_room, "a step changed more block-table entries than its requests' tokens allow"
        patch_count[0] = changed

        self._device[:cursor].copy_(host_tensor[:cursor], non_blocking=True)
        if self._copied[self._turn] is not None:
            self._copied[self._turn].record()
        dev = lambda span: self._device[span[0]:span[1]]
        paged = [PagedMeta(block_table=arrays.tables[g.index] if arrays is not None else None, slot_map=dev(s_sm),
                           width=arrays.table_width if arrays is not None else width, window=g.need.window,
                           rows=dev(s_ss))
                 for g, (_, s_sm) in zip(self.cache.groups, group_spans)]
        for arena in self.arenas:
            arena.reset()
        ctx = StepContext(
            num_tokens=n, num_seqs=r, num_decode_seqs=num_decode, token_ids=dev(s_ids), positions=dev(s_pos),
            seq_of_token=dev(s_sot), q_start=dev(s_qs), seq_lens=dev(s_sl), seq_slots=dev(s_ss),
            logit_rows=dev(s_lr), paged=paged, arena=self.arenas[0],
            host_q_start=[int(x) for x in q_start[:r + 1]], host_seq_lens=[int(x) for x in seq_lens[:r]],
            host_seq_slots=[int(x) for x in seq_slots[:r]],
            max_seq_len=int(seq_lens[:r].max()), max_new_tokens=max(len(e.tokens) for e in ordered),
            most_wanted=max(len(e.want) for e in ordered),
            arenas=self.arenas, table_pages=width, patches=dev(s_pa), patch_count=dev(s_pc), patch_room=patch_room,
            slot_state=arrays.state if arrays is not None else None,
            slot_words=arrays.words if arrays is not None else None,
            extra={name: dev(span).view(n, width_of) for name, (_, span, width_of) in extra_spans.items()},
        )
        return ctx, first_wanted_of

    def _extra_regions(self, ordered: list[StepEntry], n: int, region) -> dict:
        """Room in the step's upload for the further per-token integers the entries bring: name -> (host view, span,
        width).  All entries must agree on names and widths."""
        first = ordered[0].extra or {}
        widths = {}
        for name, rows in first.items():
            array = np.asarray(rows)
            if array.ndim != 2 or array.shape[0] != len(ordered[0].tokens) or array.dtype.kind not in "iu":
                raise ValueError(f"extra {name!r} must hold one row of integers per token")
            widths[name] = int(array.shape[1])
        for e in ordered[1:]:
            other = e.extra or {}
            if set(other) != set(widths) or any(np.asarray(other[name]).shape != (len(e.tokens), w) for name, w in widths.items()):
                raise ValueError("every entry of a step must bring the same further integers per token (names and widths)")
        if sum(widths.values()) > self.EXTRA_WORDS_PER_TOKEN:
            raise ValueError(f"{sum(widths.values())} further integers per token; the step's upload has room for "
                             f"{self.EXTRA_WORDS_PER_TOKEN}")
        spans = {}
        for name in sorted(widths):
            view, span = region(n * widths[name])
            spans[name] = (view, span, widths[name])
        return spans

    def _check_pages(self, ordered: list[StepEntry]) -> None:
        """Plays the step's registrations through in the order they will be made (a request first gives back the
        pages its window has passed, then takes what it needs) and refuses the step if the pool would run dry at
        any point of it - a sum over the whole step would let an early request count on pages a later one frees."""
        from ..cache.pages import PagePoolExhausted
        for g in self.cache.groups:
            available = g.allocator.num_free
            for e in ordered:
                table = e.seq.tables[g.index]
                required = (table.length + len(e.tokens) + self.cache.page_size - 1) // self.cache.page_size
                available += table._passed_pages(table.length) - max(0, required - table.num_pages)
                if available < 0:
                    raise PagePoolExhausted(f"the step needs {-available} more page(s) than the pool of cache group "
                                            f"{g.index} has free when request {e.seq.request_id!r} registers its "
                                            "tokens; no token of the step was registered")
