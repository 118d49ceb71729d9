"""One step's batch: portions of requests as flat device arrays.

The reference passes ``input_ids[1, T]`` for one whole prompt or ``[B, 1]`` for
decoded tokens and derives positions from ``arange(T)`` or the token counts
(somi_inference/models/qwen2_adapter.py:91, 134-137), and rebuilds block tables
in every layer (somi_inference/core/paged_attention.py:173-193 via
qwen2_adapter.py:117).  Here every token carries its request's entry index and
its position explicitly, the tables are built once per step on the host as
int32 and reach the device in one copy.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable

import numpy as np
import torch

from ..cache.manager import CacheManager


@dataclass
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""

    request_id: Hashable
    tokens: list[int]
    want: list[int] = field(default_factory=list)


@dataclass
class EntryInfo:
    request_id: Hashable
    start: int          # index of the entry's first token in the flat batch
    length: int
    first_position: int  # position of that token in its request (= tokens cached before the step)
    state_slot: int


@dataclass
class PagedView:
    """A cache group's view of the step."""

    slot_mapping: torch.Tensor      # [N] int32: page * page_size + offset where what token t keeps goes
    block_table: torch.Tensor       # [E, max_blocks] int32 physical pages of each entry's request
    page_size: int = 0              # tokens per page of this group


@dataclass
class EntrySplit:
    """The step's entries cut in two by their length, for a mixer that serves long portions and single tokens
    (or portions of a few) with different kernels.  Every token of the step lies in exactly one of the two."""

    threshold: int
    long_entry_len: torch.Tensor    # [E] int32: an entry's length if it is longer than the threshold, else 0
    short_tokens: torch.Tensor      # [Ns] int32: flat indices of the tokens of the entries of at most threshold tokens
    num_long_tokens: int
    num_short_tokens: int


@dataclass
class StepBatch:
    num_tokens: int
    num_entries: int
    num_logit_rows: int
    token_ids: torch.Tensor         # [N] int32
    positions: torch.Tensor         # [N] int32
    token_entry: torch.Tensor       # [N] int32: entry index of each token
    entry_start: torch.Tensor       # [E + 1] int32: offsets of the entries in the flat batch
    entry_first_position: torch.Tensor   # [E] int32
    context_lens: torch.Tensor      # [E] int32: tokens of each request after this step
    state_slots: torch.Tensor       # [E] int32
    logit_rows: torch.Tensor        # [R] int32 flat token indices whose logits are wanted
    paged: list[PagedView]
    entries: list[EntryInfo]        # host mirror
    max_entry_len: int
    max_context: int
    block_size: int
    splits: dict[int, EntrySplit] = field(default_factory=dict)

    def split(self, threshold: int) -> EntrySplit:
        """The entries cut at ``threshold`` tokens.  Only the thresholds that the model's mixers declared
        (``Mixer.entry_split``) are laid out: the lists travel with the step's one copy to the device."""
        try:
            return self.splits[int(threshold)]
        except KeyError:
            raise KeyError(f"this step holds no split of its entries at {threshold} tokens (it has "
                           f"{sorted(self.splits)}): a mixer declares the threshold it needs as entry_split") from None


class _Padding:
    def __repr__(self) -> str:
        return "<padding>"


PADDING = _Padding()      # request id of a padding entry


FIXED_SECTIONS = 8      # token ids, positions, token -> entry, entry offsets, first positions, contexts, slots, logit rows


def _layout(entries: list[StepEntry], cache: CacheManager, table_widths: list[int] | None, pad_to: int = 0,
            entry_splits: tuple[int, ...] = ()):
    """The step as host arrays: (sections, infos, widths).  ``table_widths`` fixes the block tables'
    widths (a captured graph needs the same layout at every replay); None = as narrow as possible.
    ``entry_splits``: the lengths at which mixers want the entries cut into long and short ones.

    ``pad_to``: entries are added until there are this many.  A padding entry is one token (id 0, position 0)
    of no request: it stores nothing (slot -1), reads page 0 through a table row of zeros, uses the state
    slot that no request gets, and its logits are computed and dropped by the caller."""
    infos: list[EntryInfo] = []
    token_ids: list[int] = []
    positions: list[int] = []
    token_entry: list[int] = []
    logit_rows: list[int] = []
    for index, entry in enumerate(entries):
        first = cache.num_tokens(entry.request_id)
        infos.append(EntryInfo(entry.request_id, len(token_ids), len(entry.tokens), first,
                               cache.state_slot(entry.request_id)))
        logit_rows.extend(len(token_ids) + w for w in entry.want)
        token_ids.extend(entry.tokens)
        positions.extend(range(first, first + len(entry.tokens)))
        token_entry.extend([index] * len(entry.tokens))
    for index in range(len(entries), pad_to):
        infos.append(EntryInfo(PADDING, len(token_ids), 1, 0, cache.padding_state_slot))
        logit_rows.append(len(token_ids))
        token_ids.append(0)
        positions.append(0)
        token_entry.append(index)
    n, e = len(token_ids), len(infos)
    nothing = np.zeros(0, dtype=np.int32)
    tables, slot_maps, widths = [], [], []
    for g in range(len(cache.groups)):
        rows = [cache.table_row(g, info.request_id) if info.request_id is not PADDING else nothing for info in infos]
        width = max(1, max((r.size for r in rows), default=1))
        if table_widths is not None:
            if width > table_widths[g]:
                raise ValueError(f"block table of width {width} does not fit the fixed width {table_widths[g]}")
            width = table_widths[g]
        table = np.zeros((e, width), dtype=np.int32)
        for r, pages in enumerate(rows):
            table[r, :pages.size] = pages                # released pages read as page 0 there
        slots: list[int] = []
        for info in infos:
            if info.request_id is PADDING:
                slots.append(-1)
            else:
                slots.extend(cache.slots(g, info.request_id, info.first_position, info.length))
        tables.append(table)
        slot_maps.append(np.asarray(slots, dtype=np.int32))
        widths.append(width)
    sections = [
        np.asarray(token_ids, dtype=np.int32), np.asarray(positions, dtype=np.int32),
        np.asarray(token_entry, dtype=np.int32),
        np.asarray([i.start for i in infos] + [n], dtype=np.int32),
        np.asarray([i.first_position for i in infos], dtype=np.int32),
        np.asarray([i.first_position + i.length for i in infos], dtype=np.int32),
        np.asarray([i.state_slot for i in infos], dtype=np.int32),
        np.asarray(logit_rows, dtype=np.int32),
    ]
    assert len(sections) == FIXED_SECTIONS
    for table, slots in zip(tables, slot_maps):
        sections += [slots, table.reshape(-1)]
    for threshold in entry_splits:
        sections += [
            np.asarray([i.length if i.length > threshold else 0 for i in infos], dtype=np.int32),
            np.asarray([t for i in infos if i.length <= threshold for t in range(i.start, i.start + i.length)],
                       dtype=np.int32),
        ]
    return sections, infos, widths


def _views(on_device: torch.Tensor, sizes: list[int], infos: list[EntryInfo], widths: list[int],
           page_sizes: list[int], block_size: int, max_context: int | None = None,
           entry_splits: tuple[int, ...] = ()) -> StepBatch:
    offsets = np.cumsum([0] + sizes)

    def part(i: int) -> torch.Tensor:
        return on_device[int(offsets[i]):int(offsets[i + 1])]

    e = len(infos)
    paged = [PagedView(part(FIXED_SECTIONS + 2 * g), part(FIXED_SECTIONS + 1 + 2 * g).view(e, widths[g]), size)
             for g, size in enumerate(page_sizes)]
    splits = {}
    for index, threshold in enumerate(entry_splits):
        at = FIXED_SECTIONS + 2 * len(page_sizes) + 2 * index
        short = sum(i.length for i in infos if i.length <= threshold)
        splits[int(threshold)] = EntrySplit(int(threshold), part(at), part(at + 1), sizes[0] - short, short)
    return StepBatch(
        num_tokens=sizes[0], num_entries=e, num_logit_rows=sizes[7],
        token_ids=part(0), positions=part(1), token_entry=part(2), entry_start=part(3),
        entry_first_position=part(4), context_lens=part(5), state_slots=part(6), logit_rows=part(7),
        paged=paged, entries=infos, splits=splits,
        max_entry_len=max((i.length for i in infos), default=0),
        max_context=max_context if max_context is not None else max((i.first_position + i.length for i in infos), default=0),
        block_size=block_size,
    )


def build_step(entries: list[StepEntry], cache: CacheManager, device: torch.device,
               entry_splits: tuple[int, ...] = ()) -> StepBatch:
    """Lay out the step on the host and copy it to the device in one transfer.

    Pages for the new tokens must already be reserved: slot mappings and block
    tables are read from the cache manager as they stand.
    """
    sections, infos, widths = _layout(entries, cache, None, entry_splits=tuple(entry_splits))
    packed = torch.from_numpy(np.concatenate(sections))
    return _views(packed.to(device), [s.size for s in sections], infos, widths,
                  [group.page_size for group in cache.groups], cache.block_size, entry_splits=tuple(entry_splits))


class StaticStep:
    """A step of fixed shape (one token and one wanted logit per entry, block tables of fixed width)
    whose device arrays stay in place, so that a captured HIP graph can be replayed on new contents."""

    def __init__(self, entries: list[StepEntry], cache: CacheManager, device: torch.device,
                 table_widths: list[int], pad_to: int = 0, entry_splits: tuple[int, ...] = ()) -> None:
        self.table_widths = list(table_widths)
        self.pad_to = int(pad_to)
        self.entry_splits = tuple(entry_splits)
        sections, infos, widths = _layout(entries, cache, self.table_widths, self.pad_to, self.entry_splits)
        self.sizes = [s.size for s in sections]
        # Staging in pinned memory, several buffers in turn: the copy to the device is asynchronous, so the
        # host can lay out the next step while the device still runs this one.  A buffer is written again
        # only after the copy that read it has finished (its event).
        self.hosts = [torch.empty(sum(self.sizes), dtype=torch.int32).pin_memory() for _ in range(self.STAGING)]
        self.copied: list[torch.cuda.Event | None] = [None] * self.STAGING
        self.turn = 0
        self.device_buffer = torch.empty(sum(self.sizes), dtype=torch.int32, device=device)
        # kernels that size their launch by the context use the widest the tables allow
        sizes = [group.page_size for group in cache.groups]
        self.batch = _views(self.device_buffer, self.sizes, infos, widths, sizes, cache.block_size,
                            max_context=min((w * s for w, s in zip(self.table_widths, sizes)), default=cache.block_size),
                            entry_splits=self.entry_splits)
        self._fill(sections, infos)

    STAGING = 4

    def _fill(self, sections, infos) -> None:
        turn, self.turn = self.turn, (self.turn + 1) % self.STAGING
        if self.copied[turn] is not None:
            self.copied[turn].synchronize()
        np.concatenate(sections, out=self.hosts[turn].numpy())
        self.device_buffer.copy_(self.hosts[turn], non_blocking=True)     # in stream order, after the last replay
        event = torch.cuda.Event()
        event.record()
        self.copied[turn] = event
        self.batch.entries = infos

    def update(self, entries: list[StepEntry], cache: CacheManager) -> StepBatch:
        sections, infos, _ = _layout(entries, cache, self.table_widths, self.pad_to, self.entry_splits)
        if [s.size for s in sections] != self.sizes:
            raise ValueError("the entries do not fit the shape this step was laid out for")
        self._fill(sections, infos)
        return self.batch
