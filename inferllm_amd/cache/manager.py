"""The cache of a model: slots, paged key/value storage per group of layers, and
fixed-size state per sequence.

Layout.  A *cache line* is the storage one run of a layer uses (the schedule
names it).  Lines with the same needs form a *group* with storage of its own:

* kind "full": every key and value of a sequence is kept;
* kind "window": only the last `window` keys are ever read, so a sequence keeps a
  ring of pages and its storage stops growing.

What a line keeps per token is a list of named tensors (`TokenTensor`: name, per-token shape,
dtype), which its mixer states: attention keeps "k" and "v" of [kv heads, head_dim]; another
mixer may keep one latent row, keys and values of different widths, or a dtype of its own.  A
tensor of per-token shape (*lead, d) is stored as [line][page][*lead][row in page][d]; a page has
`page_size` (64) rows, so for keys one kv head's part of a page is contiguous.  Each group
has its own page pool and its own page table [slot][logical page] -> page.  The
last slot and the last page of every group are spare: rows that only pad a batch
point there.  Sequence lengths live in `slot_len`, one int per slot, on the host
and on the device.

Beside the groups, `StateSpec`s describe tensors of fixed size per sequence
([slot, *shape]), zeroed when a slot is handed out.

The reference keeps, per attention op, two tensors [n_ctx, embd] and a cursor
(src/core/kvstorage.h:9-54), grown lazily in steps of 100 rows
(src/core/kvstotage.cpp:53-76), for its single sequence.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .slots import CacheError, CacheFull, FreeList

PAGE_SIZE = 64


def round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


@dataclass(frozen=True)
class TokenTensor:
    """One tensor a cache line keeps per token: its name, its per-token shape, and its dtype
    (None: the engine's)."""
    name: str
    shape: Tuple[int, ...]
    dtype: Optional[torch.dtype] = None

    def __post_init__(self):
        if not self.shape or any(int(n) <= 0 for n in self.shape):
            raise CacheError(f"per-token tensor {self.name!r} needs a shape of positive sizes")


@dataclass(frozen=True)
class KVSpec:
    """What one cache line needs: which tokens are kept ("full": all, "window": the last
    `window`) and the tensors kept of each."""
    kind: str
    tensors: Tuple[TokenTensor, ...]
    window: Optional[int] = None

    def __post_init__(self):
        if self.kind not in ("full", "window"):
            raise CacheError(f"unknown cache kind {self.kind!r}")
        if self.kind == "window" and not (self.window and self.window > 0):
            raise CacheError("a window cache needs a positive window")
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise CacheError(f"a cache line needs per-token tensors with distinct names, got {names}")

    @classmethod
    def keys_values(cls, num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> "KVSpec":
        """Attention's needs: "k" and "v" of [kv heads, head_dim] in the engine's dtype."""
        shape = (int(num_kv_heads), int(head_dim))
        return cls("window" if window else "full",
                   (TokenTensor("k", shape), TokenTensor("v", shape)), window or None)


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state per sequence for one cache line: shape and dtype."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class KVGroup:
    """Storage, page pool and page table of the lines that share one `KVSpec`."""

    def __init__(self, spec: KVSpec, lines: Sequence[int], n_slots: int, max_tokens: int,
                 max_seq_len: int, dtype: torch.dtype, device, page_size: int = PAGE_SIZE,
                 step_rows: int = 0):
        self.spec = spec
        self.lines = list(lines)
        self.page_size = page_size
        pages_full = max(1, max_tokens // page_size)
        seq_pages = max(1, round_up(max_seq_len, page_size) // page_size)
        if spec.kind == "window":
            # pages that the last `window` keys of any position can touch, and `step_rows` more
            # rows: a step stores all its keys before its rows read, so the keys of a step of n
            # tokens must not reach round the ring into the window of the step's first row
            self.ring = (spec.window + max(0, step_rows - 1) + page_size - 2) // page_size + 1
            if self.ring >= seq_pages:
                self.ring = 0           # the window never wraps: same as "full"
        else:
            self.ring = 0
        self.pages_per_seq = self.ring if self.ring else seq_pages
        self.n_pages = min(pages_full, n_slots * self.pages_per_seq)
        self.pool = FreeList(self.n_pages, "page", scatter=True)
        self.spare_page = self.n_pages
        self.tensors: Dict[str, torch.Tensor] = {}
        for t in spec.tensors:
            shape = (len(self.lines), self.n_pages + 1) + tuple(t.shape[:-1]) + (page_size, t.shape[-1])
            self.tensors[t.name] = torch.zeros(shape, dtype=t.dtype or dtype, device=device)
        self.table_host = torch.full((n_slots + 1, self.pages_per_seq), self.spare_page,
                                     dtype=torch.int32)
        self.table = self.table_host.to(device)
        self.held: Dict[int, List[int]] = {}     # slot -> pages in logical order
        self._dirty = set()

    @property
    def k(self) -> torch.Tensor:
        return self.tensors["k"]

    @property
    def v(self) -> torch.Tensor:
        return self.tensors["v"]

    @property
    def step_limit(self) -> Optional[int]:
        """Most tokens a sequence may go on by in one step so that none of the step's keys lands
        on a key that a row of the step still reads (None: no limit, nothing wraps)."""
        return self.ring * self.page_size - self.spec.window + 1 if self.ring else None

    def line_index(self, line: int) -> int:
        return self.lines.index(line)

    def _poison(self, pages: Sequence[int]) -> None:
        for t in self.tensors.values():
            if pages and t.dtype.is_floating_point:
                t[:, torch.tensor(list(pages), dtype=torch.long, device=t.device)] = float("nan")

    def pages_needed(self, length: int) -> int:
        n = (length + self.page_size - 1) // self.page_size
        return min(n, self.ring) if self.ring else n

    def reserve(self, slot: int, length: int) -> None:
        pages = self.held.setdefault(slot, [])
        need = self.pages_needed(length)
        if need > self.pages_per_seq:
            raise CacheFull(f"a sequence of {length} tokens needs {need} pages; "
                            f"{self.pages_per_seq} is the most one sequence may hold")
        if need - len(pages) > self.pool.n_free():
            raise CacheFull(f"cache full: {need - len(pages)} more pages of {self.page_size} tokens "
                            f"needed, {self.pool.n_free()} of {self.n_pages} free")
        while len(pages) < need:
            p = self.pool.alloc()
            self.table_host[slot, len(pages)] = p
            pages.append(p)
            self._dirty.add(slot)

    def shrink(self, slot: int, length: int, poison: bool = False) -> None:
        """Give back the pages that a sequence of only `length` tokens does not need."""
        pages = self.held.get(slot, [])
        need = self.pages_needed(length)
        gone = pages[need:]
        if not gone:
            return
        del pages[need:]
        if poison:
            self._poison(gone)
        for p in gone:
            self.pool.free(p)
        self.table_host[slot, need:need + len(gone)] = self.spare_page
        self._dirty.add(slot)

    def release(self, slot: int, poison: bool = False) -> None:
        pages = self.held.pop(slot, [])
        if poison:
            self._poison(pages)
        for p in pages:
            self.pool.free(p)
        self.table_host[slot].fill_(self.spare_page)
        self._dirty.add(slot)

    def upload(self) -> None:
        for slot in sorted(self._dirty):
            self.table[slot].copy_(self.table_host[slot])
        self._dirty.clear()


class CacheManager:
    """Slots, KV groups and per-sequence state for one model on one device.

    `max_tokens` is the most tokens that live sequences hold together, each
    sequence rounded up to whole pages; `max_slots` the most live sequences;
    `max_seq_len` the longest one sequence may become.
    """

    def __init__(self, kv_lines: Dict[int, KVSpec], state_lines: Dict[int, StateSpec],
                 max_tokens: int, max_slots: int, max_seq_len: int, dtype: torch.dtype, device,
                 page_size: int = PAGE_SIZE, poison_freed: bool = False, step_rows: int = 0):
        """`step_rows`: the most tokens by which a sequence that already holds tokens goes on in
        one step without the step being cut (`step_limit`); it sizes the rings of window groups
        and costs nothing where nothing is a ring."""
        if max_slots <= 0 or max_tokens <= 0 or max_seq_len <= 0:
            raise CacheError("max_slots, max_tokens and max_seq_len must be positive")
        self.page_size = page_size
        self.max_tokens = round_up(max_tokens, page_size)
        self.max_slots = max_slots
        self.max_seq_len = max_seq_len
        self.device = torch.device(device)
        self.dtype = dtype
        self.poison_freed = poison_freed
        self.slots = FreeList(max_slots, "slot")
        self.spare_slot = max_slots
        by_spec: Dict[KVSpec, List[int]] = {}
        for line in sorted(kv_lines):
            by_spec.setdefault(kv_lines[line], []).append(line)
        self.groups: List[KVGroup] = [
            KVGroup(spec, lines, max_slots, self.max_tokens, max_seq_len, dtype, device, page_size,
                    step_rows)
            for spec, lines in by_spec.items()]
        limits = [g.step_limit for g in self.groups if g.step_limit is not None]
        # most tokens a sequence may bring to a step that reads the cache (None: any number)
        self.step_limit: Optional[int] = min(limits) if limits else None
        self._group_of: Dict[int, KVGroup] = {l: g for g in self.groups for l in g.lines}
        self.states: Dict[int, torch.Tensor] = {
            line: torch.zeros((max_slots + 1,) + tuple(s.shape), dtype=s.dtype, device=device)
            for line, s in state_lines.items()}
        self.len_host = torch.zeros(max_slots + 1, dtype=torch.int32)
        self._len = self.len_host.numpy()       # the same memory; element access costs far less
        self._len[self.spare_slot] = 1          # padding rows attend to one (spare) key, not to none
        self.slot_len = self.len_host.to(device)
        self._len_dirty = False

    # ------------------------------------------------------------ slots
    def alloc_slot(self) -> int:
        slot = self.slots.alloc()
        self._len[slot] = 0
        self._len_dirty = True
        for t in self.states.values():
            t[slot].zero_()
        return slot

    def free_slot(self, slot: int) -> None:
        self.slots.free(slot)           # raises if not held
        for g in self.groups:
            g.release(slot, self.poison_freed)
        self._len[slot] = 0
        self._len_dirty = True

    def length(self, slot: int) -> int:
        return int(self._len[slot])

    # ------------------------------------------------------------ steps
    def extend(self, slot: int, start_pos: int, n_tokens: int) -> None:
        """Make room for `n_tokens` more tokens of `slot`, which must now hold `start_pos`."""
        if not self.slots.holds(slot):
            raise CacheError(f"slot {slot} is not held")
        have = int(self._len[slot])
        if start_pos != have:
            raise CacheError(f"slot {slot} holds {have} tokens; a step starting at {start_pos} "
                             "does not follow")
        new_len = have + n_tokens
        if new_len > self.max_seq_len:
            raise CacheFull(f"sequence would reach {new_len} tokens; the limit is {self.max_seq_len}")
        for g in self.groups:
            g.reserve(slot, new_len)
        self._len[slot] = new_len
        self._len_dirty = True

    def rewind(self, slot: int, n_tokens: int) -> None:
        """Take the last `n_tokens` of `slot` back: the next step goes on from the shorter
        sequence and writes over what they left.  Only keys and values can be taken back (a
        window's ring keeps everything the shorter sequence still sees as long as no more tokens
        are taken back than a step may bring); fixed-size state cannot, so a cache with state
        refuses."""
        if not self.slots.holds(slot):
            raise CacheError(f"slot {slot} is not held")
        if self.states:
            raise CacheError("per-sequence state cannot be taken back by tokens")
        have = int(self._len[slot])
        if not 0 <= n_tokens <= have:
            raise CacheError(f"slot {slot} holds {have} tokens; {n_tokens} cannot be taken back")
        for g in self.groups:
            if g.ring and n_tokens > g.step_limit:
                raise CacheError(f"a window's ring does not keep what {n_tokens} tokens wrote over")
            g.shrink(slot, have - n_tokens, self.poison_freed)
        self._len[slot] = have - n_tokens
        self._len_dirty = True

    def check_room(self, items: Sequence[Tuple[int, int, int]]) -> None:
        """Raise unless every (slot, start_pos, n_tokens) of a step follows its slot and the step
        as a whole fits; nothing is changed."""
        for g in self.groups:
            more = 0
            for slot, start, n in items:
                more += max(0, g.pages_needed(start + n) - len(g.held.get(slot, ())))
            if more > g.pool.n_free():
                raise CacheFull(f"cache full: this step needs {more} more pages of "
                                f"{g.page_size} tokens, {g.pool.n_free()} of {g.n_pages} are free")
        for slot, start, n in items:
            if not self.slots.holds(slot):
                raise CacheError(f"slot {slot} is not held")
            if start != int(self._len[slot]):
                raise CacheError(f"slot {slot} holds {int(self._len[slot])} tokens; a step "
                                 f"starting at {start} does not follow")
            if start + n > self.max_seq_len:
                raise CacheFull(f"sequence would reach {start + n} tokens; the limit is "
                                f"{self.max_seq_len}")

    def extend_all(self, items: Sequence[Tuple[int, int, int]]) -> None:
        """`extend` for every (slot, start_pos, n_tokens) of a step, or for none of them: if the
        step as a whole does not fit, CacheFull is raised and the cache is as it was."""
        self.check_room(items)
        for slot, start, n in items:
            self.extend(slot, start, n)

    def upload(self, lengths: bool = True) -> None:
        """Bring page tables (and, unless `lengths` is False, the per-slot lengths) on the
        device up to date with the host.  Steps of single tokens carry their sequences'
        lengths themselves and leave `slot_len` for the next step of whole prompts."""
        for g in self.groups:
            g.upload()
        if lengths and self._len_dirty:
            self.slot_len.copy_(self.len_host)
            self._len_dirty = False

    # ------------------------------------------------------------ views for parts
    def kv_line(self, line: int):
        """(K, V, group) of a cache line that keeps "k" and "v"; K and V are
        [page, kv head, row, head_dim]."""
        g = self._group_of[line]
        i = g.line_index(line)
        return g.k[i], g.v[i], g

    def token_line(self, line: int):
        """(name -> tensor [page, *lead, row, d], group) of a cache line: everything it keeps per
        token."""
        g = self._group_of[line]
        i = g.line_index(line)
        return {name: t[i] for name, t in g.tensors.items()}, g

    def state_line(self, line: int) -> Optional[torch.Tensor]:
        return self.states.get(line)

    def tokens_held(self) -> int:
        """Tokens held now, each sequence rounded up to whole pages."""
        return sum(round_up(int(self._len[s]), self.page_size) for s in self.slots.held())

    def check(self) -> None:
        self.slots.check()
        for g in self.groups:
            g.pool.check()
            held = [p for pages in g.held.values() for p in pages]
            if sorted(held) != g.pool.held():
                raise CacheError("pages held by slots differ from pages taken from the pool")
            if set(g.held) - set(self.slots.held()):
                raise CacheError("a freed slot still holds pages")
