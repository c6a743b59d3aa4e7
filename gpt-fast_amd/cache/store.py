"""The cache of a model: a slot for each live sequence, keys and values in pages, and
fixed-size state per sequence.

What each run of a layer needs is stated by its mixer as a *need*:

* :class:`KVNeed` - keys and values of every earlier token (or of a window of them), for
  ``n_kv_heads`` heads of ``head_dim``;
* :class:`StateNeed` - a tensor of fixed shape per sequence, zeroed when a slot is
  acquired (attention has none; a recurrent mixer would keep its state here);
* ``None`` - nothing (or the run borrows another run's entry).

Runs with equal needs form a *group* with storage of its own:

* a KV group owns ``k`` and ``v`` of shape ``[entries, n_pages, n_kv_heads, PAGE,
  head_dim]`` and a free list of pages; a sequence holds, per group, a list of pages that
  grows by one page every ``PAGE`` tokens.  A windowed group gives pages back once every
  key in them is out of reach.  Pages are reused without clearing: a reader never looks
  beyond a sequence's length (the reference relies on the same masking when it reuses its
  buffers, model.py:118-119).
* a state group owns ``[entries, n_slots + 1, *shape]``; the last slot belongs to no
  sequence (rows that only fill a recorded batch's shape use it).

The reference's cache is one ``[batch, heads, max_len, head_dim]`` buffer pair per layer
with one shared position for all rows (model.py:84-100, 117-134); here every sequence has
its own length and the pool is sized in tokens, not in rows times maximum length.
"""
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..ops.kernels import PAGE
from .slots import CacheFull, FreeList


@dataclass(frozen=True)
class KVNeed:
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    shape: Tuple[int, ...]
    dtype: str = "float32"


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE - 1) // PAGE


class KVGroup:
    def __init__(self, need: KVNeed, entries: int, n_pages: int, dtype, device):
        self.need = need
        self.entries = entries
        self.n_pages = n_pages
        # Every (page, kv head) owns PAGE * head_dim elements of keys and as many of values.
        # The last two dimensions only give that size: inside, the kernels keep the elements
        # in the order in which the matrix-core attention reads its operands (csrc/common.h:
        # key_offset, value_offset), and nothing in Python looks inside.
        # one page beyond the pool (index n_pages) belongs to no sequence: rows of a batch
        # that only fill a fixed shape are pointed at it
        self.k = torch.empty((entries, n_pages + 1, need.n_kv_heads, PAGE, need.head_dim),
                             dtype=dtype, device=device)
        self.v = torch.empty((entries, n_pages + 1, need.n_kv_heads, need.head_dim, PAGE),
                             dtype=dtype, device=device)
        self.spare_page = n_pages
        self.k[:, n_pages].zero_()
        self.v[:, n_pages].zero_()
        self.pages = FreeList(n_pages, "cache page")
        self.held: Dict[int, List[int]] = {}      # slot -> page of each PAGE tokens, -1 = given back

    def bytes_per_token(self) -> int:
        return 2 * self.entries * self.need.n_kv_heads * self.need.head_dim * self.k.element_size()


class StateGroup:
    def __init__(self, need: StateNeed, entries: int, n_slots: int, device):
        self.need = need
        self.entries = entries
        # one slot beyond the pool (index n_slots) belongs to no sequence: rows of a batch
        # that only fill a fixed shape read and write it
        self.data = torch.zeros((entries, n_slots + 1) + tuple(need.shape),
                                dtype=getattr(torch, need.dtype), device=device)


class CacheEntry:
    """What one run's mixer sees: its group and its index in it."""

    def __init__(self, group_id: int, group, index: int, writes: bool = True):
        self.group_id = group_id
        self.group = group
        self.index = index
        self.writes = writes          # False for a run that borrows another run's entry

    @property
    def k_pages(self) -> torch.Tensor:
        return self.group.k[self.index]

    @property
    def v_pages(self) -> torch.Tensor:
        return self.group.v[self.index]

    @property
    def state(self) -> torch.Tensor:
        """[n_slots + 1, *shape] of a state group; the last row is the spare slot."""
        return self.group.data[self.index]


class Cache:
    """Slots, pages and state for one model.

    ``needs`` has one item per run of the model's order; ``borrow[n]`` names the earlier
    run whose entry run ``n`` reads (or None).  ``max_tokens`` is the most tokens all live
    sequences hold together, each sequence rounded up to whole pages; ``max_sequences`` the
    most sequences alive at once.
    """

    def __init__(self, needs: Sequence[object], borrow: Sequence[Optional[int]], *,
                 max_tokens: int, max_sequences: int, dtype, device):
        if max_tokens <= 0 or max_sequences <= 0:
            raise ValueError("the cache needs room for at least one token and one sequence")
        self.n_pages = pages_for(max_tokens)
        self.max_sequences = max_sequences
        self.dtype = dtype
        self.device = device
        self.slots = FreeList(max_sequences, "sequence slot")
        self.spare_slot = max_sequences         # of state groups; belongs to no sequence
        self.lengths: List[int] = [0] * max_sequences

        order_of_need: Dict[object, int] = {}
        members: List[List[int]] = []
        for n, need in enumerate(needs):
            if need is None or borrow[n] is not None:
                continue
            if need not in order_of_need:
                order_of_need[need] = len(members)
                members.append([])
            members[order_of_need[need]].append(n)
        self.groups: List[object] = []
        for need, gid in order_of_need.items():
            count = len(members[gid])
            if isinstance(need, KVNeed):
                self.groups.append(KVGroup(need, count, self.n_pages, dtype, device))
            elif isinstance(need, StateNeed):
                self.groups.append(StateGroup(need, count, max_sequences, device))
            else:
                raise TypeError(f"a mixer's cache need must be a KVNeed, a StateNeed or None, "
                                f"not {type(need).__name__}")
        self.entries: List[Optional[CacheEntry]] = [None] * len(needs)
        for gid, runs in enumerate(members):
            for index, n in enumerate(runs):
                self.entries[n] = CacheEntry(gid, self.groups[gid], index, writes=True)
        for n, src in enumerate(borrow):
            if src is not None:
                e = self.entries[src]
                if e is None:
                    raise ValueError(f"run {n} borrows the cache of run {src}, which has none")
                self.entries[n] = CacheEntry(e.group_id, e.group, e.index, writes=False)

    # ------------------------------------------------------------------ sequences
    @property
    def kv_groups(self) -> List[Tuple[int, KVGroup]]:
        return [(i, g) for i, g in enumerate(self.groups) if isinstance(g, KVGroup)]

    def acquire(self) -> int:
        """A free slot for a new sequence: length 0, no pages, state zeroed."""
        slot = self.slots.take()
        self.lengths[slot] = 0
        for g in self.groups:
            if isinstance(g, KVGroup):
                g.held[slot] = []
            else:
                g.data[:, slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        """Give the slot and every page it holds back."""
        if not self.slots.is_held(slot):
            raise ValueError(f"sequence slot {slot} is released but is not held")
        for g in self.groups:
            if isinstance(g, KVGroup):
                for p in g.held.pop(slot):
                    if p >= 0:
                        g.pages.give(p)
        self.lengths[slot] = 0
        self.slots.give(slot)

    def length(self, slot: int) -> int:
        return self.lengths[slot]

    def extend(self, slot: int, n_new: int) -> int:
        """Make room for ``n_new`` more tokens of the sequence in ``slot`` and count them
        in.  Returns the length before.  Raises :class:`CacheFull` (nothing changed) if the
        pages do not suffice."""
        return self.extend_many([(slot, n_new)])[0]

    def extend_many(self, items: Sequence[Tuple[int, int]]) -> List[int]:
        """:meth:`extend` for several sequences at once: either all get their room or
        nothing changes.  Returns the lengths before."""
        seen = set()
        for slot, n_new in items:
            if not self.slots.is_held(slot):
                raise ValueError(f"sequence slot {slot} is not held")
            if slot in seen:
                raise ValueError(f"sequence slot {slot} appears twice in one step")
            seen.add(slot)
            if n_new <= 0:
                raise ValueError("a step brings at least one token for each of its sequences")
        plans = []
        for _, g in self.kv_groups:
            demand = 0
            for slot, n_new in items:
                start = self.lengths[slot]
                held = g.held[slot]
                first_needed = 0
                if g.need.window is not None:
                    first_needed = max(0, start - g.need.window + 1) // PAGE
                drop = [i for i in range(min(first_needed, len(held))) if held[i] >= 0]
                grow = max(pages_for(start + n_new) - len(held), 0)
                plans.append((g, slot, drop, grow))
                demand += grow - len(drop)
            if demand > g.pages.free:
                raise CacheFull(
                    f"the cache holds {self.n_pages * PAGE} tokens in pages of {PAGE}; this "
                    f"step needs {demand} more pages and {g.pages.free} are free")
        for g, slot, drop, grow in plans:
            held = g.held[slot]
            for i in drop:
                g.pages.give(held[i])
                held[i] = -1
            for _ in range(grow):
                held.append(g.pages.take())
        before = []
        for slot, n_new in items:
            before.append(self.lengths[slot])
            self.lengths[slot] += n_new
        return before

    def page_list(self, group_id: int, slot: int) -> List[int]:
        return self.groups[group_id].held[slot]

    @property
    def state_groups(self) -> List[Tuple[int, StateGroup]]:
        return [(i, g) for i, g in enumerate(self.groups) if isinstance(g, StateGroup)]

    def require_room(self, lengths: Sequence[int]) -> None:
        """Raise :class:`CacheFull` unless sequences that grow to these lengths fit together
        in an empty cache (slots and, for every group, pages)."""
        if len(lengths) > self.max_sequences:
            raise CacheFull(f"{len(lengths)} sequences at once, but the cache has "
                            f"{self.max_sequences} slots")
        need = sum(pages_for(n) for n in lengths)
        if need > self.n_pages:
            raise CacheFull(
                f"the cache holds {self.n_pages * PAGE} tokens in pages of {PAGE}; sequences "
                f"of {list(lengths)} tokens need {need * PAGE}")

    def tokens_held(self) -> int:
        """Tokens of all live sequences, each rounded up to whole pages."""
        return sum(pages_for(self.lengths[s]) * PAGE
                   for s in range(self.max_sequences) if self.slots.is_held(s))

    def check(self) -> None:
        """Bookkeeping invariants: no slot or page lost, none held twice."""
        self.slots.check()
        for _, g in self.kv_groups:
            g.pages.check()
            seen = set()
            for slot, held in g.held.items():
                if not self.slots.is_held(slot):
                    raise AssertionError(f"pages are held for slot {slot}, which is free")
                for p in held:
                    if p < 0:
                        continue
                    if p in seen:
                        raise AssertionError(f"page {p} is held by two sequences")
                    if not g.pages.is_held(p):
                        raise AssertionError(f"page {p} is in use but on the free list")
                    seen.add(p)
            if len(seen) != g.pages.held:
                raise AssertionError("a page is marked held but belongs to no sequence")
