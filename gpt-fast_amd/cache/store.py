"""The cache of a model: a slot for each live sequence, keys and values in pages, and
fixed-size state per sequence.

What each run of a layer needs is stated by its mixer as a *need*:

* :class:`KVNeed` - keys and values of every earlier token (or of a window of them), for
  ``n_kv_heads`` heads of ``head_dim`` (values of ``value_dim``, if that differs);
* :class:`StateNeed` - a tensor of fixed shape per sequence, zeroed when a slot is
  acquired (attention has none; a recurrent mixer would keep its state here);
* ``None`` - nothing (or the run borrows another run's entry);
* any other type registered with :func:`register_cache_need` together with the class of
  its groups (a compressed latent per token, a ring of recent tokens, ...).

Runs with equal needs form a *group* with storage of its own; a group is an object with the
methods of :class:`Group`, and the cache itself only hands out slots, counts lengths and
asks its groups:

* a KV group owns ``k`` ``[entries, n_pages + 1, n_kv_heads, PAGE, head_dim]`` and ``v``
  ``[entries, n_pages + 1, n_kv_heads, value_dim, PAGE]`` and a free list of pages; a
  sequence holds, per group, a list of pages that grows by one page every ``PAGE`` tokens.
  A windowed group gives pages back once every key in them is out of reach.  Pages are
  reused without clearing: a reader never looks beyond a sequence's length (the reference
  relies on the same masking when it reuses its buffers, model.py:118-119).  A group with
  ``paged = True`` gets a table of page numbers per sequence in every step's description.
* a state group owns ``[entries, n_slots + 1, *shape]``; the last slot belongs to no
  sequence (rows that only fill a recorded batch's shape use it).

The reference's cache is one ``[batch, heads, max_len, head_dim]`` buffer pair per layer
with one shared position for all rows (model.py:84-100, 117-134); here every sequence has
its own length and the pool is sized in tokens, not in rows times maximum length.
"""
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import torch

from ..ops.kernels import PAGE
from .slots import CacheFull, FreeList


@dataclass(frozen=True)
class KVNeed:
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None       # None: as head_dim

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class StateNeed:
    shape: Tuple[int, ...]
    dtype: str = "float32"


def pages_for(n_tokens: int) -> int:
    return (n_tokens + PAGE - 1) // PAGE


@dataclass(frozen=True)
class Geometry:
    """What a cache gives its groups to size themselves by."""
    n_pages: int          # pages of PAGE tokens in every paged group's pool
    n_slots: int          # sequences alive at once


class Group:
    """What the cache asks of a group.  ``paged`` groups appear in a step's description with
    a table of ``table_entries(slot)`` numbers per sequence, written by ``fill_table_row``."""

    paged = False

    def acquire(self, slot: int) -> None:
        """A new sequence takes ``slot``."""

    def release(self, slot: int) -> None:
        """The sequence in ``slot`` has ended: give back what it holds."""

    def plan_extend(self, items, lengths) -> Optional[Callable[[], None]]:
        """``items`` = (slot, new tokens) of one step, ``lengths`` the sequences' lengths
        before it.  Raise :class:`CacheFull` if the group cannot take them; else return what
        commits the reservation (or None): the cache commits only if every group agrees."""
        return None

    def check(self, slots: FreeList) -> None:
        """Bookkeeping invariants (tests)."""

    def bytes_per_token(self) -> int:
        """Bytes a one-token step reads of this group per cached token."""
        return 0

    def snapshot(self) -> Optional[Callable[[], None]]:
        """What puts the group's contents back after a step is run twice (the warm-up of a
        recording); None if a repeated step writes the same bytes."""
        return None


class KVGroup(Group):
    paged = True

    def __init__(self, need: KVNeed, entries: int, geometry: Geometry, dtype, device):
        self.need = need
        self.entries = entries
        self.n_pages = n_pages = geometry.n_pages
        # Every (page, kv head) owns PAGE * head_dim elements of keys and PAGE * value_dim of
        # values.  The last two dimensions only give that size: inside, the kernels keep the
        # elements in the order in which the matrix-core attention reads its operands
        # (csrc/common.h: key_offset, value_offset), and nothing in Python looks inside.
        # one page beyond the pool (index n_pages) belongs to no sequence: rows of a batch
        # that only fill a fixed shape are pointed at it
        self.k = torch.empty((entries, n_pages + 1, need.n_kv_heads, PAGE, need.head_dim),
                             dtype=dtype, device=device)
        self.v = torch.empty((entries, n_pages + 1, need.n_kv_heads, need.v_dim, PAGE),
                             dtype=dtype, device=device)
        self.spare_page = n_pages
        self.k[:, n_pages].zero_()
        self.v[:, n_pages].zero_()
        self.pages = FreeList(n_pages, "cache page")
        self.held: Dict[int, List[int]] = {}      # slot -> page of each PAGE tokens, -1 = given back

    def bytes_per_token(self) -> int:
        return (self.entries * self.need.n_kv_heads * (self.need.head_dim + self.need.v_dim)
                * self.k.element_size())

    def acquire(self, slot):
        self.held[slot] = []

    def release(self, slot):
        for p in self.held.pop(slot):
            if p >= 0:
                self.pages.give(p)

    def plan_extend(self, items, lengths):
        plans, demand = [], 0
        for slot, n_new in items:
            start = lengths[slot]
            held = self.held[slot]
            first_needed = 0
            if self.need.window is not None:
                first_needed = max(0, start - self.need.window + 1) // PAGE
            drop = [i for i in range(min(first_needed, len(held))) if held[i] >= 0]
            grow = max(pages_for(start + n_new) - len(held), 0)
            plans.append((held, drop, grow))
            demand += grow - len(drop)
        if demand > self.pages.free:
            raise CacheFull(
                f"the cache holds {self.n_pages * PAGE} tokens in pages of {PAGE}; this "
                f"step needs {demand} more pages and {self.pages.free} are free")

        def commit():
            for held, drop, grow in plans:
                for i in drop:
                    self.pages.give(held[i])
                    held[i] = -1
                for _ in range(grow):
                    held.append(self.pages.take())
        return commit

    # the step's description
    def table_entries(self, slot: int) -> int:
        return len(self.held[slot])

    def fill_table_row(self, row, slot: Optional[int]) -> None:
        """Page numbers of the sequence in ``slot`` (-1 where it holds none), or the spare
        page throughout for a row that belongs to no sequence."""
        if slot is None:
            row[:] = self.spare_page
            return
        pages = self.held[slot]
        row[:len(pages)] = pages
        row[len(pages):] = -1

    def check(self, slots):
        self.pages.check()
        seen = set()
        for slot, held in self.held.items():
            if not slots.is_held(slot):
                raise AssertionError(f"pages are held for slot {slot}, which is free")
            for p in held:
                if p < 0:
                    continue
                if p in seen:
                    raise AssertionError(f"page {p} is held by two sequences")
                if not self.pages.is_held(p):
                    raise AssertionError(f"page {p} is in use but on the free list")
                seen.add(p)
        if len(seen) != self.pages.held:
            raise AssertionError("a page is marked held but belongs to no sequence")


class StateGroup(Group):
    def __init__(self, need: StateNeed, entries: int, geometry: Geometry, dtype, device):
        self.need = need
        self.entries = entries
        # one slot beyond the pool (index n_slots) belongs to no sequence: rows of a batch
        # that only fill a fixed shape read and write it
        self.data = torch.zeros((entries, geometry.n_slots + 1) + tuple(need.shape),
                                dtype=getattr(torch, need.dtype), device=device)

    def acquire(self, slot):
        self.data[:, slot].zero_()

    def snapshot(self):
        saved = self.data.clone()
        return lambda: self.data.copy_(saved)


# need type -> factory(need, entries, geometry, dtype, device) of its groups
_GROUP_OF_NEED: Dict[type, Callable] = {}


def register_cache_need(need_type: type, group_factory: Callable) -> None:
    """A further kind of cache need: ``need_type`` instances (hashable, equal for runs that
    can share storage) are what a mixer's ``cache_need()`` returns, and
    ``group_factory(need, entries, geometry, dtype, device)`` builds the :class:`Group` that
    stores it for ``entries`` runs."""
    _GROUP_OF_NEED[need_type] = group_factory


register_cache_need(KVNeed, KVGroup)
register_cache_need(StateNeed, StateGroup)


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
    """Slots, lengths and the groups of one model.

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
        geometry = Geometry(self.n_pages, max_sequences)

        order_of_need: Dict[object, int] = {}
        members: List[List[int]] = []
        for n, need in enumerate(needs):
            if need is None or borrow[n] is not None:
                continue
            if need not in order_of_need:
                order_of_need[need] = len(members)
                members.append([])
            members[order_of_need[need]].append(n)
        self.groups: List[Group] = []
        for need, gid in order_of_need.items():
            factory = _GROUP_OF_NEED.get(type(need))
            if factory is None:
                known = ", ".join(sorted(t.__name__ for t in _GROUP_OF_NEED))
                raise TypeError(f"a mixer's cache need must be None or of a registered kind "
                                f"({known}), not {type(need).__name__}")
            self.groups.append(factory(need, len(members[gid]), geometry, dtype, device))
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

    # ------------------------------------------------------------------ groups by kind
    @property
    def paged_groups(self) -> List[Tuple[int, Group]]:
        """Groups that get a table per sequence in a step's description."""
        return [(i, g) for i, g in enumerate(self.groups) if g.paged]

    @property
    def kv_groups(self) -> List[Tuple[int, KVGroup]]:
        return [(i, g) for i, g in enumerate(self.groups) if isinstance(g, KVGroup)]

    @property
    def state_groups(self) -> List[Tuple[int, StateGroup]]:
        return [(i, g) for i, g in enumerate(self.groups) if isinstance(g, StateGroup)]

    # ------------------------------------------------------------------ sequences
    def acquire(self) -> int:
        """A free slot for a new sequence: length 0, no pages, state zeroed."""
        slot = self.slots.take()
        self.lengths[slot] = 0
        for g in self.groups:
            g.acquire(slot)
        return slot

    def release(self, slot: int) -> None:
        """Give the slot and everything it holds back."""
        if not self.slots.is_held(slot):
            raise ValueError(f"sequence slot {slot} is released but is not held")
        for g in self.groups:
            g.release(slot)
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
        commits = [g.plan_extend(items, self.lengths) for g in self.groups]    # may raise CacheFull
        for commit in commits:
            if commit is not None:
                commit()
        before = []
        for slot, n_new in items:
            before.append(self.lengths[slot])
            self.lengths[slot] += n_new
        return before

    def page_list(self, group_id: int, slot: int) -> List[int]:
        return self.groups[group_id].held[slot]

    def snapshots(self) -> List[Callable[[], None]]:
        """What undoes a step that is run twice: one callable per group that needs it."""
        return [r for r in (g.snapshot() for g in self.groups) if r is not None]

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
        for g in self.groups:
            g.check(self.slots)
