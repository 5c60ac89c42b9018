"""The cache: a slot for each live sequence, keys and values of every layer in pages, and state of
fixed size per sequence.

The reference keeps one run state per sequence with flat ``[layers][max_seq][kv_dim]`` arrays
(/root/reference/src/engine/tq_transformer.c:208-281) and, beside them, recurrent state of fixed size
(``delta_state``, ``conv_state``, tq_transformer.c:290-313); its block cache in ``src/cache`` hands out
blocks on demand with create / append / seq_len / free calls and status checks
(/root/reference/src/cache/tq_paged_cache.c:35-243).  This cache serves many sequences at once:

* A *slot* stands for one live sequence: its length, its pages, its row of every state tensor.
  Slots are opened when a batch starts, closed when its sequence ends, and handed out again.
* Keys and values live in *pages* of ``page_size`` positions.  Layers whose needs agree (kv heads,
  width of a key row, width of a value row, window) form a *group* with storage of its own: one pool of
  pages (a group that keeps a window has a pool for its windows only: what every sequence's window, and the
  ``window_step`` positions that one step may add to it, can hold), each page holding the rows of all the group's layers for ``page_size`` positions of one sequence:
  keys laid out ``[layer][kv head][row][head_dim]``, values transposed, ``[layer][kv head][value_dim][row]``
  (both as the attention kernels' operands want them).  Keys and values have pools of their own, so their
  rows may differ in width, and a group whose layers keep one row per position only (``value_dim`` 0) has no
  value pool at all.  A group that keeps a window gives back the pages that have fallen out of every later
  token's window, so its sequences hold pages for the window only.
* The page table of a group, ``[slot][logical page] -> page`` (-1: none), lives on the device and is
  updated only when pages change hands; kernels find a token's rows through its slot.
* A schedule entry that reads another entry's cache gets a view of that entry's storage and none
  of its own.

All bookkeeping is on the host and independent of the device, so it is tested without one.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """No page or slot is free for what was asked."""


class PagePool:
    """Free list of the pages of one group."""

    def __init__(self, n_pages: int):
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))   # pop() hands out low numbers first
        self._held = bytearray(n_pages)

    @property
    def n_free(self) -> int:
        return len(self._free)

    def take(self, n: int) -> list[int]:
        if n > len(self._free):
            raise CacheFull(f"cache needs {n} more pages, {len(self._free)} of {self.n_pages} are free")
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            self._held[p] = 1
        return pages

    def give_back(self, pages) -> None:
        for p in pages:
            if not 0 <= p < self.n_pages or not self._held[p]:
                raise CacheError(f"page {p} is given back but is not held")
            self._held[p] = 0
            self._free.append(p)


@dataclass(frozen=True)
class GroupKey:
    num_kv_heads: int
    head_dim: int
    value_dim: int
    window: int | None


@dataclass
class KVView:
    """What a mixer needs to reach its keys and values."""
    k_pages: torch.Tensor | None      # flat pool of the group's keys
    v_pages: torch.Tensor | None      # flat pool of the group's values (None: the group keeps keys only)
    table: torch.Tensor | None        # int32 [slots, logical pages]
    layer_offset: int                 # offset of the layer's key rows inside a key page, in elements
    page_size: int
    page_stride: int                  # elements per key page
    window: int | None
    owns: bool                        # False: this run reads another run's keys and values and writes none
    v_layer_offset: int = 0           # the same for values; equal to the keys' when both rows are as wide
    v_page_stride: int = 0
    value_dim: int = 0


class CacheGroup:
    def __init__(self, key: GroupKey, entries: list[int], n_pages: int, page_size: int, max_slots: int,
                 max_pages_per_seq: int, dtype: torch.dtype, device):
        self.key = key
        self.entries = entries
        self.page_size = page_size
        self.layer_elems = key.num_kv_heads * page_size * key.head_dim
        self.v_layer_elems = key.num_kv_heads * page_size * key.value_dim
        self.page_stride = len(entries) * self.layer_elems
        self.v_page_stride = len(entries) * self.v_layer_elems
        self.pool = PagePool(n_pages)
        self.max_pages_per_seq = max_pages_per_seq
        self.host_table = np.full((max_slots, max_pages_per_seq), -1, dtype=np.int32)
        self.dirty: set[int] = set()
        self.device = device
        self._staging = None
        self.k_pages = self.v_pages = self.table = None     # without a device: bookkeeping only
        if device is not None:
            # zeroed once: rows beyond a sequence's length are read by tiled kernels (and masked), so they
            # must always hold finite numbers; pages that come back from a sequence do
            self.k_pages = torch.zeros(n_pages * self.page_stride, dtype=dtype, device=device)
            if self.v_page_stride:
                self.v_pages = torch.zeros(n_pages * self.v_page_stride, dtype=dtype, device=device)
            self.table = torch.full((max_slots, max_pages_per_seq), -1, dtype=torch.int32, device=device)

    def offset_of(self, entry: int) -> int:
        return self.entries.index(entry) * self.layer_elems

    def v_offset_of(self, entry: int) -> int:
        return self.entries.index(entry) * self.v_layer_elems

    def first_needed_page(self, length: int) -> int:
        """Lowest logical page that a token at position >= length can still attend to."""
        if self.key.window is None:
            return 0
        return max(0, length - self.key.window + 1) // self.page_size

    def sync(self) -> None:
        """Sends the rows of the page table that changed to the device.  On a GPU they go through pinned memory
        with copies that the host does not wait for (a copy from ordinary memory returns only when everything
        issued before it has run, a decode step that was issued ahead included); the pinned rows are written again
        only after an event behind the last copies has passed."""
        if not self.dirty or self.table is None:
            self.dirty.clear()
            return
        rows = sorted(self.dirty)
        self.dirty.clear()
        n = len(rows)
        if torch.device(self.device).type != "cuda":
            self.table[torch.tensor(rows, dtype=torch.int64)] = torch.from_numpy(self.host_table[rows])
            return
        st = self._staging
        if st is None or st["rows"].shape[0] < n:
            cap = max(n, 8)
            st = self._staging = {"rows": torch.empty((cap, self.max_pages_per_seq), dtype=torch.int32).pin_memory(),
                                  "idx": torch.empty((cap,), dtype=torch.int64).pin_memory(),
                                  "copied": torch.cuda.Event()}
        else:
            st["copied"].synchronize()
        st["rows"].numpy()[:n] = self.host_table[rows]
        st["idx"].numpy()[:n] = rows
        dev_rows = st["rows"][:n].to(self.device, non_blocking=True)
        dev_idx = st["idx"][:n].to(self.device, non_blocking=True)
        st["copied"].record()
        self.table.index_copy_(0, dev_idx, dev_rows)


@dataclass
class Slot:
    index: int
    length: int = 0
    live: bool = False
    reserved: int = 0                 # positions reserved beyond length by the running step


class PagedCache:
    """Slots, page groups and per-sequence state for one model.

    ``needs``: for every schedule entry ``(cache_need or None, state_need or None, cache_of or None)``.
    ``max_tokens``: the most positions live sequences hold at once, each rounded up to whole pages.
    """

    def __init__(self, needs, max_tokens: int, dtype: torch.dtype, device, page_size: int = 64,
                 max_slots: int | None = None, max_positions: int | None = None, window_step: int = 2048):
        """``window_step``: the most positions that one step adds to a sequence where a group keeps a window; such a
        group's pool is sized for ``max_slots`` windows of that reach, and whoever runs longer steps cuts them
        (``step_limit`` says so: None where no pool is smaller for it)."""
        if page_size < 1 or max_tokens < 1 or window_step < 1:
            raise CacheError("page_size, max_tokens and window_step must be positive")
        self.page_size = page_size
        self.n_pages = -(-max_tokens // page_size)
        self.max_slots = min(self.n_pages, 4096) if max_slots is None else max_slots
        per_seq = self.n_pages if max_positions is None else min(self.n_pages, -(-max_positions // page_size))
        self.max_positions = per_seq * page_size if max_positions is None else min(per_seq * page_size, max_positions)
        self.dtype, self.device = dtype, device
        self.slots = [Slot(i) for i in range(self.max_slots)]
        self._free_slots = list(range(self.max_slots - 1, -1, -1))

        by_key: dict[GroupKey, list[int]] = {}
        self._entry_group: dict[int, tuple[CacheGroup, int, bool]] = {}
        self._needs = list(needs)
        for e, (cache_need, _state, cache_of) in enumerate(self._needs):
            if cache_need is not None and cache_of is None:
                by_key.setdefault(GroupKey(cache_need.num_kv_heads, cache_need.head_dim, cache_need.value_width,
                                           cache_need.window), []).append(e)
        # A sequence holds, of a group with a window, the pages that its last `window` positions touch, and during a
        # step those of the step's new positions too, until the step is committed: window + window_step positions
        # lie in at most that many pages plus two.
        self.step_limit: int | None = None
        self.groups: list[CacheGroup] = []
        for key, entries in by_key.items():
            pages = self.n_pages
            if key.window is not None:
                for_windows = self.max_slots * (-(-(key.window + window_step) // page_size) + 2)
                if for_windows < pages:
                    pages, self.step_limit = for_windows, window_step
            self.groups.append(CacheGroup(key, entries, pages, page_size, self.max_slots, per_seq, dtype, device))
        self._v_offset: dict[int, int] = {}
        for g in self.groups:
            for e in g.entries:
                self._entry_group[e] = (g, g.offset_of(e), True)
                self._v_offset[e] = g.v_offset_of(e)
        for e, (cache_need, _state, cache_of) in enumerate(self._needs):
            if cache_need is not None and cache_of is not None:
                if cache_of not in self._entry_group or not self._entry_group[cache_of][2]:
                    raise CacheError(f"schedule entry {e} reads the cache of entry {cache_of}, which keeps none of its own")
                g, off, _ = self._entry_group[cache_of]
                src = self._needs[cache_of][0]
                if (src.num_kv_heads, src.head_dim, src.value_width) != \
                        (cache_need.num_kv_heads, cache_need.head_dim, cache_need.value_width):
                    raise CacheError(f"schedule entry {e} reads the cache of entry {cache_of} but their head counts or sizes differ")
                if src.window is not None and (cache_need.window is None or cache_need.window > src.window):
                    raise CacheError(f"schedule entry {e} looks further back than entry {cache_of}, whose cache it reads, keeps")
                self._entry_group[e] = (g, off, False)
                self._v_offset[e] = self._v_offset[cache_of]

        self.states: dict[int, torch.Tensor] = {}
        for e, (_cache, state_need, _of) in enumerate(self._needs):
            if state_need is not None and device is not None:
                self.states[e] = torch.zeros((self.max_slots, *state_need.shape), dtype=state_need.dtype, device=device)

    # ------------------------------------------------------------ slots
    @property
    def n_live(self) -> int:
        return self.max_slots - len(self._free_slots)

    def open(self) -> int:
        """A slot for a new sequence of length 0 with zeroed state."""
        if not self._free_slots:
            raise CacheFull(f"all {self.max_slots} slots hold live sequences")
        i = self._free_slots.pop()
        s = self.slots[i]
        s.length, s.live, s.reserved = 0, True, 0
        for st in self.states.values():
            st[i].zero_()
        return i

    def close(self, slot: int) -> None:
        """Ends a sequence: its pages and its slot go back."""
        s = self._live(slot)
        for g in self.groups:
            row = g.host_table[slot]
            held = row[row >= 0]
            if held.size:
                g.pool.give_back(held.tolist())
                row[:] = -1
                g.dirty.add(slot)
        s.live, s.length, s.reserved = False, 0, 0
        self._free_slots.append(slot)

    def length(self, slot: int) -> int:
        return self._live(slot).length

    def _live(self, slot: int) -> Slot:
        if not 0 <= slot < self.max_slots or not self.slots[slot].live:
            raise CacheError(f"slot {slot} holds no live sequence")
        return self.slots[slot]

    # ------------------------------------------------------------ a step's positions
    def reserve(self, slot: int, n_new: int) -> int:
        """Makes room for positions length .. length+n_new-1 in every group; returns the first of them."""
        s = self._live(slot)
        if s.reserved:
            raise CacheError(f"slot {slot} already has positions reserved for a running step")
        end = s.length + n_new
        if end > self.max_positions:
            raise CacheFull(f"sequence in slot {slot} would reach {end} positions, the cache holds {self.max_positions} per sequence")
        first_page, last_page = s.length // self.page_size, (end - 1) // self.page_size
        for g in self.groups:
            row = g.host_table[slot]
            missing = [p for p in range(first_page, last_page + 1) if row[p] < 0]
            if missing:
                try:
                    pages = g.pool.take(len(missing))
                except CacheFull:
                    self._undo_reserve(slot, g)
                    raise
                row[missing] = pages
                g.dirty.add(slot)
        s.reserved = n_new
        return s.length

    def room_for(self, slots, counts) -> None:
        """Raises CacheFull if the groups that keep every position (and each sequence's own bound) have no room for
        ``counts[i]`` more positions in ``slots[i]``, all together; takes nothing.  For a step that is run in cuts:
        the groups with a window have room for every cut by the size of their pools."""
        need = 0
        for slot, n in zip(slots, counts):
            s = self._live(slot)
            if s.length + n > self.max_positions:
                raise CacheFull(f"sequence in slot {slot} would reach {s.length + n} positions, the cache holds {self.max_positions} per sequence")
            held = (s.length + self.page_size - 1) // self.page_size
            need += (s.length + n + self.page_size - 1) // self.page_size - held
        for g in self.groups:
            if g.key.window is None and need > g.pool.n_free:
                raise CacheFull(f"cache needs {need} more pages, {g.pool.n_free} of {g.pool.n_pages} are free")

    def needs_page(self, slot: int, n_new: int = 1) -> bool:
        """Whether ``n_new`` more positions would take a page that the sequence does not hold yet."""
        s = self._live(slot)
        first_page, last_page = s.length // self.page_size, (s.length + n_new - 1) // self.page_size
        if last_page >= self.groups[0].max_pages_per_seq if self.groups else False:
            return True
        return any((g.host_table[slot][first_page:last_page + 1] < 0).any() for g in self.groups)

    @property
    def n_free_slots(self) -> int:
        return len(self._free_slots)

    def _undo_reserve(self, slot: int, failed: CacheGroup | None) -> None:
        """Gives back the pages beyond the sequence's length, in the groups before ``failed`` (None: in all)."""
        s = self.slots[slot]
        keep_upto = (s.length - 1) // self.page_size if s.length else -1
        for g in self.groups:
            if g is failed:
                break
            row = g.host_table[slot]
            extra = [p for p in range(keep_upto + 1, g.max_pages_per_seq) if row[p] >= 0]
            if extra:
                g.pool.give_back(row[extra].tolist())
                row[extra] = -1
                g.dirty.add(slot)

    def cancel(self, slot: int) -> None:
        """The step that reserved positions did not run: they do not count, and pages taken for them go back."""
        s = self._live(slot)
        s.reserved = 0
        self._undo_reserve(slot, None)

    def commit(self, slot: int) -> None:
        """The step that reserved positions has run: they now count, and pages that no later token's
        window reaches go back to their pool."""
        s = self._live(slot)
        s.length += s.reserved
        s.reserved = 0
        for g in self.groups:
            first = g.first_needed_page(s.length)
            if first > 0:
                row = g.host_table[slot]
                old = [p for p in range(first) if row[p] >= 0]
                if old:
                    g.pool.give_back(row[old].tolist())
                    row[old] = -1
                    g.dirty.add(slot)

    # ------------------------------------------------------------ a sequence that outlives its request
    def truncate(self, slot: int, length: int) -> None:
        """Forgets the positions from ``length`` on, so that the sequence can go on from there with other tokens.
        Refused (CacheError) where that cannot be done: a group with a window has given back pages that a token at
        ``length`` would look at, or the model keeps fixed-size state per sequence, which has no earlier value."""
        s = self._live(slot)
        if s.reserved:
            raise CacheError(f"slot {slot} has positions reserved for a running step")
        if not 0 <= length <= s.length:
            raise CacheError(f"slot {slot} holds {s.length} positions, not {length}")
        if length == s.length:
            return
        if any(state is not None for _c, state, _o in self._needs):
            raise CacheError("a model with fixed-size state per sequence cannot go back to an earlier position")
        last = (length - 1) // self.page_size if length else -1
        for g in self.groups:
            row = g.host_table[slot]
            if any(row[p] < 0 for p in range(g.first_needed_page(length), last + 1)):
                raise CacheError(f"the window of a group has given back pages that position {length} would look at")
        for g in self.groups:
            row = g.host_table[slot]
            gone = [p for p in range(g.max_pages_per_seq) if row[p] >= 0 and (p > last or p < g.first_needed_page(length))]
            if gone:
                g.pool.give_back(row[gone].tolist())
                row[gone] = -1
                g.dirty.add(slot)
        s.length = length

    def export_slot(self, slot: int) -> dict:
        """What the cache holds of one sequence, on the host: its length, per group the logical pages it holds
        (first page, keys [pages, page elements], values) and per entry its row of fixed-size state."""
        s = self._live(slot)
        if s.reserved:
            raise CacheError(f"slot {slot} has positions reserved for a running step")
        out = {"length": s.length, "page_size": self.page_size, "groups": [], "states": {}}
        last = (s.length - 1) // self.page_size if s.length else -1
        for g in self.groups:
            first = g.first_needed_page(s.length)
            row = g.host_table[slot]
            pages = [int(row[p]) for p in range(first, last + 1)]
            if any(p < 0 for p in pages):
                raise CacheError(f"slot {slot} does not hold all pages of its {s.length} positions")
            idx = torch.tensor(pages, dtype=torch.int64, device=self.device)
            entry = {"first_page": first, "entries": list(g.entries), "key": (g.key.num_kv_heads, g.key.head_dim, g.key.value_dim, g.key.window),
                     "keys": g.k_pages.view(-1, g.page_stride)[idx].cpu(), "values": None}
            if g.v_pages is not None:
                entry["values"] = g.v_pages.view(-1, g.v_page_stride)[idx].cpu()
            out["groups"].append(entry)
        for e, st in self.states.items():
            out["states"][e] = st[slot].cpu()
        return out

    def import_slot(self, data: dict) -> int:
        """A new slot that holds what ``export_slot`` gave (of a cache of the same model, page size and type)."""
        if data["page_size"] != self.page_size or len(data["groups"]) != len(self.groups):
            raise CacheError("the saved sequence comes from a cache of another layout")
        for g, d in zip(self.groups, data["groups"]):
            if tuple(d["key"]) != (g.key.num_kv_heads, g.key.head_dim, g.key.value_dim, g.key.window) or \
                    list(d["entries"]) != list(g.entries) or d["keys"].dtype != self.dtype or \
                    d["keys"].shape[1] != g.page_stride or (d["values"] is None) != (g.v_pages is None):
                raise CacheError("the saved sequence comes from a cache of another layout")
        slot = self.open()
        try:
            length = int(data["length"])
            if length:
                self.reserve(slot, length)
                self.commit(slot)
            last = (length - 1) // self.page_size if length else -1
            for g, d in zip(self.groups, data["groups"]):
                first = g.first_needed_page(length)
                if d["first_page"] != first or d["keys"].shape[0] != last + 1 - first:
                    raise CacheError("the saved pages do not cover the saved length")
                row = g.host_table[slot]
                idx = torch.tensor([int(row[p]) for p in range(first, last + 1)], dtype=torch.int64, device=self.device)
                if idx.numel():
                    g.k_pages.view(-1, g.page_stride)[idx] = d["keys"].to(self.device)
                    if g.v_pages is not None:
                        g.v_pages.view(-1, g.v_page_stride)[idx] = d["values"].to(self.device)
            for e, st in data["states"].items():
                self.states[int(e)][slot].copy_(st.to(self.device))
        except BaseException:
            self.slots[slot].reserved = 0
            self.close(slot)
            raise
        return slot

    def sync(self) -> None:
        for g in self.groups:
            g.sync()

    # ------------------------------------------------------------ views
    def kv(self, entry: int) -> KVView:
        if entry not in self._entry_group:
            raise CacheError(f"schedule entry {entry} keeps no keys and values")
        g, off, owns = self._entry_group[entry]
        return KVView(g.k_pages, g.v_pages, g.table, off, g.page_size, g.page_stride, self._needs[entry][0].window, owns,
                      self._v_offset[entry], g.v_page_stride, g.key.value_dim)

    def state(self, entry: int) -> torch.Tensor:
        if entry not in self.states:
            raise CacheError(f"schedule entry {entry} keeps no per-sequence state")
        return self.states[entry]

    def pages_held(self) -> dict[int, int]:
        """Pages in use per group index."""
        return {i: g.pool.n_pages - g.pool.n_free for i, g in enumerate(self.groups)}

    def bytes(self) -> int:
        n = 0
        for g in self.groups:
            for pages in (g.k_pages, g.v_pages):
                if pages is not None:
                    n += pages.numel() * pages.element_size()
        return n
