"""The cache manager: keys and values in pages, a block table per request and
group, and slots for per-request state of fixed size.

A mixer states what it needs of the cache as a ``CacheNeed``.  Cache layers
with equal needs form a group; a group owns a pool of page ids, one device
tensor for keys and one for values, and one block table per request, so layers
that keep all keys and layers that keep a window of them do not share pages.
A window group gives a page back as soon as every slot of it lies before the
window of all tokens still to come; every group gives all of a request's pages
back when the request ends.  A group has as many pages as it can use: one that
keeps all keys the number asked for, a window group no more than its requests
can ever hold together (``window_group_pages``).  (The reference has one group
and no window: model/src/qwen3_kv_cache.cpp:14-44, engine/src/block_manager.cpp.)

Prefix caching (off unless asked for; the reference's block manager does the same,
engine/src/block_manager.cpp:24-64, 184-224): every full page gets a hash chained
over the hashes of the pages before it and its own token ids (FNV-1a, 64 bit).  A
new request whose leading full pages (all but its last page, so that at least one
token is always computed) are known takes those pages instead of computing them:
a page that is still held is shared (its reference count goes up), a page that is
free but not yet handed out again is revived.  A page leaves the cache when the
pool hands it out for something else.  Shared pages are never written: the tokens
of a shared prefix are not run again.  It is available only when every group keeps
all keys and no mixer keeps state, because a passed window page or a state cannot
be taken over.

What a page holds is the mixer's to say (``CacheRecord``): the manager deals in
page ids only.  The attention part keeps keys ``[cache layer in group, page, kv
head, slot, head_dim]`` and values ``[cache layer in group, page, kv head,
head_dim, slot]``.  The block table of a request maps ``position // page_size``
to a page id, -1 where no page is held.
"""
from __future__ import annotations

from array import array
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

from .pages import PageError, PagePool


class CacheFull(RuntimeError):
    """No pages (or state slots) are left for what was asked."""


PAGE = -1          # in a record's ``dims``: the axis that counts the tokens of a page


@dataclass(frozen=True)
class CacheRecord:
    """One tensor a mixer keeps per token, given as the shape of one page of it: ``dims`` with
    ``PAGE`` where the page's token slots are counted (exactly once).  ``dtype`` None: the run's
    storage type, else a torch dtype.  The engine allocates, per group of layers,
    ``[layers in group, pages, *dims]`` with ``PAGE`` replaced by the page size, zeroed."""
    name: str
    dims: Tuple[int, ...]
    dtype: object = None

    def __post_init__(self):
        if list(self.dims).count(PAGE) != 1 or any(d <= 0 for d in self.dims if d != PAGE):
            raise ValueError(f"cache record '{self.name}': dims {self.dims} must be positive sizes "
                             f"with PAGE exactly once")

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        return tuple(page_size if d == PAGE else d for d in self.dims)

    def elems_per_token(self) -> int:
        n = 1
        for d in self.dims:
            if d != PAGE:
                n *= d
        return n


@dataclass(frozen=True)
class CacheNeed:
    """What one mixer needs of the paged cache: the records it keeps for every token and
    how far back its rows read (``window`` None: everything, else the last ``window``
    tokens, so that pages before the window can be given back).  Cache layers whose needs
    are equal share a group: page ids, block tables and tensors of their own."""
    records: Tuple[CacheRecord, ...]
    window: Optional[int] = None

    def __post_init__(self):
        names = [r.name for r in self.records]
        if not names or len(set(names)) != len(names):
            raise ValueError("a cache need names at least one record, each once")

    @staticmethod
    def keys_and_values(num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> "CacheNeed":
        """The records of attention over keys and values: keys ``[kv head, slot, head_dim]``,
        values transposed ``[kv head, head_dim, slot]``, so that each matrix-core operand is
        contiguous along the index it is contracted over."""
        return CacheNeed((CacheRecord("k", (num_kv_heads, PAGE, head_dim)),
                          CacheRecord("v", (num_kv_heads, head_dim, PAGE))), window)


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size state per request: ``shape`` elements of ``dtype`` (a torch dtype)."""
    shape: Tuple[int, ...]
    dtype: object


@dataclass
class GroupLayout:
    need: CacheNeed
    cache_layers: List[int]            # global cache layer ids, in group order
    pool: PagePool
    index: int = 0

    def local_layer(self, cache_layer: int) -> int:
        return self.cache_layers.index(cache_layer)


class PageTable(array):
    """The block table of a request in one group: block -> page id or -1, 32-bit integers in
    one piece of memory, so that a step packs it into its inputs with one copy
    (``numpy.frombuffer``) however long it has grown.  Reads like a list, and is equal to any
    sequence of the same numbers."""

    def __new__(cls, pages=()):
        return super().__new__(cls, "i", pages)

    def __eq__(self, other):
        return list(self) == list(other)

    def __ne__(self, other):
        return not self.__eq__(other)

    __hash__ = None


@dataclass
class RequestCache:
    """What one live request holds."""
    key: Hashable
    slot: int
    num_tokens: int = 0                               # tokens whose keys are in the cache
    hashed_blocks: int = 0                            # leading pages already in the prefix cache
    prefix_hash: int = 0                              # chained hash of those pages
    tables: List[PageTable] = field(default_factory=list)    # per group: block -> page or -1
    reserved_tokens: int = 0                          # positions [0, reserved) are covered


def _blocks(tokens: int, page: int) -> int:
    return (tokens + page - 1) // page


_FNV_OFFSET = 1469598103934665603
_FNV_PRIME = 1099511628211
_MASK64 = (1 << 64) - 1


def page_hash(tokens: Sequence[int], prefix_hash: int) -> int:
    """FNV-1a over the 8 bytes of the previous page's hash, then the 4 bytes of
    each token id, little-endian (engine/src/block_manager.cpp:24-43)."""
    h = _FNV_OFFSET
    for shift in range(0, 64, 8):
        h = ((h ^ ((prefix_hash >> shift) & 0xFF)) * _FNV_PRIME) & _MASK64
    for t in tokens:
        v = int(t) & 0xFFFFFFFF
        for shift in range(0, 32, 8):
            h = ((h ^ ((v >> shift) & 0xFF)) * _FNV_PRIME) & _MASK64
    return h


def window_group_pages(window: int, page_size: int, max_requests: int, max_step_tokens: int) -> int:
    """The most pages that the live requests of a window group can hold together.  A request that
    has s tokens in the cache and runs c more holds the blocks from the first one a query at s
    reads to the one its last token is written to: at most (window - 1 + c) / page + 2, the
    window and the portion each straddling a page's edge.  Over ``max_requests`` requests whose
    portions of one step add up to ``max_step_tokens``."""
    blocks = lambda n: (n + page_size - 1) // page_size
    return max_requests * (blocks(window - 1) + 2) + blocks(max_step_tokens)


def group_needs(needs: Sequence[Optional["CacheNeed"]]) -> List["CacheNeed"]:
    """The distinct needs among ``needs`` in the order the groups are made."""
    out: List[CacheNeed] = []
    for need in needs:
        if need is not None and need not in out:
            out.append(need)
    return out


class CacheManager:
    def __init__(self, needs: Sequence[Optional[CacheNeed]], page_size: int, num_pages,
                 max_requests: int, prefix_caching: bool = False, max_step_tokens: Optional[int] = None):
        """``needs[i]`` is the need of cache layer i (None: that layer keeps nothing).
        ``num_pages``: the pages (of ``page_size`` slots) of a group that keeps all keys, or a
        list with one count for every group (``group_needs`` gives their order).  Given one
        number and ``max_step_tokens`` (the most tokens that the requests of one step bring
        together), a window group gets no more pages than ``window_group_pages`` says it can
        use; without it every group gets ``num_pages``."""
        per_group = None if isinstance(num_pages, int) else [int(n) for n in num_pages]
        if page_size <= 0 or max_requests <= 0 or (per_group is None and num_pages <= 0) \
                or (per_group is not None and any(n <= 0 for n in per_group)):
            raise ValueError("page_size, num_pages and max_requests must be positive")
        distinct = group_needs(needs)
        if per_group is None:
            per_group = [num_pages if (n.window is None or max_step_tokens is None) else
                         min(num_pages, window_group_pages(n.window, page_size, max_requests, max_step_tokens))
                         for n in distinct]
        if len(per_group) != len(distinct):
            raise ValueError(f"{len(per_group)} page counts for {len(distinct)} groups of cache layers")
        self.page_size = page_size
        self.num_pages = max(per_group, default=0)         # of the largest group
        self.max_requests = max_requests
        self.groups: List[GroupLayout] = []
        self.group_of_layer: Dict[int, int] = {}
        by_need: Dict[CacheNeed, GroupLayout] = {}
        for layer, need in enumerate(needs):
            if need is None:
                continue
            g = by_need.get(need)
            if g is None:
                g = GroupLayout(need, [], PagePool(per_group[len(self.groups)]), index=len(self.groups))
                by_need[need] = g
                self.groups.append(g)
            g.cache_layers.append(layer)
            self.group_of_layer[layer] = g.index
        self._no_window = all(g.need.window is None for g in self.groups)
        self._free_slots = list(range(max_requests - 1, -1, -1))   # pop() gives the lowest
        self._live: Dict[Hashable, RequestCache] = {}
        self.pages_taken_total = 0
        self.pages_returned_total = 0
        if prefix_caching and any(g.need.window is not None for g in self.groups):
            raise ValueError("prefix caching needs every layer to keep all keys (no window)")
        self.prefix_caching = prefix_caching
        # per group: hash -> page, and per page its (hash, token ids) while it is in the cache
        self._page_of_hash: List[Dict[int, int]] = [dict() for _ in self.groups]
        self._known: List[Dict[int, Tuple[int, Tuple[int, ...]]]] = [dict() for _ in self.groups]
        self.prefix_hits = 0                # pages taken over instead of computed

    # ---- requests -------------------------------------------------------
    def live(self) -> List[Hashable]:
        return list(self._live)

    def get(self, key: Hashable) -> RequestCache:
        return self._live[key]

    def __contains__(self, key: Hashable) -> bool:
        return key in self._live

    def free_slots(self) -> int:
        return len(self._free_slots)

    def admit(self, key: Hashable) -> RequestCache:
        """Give a new request a state slot and empty block tables."""
        if key in self._live:
            raise ValueError(f"request {key!r} is already live")
        if not self._free_slots:
            raise CacheFull("no state slot is free")
        slot = self._free_slots.pop()
        rc = RequestCache(key=key, slot=slot, tables=[PageTable() for _ in self.groups])
        self._live[key] = rc
        return rc

    # ---- prefix cache ---------------------------------------------------
    def _take(self, gi: int) -> int:
        """A fresh page of group gi; what the prefix cache knew of it is forgotten."""
        page = self.groups[gi].pool.take()
        known = self._known[gi].pop(page, None)
        if known is not None and self._page_of_hash[gi].get(known[0]) == page:
            del self._page_of_hash[gi][known[0]]
        self.pages_taken_total += 1
        return page

    def match_prefix(self, tokens: Sequence[int]) -> List[List[int]]:
        """Pages (per group) that hold the leading full pages of ``tokens``: as many
        as every group knows, never the last page of the sequence."""
        if not self.prefix_caching or not self.groups:
            return [[] for _ in self.groups]
        out: List[List[int]] = [[] for _ in self.groups]
        prefix = 0
        nb = _blocks(len(tokens), self.page_size)
        for b in range(nb - 1):
            chunk = tuple(int(t) for t in tokens[b * self.page_size:(b + 1) * self.page_size])
            if len(chunk) != self.page_size:
                break
            prefix = page_hash(chunk, prefix)
            found = []
            for gi in range(len(self.groups)):
                page = self._page_of_hash[gi].get(prefix)
                known = None if page is None else self._known[gi].get(page)
                if known is None or known[0] != prefix or known[1] != chunk:   # collision check
                    found = None
                    break
                found.append(page)
            if found is None:
                break
            for gi, page in enumerate(found):
                out[gi].append(page)
        return out

    def adopt_prefix(self, key: Hashable, tokens: Sequence[int]) -> int:
        """Give a just admitted request the cached pages of its prefix; returns how
        many tokens need not be computed."""
        rc = self._live[key]
        if rc.num_tokens or any(rc.tables):
            raise ValueError("a prefix can only be adopted by a request that holds nothing")
        matched = self.match_prefix(tokens)
        n = len(matched[0]) if matched else 0
        for gi, pages in enumerate(matched):
            pool = self.groups[gi].pool
            for page in pages:
                if pool.is_free(page):
                    pool.revive(page)
                    self.pages_taken_total += 1
                else:
                    pool.share(page)
                rc.tables[gi].append(page)
        rc.num_tokens = n * self.page_size
        rc.reserved_tokens = rc.num_tokens
        rc.hashed_blocks = n
        rc.prefix_hash = 0
        for b in range(n):
            rc.prefix_hash = page_hash(tokens[b * self.page_size:(b + 1) * self.page_size], rc.prefix_hash)
        self.prefix_hits += n
        return rc.num_tokens

    def register_pages(self, key: Hashable, tokens: Sequence[int]) -> None:
        """After a step: the request's newly completed full pages enter the cache
        (engine/src/block_manager.cpp:184-224).  ``tokens`` are all its tokens."""
        if not self.prefix_caching:
            return
        rc = self._live[key]
        full = min(rc.num_tokens, len(tokens)) // self.page_size
        for b in range(rc.hashed_blocks, full):
            chunk = tuple(int(t) for t in tokens[b * self.page_size:(b + 1) * self.page_size])
            rc.prefix_hash = page_hash(chunk, rc.prefix_hash)
            for gi in range(len(self.groups)):
                page = rc.tables[gi][b]
                old = self._known[gi].pop(page, None)
                if old is not None and self._page_of_hash[gi].get(old[0]) == page:
                    del self._page_of_hash[gi][old[0]]
                self._known[gi][page] = (rc.prefix_hash, chunk)
                self._page_of_hash[gi][rc.prefix_hash] = page
        rc.hashed_blocks = max(rc.hashed_blocks, full)

    # ---- pages ----------------------------------------------------------
    def _first_needed_block(self, g: GroupLayout, first_query_pos: int) -> int:
        """Lowest block a query at ``first_query_pos`` (and any later one) can read."""
        if g.need.window is None:
            return 0
        return max(0, first_query_pos - g.need.window + 1) // self.page_size

    def pages_needed(self, key: Hashable, new_total: int) -> List[int]:
        """Per group, pages that must be taken so that the request can run the
        tokens at positions [num_tokens, new_total)."""
        rc = self._live[key]
        nb = _blocks(new_total, self.page_size)
        if self._no_window:                   # (every step of every request comes through here: the short way)
            return [max(0, nb - len(table)) for table in rc.tables]
        out = []
        for gi, g in enumerate(self.groups):
            # every block from the first one a query at num_tokens reads up to the table's end is
            # held (``reserve`` filled them, ``advance`` gives back only what lies before): what is
            # missing are the blocks past the table's end
            first = self._first_needed_block(g, rc.num_tokens)
            out.append(max(0, nb - max(first, len(rc.tables[gi]))))
        return out

    def can_reserve(self, key: Hashable, new_total: int) -> bool:
        return all(n <= g.pool.free_count
                   for n, g in zip(self.pages_needed(key, new_total), self.groups))

    def most_pages_needed(self, total_tokens: int, portion: int) -> List[int]:
        """Per group, the most pages one request of ``total_tokens`` tokens ever holds when it is
        run in portions of at most ``portion`` tokens: all its blocks where all keys are kept, the
        window's and a portion's where a window passes."""
        whole = _blocks(total_tokens, self.page_size)
        out = []
        for g in self.groups:
            if g.need.window is None:
                out.append(whole)
            else:
                out.append(min(whole, _blocks(g.need.window - 1, self.page_size) + 2
                               + _blocks(min(portion, total_tokens), self.page_size)))
        return out

    def pages_per_group(self) -> List[int]:
        return [g.pool.num_pages for g in self.groups]

    def _ahead_needed(self, rc: RequestCache, total: int) -> List[int]:
        nb = _blocks(total, self.page_size)
        return [max(0, nb - len(rc.tables[gi])) if g.need.window is None else 0
                for gi, g in enumerate(self.groups)]

    def can_hold_ahead(self, key: Hashable, total: int) -> bool:
        return all(n <= g.pool.free_count
                   for n, g in zip(self._ahead_needed(self._live[key], total), self.groups))

    def hold_ahead(self, key: Hashable, total: int) -> None:
        """Take now, in the groups that keep all keys, the pages for ``total`` tokens of the
        request, so that once it is admitted no other request can take them from under it (the
        reference allocates a whole prompt at admission, engine/src/block_manager.cpp:87-119).
        Window groups take theirs portion by portion (``reserve``), since they give them back
        the same way.  All or nothing."""
        rc = self._live[key]
        if not self.can_hold_ahead(key, total):
            raise CacheFull(f"not enough free pages to hold {total} tokens of {key!r}")
        nb = _blocks(total, self.page_size)
        for gi, g in enumerate(self.groups):
            if g.need.window is None:
                table = rc.tables[gi]
                while len(table) < nb:
                    table.append(self._take(gi))

    def reserve(self, key: Hashable, new_total: int) -> None:
        """Take pages so that positions up to ``new_total`` can be written and
        everything a query in [num_tokens, new_total) reads is held.  All or
        nothing: CacheFull leaves the request as it was."""
        rc = self._live[key]
        if new_total < rc.num_tokens:
            raise ValueError("a request cannot shrink")
        needs = self.pages_needed(key, new_total)
        if not any(needs) and self._no_window:            # a token that goes into a page already held
            if new_total > rc.reserved_tokens:
                rc.reserved_tokens = new_total
            return
        if any(n > g.pool.free_count for n, g in zip(needs, self.groups)):
            raise CacheFull(f"not enough free pages to hold {new_total} tokens of {key!r}")
        nb = _blocks(new_total, self.page_size)
        for gi, g in enumerate(self.groups):
            table = rc.tables[gi]
            held = len(table)
            first = self._first_needed_block(g, rc.num_tokens)
            while len(table) < min(first, nb):
                table.append(-1)                  # (a window has jumped past these blocks)
            for b in range(max(first, held), nb):
                table.append(self._take(gi))
        rc.reserved_tokens = max(rc.reserved_tokens, new_total)

    def advance(self, key: Hashable, new_total: int) -> None:
        """Record that the tokens up to ``new_total`` are now in the cache and
        give back the pages of window groups that no later token can read."""
        rc = self._live[key]
        if new_total > rc.reserved_tokens:
            raise ValueError(f"{key!r}: {new_total} tokens were run but only "
                             f"{rc.reserved_tokens} were reserved")
        rc.num_tokens = new_total
        for gi, g in enumerate(self.groups):
            if g.need.window is None:
                continue
            table = rc.tables[gi]
            first = min(self._first_needed_block(g, new_total), len(table))
            for b in range(first):
                if table[b] >= 0:
                    g.pool.release(table[b])
                    self.pages_returned_total += 1
                    table[b] = -1

    def release(self, key: Hashable) -> None:
        """The request has ended (or is preempted): all it holds is given back,
        pages in reverse table order as the reference does
        (engine/src/block_manager.cpp:150-159)."""
        rc = self._live.pop(key)
        for gi, g in enumerate(self.groups):
            for page in reversed(rc.tables[gi]):
                if page >= 0:
                    g.pool.release(page)
                    self.pages_returned_total += 1
            rc.tables[gi] = PageTable()
        self._free_slots.append(rc.slot)
        self._free_slots.sort(reverse=True)

    # ---- inspection -----------------------------------------------------
    def free_pages(self) -> List[int]:
        return [g.pool.free_count for g in self.groups]

    def check(self) -> None:
        """No page lost, held twice or freed twice; slots likewise."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            held: Dict[int, int] = {}
            for rc in self._live.values():
                for page in rc.tables[gi]:
                    if page >= 0:
                        held[page] = held.get(page, 0) + 1
                # what ``pages_needed`` counts on: no hole from the first block that is read to the end
                first = self._first_needed_block(g, rc.num_tokens)
                if any(page < 0 for page in rc.tables[gi][first:]):
                    raise PageError(f"group {gi}: the table of {rc.key!r} has a hole at or after block {first}")
            for page in range(g.pool.num_pages):
                if g.pool.ref_count(page) != held.get(page, 0):
                    raise PageError(f"group {gi} page {page}: pool counts "
                                    f"{g.pool.ref_count(page)} holders, tables show {held.get(page, 0)}")
        slots = [rc.slot for rc in self._live.values()] + self._free_slots
        if sorted(slots) != list(range(self.max_requests)):
            raise PageError("state slots are lost or held twice")
