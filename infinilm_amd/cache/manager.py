"""The cache manager: pages of keys and values with a block table per request, in groups of cache
entries with the same need, and slots of fixed-size state per request.

Reference: data plane csrc/cache/kv_cache.cpp:113-148 (one tensor per layer, here K and V apart,
keys [pages, nkv, page, d], values [pages, nkv, d, page]); control plane python/infinilm/llm/cache_manager.py:158-191 (pages for
a prompt), :317-328 (a new page iff the new token opens one), :330-348 (giving back); fixed-size
state csrc/cache/mamba_cache.cpp:8-47 and cache_manager.py:33-68 (row 0 is the zero state, rows
from a free list).  Differences by design: pages are reserved portion by portion instead of for
the whole prompt at admission, go straight back to the free list when a request ends or a window
has passed them, and cache entries whose mixers keep all keys and those that keep a window form
groups with page pools and block tables of their own.

Prefix sharing (`prefix_caching=True`; the reference's python/infinilm/llm/prefix_cache.py and
cache_manager.py:136-156, scheduler.py:158-164,503-523): a page all of whose tokens have been
computed is published under a key chained over the tokens of the whole prefix; a request admitted
with its tokens takes the longest run of published pages from its start (never the page of its
last token: one token at least has to run to give logits) and begins after them.  Pages of a
request that ends stay findable until the pool needs them.  Only where every cache entry keeps all
keys in pages: a window's pages are given back, and a fixed-size state cannot be taken over.

The control plane (this class) holds no GPU state beyond the tensors it allocates; it can be built
with device="meta" or "cpu" and exercised without a GPU.
"""
from __future__ import annotations

import hashlib
from array import array
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

from .needs import FixedState, PagedKV
from .pages import CacheError, OutOfPages, PagePool


@dataclass
class _Group:
    """Cache entries that share a page-id space and a block table per request."""
    window: int
    entries: List[int]
    pool: PagePool


@dataclass
class _Request:
    length: int = 0                      # tokens whose keys are in the cache
    reserved: int = 0                    # tokens pages are held for (>= length)
    tables: List[List[int]] = field(default_factory=list)   # per group: logical page -> page id, -1 = given back
    state_slot: int = 0
    fresh: bool = True                   # no state written yet: reads start from the zero row
    # prefix sharing: key of the last whole page, tokens since then, whole pages whose key is known;
    # chain None = this request's tokens are unknown (committed without them): nothing is published
    chain: Optional[bytes] = None
    pending: List[int] = field(default_factory=list)
    keyed_pages: int = 0


class KVView:
    """What a mixer's forward gets for a paged entry."""
    __slots__ = ("k", "v", "page_size", "block_tables", "slots", "window")

    def __init__(self, k, v, page_size, block_tables, slots, window):
        self.k, self.v, self.page_size, self.block_tables, self.slots, self.window = k, v, page_size, block_tables, slots, window


class StateView:
    """What a mixer's forward gets for a fixed-size state entry: the pool [slots, *shape], the row
    each request reads at the start of the step (0 = zeros) and the row it writes at the end."""
    __slots__ = ("pool", "state_in", "state_out")

    def __init__(self, pool, state_in, state_out):
        self.pool, self.state_in, self.state_out = pool, state_in, state_out


class CacheManager:
    def __init__(self, needs: Sequence, page_size: int, num_pages: int, max_requests: int,
                 dtype: torch.dtype, device, num_pages_per_group: Optional[Dict[int, int]] = None,
                 prefix_caching: bool = False):
        if page_size <= 0:
            raise CacheError(f"page size must be positive, got {page_size}")
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        self.version = 0   # counts admissions and releases: what was prepared for a set of requests is stale after either
        self.device = torch.device(device)
        self.dtype = dtype
        self.needs = list(needs)
        self.groups: List[_Group] = []
        self.group_of_entry: Dict[int, int] = {}
        by_window: Dict[int, int] = {}
        for e, need in enumerate(self.needs):
            if isinstance(need, PagedKV):
                if need.window not in by_window:
                    n = (num_pages_per_group or {}).get(need.window, num_pages)
                    by_window[need.window] = len(self.groups)
                    self.groups.append(_Group(need.window, [], PagePool(n)))
                g = by_window[need.window]
                self.groups[g].entries.append(e)
                self.group_of_entry[e] = g
        # data plane
        self.k: Dict[int, torch.Tensor] = {}
        self.v: Dict[int, torch.Tensor] = {}
        self.state: Dict[int, torch.Tensor] = {}
        for e, need in enumerate(self.needs):
            if isinstance(need, PagedKV):
                n = self.groups[self.group_of_entry[e]].pool.num_pages
                # keys [pages, nkv, page, d]; values transposed [pages, nkv, d, page], so that the
                # attention kernels read consecutive keys of one dim with one load.  Zero-filled once:
                # what a reused page holds is stale but finite, and lengths bound every read.
                # One page more than the pool gives out, the last: a place for rows that belong to no request
                # (a recorded decode step of 8 rows that serves 5 requests fills up with such rows); what
                # lands there is never read by a request.
                self.k[e] = torch.zeros((n + 1, need.num_kv_heads, self.page_size, need.head_dim), dtype=dtype,
                                        device=self.device)
                self.v[e] = torch.zeros((n + 1, need.num_kv_heads, need.head_dim, self.page_size), dtype=dtype,
                                        device=self.device)
            elif isinstance(need, FixedState):
                # row 0: the zero state; rows 1..max_requests: the slots; the last row: for rows of no request
                self.state[e] = torch.zeros((self.max_requests + 2,) + tuple(need.shape),
                                            dtype=need.dtype or torch.float32, device=self.device)
            elif need is not None:
                raise CacheError(f"cache entry {e}: unknown need {need!r}")
        # state slots: row 0 is the permanent zero state
        self._free_slots = list(range(self.max_requests, 0, -1))
        self.requests: Dict[object, _Request] = {}
        # prefix sharing needs one group that keeps all keys, and no state beside it
        self.prefix_caching = bool(prefix_caching) and len(self.groups) == 1 and self.groups[0].window <= 0 \
            and not self.state
        self._root_key = hashlib.blake2b(b"infinilm_amd page chain 1 " + str(self.page_size).encode(), digest_size=16).digest()
        self.prefix_hit_tokens = 0       # tokens taken over from published pages at admissions
        self.prefix_asked_tokens = 0     # tokens of the prompts admitted with their tokens

    # ---- sizes ----------------------------------------------------------------------------------
    def bytes_per_token(self) -> int:
        total = 0
        for e, need in enumerate(self.needs):
            if isinstance(need, PagedKV):
                total += 2 * need.num_kv_heads * need.head_dim * self.k[e].element_size()
        return total

    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.num_free if self.groups else 0

    def total_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.num_pages if self.groups else 0

    def null_page(self, group: int) -> int:
        """The page of group `group` that belongs to no request (see the data plane above)."""
        return self.groups[group].pool.num_pages

    @property
    def null_state_row(self) -> int:
        return self.max_requests + 1

    def stats(self) -> dict:
        return {"requests": len(self.requests),
                "groups": [{"window": g.window, "entries": len(g.entries), "pages": g.pool.num_pages,
                            "free": g.pool.num_free, "idle": g.pool.num_idle, "evictions": g.pool.evictions,
                            "high_water": g.pool.high_water} for g in self.groups],
                "state_slots_free": len(self._free_slots),
                "prefix_caching": self.prefix_caching, "prefix_hit_tokens": self.prefix_hit_tokens,
                "prefix_asked_tokens": self.prefix_asked_tokens}

    # ---- keys of whole pages ----------------------------------------------------------------------
    def _page_key(self, parent: bytes, tokens: Sequence[int]) -> bytes:
        """Key of a whole page: a hash over the key of the page before it and its own tokens, so it
        stands for the whole prefix."""
        return hashlib.blake2b(parent + array("i", tokens).tobytes(), digest_size=16).digest()

    def _matching_pages(self, tokens: Sequence[int]):
        """(pages, key of the last one) of the longest published run from the start of `tokens` that
        leaves at least the last token to be computed."""
        pool = self.groups[0].pool
        ps = self.page_size
        pages, key = [], self._root_key
        for i in range((len(tokens) - 1) // ps):
            k = self._page_key(key, tokens[i * ps:(i + 1) * ps])
            page = pool.lookup(k)
            if page is None:
                break
            pages.append(page)
            key = k
        return pages, key

    def peek_prefix(self, tokens: Sequence[int]):
        """(tokens an admission with these tokens would take over from published pages, how many of those
        pages are idle now and would leave the pages that can be given out); nothing is pinned."""
        if not self.prefix_caching:
            return 0, 0
        pages = self._matching_pages(tokens)[0]
        pool = self.groups[0].pool
        return len(pages) * self.page_size, sum(1 for p in pages if pool.refs(p) == 0)

    # ---- requests -------------------------------------------------------------------------------
    def admit(self, req_id, tokens: Optional[Sequence[int]] = None) -> int:
        """A new request.  With prefix sharing and the request's `tokens` (all that are known), it takes
        over the published pages that hold its beginning; returns how many tokens they cover: the
        request's length, from which its first step goes on."""
        if req_id in self.requests:
            raise CacheError(f"request {req_id!r} is already admitted")
        if not self._free_slots:
            raise CacheError(f"no state slot free for request {req_id!r} ({self.max_requests} requests at most)")
        r = _Request(tables=[[] for _ in self.groups], state_slot=self._free_slots.pop())
        if self.prefix_caching and tokens is not None:
            pages, key = self._matching_pages(tokens)
            pool = self.groups[0].pool
            for p in pages:
                pool.share(p)
            r.tables[0] = list(pages)
            r.length = r.reserved = len(pages) * self.page_size
            r.chain, r.keyed_pages = key, len(pages)
            self.prefix_hit_tokens += r.length
            self.prefix_asked_tokens += len(tokens)
        self.requests[req_id] = r
        self.version += 1
        return r.length

    def has(self, req_id) -> bool:
        return req_id in self.requests

    def length(self, req_id) -> int:
        return self.requests[req_id].length

    def _first_needed_page(self, group: _Group, first_query_pos: int) -> int:
        if group.window <= 0:
            return 0
        lo = max(0, first_query_pos - group.window + 1)
        return lo // self.page_size

    def pages_needed(self, req_id, n_new: int) -> List[int]:
        """Pages each group would have to take so that `n_new` more tokens fit."""
        r = self.requests[req_id]
        upto = r.length + n_new
        out = []
        for g, table in zip(self.groups, r.tables):
            want = -(-upto // self.page_size)
            out.append(max(0, want - len(table)))
        return out

    def can_reserve(self, req_id, n_new: int) -> bool:
        return all(n <= g.pool.num_free for n, g in zip(self.pages_needed(req_id, n_new), self.groups))

    def reserve(self, req_id, n_new: int) -> None:
        """Take the pages for `n_new` tokens after the cached ones in every group, or OutOfPages
        with nothing taken."""
        r = self.requests[req_id]
        if n_new <= 0:
            raise CacheError(f"reserve of {n_new} tokens")
        need = self.pages_needed(req_id, n_new)
        for n, g in zip(need, self.groups):
            if n > g.pool.num_free:
                raise OutOfPages(f"request {req_id!r}: {n} pages needed for {n_new} tokens after {r.length}, "
                                 f"{g.pool.num_free} free of {g.pool.num_pages} (window {g.window})")
        for n, g, table in zip(need, self.groups, r.tables):
            table.extend(g.pool.take(n))
        r.reserved = max(r.reserved, r.length + n_new)

    def commit(self, req_id, n_new: int, tokens: Optional[Sequence[int]] = None) -> None:
        """`n_new` tokens have been written; give back the pages a window has passed.  With prefix
        sharing, `tokens` (the n_new token ids) let the pages they complete be published; a commit
        without them ends the publishing for this request."""
        r = self.requests[req_id]
        if r.length + n_new > r.reserved:
            raise CacheError(f"request {req_id!r}: commit of {n_new} tokens beyond what was reserved")
        r.length += n_new
        r.fresh = False
        if self.prefix_caching and r.chain is not None:
            if tokens is None or len(tokens) != n_new:
                r.chain, r.pending = None, []
            else:
                self._publish(r, tokens)
        for g, table in zip(self.groups, r.tables):
            first = self._first_needed_page(g, r.length)  # the next query sits at position `length`
            for i in range(min(first, len(table))):
                if table[i] >= 0:
                    g.pool.give_back([table[i]])
                    table[i] = -1

    def slot_of(self, req_id, group: int, position: int) -> int:
        """slot = page_id * page_size + offset (cache_manager.py:186-191)."""
        table = self.requests[req_id].tables[group]
        page = table[position // self.page_size]
        if page < 0:
            raise CacheError(f"request {req_id!r}: position {position} lies on a page already given back")
        return page * self.page_size + position % self.page_size

    def table(self, req_id, group: int) -> List[int]:
        return self.requests[req_id].tables[group]

    def state_rows(self, req_id):
        """(row read at the start of the step, row written at its end)."""
        r = self.requests[req_id]
        return (0 if r.fresh else r.state_slot), r.state_slot

    def snapshot_states(self, req_ids: Sequence) -> list:
        """Copies of the state rows these requests write, for `restore_states`: a step that has to run
        twice on the same books (the warm-up before a graph is recorded) must not advance a state twice.
        Keys and values need nothing of the kind: writing them again writes the same."""
        if not self.state:
            return []
        rows = torch.tensor([self.requests[i].state_slot for i in req_ids], dtype=torch.long, device=self.device)
        return [(pool, rows, pool.index_select(0, rows)) for pool in self.state.values()]

    def restore_states(self, snapshot: list) -> None:
        for pool, rows, saved in snapshot:
            pool.index_copy_(0, rows, saved)

    def _publish(self, r: _Request, tokens: Sequence[int]) -> None:
        ps = self.page_size
        pool = self.groups[0].pool
        r.pending.extend(tokens)
        while len(r.pending) >= ps:
            key = self._page_key(r.chain, r.pending[:ps])
            pool.publish(r.tables[0][r.keyed_pages], key)   # False: the same content is already there; ours stays private
            r.chain = key
            r.keyed_pages += 1
            del r.pending[:ps]

    def release(self, req_id) -> None:
        """The request is over (or preempted): all its pages and its slot go back.  Published pages go
        last page first, so that of a run the end loses its content before the beginning."""
        r = self.requests.pop(req_id, None)
        if r is None:
            raise CacheError(f"request {req_id!r} is not admitted (released twice?)")
        for g, table in zip(self.groups, r.tables):
            pages = [p for p in table if p >= 0]
            g.pool.give_back([p for p in pages if not g.pool.is_published(p)])
            g.pool.give_back([p for p in reversed(pages) if g.pool.is_published(p)])
        self._free_slots.append(r.state_slot)
        self.version += 1

    def check(self) -> None:
        """No page lost, none held twice: the pages in the block tables are exactly the held ones."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            held: Dict[int, int] = {}
            for r in self.requests.values():
                pages = [p for p in r.tables[gi] if p >= 0]
                if len(pages) != len(set(pages)):
                    raise CacheError(f"group {gi}: a page is twice in one block table")
                for p in pages:
                    held[p] = held.get(p, 0) + 1
            for p, n in held.items():
                if g.pool.refs(p) != n:
                    raise CacheError(f"group {gi}: page {p} is in {n} block tables and has {g.pool.refs(p)} owners")
                if n > 1 and not self.prefix_caching:
                    raise CacheError(f"group {gi}: page {p} is in two block tables")
            if len(held) != g.pool.num_held:
                raise CacheError(f"group {gi}: {g.pool.num_held} pages held, {len(held)} in block tables")
        slots = [r.state_slot for r in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots) or 0 in slots:
            raise CacheError("state slots are inconsistent")

    # ---- what a layer sees --------------------------------------------------------------------
    def view(self, entry: int, batch, writes: bool):
        need = self.needs[entry]
        if isinstance(need, PagedKV):
            g = self.group_of_entry[entry]
            return KVView(self.k[entry], self.v[entry], self.page_size, batch.block_tables[g],
                          batch.slots[g] if writes else None, need.window)
        if isinstance(need, FixedState):
            return StateView(self.state[entry], batch.state_in, batch.state_out)
        return None
