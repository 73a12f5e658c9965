"""The cache manager: pages of keys and values for every request, per group of
layers, and slots of fixed-size state.

Runs of the layer order with the same need (heads, head size, window, page size)
form a group; a group has its own pool of pages, of its own page size and its own
number of pages, its own block table for every request, and one key and one value
tensor for each of its runs, laid out [page][kv head][slot in page][head_dim].  A group with a window gives pages
back as soon as the window has passed them; every group gives all pages back
when the request ends.  Mixers that keep state of fixed size get a slot per
request instead: a row of a tensor [slots, ...], zeroed when claimed.

A step is transactional (/root/reference/src/kipp.c:3616-3635, 4043-4072): `reserve`
claims the pages of every entry of the step or none.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .needs import KVNeed, StateNeed
from .pool import PagePool


class OutOfPages(RuntimeError):
    """A step needs more pages than are free; nothing was changed."""


class OutOfSlots(RuntimeError):
    """Every request slot is taken."""


def _per_group(value, n_groups: int, what: str) -> List[int]:
    """`value` for every group: one integer for all, or a sequence with one entry a group."""
    if isinstance(value, (int, np.integer)):
        return [int(value)] * n_groups
    out = [int(v) for v in value]
    if len(out) != n_groups:
        raise ValueError(f"{what}: {len(out)} values for {n_groups} cache groups")
    return out


@dataclass
class KVCacheView:
    """What a mixer sees of the cache in one run."""
    group: int
    k: object
    v: object
    page_size: int
    writable: bool = True


@dataclass
class RequestCache:
    id: object
    slot: int
    length: int = 0
    tokens: List[int] = field(default_factory=list)
    tables: List[List[int]] = field(default_factory=list)   # per group: page id per block, -1 once given back
    adopted: List[int] = field(default_factory=list)        # per group: leading pages taken from the index
    adopted_tokens: int = 0
    rows: List[np.ndarray] = field(default_factory=list)    # per group: the table as the device sees it (int32, given-back pages 0)
    table_version: int = 0                                  # counts changes of `rows`
    publish_early: bool = False                             # full pages are published as soon as they are committed
    published: int = 0                                      # leading blocks that are adopted or published
    chain: int = 0                                          # chained hash after `published` blocks
    serial: int = 0                                         # unique among all requests the manager ever opened (ids may come again)


class CacheGroup:
    def __init__(self, index: int, need: KVNeed, runs: List[int], num_pages: int, page_size: int, page_order=None):
        self.index = index
        self.need = need
        self.runs = runs
        self.page_size = page_size
        self.pool = PagePool(num_pages, page_size, order=page_order)
        self.k: Dict[int, object] = {}
        self.v: Dict[int, object] = {}

    def bytes_per_token(self, element_size: int) -> int:
        return 2 * len(self.runs) * self.need.num_kv_heads * self.need.head_dim * element_size


class CacheManager:
    def __init__(self, kv_needs: Sequence[Optional[KVNeed]], state_needs: Sequence[Optional[StateNeed]],
                 page_size: int, num_pages, max_requests: int, max_position: int,
                 runtime=None, share_prefixes: bool = True, page_order=None):
        """`kv_needs[r]` / `state_needs[r]`: what run r of the layer order keeps
        (None: nothing).  `page_size`: tokens a page for every group whose need names none of
        its own.  `num_pages`: the pages of a pool, one number for every group (a group whose
        pages have another size gets as many as hold the same tokens) or a sequence with a number
        for each group, in the order in which the groups first appear in the run order.
        With `runtime` None no device memory is made (bookkeeping only).  `page_order`:
        the order in which every group's fresh pool hands out its pages (see `PagePool`)."""
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_position = max_position
        self.rt = runtime
        self.groups: List[CacheGroup] = []
        self.run_group: Dict[int, Tuple[int, int]] = {}
        needs: List[KVNeed] = []
        for need in kv_needs:
            if need is not None and need not in needs:
                needs.append(need)
        sizes = [need.page_size or page_size for need in needs]
        if isinstance(num_pages, (int, np.integer)):
            pages = [-(-int(num_pages) * page_size // size) for size in sizes]
        else:
            pages = _per_group(num_pages, len(needs), "num_pages")
        by_need: Dict[KVNeed, CacheGroup] = {}
        for run, need in enumerate(kv_needs):
            if need is None:
                continue
            group = by_need.get(need)
            if group is None:
                at = len(self.groups)
                order = page_order if page_order is None or len(page_order) == pages[at] else None
                group = CacheGroup(at, need, [], pages[at], sizes[at], order)
                by_need[need] = group
                self.groups.append(group)
            group.runs.append(run)
        self.max_blocks = max([-(-max_position // g.page_size) for g in self.groups] or [1])
        self.state_needs = {r: n for r, n in enumerate(state_needs) if n is not None}
        self.states: Dict[int, object] = {}
        # content sharing needs every token of the prefix to be in pages that are kept, and pages that
        # hold the same tokens in every group (one page size)
        self.share = share_prefixes and not self.state_needs and all(g.need.window is None for g in self.groups) \
            and len({g.page_size for g in self.groups}) <= 1
        if self.groups and len({g.page_size for g in self.groups}) == 1:
            self.page_size = self.groups[0].page_size
        self.free_slots = list(range(max_requests - 1, -1, -1))
        self.requests: Dict[object, RequestCache] = {}
        self._serial = 0
        if runtime is not None:
            self._allocate_device()

    # -- device memory -----------------------------------------------------------
    def _allocate_device(self) -> None:
        import torch
        rt = self.rt
        for g in self.groups:
            # one page more than the pool hands out: `scratch_page`, where rows that only pad a batch write
            shape = (g.pool.num_pages + 1, g.need.num_kv_heads, g.page_size, g.need.head_dim)
            for run in g.runs:
                # zeroed: masked slots must hold finite values
                g.k[run] = torch.zeros(shape, dtype=rt.cache_dtype, device=rt.device)
                g.v[run] = torch.zeros(shape, dtype=rt.cache_dtype, device=rt.device)
        for run, need in self.state_needs.items():
            dtype = {"float32": torch.float32, "bfloat16": torch.bfloat16}[need.dtype]
            # one slot more than requests: `scratch_slot`
            self.states[run] = torch.zeros((self.max_requests + 1,) + tuple(need.shape), dtype=dtype, device=rt.device)

    def scratch_page(self, group: int) -> int:
        """A page of the group's tensors that no request ever gets: rows that only fill a batch up to a
        recorded size keep their key and value there."""
        return self.groups[group].pool.num_pages

    @property
    def scratch_slot(self) -> int:
        """The state slot of such rows."""
        return self.max_requests

    def view(self, run: int, reads_run: Optional[int] = None) -> Optional[KVCacheView]:
        """The cache of `run`, or of `reads_run` read-only."""
        src = run if reads_run is None else reads_run
        for g in self.groups:
            if src in g.runs:
                return KVCacheView(g.index, g.k.get(src), g.v.get(src), g.page_size, writable=reads_run is None)
        return None

    def state(self, run: int):
        return self.states.get(run)

    # -- requests ------------------------------------------------------------------
    def open(self, request_id, prompt: Optional[Sequence[int]] = None, publish_early: bool = False) -> RequestCache:
        """Claim a slot (its state zeroed) and, where sharing is on and `prompt`
        is given, adopt the pages of its longest known beginning.

        The reference publishes a session's pages when it ends, which keeps
        truncation sound (/root/reference/src/kipp.c:3647-3670).  A request that
        will never be truncated may set `publish_early`: its pages are published
        as soon as they are full, so that requests running beside it can adopt
        them; it can then no longer be cut below them."""
        if request_id in self.requests:
            raise ValueError(f"request {request_id!r} is already open")
        if not self.free_slots:
            raise OutOfSlots(f"all {self.max_requests} request slots are taken")
        slot = self.free_slots.pop()
        for tensor in self.states.values():
            row = tensor[slot]
            if self.rt is not None and (row.numel() * row.element_size()) % 4 == 0:
                self.rt.ops.fill_zero(row)
            else:
                row.zero_()
        self._serial += 1
        req = RequestCache(request_id, slot, tables=[[] for _ in self.groups], adopted=[0 for _ in self.groups],
                           rows=[np.zeros(-(-self.max_position // g.page_size), dtype=np.int32) for g in self.groups],
                           serial=self._serial)
        if self.share and prompt is not None and self.groups:
            matches = [g.pool.prefix_match(prompt) for g in self.groups]
            keep = min(len(pages) for pages, _ in matches)
            for g, (pages, _) in zip(self.groups, matches):
                for page in pages[keep:]:
                    g.pool.release(page)
                req.tables[g.index] = list(pages[:keep])
                req.rows[g.index][:keep] = pages[:keep]
                req.table_version += 1
                req.adopted[g.index] = keep
            req.adopted_tokens = keep * self.page_size
            req.length = req.adopted_tokens
            req.tokens = [int(t) for t in prompt[:req.length]]
            req.published, req.chain = keep, matches[0][1] if keep == len(matches[0][0]) else self._chain(req.tokens)
        req.publish_early = publish_early and self.share
        self.requests[request_id] = req
        return req

    def _chain(self, tokens: Sequence[int]) -> int:
        parent = 0
        for block in range(len(tokens) // self.page_size):
            parent = self.groups[0].pool._hash(parent, tokens[block * self.page_size:(block + 1) * self.page_size])
        return parent

    def pages_needed(self, req: RequestCache, new_length: int) -> List[int]:
        """Pages each group still has to claim so that positions < new_length have one."""
        return [max(0, -(-new_length // g.page_size) - len(req.tables[g.index])) for g in self.groups]

    def pages_bound(self, req: Optional[RequestCache], budget_tokens: int, step_tokens: int) -> List[int]:
        """The most pages each group may still have to hand the request beyond those it holds now, if it grows to
        `budget_tokens` in steps of at most `step_tokens` (`req` None: a request that holds nothing yet).  A group
        that keeps every key: the blocks it has not claimed.  A group with a window gives pages back as the
        window passes them, so the request never holds more than the pages of window - 1 + step_tokens tokens
        and one more for where they begin: what a scheduler has to keep free for it is the distance to that."""
        out = []
        for g in self.groups:
            table = req.tables[g.index] if req is not None else []
            need = max(0, -(-budget_tokens // g.page_size) - len(table))
            if g.need.window is not None:
                most = -(-(g.need.window - 1 + step_tokens) // g.page_size) + 1
                held = sum(1 for page in table if page >= 0)
                need = min(need, max(0, most - held))
            out.append(need)
        return out

    def free_pages(self) -> List[int]:
        return [g.pool.free_count for g in self.groups]

    def reserve(self, entries: Sequence[Tuple[RequestCache, int]]) -> None:
        """Claim the pages that every (request, number of new tokens) of a step
        needs, in every group; all or nothing."""
        claimed: List[Tuple[RequestCache, int, int]] = []
        for req, n_new in entries:
            new_length = req.length + n_new
            if n_new > 0 and new_length <= self.max_position:
                if all(len(req.tables[g.index]) * g.page_size >= new_length for g in self.groups):
                    continue                                  # every position already has its page
            if n_new <= 0:
                self._rollback(claimed)
                raise ValueError("a step entry needs at least one token")
            if new_length > self.max_position:
                self._rollback(claimed)
                raise ValueError(f"request {req.id!r}: {new_length} tokens exceed the model's {self.max_position} positions")
            for g, need in zip(self.groups, self.pages_needed(req, new_length)):
                for _ in range(need):
                    page = g.pool.alloc()
                    if page is None:
                        self._rollback(claimed)
                        raise OutOfPages(f"group {g.index}: no free page for request {req.id!r}")
                    req.rows[g.index][len(req.tables[g.index])] = page
                    req.table_version += 1
                    req.tables[g.index].append(page)
                    claimed.append((req, g.index, page))

    def _rollback(self, claimed) -> None:
        for req, gi, page in reversed(claimed):
            popped = req.tables[gi].pop()
            assert popped == page
            req.rows[gi][len(req.tables[gi])] = 0
            req.table_version += 1
            self.groups[gi].pool.release(page)

    def trim(self, req: RequestCache) -> None:
        """Give back pages that were claimed for a step that did not happen."""
        for g in self.groups:
            blocks = -(-req.length // g.page_size)
            table = req.tables[g.index]
            while len(table) > blocks:
                page = table.pop()
                req.rows[g.index][len(table)] = 0
                req.table_version += 1
                if page >= 0:
                    g.pool.release(page)

    def truncate(self, req: RequestCache, length: int) -> None:
        """Keep only the first `length` tokens of the request; pages above them go
        back (/root/reference/src/kipp.c:3739-3774).  Pages adopted from the index are
        shared and complete, so a request is never cut below them; a windowed group
        or a state slot cannot be rolled back."""
        if not 0 <= length <= req.length:
            raise ValueError(f"cannot truncate {req.length} tokens to {length}")
        if self.state_needs or any(g.need.window is not None for g in self.groups):
            raise NotImplementedError("truncation needs every group to keep all keys and no per-request state")
        floor = max(req.adopted_tokens, req.published * self.page_size)
        if length < floor:
            raise ValueError(f"cannot truncate below the {floor} adopted or published tokens")
        req.length = length
        del req.tokens[length:]
        self.trim(req)

    def commit(self, req: RequestCache, tokens: Sequence[int]) -> None:
        """The step ran: the request now holds `tokens` more.  Pages that a
        window has passed are given back."""
        req.tokens.extend(int(t) for t in tokens)
        req.length += len(tokens)
        if req.publish_early:
            while (req.published + 1) * self.page_size <= req.length:
                block = req.published
                chunk = req.tokens[block * self.page_size:(block + 1) * self.page_size]
                for g in self.groups:
                    h = g.pool.seal(req.tables[g.index][block], req.chain, chunk)
                req.chain, req.published = h, block + 1
        for g in self.groups:
            window = g.need.window
            if window is None:
                continue
            first_needed = max(0, req.length - window + 1)
            table = req.tables[g.index]
            for block in range(min(first_needed // g.page_size, len(table))):
                if table[block] >= 0:
                    g.pool.release(table[block])
                    table[block] = -1
                    req.rows[g.index][block] = 0
                    req.table_version += 1

    def close(self, request_id) -> None:
        """The request ended: publish its full pages where sharing is on, give
        every page and the slot back."""
        req = self.requests.pop(request_id)
        for g in self.groups:
            table = req.tables[g.index]
            if self.share:
                parent = 0
                for block in range(req.length // self.page_size):
                    chunk = req.tokens[block * self.page_size:(block + 1) * self.page_size]
                    if block < req.adopted[g.index] or g.pool.content[table[block]] is not None:
                        parent = g.pool._hash(parent, chunk)
                    else:
                        parent = g.pool.seal(table[block], parent, chunk)
            for page in table:
                if page >= 0:
                    g.pool.release(page)
            table.clear()
        self.free_slots.append(req.slot)

    def check(self) -> None:
        """Invariants over pools and tables: a held page is held exactly as often
        as tables name it; nothing is lost."""
        for g in self.groups:
            g.pool.check()
            counts = [0] * g.pool.num_pages
            for req in self.requests.values():
                for page in req.tables[g.index]:
                    if page >= 0:
                        counts[page] += 1
            for page in range(g.pool.num_pages):
                if counts[page] != g.pool.ref[page]:
                    raise AssertionError(f"group {g.index} page {page}: named {counts[page]} times, held {g.pool.ref[page]} times")
        slots = [r.slot for r in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self.free_slots):
            raise AssertionError("a slot is held twice or both held and free")
        if len(slots) + len(self.free_slots) != self.max_requests:
            raise AssertionError("a slot was lost")
