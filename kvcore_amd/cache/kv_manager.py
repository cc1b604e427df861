"""Which pages and which slot each request holds.

Reference: kvcore/kv/kv_manager.py:90-283 and kvcore/kv/single_type_kv_manager.py:
82-183.  There every layer is a group with its own page list per request
(kv_manager.py:105-113); here a group is a set of cache planes with the same need
(all keys, or a window of them), a page id addresses ``page_size`` tokens in every
plane of its group, and each group has a pool and a page list per request of its own.
A window group gives pages back as soon as the window has passed them and leaves the
null page in their place (the reference only stubs this:
single_type_kv_manager.py:345-375).  Beside the pages, the manager owns the request
slots.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .page_pool import PagePool, SlotPool


@dataclass(frozen=True)
class GroupConfig:
    """``window`` 0: every token is kept.  ``num_pages`` counts the null page."""

    page_size: int
    num_pages: int
    window: int = 0


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def plan_groups(needs, block_size: int, num_blocks: int) -> list[GroupConfig]:
    """One ``GroupConfig`` per cache need (objects with ``page_size`` and ``window``, as
    ``parts.base.CacheNeed``).  A group whose need names no page size has pages of
    ``block_size`` tokens and ``num_blocks`` of them; a group with a page size of its own gets
    as many pages as hold the same number of tokens.  Every count includes the null page."""
    if num_blocks < 2:
        raise ValueError(f"a cache needs the null page and at least one more, got {num_blocks}")
    tokens = (num_blocks - 1) * block_size
    out = []
    for need in needs:
        size = need.page_size or block_size
        pages = num_blocks if size == block_size else cdiv(tokens, size) + 1
        out.append(GroupConfig(size, pages, need.window))
    return out


@dataclass
class _RequestPages:
    pages: list[int] = field(default_factory=list)  # entry i covers tokens [i*ps, (i+1)*ps)
    released: int = 0  # leading entries already given back (they read 0)


class KVManager:
    def __init__(self, groups: list[GroupConfig], *, max_num_seqs: int, max_model_len: int,
                 shuffle_seed: int | None = None, track_freed: bool = False) -> None:
        if max_model_len <= 0:
            raise ValueError("max_model_len must be positive")
        self.groups = list(groups)
        self.pools = [PagePool(g.num_pages, None if shuffle_seed is None else shuffle_seed + i)
                      for i, g in enumerate(self.groups)]
        self.slots = SlotPool(max_num_seqs)
        self.max_model_len = max_model_len
        self._req_pages: dict[str, list[_RequestPages]] = {}
        self._req_slot: dict[str, int] = {}
        # pages given back since the last ``drain_freed`` (a debugging aid: the runner may fill
        # them with NaN; the reference keeps the like for new blocks, kv_manager.py:441-447)
        self.track_freed = track_freed
        self._freed: list[list[int]] = [[] for _ in self.groups]

    # ---------------------------------------------------------------------- admission
    def has_free_slot(self) -> bool:
        return self.slots.num_free > 0

    def admit(self, request_id: str) -> int:
        """Take a slot for a new request.  Raises if the id is live or no slot is free."""
        if request_id in self._req_slot:
            raise ValueError(f"request {request_id!r} is already admitted")
        slot = self.slots.take()
        self._req_slot[request_id] = slot
        self._req_pages[request_id] = [_RequestPages() for _ in self.groups]
        return slot

    def is_admitted(self, request_id: str) -> bool:
        return request_id in self._req_slot

    def slot_of(self, request_id: str) -> int:
        return self._req_slot[request_id]

    # -------------------------------------------------------------------------- pages
    def _missing(self, request_id: str, total_tokens: int) -> list[int]:
        total = min(total_tokens, self.max_model_len)
        return [
            max(cdiv(total, g.page_size) - len(rp.pages), 0)
            for g, rp in zip(self.groups, self._req_pages[request_id])
        ]

    def pages_missing(self, request_id: str, total_tokens: int) -> list[int]:
        """Per group, the pages that holding ``total_tokens`` tokens still needs
        (kv_manager.py:455-478; single_type_kv_manager.py:104-116)."""
        if request_id not in self._req_pages:
            return [cdiv(min(total_tokens, self.max_model_len), g.page_size) for g in self.groups]
        return self._missing(request_id, total_tokens)

    def can_fit(self, request_id: str, total_tokens: int) -> bool:
        """True iff every group's pool holds the pages that are missing
        (kv_manager.py:179-201)."""
        need = self.pages_missing(request_id, total_tokens)
        return all(n <= pool.num_free for n, pool in zip(need, self.pools))

    def allocate(self, request_id: str, num_computed: int, num_new: int) -> list[list[int]] | None:
        """Pages so that ``num_computed + num_new`` tokens have a place.  Returns the new
        page ids per group, or None (and takes nothing) if any pool is too small
        (kv_manager.py:203-246)."""
        if num_new <= 0:
            raise ValueError(f"num_new must be positive, got {num_new}")
        total = num_computed + num_new
        need = self._missing(request_id, total)
        if any(n > pool.num_free for n, pool in zip(need, self.pools)):
            return None
        new_pages = []
        for n, pool, rp in zip(need, self.pools, self._req_pages[request_id]):
            got = pool.take(n)
            rp.pages.extend(got)
            new_pages.append(got)
        return new_pages

    def release_behind_window(self, request_id: str, num_computed: int) -> list[int]:
        """After ``num_computed`` tokens are in the cache, a window group needs keys from
        ``num_computed - window + 1`` on; pages wholly before that are given back and
        read as the null page.  Returns per group how many leading entries are now null."""
        out = []
        for gi, (g, pool, rp) in enumerate(zip(self.groups, self.pools, self._req_pages[request_id])):
            if g.window > 0:
                first_needed = max(num_computed - g.window + 1, 0)
                upto = min(first_needed // g.page_size, len(rp.pages))
                if upto > rp.released:
                    pool.give_back(rp.pages[rp.released:upto])
                    if self.track_freed:
                        self._freed[gi].extend(rp.pages[rp.released:upto])
                    for i in range(rp.released, upto):
                        rp.pages[i] = 0
                    rp.released = upto
            out.append(rp.released)
        return out

    def page_ids(self, request_id: str) -> list[list[int]]:
        """Per group, the request's page list (kv_manager.py:277-283); do not modify."""
        return [rp.pages for rp in self._req_pages[request_id]]

    def released_counts(self, request_id: str) -> list[int]:
        return [rp.released for rp in self._req_pages[request_id]]

    def free(self, request_id: str) -> None:
        """Give back everything the request holds: pages in reverse order, so that tail
        pages are reused first (single_type_kv_manager.py:177-182), then the slot."""
        pages = self._req_pages.pop(request_id)
        slot = self._req_slot.pop(request_id)
        for gi, (pool, rp) in enumerate(zip(self.pools, pages)):
            pool.give_back(reversed(rp.pages))
            if self.track_freed:
                self._freed[gi].extend(p for p in rp.pages if p)
        self.slots.give_back(slot)

    def drain_freed(self) -> list[list[int]]:
        """Per group, the pages given back since the last call (empty without ``track_freed``)."""
        out, self._freed = self._freed, [[] for _ in self.groups]
        return out

    # --------------------------------------------------------------------- inspection
    def num_free_pages(self) -> list[int]:
        return [pool.num_free for pool in self.pools]

    def live_requests(self) -> list[str]:
        return list(self._req_slot)

    def check(self) -> None:
        """No page lost, held twice or free while held; all held pages are in lists."""
        for gi, pool in enumerate(self.pools):
            pool.check()
            listed: list[int] = []
            for pages in self._req_pages.values():
                listed.extend(p for p in pages[gi].pages if p != 0)
            if len(set(listed)) != len(listed):
                raise AssertionError(f"group {gi}: a page is in two lists")
            if sorted(listed) != pool.held_pages():
                raise AssertionError(f"group {gi}: held pages and page lists disagree")
        if self.slots.num_free + len(self._req_slot) != self.slots.num_slots:
            raise AssertionError("a slot is lost")
        if len(set(self._req_slot.values())) != len(self._req_slot):
            raise AssertionError("a slot is held twice")
