"""Sharing of the pages of prompt prefixes that were computed before.

The keys and values of a position depend only on the tokens up to it, so a request that starts
with tokens an earlier request has processed can use that request's pages instead of computing
them again.  The index knows *full* pages only: an entry says "after the chain of pages that
ends in page P, the page that holds these `page_size` tokens is page B".  A lookup walks a
prompt page by page from the root, so only a true prefix matches; the tokens are compared
themselves, not their hashes.  The index holds one reference to every page it names; requests
that use a page hold their own.  Pages that only the index references can be given back when
memory runs short, least recently used leaf first.

Behaviour as the reference's prefix cache (src/model/prefix_cache.h:1-11,
src/model/prefix_cache.cpp:11-97).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Sequence, Tuple

from .pages import PagePool

ROOT = -1


@dataclass
class _Entry:
    parent: int                 # the page before this one in the chain, ROOT for a prompt's first page
    tokens: Tuple[int, ...]
    tick: int                   # last use
    children: int = 0


class PrefixIndex:
    def __init__(self, pool: PagePool, page_size: int):
        self.pool, self.page_size = pool, int(page_size)
        self._page_of: Dict[Tuple[int, Tuple[int, ...]], int] = {}      # (parent page, tokens) -> page
        self._entry: Dict[int, _Entry] = {}                              # by page
        self._clock = 0

    def __len__(self) -> int:
        return len(self._entry)

    def __contains__(self, page: int) -> bool:
        return page in self._entry

    def _touch(self, page: int) -> None:
        self._clock += 1
        self._entry[page].tick = self._clock

    def match(self, tokens: Sequence[int], limit: int) -> List[int]:
        """The longest known chain of full pages that is a prefix of tokens[:limit].  Every page returned
        is retained once for the caller (who hands them to a request, or releases them)."""
        ps, parent, found = self.page_size, ROOT, []
        for i in range(min(limit, len(tokens)) // ps):
            page = self._page_of.get((parent, tuple(int(t) for t in tokens[i * ps:(i + 1) * ps])))
            if page is None:
                break
            self.pool.retain(page)
            self._touch(page)
            found.append(page)
            parent = page
        return found

    def insert(self, tokens: Sequence[int], n_tokens: int, pages: Sequence[int]) -> int:
        """The first n_tokens positions of a request hold `tokens` in `pages` (its page table): its full
        pages become the known pages of their chain links, unless a link is known already (then the known
        page is followed, whatever the request's own copy).  Returns how many pages were newly named."""
        ps, parent, added = self.page_size, ROOT, 0
        for i in range(min(n_tokens // ps, len(pages))):
            key = (parent, tuple(int(t) for t in tokens[i * ps:(i + 1) * ps]))
            known = self._page_of.get(key)
            if known is not None:
                self._touch(known)
                parent = known
                continue
            page = int(pages[i])
            if page in self._entry:             # a page is never named twice (a consistent caller never gets here)
                break
            self.pool.retain(page)
            self._clock += 1
            self._entry[page] = _Entry(parent, key[1], self._clock)
            self._page_of[key] = page
            if parent != ROOT:
                self._entry[parent].children += 1
            parent = page
            added += 1
        return added

    def _forget(self, page: int) -> None:
        e = self._entry.pop(page)
        del self._page_of[(e.parent, e.tokens)]
        if e.parent != ROOT:
            self._entry[e.parent].children -= 1
        self.pool.release(page)

    def evictable(self) -> int:
        """Pages `evict` could give back right now: those only the index references."""
        return sum(1 for page in self._entry if self.pool.ref_count(page) == 1)

    def evict(self, count: int) -> int:
        """Gives back up to `count` pages nobody else uses, least recently used leaves first; returns how
        many.  A page only the index holds may sit above a leaf a request still uses: then that leaf is
        forgotten (the request keeps its page), which frees nothing yet but uncovers the page above."""
        freed = 0
        while freed < count:
            victim, victim_frees = None, False
            for page, e in self._entry.items():
                if e.children:
                    continue
                frees = self.pool.ref_count(page) == 1
                if not frees:
                    above, a = False, e.parent
                    while a != ROOT and not above:
                        above = self.pool.ref_count(a) == 1
                        a = self._entry[a].parent
                    if not above:
                        continue
                if victim is None or (frees and not victim_frees) or (frees == victim_frees and e.tick < self._entry[victim].tick):
                    victim, victim_frees = page, frees
            if victim is None:
                break
            self._forget(victim)
            freed += 1 if victim_frees else 0
        return freed

    def clear(self) -> None:
        """Forgets everything (pages that requests use stay with them)."""
        for page in list(self._entry):
            self.pool.release(page)
        self._entry.clear()
        self._page_of.clear()
