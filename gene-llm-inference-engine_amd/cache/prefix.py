"""Sharing of the pages of prompt beginnings that were computed before.

The keys and values of a position depend only on the tokens up to it, so a request that begins
with tokens an earlier request has processed can read that request's pages instead of computing
them again.  This index is a tree of *full* pages: the children of a node are the pages that
followed it in some request, found by the `page_size` tokens they hold (the tokens themselves, not
a hash of them); the children of the root are first pages.  A lookup walks a prompt down from the
root, so only a true beginning matches.

The index holds one reference to every page it names, requests hold their own.  It learns of every
change of a named page's reference count through the pool's `on_change` hook, and so knows at all
times how many pages nobody but itself holds (`evictable()`, constant time) and which of them are
leaves: those wait in a heap ordered by last use, and `evict(k)` pops them, least recently used
first, in O(k log n).  Heap entries are not removed when a page is used again or gains a child;
they are recognised as stale when popped (the node's stamp has moved on).

What it does is what the reference's prefix cache does (src/model/prefix_cache.h:1-11): full pages
only, one reference per named page, `match` retains for the caller, leaves nobody uses go first.

A model whose layers keep their keys in several groups of pages (other head counts or sizes, each
group with a pool of its own) has one page per group for the same positions.  The index then names
the first group's page and keeps the other groups' pages beside it (`companions`): whoever holds one
of them holds all (requests take and give back their pages of all groups together), so the first
pool's reference counts speak for the others, and what is retained, released or given back is the
whole set.
"""
from __future__ import annotations

import heapq
from typing import Dict, List, Optional, Sequence, Tuple

from .pages import PagePool


class _Node:
    __slots__ = ("page", "tokens", "parent", "children", "stamp", "only_mine", "companions")

    def __init__(self, page: int, tokens: Tuple[int, ...], parent: Optional["_Node"], stamp: int, companions: Tuple[int, ...] = ()):
        self.page, self.tokens, self.parent, self.companions = page, tokens, parent, companions
        self.children: Dict[Tuple[int, ...], "_Node"] = {}
        self.stamp = stamp                  # time of last use; also tells a fresh heap entry from a stale one
        self.only_mine = False              # the index's reference is the page's only one


class PrefixIndex:
    def __init__(self, pool: PagePool, page_size: int, other_pools: Sequence[PagePool] = ()):
        self.pool, self.page_size, self.other_pools = pool, int(page_size), tuple(other_pools)
        self._first: Dict[Tuple[int, ...], _Node] = {}       # the root's children
        self._by_page: Dict[int, _Node] = {}
        self._only_mine = 0                                   # named pages whose reference count is 1
        self._idle_leaves: List[Tuple[int, int]] = []         # heap of (stamp, page): leaves nobody else holds, and stale entries
        self._clock = 0
        self.last_walk = None                # where the last insert ended: (node of the last full page it passed, how many it passed)
        pool.on_change = self._references_changed

    def __len__(self) -> int:
        return len(self._by_page)

    def __contains__(self, page: int) -> bool:
        return page in self._by_page

    def pages(self):
        """The pages the index names (and holds a reference to)."""
        return self._by_page.keys()

    # ------------------------------------------------------------------------- bookkeeping
    def _references_changed(self, page: int, count: int) -> None:
        node = self._by_page.get(page)
        if node is None:
            return
        alone = count == 1
        if alone != node.only_mine:
            node.only_mine = alone
            self._only_mine += 1 if alone else -1
            if alone:
                self._offer(node)

    def _offer(self, node: _Node) -> None:
        if node.only_mine and not node.children:
            heapq.heappush(self._idle_leaves, (node.stamp, node.page))

    def _touch(self, node: _Node) -> None:
        self._clock += 1
        node.stamp = self._clock
        self._offer(node)                   # its older entry is stale now

    def _children_of(self, node: Optional[_Node]) -> Dict[Tuple[int, ...], _Node]:
        return self._first if node is None else node.children

    # ----------------------------------------------------------------------------- lookups
    def match(self, tokens: Sequence[int], limit: int) -> List[int]:
        """The longest known chain of full pages that is a beginning of tokens[:limit].  Every page returned
        is retained once for the caller (who hands them to a request, or releases them)."""
        ps, node, found = self.page_size, None, []
        for i in range(min(limit, len(tokens)) // ps):
            nxt = self._children_of(node).get(tuple(tokens[i * ps:(i + 1) * ps]))
            if nxt is None:
                break
            self.pool.retain(nxt.page)
            for pool, page in zip(self.other_pools, nxt.companions):
                pool.retain(page)
            self._touch(nxt)
            found.append(nxt.page)
            node = nxt
        return found

    def companions(self, page: int) -> Tuple[int, ...]:
        """The other groups' pages for the positions of a named page of the first group, in the order of `other_pools`."""
        return self._by_page[page].companions

    def insert(self, tokens: Sequence[int], n_tokens: int, pages: Sequence[int], after=None, companions: Sequence[Sequence[int]] = ()) -> int:
        """The first n_tokens positions of a request hold `tokens` in `pages` (its page table): its full pages
        are named, each under the page before it, unless that place is taken already (then the page that has
        it is followed, whatever the request's own copy).  Returns how many pages were newly named.

        `after`: what `last_walk` was after an earlier insert of the same request (its tokens up to there unchanged):
        the walk then starts behind the pages that one passed, unless the index has forgotten the last of them
        meanwhile (then it starts at the root as without it).  `companions`: the request's page tables in the other
        groups, one per pool of `other_pools`."""
        if len(companions) != len(self.other_pools):
            raise ValueError(f"the index names pages of {1 + len(self.other_pools)} groups, {1 + len(companions)} page tables were given")
        ps, node, added, first = self.page_size, None, 0, 0
        if after is not None and self._by_page.get(after[0].page) is after[0]:
            node, first = after
        self.last_walk = None
        for i in range(first, min(n_tokens // ps, len(pages))):
            key = tuple(tokens[i * ps:(i + 1) * ps])
            known = self._children_of(node).get(key)
            if known is not None:
                self._touch(known)
                node = known
                self.last_walk = (node, i + 1)
                continue
            page = int(pages[i])
            if page in self._by_page:       # a page has one place in the tree
                break
            self._clock += 1
            new = _Node(page, key, node, self._clock, tuple(int(table[i]) for table in companions))
            self._by_page[page] = new
            self._children_of(node)[key] = new
            self.pool.retain(page)          # (the hook sees a named page with at least two holders: nothing to count)
            for pool, other in zip(self.other_pools, new.companions):
                pool.retain(other)
            node = new
            added += 1
            self.last_walk = (new, i + 1)
        return added

    # ---------------------------------------------------------------------------- giving back
    def evictable(self) -> int:
        """Pages nobody but the index holds: what `evict` can give back."""
        return self._only_mine

    def _forget(self, node: _Node) -> None:
        del self._by_page[node.page]
        del self._children_of(node.parent)[node.tokens]
        if node.only_mine:
            self._only_mine -= 1
        self.pool.release(node.page)
        for pool, other in zip(self.other_pools, node.companions):
            pool.release(other)
        if node.parent is not None:
            self._offer(node.parent)        # it may have become a leaf nobody uses

    def _next_idle_leaf(self) -> Optional[_Node]:
        while self._idle_leaves:
            stamp, page = heapq.heappop(self._idle_leaves)
            node = self._by_page.get(page)
            if node is not None and node.stamp == stamp and node.only_mine and not node.children:
                return node
        return None

    def _uncover(self) -> bool:
        """No leaf can be given back, yet some page further up is held by the index alone (a request computed its
        own copy of that page and went on from the index's).  Below the least recently used such page, the leaves
        that requests still use are forgotten (the requests keep their pages; nothing is freed), and again until what
        is left below it are pages of the index alone, whose leaves `evict` can then give back."""
        buried = [n for n in self._by_page.values() if n.only_mine]
        if not buried:
            return False
        top = min(buried, key=lambda n: n.stamp)
        order, stack = [], list(top.children.values())
        while stack:                        # the pages below `top`, every page before the pages under it
            n = stack.pop()
            order.append(n)
            stack.extend(n.children.values())
        for n in reversed(order):           # ... and now every page after the pages under it
            if not n.children and not n.only_mine:
                self._forget(n)
        return True

    def evict(self, count: int) -> int:
        """Gives back up to `count` pages that nobody else holds, least recently used leaves first; returns how
        many were given back."""
        freed = 0
        while freed < count:
            node = self._next_idle_leaf()
            if node is None:
                if self._only_mine == 0 or not self._uncover():
                    break
                continue
            self._forget(node)
            freed += 1
        return freed

    def clear(self) -> None:
        """Forgets everything (pages that requests use stay with them)."""
        nodes = list(self._by_page.values())
        self._by_page.clear()
        self._first.clear()
        self._idle_leaves.clear()
        self._only_mine = 0
        for node in nodes:
            self.pool.release(node.page)
            for pool, other in zip(self.other_pools, node.companions):
                pool.release(other)
