"""Prefix index: finished requests leave the whole pages of their context
behind, and a later request whose prompt starts with the same tokens maps
those pages instead of computing them again.

The index is a tree over whole pages of tokens.  A node stands for one page:
its edge from the parent is the page's token tuple, so walking a prompt page
by page from the root finds exactly the prefixes that are held, and a match
is a match of every token before it.  Each node pins its physical page in the
cache manager (one extra holder); ``by_page`` finds a node from its page, so
dropping one costs no search.  Only *leaves* that nobody but the index holds
may be dropped: a page in the middle of a chain is what makes its
descendants reachable, and a request that maps a descendant maps the whole
chain, so holders can only thin out towards the leaves and a droppable leaf
exists whenever an index-only page does.

What the reference's index does (engine/cache/prefix.py:38-103: whole pages
only, entries added when a request finishes, entries whose page has no other
holder given up under pressure) is kept; the flat table of chained hashes it
uses is replaced by the tree, and the chained digest survives only as each
node's name in ``digest()``.
"""

from __future__ import annotations

import hashlib
import struct


class _Node:
    __slots__ = ("tokens", "page", "parent", "children", "name", "matched")

    def __init__(self, tokens: tuple, page: int, parent: "_Node | None"):
        self.tokens = tokens
        self.page = page
        self.parent = parent
        self.children: dict[tuple, _Node] = {}
        self.matched = 0
        seed = parent.name if parent is not None else b"prefix-tree"
        self.name = hashlib.sha256(seed + struct.pack(f"<{len(tokens)}q", *tokens)).digest()


class PrefixIndex:
    def __init__(self, page_size: int):
        self.page_size = page_size
        self.root = _Node((), -1, None)
        self.by_page: dict[int, _Node] = {}
        self.asked = 0            # match() calls
        self.pages_matched = 0
        self.pages_indexed = 0
        self.pages_dropped = 0

    def __len__(self) -> int:
        return len(self.by_page)

    def _pages_of(self, tokens):
        size = self.page_size
        for first in range(0, len(tokens) - size + 1, size):
            yield tuple(int(t) for t in tokens[first:first + size])

    def match(self, tokens) -> list[int]:
        """Physical pages of the longest indexed prefix of ``tokens`` (whole pages, in order)."""
        self.asked += 1
        node, pages = self.root, []
        for page_tokens in self._pages_of(tokens):
            node = node.children.get(page_tokens)
            if node is None:
                break
            node.matched += 1
            pages.append(node.page)
        self.pages_matched += len(pages)
        return pages

    def remember(self, tokens, pages, cache) -> int:
        """Index the whole pages of ``tokens``, which ``pages`` (a request's physical pages, in
        logical order) hold; pages already indexed are walked over.  Returns how many were new;
        each of those is pinned in ``cache``."""
        node, added = self.root, 0
        for logical, page_tokens in enumerate(self._pages_of(tokens)):
            if logical >= len(pages) or pages[logical] < 0:
                break
            child = node.children.get(page_tokens)
            if child is None:
                page = int(pages[logical])
                if page in self.by_page:
                    break        # the page already stands for other tokens: leave the chain here
                child = _Node(page_tokens, page, node)
                node.children[page_tokens] = child
                self.by_page[page] = child
                cache.pin(page)
                added += 1
            node = child
        self.pages_indexed += added
        return added

    def reclaimable(self, cache) -> int:
        """Pages that nobody but the index holds (all of them can be had, leaf by leaf)."""
        holders = cache.groups[0].pool.holders
        return sum(1 for page in self.by_page if holders[page] == 1)

    def droppable(self, cache) -> list[int]:
        """Pages of leaves that nobody but the index holds, ascending."""
        holders = cache.groups[0].pool.holders
        return sorted(page for page, node in self.by_page.items() if not node.children and holders[page] == 1)

    def drop(self, page: int, cache) -> bool:
        """Forget the leaf that stands for ``page`` and unpin the page."""
        node = self.by_page.get(page)
        if node is None or node.children:
            return False
        del node.parent.children[node.tokens]
        del self.by_page[page]
        cache.unpin(page)
        self.pages_dropped += 1
        return True

    def digest(self) -> tuple:
        """The held prefixes as a comparable value."""
        return tuple(sorted((node.name.hex()[:16], page) for page, node in self.by_page.items()))
