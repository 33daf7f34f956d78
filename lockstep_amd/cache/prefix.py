"""Index from a prompt's leading whole pages to the physical pages that hold
their keys and values, so a later request with the same prefix skips them.

Keys form a hash chain over whole pages of tokens: ``key_i = sha256(key_{i-1},
tokens of page i)``, so a match is a match of the whole prefix (reference
engine/cache/prefix.py:11-17,38-47).  Each entry pins its page in the cache
manager; an entry whose page has no other holder can be evicted under
pressure (reference engine/cache/prefix.py:83-103).  Entries are added when a
request finishes (reference engine/sched/scheduler.py:343-348).
"""

from __future__ import annotations

import hashlib
from dataclasses import dataclass

_ROOT = b"lockstep-prefix-root"


def page_key(parent: bytes, tokens) -> bytes:
    digest = hashlib.sha256()
    digest.update(parent)
    digest.update(b"|")
    digest.update(",".join(str(int(t)) for t in tokens).encode("ascii"))
    return digest.digest()


@dataclass
class PrefixEntry:
    page: int
    tokens: tuple
    hits: int = 0


class PrefixIndex:
    def __init__(self, page_size: int):
        self.page_size = page_size
        self.entries: dict[bytes, PrefixEntry] = {}
        self.stats = {"lookups": 0, "hit_pages": 0, "inserts": 0, "evictions": 0}

    def _chain(self, tokens):
        parent = _ROOT
        for i in range(len(tokens) // self.page_size):
            chunk = tuple(int(t) for t in tokens[i * self.page_size:(i + 1) * self.page_size])
            parent = page_key(parent, chunk)
            yield parent, chunk

    def lookup(self, tokens) -> tuple[int, list[int]]:
        """Longest indexed whole-page prefix: (token count, pages)."""
        self.stats["lookups"] += 1
        pages: list[int] = []
        for key, chunk in self._chain(tokens):
            entry = self.entries.get(key)
            if entry is None or entry.tokens != chunk:
                break
            entry.hits += 1
            pages.append(entry.page)
        self.stats["hit_pages"] += len(pages)
        return len(pages) * self.page_size, pages

    def insert(self, tokens, pages, cache) -> int:
        """Index every whole page of ``tokens`` held in ``pages``; pins each new one."""
        created = 0
        for i, (key, chunk) in enumerate(self._chain(tokens)):
            if i >= len(pages) or pages[i] < 0:
                break
            if key in self.entries:
                continue
            self.entries[key] = PrefixEntry(page=pages[i], tokens=chunk)
            cache.pin(pages[i])
            created += 1
        self.stats["inserts"] += created
        return created

    def evictable(self, cache) -> list[int]:
        """Pages whose only holder is this index."""
        holders = cache.groups[0].pool.holders
        return sorted(e.page for e in self.entries.values() if holders[e.page] == 1)

    def evict(self, page: int, cache) -> bool:
        for key, entry in list(self.entries.items()):
            if entry.page == page:
                del self.entries[key]
                cache.unpin(page)
                self.stats["evictions"] += 1
                return True
        return False

    def state_digest(self) -> tuple:
        return tuple(sorted((k.hex()[:16], e.page, e.tokens) for k, e in self.entries.items()))
