"""Counter-based random draws keyed on (seed, request id, position) and nothing
else, so a request's samples do not depend on what else is running.

Philox-4x32 with ten rounds (multipliers 0xD2511F53 / 0xCD9E8D57, Weyl
constants 0x9E3779B9 / 0xBB67AE85); counter ``(position low, position high,
index, 0)``; key = the two halves of ``seed XOR k(uid)`` where ``k(uid)`` is
the first eight bytes, big-endian, of sha256(uid); the draw is the first
output word times 2^-32 (reference engine/sampler/philox.py:9-61).
"""

from __future__ import annotations

import functools
import hashlib

_MASK = 0xFFFFFFFF
_ROUNDS = 10


@functools.lru_cache(maxsize=65536)
def uid_key(uid: str) -> int:
    return int.from_bytes(hashlib.sha256(uid.encode("utf-8")).digest()[:8], "big")


def philox_4x32(counter, key) -> tuple[int, int, int, int]:
    c0, c1, c2, c3 = (int(x) & _MASK for x in counter)
    k0, k1 = (int(x) & _MASK for x in key)
    for round_index in range(_ROUNDS):
        prod0 = 0xD2511F53 * c0
        prod1 = 0xCD9E8D57 * c2
        c0, c1, c2, c3 = (
            ((prod1 >> 32) ^ c1 ^ k0) & _MASK,
            prod1 & _MASK,
            ((prod0 >> 32) ^ c3 ^ k1) & _MASK,
            prod0 & _MASK,
        )
        if round_index + 1 < _ROUNDS:
            k0 = (k0 + 0x9E3779B9) & _MASK
            k1 = (k1 + 0xBB67AE85) & _MASK
    return c0, c1, c2, c3


def uniform(seed: int, uid: str, position: int, index: int = 0) -> float:
    """A draw in [0, 1), a pure function of its arguments."""
    mixed = int(seed) ^ uid_key(uid)
    words = philox_4x32((position & _MASK, (position >> 32) & _MASK, index & _MASK, 0),
                        (mixed & _MASK, (mixed >> 32) & _MASK))
    return words[0] * 2.0 ** -32
