"""A counter-based random stream per request: Philox4x32-10 keyed by the request's seed,
counted by the index of the token being drawn.  The number for token ``i`` of a request
is a pure function of (seed, i): it does not depend on the batch the request runs in,
on how its prompt was cut, or on what other requests draw."""
from __future__ import annotations

_M0, _M1 = 0xD2511F53, 0xCD9E8D57
_W0, _W1 = 0x9E3779B9, 0xBB67AE85
_MASK = 0xFFFFFFFF


def philox4x32(counter, key, rounds: int = 10):
    c0, c1, c2, c3 = counter
    k0, k1 = key
    for _ in range(rounds):
        p0 = _M0 * c0
        p1 = _M1 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0) & _MASK, p1 & _MASK, ((p0 >> 32) ^ c3 ^ k1) & _MASK, p0 & _MASK
        k0 = (k0 + _W0) & _MASK
        k1 = (k1 + _W1) & _MASK
    return c0, c1, c2, c3


def uniform(seed: int, index: int) -> float:
    """A number in [0, 1) with 24 random bits, for draw ``index`` of stream ``seed``."""
    word = philox4x32((index & _MASK, (index >> 32) & _MASK, 0, 0), (seed & _MASK, (seed >> 32) & _MASK))[0]
    return (word >> 8) * (1.0 / (1 << 24))
