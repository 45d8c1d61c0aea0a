"""Counter-based noise for the KeyFormer score path (oracle side, numpy).

Philox4x32 as published by Salmon et al. (Random123): R rounds of
    hi0:lo0 = M0 * c0 ; hi1:lo1 = M1 * c2
    c = (hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0)
with the key bumped by the Weyl constants between rounds.  The kernels use
R = 7 (NOISE_ROUNDS): the fewest rounds at which the authors report the
generator passing BigCrush; R = 10 is Random123's default.

Counter layout used by the kernels (one call yields sixteen bits for each of
eight keys of one query row: two groups of four consecutive keys, eight apart):
    counter = (2 * (key_index // 16) + (key_index // 4) % 2, query_index, head, 0)
    key     = (seed & 0xffffffff, seed >> 32)
    key index k takes output word k % 4, its low half if (k // 8) % 2 == 0, else its high half
The reference takes its noise as an input tensor (convert_eval_rms.py:163);
the seeded form exists because a [heads, S, S] tensor is 1 GiB at S = 4096.
"""
import numpy as np

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_W0 = np.uint32(0x9E3779B9)
_W1 = np.uint32(0xBB67AE85)
_MASK = np.uint64(0xFFFFFFFF)


NOISE_ROUNDS = 7


def philox4x32(c0, c1, c2, c3, k0, k1, rounds=NOISE_ROUNDS):
    """Vectorised Philox4x32 with `rounds` rounds.  All arguments broadcastable uint32 arrays.

    Returns a tuple of four uint32 arrays.
    """
    c0, c1, c2, c3, k0, k1 = np.broadcast_arrays(
        *[np.asarray(a, dtype=np.uint32) for a in (c0, c1, c2, c3, k0, k1)]
    )
    c0, c1, c2, c3, k0, k1 = [a.copy() for a in (c0, c1, c2, c3, k0, k1)]
    with np.errstate(over="ignore"):
        for _ in range(rounds):
            p0 = _M0 * c0.astype(np.uint64)
            p1 = _M1 * c2.astype(np.uint64)
            hi0 = (p0 >> np.uint64(32)).astype(np.uint32)
            lo0 = (p0 & _MASK).astype(np.uint32)
            hi1 = (p1 >> np.uint64(32)).astype(np.uint32)
            lo1 = (p1 & _MASK).astype(np.uint32)
            c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
            k0 = k0 + _W0
            k1 = k1 + _W1
    return c0, c1, c2, c3


def philox4x32_10(c0, c1, c2, c3, k0, k1):
    """Random123's default round count (kept for its known-answer vectors)."""
    return philox4x32(c0, c1, c2, c3, k0, k1, rounds=10)


def uniform_from_bits(x):
    """16 random bits -> float64 in (0, 1): centred in their bin (so that the
    value is exact in fp32 as well)."""
    return (np.asarray(x, dtype=np.uint32).astype(np.float64) + 0.5) * 2.0 ** -16


def noise_bits(seed, n_heads, n_queries, n_keys, heads=None):
    """The sixteen random bits of every (head, query, key) as uint32.

    One generator call serves eight keys - two groups of four consecutive
    keys, eight apart: counter word 0 = 2 * (key // 16) + (key // 4) % 2;
    key k takes output word k % 4, low half if (k // 8) % 2 == 0 else high.
    """
    seed = int(seed)
    k0 = np.uint32(seed & 0xFFFFFFFF)
    k1 = np.uint32((seed >> 32) & 0xFFFFFFFF)
    hs = np.arange(n_heads, dtype=np.uint32) if heads is None else np.asarray(list(heads), dtype=np.uint32)
    ncall = 2 * ((n_keys + 15) // 16)
    cb = np.arange(ncall, dtype=np.uint32)[None, None, :]
    q = np.arange(n_queries, dtype=np.uint32)[None, :, None]
    h = hs[:, None, None]
    words = np.stack(philox4x32(cb, q, h, np.uint32(0), k0, k1), axis=-1)  # [H, Q, call, 4]
    key = np.arange(n_keys)
    call = 2 * (key // 16) + (key // 4) % 2
    w = words[:, :, call, key % 4]
    hi = ((key // 8) % 2).astype(bool)
    return np.where(hi[None, None, :], w >> np.uint32(16), w & np.uint32(0xFFFF)).astype(np.uint32)


def gumbel_noise(seed, n_heads, n_queries, n_keys, heads=None):
    """Standard Gumbel noise g[h, q, k] = -log(-log(u)) as float32.

    `heads` optionally restricts the head axis to the given iterable (memory).
    """
    u = uniform_from_bits(noise_bits(seed, n_heads, n_queries, n_keys, heads))
    return (-np.log(-np.log(u))).astype(np.float32)
