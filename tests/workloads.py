"""Seeded synthetic inputs shared by the parity tests and the benchmark.

All streams come from splitmix64; keys that fall in the reserved range
((k & ~3) == ~3 at the default start bit) are remapped, and batches are unique
by construction or by an explicit de-duplication.
"""
import numpy as np

MASK64 = (1 << 64) - 1


def splitmix64(state):
    """Vectorised splitmix64 output function on a uint64 array of states."""
    with np.errstate(over="ignore"):
        z = state + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def stream(seed, start, n):
    """n outputs of the splitmix64 stream `seed`, positions start..start+n-1."""
    with np.errstate(over="ignore"):
        idx = np.arange(start, start + n, dtype=np.uint64)
        return splitmix64(np.uint64(seed) + idx * np.uint64(0x9E3779B97F4A7C15))


def unique_keys(seed, start, n):
    """n distinct non-reserved uint64 keys: a bijective mix of the counter
    start..start+n-1 (distinct counters give distinct keys across calls with
    the same seed), with the four reserved patterns moved out of the way."""
    with np.errstate(over="ignore"):
        ctr = np.arange(start, start + n, dtype=np.uint64) + np.uint64(seed) * np.uint64(0x100000001B3)
        k = splitmix64(ctr)  # splitmix64's finaliser is a bijection on uint64
    reserved = (k & np.uint64(0xFFFFFFFFFFFFFFFC)) == np.uint64(0xFFFFFFFFFFFFFFFC)
    # clear bit 63 of a reserved output: lands outside the reserved range; the
    # (astronomically unlikely) collision with another key is tolerated by callers
    k[reserved] &= np.uint64(0x7FFFFFFFFFFFFFFF)
    return k


def values_from_keys(keys, dim, dtype=np.float32):
    """C1's key-derived values: value[i][d] = float(key % 1000) + d."""
    base = (keys % np.uint64(1000)).astype(dtype)
    return (base[:, None] + np.arange(dim, dtype=dtype)[None, :]).astype(dtype)


def uniform_values(seed, start, n, dim):
    """fp32 in [-1, 1) from the stream."""
    r = stream(seed ^ 0xA5A5A5A5, start * dim, n * dim)
    return ((r >> np.uint64(40)).astype(np.float32) / np.float32(1 << 23) - np.float32(1.0)).reshape(n, dim)


def zipf_unique_keys(seed, start, n, universe_bits=31, alpha=1.05):
    """About n unique Zipf(alpha)-distributed keys over [1, 2^universe_bits].

    Inverse-CDF sampling of the continuous power law on [1, U] gives rank r with
    density ~ r^-alpha; ranks are mixed to spread hot keys over buckets, then the
    batch is de-duplicated (order of first occurrence kept) and truncated to n.
    """
    U = float(1 << universe_bits)
    out = np.zeros(0, np.uint64)
    pos = start
    a = 1.0 - alpha
    while len(out) < n:
        m = int((n - len(out)) * 1.6) + 1024
        u = (stream(seed ^ 0x5A5A, pos, m) >> np.uint64(11)).astype(np.float64) / float(1 << 53)
        pos += m
        r = np.floor((1.0 + u * (U ** a - 1.0)) ** (1.0 / a)).astype(np.uint64)
        k = splitmix64(r)  # rank -> key, bijective
        k[(k & np.uint64(0xFFFFFFFFFFFFFFFC)) == np.uint64(0xFFFFFFFFFFFFFFFC)] &= np.uint64(0x7FFFFFFFFFFFFFFF)
        out = np.concatenate([out, k])
        _, first = np.unique(out, return_index=True)
        out = out[np.sort(first)]
    return out[:n], pos


def monotone_scores(batch_seq, n, seed=0):
    """Distinct scores that grow with the batch number: (batch << 40) | perm.
    Within a batch the low part is a seeded permutation of 0..n-1, so scores
    are pairwise distinct and no later batch ever scores below an earlier one."""
    rng = np.random.Generator(np.random.PCG64(seed * 1000003 + batch_seq))
    perm = rng.permutation(n).astype(np.uint64)
    return (np.uint64(batch_seq) << np.uint64(40)) | perm
