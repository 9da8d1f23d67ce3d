"""Device-side generators for workloads too large for host arrays: keys, scores and rows are
functions of a counter (or of the key), computed with torch on the GPU, so that a 2^28-slot
table is filled in seconds and every row that comes back can be checked from its key alone.
Shared by the full-size tests and by bench.py's per-configuration mode."""
import torch

DEV = "cuda:0"
M63 = (1 << 63) - 1


def _lsr(x, k):
    return (x >> k) & ((1 << (64 - k)) - 1)


def _s64(c):
    return c - (1 << 64) if c >= (1 << 63) else c


def mix64(x):
    """splitmix64 finaliser on int64 tensors (bit patterns of uint64): a bijection."""
    z = x + _s64(0x9E3779B97F4A7C15)
    z = (z ^ _lsr(z, 30)) * _s64(0xBF58476D1CE4E5B9)
    z = (z ^ _lsr(z, 27)) * _s64(0x94D049BB133111EB)
    return z ^ _lsr(z, 31)


def fold_reserved(k):
    """The four reserved patterns (top 62 bits all ones) are folded away by clearing bit 63."""
    return torch.where((k | 3) == -1, k & M63, k)


def dev_keys(seed, start, n):
    """n unique keys: the mix of the counters start..start+n-1."""
    c = torch.arange(start, start + n, dtype=torch.int64, device=DEV) + (seed << 40)
    return fold_reserved(mix64(c))


def value_of(keys, dim):
    """fp32 row of a key: float(key & 1023) + d."""
    return (keys & 1023).to(torch.float32)[:, None] + torch.arange(dim, dtype=torch.float32, device=DEV)[None, :]


def score_of(keys):
    """Customized-strategy score of a key: 63-bit mix, distinct for practical purposes."""
    return _lsr(mix64(keys ^ 0x5555), 1)


def batch_scores(keys, batch):
    """Customized scores that grow with the batch number and are distinct inside a batch for
    practical purposes: (batch << 40) | 40 bits of a mix of the key."""
    return (batch << 40) | (mix64(keys ^ 0x3333) & ((1 << 40) - 1))


def zipf_keys(gen, n, universe_bits=31, alpha=1.05):
    """n unique keys whose ranks follow a power law with exponent alpha over [1, 2^universe_bits]
    (inverse-CDF sampling of the continuous law), rank -> key by the mixing bijection, the
    batch de-duplicated and cut to n in random order."""
    U = float(1 << universe_bits)
    a = 1.0 - alpha
    out = torch.zeros(0, dtype=torch.int64, device=DEV)
    while out.numel() < n:
        m = int((n - out.numel()) * 1.7) + 4096
        u = torch.rand(m, dtype=torch.float64, device=DEV, generator=gen)
        r = torch.floor((1.0 + u * (U ** a - 1.0)) ** (1.0 / a)).to(torch.int64)
        out = torch.unique(torch.cat([out, fold_reserved(mix64(r))]))
    perm = torch.randperm(out.numel(), device=DEV, generator=gen)
    return out[perm[:n]].contiguous()
