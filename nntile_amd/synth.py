"""Seeded synthetic inputs for the attention tiles.

A counter-based generator (splitmix64 -> Box-Muller) so that any slice of a
stream can be produced without producing what precedes it, and so that the
benchmark, the tests and the CPU checker all see the same values.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _splitmix64(x):
    with np.errstate(over="ignore"):
        z = x + _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def randn(seed, stream, n, offset=0, chunk=1 << 22):
    """n i.i.d. N(0,1) fp32 values: elements [offset, offset+n) of the stream
    named by (seed, stream)."""
    out = np.empty(n, np.float32)
    with np.errstate(over="ignore"):
        key = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3)
                          + np.uint64(stream))
    for start in range(0, n, chunk):
        m = min(chunk, n - start)
        ctr = np.arange(offset + start, offset + start + m, dtype=np.uint64)
        with np.errstate(over="ignore"):
            a = _splitmix64(key ^ (ctr * np.uint64(2)))
            b = _splitmix64(key ^ (ctr * np.uint64(2) + np.uint64(1)))
        u1 = ((a >> np.uint64(11)).astype(np.float64) + 1.0) * (2.0 ** -53)
        u2 = (b >> np.uint64(11)).astype(np.float64) * (2.0 ** -53)
        out[start:start + m] = (np.sqrt(-2.0 * np.log(u1))
                                * np.cos(2.0 * np.pi * u2)).astype(np.float32)
    return out


def _signed(u):
    """A 64-bit pattern as the int64 with the same bits."""
    u = int(u)
    return u - (1 << 64) if u >= (1 << 63) else u


def randn_torch(seed, stream, n, device="cuda", offset=0, chunk=1 << 24):
    """`randn` evaluated with torch on `device` (int64 arithmetic wraps like
    uint64; the logical right shifts are masked arithmetic ones): the same
    stream of values, produced where they are needed.  The uniform variates
    are bit-identical to the numpy version's; log, sqrt and cos are the
    device's, so a value may differ from numpy's in its last bit."""
    import torch
    key = _signed(_splitmix64(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(stream)))
    golden, m1, m2 = _signed(_GOLDEN), _signed(_M1), _signed(_M2)

    def lsr(z, k):
        return (z >> k) & ((1 << (64 - k)) - 1)

    def mix(x):
        z = x + golden
        z = (z ^ lsr(z, 30)) * m1
        z = (z ^ lsr(z, 27)) * m2
        return z ^ lsr(z, 31)

    out = torch.empty(n, dtype=torch.float32, device=device)
    for start in range(0, n, chunk):
        m = min(chunk, n - start)
        ctr = torch.arange(offset + start, offset + start + m, dtype=torch.int64, device=device)
        a = mix((ctr * 2) ^ key)
        b = mix((ctr * 2 + 1) ^ key)
        u1 = (lsr(a, 11).to(torch.float64) + 1.0) * (2.0 ** -53)
        u2 = lsr(b, 11).to(torch.float64) * (2.0 ** -53)
        out[start:start + m] = (torch.sqrt(-2.0 * torch.log(u1))
                                * torch.cos(2.0 * np.pi * u2)).to(torch.float32)
    return out


def permutation(seed, stream, n):
    """A seeded permutation of range(n) (argsort of a hashed counter)."""
    with np.errstate(over="ignore"):
        key = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3)
                          + np.uint64(stream))
        h = _splitmix64(key ^ np.arange(n, dtype=np.uint64))
    return np.argsort(h, kind="stable")


def round_bf16(x):
    """Round fp32 values to the nearest bf16 (ties to even); returns
    (uint16 storage, the rounded values as fp32)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
         ) >> np.uint32(16)
    bits = r.astype(np.uint16)
    return bits, (r << np.uint32(16)).astype(np.uint32).view(np.float32)


def bf16_bits_to_f32(bits):
    return (np.ascontiguousarray(bits, np.uint16).astype(np.uint32)
            << np.uint32(16)).view(np.float32)


def round_fp16(x):
    h = np.ascontiguousarray(x, np.float32).astype(np.float16)
    return h.view(np.uint16), h.astype(np.float32)


def causal_mask(q_seq, k_seq, offset=0):
    """Boolean visibility [q_seq, k_seq] (C order = the reference's Fortran
    [k_seq, q_seq]): key k is visible to query q iff k <= q + offset."""
    q = np.arange(q_seq)[:, None]
    k = np.arange(k_seq)[None, :]
    return k <= q + offset
