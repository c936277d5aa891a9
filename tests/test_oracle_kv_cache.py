"""Pins of the checker's key/value-cache functions (CPU only).

copy_intersection is checked against its definition, element by element, on
tiny arrays; the cache against plain concatenation; the mask slice against
the closed form for a causal mask; and the composition against what the
reference's own tests assert (wrappers/python/tests/model/test_llama_attention.py:
320-345: prefill, then decode chunk by chunk, equals the rows of one pass over
the whole sequence)."""
import itertools
import ctypes

import numpy as np
import pytest

from nntile_amd import hip_sdpa as h, synth


def _brute_copy(src, so, dst, do):
    """dst[g - do] = src[g - so] for every global index g inside both."""
    out = dst.copy()
    for idx in itertools.product(*[range(n) for n in dst.shape]):
        g = [i + o for i, o in zip(idx, do)]
        s = [gi - o for gi, o in zip(g, so)]
        if all(0 <= si < n for si, n in zip(s, src.shape)):
            out[idx] = src[tuple(s)]
    return out


@pytest.mark.parametrize("seed", range(40))
def test_copy_intersection_is_the_global_index_copy(oracle, seed):
    rng = np.random.default_rng(seed)
    ndim = int(rng.integers(1, 4))
    s_shape = rng.integers(1, 6, ndim)
    d_shape = rng.integers(1, 6, ndim)
    so = [int(v) for v in rng.integers(0, 5, ndim)]
    do = [int(v) for v in rng.integers(0, 5, ndim)]
    src = rng.standard_normal(s_shape).astype(np.float32)
    dst = rng.standard_normal(d_shape).astype(np.float32)
    want = _brute_copy(src, so, dst, do)
    got = oracle.copy_intersection(src, so, dst.copy(), do)
    assert np.array_equal(got, want)


def test_copy_intersection_disjoint_leaves_dst(oracle):
    src, dst = np.ones((3, 3), np.float32), np.zeros((3, 3), np.float32)
    assert not oracle.copy_intersection(src, [0, 3], dst, [0, 0]).any()
    assert not oracle.copy_intersection(src, [0, 0], dst, [3, 0]).any()


def test_cache_append_is_concatenation(oracle):
    rng = np.random.default_rng(3)
    head, n_batch, n_kv, cap = 4, 2, 3, 11
    cache = oracle.KVCache(cap, 1)
    ks, vs = [], []
    for rows in (5, 1, 3, 2):
        k = rng.standard_normal((head, rows, n_batch, n_kv)).astype(np.float32)
        v = rng.standard_normal((head, rows, n_batch, n_kv)).astype(np.float32)
        cache.append(k, v)
        ks.append(k)
        vs.append(v)
        assert len(cache) == sum(a.shape[1] for a in ks)
        assert cache.k.shape == (head, cap, n_batch, n_kv)
        assert np.array_equal(cache.k_partial, np.concatenate(ks, axis=1))
        assert np.array_equal(cache.v_partial, np.concatenate(vs, axis=1))
        assert not cache.k[:, len(cache):].any()        # the rest stays zero


@pytest.mark.parametrize("k_seq,q_seq,full", [(6, 2, 8), (8, 8, 8), (9, 1, 16), (5, 5, 12), (16, 3, 16)])
def test_mask_slice_of_a_causal_mask_is_the_offset_rule(oracle, k_seq, q_seq, full):
    k = np.arange(full)[:, None]
    q = np.arange(full)[None, :]
    causal = k <= q                                        # [keys, queries]
    got = oracle.prepare_mask_for_kv_cache(causal, k_seq, q_seq)
    kk = np.arange(k_seq)[:, None]
    jj = np.arange(q_seq)[None, :]
    assert np.array_equal(got, kk <= jj + (k_seq - q_seq))
    # the same rule in the [q_seq, k_seq] orientation the kernels take
    assert np.array_equal(got.T, synth.causal_mask(q_seq, k_seq, k_seq - q_seq))


def test_mask_of_the_right_shape_passes_through(oracle):
    m = np.random.default_rng(0).random((7, 3)) < 0.5
    assert oracle.prepare_mask_for_kv_cache(m, 7, 3) is not None
    assert np.array_equal(oracle.prepare_mask_for_kv_cache(m, 7, 3), m)


def test_cached_decode_equals_rows_of_the_full_pass(oracle):
    """Prefill then two decode chunks through the cache and the mask slice give
    the rows of one causal pass over the whole sequence."""
    head, n_batch, n_kv, group, total, prefill = 16, 2, 2, 2, 24, 17
    kv_batch, batch = n_batch * n_kv, n_batch * n_kv * group
    q = synth.randn(5, 0, batch * total * head).reshape(batch, total, head)
    k = synth.randn(5, 1, kv_batch * total * head).reshape(kv_batch, total, head)
    v = synth.randn(5, 2, kv_batch * total * head).reshape(kv_batch, total, head)
    full_mask = synth.causal_mask(total, total)            # [q, k]
    want, want_lse = oracle.sdpa_vanilla(k, q, v, full_mask, n_batch=n_batch, kv_repeat=group)
    cache = oracle.KVCache(total, 1)
    # the reference's axis order is the reverse of the C order used here
    to_ref = lambda a: np.ascontiguousarray(a.transpose(2, 1, 0))
    to_c = lambda a: np.ascontiguousarray(a.transpose(2, 1, 0))
    pos = 0
    for rows in (prefill, 1, total - prefill - 1):
        cache.append(to_ref(k[:, pos:pos + rows]), to_ref(v[:, pos:pos + rows]))
        k_seq = len(cache)
        m = oracle.prepare_mask_for_kv_cache(full_mask.T, k_seq, rows)      # [k, q]
        got, got_lse = oracle.sdpa_vanilla(to_c(cache.k_partial), q[:, pos:pos + rows],
                                           to_c(cache.v_partial), m.T, n_batch=n_batch,
                                           kv_repeat=group)
        assert np.allclose(got, want[:, pos:pos + rows], rtol=1e-5, atol=1e-6)
        assert np.allclose(got_lse, want_lse[:, pos:pos + rows], rtol=1e-5, atol=1e-6)
        pos += rows


def test_append_and_cache_decode_argument_checks():
    """Checked before anything touches HIP."""
    L = h.lib()
    for t in ("bf16", "fp16", "fp32"):
        f = getattr(L, "nntile_hip_kv_cache_append_" + t)
        # head, rows, entries, capacity, filled
        assert f(None, 64, 3, 2, 8, 6, 4096, 4096, 4096, 4096) == h.EINVAL     # 3 > 8 - 6
        assert f(None, 64, 0, 2, 8, 8, None, None, None, None) == h.OK         # nothing to add
        assert f(None, 64, 1, 0, 8, 0, None, None, None, None) == h.OK
        assert f(None, 0, 1, 2, 8, 0, 4096, 4096, 4096, 4096) == h.EINVAL
        assert f(None, 64, 1, 2, 8, -1, 4096, 4096, 4096, 4096) == h.EINVAL
        assert f(None, 64, 1, 2, 8, 0, None, 4096, 4096, 4096) == h.EINVAL
    a = h.TileArgs()
    a.q_seq, a.k_seq, a.head, a.batch, a.n_batch, a.kv_group = 1, 512, 128, 16, 2, 4
    a.mask_mode = h.MASK_CAUSAL
    a.K = a.Q = a.V = a.lse = a.A = 4096
    dec = L.nntile_hip_sdpa_fwd_decode_cache_bf16
    assert dec(None, ctypes.byref(a), 511, 4096, 1 << 30) == h.EINVAL            # capacity < k_seq
    assert dec(None, ctypes.byref(a), 1024, None, 0) == h.EWORKSPACE
    assert dec(None, None, 1024, 4096, 1 << 30) == h.EINVAL
    for t in ("bf16", "fp16", "fp32"):
        tile = getattr(L, "nntile_hip_sdpa_fwd_tile_cache_" + t)
        assert tile(None, ctypes.byref(a), 511) == h.EINVAL                      # capacity < k_seq
        assert tile(None, None, 1024) == h.EINVAL
        a.head = 48
        assert tile(None, ctypes.byref(a), 1024) == h.EUNSUPPORTED
        a.head = 128
