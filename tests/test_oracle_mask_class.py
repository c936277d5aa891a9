"""Pins of the checker's mask-tile classification (CPU only): brute force over
the definition on tiny tiles, and the property that makes it safe to act on -
attention with the class's analytic stand-in equals attention with the mask."""
import ctypes
import itertools

import numpy as np
import pytest

from nntile_amd import hip_sdpa as h


def _brute(mask, offset):
    kr, qc = mask.shape
    vis = hid = other = off_rule = False
    for k, q in itertools.product(range(kr), range(qc)):
        v = mask[k, q]
        if mask.dtype == bool:
            is_vis, is_hid = bool(v), not bool(v)
        else:
            is_vis, is_hid = v == 0.0, v == -np.inf
        vis |= is_vis
        hid |= is_hid
        other |= not (is_vis or is_hid)
        off_rule |= is_vis != (k <= q + offset)
    if other:
        return 0
    if not hid:
        return 1
    if not vis:
        return 2
    return 0 if off_rule else 3


@pytest.mark.parametrize("seed", range(60))
def test_class_equals_brute_force(oracle, seed):
    rng = np.random.default_rng(seed)
    kr, qc = int(rng.integers(1, 7)), int(rng.integers(1, 7))
    offset = int(rng.integers(-4, 5))
    kind = seed % 6
    k, q = np.arange(kr)[:, None], np.arange(qc)[None, :]
    if kind == 0:
        vis = np.ones((kr, qc), bool)
    elif kind == 1:
        vis = np.zeros((kr, qc), bool)
    elif kind in (2, 3):
        vis = k <= q + offset
        if kind == 3:                                  # one element off the rule
            vis = vis.copy()
            vis[rng.integers(kr), rng.integers(qc)] ^= True
    else:
        vis = rng.random((kr, qc)) < 0.5
    if seed % 2:
        mask = vis
    else:
        mask = np.where(vis, 0.0, -np.inf).astype(np.float32)
        if kind == 5:
            mask[rng.integers(kr), rng.integers(qc)] = -0.5      # a bias
    assert oracle.mask_tile_class(mask, offset) == _brute(mask, offset)


def test_negative_zero_is_visible_and_nan_is_other(oracle):
    m = np.array([[0.0, -0.0], [-0.0, 0.0]], np.float32)
    assert oracle.mask_tile_class(m) == oracle.TILE_OPEN
    m[0, 0] = np.nan
    assert oracle.mask_tile_class(m) == oracle.TILE_MIXED
    m[0, 0] = np.inf
    assert oracle.mask_tile_class(m) == oracle.TILE_MIXED


@pytest.mark.parametrize("offset", [-3, 0, 2])
def test_acting_on_the_class_keeps_the_attention(oracle, offset):
    """A tile classified CAUSAL / OPEN gives the same attention through the
    rule it names as through its values."""
    from nntile_amd import synth
    q_seq, k_seq, head, batch = 9, 11, 8, 2
    q = synth.randn(3, 0, batch * q_seq * head).reshape(batch, q_seq, head)
    k = synth.randn(3, 1, batch * k_seq * head).reshape(batch, k_seq, head)
    v = synth.randn(3, 2, batch * k_seq * head).reshape(batch, k_seq, head)
    kk, qq = np.arange(k_seq)[:, None], np.arange(q_seq)[None, :]
    tile = kk <= qq + offset                                       # [k, q]
    assert oracle.mask_tile_class(tile, offset) == oracle.TILE_CAUSAL
    assert oracle.mask_tile_class(tile, offset + 1) == oracle.TILE_MIXED
    want = oracle.sdpa_vanilla(k, q, v, tile.T)
    got = oracle.sdpa_vanilla(k, q, v, synth.causal_mask(q_seq, k_seq, offset))
    assert np.array_equal(want[0], got[0]) and np.array_equal(want[1], got[1])
    open_tile = np.ones((k_seq, q_seq), bool)
    assert oracle.mask_tile_class(open_tile, offset) == oracle.TILE_OPEN
    a = oracle.sdpa_vanilla(k, q, v, open_tile.T)
    b = oracle.sdpa_vanilla(k, q, v, None)
    assert np.allclose(a[0], b[0], rtol=1e-6, atol=1e-7)


def test_argument_checks_before_any_launch():
    L = h.lib()
    out = ctypes.c_int32(-7)
    for t in ("bf16", "fp16", "fp32", "bool"):
        f = getattr(L, "nntile_hip_mask_tile_class_" + t)
        assert f(None, 0, 4, 4096, 0, 4096, ctypes.byref(out)) == h.EINVAL
        assert f(None, 4, 4, None, 0, 4096, ctypes.byref(out)) == h.EINVAL
        assert f(None, 4, 4, 4096, 0, None, ctypes.byref(out)) == h.EINVAL
        assert f(None, 4, 4, 4096, 0, 4098, ctypes.byref(out)) == h.EINVAL        # misaligned word
        assert f(None, 4, 4, 4096, 0, 4096, None) == h.EINVAL
    assert out.value == -7


def _classes(oracle, mask_kq, k_tile, q_tile, offset):
    """Classes of the tiles of a [k, q] mask in the grid's linear order (key
    tile fastest), each against the rule moved into the tile."""
    k_seq, q_seq = mask_kq.shape
    out = []
    for q0 in range(0, q_seq, q_tile):
        for k0 in range(0, k_seq, k_tile):
            out.append(oracle.mask_tile_class(mask_kq[k0:k0 + k_tile, q0:q0 + q_tile],
                                              q0 - k0 + offset))
    return out


@pytest.mark.parametrize("seed", range(30))
def test_whole_mask_rule_from_the_classes(oracle, seed):
    """tensor::flash_sdpa_mask_rule (host library, no GPU): the classes of a
    mask that is the causal rule say so on any tiling, ragged last tiles
    included; one element off the rule anywhere and they do not."""
    from nntile_amd import host_mirror as hm
    rng = np.random.default_rng(seed)
    k_seq, q_seq = int(rng.integers(3, 40)), int(rng.integers(3, 40))
    k_tile, q_tile = int(rng.integers(1, k_seq + 1)), int(rng.integers(1, q_seq + 1))
    offset = int(rng.integers(-q_seq, k_seq))
    k, q = np.arange(k_seq)[:, None], np.arange(q_seq)[None, :]
    rule = k <= q + offset
    cls = _classes(oracle, rule, k_tile, q_tile, offset)
    want = 1
    if not rule.all():
        want = 2
    assert hm.mask_rule(k_seq, q_seq, k_tile, q_tile, cls, offset) == want
    if rule.any() and not rule.all():
        dent = rule.copy()
        dent[rng.integers(k_seq), rng.integers(q_seq)] ^= True
        cls = _classes(oracle, dent, k_tile, q_tile, offset)
        got = hm.mask_rule(k_seq, q_seq, k_tile, q_tile, cls, offset)
        assert got == (1 if dent.all() else -1)
    open_cls = _classes(oracle, np.ones((k_seq, q_seq), bool), k_tile, q_tile, offset)
    assert hm.mask_rule(k_seq, q_seq, k_tile, q_tile, open_cls, offset) == 1
    with pytest.raises(hm.HostError):
        hm.mask_rule(k_seq, q_seq, k_tile, q_tile, open_cls + [1], offset)
