"""GPU checks of the mask-tile classification and of the tensor-level forward
that acts on it: classes equal the checker's on every pattern, and the
classified submission gives the reference submission's result with fewer
tasks (src/tensor/flash_sdpa_fwd_cudnn.cc:246-274 submits every pair)."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, host_mirror as hm, synth
from . import helpers as H
from .test_host_mirror import _case, _fortran5

pytestmark = pytest.mark.gpu


def _patterns(kr, qc, offset, rng):
    k, q = np.arange(kr)[:, None], np.arange(qc)[None, :]
    rule = k <= q + offset
    out = {"open": np.ones((kr, qc), bool), "hidden": np.zeros((kr, qc), bool), "rule": rule,
           "window": np.abs(k - q) <= 32, "random": rng.random((kr, qc)) < 0.5}
    for name, (kk, qq) in {"first": (0, 0), "last": (kr - 1, qc - 1),
                           "inner": (int(rng.integers(kr)), int(rng.integers(qc)))}.items():
        for base in ("open", "hidden", "rule"):
            m = out[base].copy()
            m[kk, qq] ^= True
            out[base + "_flip_" + name] = m
    return out


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32", "bool"])
@pytest.mark.parametrize("kr,qc,offset", [(1, 1, 0), (64, 64, 0), (128, 128, -5), (70, 4200, 100),
                                          (4200, 70, -4000), (1024, 1024, 0), (333, 257, 40),
                                          (1024, 1024, 1024), (1024, 1024, -1024)])
def test_classes_equal_the_checker(oracle, dtype, kr, qc, offset):
    print("case", dtype, kr, qc, offset, flush=True)
    rng = np.random.default_rng(kr * 7 + qc)
    ws = torch.empty(1, dtype=torch.int32, device="cuda")
    for name, vis in _patterns(kr, qc, offset, rng).items():
        if dtype == "bool":
            ref_mask = vis
            dev = torch.from_numpy(np.ascontiguousarray(vis.T)).cuda()
        else:
            ref_mask = np.where(vis, 0.0, -np.inf).astype(np.float32)
            dev = torch.from_numpy(np.ascontiguousarray(ref_mask.T)).to(H.TORCH_DT[dtype]).cuda()
        want = oracle.mask_tile_class(ref_mask, offset)
        got = hip_sdpa.mask_tile_class(dev, offset, ws)
        assert got == want, (name, got, want)
    if dtype != "bool":                                  # a bias anywhere makes the tile MIXED
        m = np.where(np.ones((kr, qc), bool), 0.0, 0.0).astype(np.float32)
        m[kr - 1, qc // 2] = -0.5
        dev = torch.from_numpy(np.ascontiguousarray(m.T)).to(H.TORCH_DT[dtype]).cuda()
        assert hip_sdpa.mask_tile_class(dev, offset, ws) == hip_sdpa.TILE_MIXED
        m[kr - 1, qc // 2] = -0.0                        # minus zero is visible
        dev = torch.from_numpy(np.ascontiguousarray(m.T)).to(H.TORCH_DT[dtype]).cuda()
        assert hip_sdpa.mask_tile_class(dev, offset, ws) == hip_sdpa.TILE_OPEN


def _tensors(dtype, arrs, mask_bool, head, seq, nb, grp, nkv, tile):
    s5 = [head, seq, nb, grp, nkv]
    b5 = [head, tile, max(1, nb // 2), 1, max(1, nkv // 2)]
    T = {n: hm.Tensor(dtype, s5, b5).from_array(arrs[n]) for n in ("K", "Q", "V")}
    A = hm.Tensor(dtype, s5, b5).from_array(np.zeros(s5, np.float32 if dtype == "fp32" else np.uint16))
    lse = hm.Tensor("fp32", s5[1:], b5[1:]).from_array(np.full(s5[1:], -np.inf, np.float32))
    add = np.where(mask_bool, 0.0, -np.inf).astype(np.float32).T               # [k_seq, q_seq]
    m_t, _ = H.rounded(add, dtype)
    m_np = m_t.numpy() if dtype == "fp32" else m_t.view(torch.int16).numpy().view(np.uint16)
    mask = hm.Tensor(dtype, [seq, seq], [tile, tile]).from_array(np.asfortranarray(m_np))
    return T, A, lse, mask


def _read(dtype, A, lse, head, seq):
    a = A.to_array()
    if dtype != "fp32":
        a = H.to_np(torch.from_numpy(a.view(np.int16).copy()).view(H.TORCH_DT[dtype]))
    a = np.ascontiguousarray(a.transpose(4, 3, 2, 1, 0)).reshape(-1, seq, head)
    l = np.ascontiguousarray(lse.to_array().transpose(3, 2, 1, 0)).reshape(-1, seq)
    return a, l


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("kind,want_classes", [
    ("causal", {"hidden": 6, "open": 6, "causal": 4, "mixed": 0}),
    ("window", None), ("full", {"hidden": 0, "open": 16, "causal": 0, "mixed": 0}),
    ("causal_dent", {"hidden": 6, "open": 5, "causal": 4, "mixed": 1})])
def test_classified_submission_equals_the_reference_submission(oracle, dtype, kind, want_classes):
    head, seq, nb, grp, nkv, tile = 64, 512, 2, 1, 2, 128
    arrs, (qf, kf, vf) = _case(dtype, head, seq, nb, grp, nkv, seed=11)
    k, q = np.arange(seq)[None, :], np.arange(seq)[:, None]
    mask = {"causal": synth.causal_mask(seq, seq), "window": np.abs(k - q) <= 100,
            "full": np.ones((seq, seq), bool), "causal_dent": synth.causal_mask(seq, seq)}[kind]  # [q, k]
    if kind == "causal_dent":
        mask = mask.copy()
        mask[400, 3] = False            # one key hidden far below the diagonal
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, k_tile=tile)
    # the reference's submission: every pair with its mask tile
    T, A0, lse0, M = _tensors(dtype, arrs, mask, head, seq, nb, grp, nkv, tile)
    before = hm.tasks_submitted(dtype)
    hm.flash_sdpa_fwd(hm.OP_PAIRS, T["K"], T["Q"], M, lse0, T["V"], A0)
    all_pairs = hm.tasks_submitted(dtype) - before
    ref_a, ref_lse = _read(dtype, A0, lse0, head, seq)
    # the classified submission
    T, A1, lse1, M = _tensors(dtype, arrs, mask, head, seq, nb, grp, nkv, tile)
    classes, submitted = hm.flash_sdpa_fwd_classified(T["K"], T["Q"], M, lse1, T["V"], A1)
    got_a, got_lse = _read(dtype, A1, lse1, head, seq)
    n_t = seq // tile
    assert len(classes) == n_t * n_t and all_pairs == A1.ntiles * n_t
    # classes against the checker, tile by tile (mask grid is [key tile, query tile], Fortran order)
    for lin, cls in enumerate(classes):
        kt, qt = lin % n_t, lin // n_t
        sub = mask[qt * tile:(qt + 1) * tile, kt * tile:(kt + 1) * tile].T
        assert cls == oracle.mask_tile_class(sub, (qt - kt) * tile), (kt, qt)
    count = {"hidden": classes.count(hip_sdpa.TILE_HIDDEN), "open": classes.count(hip_sdpa.TILE_OPEN),
             "causal": classes.count(hip_sdpa.TILE_CAUSAL), "mixed": classes.count(hip_sdpa.TILE_MIXED)}
    if want_classes is not None:
        assert count == want_classes
    else:
        assert count["hidden"] > 0 and count["mixed"] > 0
    slabs = A1.ntiles // n_t
    if kind in ("causal", "full"):
        # the mask is the causal rule itself / hides nothing: the slabs share
        # launches, as many as the launch's tile tables hold
        per_launch = hip_sdpa.MAX_TILES // n_t
        assert submitted == -(-slabs // per_launch)
    else:
        assert submitted == slabs * (n_t * n_t - count["hidden"])
    assert H.rel_fro(got_a, want) < H.TOL[dtype] and H.rel_fro(got_lse, want_lse) < H.TOL[dtype]
    assert H.rel_fro(got_a, ref_a) < H.TOL[dtype] and H.rel_fro(got_lse, ref_lse) < H.TOL[dtype]


def test_a_bias_mask_is_submitted_as_the_reference_does(oracle):
    """Additive values other than 0 and -inf: every tile MIXED, every pair
    submitted with its mask, bit-identical to the reference submission."""
    dtype, head, seq, nb, grp, nkv, tile = "bf16", 64, 256, 2, 1, 2, 128
    arrs, _ = _case(dtype, head, seq, nb, grp, nkv, seed=12)
    s5 = [head, seq, nb, grp, nkv]
    b5 = [head, tile, 1, 1, 1]
    bias = (-0.25 * np.abs(np.arange(seq)[:, None] - np.arange(seq)[None, :]) - 0.25).astype(np.float32)
    m_t, _ = H.rounded(bias, dtype)
    m_np = np.asfortranarray(m_t.view(torch.int16).numpy().view(np.uint16))
    outs = []
    for classified in (False, True):
        T = {n: hm.Tensor(dtype, s5, b5).from_array(arrs[n]) for n in ("K", "Q", "V")}
        A = hm.Tensor(dtype, s5, b5).from_array(np.zeros(s5, np.uint16))
        lse = hm.Tensor("fp32", s5[1:], b5[1:]).from_array(np.full(s5[1:], -np.inf, np.float32))
        M = hm.Tensor(dtype, [seq, seq], [tile, tile]).from_array(m_np)
        if classified:
            classes, submitted = hm.flash_sdpa_fwd_classified(T["K"], T["Q"], M, lse, T["V"], A)
            assert classes == [hip_sdpa.TILE_MIXED] * 4 and submitted == A.ntiles * 2
        else:
            hm.flash_sdpa_fwd(hm.OP_PAIRS, T["K"], T["Q"], M, lse, T["V"], A)
        outs.append((A.to_array().copy(), lse.to_array().copy()))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
