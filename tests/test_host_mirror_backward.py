"""The C++ host mirror of the reference's backward layers (codelet, tile,
tensor).

CPU part: the shape rules and their messages (src/tile/flash_sdpa_bwd_cudnn.cc:
24-89, src/tensor/flash_sdpa_bwd_cudnn.cc:22-161).
GPU part: multi-tile tensors against the single-tile result, on the data of
the reference's own test (tests/tensor/flash_sdpa_bwd_cudnn.cc:46-324), and
both against the fp64 checker."""
import numpy as np
import pytest

from nntile_amd import hip_sdpa, host_mirror as hm, synth
from . import helpers as H

ORDER = ("K", "Q", "V", "A", "dA", "mask", "lse", "dK", "dQ", "dV")


def _specs(head=64, seq=128, nb=2, grp=1, nkv=3, tile=None, **over):
    tile = tile or seq
    s5, b5 = [head, seq, nb, grp, nkv], [head, tile, nb, grp, nkv]
    d = {n: (list(s5), list(b5)) for n in ORDER}
    d["mask"] = ([seq, seq], [tile, tile])
    d["lse"] = ([seq, nb, grp, nkv], [tile, nb, grp, nkv])
    d.update(over)
    return [d[k] for k in ORDER]


def test_shape_rules_accept_the_reference_cases():
    # tests/tensor/flash_sdpa_bwd_cudnn.cc:322-324
    hm.check_shapes_bwd(0, _specs(32, 64, 1, 1, 1))
    hm.check_shapes_bwd(1, _specs(32, 128, 1, 1, 1, tile=64))
    s5, b5 = [64, 256, 3, 2, 4], [64, 64, 1, 1, 2]
    d = {n: (s5, b5) for n in ORDER}
    d["mask"] = ([256, 256], [64, 64])
    d["lse"] = (s5[1:], b5[1:])
    hm.check_shapes_bwd(1, [d[k] for k in ORDER])


@pytest.mark.parametrize("level", [0, 1])
@pytest.mark.parametrize("change,message", [
    ({"dA": ([64, 128, 2, 1], [64, 128, 2, 1])}, "dA.ndim != 5"),
    ({"dV": ([64, 128, 2, 1, 3, 1], [64, 128, 2, 1, 3, 1])}, "dV.ndim != 5"),
    ({"mask": ([128, 128, 1], [128, 128, 1])}, "mask.ndim != 2"),
    ({"lse": ([128, 2, 1, 3, 1], [128, 2, 1, 3, 1])}, "logsumexp.ndim != 4"),
    ({"Q": ([32, 128, 2, 1, 3], [32, 128, 2, 1, 3])}, "K.shape != Q.shape"),
    ({"A": ([64, 64, 2, 1, 3], [64, 64, 2, 1, 3])}, "K.shape != A.shape"),
    ({"dQ": ([64, 128, 4, 1, 3], [64, 128, 4, 1, 3])}, "K.shape != dQ.shape"),
    ({"mask": ([64, 128], [64, 128])}, "Mask shape mismatch"),
    ({"lse": ([64, 2, 1, 3], [64, 2, 1, 3])}, "logsumexp axis 0 must match sequence length"),
    ({"lse": ([128, 4, 1, 3], [128, 4, 1, 3])}, "logsumexp axis 1 must match batch"),
    ({"lse": ([128, 2, 2, 3], [128, 2, 2, 3])}, "logsumexp axis 2 must match kv_group_size"),
    ({"lse": ([128, 2, 1, 5], [128, 2, 1, 5])}, "logsumexp axis 3 must match n_head_kv"),
])
def test_shape_rules_reject_with_reference_messages(level, change, message):
    with pytest.raises(hm.HostError) as e:
        hm.check_shapes_bwd(level, _specs(**change))
    assert str(e.value) == message


@pytest.mark.parametrize("change,message", [
    ({"dQ": ([64, 128, 2, 1, 3], [64, 64, 2, 1, 3])}, "Q, dQ, A, dA basetile shapes must match"),
    ({"dA": ([64, 128, 2, 1, 3], [64, 128, 1, 1, 3])}, "Q, dQ, A, dA basetile shapes must match"),
    ({"K": ([64, 128, 2, 1, 3], [64, 128, 1, 1, 3])}, "K and Q basetile shapes mismatch"),
    ({"V": ([64, 128, 2, 1, 3], [64, 128, 2, 1, 1])}, "V and Q basetile shapes mismatch"),
    ({"dK": ([64, 128, 2, 1, 3], [64, 128, 1, 1, 3])}, "dK and Q basetile shapes mismatch"),
    ({"dV": ([64, 128, 2, 1, 3], [64, 128, 2, 1, 1])}, "dV and Q basetile shapes mismatch"),
    ({"mask": ([128, 128], [64, 128])},
     "mask basetile axis 0 must match K basetile sequence dimension"),
    ({"mask": ([128, 128], [128, 64])},
     "mask basetile axis 1 must match Q basetile sequence dimension"),
    ({"lse": ([128, 2, 1, 3], [64, 2, 1, 3])},
     "logsumexp basetile shape must match Q basetile shape (excluding head dimension)"),
])
def test_tensor_level_basetile_rules(change, message):
    with pytest.raises(hm.HostError) as e:
        hm.check_shapes_bwd(1, _specs(**change))
    assert str(e.value) == message


def test_head_axis_must_not_be_tiled():
    s5, b5 = [64, 128, 2, 1, 3], [32, 128, 2, 1, 3]
    with pytest.raises(hm.HostError, match="head dimension must not be tiled"):
        hm.check_shapes_bwd(1, _specs(**{n: (s5, b5) for n in ORDER if n not in ("mask", "lse")}))


def test_footprint_and_codelet_names():
    # the footprint hashes (seq, head, batch), as the forward's does
    # (src/starpu/flash_sdpa_bwd_cudnn.cc:143-166)
    assert hm.footprint_bwd(64, 32, 1) == hm.footprint(64, 32, 1)
    assert hm.footprint_bwd(64, 32, 1) != hm.footprint_bwd(64, 32, 2)
    assert hm.codelet_name_bwd("bf16") == "nntile_flash_sdpa_bwd_cudnn_bf16"
    assert hm.codelet_name_bwd("fp16") == "nntile_flash_sdpa_bwd_cudnn_fp16"


# ---- GPU ---------------------------------------------------------------------

def _bits(t):
    import torch
    return t.view(torch.int16).numpy().view(np.uint16)


def _values(bits, dtype):
    import torch
    return H.to_np(torch.from_numpy(bits.view(np.int16).copy()).view(H.TORCH_DT[dtype]))


def _fortran5(x, head, seq, nb, grp, nkv):
    """C-ordered [batch_flat, seq, head] -> Fortran [head, seq, nb, grp, nkv]."""
    return np.asfortranarray(x.reshape(nkv, grp, nb, seq, head).transpose(4, 3, 2, 1, 0))


def _flat(x, head, seq):
    """Fortran [head, seq, nb, grp, nkv] -> C-ordered [batch_flat, seq, head]."""
    return np.ascontiguousarray(x.transpose(4, 3, 2, 1, 0)).reshape(-1, seq, head)


def _run(op, dtype, data, lse, add_mask, shape5, base5, grads0=None, mask_mode=0, offset=0):
    """data: fp32 C-ordered [batch_flat, seq, head] arrays of tile-dtype values
    for K, Q, V, A, dA.  Returns (dK, dQ, dV) the same way, and the task count."""
    head, seq, nb, grp, nkv = shape5
    T = {}
    for n in ("K", "Q", "V", "A", "dA"):
        t, _ = H.rounded(data[n], dtype)
        T[n] = hm.Tensor(dtype, shape5, base5).from_array(_fortran5(_bits(t), *shape5))
    for n in ("dK", "dQ", "dV"):
        start = np.zeros((nb * grp * nkv, seq, head), np.float32) if grads0 is None else grads0[n]
        t, _ = H.rounded(start, dtype)
        T[n] = hm.Tensor(dtype, shape5, base5).from_array(_fortran5(_bits(t), *shape5))
    L = hm.Tensor("fp32", shape5[1:], base5[1:]).from_array(
        np.asfortranarray(lse.reshape(nkv, grp, nb, seq).transpose(3, 2, 1, 0)))
    m, _ = H.rounded(add_mask, dtype)                       # [q, k] C order
    M = hm.Tensor(dtype, [seq, seq], [base5[1], base5[1]]).from_array(
        np.asfortranarray(_bits(m).T))                      # Fortran [k, q]
    before = hm.tasks_submitted_bwd(dtype)
    if op == hm.OP_HIP:
        pairs = hm.flash_sdpa_bwd(op, T["K"], T["Q"], T["V"], T["A"], T["dA"], None, L, T["dK"], T["dQ"],
                                  T["dV"], mask_mode=mask_mode, offset=offset)
    elif op == hm.OP_CLASSIFIED:
        pairs = hm.flash_sdpa_bwd(op, T["K"], T["Q"], T["V"], T["A"], T["dA"], M, L, T["dK"], T["dQ"],
                                  T["dV"], offset=offset)
    else:
        if op == hm.OP_TENSOR:
            hm.mask_declare_constant(M)     # what the layer says once after building its mask
        hm.flash_sdpa_bwd(op, T["K"], T["Q"], T["V"], T["A"], T["dA"], M, L, T["dK"], T["dQ"], T["dV"])
        pairs = hm.tasks_submitted_bwd(dtype) - before
    out = [_flat(_values(T[n].to_array(), dtype), head, seq) for n in ("dK", "dQ", "dV")]
    return out, pairs, T["dQ"].ntiles


def _reference_data(n, dtype):
    # tests/tensor/flash_sdpa_bwd_cudnn.cc:121-139: element i of every tile in
    # memory order; A and logsumexp are NOT those of a forward pass
    i = np.arange(n)
    data = {name: H.rounded((0.1 * ((i + s) % 10 - 5)).astype(np.float32), dtype)[1]
            for s, name in enumerate(("K", "Q", "V", "A", "dA"))}
    return data


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("case", [(32, 64, 64, 1, 1, 1, 1, 1, 1), (32, 128, 64, 1, 1, 1, 1, 1, 1),
                                  (64, 256, 64, 3, 1, 2, 1, 4, 2)])
def test_reference_tensor_test_multi_tile_equals_single_tile(oracle, dtype, case):
    head, seq, seq_tile, nb, nb_tile, grp, grp_tile, nkv, nkv_tile = case
    print("case host bwd", dtype, case, flush=True)
    batch = nb * grp * nkv
    shape5 = [head, seq, nb, grp, nkv]
    data = {k: v.reshape(batch, seq, head) for k, v in _reference_data(batch * seq * head, dtype).items()}
    lse = (0.1 * (np.arange(batch * seq) % 10 - 5)).astype(np.float32).reshape(batch, seq)
    i = np.arange(seq)
    add = np.where(np.abs(i[:, None] - i[None, :]) <= 32, 0.0, -np.inf).astype(np.float32)
    single, tasks1, _ = _run(hm.OP_PAIRS_BWD, dtype, data, lse, add, shape5, shape5)
    assert tasks1 == 1
    multi, tasks, ntiles = _run(hm.OP_PAIRS_BWD, dtype, data, lse, add, shape5,
                                [head, seq_tile, nb_tile, grp_tile, nkv_tile])
    # one task per (dQ tile, key tile), none skipped (src/tensor/...:172-247)
    assert tasks == ntiles * (seq // seq_tile)
    want = oracle.sdpa_bwd_flash_f64(data["K"], data["Q"], data["V"], data["A"], data["dA"], lse, add)
    for s, m, w, name in zip(single, multi, want, ("dK", "dQ", "dV")):
        # the reference's bound between the two tilings (:281-301), and each
        # against the fp64 checker
        assert np.linalg.norm(m - s) <= 1e-2 * np.linalg.norm(s), name
        assert H.rel_fro(s, w) < 1e-2, name
        assert H.rel_fro(m, w) < 1e-2, name


@pytest.mark.gpu
def test_tile_level_adds_to_the_gradients_and_reads_the_mask_as_key_by_query(oracle):
    """A mask that is not symmetric (causal) pins the [k, q] orientation of
    the mask tile; gradients that start non-zero pin the accumulation."""
    dtype, head, seq, nb, grp, nkv = "bf16", 64, 128, 2, 1, 2
    batch = nb * grp * nkv
    shape5 = [head, seq, nb, grp, nkv]
    (Q, K, V), (qf, kf, vf) = H.make_qkv(31, batch, seq, seq, head, dtype)
    _, gf = H.rounded(synth.randn(32, 0, batch * seq * head).reshape(batch, seq, head), dtype)
    mask = synth.causal_mask(seq, seq)
    add = np.where(mask, 0.0, -np.inf).astype(np.float32)
    A64, lse64 = oracle.sdpa_bruteforce_f64(kf, qf, vf, add)
    _, af = H.rounded(A64, dtype)
    lse = lse64.astype(np.float32)
    data = {"K": kf, "Q": qf, "V": vf, "A": af, "dA": gf}
    start = {n: H.rounded(0.5 * synth.randn(40 + j, 0, batch * seq * head).reshape(batch, seq, head),
                          dtype)[1] for j, n in enumerate(("dK", "dQ", "dV"))}
    got, tasks, _ = _run(hm.OP_TILE, dtype, data, lse, add, shape5, shape5, grads0=start)
    assert tasks == 1
    want = oracle.sdpa_bwd_flash_f64(kf, qf, vf, af, gf, lse, add)
    for g, w, n in zip(got, want, ("dK", "dQ", "dV")):
        assert H.rel_fro(g, w + start[n]) < 1e-2, n
    # shape errors come from the tile-level check, with the reference's text
    bad = hm.Tensor(dtype, [head, seq // 2, nb, grp, nkv], [head, seq // 2, nb, grp, nkv])
    ok = {n: hm.Tensor(dtype, shape5, shape5) for n in ("K", "V", "A", "dA", "dK", "dQ", "dV")}
    L = hm.Tensor("fp32", shape5[1:], shape5[1:])
    M = hm.Tensor(dtype, [seq, seq], [seq, seq])
    with pytest.raises(hm.HostError, match=r"K.shape != Q.shape"):
        hm.flash_sdpa_bwd(hm.OP_TILE, ok["K"], bad, ok["V"], ok["A"], ok["dA"], M, L,
                          ok["dK"], ok["dQ"], ok["dV"])
    f32 = hm.Tensor("fp32", shape5, shape5)
    with pytest.raises(hm.HostError, match="no fp32 instance"):
        hm.flash_sdpa_bwd(hm.OP_TILE, f32, f32, f32, f32, f32, f32, L, f32, f32, f32)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("mode,offset", [("causal", 0), ("causal", -70), ("none", 0)])
def test_analytic_mask_form_skips_hidden_tile_pairs(oracle, dtype, mode, offset):
    """tensor::flash_sdpa_bwd_hip_async: no mask tensor, the tile pairs a
    causal mask hides are not launched, gradients as the checker's with the
    same mask written out."""
    head, seq, tile, nb, grp, nkv = 64, 320, 64, 2, 1, 2
    batch = nb * grp * nkv
    shape5, base5 = [head, seq, nb, grp, nkv], [head, tile, 1, 1, 2]
    (Q, K, V), (qf, kf, vf) = H.make_qkv(51, batch, seq, seq, head, dtype)
    _, gf = H.rounded(synth.randn(52, 0, batch * seq * head).reshape(batch, seq, head), dtype)
    i = np.arange(seq)
    mask = (i[None, :] <= i[:, None] + offset) if mode == "causal" else np.ones((seq, seq), bool)
    add = np.where(mask, 0.0, -np.inf).astype(np.float32)
    vis = mask.any(axis=1)
    with np.errstate(all="ignore"):
        A64, lse64 = oracle.sdpa_bruteforce_f64(kf, qf, vf, add)
    A64 = np.where(vis[None, :, None], A64, 0.0)
    lse = np.where(vis[None, :], lse64, -np.inf).astype(np.float32)
    _, af = H.rounded(A64, dtype)
    data = {"K": kf, "Q": qf, "V": vf, "A": af, "dA": gf}
    got, pairs, ntiles = _run(hm.OP_HIP, dtype, data, lse, add, shape5, base5,
                              mask_mode=2 if mode == "causal" else 1, offset=offset)
    nt = seq // tile
    slabs = ntiles // nt
    if mode == "none":
        assert pairs == slabs * nt * nt
    else:
        visible_pairs = sum(1 for q in range(nt) for k in range(nt)
                            if k * tile <= q * tile + tile - 1 + offset)
        assert pairs == slabs * visible_pairs and visible_pairs < nt * nt
    with np.errstate(all="ignore"):
        want = oracle.sdpa_bwd_flash_f64(kf, qf, vf, af, gf, np.where(vis[None, :], lse, 0.0),
                                         np.where(vis[:, None], add, -np.inf))
    for g, w, n in zip(got, want, ("dK", "dQ", "dV")):
        assert H.rel_fro(g, w) < (1e-2 if dtype == "bf16" else 2e-3), n


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("kind,offset", [("causal", 0), ("causal", -70), ("window", 0), ("full", 0)])
def test_classified_submission_skips_hidden_tile_pairs(oracle, dtype, kind, offset):
    """The tensor-level overload that takes the classes of the mask's tiles:
    the gradients of the reference submission (every pair with its mask tile)
    and of the checker, with no call for pairs whose mask tile hides
    everything."""
    head, seq, tile, nb, grp, nkv = 64, 320, 64, 2, 1, 2
    batch = nb * grp * nkv
    shape5, base5 = [head, seq, nb, grp, nkv], [head, tile, 1, 1, 2]
    (Q, K, V), (qf, kf, vf) = H.make_qkv(61, batch, seq, seq, head, dtype)
    _, gf = H.rounded(synth.randn(62, 0, batch * seq * head).reshape(batch, seq, head), dtype)
    i = np.arange(seq)
    mask = {"causal": i[None, :] <= i[:, None] + offset, "window": np.abs(i[None, :] - i[:, None]) <= 90,
            "full": np.ones((seq, seq), bool)}[kind]
    add = np.where(mask, 0.0, -np.inf).astype(np.float32)
    vis = mask.any(axis=1)
    with np.errstate(all="ignore"):
        A64, lse64 = oracle.sdpa_bruteforce_f64(kf, qf, vf, add)
    A64 = np.where(vis[None, :, None], A64, 0.0)
    lse = np.where(vis[None, :], lse64, -np.inf).astype(np.float32)
    _, af = H.rounded(A64, dtype)
    data = {"K": kf, "Q": qf, "V": vf, "A": af, "dA": gf}
    got, pairs, ntiles = _run(hm.OP_CLASSIFIED, dtype, data, lse, add, shape5, base5, offset=offset)
    ref, all_pairs, _ = _run(hm.OP_PAIRS_BWD, dtype, data, lse, add, shape5, base5)
    nt = seq // tile
    slabs = ntiles // nt
    live = sum(1 for q in range(nt) for k in range(nt)
               if mask[q * tile:(q + 1) * tile, k * tile:(k + 1) * tile].any())
    assert all_pairs == slabs * nt * nt and pairs == slabs * live
    assert (live < nt * nt) == (kind != "full")
    with np.errstate(all="ignore"):
        want = oracle.sdpa_bwd_flash_f64(kf, qf, vf, af, gf, np.where(vis[None, :], lse, 0.0),
                                         np.where(vis[:, None], add, -np.inf))
    tol = 1e-2 if dtype == "bf16" else 2e-3
    for g, r, w, n in zip(got, ref, want, ("dK", "dQ", "dV")):
        assert H.rel_fro(g, w) < tol, n
        assert H.rel_fro(g, r) < tol, n
    if offset == 0:
        # the reference's signature on the mask declared constant (classified
        # against the rule key <= query) submits the same calls: same bits, and
        # only MIXED pairs as tile tasks
        dflt, tile_tasks, _ = _run(hm.OP_TENSOR, dtype, data, lse, add, shape5, base5)
        for g, d, n in zip(got, dflt, ("dK", "dQ", "dV")):
            assert np.array_equal(g, d), n
        mixed = sum(1 for q in range(nt) for k in range(nt)
                    if mask[q * tile:(q + 1) * tile, k * tile:(k + 1) * tile].any()
                    and not mask[q * tile:(q + 1) * tile, k * tile:(k + 1) * tile].all()
                    and not (kind == "causal" and q == k))
        assert tile_tasks == slabs * mixed


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("kind,offset", [("causal", 0), ("causal", -70), ("full", 0), ("window", 0)])
def test_tiles_of_128_rows_take_one_call_per_slab(oracle, dtype, kind, offset):
    """Sequence tiles that are multiples of 128 rows: a mask whose tile classes say it is the causal rule, or hides nothing,
    costs one call per slab of the batch grid instead of one per tile pair -
    through the overload that takes the classes, through the reference's own
    signature, and through the analytic form; any other mask still goes pair
    by pair.  Gradients as the checker's and as the literal submission's."""
    head, seq, tile, nb, grp, nkv = 64, 384, 128, 2, 1, 2
    batch = nb * grp * nkv
    shape5, base5 = [head, seq, nb, grp, nkv], [head, tile, 1, 1, 2]
    (Q, K, V), (qf, kf, vf) = H.make_qkv(71, batch, seq, seq, head, dtype)
    _, gf = H.rounded(synth.randn(72, 0, batch * seq * head).reshape(batch, seq, head), dtype)
    i = np.arange(seq)
    mask = {"causal": i[None, :] <= i[:, None] + offset, "window": np.abs(i[None, :] - i[:, None]) <= 150,
            "full": np.ones((seq, seq), bool)}[kind]
    add = np.where(mask, 0.0, -np.inf).astype(np.float32)
    vis = mask.any(axis=1)
    with np.errstate(all="ignore"):
        A64, lse64 = oracle.sdpa_bruteforce_f64(kf, qf, vf, add)
    A64 = np.where(vis[None, :, None], A64, 0.0)
    lse = np.where(vis[None, :], lse64, -np.inf).astype(np.float32)
    _, af = H.rounded(A64, dtype)
    data = {"K": kf, "Q": qf, "V": vf, "A": af, "dA": gf}
    start = {n: 0.25 * synth.randn(73, j, batch * seq * head).reshape(batch, seq, head)
             for j, n in enumerate(("dK", "dQ", "dV"))}
    start = {n: H.rounded(x, dtype)[1] for n, x in start.items()}
    got, calls, ntiles = _run(hm.OP_CLASSIFIED, dtype, data, lse, add, shape5, base5, grads0=start,
                              offset=offset)
    ref, all_pairs, _ = _run(hm.OP_PAIRS_BWD, dtype, data, lse, add, shape5, base5, grads0=start)
    nt = -(-seq // tile)
    slabs = ntiles // nt
    live = sum(1 for q in range(nt) for k in range(nt)
               if mask[q * tile:(q + 1) * tile, k * tile:(k + 1) * tile].any())
    assert all_pairs == slabs * nt * nt
    # (a mask on the causal rule, or none: the slabs share calls, as many as
    # the tile tables of a call hold)
    grid_calls = -(-slabs // (hip_sdpa.BWD_MAX_TILES // nt))
    assert calls == (slabs * live if kind == "window" else grid_calls)
    with np.errstate(all="ignore"):
        want = oracle.sdpa_bwd_flash_f64(kf, qf, vf, af, gf, np.where(vis[None, :], lse, 0.0),
                                         np.where(vis[:, None], add, -np.inf))
    tol = 1e-2 if dtype == "bf16" else 2e-3
    for g, r, w, n in zip(got, ref, want, ("dK", "dQ", "dV")):
        assert H.rel_fro(g, w + start[n]) < tol, n
        assert H.rel_fro(g, r) < tol, n
    if kind != "window":
        hip, hip_calls, _ = _run(hm.OP_HIP, dtype, data, lse, add, shape5, base5, grads0=start,
                                 mask_mode=2 if kind == "causal" else 1, offset=offset)
        assert hip_calls == grid_calls
        for g, d, n in zip(got, hip, ("dK", "dQ", "dV")):
            assert np.array_equal(g, d), n
    if offset == 0:
        dflt, tile_tasks, _ = _run(hm.OP_TENSOR, dtype, data, lse, add, shape5, base5, grads0=start)
        for g, d, n in zip(got, dflt, ("dK", "dQ", "dV")):
            assert np.array_equal(g, d), n
        if kind != "window":
            assert tile_tasks == 0


@pytest.mark.gpu
def test_slabs_of_unequal_size_share_calls_only_with_their_like(oracle):
    """A batch grid whose last tiles are smaller: slabs of 4, 2, 2 and 1
    entries.  Only neighbours of equal size share a call (4 | 2, 2 | 1), and
    the gradients are those of the pair-by-pair submission and the checker."""
    dtype, head, seq, tile, nb, grp, nkv = "bf16", 64, 256, 128, 3, 1, 3
    batch = nb * grp * nkv
    shape5, base5 = [head, seq, nb, grp, nkv], [head, tile, 2, 1, 2]
    (Q, K, V), (qf, kf, vf) = H.make_qkv(91, batch, seq, seq, head, dtype)
    _, gf = H.rounded(synth.randn(92, 0, batch * seq * head).reshape(batch, seq, head), dtype)
    i = np.arange(seq)
    mask = i[None, :] <= i[:, None]
    add = np.where(mask, 0.0, -np.inf).astype(np.float32)
    A64, lse64 = oracle.sdpa_bruteforce_f64(kf, qf, vf, add)
    lse = lse64.astype(np.float32)
    _, af = H.rounded(A64, dtype)
    data = {"K": kf, "Q": qf, "V": vf, "A": af, "dA": gf}
    got, calls, ntiles = _run(hm.OP_CLASSIFIED, dtype, data, lse, add, shape5, base5)
    ref, all_pairs, _ = _run(hm.OP_PAIRS_BWD, dtype, data, lse, add, shape5, base5)
    nt = seq // tile
    assert ntiles // nt == 4 and all_pairs == 4 * nt * nt
    assert calls == 3
    want = oracle.sdpa_bwd_flash_f64(kf, qf, vf, af, gf, lse, add)
    for g, r, w, n in zip(got, ref, want, ("dK", "dQ", "dV")):
        assert H.rel_fro(g, w) < 1e-2, n
        assert H.rel_fro(g, r) < 1e-2, n
