"""The C++ host mirror of the reference's tile/tensor/codelet layers.

CPU part: the shape rules and their error messages (the reference's own tests
check them with TEST_THROW, tests/tile/flash_sdpa_fwd_cudnn.cc:196-262).
GPU part: multi-tile tensors against the single-tile result and the CPU
checker, as tests/tensor/flash_sdpa_fwd_cudnn.cc:45-253 does."""
import numpy as np
import pytest

from nntile_amd import host_mirror as hm, synth
from . import helpers as H


def _specs(head=64, seq=128, nb=2, grp=1, nkv=3, tile=None, **over):
    tile = tile or seq
    s5, b5 = [head, seq, nb, grp, nkv], [head, tile, nb, grp, nkv]
    d = {"K": (list(s5), list(b5)), "Q": (list(s5), list(b5)), "mask": ([seq, seq], [tile, tile]),
         "lse": ([seq, nb, grp, nkv], [tile, nb, grp, nkv]), "V": (list(s5), list(b5)),
         "A": (list(s5), list(b5))}
    for k, v in over.items():
        d[k] = v
    return [d[k] for k in ("K", "Q", "mask", "lse", "V", "A")]


def test_shape_rules_accept_the_reference_cases():
    # tests/tensor/flash_sdpa_fwd_cudnn.cc:244-246
    hm.check_shapes(0, _specs(32, 64, 64, 1, 1))
    hm.check_shapes(1, _specs(128, 256, 2, 1, 2, tile=128))
    hm.check_shapes(1, [([32, 512, 4, 3, 4], [32, 64, 4, 1, 2]), ([32, 512, 4, 3, 4], [32, 64, 4, 1, 2]),
                        ([512, 512], [64, 64]), ([512, 4, 3, 4], [64, 4, 1, 2]),
                        ([32, 512, 4, 3, 4], [32, 64, 4, 1, 2]), ([32, 512, 4, 3, 4], [32, 64, 4, 1, 2])])


@pytest.mark.parametrize("level", [0, 1])
@pytest.mark.parametrize("change,message", [
    ({"K": ([64, 128, 2, 1], [64, 128, 2, 1])}, "K.ndim != 5"),
    ({"mask": ([128, 128, 1], [128, 128, 1])}, "mask.ndim != 2"),
    ({"lse": ([128, 2, 1, 3, 1], [128, 2, 1, 3, 1])}, "logsumexp.ndim != 4"),
    ({"Q": ([32, 128, 2, 1, 3], [32, 128, 2, 1, 3])}, "K.shape[0] != Q.shape[0]"),
    ({"V": ([64, 64, 2, 1, 3], [64, 64, 2, 1, 3])}, "K.shape[1] != V.shape[1]"),
    ({"A": ([64, 128, 4, 1, 3], [64, 128, 4, 1, 3])}, "K.shape[2] != A.shape[2]"),
    ({"lse": ([128, 2, 1, 5], [128, 2, 1, 5])}, "K.shape[4] != logsumexp.shape[3]"),
])
def test_shape_rules_reject_with_reference_messages(level, change, message):
    with pytest.raises(hm.HostError) as e:
        hm.check_shapes(level, _specs(**change))
    assert str(e.value) == message


def test_tile_level_needs_square_tiles_tensor_level_names_the_axis():
    bad = _specs(mask=([64, 128], [64, 128]))
    with pytest.raises(hm.HostError, match=r"K.shape\[1\] != mask.shape\[0\]"):
        hm.check_shapes(0, bad)
    with pytest.raises(hm.HostError, match="K sequence dimension must match mask axis 0"):
        hm.check_shapes(1, bad)


@pytest.mark.parametrize("change,message", [
    ({"K": ([64, 128, 2, 1, 3], [32, 128, 2, 1, 3])}, "K and Q basetile shapes mismatch"),
    ({"A": ([64, 128, 2, 1, 3], [64, 64, 2, 1, 3])}, "Q and A basetile shapes must match"),
    ({"mask": ([128, 128], [64, 128])}, "mask basetile axis 0 must match K basetile sequence dimension"),
    ({"lse": ([128, 2, 1, 3], [128, 1, 1, 3])},
     "logsumexp basetile shape must match Q basetile shape (excluding head dimension)"),
])
def test_tensor_level_basetile_rules(change, message):
    with pytest.raises(hm.HostError) as e:
        hm.check_shapes(1, _specs(**change))
    assert str(e.value) == message


def test_head_axis_must_not_be_tiled():
    s = ([64, 128, 2, 1, 3], [32, 128, 2, 1, 3])
    with pytest.raises(hm.HostError, match="head dimension must not be tiled"):
        hm.check_shapes(1, _specs(K=s, Q=s, V=s, A=s))


def test_footprint_and_codelet_names():
    # equal sizes <=> equal footprint (src/starpu/flash_sdpa_fwd_cudnn.cc:159-179)
    assert hm.footprint(1024, 128, 32) == hm.footprint(1024, 128, 32)
    seen = {hm.footprint(s, h, b) for s in (64, 128, 1024) for h in (32, 64, 128) for b in (1, 8, 32)}
    assert len(seen) == 27
    assert hm.codelet_name("bf16") == "nntile_flash_sdpa_fwd_cudnn_bf16"
    assert hm.codelet_name("fp32") == "nntile_flash_sdpa_fwd_cudnn_fp32"


# ---- GPU ---------------------------------------------------------------------

def _fortran5(x, head, seq, nb, grp, nkv):
    """C-ordered [batch_flat, seq, head] -> Fortran [head, seq, nb, grp, nkv]."""
    return np.asfortranarray(x.reshape(nkv, grp, nb, seq, head).transpose(4, 3, 2, 1, 0))


def _case(dtype, head, seq, nb, grp, nkv, seed=5):
    batch = nb * grp * nkv
    (Q, K, V), f32 = H.make_qkv(seed, batch, seq, seq, head, dtype)
    store = (lambda t: t.numpy()) if dtype == "fp32" else (lambda t: t.view(__import__("torch").int16).numpy().view(np.uint16))
    arrs = {n: _fortran5(store(t), head, seq, nb, grp, nkv) for n, t in (("Q", Q), ("K", K), ("V", V))}
    return arrs, f32


def _run(dtype, arrs, mask_bool, head, seq, nb, grp, nkv, tile, op, **kw):
    s5 = [head, seq, nb, grp, nkv]
    b5 = [head, tile, max(1, nb // 2), 1, max(1, nkv // 2)]     # the batch axes are tiled too
    T = {n: hm.Tensor(dtype, s5, b5).from_array(arrs[n]) for n in ("K", "Q", "V")}
    A = hm.Tensor(dtype, s5, b5).from_array(np.zeros(s5, np.float32 if dtype == "fp32" else np.uint16))
    lse = hm.Tensor("fp32", s5[1:], b5[1:]).from_array(np.full(s5[1:], -np.inf, np.float32))
    mask = None
    if op != hm.OP_HIP:     # (OP_TENSOR, OP_PAIRS: a materialised additive mask)
        add = np.where(mask_bool, 0.0, -np.inf).astype(np.float32).T       # [k_seq, q_seq] Fortran
        m_t, _ = H.rounded(add, dtype)
        m_np = m_t.numpy() if dtype == "fp32" else m_t.view(__import__("torch").int16).numpy().view(np.uint16)
        mask = hm.Tensor(dtype, [seq, seq], [tile, tile]).from_array(np.asfortranarray(m_np))
    if op == hm.OP_TENSOR and kw.pop("declare", True):
        # what the layer says once after building its mask
        hm.mask_declare_constant(mask)
    before = hm.tasks_submitted(dtype)
    hm.flash_sdpa_fwd(op, T["K"], T["Q"], mask, lse, T["V"], A, **kw)
    a = A.to_array()
    if dtype != "fp32":
        a = H.to_np(__import__("torch").from_numpy(a.view(np.int16).copy()).view(H.TORCH_DT[dtype]))
    back = lambda x: np.ascontiguousarray(x.transpose(4, 3, 2, 1, 0)).reshape(-1, seq, head)
    lse_np = np.ascontiguousarray(lse.to_array().transpose(3, 2, 1, 0)).reshape(-1, seq)
    return back(a), lse_np, hm.tasks_submitted(dtype) - before, A.ntiles


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("head,seq,nb,grp,nkv,tile", [(32, 64, 2, 1, 2, 64), (128, 256, 2, 1, 2, 128),
                                                     (32, 512, 4, 3, 4, 64), (64, 200, 2, 1, 2, 96),
                                                     # batch tiles of 2, 2 and 1 entries: slabs of unequal size
                                                     (64, 256, 5, 1, 3, 128)])
def test_tensor_level_tiles_match_oracle(oracle, dtype, head, seq, nb, grp, nkv, tile):
    arrs, (qf, kf, vf) = _case(dtype, head, seq, nb, grp, nkv)
    mask = synth.causal_mask(seq, seq)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, k_tile=tile)
    if seq % tile == 0:
        got, got_lse, tasks, ntiles = _run(dtype, arrs, mask, head, seq, nb, grp, nkv, tile, hm.OP_PAIRS)
        # one task per (output tile, key tile), none skipped (src/tensor/...:221-274)
        assert tasks == ntiles * (seq // tile)
        assert H.rel_fro(got, want) < H.TOL[dtype] and H.rel_fro(got_lse, want_lse) < H.TOL[dtype]
        # the reference's signature on a mask declared constant: its tiles were
        # classified at the declaration, a causal mask needs no tile tasks at all
        got, got_lse, tasks, ntiles = _run(dtype, arrs, mask, head, seq, nb, grp, nkv, tile, hm.OP_TENSOR)
        assert tasks == 0
        assert H.rel_fro(got, want) < H.TOL[dtype] and H.rel_fro(got_lse, want_lse) < H.TOL[dtype]
        # ... and on a mask nothing was said about: the reference's submission
        got, got_lse, tasks, ntiles = _run(dtype, arrs, mask, head, seq, nb, grp, nkv, tile,
                                           hm.OP_TENSOR, declare=False)
        assert tasks == ntiles * (seq // tile)
        assert H.rel_fro(got, want) < H.TOL[dtype] and H.rel_fro(got_lse, want_lse) < H.TOL[dtype]
    # the single-launch path on the same tiling, ragged last tile included
    got, got_lse, tasks, _ = _run(dtype, arrs, mask, head, seq, nb, grp, nkv, tile, hm.OP_HIP,
                                  mask_mode=2, offset=0, overwrite=True)
    assert tasks == 0
    assert H.rel_fro(got, want) < H.TOL[dtype] and H.rel_fro(got_lse, want_lse) < H.TOL[dtype]


@pytest.mark.gpu
def test_tile_level_entry_and_its_errors(oracle):
    head, seq, nb, grp, nkv = 64, 128, 2, 1, 2
    arrs, (qf, kf, vf) = _case("bf16", head, seq, nb, grp, nkv)
    mask = np.abs(np.arange(seq)[:, None] - np.arange(seq)[None, :]) <= 32   # tests/tile/...:57-86
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask)
    s5 = [head, seq, nb, grp, nkv]
    T = {n: hm.Tensor("bf16", s5, s5).from_array(arrs[n]) for n in ("K", "Q", "V")}
    A = hm.Tensor("bf16", s5, s5).from_array(np.zeros(s5, np.uint16))
    lse = hm.Tensor("fp32", s5[1:], s5[1:]).from_array(np.full(s5[1:], -np.inf, np.float32))
    import torch
    m = H.additive_mask(mask, "bf16").view(torch.int16).numpy().view(np.uint16).T
    M = hm.Tensor("bf16", [seq, seq], [seq, seq]).from_array(np.asfortranarray(m))
    hm.flash_sdpa_fwd(hm.OP_TILE, T["K"], T["Q"], M, lse, T["V"], A)
    a = H.to_np(torch.from_numpy(A.to_array().view(np.int16).copy()).view(torch.bfloat16))
    got = np.ascontiguousarray(a.transpose(4, 3, 2, 1, 0)).reshape(-1, seq, head)
    got_lse = np.ascontiguousarray(lse.to_array().transpose(3, 2, 1, 0)).reshape(-1, seq)
    assert H.rel_fro(got, want) < 1e-2 and H.rel_fro(got_lse, want_lse) < 1e-2
    bad = hm.Tensor("bf16", [head, seq // 2, nb, grp, nkv], [head, seq // 2, nb, grp, nkv])
    with pytest.raises(hm.HostError, match=r"K.shape\[1\] != Q.shape\[1\]"):
        hm.flash_sdpa_fwd(hm.OP_TILE, T["K"], bad, M, lse, T["V"], A)


# ---- the reference's signature and what it learns about its mask ---------------

def _mask_tensor(dtype, mask_bool, tile, values=None):
    import torch
    seq = mask_bool.shape[0]
    add = np.where(mask_bool, 0.0, -np.inf).astype(np.float32) if values is None else values
    m_t, _ = H.rounded(add.T, dtype)                        # [k_seq, q_seq]
    m_np = m_t.numpy() if dtype == "fp32" else m_t.view(torch.int16).numpy().view(np.uint16)
    return np.asfortranarray(m_np), hm.Tensor(dtype, [seq, seq], [tile, tile])


def _outputs(dtype, s5, b5):
    A = hm.Tensor(dtype, s5, b5).from_array(np.zeros(s5, np.float32 if dtype == "fp32" else np.uint16))
    lse = hm.Tensor("fp32", s5[1:], b5[1:]).from_array(np.full(s5[1:], -np.inf, np.float32))
    return A, lse


def _read_out(dtype, A, lse, head, seq):
    import torch
    a = A.to_array()
    if dtype != "fp32":
        a = H.to_np(torch.from_numpy(a.view(np.int16).copy()).view(H.TORCH_DT[dtype]))
    got = np.ascontiguousarray(a.transpose(4, 3, 2, 1, 0)).reshape(-1, seq, head)
    got_lse = np.ascontiguousarray(lse.to_array().transpose(3, 2, 1, 0)).reshape(-1, seq)
    return got, got_lse


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_reference_signature_uses_the_classes_of_a_declared_mask_and_drops_them_on_a_write(oracle, dtype):
    head, seq, nb, grp, nkv, tile = 64, 256, 2, 1, 2, 64
    arrs, (qf, kf, vf) = _case(dtype, head, seq, nb, grp, nkv, seed=21)
    s5, b5 = [head, seq, nb, grp, nkv], [head, tile, 1, 1, 1]
    T = {n: hm.Tensor(dtype, s5, b5).from_array(arrs[n]) for n in ("K", "Q", "V")}
    causal = synth.causal_mask(seq, seq)
    i = np.arange(seq)
    window = np.abs(i[None, :] - i[:, None]) <= 40
    n_t = seq // tile
    slabs = nb * grp * nkv
    every_pair = slabs * n_t * n_t

    def run(M, mask_bool):
        """(tile tasks, look-ups that found classes, look-ups that did not,
        blocking classifications) of one call with the reference's signature"""
        A, lse = _outputs(dtype, s5, b5)
        tasks0, (h0, m0), c0 = hm.tasks_submitted(dtype), hm.mask_cache_stats(), hm.mask_classifications()
        hm.flash_sdpa_fwd(hm.OP_TENSOR, T["K"], T["Q"], M, lse, T["V"], A)
        (h1, m1), c1 = hm.mask_cache_stats(), hm.mask_classifications()
        got, got_lse = _read_out(dtype, A, lse, head, seq)
        want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask_bool, k_tile=tile)
        assert H.rel_fro(got, want) < H.TOL[dtype] and H.rel_fro(got_lse, want_lse) < H.TOL[dtype]
        return hm.tasks_submitted(dtype) - tasks0, h1 - h0, m1 - m0, c1 - c0

    arr, M = _mask_tensor(dtype, causal, tile)
    M.from_array(arr)
    # nothing said about the mask: the reference's submission, and the call
    # never classifies anything itself
    assert run(M, causal) == (every_pair, 0, 1, 0)
    # declared constant: classified once, there and then; the causal rule needs
    # no tile tasks, one task of the whole-grid codelet instead (all slabs have
    # the same extents)
    c0 = hm.mask_classifications()
    hm.mask_declare_constant(M)
    assert hm.mask_classifications() - c0 == 1
    grid0 = hm.grid_tasks_submitted(dtype)
    assert run(M, causal) == (0, 1, 0, 0)
    assert hm.grid_tasks_submitted(dtype) - grid0 == 1
    assert hm.grid_codelet_name(dtype) == "nntile_sdpa_fwd_grid_hip_" + dtype
    assert run(M, causal) == (0, 1, 0, 0)
    # the mask is rewritten through the runtime with a window: the classes are
    # dropped with the write, the call goes back to the reference's submission
    # and follows the new contents
    arr_w, _ = _mask_tensor(dtype, window, tile)
    M.from_array(arr_w)
    assert run(M, window) == (every_pair, 0, 1, 0)
    # declared again: pairs the window hides are not submitted, the others take
    # the tile path (their tiles are MIXED) or the open path
    hm.mask_declare_constant(M)
    tasks, hits, misses, classified = run(M, window)
    assert (hits, misses, classified) == (1, 0, 0)
    live = sum(1 for q in range(n_t) for k in range(n_t)
               if window[q * tile:(q + 1) * tile, k * tile:(k + 1) * tile].any())
    mixed = sum(1 for q in range(n_t) for k in range(n_t)
                if window[q * tile:(q + 1) * tile, k * tile:(k + 1) * tile].any()
                and not window[q * tile:(q + 1) * tile, k * tile:(k + 1) * tile].all())
    assert live < n_t * n_t and 0 < tasks <= slabs * mixed
    # a writer got the tiles (same contents): dropped again
    M.mark_written()
    assert run(M, window)[1:] == (0, 1, 0)
    # forgotten on request
    hm.mask_declare_constant(M)
    assert run(M, window)[1:] == (1, 0, 0)
    hm.mask_forget(M)
    assert run(M, window) == (every_pair, 0, 1, 0)
    # another tensor, freed and re-created in between (its memory may be
    # the one the freed tensor had): never served from the old entry
    hm.mask_declare_constant(M)
    for mask_bool in (window, causal, window):
        arr2, M2 = _mask_tensor(dtype, mask_bool, tile)
        M2.from_array(arr2)
        assert run(M2, mask_bool)[1:] == (0, 1, 0)
        hm.mask_declare_constant(M2)
        assert run(M2, mask_bool)[1:] == (1, 0, 0)
        del M2


@pytest.mark.gpu
def test_a_mask_rewritten_behind_the_runtimes_back_is_honoured(oracle):
    """The mask's tiles are overwritten by a kernel the runtime knows nothing
    about (the transpose kernel of the C ABI, launched by the test on the
    tiles' device addresses): the next call with the reference's signature
    reads the mask as it then is, because an undeclared mask is never
    classified ahead of time."""
    import ctypes
    import torch
    from nntile_amd import hip_sdpa
    dtype, head, seq, nb, grp, nkv, tile = "bf16", 64, 256, 2, 1, 2, 128
    arrs, (qf, kf, vf) = _case(dtype, head, seq, nb, grp, nkv, seed=23)
    s5, b5 = [head, seq, nb, grp, nkv], [head, tile, 1, 1, 1]
    T = {n: hm.Tensor(dtype, s5, b5).from_array(arrs[n]) for n in ("K", "Q", "V")}
    causal = synth.causal_mask(seq, seq)
    i = np.arange(seq)
    window = np.abs(i[None, :] - i[:, None]) <= 40
    arr, M = _mask_tensor(dtype, causal, tile)
    M.from_array(arr)

    def run(mask_bool):
        A, lse = _outputs(dtype, s5, b5)
        hm.flash_sdpa_fwd(hm.OP_TENSOR, T["K"], T["Q"], M, lse, T["V"], A)
        got, got_lse = _read_out(dtype, A, lse, head, seq)
        want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask_bool, k_tile=tile)
        return H.rel_fro(got, want), H.rel_fro(got_lse, want_lse)

    assert max(run(causal)) < H.TOL[dtype]
    # tile (kt, qt) of the mask is Fortran [k, q] = the transpose of the C-ordered
    # [k, q] block the test builds; dst = 1.0 * src^T writes it in place
    add = np.where(window, 0.0, -np.inf).astype(np.float32)          # [q, k]
    n_t = seq // tile
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # (the calls above are blocking: nothing of the runtime's is in flight)
    keep = []
    for qt in range(n_t):
        for kt in range(n_t):
            block = add[qt * tile:(qt + 1) * tile, kt * tile:(kt + 1) * tile]    # [q, k]
            src = torch.from_numpy(np.ascontiguousarray(block.T)).to(torch.bfloat16).cuda()   # C [k, q]
            ptr, nbytes = hm.tile_ptr(M, kt + qt * n_t)
            assert nbytes == tile * tile * 2
            # src as Fortran [q, k] (m = q, n = k) -> dst Fortran [k, q]
            rc = hip_sdpa.lib().nntile_hip_transpose_bf16(stream, tile, tile, ctypes.c_float(1.0),
                                                          ctypes.c_void_p(src.data_ptr()),
                                                          ctypes.c_void_p(ptr))
            assert rc == 0
            keep.append(src)
    torch.cuda.synchronize()
    assert max(run(window)) < H.TOL[dtype]
    # the same write behind a DECLARED mask breaks the caller's contract, and
    # the caller's remedy is to say so before writing: forget, write, declare
    hm.mask_declare_constant(M)
    assert max(run(window)) < H.TOL[dtype]


@pytest.mark.gpu
def test_reference_signature_with_a_bias_mask_is_the_reference_submission_bit_for_bit():
    dtype, head, seq, nb, grp, nkv, tile = "bf16", 64, 256, 2, 1, 2, 128
    arrs, _ = _case(dtype, head, seq, nb, grp, nkv, seed=22)
    s5, b5 = [head, seq, nb, grp, nkv], [head, tile, 1, 1, 1]
    i = np.arange(seq)
    bias = (-0.25 * np.abs(i[:, None] - i[None, :]) - 0.25).astype(np.float32)
    outs = []
    for declare, op in ((False, hm.OP_PAIRS), (False, hm.OP_TENSOR), (True, hm.OP_TENSOR)):
        T = {n: hm.Tensor(dtype, s5, b5).from_array(arrs[n]) for n in ("K", "Q", "V")}
        arr, M = _mask_tensor(dtype, np.ones((seq, seq), bool), tile, values=bias)
        M.from_array(arr)
        if declare:
            hm.mask_declare_constant(M)
        A, lse = _outputs(dtype, s5, b5)
        before = hm.tasks_submitted(dtype)
        hm.flash_sdpa_fwd(op, T["K"], T["Q"], M, lse, T["V"], A)
        # every pair is a tile task with its mask tile, in both forms
        assert hm.tasks_submitted(dtype) - before == A.ntiles * (seq // tile)
        outs.append((A.to_array().copy(), lse.to_array().copy()))
    for a, l in outs[1:]:
        assert np.array_equal(outs[0][0], a) and np.array_equal(outs[0][1], l)
