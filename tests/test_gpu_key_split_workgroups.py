"""The 16-bit prefill kernel with the key steps of a workgroup's 128 queries
split over two groups of four wavefronts (NNTILE_HIP_SDPA_FORM_SPLIT; what a
launch of at most one workgroup per CU takes by itself) against the checker
and beside the four-wavefront form of the same call.  The two groups see
different keys, so their partial softmaxes are combined at the end and the
result agrees with the other form within the tolerance, not bit for bit."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from . import helpers as H

pytestmark = pytest.mark.gpu


def _tiles(x, step):
    return [x[:, s:s + step].contiguous().cuda() for s in range(0, x.shape[1], step)]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("head", [64, 128])
@pytest.mark.parametrize("q_seq,k_seq,q_tile,k_tile,n_batch,group,n_kv,causal", [
    (256, 1024, 256, 1024, 2, 1, 2, False),     # 16 steps: both groups in the pipelined loop
    (256, 1088, 256, 1088, 1, 1, 2, False),     # 17 steps: the second group idles through the last round
    (128, 64, 128, 64, 1, 1, 3, False),         # one step: the second group has nothing at all
    (130, 128, 130, 128, 1, 1, 2, False),       # one step each
    (200, 333, 200, 333, 2, 2, 1, False),       # ragged last step (in the second group's hands), GQA
    (300, 397, 300, 397, 1, 1, 2, False),       # ragged last step in the first group's
    (512, 512, 512, 512, 2, 1, 2, True),        # causal: diagonal steps in both groups
    (1000, 1000, 384, 320, 1, 2, 2, True),      # ragged tiles, key tiles that are not whole steps
    (300, 700, 300, 256, 2, 1, 1, True),        # rectangular with an offset, several key tiles
    (64, 4160, 64, 4160, 1, 1, 2, True),        # 65 steps
])
def test_key_split_workgroups(oracle, dtype, head, q_seq, k_seq, q_tile, k_tile, n_batch, group,
                              n_kv, causal):
    print("case", dtype, head, q_seq, k_seq, q_tile, k_tile, n_batch, group, n_kv, causal, flush=True)
    batch = n_batch * group * n_kv
    offset = k_seq - q_seq
    (Q, K, V), (qf, kf, vf) = H.make_qkv(71, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    mask = synth.causal_mask(q_seq, k_seq, offset) if causal else None
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, k_tile=k_tile, n_batch=n_batch,
                                         kv_repeat=group)
    mode = hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE
    Kt, Vt, Qt = _tiles(K, k_tile), _tiles(V, k_tile), _tiles(Q, q_tile)
    outs = {}
    for name, flags in (("four", hip_sdpa.FORM_SHARED), ("split", hip_sdpa.FORM_SPLIT),
                        ("split_overwrite", hip_sdpa.FORM_SPLIT | hip_sdpa.OVERWRITE),
                        ("split_again", hip_sdpa.FORM_SPLIT)):
        o = [H.fresh_outputs(batch, t.shape[1], head, dtype) for t in Qt]
        hip_sdpa.sdpa_fwd_grid(Kt, Qt, [x[0] for x in o], Vt, [x[1] for x in o], q_seq, k_seq, q_tile,
                               k_tile, mode, n_batch=n_batch, kv_group=group, causal_offset=offset,
                               flags=flags)
        torch.cuda.synchronize()
        outs[name] = (np.concatenate([H.to_np(x[1]) for x in o], axis=1),
                      np.concatenate([H.to_np(x[0]) for x in o], axis=1))
    for name, (A, lse) in outs.items():
        assert H.rel_fro(A, want) < H.TOL[dtype], name
        assert H.rel_fro(lse, want_lse) < H.TOL[dtype], name
        H.check_rows(A, want, lse, want_lse, dtype, name)
    assert H.rel_fro(outs["split"][0], outs["four"][0]) < H.TOL[dtype]
    # no dependence on timing, and the overwrite flag changes nothing here
    assert np.array_equal(outs["split"][0], outs["split_again"][0])
    assert np.array_equal(outs["split"][1], outs["split_again"][1])
    assert np.array_equal(outs["split"][0], outs["split_overwrite"][0])
    assert np.array_equal(outs["split"][1], outs["split_overwrite"][1])


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("form", ["additive", "bool"])
@pytest.mark.parametrize("head", [64, 128])
@pytest.mark.parametrize("q_seq,k_seq,pattern", [
    (256, 1024, "causal"), (200, 712, "band"), (128, 520, "holes"), (130, 333, "band"),
    (130, 1001, "causal"), (256, 1024, "all_open"), (128, 576, "all_hidden"), (130, 4232, "band")])
def test_key_split_with_masks_given_as_values(oracle, dtype, form, head, q_seq, k_seq, pattern):
    """Scan of the mask rows, open leading steps in the pipelined loop, mixed
    and hidden steps, ragged rows: every path of the explicit masks with the
    steps dealt to two groups."""
    print("case", dtype, form, head, q_seq, k_seq, pattern, flush=True)
    batch = 3
    i = np.arange(q_seq)[:, None]
    j = np.arange(k_seq)[None, :]
    if pattern == "causal":
        mask = j <= i + (k_seq - q_seq)
    elif pattern == "band":
        mask = j <= (k_seq // 3 + 2 * i)
    elif pattern == "holes":
        mask = ((j < 100) | (j >= 300)) & (i % 50 != 49)
    elif pattern == "all_hidden":
        mask = np.zeros((q_seq, k_seq), bool)
    else:
        mask = np.ones((q_seq, k_seq), bool)
    mask = np.ascontiguousarray(np.broadcast_to(mask, (q_seq, k_seq)))
    (Q, K, V), f32 = H.make_qkv(73, batch, q_seq, k_seq, head, dtype)
    qf, kf, vf = f32
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask)
    m = (H.additive_mask(mask, dtype) if form == "additive" else torch.from_numpy(mask.copy())).cuda()
    mode = hip_sdpa.MASK_ADDITIVE if form == "additive" else hip_sdpa.MASK_BOOL
    vis = mask.any(axis=1)
    got = {}
    for name, flags in (("four", hip_sdpa.FORM_SHARED | hip_sdpa.OVERWRITE),
                        ("split", hip_sdpa.FORM_SPLIT | hip_sdpa.OVERWRITE)):
        lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
        hip_sdpa.sdpa_fwd_tile(K.cuda(), Q.cuda(), m, lse, V.cuda(), A, mode, flags=flags)
        torch.cuda.synchronize()
        a, l = H.to_np(A), H.to_np(lse)
        assert np.all(a[:, ~vis] == 0) and np.all(np.isneginf(l[:, ~vis])), name
        if vis.any():
            assert H.rel_fro(a[:, vis], want[:, vis]) < H.TOL[dtype], name
            assert H.rel_fro(l[:, vis], want_lse[:, vis]) < H.TOL[dtype], name
        got[name] = a
    if vis.any():
        assert H.rel_fro(got["split"][:, vis], got["four"][:, vis]) < H.TOL[dtype]


def test_key_split_merges_into_a_running_pair(oracle):
    """Key tiles one call at a time through the tile entry point, each call's
    two groups merged first and then into the running pair."""
    dtype, head, seq, k_tile, batch = "bf16", 128, 640, 320, 2
    (Q, K, V), (qf, kf, vf) = H.make_qkv(72, batch, seq, seq, head, dtype)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, synth.causal_mask(seq, seq), k_tile=k_tile)
    lse, A = H.fresh_outputs(batch, seq, head, dtype)
    for i, (kt, vt) in enumerate(zip(_tiles(K, k_tile), _tiles(V, k_tile))):
        hip_sdpa.sdpa_fwd_tile(kt, Q.cuda(), None, lse, vt, A, hip_sdpa.MASK_CAUSAL,
                               k_pos0=i * k_tile, flags=hip_sdpa.FORM_SPLIT)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
