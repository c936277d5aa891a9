"""The 16-bit prefill kernel with workgroups of 256 queries (eight wavefronts
sharing every K/V step, NNTILE_HIP_SDPA_FORM_WIDE) against the checker and
beside the 128-query form of the same call.  (Which key steps of a query run
in the pipelined loop depends on the first query of its workgroup, so the two
forms round differently and agree within the tolerance, not bit for bit.)"""
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
    (512, 512, 512, 512, 2, 1, 2, True),        # one tile, whole 256-query blocks
    (768, 768, 256, 256, 1, 1, 2, True),        # a tile is one block
    (1000, 1000, 384, 320, 1, 2, 2, True),      # ragged tiles, blocks with fewer than 256 rows, GQA
    (300, 700, 300, 256, 2, 1, 1, True),        # rectangular with an offset
    (520, 260, 520, 260, 3, 1, 1, False),       # no mask, ragged last key step
    (130, 64, 130, 64, 1, 1, 3, False),
])
def test_wide_workgroups(oracle, dtype, head, q_seq, k_seq, q_tile, k_tile, n_batch, group, n_kv,
                         causal):
    print("case", dtype, head, q_seq, k_seq, q_tile, k_tile, n_batch, group, n_kv, causal, flush=True)
    batch = n_batch * group * n_kv
    offset = k_seq - q_seq
    (Q, K, V), (qf, kf, vf) = H.make_qkv(61, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    mask = synth.causal_mask(q_seq, k_seq, offset) if causal else None
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, k_tile=k_tile, n_batch=n_batch,
                                         kv_repeat=group)
    mode = hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE
    Kt, Vt, Qt = _tiles(K, k_tile), _tiles(V, k_tile), _tiles(Q, q_tile)
    outs = {}
    for name, flags in (("narrow", hip_sdpa.FORM_SHARED), ("wide", hip_sdpa.FORM_WIDE),
                        ("wide_overwrite", hip_sdpa.FORM_WIDE | hip_sdpa.OVERWRITE)):
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
    assert H.rel_fro(outs["wide"][0], outs["narrow"][0]) < H.TOL[dtype]
    assert np.array_equal(outs["wide"][0], outs["wide_overwrite"][0])
    assert np.array_equal(outs["wide"][1], outs["wide_overwrite"][1])


def test_wide_workgroups_merge_into_a_running_pair(oracle):
    """Key tiles one call at a time through the tile entry point, merged into
    the running pair."""
    dtype, head, seq, k_tile, batch = "bf16", 128, 640, 256, 2
    (Q, K, V), (qf, kf, vf) = H.make_qkv(62, batch, seq, seq, head, dtype)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, synth.causal_mask(seq, seq), k_tile=k_tile)
    lse, A = H.fresh_outputs(batch, seq, head, dtype)
    for i, (kt, vt) in enumerate(zip(_tiles(K, k_tile), _tiles(V, k_tile))):
        hip_sdpa.sdpa_fwd_tile(kt, Q.cuda(), None, lse, vt, A, hip_sdpa.MASK_CAUSAL,
                               k_pos0=i * k_tile, flags=hip_sdpa.FORM_WIDE)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
