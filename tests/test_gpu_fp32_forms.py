"""The two workgroup shapes of the fp32 prefill kernel (128 queries sharing
every key step; 32 queries whose wavefronts split the key steps), each forced
with its flag on shapes where the launcher would pick the other, against the
CPU composition - the size of a launch decides the shape, so most small test
shapes would otherwise only ever see one of them."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from tests import helpers as H

pytestmark = pytest.mark.gpu

FORMS = {"shared": hip_sdpa.FORM_SHARED, "split": hip_sdpa.FORM_SPLIT}


@pytest.mark.parametrize("form", ["shared", "split"])
@pytest.mark.parametrize("head", [32, 64, 128])
@pytest.mark.parametrize("mode", ["causal", "none", "additive", "bool"])
@pytest.mark.parametrize("batch,q_seq,k_seq", [(3, 200, 200), (2, 128, 333), (5, 70, 96), (1, 257, 64)])
def test_tile_call_in_both_forms(oracle, form, head, mode, batch, q_seq, k_seq):
    print("case", form, head, mode, batch, q_seq, k_seq, flush=True)
    offset = k_seq - q_seq
    (Q, K, V), f32 = H.make_qkv(31, batch, q_seq, k_seq, head, "fp32")
    if mode == "none":
        mask_bool = None
    elif mode == "causal":
        mask_bool = synth.causal_mask(q_seq, k_seq, offset)
    else:       # a window with a few rows that see nothing
        q, k = np.arange(q_seq)[:, None], np.arange(k_seq)[None, :]
        mask_bool = (np.abs(k - q - offset) <= 40) & (q % 17 != 3)
    want, want_lse = oracle.sdpa_vanilla(f32[1], f32[0], f32[2], mask_bool)
    m, mm = {"none": (None, hip_sdpa.MASK_NONE), "causal": (None, hip_sdpa.MASK_CAUSAL),
             "additive": (None if mask_bool is None else H.additive_mask(mask_bool, "fp32").cuda(),
                          hip_sdpa.MASK_ADDITIVE),
             "bool": (None if mask_bool is None else torch.from_numpy(mask_bool).cuda(),
                      hip_sdpa.MASK_BOOL)}[mode]
    lse, A = H.fresh_outputs(batch, q_seq, head, "fp32")
    hip_sdpa.sdpa_fwd_tile(K.cuda(), Q.cuda(), m, lse, V.cuda(), A, mm, causal_offset=offset,
                           flags=FORMS[form])
    torch.cuda.synchronize()
    got, got_lse = H.to_np(A), H.to_np(lse)
    # rows without a visible key keep what they had (lse -inf, A poisoned)
    dead = np.isneginf(want_lse)
    assert np.array_equal(np.isneginf(got_lse), dead)
    got = np.where(dead[..., None], 0.0, got)
    want = np.where(dead[..., None], 0.0, want)
    assert H.rel_fro(got, want) < 1e-4
    assert H.rel_fro(got_lse, want_lse) < 1e-4


@pytest.mark.parametrize("form", ["shared", "split"])
def test_grid_call_in_both_forms_merges_into_the_running_pair(oracle, form):
    """Two key tiles in two calls (the second merges), ragged tiles, several
    slabs: the hand-off between calls is the same in both forms."""
    head, batch, n_slabs, q_seq, k_seq, q_tile, k_tile = 64, 2, 3, 300, 300, 128, 160
    mask = synth.causal_mask(q_seq, k_seq)
    Kt, Vt, Qt, outs, want = [], [], [], [], []
    for s in range(n_slabs):
        (Q, K, V), f32 = H.make_qkv(40 + s, batch, q_seq, k_seq, head, "fp32")
        want.append(oracle.sdpa_vanilla(f32[1], f32[0], f32[2], mask, k_tile=k_tile))
        tiles = lambda x, step: [x[:, i:i + step].contiguous().cuda() for i in range(0, x.shape[1], step)]
        Kt += tiles(K, k_tile)
        Vt += tiles(V, k_tile)
        q = tiles(Q, q_tile)
        Qt += q
        outs += [H.fresh_outputs(batch, t.shape[1], head, "fp32") for t in q]
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in outs], Vt, [o[1] for o in outs], q_seq, k_seq,
                           q_tile, k_tile, hip_sdpa.MASK_CAUSAL, n_slabs=n_slabs, flags=FORMS[form])
    torch.cuda.synchronize()
    n_q = len(Qt) // n_slabs
    for s in range(n_slabs):
        A = np.concatenate([H.to_np(o[1]) for o in outs[s * n_q:(s + 1) * n_q]], axis=1)
        lse = np.concatenate([H.to_np(o[0]) for o in outs[s * n_q:(s + 1) * n_q]], axis=1)
        assert H.rel_fro(A, want[s][0]) < 1e-4
        assert H.rel_fro(lse, want[s][1]) < 1e-4
