"""The fp32 split-key decode entry (nntile_hip_sdpa_fwd_decode_fp32, the
shape of LlamaAttention.forward_dynamic in fp32) against the checker at the
fp32 tolerance, against the tile kernel on the same inputs, merged into a
running pair, and reading a key/value cache in place."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from . import helpers as H

pytestmark = pytest.mark.gpu


def _workspace(Kd, Qd, n_batch, group):
    return torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group), dtype=torch.uint8,
                       device="cuda")


@pytest.mark.parametrize("q_seq,k_seq,n_batch,group,n_kv,head", [
    (16, 512, 2, 4, 2, 128), (1, 300, 3, 4, 2, 128), (16, 1000, 1, 4, 1, 64),
    (5, 77, 2, 8, 3, 128), (16, 64, 1, 2, 2, 128), (64, 200, 2, 1, 2, 64),
    (3, 31, 1, 2, 1, 64), (16, 2048, 4, 4, 2, 128), (7, 4100, 8, 1, 1, 64)])
@pytest.mark.parametrize("mode", ["causal", "bool", "additive", "none"])
def test_decode_fp32_matches_oracle(oracle, q_seq, k_seq, n_batch, group, n_kv, head, mode):
    print("case fp32 decode", q_seq, k_seq, n_batch, group, n_kv, head, mode, flush=True)
    batch = n_batch * group * n_kv
    (Q, K, V), f32 = H.make_qkv(17, batch, q_seq, k_seq, head, "fp32", kv_batch=n_batch * n_kv)
    offset = k_seq - q_seq            # layer/sdpa.py:516-531: new tokens are the last keys
    if mode == "none":
        mask = None
    elif mode == "causal":
        mask = synth.causal_mask(q_seq, k_seq, offset)
    else:                             # holes and hidden stretches: a wrong element changes the result
        i = np.arange(q_seq)[:, None]
        j = np.arange(k_seq)[None, :]
        mask = np.ascontiguousarray(((i * 5 + j) % 7 != 0) & ((j // 50) % 3 != (i % 3))
                                    & (j <= i + offset))
    qf, kf, vf = f32
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, n_batch=n_batch, kv_repeat=group)
    Kd, Qd, Vd = K.cuda(), Q.cuda(), V.cuda()
    ws = _workspace(Kd, Qd, n_batch, group)
    m, mm = {"causal": (None, hip_sdpa.MASK_CAUSAL), "none": (None, hip_sdpa.MASK_NONE),
             "bool": (None if mask is None else torch.from_numpy(mask).cuda(), hip_sdpa.MASK_BOOL),
             "additive": (None if mask is None else H.additive_mask(mask, "fp32").cuda(),
                          hip_sdpa.MASK_ADDITIVE)}[mode]
    vis = np.ones(q_seq, bool) if mask is None else mask.any(axis=1)
    outs = []
    for flags in (0, hip_sdpa.OVERWRITE):
        lse, A = H.fresh_outputs(batch, q_seq, head, "fp32")
        hip_sdpa.sdpa_fwd_decode(Kd, Qd, m, lse, Vd, A, mm, n_batch, group, ws, causal_offset=offset,
                                 flags=flags)
        torch.cuda.synchronize()
        a, l = H.to_np(A), H.to_np(lse)
        assert np.all(np.isneginf(l[:, ~vis]))
        assert H.rel_fro(a[:, vis], want[:, vis]) < H.TOL["fp32"]
        assert H.rel_fro(l[:, vis], want_lse[:, vis]) < H.TOL["fp32"]
        outs.append((a, l))
    assert np.all(outs[1][0][:, ~vis] == 0)
    assert np.array_equal(outs[0][0][:, vis], outs[1][0][:, vis])
    # the tile kernel on the same inputs (analytic and bool forms)
    if mode != "additive":
        lse2, A2 = H.fresh_outputs(batch, q_seq, head, "fp32")
        hip_sdpa.sdpa_fwd_tile(Kd, Qd, m, lse2, Vd, A2, mm, n_batch=n_batch, kv_group=group,
                               causal_offset=offset, flags=hip_sdpa.OVERWRITE)
        torch.cuda.synchronize()
        assert H.rel_fro(outs[1][0][:, vis], H.to_np(A2)[:, vis]) < H.TOL["fp32"]


def test_decode_fp32_merges_into_running_pair(oracle):
    """Two decode calls over two halves of the keys == one call over all of them."""
    q_seq, k_seq, n_batch, group, n_kv, head = 16, 512, 2, 4, 2, 128
    batch = n_batch * group * n_kv
    (Q, K, V), f32 = H.make_qkv(19, batch, q_seq, k_seq, head, "fp32", kv_batch=n_batch * n_kv)
    offset = k_seq - q_seq
    qf, kf, vf = f32
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, synth.causal_mask(q_seq, k_seq, offset),
                                         n_batch=n_batch, kv_repeat=group)
    Qd = Q.cuda()
    lse, A = H.fresh_outputs(batch, q_seq, head, "fp32")
    for lo, hi in [(256, 512), (0, 256)]:
        Kd, Vd = K[:, lo:hi].contiguous().cuda(), V[:, lo:hi].contiguous().cuda()
        hip_sdpa.sdpa_fwd_decode(Kd, Qd, None, lse, Vd, A, hip_sdpa.MASK_CAUSAL, n_batch, group,
                                 _workspace(Kd, Qd, n_batch, group), k_pos0=lo, causal_offset=offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL["fp32"]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL["fp32"]


@pytest.mark.parametrize("head", [64, 128])
def test_decode_fp32_from_a_cache_equals_the_dense_decode(oracle, head):
    """The cache form reads the first k_seq rows of every entry where they lie
    (rows behind them hold NaN): bit-identical to the dense call."""
    q_seq, k_seq, cap, n_batch, group, n_kv = 4, 333, 512, 2, 4, 2
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), f32 = H.make_qkv(21, batch, q_seq, k_seq, head, "fp32", kv_batch=kvb)
    Kc = torch.full((kvb, cap, head), float("nan"), device="cuda")
    Vc = torch.full((kvb, cap, head), float("nan"), device="cuda")
    Kc[:, :k_seq], Vc[:, :k_seq] = K.cuda(), V.cuda()
    Qd = Q.cuda()
    offset = k_seq - q_seq
    lse0, A0 = H.fresh_outputs(batch, q_seq, head, "fp32")
    hip_sdpa.sdpa_fwd_decode(K.cuda(), Qd, None, lse0, V.cuda(), A0, hip_sdpa.MASK_CAUSAL, n_batch,
                             group, _workspace(K.cuda(), Qd, n_batch, group), causal_offset=offset,
                             flags=hip_sdpa.OVERWRITE)
    lse1, A1 = H.fresh_outputs(batch, q_seq, head, "fp32")
    ws = torch.empty(hip_sdpa.decode_cache_workspace_bytes(k_seq, Qd, n_batch, group),
                     dtype=torch.uint8, device="cuda")
    hip_sdpa.sdpa_fwd_decode_cache(Kc, Vc, k_seq, Qd, None, lse1, A1, hip_sdpa.MASK_CAUSAL, n_batch,
                                   group, ws, causal_offset=offset, flags=hip_sdpa.OVERWRITE)
    torch.cuda.synchronize()
    assert torch.equal(A0, A1) and torch.equal(lse0, lse1)
    qf, kf, vf = f32
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, synth.causal_mask(q_seq, k_seq, offset),
                                         n_batch=n_batch, kv_repeat=group)
    assert H.rel_fro(H.to_np(A1), want) < H.TOL["fp32"]
    assert H.rel_fro(H.to_np(lse1), want_lse) < H.TOL["fp32"]


def test_decode_fp32_at_the_decode_benchmark_shape(oracle):
    """cfg4's shape with fp32 tiles, four (batch, kv head) units against the
    checker and all of them through an exact property: doubling V doubles A."""
    q_seq, k_seq, n_batch, group, n_kv, head = 16, 8192, 8, 4, 8, 128
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), f32 = H.make_qkv(23, batch, q_seq, k_seq, head, "fp32", kv_batch=kvb)
    offset = k_seq - q_seq
    Kd, Qd, Vd = K.cuda(), Q.cuda(), V.cuda()
    ws = _workspace(Kd, Qd, n_batch, group)
    lse, A = H.fresh_outputs(batch, q_seq, head, "fp32")
    hip_sdpa.sdpa_fwd_decode(Kd, Qd, None, lse, Vd, A, hip_sdpa.MASK_CAUSAL, n_batch, group, ws,
                             causal_offset=offset, flags=hip_sdpa.OVERWRITE)
    lse2, A2 = H.fresh_outputs(batch, q_seq, head, "fp32")
    hip_sdpa.sdpa_fwd_decode(Kd, Qd, None, lse2, 2.0 * Vd, A2, hip_sdpa.MASK_CAUSAL, n_batch, group,
                             ws, causal_offset=offset, flags=hip_sdpa.OVERWRITE)
    torch.cuda.synchronize()
    assert torch.equal(2.0 * A, A2) and torch.equal(lse, lse2)
    qf, kf, vf = f32
    mask = synth.causal_mask(q_seq, k_seq, offset)
    got, got_lse = H.to_np(A), H.to_np(lse)
    for nb, hkv in ((0, 0), (3, 1), (7, 7), (5, 4)):
        kv = nb + n_batch * hkv
        qs = [nb + n_batch * (g + group * hkv) for g in range(group)]
        want, want_lse = oracle.sdpa_vanilla(kf[kv:kv + 1], qf[qs], vf[kv:kv + 1], mask, n_batch=1,
                                             kv_repeat=group)
        assert H.rel_fro(got[qs], want) < H.TOL["fp32"]
        assert H.rel_fro(got_lse[qs], want_lse) < H.TOL["fp32"]
