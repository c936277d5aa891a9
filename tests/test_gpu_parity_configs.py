"""The five workload shapes at full size: HIP path vs the CPU checker on the
same seeded (and, for bf16, rounded) inputs, within the stated tolerances
(fp32 1e-4, bf16 1e-2 relative Frobenius error on the output and on
logsumexp), plus size-independent properties where the checker would take too
long on everything."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from nntile_amd.configs import BY_NAME
from . import helpers as H

pytestmark = pytest.mark.gpu


def _inputs(cfg, kv_batch=None):
    """Q, K, V drawn in that order, each in Fortran element order of its tile
    ([head, seq, batch...] == C order [batch..., seq, head])."""
    kvb = cfg.batch_flat if kv_batch is None else kv_batch
    q = synth.randn(cfg.seed, 0, cfg.batch_flat * cfg.q_seq * cfg.head).reshape(
        cfg.batch_flat, cfg.q_seq, cfg.head)
    if cfg.outlier_frac > 0:
        n = int(cfg.outlier_frac * cfg.q_seq)
        rows = synth.permutation(cfg.seed, 7, cfg.q_seq)[:n]
        q[:, rows, :] *= np.float32(cfg.outlier_scale)
    k = synth.randn(cfg.seed, 1, kvb * cfg.k_seq * cfg.head).reshape(kvb, cfg.k_seq, cfg.head)
    v = synth.randn(cfg.seed, 2, kvb * cfg.k_seq * cfg.head).reshape(kvb, cfg.k_seq, cfg.head)
    (Q, qf), (K, kf), (V, vf) = H.rounded(q, cfg.dtype), H.rounded(k, cfg.dtype), H.rounded(v, cfg.dtype)
    return (Q, K, V), (qf, kf, vf)


def test_cfg1_single_head_fp32(oracle):
    cfg = BY_NAME["cfg1_single_head_fp32"]
    (Q, K, V), (qf, kf, vf) = _inputs(cfg)
    mask = synth.causal_mask(cfg.q_seq, cfg.k_seq)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask)
    lse, A = H.fresh_outputs(1, cfg.q_seq, cfg.head, "fp32")
    hip_sdpa.flash_sdpa_fwd(K.cuda(), Q.cuda(), H.additive_mask(mask, "fp32").cuda(), lse, V.cuda(), A)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < 1e-4
    assert H.rel_fro(H.to_np(lse), want_lse) < 1e-4
    H.check_rows(H.to_np(A), want, H.to_np(lse), want_lse, "fp32", "cfg1")


def test_cfg2_gpt2_small_fp32(oracle):
    """seq-tile 1024, head-tile 12: one kernel call per batch entry with
    batch_flat = 12 (Q laid out [head, seq, n_batch, 1, n_head])."""
    cfg = BY_NAME["cfg2_gpt2_small_fp32"]
    (Q, K, V), (qf, kf, vf) = _inputs(cfg)
    mask = synth.causal_mask(cfg.q_seq, cfg.k_seq)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask)
    md = H.additive_mask(mask, "fp32").cuda()
    shape5 = (cfg.n_head_kv, cfg.n_batch, cfg.q_seq, cfg.head)
    A_all = np.empty(shape5, np.float32)
    lse_all = np.empty(shape5[:3], np.float32)
    for nb in range(cfg.n_batch):
        sl = lambda t: t.view(shape5)[:, nb].contiguous().cuda()
        lse, A = H.fresh_outputs(cfg.n_head_kv, cfg.q_seq, cfg.head, "fp32")
        hip_sdpa.flash_sdpa_fwd(sl(K), sl(Q), md, lse, sl(V), A)
        torch.cuda.synchronize()
        A_all[:, nb], lse_all[:, nb] = H.to_np(A), H.to_np(lse)
    assert H.rel_fro(A_all.reshape(want.shape), want) < 1e-4
    assert H.rel_fro(lse_all.reshape(want_lse.shape), want_lse) < 1e-4
    H.check_rows(A_all.reshape(want.shape), want, lse_all.reshape(want_lse.shape), want_lse, "fp32", "cfg2")


def test_cfg2_gpt2_small_fp32_one_launch(oracle):
    """The same four (batch, head-tile) slabs as separate allocations in ONE
    launch with the analytic causal mask (what the tensor-level call submits
    once the mask's tiles are known to be the causal rule)."""
    cfg = BY_NAME["cfg2_gpt2_small_fp32"]
    (Q, K, V), (qf, kf, vf) = _inputs(cfg)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, synth.causal_mask(cfg.q_seq, cfg.k_seq))
    shape5 = (cfg.n_head_kv, cfg.n_batch, cfg.q_seq, cfg.head)
    slab = lambda t: [t.view(shape5)[:, nb].contiguous().cuda() for nb in range(cfg.n_batch)]
    outs = [H.fresh_outputs(cfg.n_head_kv, cfg.q_seq, cfg.head, "fp32") for _ in range(cfg.n_batch)]
    hip_sdpa.sdpa_fwd_grid(slab(K), slab(Q), [o[0] for o in outs], slab(V), [o[1] for o in outs],
                           cfg.q_seq, cfg.k_seq, cfg.seq_tile, cfg.seq_tile, hip_sdpa.MASK_CAUSAL,
                           n_slabs=cfg.n_batch)
    torch.cuda.synchronize()
    A = np.stack([H.to_np(o[1]) for o in outs], axis=1).reshape(want.shape)
    lse = np.stack([H.to_np(o[0]) for o in outs], axis=1).reshape(want_lse.shape)
    assert H.rel_fro(A, want) < 1e-4
    assert H.rel_fro(lse, want_lse) < 1e-4
    H.check_rows(A, want, lse, want_lse, "fp32", "cfg2 one launch")


def _split(t, tile):
    return [t[:, s:s + tile].contiguous().cuda() for s in range(0, t.shape[1], tile)]


def test_cfg3_llama_prefill_bf16(oracle):
    cfg = BY_NAME["cfg3_llama_prefill_bf16"]
    (Q, K, V), (qf, kf, vf) = _inputs(cfg)
    mask = synth.causal_mask(cfg.q_seq, cfg.k_seq)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, k_tile=cfg.seq_tile)
    t = cfg.seq_tile
    Qt, Kt, Vt = _split(Q, t), _split(K, t), _split(V, t)
    nt = len(Qt)
    # (a) one fused launch over the 4x4 tile grid
    outs = [H.fresh_outputs(cfg.batch_flat, t, cfg.head, "bf16") for _ in range(nt)]
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in outs], Vt, [o[1] for o in outs], cfg.q_seq,
                           cfg.k_seq, t, t, hip_sdpa.MASK_CAUSAL)
    torch.cuda.synchronize()
    A = np.concatenate([H.to_np(o[1]) for o in outs], axis=1)
    lse = np.concatenate([H.to_np(o[0]) for o in outs], axis=1)
    assert H.rel_fro(A, want) < 1e-2
    assert H.rel_fro(lse, want_lse) < 1e-2
    H.check_rows(A, want, lse, want_lse, "bf16", "cfg3 one launch")
    # (b) the reference's task structure: 16 calls, additive mask tiles, the
    # running (lse, A) carried through memory across the 4 key tiles
    outs2 = [H.fresh_outputs(cfg.batch_flat, t, cfg.head, "bf16") for _ in range(nt)]
    for qi in range(nt):
        for ki in range(nt):
            m = H.additive_mask(mask[qi * t:(qi + 1) * t, ki * t:(ki + 1) * t], "bf16").contiguous().cuda()
            hip_sdpa.flash_sdpa_fwd(Kt[ki], Qt[qi], m, outs2[qi][0], Vt[ki], outs2[qi][1])
    torch.cuda.synchronize()
    A2 = np.concatenate([H.to_np(o[1]) for o in outs2], axis=1)
    lse2 = np.concatenate([H.to_np(o[0]) for o in outs2], axis=1)
    assert H.rel_fro(A2, want) < 1e-2
    assert H.rel_fro(lse2, want_lse) < 1e-2
    H.check_rows(A2, want, lse2, want_lse, "bf16", "cfg3 sixteen tasks")


def test_cfg4_gqa_decode_bf16(oracle):
    cfg = BY_NAME["cfg4_gqa_decode_bf16"]
    (Q, K, V), (qf, kf, vf) = _inputs(cfg, kv_batch=cfg.n_batch * cfg.n_head_kv)
    mask = synth.causal_mask(cfg.q_seq, cfg.k_seq, cfg.causal_offset)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, n_batch=cfg.n_batch, kv_repeat=cfg.kv_group)
    Kd, Qd, Vd = K.cuda(), Q.cuda(), V.cuda()
    ws = torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, cfg.n_batch, cfg.kv_group),
                     dtype=torch.uint8, device="cuda")
    lse, A = H.fresh_outputs(cfg.batch_flat, cfg.q_seq, cfg.head, "bf16")
    hip_sdpa.sdpa_fwd_decode(Kd, Qd, None, lse, Vd, A, hip_sdpa.MASK_CAUSAL, cfg.n_batch,
                             cfg.kv_group, ws, causal_offset=cfg.causal_offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < 1e-2
    assert H.rel_fro(H.to_np(lse), want_lse) < 1e-2
    H.check_rows(H.to_np(A), want, H.to_np(lse), want_lse, "bf16", "cfg4 decode")
    # the same answer from the prefill tile kernel with the GQA index map
    lse2, A2 = H.fresh_outputs(cfg.batch_flat, cfg.q_seq, cfg.head, "bf16")
    hip_sdpa.sdpa_fwd_tile(Kd, Qd, None, lse2, Vd, A2, hip_sdpa.MASK_CAUSAL, n_batch=cfg.n_batch,
                           kv_group=cfg.kv_group, causal_offset=cfg.causal_offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A2), want) < 1e-2
    assert H.rel_fro(H.to_np(lse2), want_lse) < 1e-2
    H.check_rows(H.to_np(A2), want, H.to_np(lse2), want_lse, "bf16", "cfg4 tile kernel")


def test_cfg5_long_sequence_bf16(oracle):
    """16x16 tile grid, 1% of the query rows scaled x8.  The checker runs on
    every one of the sixteen query tiles (1 to 16 accumulated key tiles) for
    every head, over the keys a tile can see; exact properties over the whole
    output follow."""
    cfg = BY_NAME["cfg5_long_seq_bf16"]
    (Q, K, V), (qf, kf, vf) = _inputs(cfg)
    t = cfg.seq_tile
    Qt, Kt, Vt = _split(Q, t), _split(K, t), _split(V, t)
    nt = len(Qt)
    outs = [H.fresh_outputs(cfg.batch_flat, t, cfg.head, "bf16") for _ in range(nt)]
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in outs], Vt, [o[1] for o in outs], cfg.q_seq,
                           cfg.k_seq, t, t, hip_sdpa.MASK_CAUSAL)
    torch.cuda.synchronize()
    mask = synth.causal_mask(cfg.q_seq, cfg.k_seq)
    outliers = synth.permutation(cfg.seed, 7, cfg.q_seq)[:int(cfg.outlier_frac * cfg.q_seq)]
    seen = 0
    for qi in range(nt):
        rows = slice(qi * t, (qi + 1) * t)
        seen += int(np.count_nonzero((outliers >= rows.start) & (outliers < rows.stop)))
        hi = rows.stop          # the keys beyond are hidden from every row of the tile
        want, want_lse = oracle.sdpa_vanilla(np.ascontiguousarray(kf[:, :hi]),
                                             np.ascontiguousarray(qf[:, rows]),
                                             np.ascontiguousarray(vf[:, :hi]),
                                             np.ascontiguousarray(mask[rows, :hi]), k_tile=t)
        assert H.rel_fro(H.to_np(outs[qi][1]), want) < 1e-2
        assert H.rel_fro(H.to_np(outs[qi][0]), want_lse) < 1e-2
        H.check_rows(H.to_np(outs[qi][1]), want, H.to_np(outs[qi][0]), want_lse, "bf16",
                     "cfg5 query tile %d" % qi)
    assert seen == len(outliers) > 0
    # exact property over the whole output: doubling V doubles A bit for bit
    # and leaves lse unchanged (a power-of-two scale commutes with rounding)
    V2 = [v * 2 for v in Vt]
    outs2 = [H.fresh_outputs(cfg.batch_flat, t, cfg.head, "bf16") for _ in range(nt)]
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in outs2], V2, [o[1] for o in outs2], cfg.q_seq,
                           cfg.k_seq, t, t, hip_sdpa.MASK_CAUSAL)
    torch.cuda.synchronize()
    for a, b in zip(outs, outs2):
        assert torch.equal(a[1] * 2, b[1]) and torch.equal(a[0], b[0])
        assert torch.isfinite(a[1].float()).all() and torch.isfinite(a[0]).all()
    # constant V: every output equals that constant (softmax weights sum to 1)
    ones = [torch.ones_like(v) for v in Vt]
    outs3 = [H.fresh_outputs(cfg.batch_flat, t, cfg.head, "bf16") for _ in range(nt)]
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in outs3], ones, [o[1] for o in outs3], cfg.q_seq,
                           cfg.k_seq, t, t, hip_sdpa.MASK_CAUSAL)
    torch.cuda.synchronize()
    for o3 in outs3:
        assert (o3[1].float() - 1.0).abs().max().item() <= 2 ** -7
    # per-task path on the last query tile (16 hand-offs through bf16)
    lse_pt, A_pt = H.fresh_outputs(cfg.batch_flat, t, cfg.head, "bf16")
    for ki in range(nt):
        hip_sdpa.sdpa_fwd_tile(Kt[ki], Qt[15], None, lse_pt, Vt[ki], A_pt, hip_sdpa.MASK_CAUSAL,
                               q_pos0=15 * t, k_pos0=ki * t)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A_pt), want) < 1e-2
    assert H.rel_fro(H.to_np(lse_pt), want_lse) < 1e-2
    H.check_rows(H.to_np(A_pt), want, H.to_np(lse_pt), want_lse, "bf16", "cfg5 sixteen hand-offs")
