"""GPU parity of the HIP path against the CPU checker, through the C ABI, on
shapes the checker finishes in well under a second.  Covers every entry point,
every mask mode, the three dtypes, ragged and tiny extents, hidden rows and
the running (lse, A) hand-off."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from . import helpers as H

pytestmark = pytest.mark.gpu


def _oracle(oracle, f32, mask_bool, **kw):
    qf, kf, vf = f32
    return oracle.sdpa_vanilla(kf, qf, vf, mask_bool, **kw)


def _mask(kind, q_seq, k_seq):
    if kind == "causal":
        return synth.causal_mask(q_seq, k_seq)
    if kind == "full":
        return np.ones((q_seq, k_seq), bool)
    if kind == "window":      # tests/tile/flash_sdpa_fwd_cudnn.cc:57-86
        return np.abs(np.arange(q_seq)[:, None] - np.arange(k_seq)[None, :]) <= 32
    raise ValueError(kind)


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("seq,head,batch", [(32, 32, 1), (64, 64, 2), (128, 64, 3),
                                            (256, 128, 2), (96, 128, 1), (200, 64, 2),
                                            (1, 64, 1), (33, 32, 5)])
@pytest.mark.parametrize("kind", ["causal", "full", "window"])
def test_flash_entry_matches_oracle(oracle, dtype, seq, head, batch, kind):
    print("case", dtype, seq, head, batch, kind, flush=True)
    (Q, K, V), f32 = H.make_qkv(42, batch, seq, seq, head, dtype)
    mask = _mask(kind, seq, seq)
    want, want_lse = _oracle(oracle, f32, mask)
    lse, A = H.fresh_outputs(batch, seq, head, dtype)
    hip_sdpa.flash_sdpa_fwd(K.cuda(), Q.cuda(), H.additive_mask(mask, dtype).cuda(),
                            lse, V.cuda(), A)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_reference_preset_data(oracle, dtype):
    # tests/kernel/flash_sdpa_fwd_cudnn.cc:211-219: K=(i%20-10)*0.1, Q=0.8K, V=1.2K
    seq, head, batch = 128, 64, 3
    i = np.arange(batch * seq * head)
    k = ((i % 20 - 10) * 0.1).astype(np.float32).reshape(batch, seq, head)
    (K, kf), (Q, qf), (V, vf) = H.rounded(k, dtype), H.rounded(k * np.float32(0.8), dtype), \
        H.rounded(k * np.float32(1.2), dtype)
    mask = synth.causal_mask(seq, seq)
    want, want_lse = oracle.sdpa_bruteforce_f64(kf, qf, vf,
                                                np.where(mask, 0, -np.inf).astype(np.float32))
    lse, A = H.fresh_outputs(batch, seq, head, dtype)
    hip_sdpa.flash_sdpa_fwd(K.cuda(), Q.cuda(), H.additive_mask(mask, dtype).cuda(),
                            lse, V.cuda(), A)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("q_seq,k_seq,offset", [(128, 128, 0), (100, 260, 160), (64, 300, 100),
                                                (130, 70, -20), (16, 512, 496)])
def test_mask_modes_agree(oracle, dtype, q_seq, k_seq, offset):
    """Analytic causal, boolean and additive masks give the oracle's answer on
    non-square tiles, including queries that see nothing (negative offset)."""
    print("case", dtype, q_seq, k_seq, offset, flush=True)
    head, batch = 64, 2
    (Q, K, V), f32 = H.make_qkv(7, batch, q_seq, k_seq, head, dtype)
    mask = synth.causal_mask(q_seq, k_seq, offset)
    want, want_lse = _oracle(oracle, f32, mask)
    Kd, Qd, Vd = K.cuda(), Q.cuda(), V.cuda()
    outs = []
    for mode, m in [(hip_sdpa.MASK_CAUSAL, None),
                    (hip_sdpa.MASK_BOOL, torch.from_numpy(mask).cuda()),
                    (hip_sdpa.MASK_ADDITIVE, H.additive_mask(mask, dtype).cuda())]:
        lse, A = H.fresh_outputs(batch, q_seq, head, dtype, poison=False)
        hip_sdpa.sdpa_fwd_tile(Kd, Qd, m, lse, Vd, A, mode, causal_offset=offset)
        torch.cuda.synchronize()
        assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
        assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
        outs.append((H.to_np(lse), H.to_np(A)))
    hidden = ~mask.any(axis=1)
    if hidden.any():       # hidden queries: lse stays -inf, A untouched (0 here)
        assert np.all(np.isneginf(outs[0][0][:, hidden])) and np.all(outs[0][1][:, hidden] == 0)


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_no_mask_mode(oracle, dtype):
    (Q, K, V), f32 = H.make_qkv(9, 3, 70, 150, 128, dtype)
    want, want_lse = _oracle(oracle, f32, None)
    lse, A = H.fresh_outputs(3, 70, 128, dtype)
    hip_sdpa.sdpa_fwd_tile(K.cuda(), Q.cuda(), None, lse, V.cuda(), A, hip_sdpa.MASK_NONE)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
def test_running_merge_over_key_tiles(oracle, dtype):
    """One call per key tile, (lse, A) carried in memory between calls as
    between NNTile tasks (src/tensor/flash_sdpa_fwd_cudnn.cc:246-274), in a
    shuffled order: equals attention over all keys at once."""
    seq, head, batch, tile = 256, 64, 2, 64
    (Q, K, V), f32 = H.make_qkv(11, batch, seq, seq, head, dtype)
    mask = synth.causal_mask(seq, seq)
    want, want_lse = _oracle(oracle, f32, mask)
    lse, A = H.fresh_outputs(batch, seq, head, dtype)
    Qd = Q.cuda()
    for t in [2, 0, 3, 1]:
        Kt = K[:, t * tile:(t + 1) * tile].contiguous().cuda()
        Vt = V[:, t * tile:(t + 1) * tile].contiguous().cuda()
        mt = H.additive_mask(mask[:, t * tile:(t + 1) * tile], dtype).contiguous().cuda()
        hip_sdpa.sdpa_fwd_tile(Kt, Qd, mt, lse, Vt, A, hip_sdpa.MASK_ADDITIVE)
    torch.cuda.synchronize()
    # each hand-off rounds A to the tile dtype once more
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("q_seq,k_seq,q_tile,k_tile", [(256, 256, 64, 64), (300, 300, 128, 96),
                                                       (200, 520, 200, 128), (512, 512, 128, 256)])
@pytest.mark.parametrize("causal", [True, False])
def test_grid_entry_matches_oracle(oracle, dtype, q_seq, k_seq, q_tile, k_tile, causal):
    print("case", dtype, q_seq, k_seq, q_tile, k_tile, causal, flush=True)
    head, batch = 64, 3
    offset = k_seq - q_seq
    (Q, K, V), f32 = H.make_qkv(13, batch, q_seq, k_seq, head, dtype)
    mask = synth.causal_mask(q_seq, k_seq, offset) if causal else None
    want, want_lse = _oracle(oracle, f32, mask, k_tile=k_tile)
    Kt = [K[:, s:s + k_tile].contiguous().cuda() for s in range(0, k_seq, k_tile)]
    Vt = [V[:, s:s + k_tile].contiguous().cuda() for s in range(0, k_seq, k_tile)]
    Qt = [Q[:, s:s + q_tile].contiguous().cuda() for s in range(0, q_seq, q_tile)]
    outs = [H.fresh_outputs(batch, q.shape[1], head, dtype) for q in Qt]
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in outs], Vt, [o[1] for o in outs], q_seq, k_seq,
                           q_tile, k_tile, hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE,
                           causal_offset=offset)
    torch.cuda.synchronize()
    A = np.concatenate([H.to_np(o[1]) for o in outs], axis=1)
    lse = np.concatenate([H.to_np(o[0]) for o in outs], axis=1)
    assert H.rel_fro(A, want) < H.TOL[dtype]
    assert H.rel_fro(lse, want_lse) < H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("q_seq,k_seq,n_batch,group,n_kv,head", [
    (16, 512, 2, 4, 2, 128), (1, 300, 3, 4, 2, 128), (16, 1000, 1, 4, 1, 64),
    (5, 77, 2, 8, 3, 128), (16, 64, 1, 2, 2, 128), (64, 200, 2, 1, 2, 64)])
@pytest.mark.parametrize("mode", ["causal", "bool", "additive", "none"])
def test_decode_entry_matches_oracle(oracle, dtype, q_seq, k_seq, n_batch, group, n_kv, head, mode):
    print("case", dtype, q_seq, k_seq, n_batch, group, n_kv, head, mode, flush=True)
    batch = n_batch * group * n_kv
    (Q, K, V), f32 = H.make_qkv(17, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    offset = k_seq - q_seq            # layer/sdpa.py:516-531: new tokens are the last keys
    mask = None if mode == "none" else synth.causal_mask(q_seq, k_seq, offset)
    want, want_lse = _oracle(oracle, f32, mask, n_batch=n_batch, kv_repeat=group)
    Kd, Qd, Vd = K.cuda(), Q.cuda(), V.cuda()
    ws = torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group), dtype=torch.uint8,
                     device="cuda")
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    m, mm = {"causal": (None, hip_sdpa.MASK_CAUSAL), "none": (None, hip_sdpa.MASK_NONE),
             "bool": (None if mask is None else torch.from_numpy(mask).cuda(), hip_sdpa.MASK_BOOL),
             "additive": (None if mask is None else H.additive_mask(mask, dtype).cuda(),
                          hip_sdpa.MASK_ADDITIVE)}[mode]
    hip_sdpa.sdpa_fwd_decode(Kd, Qd, m, lse, Vd, A, mm, n_batch, group, ws, causal_offset=offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("form", ["additive", "bool"])
@pytest.mark.parametrize("q_seq,k_seq,shift,head", [(16, 1001, 0, 128), (5, 333, 1, 128), (16, 2050, 3, 64),
                                                    (3, 67, 1, 128), (16, 1024, 1, 128), (7, 130, 0, 64)])
def test_decode_explicit_masks_of_any_alignment(oracle, dtype, form, q_seq, k_seq, shift, head):
    """Decode with a mask given as values that is not a causal one (holes and
    hidden stretches, so that a wrong mask element changes the result), whose
    rows are not a multiple of 4 elements, that starts `shift` elements into
    its allocation, and whose last key step is ragged; both mask tile types."""
    print("case decode mask", dtype, form, q_seq, k_seq, shift, head, flush=True)
    n_batch, group, n_kv = 2, 4, 2
    batch = n_batch * group * n_kv
    (Q, K, V), f32 = H.make_qkv(29, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    i = np.arange(q_seq)[:, None]
    j = np.arange(k_seq)[None, :]
    mask = np.ascontiguousarray(((i * 5 + j) % 7 != 0) & ((j // 50) % 3 != (i % 3)) & (j >= i))
    want, want_lse = _oracle(oracle, f32, mask, n_batch=n_batch, kv_repeat=group)
    flat = (H.additive_mask(mask, dtype) if form == "additive" else torch.from_numpy(mask.copy())).reshape(-1)
    room = torch.zeros(flat.numel() + 8, dtype=flat.dtype)
    room[shift:shift + flat.numel()] = flat
    m = room.cuda()[shift:shift + flat.numel()].view(q_seq, k_seq)
    Kd, Qd, Vd = K.cuda(), Q.cuda(), V.cuda()
    ws = torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group), dtype=torch.uint8,
                     device="cuda")
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    mode = hip_sdpa.MASK_ADDITIVE if form == "additive" else hip_sdpa.MASK_BOOL
    hip_sdpa.sdpa_fwd_decode(Kd, Qd, m, lse, Vd, A, mode, n_batch, group, ws)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]


def test_decode_merges_into_running_pair(oracle):
    """Two decode calls over two halves of the cache == one call over all of it."""
    dtype, q_seq, k_seq, n_batch, group, n_kv, head = "bf16", 16, 512, 2, 4, 2, 128
    batch = n_batch * group * n_kv
    (Q, K, V), f32 = H.make_qkv(19, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    offset = k_seq - q_seq
    want, want_lse = _oracle(oracle, f32, synth.causal_mask(q_seq, k_seq, offset),
                             n_batch=n_batch, kv_repeat=group)
    Qd = Q.cuda()
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    for lo, hi in [(256, 512), (0, 256)]:
        Kd, Vd = K[:, lo:hi].contiguous().cuda(), V[:, lo:hi].contiguous().cuda()
        ws = torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group),
                         dtype=torch.uint8, device="cuda")
        hip_sdpa.sdpa_fwd_decode(Kd, Qd, None, lse, Vd, A, hip_sdpa.MASK_CAUSAL, n_batch, group,
                                 ws, k_pos0=lo, causal_offset=offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("head,seq,batch", [(8, 5, 3), (64, 33, 2), (128, 7, 4), (5, 9, 1), (128, 1024, 8)])
def test_accumulate_attn_output_preset(oracle, dtype, head, seq, batch):
    # data formulas of tests/kernel/accumulate_attn_output.cc:98-128
    lin = np.arange(seq * batch)
    base = -3.0 + 0.25 * (lin % 17)
    d_on, s_on = ((lin + 1) % 3) != 0, ((lin + 2) % 4) != 0
    dst_lse = np.where(d_on, base, -np.inf).astype(np.float32)
    src_lse = np.where(s_on, base + 0.5, -np.inf).astype(np.float32)
    h = np.arange(head)[None, :]
    dst = np.where(d_on[:, None], 0.1 * ((lin[:, None] + h) % 11) - 1.0, 0.0).astype(np.float32)
    src = np.where(s_on[:, None], 0.2 * ((lin[:, None] + h + 3) % 13) - 0.5, 0.0).astype(np.float32)
    (D, df), (S, sf) = H.rounded(dst.reshape(batch, seq, head), dtype), \
        H.rounded(src.reshape(batch, seq, head), dtype)
    want_lse, want = dst_lse.copy(), df.copy()
    oracle.accumulate_attn_output("fp32", head, seq, batch, src_lse, sf, want_lse, want)
    Dd, dl = D.cuda(), torch.from_numpy(dst_lse.reshape(batch, seq)).cuda()
    hip_sdpa.accumulate_attn_output(torch.from_numpy(src_lse.reshape(batch, seq)).cuda(), S.cuda(), dl, Dd)
    torch.cuda.synchronize()
    tol = 1e-5 if dtype == "fp32" else 5e-3       # :176-184
    assert np.max(np.abs(H.to_np(Dd) - want)) < tol * max(1.0, np.abs(want).max())
    got_lse = H.to_np(dl).ravel()
    assert np.array_equal(np.isneginf(got_lse), np.isneginf(want_lse))
    fin = np.isfinite(want_lse)
    assert np.max(np.abs(got_lse[fin] - want_lse[fin])) < 1e-5


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("head", [128, 6])      # the 16-byte path and the element path
def test_accumulate_attn_output_skips_rows_whose_source_logsumexp_is_not_finite(dtype, head):
    """src/kernel/accumulate_attn_output/cuda.cu:43-50: a source row with a
    non-finite logsumexp (-inf, NaN, +inf) has no influence; its destination
    row - values and logsumexp, even a -inf one with NaN values behind it - stays
    bit for bit.  (The reference's CPU statement only knows -inf, cpu.cc:73-97;
    the GPU kernel is what this entry point replaces.)"""
    seq, batch = 9, 2
    rows = seq * batch
    src_lse = np.linspace(-1.0, 1.0, rows).astype(np.float32)
    bad = {1: np.nan, 4: np.inf, 7: -np.inf, 10: np.nan, 13: -np.inf}
    for r, v in bad.items():
        src_lse[r] = v
    dst_lse = np.linspace(0.5, -0.5, rows).astype(np.float32)
    dst_lse[10] = -np.inf
    dt = H.TORCH_DT[dtype]
    g = torch.Generator().manual_seed(5)
    src = torch.randn(batch, seq, head, generator=g).to(dt)
    dst = torch.randn(batch, seq, head, generator=g).to(dt)
    dst.view(rows, head)[10] = float("nan")        # never read: its logsumexp is -inf
    Dd, dl = dst.clone().cuda(), torch.from_numpy(dst_lse.reshape(batch, seq)).cuda()
    hip_sdpa.accumulate_attn_output(torch.from_numpy(src_lse.reshape(batch, seq)).cuda(), src.cuda(), dl, Dd)
    torch.cuda.synchronize()
    bits = lambda t: t.cpu().contiguous().view(torch.int32 if t.element_size() == 4 else torch.int16)
    got, got_lse = Dd.cpu().view(rows, head), dl.cpu().view(rows)
    for r in range(rows):
        if r in bad:
            assert torch.equal(bits(got[r]), bits(dst.view(rows, head)[r])), r
            assert np.array_equal(got_lse[r:r + 1].numpy().view(np.int32),
                                  dst_lse[r:r + 1].view(np.int32)), r
        else:
            want_lse = np.logaddexp(np.float64(dst_lse[r]), np.float64(src_lse[r]))
            assert abs(float(got_lse[r]) - want_lse) < 1e-5, r
            assert torch.isfinite(got[r].float()).all(), r


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_codelet_body(oracle, dtype):
    """The StarPU-shaped body with the reference's buffer order, run twice on
    two key tiles; a bad argument makes the task a no-op."""
    seq, head, batch = 64, 64, 2
    (Q, K, V), f32 = H.make_qkv(23, batch, seq, seq, head, dtype)
    mask = synth.causal_mask(seq, seq)
    want, want_lse = _oracle(oracle, f32, mask)
    lse, A = H.fresh_outputs(batch, seq, head, dtype)
    Kd, Qd, Vd, md = K.cuda(), Q.cuda(), V.cuda(), H.additive_mask(mask, dtype).cuda()
    s_lse, s_A = torch.empty_like(lse), torch.empty_like(A)
    torch.cuda.synchronize()
    hip_sdpa.flash_sdpa_fwd_codelet(Kd, Qd, md, lse, Vd, A, s_lse, s_A, head=48)   # unsupported head
    torch.cuda.synchronize()
    assert torch.isneginf(lse).all()
    hip_sdpa.flash_sdpa_fwd_codelet(Kd, Qd, md, lse, Vd, A, s_lse, s_A)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]


def test_inputs_are_not_modified():
    # tests/kernel/flash_sdpa_fwd_cudnn.cc:345-362 asserts bit-identical inputs afterwards
    (Q, K, V), _ = H.make_qkv(29, 2, 128, 128, 64, "bf16")
    mask = H.additive_mask(synth.causal_mask(128, 128), "bf16")
    Kd, Qd, Vd, md = K.cuda(), Q.cuda(), V.cuda(), mask.cuda()
    lse, A = H.fresh_outputs(2, 128, 64, "bf16")
    hip_sdpa.flash_sdpa_fwd(Kd, Qd, md, lse, Vd, A)
    torch.cuda.synchronize()
    for d, h in [(Kd, K), (Qd, Q), (Vd, V), (md, mask)]:
        assert torch.equal(d.cpu().view(torch.int16), h.view(torch.int16))


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_overwrite_flag_ignores_running_pair(oracle, dtype):
    """OVERWRITE: lse and A hold garbage on entry, every row is written; rows
    that see no key get lse = -inf and A = 0."""
    q_seq, k_seq, head, batch, offset = 200, 150, 64, 2, -70
    (Q, K, V), f32 = H.make_qkv(31, batch, q_seq, k_seq, head, dtype)
    mask = synth.causal_mask(q_seq, k_seq, offset)
    want, want_lse = _oracle(oracle, f32, mask)
    hidden = ~mask.any(axis=1)
    assert hidden.sum() >= 64          # a whole wavefront and more sees nothing
    for entry in ("tile", "grid"):
        lse = torch.full((batch, q_seq), 123.0, device="cuda")
        A = torch.full((batch, q_seq, head), float("nan"), dtype=H.TORCH_DT[dtype], device="cuda")
        if entry == "tile":
            hip_sdpa.sdpa_fwd_tile(K.cuda(), Q.cuda(), None, lse, V.cuda(), A, hip_sdpa.MASK_CAUSAL,
                                   causal_offset=offset, flags=hip_sdpa.OVERWRITE)
        else:
            hip_sdpa.sdpa_fwd_grid([K.cuda()], [Q.cuda()], [lse], [V.cuda()], [A], q_seq, k_seq,
                                   q_seq, k_seq, hip_sdpa.MASK_CAUSAL, causal_offset=offset,
                                   flags=hip_sdpa.OVERWRITE)
        torch.cuda.synchronize()
        assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
        assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
        assert np.all(H.to_np(A)[:, hidden] == 0)


def test_overwrite_flag_decode(oracle):
    dtype, q_seq, k_seq, n_batch, group, n_kv, head = "bf16", 16, 300, 2, 4, 2, 128
    batch = n_batch * group * n_kv
    (Q, K, V), f32 = H.make_qkv(37, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    offset = -8                         # tokens 0..7 see nothing
    mask = synth.causal_mask(q_seq, k_seq, offset)
    want, want_lse = _oracle(oracle, f32, mask, n_batch=n_batch, kv_repeat=group)
    Kd, Qd, Vd = K.cuda(), Q.cuda(), V.cuda()
    ws = torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group), dtype=torch.uint8,
                     device="cuda")
    lse = torch.full((batch, q_seq), 5.0, device="cuda")
    A = torch.full((batch, q_seq, head), float("nan"), dtype=torch.bfloat16, device="cuda")
    hip_sdpa.sdpa_fwd_decode(Kd, Qd, None, lse, Vd, A, hip_sdpa.MASK_CAUSAL, n_batch, group, ws,
                             causal_offset=offset, flags=hip_sdpa.OVERWRITE)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < 1e-2
    assert H.rel_fro(H.to_np(lse), want_lse) < 1e-2


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("head", [32, 64, 128])
@pytest.mark.parametrize("q_seq,k_seq,k_tile", [(192, 448, 448), (130, 397, 397), (256, 576, 192),
                                                (96, 480, 160), (128, 128, 128)])
@pytest.mark.parametrize("causal", [True, False])
def test_unmasked_steps_loop(oracle, dtype, head, q_seq, k_seq, k_tile, causal):
    """Shapes chosen for the pipelined loop over complete, fully visible key
    steps: odd and even numbers of such steps, a ragged last step, key tiles
    that are and are not multiples of the step, every head size, GQA, and a
    running pair that is merged into rather than overwritten."""
    print("case", dtype, head, q_seq, k_seq, k_tile, causal, flush=True)
    n_batch, group, n_kv = 2, 2, 2
    batch = n_batch * group * n_kv
    offset = k_seq - q_seq
    (Q, K, V), f32 = H.make_qkv(23, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    mask = synth.causal_mask(q_seq, k_seq, offset) if causal else None
    want, want_lse = _oracle(oracle, f32, mask, k_tile=k_tile, n_batch=n_batch, kv_repeat=group)
    Kt = [K[:, s:s + k_tile].contiguous().cuda() for s in range(0, k_seq, k_tile)]
    Vt = [V[:, s:s + k_tile].contiguous().cuda() for s in range(0, k_seq, k_tile)]
    mode = hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    hip_sdpa.sdpa_fwd_grid(Kt, [Q.cuda()], [lse], Vt, [A], q_seq, k_seq, q_seq, k_tile, mode,
                           n_batch=n_batch, kv_group=group, causal_offset=offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
    # the same through per-tile calls that merge into the running pair, and twice
    # in a row: bit-identical results (no dependence on timing)
    runs = []
    for _ in range(2):
        lse2, A2 = H.fresh_outputs(batch, q_seq, head, dtype)
        for i, (kt, vt) in enumerate(zip(Kt, Vt)):
            hip_sdpa.sdpa_fwd_tile(kt, Q.cuda(), None, lse2, vt, A2, mode, n_batch=n_batch,
                                   kv_group=group, k_pos0=i * k_tile, causal_offset=offset)
        torch.cuda.synchronize()
        runs.append((lse2, A2))
    assert torch.equal(runs[0][0], runs[1][0])
    assert torch.equal(runs[0][1].view(torch.int16), runs[1][1].view(torch.int16))
    assert H.rel_fro(H.to_np(runs[0][1]), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(runs[0][0]), want_lse) < H.TOL[dtype]


@pytest.mark.parametrize("head", [32, 64, 128])
@pytest.mark.parametrize("batch,q_seq,k_seq,k_tile", [(3, 200, 333, 333), (2, 64, 1000, 250),
                                                      (40, 1024, 320, 320), (70, 512, 200, 96)])
@pytest.mark.parametrize("causal", [True, False])
def test_fp32_launch_forms(oracle, head, batch, q_seq, k_seq, k_tile, causal):
    """The fp32 kernel has two launch forms: 128-query workgroups, and - for
    launches with fewer of those than the GPU has CUs - 32-query workgroups
    whose four wavefronts share the keys and merge at the end.  Small batches
    take the second form, the large ones the first; both against the checker,
    over one and several key tiles (ragged ones included), with key counts
    that leave some wavefronts of the second form without a step."""
    print("case fp32", head, batch, q_seq, k_seq, k_tile, causal, flush=True)
    offset = max(k_seq - q_seq, 0)
    (Q, K, V), f32 = H.make_qkv(31, batch, q_seq, k_seq, head, "fp32")
    mask = synth.causal_mask(q_seq, k_seq, offset) if causal else None
    want, want_lse = _oracle(oracle, f32, mask, k_tile=k_tile)
    Kt = [K[:, s:s + k_tile].contiguous().cuda() for s in range(0, k_seq, k_tile)]
    Vt = [V[:, s:s + k_tile].contiguous().cuda() for s in range(0, k_seq, k_tile)]
    mode = hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE
    lse, A = H.fresh_outputs(batch, q_seq, head, "fp32")
    hip_sdpa.sdpa_fwd_grid(Kt, [Q.cuda()], [lse], Vt, [A], q_seq, k_seq, q_seq, k_tile, mode,
                           causal_offset=offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL["fp32"]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL["fp32"]
    # per key tile, merged into the running pair
    lse2, A2 = H.fresh_outputs(batch, q_seq, head, "fp32")
    for i, (kt, vt) in enumerate(zip(Kt, Vt)):
        hip_sdpa.sdpa_fwd_tile(kt, Q.cuda(), None, lse2, vt, A2, mode, k_pos0=i * k_tile,
                               causal_offset=offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A2), want) < H.TOL["fp32"]
    assert H.rel_fro(H.to_np(lse2), want_lse) < H.TOL["fp32"]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("form", ["additive", "bool"])
@pytest.mark.parametrize("q_seq,k_seq", [(256, 1024), (200, 712), (128, 520), (130, 333),
                                         (130, 4232)])      # more than 64 key steps: the last bit is shared
@pytest.mark.parametrize("pattern", ["band", "late_start", "holes", "all_hidden", "all_open"])
def test_explicit_mask_scan_paths(oracle, dtype, form, q_seq, k_seq, pattern):
    """Masks given as values are scanned once per workgroup: leading key steps
    in which nothing is masked run in the unmasked pipelined loop, trailing
    steps in which everything is hidden are dropped.  The patterns put the
    boundaries of those runs at, before and after multiples of the 64-key
    step, per 128-query block differently; 333 keys make rows that are not a
    multiple of 16 bytes (no scan), 712 and 520 a ragged last step."""
    print("case scan", dtype, form, q_seq, k_seq, pattern, flush=True)
    batch, head = 3, 128
    i = np.arange(q_seq)[:, None]
    j = np.arange(k_seq)[None, :]
    if pattern == "band":            # open prefix, mixed band, hidden suffix
        mask = j <= (k_seq // 3 + 2 * i)
    elif pattern == "late_start":    # first keys hidden for some rows, rest open
        mask = j >= (i % 7) * 3
    elif pattern == "holes":         # a hidden stretch in the middle, rows with nothing visible
        mask = ((j < 100) | (j >= 300)) & (i % 50 != 49)
    elif pattern == "all_hidden":
        mask = np.zeros((q_seq, k_seq), bool)
    else:
        mask = np.ones((q_seq, k_seq), bool)
    mask = np.ascontiguousarray(np.broadcast_to(mask, (q_seq, k_seq)))
    (Q, K, V), f32 = H.make_qkv(77, batch, q_seq, k_seq, head, dtype)
    want, want_lse = _oracle(oracle, f32, mask)
    m = (H.additive_mask(mask, dtype) if form == "additive" else torch.from_numpy(mask.copy())).cuda()
    mode = hip_sdpa.MASK_ADDITIVE if form == "additive" else hip_sdpa.MASK_BOOL
    # merged into a running pair that starts empty ...
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    hip_sdpa.sdpa_fwd_tile(K.cuda(), Q.cuda(), m, lse, V.cuda(), A, mode)
    torch.cuda.synchronize()
    got, got_lse = H.to_np(A), H.to_np(lse)
    vis = mask.any(axis=1)
    assert np.all(np.isneginf(got_lse[:, ~vis]))
    assert H.rel_fro(got[:, vis], want[:, vis]) < H.TOL[dtype] or not vis.any()
    assert H.rel_fro(got_lse[:, vis], want_lse[:, vis]) < H.TOL[dtype] or not vis.any()
    # ... and in overwrite mode, where rows without a visible key become 0 / -inf
    lse2, A2 = H.fresh_outputs(batch, q_seq, head, dtype)
    hip_sdpa.sdpa_fwd_tile(K.cuda(), Q.cuda(), m, lse2, V.cuda(), A2, mode, flags=hip_sdpa.OVERWRITE)
    torch.cuda.synchronize()
    got2, got2_lse = H.to_np(A2), H.to_np(lse2)
    assert np.all(got2[:, ~vis] == 0) and np.all(np.isneginf(got2_lse[:, ~vis]))
    assert np.array_equal(got2[:, vis], got[:, vis]) and np.array_equal(got2_lse[:, vis], got_lse[:, vis])


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("form", ["additive", "bool"])
@pytest.mark.parametrize("head", [64, 128])
@pytest.mark.parametrize("q_seq,k_seq,shift", [(130, 333, 0), (130, 1001, 0), (257, 1001, 1),
                                               (64, 67, 3), (200, 130, 1), (128, 1024, 1)])
def test_explicit_mask_rows_of_any_alignment(oracle, dtype, form, head, q_seq, k_seq, shift):
    """Mask rows whose length is not a multiple of 4 elements, and a mask that
    starts `shift` elements into its allocation: the full key steps still take
    the wide mask loads (at the alignment of one element), only the ragged
    last step goes element by element.  A band pattern, so that steps with
    nothing masked, mixed steps and fully hidden steps all occur."""
    print("case unaligned mask", dtype, form, head, q_seq, k_seq, shift, flush=True)
    batch = 3
    i = np.arange(q_seq)[:, None]
    j = np.arange(k_seq)[None, :]
    mask = np.ascontiguousarray((j <= (k_seq // 3 + 2 * i)) & ((i + j) % 11 != 0))
    (Q, K, V), f32 = H.make_qkv(91, batch, q_seq, k_seq, head, dtype)
    want, want_lse = _oracle(oracle, f32, mask)
    flat = (H.additive_mask(mask, dtype) if form == "additive" else torch.from_numpy(mask.copy())).reshape(-1)
    room = torch.zeros(flat.numel() + 8, dtype=flat.dtype)
    room[shift:shift + flat.numel()] = flat
    m = room.cuda()[shift:shift + flat.numel()].view(q_seq, k_seq)
    assert m.is_contiguous() and m.data_ptr() % 8 == (shift * m.element_size()) % 8
    mode = hip_sdpa.MASK_ADDITIVE if form == "additive" else hip_sdpa.MASK_BOOL
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    hip_sdpa.sdpa_fwd_tile(K.cuda(), Q.cuda(), m, lse, V.cuda(), A, mode, flags=hip_sdpa.OVERWRITE)
    torch.cuda.synchronize()
    got, got_lse = H.to_np(A), H.to_np(lse)
    vis = mask.any(axis=1)
    assert np.all(got[:, ~vis] == 0) and np.all(np.isneginf(got_lse[:, ~vis]))
    assert H.rel_fro(got[:, vis], want[:, vis]) < H.TOL[dtype]
    assert H.rel_fro(got_lse[:, vis], want_lse[:, vis]) < H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("overwrite", [True, False])
def test_decode_with_one_key_split_per_unit(oracle, dtype, overwrite):
    """512 (batch, kv head) units: every unit gets one key split and the main
    kernel writes (lse, A) itself.  Both forms: overwrite, and two calls over
    two halves of the keys merged into the running pair."""
    q_seq, k_seq, n_batch, group, n_kv, head = 3, 200, 64, 2, 8, 64
    batch = n_batch * group * n_kv
    (Q, K, V), f32 = H.make_qkv(23, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    offset = k_seq - q_seq
    want, want_lse = _oracle(oracle, f32, synth.causal_mask(q_seq, k_seq, offset),
                             n_batch=n_batch, kv_repeat=group)
    Qd = Q.cuda()
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    pieces = [(0, k_seq)] if overwrite else [(96, k_seq), (0, 96)]
    for lo, hi in pieces:
        Kd, Vd = K[:, lo:hi].contiguous().cuda(), V[:, lo:hi].contiguous().cuda()
        ws = torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group),
                         dtype=torch.uint8, device="cuda")
        hip_sdpa.sdpa_fwd_decode(Kd, Qd, None, lse, Vd, A, hip_sdpa.MASK_CAUSAL, n_batch, group, ws,
                                 k_pos0=lo, causal_offset=offset,
                                 flags=hip_sdpa.OVERWRITE if overwrite else 0)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
