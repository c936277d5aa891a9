"""The decode entry with the merge of the key splits inside the main launch
(units in multiples of 8, several splits) against the checker, against the
two-launch form and against the form that exchanges the partials through
device-scope fences: same bits; repeated calls on one workspace, workspaces
that hold arbitrary bytes, merge into a running pair."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from . import helpers as H

pytestmark = pytest.mark.gpu


def _case(oracle, dtype, q_seq, k_seq, n_batch, group, n_kv, head, mode, seed=23):
    batch = n_batch * group * n_kv
    (Q, K, V), (qf, kf, vf) = H.make_qkv(seed, batch, q_seq, k_seq, head, dtype,
                                         kv_batch=n_batch * n_kv)
    offset = k_seq - q_seq
    mask = None if mode == "none" else synth.causal_mask(q_seq, k_seq, offset)
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, mask, n_batch=n_batch, kv_repeat=group)
    m, mm = {"causal": (None, hip_sdpa.MASK_CAUSAL), "none": (None, hip_sdpa.MASK_NONE),
             "bool": (None if mask is None else torch.from_numpy(mask).cuda(), hip_sdpa.MASK_BOOL),
             "additive": (None if mask is None else H.additive_mask(mask, dtype).cuda(),
                          hip_sdpa.MASK_ADDITIVE)}[mode]
    return (K.cuda(), Q.cuda(), V.cuda()), (m, mm, offset), (want, want_lse)


def _run(dev, msk, n_batch, group, head, dtype, flags, ws=None, out=None):
    Kd, Qd, Vd = dev
    m, mm, offset = msk
    if ws is None:
        ws = torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group), dtype=torch.uint8,
                         device="cuda")
    lse, A = out if out is not None else H.fresh_outputs(Qd.shape[0], Qd.shape[1], head, dtype)
    hip_sdpa.sdpa_fwd_decode(Kd, Qd, m, lse, Vd, A, mm, n_batch, group, ws, causal_offset=offset,
                             flags=flags)
    torch.cuda.synchronize()
    return lse, A


def _bits(t):
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32).cpu().numpy()


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("q_seq,k_seq,n_batch,group,n_kv,head", [
    (16, 512, 4, 4, 2, 128), (1, 300, 8, 4, 1, 128), (16, 1000, 2, 4, 4, 64),
    (5, 777, 8, 8, 2, 128), (64, 200, 4, 1, 2, 64), (3, 4100, 2, 2, 4, 128)])
@pytest.mark.parametrize("mode", ["causal", "bool", "additive", "none"])
def test_merge_inside_the_launch(oracle, dtype, q_seq, k_seq, n_batch, group, n_kv, head, mode):
    print("case", dtype, q_seq, k_seq, n_batch, group, n_kv, head, mode, flush=True)
    before = hip_sdpa.decode_sync_timeouts(), hip_sdpa.decode_sync_misplaced()
    dev, msk, (want, want_lse) = _case(oracle, dtype, q_seq, k_seq, n_batch, group, n_kv, head, mode)
    lse, A = _run(dev, msk, n_batch, group, head, dtype, 0)
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
    for flags in (hip_sdpa.DECODE_SEPARATE_MERGE, hip_sdpa.DECODE_FENCED):
        lse2, A2 = _run(dev, msk, n_batch, group, head, dtype, flags)
        assert np.array_equal(_bits(A), _bits(A2)), flags
        assert np.array_equal(_bits(lse), _bits(lse2)), flags
    assert (hip_sdpa.decode_sync_timeouts(), hip_sdpa.decode_sync_misplaced()) == before


@pytest.mark.parametrize("fill", [0x00, 0xFF, "random"])
def test_workspace_contents_do_not_matter_and_calls_repeat(oracle, fill):
    """The flags of the in-launch merge live in the workspace: whatever bytes
    it holds before the first call, and after any number of calls, the result
    is the same."""
    dtype, q_seq, k_seq, n_batch, group, n_kv, head = "bf16", 16, 2048, 4, 4, 4, 128
    dev, msk, (want, want_lse) = _case(oracle, dtype, q_seq, k_seq, n_batch, group, n_kv, head,
                                       "causal", seed=29)
    n = hip_sdpa.decode_workspace_bytes(dev[0], dev[1], n_batch, group)
    if fill == "random":
        g = torch.Generator(device="cuda").manual_seed(5)
        ws = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    else:
        ws = torch.full((n,), fill, dtype=torch.uint8, device="cuda")
    first = None
    for rep in range(4):
        lse, A = _run(dev, msk, n_batch, group, head, dtype, 0, ws=ws)
        if first is None:
            first = (_bits(lse), _bits(A))
            assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
            assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]
        else:
            assert np.array_equal(first[0], _bits(lse)) and np.array_equal(first[1], _bits(A)), rep
    # a smaller shape on the same workspace afterwards (other flag positions)
    dev2, msk2, (want2, want_lse2) = _case(oracle, dtype, 4, 600, 8, 2, 1, head, "causal", seed=31)
    lse, A = _run(dev2, msk2, 8, 2, head, dtype, 0, ws=ws)
    assert H.rel_fro(H.to_np(A), want2) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse2) < H.TOL[dtype]


def test_other_inputs_on_the_same_workspace(oracle):
    """Calls with different inputs take turns on one workspace: every call
    must merge the partials written by this call, not what an earlier call
    left at the same addresses."""
    dtype, q_seq, k_seq, n_batch, group, n_kv, head = "bf16", 16, 1536, 4, 4, 2, 128
    cases = [_case(oracle, dtype, q_seq, k_seq, n_batch, group, n_kv, head, "causal", seed=40 + i)
             for i in range(3)]
    ws = torch.empty(hip_sdpa.decode_workspace_bytes(cases[0][0][0], cases[0][0][1], n_batch, group),
                     dtype=torch.uint8, device="cuda")
    outs = [H.fresh_outputs(cases[0][0][1].shape[0], q_seq, head, dtype) for _ in range(9)]
    # enqueued back to back, checked afterwards
    for rep, out in enumerate(outs):
        (Kd, Qd, Vd), (m, mm, offset), _ = cases[rep % 3]
        hip_sdpa.sdpa_fwd_decode(Kd, Qd, m, out[0], Vd, out[1], mm, n_batch, group, ws,
                                 causal_offset=offset)
    torch.cuda.synchronize()
    for rep, (lse, A) in enumerate(outs):
        want, want_lse = cases[rep % 3][2]
        assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype], rep
        assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype], rep
        H.check_rows(H.to_np(A), want, H.to_np(lse), want_lse, dtype, "rep %d" % rep)


def test_merge_inside_the_launch_into_running_pair(oracle):
    """Two calls over two halves of the cache == one call over all of it."""
    dtype, q_seq, k_seq, n_batch, group, n_kv, head = "bf16", 16, 1024, 4, 4, 2, 128
    batch = n_batch * group * n_kv
    (Q, K, V), (qf, kf, vf) = H.make_qkv(19, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    offset = k_seq - q_seq
    want, want_lse = oracle.sdpa_vanilla(kf, qf, vf, synth.causal_mask(q_seq, k_seq, offset),
                                         n_batch=n_batch, kv_repeat=group)
    Qd = Q.cuda()
    lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
    for lo, hi in [(512, 1024), (0, 512)]:
        Kd, Vd = K[:, lo:hi].contiguous().cuda(), V[:, lo:hi].contiguous().cuda()
        ws = torch.empty(hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group),
                         dtype=torch.uint8, device="cuda")
        hip_sdpa.sdpa_fwd_decode(Kd, Qd, None, lse, Vd, A, hip_sdpa.MASK_CAUSAL, n_batch, group,
                                 ws, k_pos0=lo, causal_offset=offset)
    torch.cuda.synchronize()
    assert H.rel_fro(H.to_np(A), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse), want_lse) < H.TOL[dtype]


def test_merge_inside_the_launch_wherever_the_round_of_the_xcds_starts(oracle):
    """A launch's workgroups go round the XCDs in index order, but the XCD of
    workgroup 0 depends on the queue and on what ran on it before (a graph
    launch moves it).  The in-launch merge only needs a unit's main and merge
    workgroups on one XCD, whichever: on the default stream, on side streams,
    after a graph launch, and with two streams running decode calls at the
    same time (each on a workspace of its own) the results are those of the
    two-launch form, bit for bit, and no merge workgroup reports a split on
    another XCD."""
    dtype, q_seq, k_seq, n_batch, group, n_kv, head = "bf16", 16, 4096, 4, 4, 2, 128
    before = hip_sdpa.decode_sync_timeouts(), hip_sdpa.decode_sync_misplaced()
    dev, msk, (want, want_lse) = _case(oracle, dtype, q_seq, k_seq, n_batch, group, n_kv, head,
                                       "causal", seed=57)
    Kd, Qd, Vd = dev
    m, mm, offset = msk
    lse0, A0 = _run(dev, msk, n_batch, group, head, dtype,
                    hip_sdpa.DECODE_SEPARATE_MERGE | hip_sdpa.OVERWRITE)
    assert H.rel_fro(H.to_np(A0), want) < H.TOL[dtype]
    nbytes = hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group)

    def call(out, ws, stream=None):
        hip_sdpa.sdpa_fwd_decode(Kd, Qd, m, out[0], Vd, out[1], mm, n_batch, group, ws,
                                 causal_offset=offset, flags=hip_sdpa.OVERWRITE, stream=stream)

    def same(out):
        return np.array_equal(_bits(out[0]), _bits(lse0)) and np.array_equal(_bits(out[1]), _bits(A0))

    ws = [torch.empty(nbytes, dtype=torch.uint8, device="cuda") for _ in range(3)]
    out = H.fresh_outputs(Qd.shape[0], q_seq, head, dtype)
    call(out, ws[0])
    torch.cuda.synchronize()
    assert same(out)
    # a graph launch, then the default stream again
    gout = H.fresh_outputs(Qd.shape[0], q_seq, head, dtype)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(gout, ws[0])
    for _ in range(2):
        gout[0].fill_(float("nan"))
        gout[1].fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert same(gout)
    out = H.fresh_outputs(Qd.shape[0], q_seq, head, dtype)
    call(out, ws[0])
    torch.cuda.synchronize()
    assert same(out)
    # two side streams at the same time, several calls each
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[H.fresh_outputs(Qd.shape[0], q_seq, head, dtype) for _ in range(4)] for _ in streams]
    torch.cuda.synchronize()
    for rep in range(4):
        for k, st in enumerate(streams):
            call(outs[k][rep], ws[1 + k], stream=st)
    torch.cuda.synchronize()
    for k in range(2):
        for rep in range(4):
            assert same(outs[k][rep]), (k, rep)
    assert (hip_sdpa.decode_sync_timeouts(), hip_sdpa.decode_sync_misplaced()) == before
