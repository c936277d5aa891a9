"""The decode entry point that allocates nothing
(nntile_hip_sdpa_fwd_decode_static: split partials in a device array the
library owns) against nntile_hip_sdpa_fwd_decode_* with a caller's workspace,
through the C ABI: same kernels, so the results must agree bit for bit, on two
calls in a row, the second on a smaller input (the array keeps the first
call's partials), and against the checker within the tolerance.  A shape
whose partials exceed the array is refused before anything is enqueued."""
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from . import helpers as H

pytestmark = pytest.mark.gpu


def _oracle(oracle, f32, mask, n_batch, group):
    qf, kf, vf = f32
    return oracle.sdpa_vanilla(kf, qf, vf, mask, n_batch=n_batch, kv_repeat=group)


def _both(oracle, dtype, q_seq, k_seq, n_batch, group, n_kv, head, seed, overwrite):
    print("case", dtype, q_seq, k_seq, n_batch, group, n_kv, head, seed, overwrite, flush=True)
    batch = n_batch * group * n_kv
    (Q, K, V), f32 = H.make_qkv(seed, batch, q_seq, k_seq, head, dtype, kv_batch=n_batch * n_kv)
    offset = k_seq - q_seq
    want, want_lse = _oracle(oracle, f32, synth.causal_mask(q_seq, k_seq, offset), n_batch, group)
    Kd, Qd, Vd = K.cuda(), Q.cuda(), V.cuda()
    need = hip_sdpa.decode_workspace_bytes(Kd, Qd, n_batch, group)
    assert 0 < need <= hip_sdpa.DECODE_STATIC_SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    flags = hip_sdpa.OVERWRITE if overwrite else 0
    lse0, A0 = H.fresh_outputs(batch, q_seq, head, dtype)
    lse1, A1 = H.fresh_outputs(batch, q_seq, head, dtype)
    hip_sdpa.sdpa_fwd_decode(Kd, Qd, None, lse0, Vd, A0, hip_sdpa.MASK_CAUSAL, n_batch, group, ws,
                             causal_offset=offset, flags=flags)
    hip_sdpa.sdpa_fwd_decode_static(Kd, Qd, None, lse1, Vd, A1, hip_sdpa.MASK_CAUSAL, n_batch,
                                    group, causal_offset=offset, flags=flags)
    torch.cuda.synchronize()
    assert torch.equal(lse0, lse1)
    assert torch.equal(A0.view(torch.int16), A1.view(torch.int16))
    assert H.rel_fro(H.to_np(A1), want) < H.TOL[dtype]
    assert H.rel_fro(H.to_np(lse1), want_lse) < H.TOL[dtype]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_static_scratch_decode_twice_second_smaller(oracle, dtype):
    # several key splits per unit (partials go through the array), then a
    # smaller input whose partials cover only the start of what the first left
    _both(oracle, dtype, 16, 2048, 2, 4, 2, 128, 51, False)
    _both(oracle, dtype, 5, 700, 1, 4, 2, 128, 52, True)
    # and the larger one again: nothing of the small call's leftovers shows
    _both(oracle, dtype, 16, 2048, 2, 4, 2, 128, 53, True)


def test_static_scratch_decode_head64_and_merge(oracle):
    _both(oracle, "bf16", 16, 1000, 1, 4, 1, 64, 54, False)
    _both(oracle, "bf16", 1, 300, 3, 4, 2, 64, 55, False)


def test_static_scratch_decode_with_the_merge_inside_the_launch(oracle):
    # 8 units: the merge rides in the main launch and its flags live in the
    # array as well; then a smaller input
    _both(oracle, "bf16", 16, 2048, 4, 4, 2, 128, 56, False)
    _both(oracle, "bf16", 3, 900, 8, 2, 1, 128, 57, True)


def _inputs(n_batch, group, n_kv, q_seq, k_seq, head, seed):
    batch = n_batch * group * n_kv
    (Q, K, V), _ = H.make_qkv(seed, batch, q_seq, k_seq, head, "bf16", kv_batch=n_batch * n_kv)
    return K.cuda(), Q.cuda(), V.cuda(), batch


def test_static_scratch_decode_allocates_nothing():
    """Across a call (after the warm-up call that looks the array up) the
    device's free memory as the runtime reports it, and what torch's allocator
    holds, stay what they were - for the form with the merge in a launch of
    its own and for the one with the merge inside the main launch."""
    for n_batch in (2, 4):
        Kd, Qd, Vd, batch = _inputs(n_batch, 4, 2, 16, 2048, 128, 60 + n_batch)
        lse, A = H.fresh_outputs(batch, 16, 128, "bf16")
        call = lambda: hip_sdpa.sdpa_fwd_decode_static(
            Kd, Qd, None, lse, Vd, A, hip_sdpa.MASK_CAUSAL, n_batch, 4, causal_offset=2032,
            flags=hip_sdpa.OVERWRITE)
        call()
        torch.cuda.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        reserved0, allocated0 = torch.cuda.memory_reserved(), torch.cuda.memory_allocated()
        for _ in range(3):
            call()
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        # (a workspace for this shape would be 8 MiB and more; the runtime's own
        # pools may move by a page or two)
        assert free1 >= free0 - (1 << 20)
        assert torch.cuda.memory_reserved() == reserved0
        assert torch.cuda.memory_allocated() == allocated0


@pytest.mark.parametrize("n_batch", [2, 4])
def test_static_scratch_decode_under_stream_capture(n_batch):
    """One call recorded into a graph, after a warm-up call outside the capture
    (the look-up of the array's address is not legal inside one).  Replays
    with eager work and synchronisations in between, each compared bit for
    bit with the eager result."""
    q_seq, k_seq, head, group = 16, 2048, 128, 4
    Kd, Qd, Vd, batch = _inputs(n_batch, group, 2, q_seq, k_seq, head, 70 + n_batch)
    offset = k_seq - q_seq
    lse0, A0 = H.fresh_outputs(batch, q_seq, head, "bf16")
    hip_sdpa.sdpa_fwd_decode_static(Kd, Qd, None, lse0, Vd, A0, hip_sdpa.MASK_CAUSAL, n_batch, group,
                                    causal_offset=offset, flags=hip_sdpa.OVERWRITE)
    torch.cuda.synchronize()
    lse, A = H.fresh_outputs(batch, q_seq, head, "bf16")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hip_sdpa.sdpa_fwd_decode_static(Kd, Qd, None, lse, Vd, A, hip_sdpa.MASK_CAUSAL, n_batch,
                                        group, causal_offset=offset, flags=hip_sdpa.OVERWRITE)
    small = _inputs(1, group, 2, 3, 500, head, 79)
    for _ in range(3):
        A.fill_(float("nan"))
        lse.fill_(float("nan"))
        # an eager call on another shape leaves its partials (and flags) in the array
        lse_s, A_s = H.fresh_outputs(small[3], 3, head, "bf16")
        hip_sdpa.sdpa_fwd_decode_static(small[0], small[1], None, lse_s, small[2], A_s,
                                        hip_sdpa.MASK_CAUSAL, 1, group, causal_offset=497,
                                        flags=hip_sdpa.OVERWRITE)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(A.view(torch.int16), A0.view(torch.int16)) and torch.equal(lse, lse0)


def test_static_scratch_refuses_what_does_not_fit():
    # 64 rows x 4096 units x 1 split of bf16 partials alone are 64 MiB
    n_batch, group, n_kv, head, q_seq, k_seq = 1024, 4, 4, 128, 16, 8192
    batch = n_batch * group * n_kv
    a = hip_sdpa.TileArgs()
    a.q_seq, a.k_seq, a.head, a.batch = q_seq, k_seq, head, batch
    a.n_batch, a.kv_group, a.mask_mode = n_batch, group, hip_sdpa.MASK_CAUSAL
    import ctypes
    need = int(hip_sdpa.lib().nntile_hip_sdpa_fwd_decode_workspace_bytes(ctypes.byref(a)))
    if need <= hip_sdpa.DECODE_STATIC_SCRATCH_BYTES:
        pytest.skip("this shape's partials fit the array")
    # the pointers are never touched: the size check comes first
    dummy = torch.zeros(16, dtype=torch.bfloat16, device="cuda")
    a.K = a.Q = a.V = a.A = dummy.data_ptr()
    a.lse = dummy.data_ptr()
    code = hip_sdpa.lib().nntile_hip_sdpa_fwd_decode_static(
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), 0, ctypes.byref(a))
    assert code == hip_sdpa.EWORKSPACE
    # an unknown dtype code is an argument error
    code = hip_sdpa.lib().nntile_hip_sdpa_fwd_decode_static(
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), 7, ctypes.byref(a))
    assert code == hip_sdpa.EINVAL
