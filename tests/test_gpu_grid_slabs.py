"""Several slabs of the batch grid in one launch (n_slabs of
nntile_hip_sdpa_grid_args): the tiles that tensor::flash_sdpa_fwd_cudnn_async
(src/tensor/flash_sdpa_fwd_cudnn.cc:246-274) walks along the batch axes.  One
launch over all slabs must give, bit for bit, what one launch per slab gives,
and that must match the CPU composition."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _tiles(x, step):
    return [x[:, s:s + step].contiguous().cuda() for s in range(0, x.shape[1], step)]


@pytest.mark.parametrize("dtype,head", [("fp32", 64), ("fp32", 128), ("fp32", 32), ("bf16", 128),
                                        ("bf16", 64), ("fp16", 128), ("fp16", 32)])
@pytest.mark.parametrize("n_slabs,batch,q_seq,k_seq,q_tile,k_tile,causal", [
    (4, 3, 256, 256, 256, 256, True),       # cfg2's form: one sequence tile, slabs along the batch
    (3, 2, 320, 320, 128, 128, True),       # sequence tiles as well, last ones ragged
    (2, 5, 96, 200, 96, 64, False),         # rectangular, no mask
    (8, 8, 128, 128, 64, 128, True),        # 64 entries: the per-XCD order of the workgroups
    (5, 1, 200, 264, 200, 264, True),       # causal offset, one entry per slab
])
def test_slabs_in_one_launch(oracle, dtype, head, n_slabs, batch, q_seq, k_seq, q_tile, k_tile, causal):
    print("case", dtype, head, n_slabs, batch, q_seq, k_seq, q_tile, k_tile, causal, flush=True)
    offset = k_seq - q_seq
    mode = hip_sdpa.MASK_CAUSAL if causal else hip_sdpa.MASK_NONE
    mask = synth.causal_mask(q_seq, k_seq, offset) if causal else None
    Kt, Vt, Qt, outs_all, outs_one, want, want_lse = [], [], [], [], [], [], []
    for s in range(n_slabs):
        (Q, K, V), f32 = H.make_qkv(100 + s, batch, q_seq, k_seq, head, dtype)
        w, wl = oracle.sdpa_vanilla(f32[1], f32[0], f32[2], mask, k_tile=k_tile)
        want.append(w), want_lse.append(wl)
        k, v, q = _tiles(K, k_tile), _tiles(V, k_tile), _tiles(Q, q_tile)
        Kt += k
        Vt += v
        Qt += q
        outs_all += [H.fresh_outputs(batch, t.shape[1], head, dtype) for t in q]
        one = [H.fresh_outputs(batch, t.shape[1], head, dtype) for t in q]
        outs_one += one
        hip_sdpa.sdpa_fwd_grid(k, q, [o[0] for o in one], v, [o[1] for o in one], q_seq, k_seq,
                               q_tile, k_tile, mode, causal_offset=offset)
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in outs_all], Vt, [o[1] for o in outs_all], q_seq,
                           k_seq, q_tile, k_tile, mode, causal_offset=offset, n_slabs=n_slabs)
    torch.cuda.synchronize()
    for a, b in zip(outs_all, outs_one):
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    n_q = len(Qt) // n_slabs
    for s in range(n_slabs):
        A = np.concatenate([H.to_np(o[1]) for o in outs_all[s * n_q:(s + 1) * n_q]], axis=1)
        lse = np.concatenate([H.to_np(o[0]) for o in outs_all[s * n_q:(s + 1) * n_q]], axis=1)
        assert H.rel_fro(A, want[s]) < H.TOL[dtype]
        assert H.rel_fro(lse, want_lse[s]) < H.TOL[dtype]


def test_slabs_with_grouped_queries(oracle):
    """Every slab keeps its own (n_batch, kv_group) mapping of query entries
    to key/value entries."""
    dtype, head, n_slabs, n_batch, group, n_kv, seq = "bf16", 128, 3, 2, 2, 2, 192
    batch = n_batch * group * n_kv
    Kt, Vt, Qt, outs, want = [], [], [], [], []
    mask = synth.causal_mask(seq, seq, 0)
    for s in range(n_slabs):
        (Q, K, V), f32 = H.make_qkv(200 + s, batch, seq, seq, head, dtype, kv_batch=n_batch * n_kv)
        want.append(oracle.sdpa_vanilla(f32[1], f32[0], f32[2], mask, n_batch=n_batch,
                                        kv_repeat=group))
        Kt.append(K.cuda()), Vt.append(V.cuda()), Qt.append(Q.cuda())
        outs.append(H.fresh_outputs(batch, seq, head, dtype))
    hip_sdpa.sdpa_fwd_grid(Kt, Qt, [o[0] for o in outs], Vt, [o[1] for o in outs], seq, seq, seq,
                           seq, hip_sdpa.MASK_CAUSAL, n_batch=n_batch, kv_group=group,
                           n_slabs=n_slabs)
    torch.cuda.synchronize()
    for s in range(n_slabs):
        assert H.rel_fro(H.to_np(outs[s][1]), want[s][0]) < H.TOL[dtype]
        assert H.rel_fro(H.to_np(outs[s][0]), want[s][1]) < H.TOL[dtype]
