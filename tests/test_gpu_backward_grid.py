"""The backward over a grid of separately allocated tiles in one call
(nntile_hip_sdpa_bwd_grid_*), through the C ABI.

Two checks.  Against the one-call form on the same rows held in one
allocation the results must be identical bit for bit: both forms walk the
same 64-row steps in the same order, only the addresses differ, so any
difference is an addressing mistake.  Against the fp64 flash-form checker the
tolerances are the reference's own for its backward kernel
(tests/kernel/flash_sdpa_bwd_cudnn.cc:312-327): relative Frobenius error 1e-2
for bf16 and 2e-3 for fp16."""
import ctypes

import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from . import helpers as H

pytestmark = pytest.mark.gpu

BWD_TOL = {"bf16": 1e-2, "fp16": 2e-3}


def _rounded(x, dtype):
    return H.rounded(np.ascontiguousarray(x, dtype=np.float32), dtype)


def _split(t, tile):
    return [t[:, s:s + tile].contiguous() for s in range(0, t.shape[1], tile)]


def _join(tiles):
    return torch.cat(tiles, dim=1)


def _bits(t):
    return t.view(torch.int16)


def _case(seed, n_batch, group, n_kv, q_seq, k_seq, head, dtype):
    """Inputs on the GPU as whole tensors, plus their fp32 values: Q, dA of
    every query head, K, V of every key/value head, A and lse from a forward
    pass of the same inputs under the causal rule with the keys' surplus as
    offset, and non-zero gradients to accumulate onto."""
    batch = n_batch * group * n_kv
    (Q, K, V), (qf, kf, vf) = H.make_qkv(seed, batch, q_seq, k_seq, head, dtype,
                                          kv_batch=n_batch * n_kv)
    G, gf = _rounded(synth.randn(seed + 1, 0, batch * q_seq * head).reshape(batch, q_seq, head),
                     dtype)
    init = [_rounded(0.25 * synth.randn(seed + 2, i, t.numel()).reshape(t.shape), dtype)
            for i, t in enumerate((K, Q, V))]
    return (Q, K, V, G), (qf, kf, vf, gf), init


def _forward(oracle, kf, qf, vf, add, n_batch, group, dtype):
    batch = qf.shape[0]
    kv_of = [(b % n_batch) + n_batch * ((b // n_batch) // group) for b in range(batch)]
    A64, lse64 = oracle.sdpa_bruteforce_f64(kf[kv_of], qf, vf[kv_of], add)
    A, af = _rounded(A64, dtype)
    return A, af, lse64.astype(np.float32)


SHAPES = [
    # q_seq, k_seq, q_tile, k_tile, n_batch, group, n_kv
    (512, 512, 128, 128, 2, 1, 1),
    (512, 512, 256, 128, 1, 2, 2),      # grouped queries: dK, dV sum over the group
    (640, 896, 256, 384, 2, 1, 1),      # last tiles shorter, still multiples of 128
    (600, 520, 256, 128, 1, 1, 2),      # ragged last tiles (88 and 8 rows)
    (300, 200, 300, 200, 2, 1, 1),      # one tile an axis, any size
    (128, 1100, 128, 256, 1, 4, 1),     # one query tile against many key tiles
    (1100, 128, 128, 128, 1, 1, 1),     # many query tiles against one key tile
]


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("head", [32, 64, 128])
@pytest.mark.parametrize("mode", ["causal", "none"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "q%d_k%d_qt%d_kt%d_n%d_g%d_kv%d" % s)
def test_grid_is_the_one_call_form_bit_for_bit(oracle, dtype, head, mode, shape):
    q_seq, k_seq, q_tile, k_tile, n_batch, group, n_kv = shape
    print("case bwd grid", dtype, head, mode, shape, flush=True)
    (Q, K, V, G), (qf, kf, vf, gf), init = _case(301, n_batch, group, n_kv, q_seq, k_seq, head,
                                                 dtype)
    offset = max(k_seq - q_seq, 0)
    mask = (synth.causal_mask(q_seq, k_seq, offset) if mode == "causal"
            else np.ones((q_seq, k_seq), bool))
    add = np.where(mask, 0, -np.inf).astype(np.float32)
    A, af, lse = _forward(oracle, kf, qf, vf, add, n_batch, group, dtype)
    mm = hip_sdpa.MASK_CAUSAL if mode == "causal" else hip_sdpa.MASK_NONE
    Qc, Kc, Vc, Gc, Ac = (t.cuda() for t in (Q, K, V, G, A))
    lc = torch.from_numpy(lse).cuda()

    for flags in (0, hip_sdpa.OVERWRITE):
        # one allocation per operand
        dK1, dQ1, dV1 = (x[0].clone().cuda() for x in init)
        hip_sdpa.sdpa_bwd_tile(Kc, Qc, Vc, Ac, Gc, None, lc, dK1, dQ1, dV1, mm, n_batch=n_batch,
                               kv_group=group, causal_offset=offset, flags=flags)
        # the same rows in tiles
        Kt, Vt = _split(Kc, k_tile), _split(Vc, k_tile)
        Qt, At, Gt, Lt = (_split(t, q_tile) for t in (Qc, Ac, Gc, lc))
        dKt, dQt, dVt = (_split(x[0].clone().cuda(), tile)
                         for x, tile in zip(init, (k_tile, q_tile, k_tile)))
        keep = [t.clone() for t in (*Kt, *Vt, *Qt, *At, *Gt, *Lt)]
        hip_sdpa.sdpa_bwd_grid(Kt, Qt, Vt, At, Gt, Lt, dKt, dQt, dVt, q_seq, k_seq, q_tile,
                               k_tile, mm, n_batch=n_batch, kv_group=group,
                               causal_offset=offset, flags=flags)
        torch.cuda.synchronize()
        for got, one, name in ((dKt, dK1, "dK"), (dQt, dQ1, "dQ"), (dVt, dV1, "dV")):
            assert torch.equal(_bits(_join(got)), _bits(one)), (name, flags)
        for a, b in zip((*Kt, *Vt, *Qt, *At, *Gt, *Lt), keep):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), "an input changed"

    # the overwrite pass against the checker
    want = oracle.sdpa_bwd_flash_f64(kf, qf, vf, af, gf, lse, add, kv_repeat=group,
                                     n_batch=n_batch)
    for got, w, name in ((dKt, want[0], "dK"), (dQt, want[1], "dQ"), (dVt, want[2], "dV")):
        err = H.rel_fro(H.to_np(_join(got)), w)
        assert err < BWD_TOL[dtype], (name, err)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_positions_and_offset(oracle, dtype):
    """q_pos0, k_pos0 and causal_offset shift the diagonal as they do for a
    single pair: a grid whose rule is key + 96 <= query + 160 + 30."""
    q_seq, k_seq, q_tile, k_tile, head, batch = 384, 512, 128, 256, 64, 2
    (Q, K, V, G), (qf, kf, vf, gf), _ = _case(311, batch, 1, 1, q_seq, k_seq, head, dtype)
    q_pos0, k_pos0, offset = 160, 96, 30
    i = np.arange(q_seq)[:, None]
    j = np.arange(k_seq)[None, :]
    mask = (j + k_pos0) <= (i + q_pos0 + offset)
    add = np.where(mask, 0, -np.inf).astype(np.float32)
    A, af, lse = _forward(oracle, kf, qf, vf, add, batch, 1, dtype)
    want = oracle.sdpa_bwd_flash_f64(kf, qf, vf, af, gf, lse, add)
    Qc, Kc, Vc, Gc, Ac = (t.cuda() for t in (Q, K, V, G, A))
    lc = torch.from_numpy(lse).cuda()
    Kt, Vt = _split(Kc, k_tile), _split(Vc, k_tile)
    Qt, At, Gt, Lt = (_split(t, q_tile) for t in (Qc, Ac, Gc, lc))
    dKt, dVt = ([torch.zeros_like(t) for t in Kt] for _ in range(2))
    dQt = [torch.zeros_like(t) for t in Qt]
    hip_sdpa.sdpa_bwd_grid(Kt, Qt, Vt, At, Gt, Lt, dKt, dQt, dVt, q_seq, k_seq, q_tile, k_tile,
                           hip_sdpa.MASK_CAUSAL, q_pos0=q_pos0, k_pos0=k_pos0,
                           causal_offset=offset)
    torch.cuda.synchronize()
    for got, w, name in ((dKt, want[0], "dK"), (dQt, want[1], "dQ"), (dVt, want[2], "dV")):
        err = H.rel_fro(H.to_np(_join(got)), w)
        assert err < BWD_TOL[dtype], (name, err)


def test_refusals():
    """What the grid form does not take is refused before anything is
    launched, with the code the header documents."""
    batch, head, q_seq, k_seq = 2, 64, 256, 256
    mk = lambda rows: torch.zeros(batch, rows, head, dtype=torch.bfloat16, device="cuda")
    lse = lambda rows: torch.zeros(batch, rows, device="cuda")

    def call(q_tile, k_tile, mode=hip_sdpa.MASK_CAUSAL, workspace=None, n_q=None, n_kv=None,
             q_seq=q_seq, k_seq=k_seq):
        n_q = -(-q_seq // q_tile) if n_q is None else n_q
        n_kv = -(-k_seq // k_tile) if n_kv is None else n_kv
        Kt = [mk(k_tile) for _ in range(n_kv)]
        Qt = [mk(q_tile) for _ in range(n_q)]
        Lt = [lse(q_tile) for _ in range(n_q)]
        hip_sdpa.sdpa_bwd_grid(Kt, Qt, Kt, Qt, Qt, Lt, [mk(k_tile) for _ in Kt],
                               [mk(q_tile) for _ in Qt], [mk(k_tile) for _ in Kt], q_seq, k_seq,
                               q_tile, k_tile, mode, workspace=workspace)

    call(128, 128)      # the shape itself is fine
    torch.cuda.synchronize()
    for q_tile, k_tile in ((64, 128), (128, 64), (96, 128)):
        with pytest.raises(hip_sdpa.SdpaError) as e:
            call(q_tile, k_tile)
        assert e.value.code == hip_sdpa.EUNSUPPORTED, (q_tile, k_tile)
    for mode in (hip_sdpa.MASK_ADDITIVE, hip_sdpa.MASK_BOOL):
        with pytest.raises(hip_sdpa.SdpaError) as e:
            call(128, 128, mode=mode)
        assert e.value.code == hip_sdpa.EUNSUPPORTED
    with pytest.raises(hip_sdpa.SdpaError) as e:
        call(128, 128, mode=17)
    assert e.value.code == hip_sdpa.EINVAL
    with pytest.raises(hip_sdpa.SdpaError) as e:
        call(128, 128, n_q=3)       # tile count does not match the extent
    assert e.value.code == hip_sdpa.EINVAL
    with pytest.raises(hip_sdpa.SdpaError) as e:
        call(128, 128, workspace=torch.empty(4 * q_seq * batch - 4, dtype=torch.uint8,
                                             device="cuda"))
    assert e.value.code == hip_sdpa.EWORKSPACE
    # more tiles than the argument block holds
    with pytest.raises(hip_sdpa.SdpaError) as e:
        call(128, 128, q_seq=128 * (hip_sdpa.BWD_MAX_TILES + 1))
    assert e.value.code == hip_sdpa.EINVAL
    # a null tile pointer
    a = hip_sdpa.BwdGridArgs()
    a.q_seq = a.k_seq = a.q_tile = a.k_tile = 128
    a.head, a.batch, a.n_batch, a.kv_group = head, batch, batch, 1
    a.mask_mode, a.n_q_tiles, a.n_kv_tiles = hip_sdpa.MASK_NONE, 1, 1
    ws = torch.empty(4 * 128 * batch, dtype=torch.uint8, device="cuda")
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    assert hip_sdpa.lib().nntile_hip_sdpa_bwd_grid_bf16(None, ctypes.byref(a)) == hip_sdpa.EINVAL
    assert hip_sdpa.lib().nntile_hip_sdpa_bwd_grid_workspace_bytes(ctypes.byref(a)) == 4 * 128 * batch


@pytest.mark.parametrize("dtype,head", [("bf16", 64), ("bf16", 128), ("fp16", 32)])
@pytest.mark.parametrize("mode", ["causal", "none"])
@pytest.mark.parametrize("n_slabs,shape", [
    (4, (256, 256, 256, 256, 3, 1, 1)),     # one tile an axis, slabs along the batch
    (3, (384, 640, 128, 256, 1, 2, 2)),     # sequence tiles as well, grouped queries
    (2, (300, 520, 128, 384, 2, 1, 1)),     # ragged last tiles
    (8, (200, 200, 200, 200, 1, 1, 1)),     # one entry per slab
    # more workgroups than the chip holds at once: at head sizes up to 64 the
    # call over all slabs takes the workgroups that compute dK and dV
    # together, the calls per slab the separate ones
    (4, (1024, 1024, 1024, 1024, 12, 1, 1)),
])
def test_slabs_in_one_call(dtype, head, mode, n_slabs, shape):
    """Several slabs of the batch grid in one call (n_slabs) give, bit for
    bit, what one call per slab gives; the workspace grows with the slabs."""
    q_seq, k_seq, q_tile, k_tile, n_batch, group, n_kv = shape
    print("case bwd slabs", dtype, head, mode, n_slabs, shape, flush=True)
    offset = max(k_seq - q_seq, 0)
    mm = hip_sdpa.MASK_CAUSAL if mode == "causal" else hip_sdpa.MASK_NONE
    ins_all = [[] for _ in range(6)]        # K, Q, V, A, dA, lse
    acc_all, acc_one = [[] for _ in range(3)], [[] for _ in range(3)]
    for s in range(n_slabs):
        (Q, K, V, G), _, init = _case(400 + 3 * s, n_batch, group, n_kv, q_seq, k_seq, head, dtype)
        # any A and lse of the right shape do: both ways read the same ones
        A, _ = _rounded(0.5 * synth.randn(900 + s, 0, Q.numel()).reshape(Q.shape), dtype)
        lse = torch.from_numpy(np.log(np.arange(1, q_seq + 1, dtype=np.float32)
                                      )[None].repeat(Q.shape[0], 0).copy())
        tiles = [_split(t.cuda(), step) for t, step in
                 ((K, k_tile), (Q, q_tile), (V, k_tile), (A, q_tile), (G, q_tile), (lse, q_tile))]
        one = [_split(x[0].clone().cuda(), step)
               for x, step in zip(init, (k_tile, q_tile, k_tile))]
        hip_sdpa.sdpa_bwd_grid(*tiles, *one, q_seq, k_seq, q_tile, k_tile, mm, n_batch=n_batch,
                               kv_group=group, causal_offset=offset)
        for dst, src in zip(ins_all, tiles):
            dst += src
        for dst, src in zip(acc_one, one):
            dst += src
        for dst, x, step in zip(acc_all, init, (k_tile, q_tile, k_tile)):
            dst += _split(x[0].clone().cuda(), step)
    batch = n_batch * group * n_kv
    a = hip_sdpa.plan_bwd_grid(*ins_all, *acc_all, q_seq, k_seq, q_tile, k_tile, mm,
                               n_batch=n_batch, kv_group=group, causal_offset=offset,
                               n_slabs=n_slabs, workspace=torch.empty(1, dtype=torch.uint8,
                                                                      device="cuda"))
    assert (hip_sdpa.lib().nntile_hip_sdpa_bwd_grid_workspace_bytes(ctypes.byref(a._args))
            == 4 * n_slabs * q_seq * batch)
    hip_sdpa.sdpa_bwd_grid(*ins_all, *acc_all, q_seq, k_seq, q_tile, k_tile, mm, n_batch=n_batch,
                           kv_group=group, causal_offset=offset, n_slabs=n_slabs)
    torch.cuda.synchronize()
    for got, want, name in zip(acc_all, acc_one, ("dK", "dQ", "dV")):
        for t, (x, y) in enumerate(zip(got, want)):
            assert torch.equal(_bits(x), _bits(y)), (name, t)
    if q_tile == q_seq and k_tile == k_seq and group == 1:
        # one tile an axis: the slabs side by side in one allocation are a
        # batch of n_slabs * batch entries for the one-allocation form
        K1, Q1, V1, A1, G1, L1 = (torch.cat(t, dim=0) for t in ins_all)
        init1 = [torch.cat(t, dim=0) for t in acc_one]      # (shapes only)
        start = []
        for s in range(n_slabs):
            _, _, init = _case(400 + 3 * s, n_batch, group, n_kv, q_seq, k_seq, head, dtype)
            start.append([x[0].clone().cuda() for x in init])
        dK1, dQ1, dV1 = (torch.cat([st[i] for st in start], dim=0) for i in range(3))
        assert dK1.shape == init1[0].shape
        hip_sdpa.sdpa_bwd_tile(K1, Q1, V1, A1, G1, None, L1, dK1, dQ1, dV1, mm,
                               causal_offset=offset)
        torch.cuda.synchronize()
        for got, one, name in zip(acc_all, (dK1, dQ1, dV1), ("dK", "dQ", "dV")):
            assert torch.equal(_bits(torch.cat(got, dim=0)), _bits(one)), name
    # a workspace sized for one slab is refused
    with pytest.raises(hip_sdpa.SdpaError) as e:
        hip_sdpa.sdpa_bwd_grid(*ins_all, *acc_all, q_seq, k_seq, q_tile, k_tile, mm,
                               n_batch=n_batch, kv_group=group, causal_offset=offset,
                               n_slabs=n_slabs,
                               workspace=torch.empty(4 * q_seq * batch, dtype=torch.uint8,
                                                     device="cuda"))
    assert e.value.code == hip_sdpa.EWORKSPACE
