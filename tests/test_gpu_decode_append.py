"""The append and the attention of a decode step in one launch: the caches
afterwards and (lse, A) are, bit for bit, what the append entry point followed
by the decode entry point make them."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa
from nntile_amd.kv_cache import KVCache
from . import helpers as H

pytestmark = pytest.mark.gpu


def _bits(t):
    t = t.detach().cpu().contiguous()
    return t.view(torch.int16 if t.element_size() == 2 else torch.int32).numpy()


def _two_ways(dtype, q_seq, rows_new, k_seq, cap, n_batch, group, n_kv, head, mode, flags=0, seed=5):
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), _ = H.make_qkv(seed, batch, q_seq, k_seq, head, dtype, kv_batch=kvb)
    Qd, Kd, Vd = Q.cuda(), K.cuda(), V.cuda()
    filled = k_seq - rows_new
    offset = k_seq - q_seq
    mask, mm = None, {"causal": hip_sdpa.MASK_CAUSAL, "none": hip_sdpa.MASK_NONE,
                      "bool": hip_sdpa.MASK_BOOL, "additive": hip_sdpa.MASK_ADDITIVE}[mode]
    if mode in ("bool", "additive"):
        rng = np.random.default_rng(seed)
        vis = rng.random((q_seq, k_seq)) < 0.7
        vis[:, 0] = True
        mask = torch.from_numpy(vis).cuda() if mode == "bool" else H.additive_mask(vis, dtype).cuda()
    ws = torch.empty(hip_sdpa.decode_cache_workspace_bytes(k_seq, Qd, n_batch, group),
                     dtype=torch.uint8, device="cuda")
    out = []
    for one_launch in (False, True):
        # rows behind the filled ones hold NaN: they must never reach a result
        Kc = torch.full((kvb, cap, head), float("nan"), dtype=H.TORCH_DT[dtype], device="cuda")
        Vc = torch.full_like(Kc, float("nan"))
        Kc[:, :filled] = Kd[:, :filled]
        Vc[:, :filled] = Vd[:, :filled]
        k_new = Kd[:, filled:].contiguous()
        v_new = Vd[:, filled:].contiguous()
        lse, A = H.fresh_outputs(batch, q_seq, head, dtype)
        if one_launch:
            hip_sdpa.sdpa_fwd_decode_append_cache(k_new, v_new, Kc, Vc, k_seq, Qd, mask, lse, A, mm,
                                                  n_batch, group, ws, causal_offset=offset, flags=flags)
        else:
            hip_sdpa.kv_cache_append(k_new, v_new, Kc, Vc, filled)
            hip_sdpa.sdpa_fwd_decode_cache(Kc, Vc, k_seq, Qd, mask, lse, A, mm, n_batch, group, ws,
                                           causal_offset=offset, flags=flags)
        torch.cuda.synchronize()
        out.append((_bits(lse), _bits(A), _bits(Kc), _bits(Vc)))
    return out


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("q_seq,rows_new,k_seq,cap,n_batch,group,n_kv,head", [
    (16, 16, 512, 1024, 2, 4, 4, 128),      # new rows fill the last part of a key step
    (1, 1, 300, 301, 3, 4, 2, 128),         # one token, ragged last step, units not a multiple of 8
    (1, 1, 257, 4096, 8, 4, 1, 64),         # the new row alone in its step
    (5, 5, 77, 77, 2, 8, 3, 128),           # the cache exactly full afterwards
    (16, 16, 1000, 4096, 1, 4, 8, 64),      # new rows straddle two key steps
    (4, 70, 200, 333, 2, 1, 4, 64),         # more new rows than queries and than a key step
    (3, 3, 3, 64, 1, 2, 8, 128),            # an empty cache: every row is new
    (16, 16, 2064, 4096, 8, 4, 1, 128),     # many splits per unit
])
@pytest.mark.parametrize("mode", ["causal", "none", "bool", "additive"])
def test_one_launch_equals_append_then_decode(dtype, q_seq, rows_new, k_seq, cap, n_batch, group, n_kv,
                                              head, mode):
    print("case", dtype, q_seq, rows_new, k_seq, cap, n_batch, group, n_kv, head, mode, flush=True)
    two, one = _two_ways(dtype, q_seq, rows_new, k_seq, cap, n_batch, group, n_kv, head, mode)
    for a, b, what in zip(two, one, ("lse", "A", "K cache", "V cache")):
        assert np.array_equal(a, b), what


@pytest.mark.parametrize("flags", [hip_sdpa.DECODE_SEPARATE_MERGE, hip_sdpa.DECODE_FENCED,
                                   hip_sdpa.OVERWRITE])
def test_one_launch_in_every_form_of_the_merge(flags):
    print("case flags", flags, flush=True)
    two, one = _two_ways("bf16", 16, 16, 1500, 2048, 4, 4, 2, 128, "causal", flags=flags)
    for a, b, what in zip(two, one, ("lse", "A", "K cache", "V cache")):
        assert np.array_equal(a, b), what


def test_refusals_leave_everything_alone():
    (Q, K, V), _ = H.make_qkv(1, 8, 1, 40, 128, "bf16", kv_batch=2)
    Qd = Q.cuda()
    Kc = torch.zeros((2, 64, 128), dtype=torch.bfloat16, device="cuda")
    Vc = torch.zeros_like(Kc)
    new = K.cuda()[:, :1].contiguous()
    ws = torch.empty(hip_sdpa.decode_cache_workspace_bytes(64, Qd, 1, 4), dtype=torch.uint8, device="cuda")
    lse, A = H.fresh_outputs(8, 1, 128, "bf16")
    before = _bits(A).copy()
    with pytest.raises(hip_sdpa.SdpaError):       # more rows than the cache holds
        hip_sdpa.sdpa_fwd_decode_append_cache(new, new, Kc, Vc, 65, Qd, None, lse, A, hip_sdpa.MASK_NONE,
                                              1, 4, ws)
    with pytest.raises(hip_sdpa.SdpaError):       # more new rows than rows
        big = K.cuda()[:, :8].contiguous()
        hip_sdpa.sdpa_fwd_decode_append_cache(big, big, Kc, Vc, 4, Qd, None, lse, A, hip_sdpa.MASK_NONE,
                                              1, 4, ws)
    torch.cuda.synchronize()
    assert not bool(Kc.any()) and not bool(Vc.any())
    assert np.array_equal(_bits(A), before)


@pytest.mark.parametrize("dtype", ["bf16", "fp16", "fp32"])
def test_cache_object_steps_one_launch_against_two(dtype):
    """Token by token through two KVCache objects, one with append + attend,
    one with append_attend: same caches, same outputs at every step."""
    n_batch, group, n_kv, head, cap = 2, 4, 4, 128, 160
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), _ = H.make_qkv(9, batch, cap, cap, head, dtype, kv_batch=kvb)
    Qd, Kd, Vd = Q.cuda(), K.cuda(), V.cuda()
    a, b = KVCache(cap), KVCache(cap)
    pos = 0
    for chunk in (37, 1, 1, 16, 1, 64, 1, 1, 3, 1):
        print("chunk", dtype, pos, chunk, flush=True)
        kn, vn = Kd[:, pos:pos + chunk].contiguous(), Vd[:, pos:pos + chunk].contiguous()
        q = Qd[:, pos:pos + chunk].contiguous()
        res = []
        for cache, fused in ((a, False), (b, True)):
            lse, A = H.fresh_outputs(batch, chunk, head, dtype)
            if fused:
                cache.append_attend(kn, vn, q, lse, A, n_batch, group)
            else:
                cache.append(kn, vn)
                cache.attend(q, lse, A, n_batch, group)
            torch.cuda.synchronize()
            res.append((_bits(lse), _bits(A)))
        pos += chunk
        assert len(a) == len(b) == pos
        assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1])
        assert np.array_equal(_bits(a.k[:, :pos]), _bits(b.k[:, :pos]))
        assert np.array_equal(_bits(a.v[:, :pos]), _bits(b.v[:, :pos]))


def test_cache_object_on_a_side_stream():
    """append_attend enqueued on a stream of its own (default priority) while
    the default stream is busy with something else: same bits as on the
    default stream."""
    n_batch, group, n_kv, head, cap = 2, 4, 4, 128, 96
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), _ = H.make_qkv(13, batch, cap, cap, head, "bf16", kv_batch=kvb)
    Qd, Kd, Vd = Q.cuda(), K.cuda(), V.cuda()
    side = torch.cuda.Stream()
    out = []
    for stream in (None, side):
        cache = KVCache(cap)
        cache.append(Kd[:, :40].contiguous(), Vd[:, :40].contiguous())
        torch.cuda.synchronize()
        res, pos = [], 40
        for chunk in (1, 16, 1, 3):
            kn, vn = Kd[:, pos:pos + chunk].contiguous(), Vd[:, pos:pos + chunk].contiguous()
            q = Qd[:, pos:pos + chunk].contiguous()
            lse, A = H.fresh_outputs(batch, chunk, head, "bf16")
            torch.cuda.synchronize()
            busy = torch.ones(1 << 22, device="cuda").cumsum(0)      # the default stream's own work
            cache.append_attend(kn, vn, q, lse, A, n_batch, group, stream=stream)
            torch.cuda.synchronize()
            res.append((_bits(lse), _bits(A)))
            pos += chunk
            del busy
        out.append((res, _bits(cache.k[:, :pos]), _bits(cache.v[:, :pos])))
    for (a_lse, a_A), (b_lse, b_A) in zip(out[0][0], out[1][0]):
        assert np.array_equal(a_lse, b_lse) and np.array_equal(a_A, b_A)
    assert np.array_equal(out[0][1], out[1][1]) and np.array_equal(out[0][2], out[1][2])


def test_cache_object_with_a_mask_given_as_values():
    """append_attend with a bool mask of the whole sequence (a window): the
    slice that goes with the cache AFTER the append, same bits as append +
    attend; a refused call leaves the cache object as it was."""
    n_batch, group, n_kv, head, cap = 1, 4, 8, 64, 80
    batch, kvb = n_batch * group * n_kv, n_batch * n_kv
    (Q, K, V), _ = H.make_qkv(17, batch, cap, cap, head, "fp16", kv_batch=kvb)
    Qd, Kd, Vd = Q.cuda(), K.cuda(), V.cuda()
    i, j = np.arange(cap)[:, None], np.arange(cap)[None, :]
    mask = torch.from_numpy((j <= i) & (i - j <= 24)).cuda()
    a, b = KVCache(cap), KVCache(cap)
    pos = 0
    for chunk in (30, 1, 7, 1, 16):
        kn, vn = Kd[:, pos:pos + chunk].contiguous(), Vd[:, pos:pos + chunk].contiguous()
        q = Qd[:, pos:pos + chunk].contiguous()
        res = []
        for cache, fused in ((a, False), (b, True)):
            lse, A = H.fresh_outputs(batch, chunk, head, "fp16")
            if fused:
                cache.append_attend(kn, vn, q, lse, A, n_batch, group, causal=False, mask=mask)
            else:
                cache.append(kn, vn)
                cache.attend(q, lse, A, n_batch, group, causal=False, mask=mask)
            torch.cuda.synchronize()
            res.append((_bits(lse), _bits(A)))
        pos += chunk
        assert len(a) == len(b) == pos
        assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1])
    # 25 rows left; 26 are refused by the two-launch path taken for them, and nothing moves
    kn = Kd[:, :26].contiguous()
    lse, A = H.fresh_outputs(batch, 26, head, "fp16")
    with pytest.raises(hip_sdpa.SdpaError):
        b.append_attend(kn, kn, Qd[:, :26].contiguous(), lse, A, n_batch, group)
    assert len(b) == pos
