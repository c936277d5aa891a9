#!/usr/bin/env python3
"""Benchmark of the MI355X tile-level attention forward.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only NAME]

A "step" is one pass of the hot path over one batch of synthetic input that is
already resident in HBM: every launch that the workload needs (all tile pairs
of the Llama-shape prefill, cfg3).  Prints ONE JSON line.  `value` is the
whole-job SDPA-forward throughput in TFLOP/s on cfg3 counted on causal-exact
FLOPs; `roofline` prices the dominant kernel of that workload against the
dense bf16 MFMA peak; `decode` carries the HBM-bound GQA decode shape (cfg4)
with its own roofline; `cpu_baseline` is the CPU checker (a port of the
reference's CPU codelet composition) timed on this host on a bounded sample.
One GPU only.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_FP32_TFLOPS = 157.3      # MI355X fp32 matrix
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E


# HBM bytes per launch from the hardware counters (FETCH_SIZE x 2.000 +
# WRITE_SIZE x 1.000, the factors a 1 GiB device copy calibrates).  They are
# properties of the kernel and the workload, not of one timing run; each names
# the committed rocprofv3 summary it was read from.
TRAFFIC = {
    "cfg3_llama_prefill_bf16": (176977920, "profiles/sdpa_prefill_16bit_kernel_cfg3_llama_prefill_bf16.txt"),
    "cfg4_gqa_decode_bf16": (288403456, "profiles/sdpa_decode_16bit_kernel_cfg4_gqa_decode_bf16.txt"),
    "cfg2_gpt2_small_fp32": (55549952, "profiles/sdpa_prefill_fp32_kernel_cfg2_gpt2_small_fp32.txt"),
    # row dots (64 MiB read, 0.5 MiB written) + the gradient launch (488.9 MiB read, 96.1 MiB written)
    "cfg3_backward": (680994816, "profiles/sdpa_bwd_kernels_cfg3_llama_prefill_bf16.txt"),
}


def roofline(bound, kernel, work, ms, peak, unit, traffic=None, extra=None):
    """The roofline object of one leg: work (FLOPs or bytes) per step over the
    device time per step, against the published peak."""
    scale = 1e12 if bound == "mfma" else 1e9
    achieved = work / (ms * 1e-3) / scale
    r = {"bound": bound, "kernel": kernel, "achieved": round(achieved, 2), "peak": peak,
         "unit": unit, "frac": round(achieved / peak, 4), "kernel_ms": round(ms, 4),
         "traffic": None, "traffic_source": None}
    if traffic is not None:
        r["traffic"], r["traffic_source"] = traffic
    if extra:
        r.update(extra)
    return r


def time_steps(step, steps, warmup):
    """Runs `step` warmup times untimed, then exactly `steps` times between
    two device synchronisations.  Returns (wall ms per step, device ms per
    step); the device figure is one pair of HIP events recorded around the
    timed region on the stream the kernels are launched on (torch's current
    stream, which the library's stream argument is taken from)."""
    import torch
    for _ in range(warmup):
        step()
    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    a.record()
    for _ in range(steps):
        step()
    b.record()
    # spin on the closing event first: a blocking synchronize alone adds its
    # wake-up latency (of the order of a millisecond here) to the timed region
    while not b.query():
        pass
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    # the events sit inside the two host time stamps
    dev = min(a.elapsed_time(b) / steps, wall)
    return wall, dev


def _randn(shape, dtype, seed, stream=0):
    """i.i.d. N(0,1) values of stream (seed, stream) of the counter-based
    generator the parity tests use (nntile_amd/synth.py), evaluated on the
    GPU, in C order of `shape` (= Fortran order of the NNTile tile), rounded
    to the tile type."""
    import numpy as np
    from nntile_amd import synth
    n = int(np.prod(shape))
    return synth.randn_torch(seed, stream, n, "cuda").view(shape).to(dtype)


DATA = ("synthetic: i.i.d. N(0,1) from the counter-based generator of the parity tests "
        "(nntile_amd/synth.py: splitmix64 -> Box-Muller) evaluated on the GPU, seed 42 + config "
        "index, streams Q, K, V in that order, each tensor drawn in Fortran element order and "
        "rounded to the tile type; legs that rotate buffer sets draw the further sets from "
        "further streams")


def _outliers(cfg, q):
    """cfg5: the query positions (first floor(frac * seq) of a seeded
    permutation) scaled across all heads, as in the parity test."""
    if cfg.outlier_frac > 0:
        import torch
        from nntile_amd import synth
        rows = synth.permutation(cfg.seed, 7, cfg.q_seq)[:int(cfg.outlier_frac * cfg.q_seq)]
        q[:, torch.from_numpy(rows.copy()).cuda(), :] *= cfg.outlier_scale
    return q


class PowerSampler:
    """Board power in W from the amdgpu hwmon file, sampled every 50 ms by a
    thread while a loop runs; None where the file cannot be read."""

    def __init__(self):
        import glob
        files = glob.glob("/sys/class/drm/card*/device/hwmon/*/power1_input")
        self.path = files[0] if files else None
        self.samples = []

    def __enter__(self):
        import threading
        self.stop = threading.Event()

        def loop():
            while not self.stop.is_set():
                try:
                    with open(self.path) as f:
                        self.samples.append(int(f.read()) / 1e6)
                except (OSError, ValueError, TypeError):
                    pass
                time.sleep(0.05)
        self.thread = threading.Thread(target=loop)
        if self.path:
            self.thread.start()
        return self

    def __exit__(self, *exc):
        self.stop.set()
        if self.path:
            self.thread.join()

    def watts(self):
        # the first quarter of the samples is the ramp
        tail = self.samples[len(self.samples) // 4:]
        return round(sum(tail) / len(tail), 0) if tail else None


def bench_prefill(cfg, steps, warmup, zeros=False, settle_s=0.0, one_launch=True, more_flags=0):
    """The tensor-level call over cfg's whole tile grid (analytic causal mask,
    hidden tile pairs skipped, overwrite mode): one fused launch over all
    sequence tiles of all slabs of the batch grid (one_launch=False: one
    launch per slab).  Tiles are separate allocations, as NNTile tensors are.
    zeros=True replaces the inputs by zeros (for the power comparison only).
    settle_s: seconds of the same step run untimed before the warm-up steps,
    so that clock and power have settled on this load whatever ran before."""
    import torch
    from nntile_amd import hip_sdpa as h
    dt = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[cfg.dtype]
    per_call = cfg.batch_flat // cfg.calls
    nt = cfg.q_seq // cfg.seq_tile
    shape = (cfg.batch_flat, cfg.q_seq, cfg.head)
    q_all = _outliers(cfg, _randn(shape, torch.float32, cfg.seed, 0)).to(dt)
    k_all, v_all = _randn(shape, dt, cfg.seed, 1), _randn(shape, dt, cfg.seed, 2)
    if zeros:
        q_all.zero_(), k_all.zero_(), v_all.zero_()
    plans = []
    keep = []
    for c in range(cfg.calls):
        sl = slice(c * per_call, (c + 1) * per_call)
        tiles = lambda x: [x[sl, i * cfg.seq_tile:(i + 1) * cfg.seq_tile].contiguous() for i in range(nt)]
        Q, K, V = tiles(q_all), tiles(k_all), tiles(v_all)
        A = [torch.zeros_like(q) for q in Q]
        lse = [torch.full((per_call, cfg.seq_tile), float("-inf"), device="cuda") for _ in range(nt)]
        keep.append((Q, K, V, A, lse))
    if one_launch and cfg.calls * nt <= h.MAX_TILES:
        cat = lambda i: [t for slab in keep for t in slab[i]]
        plans.append(h.plan_grid(cat(1), cat(0), cat(4), cat(2), cat(3), cfg.q_seq, cfg.k_seq,
                                 cfg.seq_tile, cfg.seq_tile, h.MASK_CAUSAL,
                                 flags=h.OVERWRITE | more_flags, n_slabs=cfg.calls))
    else:
        for Q, K, V, A, lse in keep:
            plans.append(h.plan_grid(K, Q, lse, V, A, cfg.q_seq, cfg.k_seq, cfg.seq_tile,
                                     cfg.seq_tile, h.MASK_CAUSAL, flags=h.OVERWRITE | more_flags))
    del q_all, k_all, v_all

    def step():
        for pl in plans:
            pl.launch()

    if settle_s > 0:
        t_end = time.perf_counter() + settle_s
        while time.perf_counter() < t_end:
            for _ in range(100):
                step()
            torch.cuda.synchronize()
    wall, dev = time_steps(step, steps, warmup)
    return {"ms_per_step": wall, "device_ms_per_step": dev, "launches_per_step": len(plans),
            "tflops": cfg.flops() / (wall * 1e-3) / 1e12}


def bench_library_gemm(seconds, zeros=False):
    """A plain library GEMM (torch.matmul, 8192^3 bf16) in a loop of about
    `seconds` with the board power read beside it: the matrix rate this GPU
    sustains under its power cap on the benchmark's kind of data."""
    import torch
    n = 8192
    a = torch.zeros(n, n, dtype=torch.bfloat16, device="cuda") if zeros else \
        _randn((n, n), torch.bfloat16, 7, 0)
    b = torch.zeros_like(a) if zeros else _randn((n, n), torch.bfloat16, 7, 1)
    c = torch.empty_like(a)
    with PowerSampler() as ps:
        _, dev = time_steps(lambda: torch.matmul(a, b.t(), out=c), max(20, int(seconds / 0.6e-3)), 20)
    return {"tflops": round(2.0 * n ** 3 / (dev * 1e-3) / 1e12, 1), "kernel_ms": round(dev, 4),
            "watts": ps.watts()}


def bench_power_context(cfg, seconds=1.5, probe_lib=None):
    """What the chip sustains under its power cap, for context (--only
    power_context): the cfg3 prefill launch and a plain library GEMM, each on
    N(0,1) data and on zeros, in loops of about `seconds`, with the board power
    read beside them; with --probe-lib PATH also the matrix instruction alone
    on operands that stay in registers (PATH: a shared library that exports
    nntile_hip_probe_mfma(stream, operands, sink, iters, workgroups); none is
    built or shipped with the product).  The matrix units' power depends on
    the data: on zeros both run at the full clock, on random data both are
    held at the power cap.  Not a roofline - the published peak stays the
    yardstick."""
    import torch
    out = {"what": "loops of ~%.1f s; TFLOP/s and board power (W, amdgpu hwmon); the GEMM is the "
                   "library's (torch.matmul 8192^3 bf16); mfma_only: v_mfma_f32_32x32x16_bf16 on "
                   "operands held in registers, two wavefronts per SIMD, nothing else" % seconds}
    for key, zeros in (("prefill_cfg3_randn", False), ("prefill_cfg3_zeros", True)):
        with PowerSampler() as ps:
            r = bench_prefill(cfg, int(seconds / 130e-6), 50, zeros=zeros)
        out[key] = {"tflops": round(cfg.flops() / (r["device_ms_per_step"] * 1e-3) / 1e12, 1),
                    "kernel_ms": round(r["device_ms_per_step"], 4), "watts": ps.watts()}
    out["library_gemm_randn"] = bench_library_gemm(seconds)
    out["library_gemm_zeros"] = bench_library_gemm(seconds, zeros=True)
    if probe_lib:
        import ctypes
        probe = ctypes.CDLL(os.path.abspath(probe_lib)).nntile_hip_probe_mfma
        probe.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32,
                          ctypes.c_int32]
        sink = torch.zeros(1, device="cuda")
        iters, wgs = 20000, 512
        for key, zeros in (("mfma_only_randn", False), ("mfma_only_zeros", True)):
            ops = torch.zeros(8192, dtype=torch.bfloat16, device="cuda") if zeros else \
                _randn((8192,), torch.bfloat16, 9, 0)
            stream = torch.cuda.current_stream().cuda_stream

            def step():
                if probe(stream, ops.data_ptr(), sink.data_ptr(), iters, wgs) != 0:
                    raise RuntimeError("mfma probe failed")

            with PowerSampler() as ps:
                _, dev = time_steps(step, max(3, int(seconds / 2.5e-3)), 3)
            fl = wgs * 4 * iters * 4 * 32768.0
            out[key] = {"tflops": round(fl / (dev * 1e-3) / 1e12, 1), "kernel_ms": round(dev, 4),
                        "watts": ps.watts()}
    return out


def bench_copy_context(steps, warmup):
    """The runtime's plain device-to-device copy (torch's copy_) of 32 MiB and
    128 MiB, buffers rotating: what a read-once / write-once stream of the size
    of the rotary-embedding and transpose workloads reaches on this GPU."""
    import torch
    out = {"what": "hipMemcpy-class device copy, read + written bytes over device time; the "
                   "HBM-bound helper kernels (rope, transpose, accumulate) move the same kind "
                   "of stream"}
    for mib, nrot in ((32, 8), (128, 4)):
        srcs = [torch.empty(mib << 20, dtype=torch.uint8, device="cuda").fill_(j + 1) for j in range(nrot)]
        dsts = [torch.empty_like(x) for x in srcs]
        i = [0]

        def step():
            j = i[0] % nrot
            dsts[j].copy_(srcs[j])
            i[0] += 1
        _, dev = time_steps(step, steps, warmup)
        gbs = 2.0 * (mib << 20) / (dev * 1e-3) / 1e9
        out["%d_MiB" % mib] = {"device_ms": round(dev, 4), "gbs": round(gbs, 1),
                               "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4)}
    return out


def bench_reference_grid(steps, warmup, case=None):
    """The reference's own benchmark grid for this kernel
    (tests/kernel/flash_sdpa_fwd_cudnn.cc:591-613): seq in {128, 1024, 4096} x
    head in {64, 128} x batch in {4, 8} x {causal, full} x {bf16, fp16}, one
    square tile, random data.  Each case twice: through
    nntile_hip_flash_sdpa_fwd_* with the additive mask tile and the two scratch
    tiles the reference passes (merge into an lse of -inf, as its test does;
    masks of 1 MiB and more are scanned once per call into the scratch
    logsumexp tile by a small kernel of its own), and through the tile
    entry point with the same mask given analytically (overwrite mode).
    FLOPs: 4 * head * visible pairs * batch (causal-exact for the causal mask).
    `case` = "dtype,seq,head,batch,mask" restricts the run to that one case
    (for a profiler)."""
    import numpy as np
    import torch
    from nntile_amd import hip_sdpa as h, synth
    rows = []
    want = case.split(",") if case else None
    take = lambda i, v: want is None or i >= len(want) or want[i] in ("", "*", str(v))
    for dtype, dt in (("bf16", torch.bfloat16), ("fp16", torch.float16)):
        if not take(0, dtype):
            continue
        for seq in (128, 1024, 4096):
            if not take(1, seq):
                continue
            vis = synth.causal_mask(seq, seq)
            masks = {"causal": torch.from_numpy(np.where(vis, 0.0, -np.inf).astype(np.float32)).to(dt).cuda(),
                     "full": torch.zeros((seq, seq), dtype=dt, device="cuda")}
            for head in (64, 128):
                for batch in (4, 8):
                    if not (take(2, head) and take(3, batch)):
                        continue
                    shape = (batch, seq, head)
                    Q, K, V = (_randn(shape, dt, 42, i) for i in range(3))
                    A = torch.zeros_like(Q)
                    lse = torch.empty((batch, seq), dtype=torch.float32, device="cuda")
                    # the reference's two scratch tiles (STARPU_SCRATCH handles)
                    scratch_lse, scratch_A = torch.empty_like(lse), torch.empty_like(A)
                    for mask_type in ("causal", "full"):
                        if not take(4, mask_type):
                            continue
                        pairs = seq * (seq + 1) // 2 if mask_type == "causal" else seq * seq
                        flops = 4.0 * head * pairs * batch
                        m = masks[mask_type]
                        additive = h.FlashPlan(K, Q, m, lse, V, A, scratch_lse, scratch_A)

                        def with_mask():
                            lse.fill_(float("-inf"))
                            additive.launch()

                        analytic = h.plan_tile(K, Q, None, lse, V, A,
                                               h.MASK_CAUSAL if mask_type == "causal" else h.MASK_NONE,
                                               flags=h.OVERWRITE)
                        _, dev_mask = time_steps(with_mask, steps, warmup)
                        _, dev_an = time_steps(analytic.launch, steps, warmup)
                        tf_mask = flops / (dev_mask * 1e-3) / 1e12
                        tf_an = flops / (dev_an * 1e-3) / 1e12
                        rows.append({"dtype": dtype, "seq": seq, "head": head, "batch": batch,
                                     "mask": mask_type,
                                     "additive_mask_ms": round(dev_mask, 4),
                                     "additive_mask_tflops": round(tf_mask, 1),
                                     "additive_mask_frac": round(tf_mask / PEAK_BF16_TFLOPS, 4),
                                     "analytic_ms": round(dev_an, 4),
                                     "analytic_tflops": round(tf_an, 1),
                                     "analytic_frac": round(tf_an / PEAK_BF16_TFLOPS, 4)})
    return {"what": "the reference's benchmark grid (tests/kernel/flash_sdpa_fwd_cudnn.cc:591-613), one "
                    "square tile per case: additive_mask = nntile_hip_flash_sdpa_fwd_* with the "
                    "materialised mask (plus the -inf fill of lse), analytic = the same mask as a rule "
                    "(overwrite mode); device ms per call, TFLOP/s on causal-exact / dense FLOPs, "
                    "fraction of the 2.5 PFLOP/s bf16/fp16 MFMA peak",
            "cases": rows}


def bench_reference_api(cfg, steps, warmup):
    """cfg as an unchanged caller runs it: tensors tiled as the config says,
    a materialised additive causal mask [k_seq, q_seq], and per pass what
    Sdpa._forward_flash does (layer/sdpa.py:533-557) - logsumexp filled with
    -inf, then tensor::flash_sdpa_fwd_cudnn_async(K, Q, mask, logsumexp, V, A)
    with the reference's six arguments - through the C++ host mirror.  Timed
    with HIP events on the mirror's stream.  The mask is declared constant
    once, as a layer would after building it (its tiles are classified there
    and then); then the call with the reference's signature, the reference's
    submission literally (one task per tile pair), and the first again on a
    mask nothing was said about."""
    import numpy as np
    from nntile_amd import host_mirror as hm, synth
    assert cfg.dtype == "bf16" and cfg.kv_group == 1
    s5 = [cfg.head, cfg.q_seq, cfg.n_batch, 1, cfg.n_head_kv]
    b5 = [cfg.head, cfg.seq_tile, cfg.n_batch, 1, cfg.n_head_kv]
    n = int(np.prod(s5))
    T = {}
    import torch
    for i, name in enumerate(("Q", "K", "V")):
        bits = synth.randn_torch(cfg.seed, i, n, "cuda").to(torch.bfloat16).view(torch.int16) \
            .cpu().numpy().view(np.uint16)
        T[name] = hm.Tensor("bf16", s5, b5).from_array(bits.reshape(s5, order="F"))
    A = hm.Tensor("bf16", s5, b5).from_array(np.zeros(s5, np.uint16))
    lse = hm.Tensor("fp32", s5[1:], b5[1:]).from_array(np.full(s5[1:], -np.inf, np.float32))
    vis = synth.causal_mask(cfg.q_seq, cfg.k_seq)                # [q, k]
    add = synth.round_bf16(np.where(vis, 0.0, -np.inf).astype(np.float32).T)[0]   # [k, q]
    M = hm.Tensor("bf16", [cfg.k_seq, cfg.q_seq], [cfg.seq_tile, cfg.seq_tile]).from_array(
        np.asfortranarray(add))
    out = {}
    # what the layer says once after building its mask (blocking, untimed):
    # its contents stay as they are
    c0 = hm.mask_classifications()
    hm.mask_declare_constant(M)
    for key, op in (("default_overload", hm.OP_TENSOR), ("every_pair", hm.OP_PAIRS)):
        h0, m0 = hm.mask_cache_stats()
        ms, launches = hm.time_flash_sdpa_fwd(op, T["K"], T["Q"], M, lse, T["V"], A, steps, warmup)
        h1, m1 = hm.mask_cache_stats()
        out[key] = {"ms_per_step": round(ms, 4), "launches_per_step": launches,
                    "tflops": round(cfg.flops() / (ms * 1e-3) / 1e12, 2),
                    "mask_classifications": hm.mask_classifications() - c0,
                    "mask_cache_hits": h1 - h0}
    hm.mask_forget(M)
    ms, launches = hm.time_flash_sdpa_fwd(hm.OP_TENSOR, T["K"], T["Q"], M, lse, T["V"], A, steps, warmup)
    out["undeclared_mask"] = {"ms_per_step": round(ms, 4), "launches_per_step": launches,
                              "what": "the same call on a mask nothing was said about: the "
                                      "reference's submission, one task per tile pair"}
    return out


def bench_decode(cfg, steps, warmup, more_flags=0, fp32=False, settle_s=0.0):
    """The GQA decode shape: one launch per step (the key splits of a unit
    are merged inside it).  Four (K, V) sets rotate (4 x 256 MiB at cfg4: the
    256 MiB last-level cache cannot serve a pass).  more_flags: further flags
    of the decode call (the merge as a second launch).  fp32: the same shape
    on fp32 tiles through the fp32 decode kernel (twice the bytes).
    settle_s: seconds of the same step run untimed before the warm-up steps
    (the first loop of a process runs before the clocks have settled)."""
    import torch
    from nntile_amd import hip_sdpa as h
    kvb = cfg.n_batch * cfg.n_head_kv
    dt = torch.float32 if fp32 else torch.bfloat16
    nrot = 2 if fp32 else 4
    Ks = [_randn((kvb, cfg.k_seq, cfg.head), dt, cfg.seed, 1 + 10 * j) for j in range(nrot)]
    Vs = [_randn((kvb, cfg.k_seq, cfg.head), dt, cfg.seed, 2 + 10 * j) for j in range(nrot)]
    Q = _randn((cfg.batch_flat, cfg.q_seq, cfg.head), dt, cfg.seed, 0)
    A = torch.zeros_like(Q)
    lse = torch.full((cfg.batch_flat, cfg.q_seq), float("-inf"), device="cuda")
    ws = torch.empty(h.decode_workspace_bytes(Ks[0], Q, cfg.n_batch, cfg.kv_group),
                     dtype=torch.uint8, device="cuda")
    plans = [h.plan_decode(Ks[j], Q, None, lse, Vs[j], A, h.MASK_CAUSAL, cfg.n_batch, cfg.kv_group,
                           ws, causal_offset=cfg.causal_offset, flags=h.OVERWRITE | more_flags)
             for j in range(nrot)]
    i = [0]

    def step():
        plans[i[0] % nrot].launch()
        i[0] += 1

    if settle_s > 0:
        t_end = time.perf_counter() + settle_s
        while time.perf_counter() < t_end:
            for _ in range(50):
                step()
            torch.cuda.synchronize()
    wall, dev = time_steps(step, steps, warmup)
    nbytes = cfg.algorithmic_bytes()
    if fp32:
        # K, V, Q, A at 4 bytes an element; lse as before
        lse_bytes = 4 * cfg.batch_flat * cfg.q_seq
        nbytes = 2 * (nbytes - lse_bytes) + lse_bytes
    return {"ms_per_step": wall, "device_ms_per_step": dev,
            "gbs": nbytes / (wall * 1e-3) / 1e9, "algorithmic_bytes": nbytes,
            "workspace_bytes": ws.numel(), "tflops": cfg.flops() / (wall * 1e-3) / 1e12}


def bench_backward(cfg, steps, warmup):
    """Backward of the same attention (dQ, dK, dV from dA, A and lse) as one
    call over the whole sequence with the analytic causal mask: the row dots,
    then one launch for the three gradients.  FLOPs counted as 2.5 x the
    forward's (five products where the forward has two); the workgroups
    execute eight, recomputing the scores for each gradient."""
    import torch
    from nntile_amd import hip_sdpa as h
    dt = {"bf16": torch.bfloat16, "fp16": torch.float16}[cfg.dtype]
    shape = (cfg.batch_flat, cfg.q_seq, cfg.head)
    Q, K, V, G = (_randn(shape, dt, cfg.seed, i) for i in range(4))
    A = torch.zeros_like(Q)
    lse = torch.full((cfg.batch_flat, cfg.q_seq), float("-inf"), device="cuda")
    h.sdpa_fwd_tile(K, Q, None, lse, V, A, h.MASK_CAUSAL, flags=h.OVERWRITE)
    dK, dQ, dV = (torch.zeros_like(Q) for _ in range(3))
    ws = torch.empty(h.sdpa_bwd_workspace_bytes(cfg.q_seq, cfg.q_seq, cfg.batch_flat, h.MASK_CAUSAL),
                     dtype=torch.uint8, device="cuda")

    def step():
        h.sdpa_bwd_tile(K, Q, V, A, G, None, lse, dK, dQ, dV, h.MASK_CAUSAL,
                        flags=h.OVERWRITE, workspace=ws)

    wall, dev = time_steps(step, steps, warmup)
    fl = 2.5 * cfg.flops()
    # the same gradients over the reference's tiling (separately allocated
    # sequence tiles, gradients added to the tiles as the reference's
    # operation does): one call for all tile pairs
    tile = cfg.seq_tile
    cut = lambda t: [t[:, s:s + tile].contiguous() for s in range(0, cfg.q_seq, tile)]
    Kt, Qt, Vt, At, Gt, Lt = (cut(t) for t in (K, Q, V, A, G, lse))
    dKt, dQt, dVt = ([torch.zeros_like(t) for t in Qt] for _ in range(3))
    plan = h.plan_bwd_grid(Kt, Qt, Vt, At, Gt, Lt, dKt, dQt, dVt, cfg.q_seq, cfg.q_seq, tile, tile,
                           h.MASK_CAUSAL, ws)
    wall_t, dev_t = time_steps(plan.launch, steps, warmup)
    return {"workload": cfg.name, "ms_per_step": round(wall, 4), "flops_per_step": fl,
            "what": "backward of %s in one call (row dots + one launch for dQ, dK, dV), analytic "
                    "causal mask, gradients written; 2.5 x the forward's causal-exact FLOPs" % cfg.name,
            "roofline": roofline("mfma", "sdpa_bwd_rowdot_kernel + sdpa_bwd_kernel<bf16,128,causal>",
                                 fl, dev, PEAK_BF16_TFLOPS, "TFLOP/s", TRAFFIC["cfg3_backward"]),
            "reference_tiling": {
                "what": "the same over %d x %d separately allocated tiles of %d rows, gradients "
                        "added to the tiles: nntile_hip_sdpa_bwd_grid, one call for all tile pairs "
                        "(row dots per query tile + one launch)" % (len(Qt), len(Kt), tile),
                "ms_per_step": round(wall_t, 4), "device_ms_per_step": round(dev_t, 4),
                "frac_of_peak": round(fl / (dev_t * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)}}


def bench_backward_slabs(cfg, steps, warmup):
    """Backward over a tensor whose batch axes are tiled (cfg.calls slabs of
    the batch grid, one sequence tile each): all slabs in one call (n_slabs of
    nntile_hip_sdpa_bwd_grid_args) against one call per slab."""
    import torch
    from nntile_amd import hip_sdpa as h
    dt = {"bf16": torch.bfloat16, "fp16": torch.float16}[cfg.dtype]
    per = cfg.batch_flat // cfg.calls
    seq = cfg.q_seq
    mk = lambda i: [_randn((per, seq, cfg.head), dt, cfg.seed, 10 * s + i) for s in range(cfg.calls)]
    Q, K, V, G = mk(0), mk(1), mk(2), mk(3)
    A = [torch.zeros_like(q) for q in Q]
    L = [torch.full((per, seq), float("-inf"), device="cuda") for _ in Q]
    h.sdpa_fwd_grid(K, Q, L, V, A, seq, seq, seq, seq, h.MASK_CAUSAL, flags=h.OVERWRITE,
                    n_slabs=cfg.calls)
    dK, dQ, dV = ([torch.zeros_like(q) for q in Q] for _ in range(3))
    ws = torch.empty(4 * cfg.calls * seq * per, dtype=torch.uint8, device="cuda")
    one = h.plan_bwd_grid(K, Q, V, A, G, L, dK, dQ, dV, seq, seq, seq, seq, h.MASK_CAUSAL, ws,
                          flags=h.OVERWRITE, n_slabs=cfg.calls)
    each = [h.plan_bwd_grid([K[i]], [Q[i]], [V[i]], [A[i]], [G[i]], [L[i]], [dK[i]], [dQ[i]],
                            [dV[i]], seq, seq, seq, seq, h.MASK_CAUSAL, ws, flags=h.OVERWRITE)
            for i in range(cfg.calls)]

    def per_slab():
        for pl in each:
            pl.launch()

    _, dev1 = time_steps(one.launch, steps, warmup)
    _, dev2 = time_steps(per_slab, steps, warmup)
    fl = 2.5 * cfg.flops()
    return {"what": "backward of %d slabs of %d heads x %d x %d (%s), causal, gradients written: one "
                    "call for all slabs against one call per slab" % (cfg.calls, per, seq, cfg.head,
                                                                       cfg.dtype),
            "one_call": {"device_ms_per_step": round(dev1, 4),
                         "tflops": round(fl / (dev1 * 1e-3) / 1e12, 1)},
            "one_call_per_slab": {"device_ms_per_step": round(dev2, 4),
                                  "tflops": round(fl / (dev2 * 1e-3) / 1e12, 1)}}


def bench_rope(cfg, steps, warmup):
    """Rotary embedding of the Q tensor of the workload (the step before the
    attention kernel): sin, cos of shape [head/2, seq], src and dst
    [head, seq, heads].  HBM-bound: reads src, writes dst; sin and cos are
    re-read from cache.  Eight buffer pairs rotate so that the 256 MiB
    last-level cache cannot serve a pass."""
    import torch
    from nntile_amd import hip_sdpa as h
    dt = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[cfg.dtype]
    half = cfg.head // 2
    # the angles of rotary embedding: position x 10000^(-2i/head)
    freq = 10000.0 ** (-torch.arange(half, device="cuda", dtype=torch.float64) * 2.0 / cfg.head)
    ang = (torch.arange(cfg.q_seq, device="cuda", dtype=torch.float64)[:, None] * freq[None, :]).float()
    sin, cos = torch.sin(ang).to(dt).contiguous(), torch.cos(ang).to(dt).contiguous()
    nrot = 8
    src = [_randn((cfg.batch_flat, cfg.q_seq, cfg.head), dt, cfg.seed, 10 * i) for i in range(nrot)]
    dst = [torch.empty_like(x) for x in src]
    i = [0]

    def step():
        j = i[0] % nrot
        h.rope(sin, cos, src[j], dst[j])
        i[0] += 1

    wall, dev = time_steps(step, steps, warmup)
    nbytes = 2 * src[0].numel() * src[0].element_size() + 2 * sin.numel() * sin.element_size()
    return {"what": "rotary embedding of the Q tensor of %s (%d MiB in, %d MiB out)"
                    % (cfg.name, src[0].numel() * src[0].element_size() >> 20,
                       src[0].numel() * src[0].element_size() >> 20),
            "device_ms_per_step": round(dev, 4), "algorithmic_bytes": nbytes,
            "gbs": round(nbytes / (dev * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (dev * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}


def bench_transpose(cfg, steps, warmup):
    """The transpose that follows the attention kernel (attention output
    [head, seq, heads] -> [heads, head, seq], llama_attention.py:622-625):
    m = head * seq, n = heads as one m x n matrix.  HBM-bound: reads and
    writes the tensor once; eight buffer pairs rotate."""
    import torch
    from nntile_amd import hip_sdpa as h
    dt = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[cfg.dtype]
    m, n = cfg.head * cfg.q_seq, cfg.batch_flat
    nrot = 8
    src = [_randn((n, m), dt, cfg.seed, 10 * i + 5) for i in range(nrot)]
    dst = [torch.empty_like(x) for x in src]
    i = [0]

    def step():
        j = i[0] % nrot
        h.transpose(1.0, src[j], dst[j], m, n)
        i[0] += 1

    wall, dev = time_steps(step, steps, warmup)
    nbytes = 2 * src[0].numel() * src[0].element_size()
    return {"what": "transpose of the attention output of %s (%d x %d, %d MiB)"
                    % (cfg.name, m, n, src[0].numel() * src[0].element_size() >> 20),
            "device_ms_per_step": round(dev, 4), "algorithmic_bytes": nbytes,
            "gbs": round(nbytes / (dev * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (dev * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}


def bench_accumulate(cfg, steps, warmup):
    """The running-pair merge on its own (accumulate_attn_output) on one
    attention tile of cfg: [head, seq_tile, heads] in the tile type plus the
    fp32 logsumexp rows.  HBM-bound: reads the two attention tiles and the two
    lse rows, writes one of each.  Eight buffer sets rotate."""
    import torch
    from nntile_amd import hip_sdpa as h
    dt = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[cfg.dtype]
    nrot = 8
    shape = (cfg.batch_flat, cfg.seq_tile, cfg.head)
    src = [_randn(shape, dt, cfg.seed, 10 * i + 6) for i in range(nrot)]
    dst = [_randn(shape, dt, cfg.seed, 10 * i + 7) for i in range(nrot)]
    src_lse = [_randn(shape[:2], torch.float32, cfg.seed, 10 * i + 8) for i in range(nrot)]
    dst_lse = [_randn(shape[:2], torch.float32, cfg.seed, 10 * i + 9) for i in range(nrot)]
    i = [0]

    def step():
        j = i[0] % nrot
        h.accumulate_attn_output(src_lse[j], src[j], dst_lse[j], dst[j])
        i[0] += 1

    wall, dev = time_steps(step, steps, warmup)
    nbytes = 3 * src[0].numel() * src[0].element_size() + 3 * src_lse[0].numel() * 4
    return {"what": "accumulate_attn_output on one %d x %d x %d tile of %s"
                    % (cfg.head, cfg.seq_tile, cfg.batch_flat, cfg.name),
            "device_ms_per_step": round(dev, 4), "algorithmic_bytes": nbytes,
            "gbs": round(nbytes / (dev * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (dev * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}


def bench_kv_cache(cfg, steps, warmup, one_launch_only=False):
    """One decode step through a preallocated key/value cache: the keys and
    values of the q_seq new tokens are appended (one launch for both), then
    the decode kernel reads the filled rows of the caches where they lie.  The
    caches hold twice the filled rows (capacity 2 x k_seq); four cache pairs
    rotate, as in the decode leg.  The reference's step copies the filled part
    of both caches out first (cache_utils.py:177-215): twice the bytes of the
    attention itself, which this path does not move."""
    import torch
    from nntile_amd import hip_sdpa as h
    kvb = cfg.n_batch * cfg.n_head_kv
    cap, nrot = 2 * cfg.k_seq, 4
    Ks = [_randn((kvb, cap, cfg.head), torch.bfloat16, cfg.seed, 1 + 10 * i) for i in range(nrot)]
    Vs = [_randn((kvb, cap, cfg.head), torch.bfloat16, cfg.seed, 2 + 10 * i) for i in range(nrot)]
    k_new = _randn((kvb, cfg.q_seq, cfg.head), torch.bfloat16, cfg.seed, 3)
    v_new = _randn((kvb, cfg.q_seq, cfg.head), torch.bfloat16, cfg.seed, 4)
    Q = _randn((cfg.batch_flat, cfg.q_seq, cfg.head), torch.bfloat16, cfg.seed, 0)
    A = torch.zeros_like(Q)
    lse = torch.full((cfg.batch_flat, cfg.q_seq), float("-inf"), device="cuda")
    ws = torch.empty(h.decode_cache_workspace_bytes(cfg.k_seq, Q, cfg.n_batch, cfg.kv_group),
                     dtype=torch.uint8, device="cuda")
    filled = cfg.k_seq - cfg.q_seq
    plans = [h.plan_decode_cache(Ks[j], Vs[j], cfg.k_seq, Q, None, lse, A, h.MASK_CAUSAL,
                                 cfg.n_batch, cfg.kv_group, ws, causal_offset=cfg.causal_offset,
                                 flags=h.OVERWRITE) for j in range(nrot)]
    i = [0]

    appends = [h.plan_kv_cache_append(k_new, v_new, Ks[j], Vs[j], filled) for j in range(nrot)]

    def step():
        j = i[0] % nrot
        appends[j].launch()
        plans[j].launch()
        i[0] += 1

    def append_only():
        appends[i[0] % nrot].launch()
        i[0] += 1

    fused = [h.plan_decode_append_cache(k_new, v_new, Ks[j], Vs[j], cfg.k_seq, Q, None, lse, A,
                                        h.MASK_CAUSAL, cfg.n_batch, cfg.kv_group, ws,
                                        causal_offset=cfg.causal_offset, flags=h.OVERWRITE)
             for j in range(nrot)]

    def one_launch():
        fused[i[0] % nrot].launch()
        i[0] += 1

    append_bytes = 2 * 2 * k_new.numel() * k_new.element_size()
    nbytes = cfg.algorithmic_bytes() + append_bytes
    if one_launch_only:
        # (for the profiler: the launch that appends and attends, nothing else)
        wall, dev_one = time_steps(one_launch, steps, warmup)
        return {"what": "append %d new tokens + decode over %d cached rows of %s in one launch"
                        % (cfg.q_seq, cfg.k_seq, cfg.name),
                "ms_per_step": round(wall, 4), "device_ms_per_step": round(dev_one, 4),
                "algorithmic_bytes": nbytes,
                "frac_of_hbm_peak": round(nbytes / (dev_one * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
    wall, dev = time_steps(step, steps, warmup)
    _, dev_append = time_steps(append_only, steps, 2)
    _, dev_one = time_steps(one_launch, steps, 5)
    # the same step as a HIP graph (one per cache pair), replayed
    graphs = []
    for j in range(nrot):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            appends[j].launch()
            plans[j].launch()
        graphs.append(g)

    def replay():
        graphs[i[0] % nrot].replay()
        i[0] += 1

    _, dev_graph = time_steps(replay, steps, 5)
    return {"what": "append %d new tokens + decode over %d cached rows of %s, cache capacity %d"
                    % (cfg.q_seq, cfg.k_seq, cfg.name, cap),
            "ms_per_step": round(wall, 4), "device_ms_per_step": round(dev, 4),
            "append_device_ms": round(dev_append, 4),
            "one_launch_device_ms_per_step": round(dev_one, 4),
            "one_launch_frac_of_hbm_peak": round(nbytes / (dev_one * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "graph_replay_device_ms_per_step": round(dev_graph, 4), "algorithmic_bytes": nbytes,
            "gbs": round(nbytes / (dev * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(nbytes / (dev * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "reference_copy_out_bytes_not_moved": 2 * 2 * kvb * cfg.k_seq * cfg.head * 2}


def cpu_baseline(cfg, target_seconds=15.0):
    """The CPU checker (port of the reference's gemm -> mask_scalar ->
    maxsumexp -> softmax_inplace -> gemm composition) on a bounded sample of
    cfg: a few (batch, head) slabs, all queries, key tiles as in cfg."""
    import numpy as np
    from oracle import cpu_oracle as o
    from nntile_amd import synth
    threads = o.max_threads()
    slabs = max(1, min(cfg.batch_flat, threads))
    shape = (slabs, cfg.q_seq, cfg.head)
    q = synth.round_bf16(synth.randn(cfg.seed, 0, int(np.prod(shape))).reshape(shape))[1]
    k = synth.round_bf16(synth.randn(cfg.seed, 1, int(np.prod(shape))).reshape(shape))[1]
    v = synth.round_bf16(synth.randn(cfg.seed, 2, int(np.prod(shape))).reshape(shape))[1]
    mask = synth.causal_mask(cfg.q_seq, cfg.k_seq)
    t0 = time.perf_counter()
    reps = 0
    while True:
        o.sdpa_vanilla(k, q, v, mask, k_tile=cfg.seq_tile)
        reps += 1
        dt = time.perf_counter() - t0
        if dt > target_seconds or reps >= 20:
            break
    per_slab = dt / (reps * slabs)
    fl = cfg.flops() / cfg.batch_flat
    return {"value": fl / per_slab / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sgemm": "builtin (the checker's own blocked kernel; no CBLAS headers in the image)",
            "sample": "%d of %d (batch,head) slabs of %s x %d passes, all %d queries, key tiles of %d; "
                      "FLOPs counted causal-exact as for the GPU (the CPU path computes the dense "
                      "score matrix)" % (slabs, cfg.batch_flat, cfg.name, reps, cfg.q_seq, cfg.seq_tile),
            "seconds": dt}


DETAIL_FILE = os.path.join("gpurun_out", "bench_detail.json")
LINE_LIMIT = 4000     # bytes; the driver keeps only the tail of stdout


def compact_line(main_leg, dec, ref_api, backward, gemm, cpu, args, cfg3, cfg4, watts=None,
                 kv_cache=None):
    """The ONE line printed last: the headline, both rooflines, the
    reference-signature path, the backward and the CPU baseline.  Everything
    else goes to DETAIL_FILE."""
    r3 = lambda x: round(x, 3)
    out = {
        "metric": "sdpa_fwd_tflops",
        "value": round(main_leg["tflops"], 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_leg["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic N(0,1), counter-based generator of the parity tests, seed 42 + config index, "
                "rounded to bf16",
        "config": {"workload": cfg3.name, "head_size": cfg3.head, "n_head": cfg3.n_head_kv,
                   "seq_len": cfg3.q_seq, "batch": cfg3.n_batch, "seq_tile": cfg3.seq_tile,
                   "mask": "causal", "flops_per_step_causal_exact": cfg3.flops(),
                   "launches_per_step": main_leg["launches_per_step"],
                   "timed": "one fused launch over the 4x4 grid of separately allocated tiles, analytic "
                            "causal mask, overwrite mode; value = causal-exact FLOPs / wall time per step"},
        "roofline": roofline("mfma", "sdpa_prefill_16bit_kernel<bf16,128,causal,8 wavefronts>", cfg3.flops(),
                             main_leg["device_ms_per_step"], PEAK_BF16_TFLOPS, "TFLOP/s",
                             TRAFFIC[cfg3.name]),
        "decode": {"workload": cfg4.name, "ms_per_step": round(dec["ms_per_step"], 4),
                   "value": round(dec["gbs"], 1), "unit": "GB/s",
                   "roofline": roofline("hbm", dec.get("kernel", "sdpa_decode_16bit_kernel"),
                                        dec["algorithmic_bytes"], dec["device_ms_per_step"],
                                        PEAK_HBM_GBS, "GB/s", TRAFFIC[cfg4.name])},
        "detail_file": DETAIL_FILE,
    }
    if gemm is not None:
        # the matrix rate the board sustains on this kind of data under its
        # power cap, measured in this run: context for roofline.frac, no
        # replacement for the published peak
        out["roofline"]["context"] = {"library_gemm_randn_tflops": gemm["tflops"],
                                      "library_gemm_watts": gemm["watts"], "prefill_watts": watts}
    if ref_api is not None:
        out["per_task_path"] = {
            "what": "cfg3 through tensor::flash_sdpa_fwd_cudnn_async with the reference's six arguments "
                    "(C++ host mirror) and a materialised causal mask that was declared constant once "
                    "(its tiles classified then): one task of the whole-grid codelet; every_pair = the "
                    "reference's one-task-per-tile-pair submission, also what an undeclared mask gets",
            "ms_per_step": ref_api["default_overload"]["ms_per_step"],
            "launches": ref_api["default_overload"]["launches_per_step"],
            "every_pair_ms_per_step": ref_api["every_pair"]["ms_per_step"],
            "every_pair_launches": ref_api["every_pair"]["launches_per_step"]}
    if backward is not None:
        out["backward"] = {"ms_per_step": backward["ms_per_step"],
                           "frac": backward["roofline"]["frac"],
                           "kernel_ms": backward["roofline"]["kernel_ms"]}
    if kv_cache is not None:
        # the decode step through the key/value cache: append + decode as two
        # launches and as one
        out["decode"]["through_cache"] = {
            "two_launches_ms": kv_cache["device_ms_per_step"],
            "one_launch_ms": kv_cache["one_launch_device_ms_per_step"],
            "one_launch_frac": kv_cache["one_launch_frac_of_hbm_peak"]}
    if cpu is not None:
        out["cpu_baseline"] = {"value": round(cpu["value"], 5), "unit": cpu["unit"], "cores": cpu["cores"],
                               "kind": cpu["kind"], "sample": cpu["sample"],
                               "seconds": round(cpu["seconds"], 2)}
    line = json.dumps(out)
    if len(line) > LINE_LIMIT:
        raise RuntimeError("bench.py: the result line is %d bytes, limit %d" % (len(line), LINE_LIMIT))
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--brief", action="store_true",
                    help="only the legs of the result line (headline, decode, reference signature, "
                         "backward, CPU baseline); no detail file")
    ap.add_argument("--case", default=None,
                    help="with --only reference_grid: one case, as dtype,seq,head,batch,mask "
                         "(e.g. bf16,4096,64,8,causal)")
    ap.add_argument("--probe-lib", default=None,
                    help="with --only power_context: a shared library exporting nntile_hip_probe_mfma "
                         "(the matrix instruction alone); not part of the product")
    ap.add_argument("--only", default=None,
                    help="run only this leg (for profiling): prefill | prefill_128_queries | cfg5 | cfg2 | decode | decode_separate_merge | decode_wide | decode_fp32 | "
                         "reference_api | reference_grid | power_context | copy_context | backward | backward_slabs | rope | transpose | accumulate | "
                         "kv_cache | kv_cache_one_launch | copy")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py: this path runs on ONE GPU; --gpus %d is not supported "
                         "(the path shards over (batch, kv head) with no exchange between GPUs)\n"
                         % args.gpus)
        sys.exit(2)

    import torch
    from nntile_amd import hip_sdpa as h
    from nntile_amd.configs import BY_NAME, Workload
    h.lib()      # fails loudly if the HIP library is not built
    torch.cuda.set_device(0)

    cfg3 = BY_NAME["cfg3_llama_prefill_bf16"]
    cfg4 = BY_NAME["cfg4_gqa_decode_bf16"]
    # cfg4's bytes as 64 sequences of 1024 cached keys: 512 (sequence, kv head)
    # units, one key split each, (lse, A) written by the main kernel
    cfg4_wide = Workload("cfg4_bytes_as_64_sequences_of_1024_keys", "bf16", 128, 16, 1024, 64, 4, 8,
                         1024, 1, 45, decode=True)
    only = args.only
    show = lambda r: print(json.dumps({k: (round(v, 4) if isinstance(v, float) else v)
                                       for k, v in r.items()}))
    legs = {"prefill": lambda: bench_prefill(cfg3, args.steps, args.warmup),
            "prefill_128_queries": lambda: bench_prefill(cfg3, args.steps, args.warmup,
                                                         more_flags=h.FORM_SHARED),
            "cfg5_128_queries": lambda: bench_prefill(BY_NAME["cfg5_long_seq_bf16"], args.steps,
                                                      args.warmup, more_flags=h.FORM_SHARED),
            "cfg5": lambda: bench_prefill(BY_NAME["cfg5_long_seq_bf16"], args.steps, args.warmup),
            "cfg2": lambda: bench_prefill(BY_NAME["cfg2_gpt2_small_fp32"], args.steps, args.warmup),
            "cfg2_per_slab": lambda: bench_prefill(BY_NAME["cfg2_gpt2_small_fp32"], args.steps,
                                                   args.warmup, one_launch=False),
            "decode": lambda: bench_decode(cfg4, args.steps, args.warmup),
            "decode_separate_merge": lambda: bench_decode(cfg4, args.steps, args.warmup,
                                                          h.DECODE_SEPARATE_MERGE),
            "decode_wide": lambda: bench_decode(cfg4_wide, args.steps, args.warmup),
            "decode_fp32": lambda: bench_decode(cfg4, args.steps, args.warmup, fp32=True),
            "reference_api": lambda: bench_reference_api(cfg3, args.steps, args.warmup),
            "reference_grid": lambda: bench_reference_grid(args.steps, args.warmup, args.case),
            "power_context": lambda: bench_power_context(cfg3, probe_lib=args.probe_lib),
            "copy_context": lambda: bench_copy_context(args.steps, args.warmup),
            "backward": lambda: bench_backward(cfg3, args.steps, args.warmup),
            "rope": lambda: bench_rope(cfg3, args.steps, args.warmup),
            "transpose": lambda: bench_transpose(cfg3, args.steps, args.warmup),
            "accumulate": lambda: bench_accumulate(cfg3, args.steps, args.warmup),
            "backward_slabs": lambda: bench_backward_slabs(
                __import__("dataclasses").replace(BY_NAME["cfg2_gpt2_small_fp32"],
                                                  name="cfg2_shape_in_bf16", dtype="bf16"),
                args.steps, args.warmup),
            "kv_cache": lambda: bench_kv_cache(cfg4, args.steps, args.warmup),
            "kv_cache_one_launch": lambda: bench_kv_cache(cfg4, args.steps, args.warmup, True)}
    if only == "copy":
        # calibration leg for the HBM traffic counters: a plain device copy
        # of 1 GiB (reads 2^30 bytes, writes 2^30 bytes per launch)
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(args.warmup + args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        return
    if only is not None:
        if only not in legs:
            sys.stderr.write("bench.py: unknown leg %r\n" % only)
            sys.exit(2)
        show(legs[only]())
        return

    # every leg is timed over at least 20 steps after at least 5 warm-up
    # steps, whatever --steps says; the secondary legs take a fifth of it
    steps = max(20, args.steps)
    warmup = max(5, args.warmup)
    few = max(20, args.steps // 5)
    dec = bench_decode(cfg4, max(steps, 100), max(warmup, 20), settle_s=0.3)
    ref_api = bench_reference_api(cfg3, few, 5)
    backward = bench_backward(cfg3, max(20, args.steps // 10), 5)
    detail = {}
    if not args.brief:
        detail["decode_many_sequences"] = (lambda r: {
            "workload": cfg4_wide.name,
            "what": "for information: cfg4's bytes as 64 sequences x 8 kv heads x 1024 keys, 16 new "
                    "tokens each; one key split per unit, no merge launch",
            "roofline": roofline("hbm", "sdpa_decode_16bit_kernel (single split)",
                                 r["algorithmic_bytes"], r["device_ms_per_step"],
                                 PEAK_HBM_GBS, "GB/s")})(bench_decode(cfg4_wide, few, 5))
        detail["decode_fp32"] = (lambda r: {
            "what": "for information: cfg4's shape on fp32 tiles through the fp32 split-key decode "
                    "(twice the bytes; 17.2 GFLOP of fp32 matrix work)",
            "device_ms_per_step": round(r["device_ms_per_step"], 4),
            "algorithmic_bytes": r["algorithmic_bytes"],
            "gbs": round(r["algorithmic_bytes"] / (r["device_ms_per_step"] * 1e-3) / 1e9, 1),
            "tflops": round(cfg4.flops() / (r["device_ms_per_step"] * 1e-3) / 1e12, 1),
            "frac_of_fp32_mfma_peak": round(cfg4.flops() / (r["device_ms_per_step"] * 1e-3) / 1e12
                                            / PEAK_FP32_TFLOPS, 4)})(
            bench_decode(cfg4, few, 5, fp32=True))
        detail["reference_bench_grid"] = bench_reference_grid(20, 5)
        extras = {}
        for name in ("cfg1_single_head_fp32", "cfg2_gpt2_small_fp32", "cfg5_long_seq_bf16"):
            c = BY_NAME[name]
            r = bench_prefill(c, few, 5)
            fp32 = c.dtype == "fp32"
            extras[name] = {
                "ms_per_step": round(r["ms_per_step"], 4), "tflops": round(r["tflops"], 2),
                "flops_causal_exact": c.flops(), "launches_per_step": r["launches_per_step"],
                "roofline": roofline("mfma", "sdpa_prefill_fp32_kernel<%d,causal>" % c.head if fp32
                                     else "sdpa_prefill_16bit_kernel<bf16,%d,causal>" % c.head,
                                     c.flops(), r["device_ms_per_step"],
                                     PEAK_FP32_TFLOPS if fp32 else PEAK_BF16_TFLOPS, "TFLOP/s",
                                     TRAFFIC.get(name))}
            if c.calls > 1:
                r1 = bench_prefill(c, few, 5, one_launch=False)
                extras[name]["one_launch_per_slab"] = {
                    "what": "the same with one launch per slab of the batch grid (%d launches)" % c.calls,
                    "ms_per_step": round(r1["ms_per_step"], 4), "tflops": round(r1["tflops"], 2),
                    "launches_per_step": r1["launches_per_step"]}
        # cfg2's tiling on 16-bit tiles (the shape of the reference's GPT-2 flash
        # path): the slabs of the batch grid in one launch and one by one
        import dataclasses
        gpt2_bf16 = dataclasses.replace(BY_NAME["cfg2_gpt2_small_fp32"], name="cfg2_shape_in_bf16",
                                        dtype="bf16")
        r, r1 = bench_prefill(gpt2_bf16, few, 5), bench_prefill(gpt2_bf16, few, 5, one_launch=False)
        extras[gpt2_bf16.name] = {
            "what": "for information: cfg2's shape and tiling on bf16 tiles",
            "ms_per_step": round(r["ms_per_step"], 4), "tflops": round(r["tflops"], 2),
            "launches_per_step": r["launches_per_step"],
            "frac_of_peak": round(r["tflops"] / PEAK_BF16_TFLOPS, 4),
            "one_launch_per_slab": {"ms_per_step": round(r1["ms_per_step"], 4),
                                    "tflops": round(r1["tflops"], 2),
                                    "launches_per_step": r1["launches_per_step"]},
            "backward": bench_backward_slabs(gpt2_bf16, few, 5)}
        detail["other_configs"] = extras
        detail["rope"] = bench_rope(cfg3, few, 5)
        detail["transpose"] = bench_transpose(cfg3, few, 5)
        detail["kv_cache"] = bench_kv_cache(cfg4, few, 5)
        detail["accumulate_attn_output"] = bench_accumulate(cfg3, few, 5)
    # the sustained matrix rate of the board on the same kind of data, for
    # roofline.context (a library GEMM for about half a second)
    gemm = bench_library_gemm(0.5)
    # The headline leg runs last and after 0.3 s of its own launch, untimed:
    # the first timed loop of a process, and a loop that follows another kind
    # of load (a copy, a library GEMM), measure up to 5 % slower than the same
    # loop a moment later (clock and power still settling), whatever the
    # warm-up count.  The W warm-up steps and the K timed steps follow.
    with PowerSampler() as ps:
        main_leg = bench_prefill(cfg3, args.steps, args.warmup, settle_s=0.3)
    cpu = None if args.no_cpu else cpu_baseline(cfg3)
    line = compact_line(main_leg, dec, ref_api, backward, gemm, cpu, args, cfg3, cfg4, ps.watts(),
                        detail.get("kv_cache"))
    if not args.brief:
        detail = dict({"headline": json.loads(line), "per_task_path": ref_api, "backward": backward,
                       "decode": dec}, **detail)
        try:
            os.makedirs(os.path.dirname(DETAIL_FILE), exist_ok=True)
            with open(DETAIL_FILE, "w") as f:
                json.dump(detail, f, indent=1)
        except OSError as e:
            sys.stderr.write("bench.py: detail file not written: %s\n" % e)
    print(line)


if __name__ == "__main__":
    main()
