"""The benchmark's result line must stay short: a driver that keeps only the
tail of stdout has to find the whole line there."""
import argparse
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_result_line_is_short_and_complete():
    b = _bench()
    from nntile_amd.configs import BY_NAME
    cfg3, cfg4 = BY_NAME["cfg3_llama_prefill_bf16"], BY_NAME["cfg4_gqa_decode_bf16"]
    args = argparse.Namespace(steps=500, warmup=50)
    main_leg = {"tflops": 1234.5678, "ms_per_step": 0.123456, "device_ms_per_step": 0.123123,
                "launches_per_step": 1}
    dec = {"ms_per_step": 0.0512345, "device_ms_per_step": 0.0501234, "gbs": 5432.123,
           "algorithmic_bytes": cfg4.algorithmic_bytes(), "workspace_bytes": 8650752, "tflops": 333.3}
    leg = {"ms_per_step": 0.151234, "launches_per_step": 16, "tflops": 912.34,
           "mask_classifications": 16, "mask_cache_hits": 123}
    ref_api = {"default_overload": leg, "every_pair": leg}
    backward = {"ms_per_step": 0.4567, "roofline": b.roofline("mfma", "k", 3.4e11, 0.4567, 2500.0, "TFLOP/s")}
    gemm = {"tflops": 1650.1, "kernel_ms": 0.6661, "watts": 1390.0}
    cpu = {"value": 0.07351234, "unit": "TFLOP/s", "cores": 16, "kind": "port",
           "sample": "16 of 32 (batch,head) slabs of cfg3_llama_prefill_bf16 x 1 passes, all 4096 "
                     "queries, key tiles of 1024; FLOPs counted causal-exact as for the GPU (the CPU "
                     "path computes the dense score matrix)", "seconds": 15.912345}
    kv = {"device_ms_per_step": 0.0531, "one_launch_device_ms_per_step": 0.0487,
          "one_launch_frac_of_hbm_peak": 0.6971}
    line = b.compact_line(main_leg, dec, ref_api, backward, gemm, cpu, args, cfg3, cfg4, 1300.0, kv)
    assert "\n" not in line and len(line) < b.LINE_LIMIT <= 4096
    out = json.loads(line)
    assert out["decode"]["through_cache"]["one_launch_ms"] == 0.0487
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline",
                "decode", "cpu_baseline"):
        assert key in out, key
    assert out["config"]["workload"] == "cfg3_llama_prefill_bf16"
    for r in (out["roofline"], out["decode"]["roofline"]):
        for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
            assert key in r, key
    assert out["roofline"]["bound"] == "mfma" and out["decode"]["roofline"]["bound"] == "hbm"
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in out["cpu_baseline"], key
