"""Builds libnntile_hip_sdpa.so (hand-written HIP for gfx950) in-tree.

    python -m nntile_amd.build [--force]
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libnntile_hip_sdpa.so")
SOURCES = ["sdpa_prefill_16bit.hip", "sdpa_prefill_fp32.hip",
           "sdpa_decode_16bit.hip", "sdpa_decode_fp32.hip", "sdpa_bwd_16bit.hip", "rope.hip", "transpose.hip", "kv_cache.hip", "mask_classify.hip",
           "accumulate_attn_output.hip", "capi.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function"]


def _stale(obj, src):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [src] + [os.path.join(CSRC, f) for f in os.listdir(CSRC)
                    if f.endswith(".hpp")]
    deps.append(os.path.join(HERE, "..", "include", "nntile_hip_sdpa.h"))
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=True):
    objs = []
    procs = []
    for name in SOURCES:
        src = os.path.join(CSRC, name)
        obj = os.path.join(CSRC, name.replace(".hip", ".o"))
        objs.append(obj)
        if force or _stale(obj, src):
            cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
            if verbose:
                print(" ".join(cmd), flush=True)
            procs.append((name, subprocess.Popen(
                cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)))
    failed = False
    for name, proc in procs:
        out = proc.communicate()[0].decode()
        out = "\n".join(l for l in out.splitlines()
                        if "packed-fp32-ops" not in l and l.strip())
        if out and verbose:
            print(out)
        if proc.returncode != 0:
            failed = True
            print("FAILED: " + name, file=sys.stderr)
    if failed:
        raise RuntimeError("hipcc failed")
    if force or procs or not os.path.exists(LIB):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-o", LIB] + objs
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
