"""Checks on the generated GPU code that no run-time test would catch.

The kernels move K and V from global memory into LDS with
`global_load_lds_dwordx4`, issued from assembly text that writes M0 (the LDS
target) without the compiler knowing.  That is safe only while the compiler
itself never uses M0 in these kernels; this test compiles every kernel source
to gfx950 assembly and looks.  It also checks that the packed-fp32
instructions, which the build switches off, do not appear."""
import os
import re
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

import pytest

from nntile_amd import build as B

KERNEL_SOURCES = [s for s in B.SOURCES if s != "capi.hip"]
# the helper's first line: the LDS target from a scalar register (which may be
# one half of VCC when the kernel is short of SGPRs)
M0_WRITE = r"s_mov_b32 m0, (s\d+|vcc_lo|vcc_hi)"


def _assembly(name, outdir):
    src = os.path.join(B.CSRC, name)
    out = os.path.join(outdir, name + ".s")
    flags = [f for f in B.FLAGS if f != "-fPIC"]
    subprocess.run([B.HIPCC] + flags + ["-S", "--cuda-device-only", "-o", out, src],
                   check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    with open(out) as f:
        return f.read()


@pytest.fixture(scope="module")
def assemblies():
    if not os.path.exists(B.HIPCC):
        pytest.skip("hipcc not found")
    with tempfile.TemporaryDirectory() as d:
        with ThreadPoolExecutor(max_workers=4) as ex:
            texts = list(ex.map(lambda n: _assembly(n, d), KERNEL_SOURCES))
    return dict(zip(KERNEL_SOURCES, texts))


def _instructions(text):
    for line in text.splitlines():
        line = line.split(";")[0].strip()
        if line and not line.startswith(".") and not line.endswith(":"):
            yield line


def test_m0_is_written_only_by_the_lds_load_helper(assemblies):
    uses = 0
    for name, text in assemblies.items():
        ins = list(_instructions(text))
        for i, line in enumerate(ins):
            if not re.search(r"\bm0\b", line):
                continue
            # the helper's three lines: s_mov_b32 m0, sN / s_nop 0 / global_load_lds_dwordx4
            assert re.fullmatch(M0_WRITE, line), (name, line)
            assert ins[i + 1] == "s_nop 0", (name, ins[i + 1])
            assert ins[i + 2].startswith("global_load_lds_dwordx4 "), (name, ins[i + 2])
            uses += 1
    assert uses > 0     # the prefill and decode kernels do use the helper


# Instructions that read or write M0 without naming it: relative register
# addressing, the GPR index mode, messages, global wave sync, LDS parameter
# and direct loads, and LDS instructions in the add-TID form.  (An "m0"
# clobber on the helper's assembly text is not an alternative: M0 is a
# reserved register for the compiler, which warns that such a clobber is not
# honoured.)
IMPLICIT_M0 = (r"^(s_movrel[sd]_|v_movrel[sd]|v_movrelsd|s_set_gpr_idx_|s_sendmsg|s_sendmsghalt|"
               r"ds_gws_|v_interp_|lds_param_load|lds_direct_load|ds_\w+_addtid_|s_ttracedata|"
               r"v_readlane_b32 \S+ \S+ m0|v_writelane_b32 \S+ \S+ m0)")


def test_no_instruction_uses_m0_implicitly(assemblies):
    for name, text in assemblies.items():
        for line in _instructions(text):
            assert not re.match(IMPLICIT_M0, line), (name, line)


def test_every_lds_load_sets_m0_first(assemblies):
    for name, text in assemblies.items():
        ins = list(_instructions(text))
        for i, line in enumerate(ins):
            if line.startswith("global_load_lds_"):
                assert i >= 2 and ins[i - 1] == "s_nop 0" \
                    and re.fullmatch(M0_WRITE, ins[i - 2]), (name, line)


def test_no_packed_fp32_instructions(assemblies):
    for name, text in assemblies.items():
        for line in _instructions(text):
            assert not re.match(r"v_pk_(add|mul|fma)_f32\b", line), (name, line)


def test_forward_kernels_use_no_scratch_memory(assemblies):
    """An array that the compiler could not keep in registers (a loop it did
    not unroll, a register index known only at run time) shows up as private
    scratch memory: slow, and with run-time indexing an implicit M0 user.  The
    fp32 and the decode kernels need none; of the 16-bit prefill kernel only
    the explicit-mask variants at head 128 spill a few registers (at most 16
    dwords a lane, written before the loop and read back after it)."""
    limits = {"sdpa_prefill_fp32.hip": 0, "sdpa_decode_16bit.hip": 0, "sdpa_decode_fp32.hip": 0,
              "sdpa_prefill_16bit.hip": 64}
    for name, limit in limits.items():
        sizes = re.findall(r"\.private_segment_fixed_size:\s*(\d+)", assemblies[name])
        assert sizes, name
        assert all(int(x) <= limit for x in sizes), (name, sorted(set(sizes)))


def test_backward_kernels_use_no_scratch_memory_without_an_explicit_mask(assemblies):
    """The backward at head 128 holds K and V fragments and both accumulators
    in 192 registers of a lane; what else lives through its loops was arranged
    so that nothing spills in the kernels without a mask and with the causal
    rule (every head size), and in every kernel below head 128.  The kernels
    that read mask values at head 128 keep at most 28 dwords a lane in
    scratch memory."""
    text = assemblies["sdpa_bwd_16bit.hip"].split("amdhsa.kernels:")[1]
    seen = 0
    for entry in text.split(".agpr_count:")[1:]:
        name = re.search(r"\.name:\s+(\S+)", entry).group(1)
        size = int(re.search(r"\.private_segment_fixed_size:\s*(\d+)", entry).group(1))
        m = re.match(r"_ZN10nntile_hip15sdpa_bwd_kernelINS_\w+?ELi(\d+)ELi(\d+)E", name)
        if m is None:
            assert size == 0, (name, size)
            continue
        seen += 1
        head, mode = int(m.group(1)), int(m.group(2))
        explicit = mode in (0, 3)           # NNTILE_HIP_MASK_ADDITIVE, NNTILE_HIP_MASK_BOOL
        assert size <= (112 if explicit and head == 128 else 0), (name, size)
    assert seen >= 48
