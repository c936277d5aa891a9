"""GPU parity of the scaled transpose against the CPU checker, through the C
ABI.  Bound: the reference's |val / ref - 1| <= 10 eps
(tests/kernel/transpose.cc:57,88-91); the kernel does one product and one
rounding, so the results must in fact equal the rounded checker values."""
import numpy as np
import pytest
import torch

from nntile_amd import hip_sdpa, synth
from . import helpers as H
from .test_oracle_transpose import reference_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["fp32", "fp16", "bf16"])
@pytest.mark.parametrize("m,n", [(1, 9), (8, 9), (8, 1), (4, 7), (64, 64), (65, 129), (1000, 37),
                                 (4096, 512), (1024, 32), (136, 40), (8, 8), (524288, 32)])
@pytest.mark.parametrize("alpha", [-2.0, 1.0])
def test_against_checker(oracle, dtype, m, n, alpha):
    print("case transpose", dtype, m, n, alpha, flush=True)
    x = reference_case(m, n) if m * n < 100 else synth.randn(80, 0, m * n)
    X, xf = H.rounded(x, dtype)
    want, _ = H.rounded(oracle.transpose(m, n, alpha, xf), dtype)
    D = torch.full((m * n,), float("nan"), dtype=H.TORCH_DT[dtype], device="cuda")
    Xc = X.cuda()
    hip_sdpa.transpose(alpha, Xc, D, m, n)
    torch.cuda.synchronize()
    assert torch.equal(D.cpu().view(torch.int16 if dtype != "fp32" else torch.int32),
                       want.view(torch.int16 if dtype != "fp32" else torch.int32))
    assert torch.equal(Xc.cpu(), X)        # the source is not touched


def test_errors():
    x = torch.zeros(16, device="cuda")
    y = torch.zeros(16, device="cuda")
    fn = hip_sdpa.lib().nntile_hip_transpose_fp32
    assert fn(None, -1, 4, 1.0, x.data_ptr(), y.data_ptr()) == hip_sdpa.EINVAL
    assert fn(None, 4, 4, 1.0, x.data_ptr(), x.data_ptr()) == hip_sdpa.EINVAL
    assert fn(None, 4, 4, 1.0, None, y.data_ptr()) == hip_sdpa.EINVAL
    assert fn(None, 0, 4, 1.0, None, None) == hip_sdpa.OK
