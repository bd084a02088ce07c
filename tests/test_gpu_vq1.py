"""GPU parity of the VQ1 LUT GEMV (mk_dev_vq1_matvec) against the oracle."""
import numpy as np
import pytest

import oracle
from gpu_util import dev, rel_l2, torch_cuda
from test_oracle_vq1 import SHAPES, Rng, case, nt_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols", SHAPES + [(2048, 7168), (7168, 2048), (5, 48), (300, 4112)])
def test_vq1_matvec(rows, cols):
    torch_cuda()
    from microkimi_amd import quant
    cb, idx, x = case(rows, cols, Rng(rows * 1000 + cols))
    want = oracle.vq1_matvec(cb, idx, rows, cols, x)
    exact = quant.matvec_vq(dev(cb), dev(idx), rows, cols, dev(x), exact=True).cpu().numpy()
    assert np.array_equal(exact.view(np.uint32), want.view(np.uint32))      # the reference's own bit-exactness contract
    fast = quant.matvec_vq(dev(cb), dev(idx), rows, cols, dev(x)).cpu().numpy()
    assert rel_l2(fast, want) <= 1e-5


def test_vq1_argument_checks():
    torch = torch_cuda()
    from microkimi_amd import quant
    cb = torch.zeros((256, 16), device="cuda")
    with pytest.raises(ValueError):
        quant.matvec_vq(cb, torch.zeros((4, 3), dtype=torch.uint8, device="cuda"), 4, 40, torch.zeros(40, device="cuda"))


@pytest.mark.parametrize("rows,cols,m", [(1, 16, 8), (7, 64, 8), (300, 208, 24), (512, 1408, 16), (2048, 7168, 8), (1000, 512, 64)])
def test_vq1_matvec_nt(rows, cols, m):
    torch_cuda()
    from microkimi_amd import quant
    cb, idx, xt = nt_case(rows, cols, m, rows * 131 + cols + m)
    want = oracle.vq1_matvec_nt(cb, idx, rows, cols, xt, m)
    got = quant.matvec_vq_nt(dev(cb), dev(idx), rows, cols, dev(xt), m).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))        # one multiply-add chain per (row, position)


def test_vq1_nt_argument_checks():
    torch = torch_cuda()
    from microkimi_amd import quant
    cb = torch.zeros((256, 16), device="cuda")
    with pytest.raises(ValueError):                                          # m must be a multiple of 8
        quant.matvec_vq_nt(cb, torch.zeros((4, 2), dtype=torch.uint8, device="cuda"), 4, 32, torch.zeros((32, 4), device="cuda"), 4)
