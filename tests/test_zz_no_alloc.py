"""The entry point that allocates nothing (mk_dev_mla_q8_decode_static: scratch in a device array inside the library)
against mk_dev_mla_q8_decode with a caller's workspace, through the C ABI: two calls in a row, the second on a smaller
input, each within relative L2 1e-5 of the existing entry point (the same kernels run, so the outputs are in fact equal
bit for bit) and, on the smaller inputs, of the CPU oracle, plus the size limit.  Collected last: it must pass alone in a fresh process and after all other tests."""
import ctypes as C

import numpy as np
import pytest

from gpu_util import dev, rel_l2, torch_cuda

pytestmark = pytest.mark.gpu


def run_both(ctx, nh, seed, oracle_check=False):
    torch = torch_cuda()
    from microkimi_amd import _lib, workloads
    from microkimi_amd._lib import check, cur_stream, lib, ptr
    _lib.require_device()
    L, R = workloads.MLA_LATENT, workloads.MLA_ROPE
    rng = np.random.default_rng(seed)
    lq, ls = workloads.q8_0_rows(rng.standard_normal((ctx, L)).astype(np.float32))
    rq, rs = workloads.q8_0_rows(rng.standard_normal((ctx, R)).astype(np.float32))
    q = dev(rng.standard_normal((nh, L + R)).astype(np.float32))
    lq, ls, rq, rs = dev(lq), dev(ls), dev(rq), dev(rs)
    ws = torch.empty(lib.mk_mla_decode_workspace_bytes(nh, L, ctx), dtype=torch.uint8, device="cuda")
    want = torch.empty((nh, L), device="cuda")
    check(lib.mk_dev_mla_q8_decode(ptr(lq), ptr(ls), ptr(rq), ptr(rs), ctx - 1, ptr(q), nh, L, R, workloads.MLA_SCALE, ptr(ws), ptr(want),
                                   cur_stream()))
    got = torch.full((nh, L), float("nan"), device="cuda")
    check(lib.mk_dev_mla_q8_decode_static(ptr(lq), ptr(ls), ptr(rq), ptr(rs), ctx - 1, ptr(q), nh, L, R, workloads.MLA_SCALE, ptr(got),
                                          cur_stream()))
    torch.cuda.synchronize()
    if oracle_check:
        # the existing entry point is itself held to the CPU restatement here, so that a mistake shared by both
        # entry points (they run the same kernels) cannot pass
        import oracle
        ref = oracle.mla_absorbed_decode(lq.cpu().numpy(), ls.cpu().numpy().astype(np.float32), rq.cpu().numpy(),
                                         rs.cpu().numpy().astype(np.float32), q.cpu().numpy(), nh, workloads.MLA_SCALE)
        assert rel_l2(got.cpu().numpy(), ref) <= 1e-5
    return got.cpu().numpy(), want.cpu().numpy()


def test_static_scratch_entry_point_two_calls_second_smaller():
    got, want = run_both(5000, 128, 1)   # many splits: partial outputs and statistics go through the scratch
    assert np.isfinite(got).all() and rel_l2(got, want) <= 1e-5
    got2, want2 = run_both(300, 20, 2, oracle_check=True)   # smaller: fewer splits, fewer heads; the scratch still holds the first call's data
    assert np.isfinite(got2).all() and rel_l2(got2, want2) <= 1e-5
    got3, want3 = run_both(40, 3, 3, oracle_check=True)     # a single split: no merge
    assert np.isfinite(got3).all() and rel_l2(got3, want3) <= 1e-5


def test_static_scratch_entry_point_rejects_what_it_cannot_hold():
    torch = torch_cuda()
    from microkimi_amd import _lib
    from microkimi_amd._lib import cur_stream, lib, ptr
    _lib.require_device()
    nh = lib.mk_mla_decode_static_max_heads() + 1
    L, R, ctx = 512, 64, 64
    z8 = torch.zeros((ctx, L), dtype=torch.int8, device="cuda")
    zs = torch.zeros((ctx, L // 32), dtype=torch.float16, device="cuda")
    q = torch.zeros((nh, L + R), device="cuda")
    out = torch.full((nh, L), 7.0, device="cuda")
    st = lib.mk_dev_mla_q8_decode_static(ptr(z8), ptr(zs), ptr(z8), ptr(zs), ctx - 1, ptr(q), nh, L, R, 1.0, ptr(out), cur_stream())
    assert st == -4 and b"at most" in lib.mk_last_error()   # MK_ERR_UNSUPPORTED, with a message that names the limit
    torch.cuda.synchronize()
    assert float(out.min()) == 7.0 and float(out.max()) == 7.0  # nothing written
