"""The entry point that allocates nothing (msamp_cast_to_fp8_intime_static: library-owned static workspace) against
msamp_cast_to_fp8_intime, through the C ABI: payload, amax, scale and scale_inv bit for bit, on two calls in a row,
the second with a smaller input, for the one-pass and the two-pass kernels."""

import ctypes

import pytest
import torch

from tests.gpu_util import same_float

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def be():
    from msamp import _backend
    _backend.load()
    return _backend


def _meta():
    return torch.full((), 3.0, device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')


def _pair(be, x, fp8_dt, two_pass):
    s0, si0, am0 = _meta()
    want = be.cast_to_fp8_intime(x, s0, am0, si0, fp8_dt, two_pass=two_pass)
    s1, si1, am1 = _meta()
    out = torch.full((x.numel(), ), 0xAA, dtype=torch.uint8, device='cuda')
    be.cast_to_fp8_intime_static(x, s1, am1, si1, out, fp8_dt, two_pass=two_pass)
    torch.cuda.synchronize()
    assert torch.equal(out.view(x.shape), want)
    assert same_float(am1, am0) and same_float(s1, s0) and same_float(si1, si0)


@pytest.mark.parametrize('two_pass', [False, True])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_static_workspace_matches_caller_workspace(be, dtype, two_pass):
    g = torch.Generator(device='cuda').manual_seed(7)
    big = (torch.randn(3 * 1024 * 1024 + 5, device='cuda', generator=g) * 2.5).to(dtype)
    small = (torch.randn(70001, device='cuda', generator=g) * 1e-3).to(dtype)
    # two calls in a row on the same static array, the second smaller: what the first left behind must not matter
    _pair(be, big, be.DT_E4M3, two_pass)
    _pair(be, small, be.DT_E5M2, two_pass)
    _pair(be, small[:3], be.DT_E4M3, two_pass)


def test_static_workspace_large_then_special_values(be):
    # beyond what the one-pass kernel holds (64 MiB): the two-pass kernels on the static array
    g = torch.Generator(device='cuda').manual_seed(8)
    x = torch.randn(40 * 1024 * 1024 + 17, device='cuda', generator=g)
    _pair(be, x, be.DT_E4M3, False)
    y = torch.randn(4099, device='cuda', generator=g)
    y[5], y[77], y[4098] = float('nan'), float('inf'), -float('inf')
    _pair(be, y, be.DT_E5M2, False)
    _pair(be, torch.zeros(513, device='cuda'), be.DT_E4M3, False)


def test_static_workspace_rejects_oversize_and_bad_arguments(be):
    lib = be.load()
    s, si, am = _meta()
    x = torch.zeros(16, device='cuda')
    out = torch.zeros(16, dtype=torch.uint8, device='cuda')
    args = lambda n: (x.data_ptr(), be.DT_F32, ctypes.c_size_t(n), s.data_ptr(), am.data_ptr(), si.data_ptr(), out.data_ptr(),
                      be.DT_E4M3, 0, 0, None)
    assert lib.msamp_cast_to_fp8_intime_static(*args(be.STATIC_MAX_ELEMS + 1)) == -2
    assert b'exceeds the limit' in lib.msamp_last_error()
    assert lib.msamp_cast_to_fp8_intime_static(x.data_ptr(), be.DT_F32, 16, None, am.data_ptr(), si.data_ptr(), out.data_ptr(),
                                               be.DT_E4M3, 0, 0, None) == -3
    assert lib.msamp_cast_to_fp8_intime_static(*args(0)) == 0
    torch.cuda.synchronize()


def test_static_workspace_reports_a_wait_that_ran_out(be):
    """With the spin limit forced to zero every wait of the one-pass kernel gives up at once (every kernel still runs
    to its end); the sticky word then sits in the library's own workspace, which a null workspace pointer stands for."""
    lib = be.load()
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.msamp_check_async_error(None, stream) == 0
    x = torch.randn(3 * 1024 * 1024 + 11, device='cuda')
    s, si, am = _meta()
    out = torch.empty(x.numel(), dtype=torch.uint8, device='cuda')
    be.set_spin_limit(0)
    try:
        be.cast_to_fp8_intime_static(x, s, am, si, out, be.DT_E4M3)
        torch.cuda.synchronize()
    finally:
        be.set_spin_limit(1 << 20)
    assert torch.isnan(am[0]).item() and s.item() == 3.0
    try:
        with pytest.raises(be.WaitExpiredError):
            be.check_async_error(block=True)
        assert be._force_two_pass
    finally:
        be._force_two_pass = False
    assert lib.msamp_check_async_error(None, stream) == 0    # reported once, then clear
    _pair(be, x, be.DT_E4M3, False)    # and the static array is as good as before
