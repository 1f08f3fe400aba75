"""The failure path of the kernels whose workgroups wait for each other (one-pass in-time cast, fused GEMM + cast),
forced from the host: with a spin limit of 0 every wait gives up at once, every kernel still runs to its end, the
sticky error word of the workspace is set, msamp_check_async_error / _backend.check_async_error report it, and the
two-pass kernels the process then switches to give the oracle's bytes."""

import pytest
import torch

from oracle import cast as ocast, fp8
from tests.gpu_util import make_meta, oracle_meta, same_float

pytestmark = pytest.mark.gpu


@pytest.fixture()
def be():
    from msamp import _backend
    _backend.load()
    _backend.check_async_error(block=True)    # start from clean workspaces
    yield _backend
    _backend.set_spin_limit(1 << 20)
    _backend._force_two_pass = False
    try:
        _backend.check_async_error(block=True)
    except _backend.WaitExpiredError:
        pass
    _backend._force_two_pass = False


def test_expired_wait_of_the_one_pass_cast_is_reported_and_the_two_pass_path_recovers(be):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3 * 1024 * 1024 + 11, generator=g)    # several workgroups of the one-pass kernel
    xd = x.cuda()
    s, si, am = make_meta(scale=4.0)
    be.set_spin_limit(0)
    be.cast_to_fp8_intime(xd, s, am[0:1], si, be.DT_E4M3)
    torch.cuda.synchronize()    # the kernel ran to its end although nobody waited for anybody
    assert torch.isnan(am[0]).item()              # the collecting workgroup posted its failure
    assert s.item() == 4.0 and si.item() == 0.25    # and kept the old scale
    with pytest.raises(be.WaitExpiredError):
        be.check_async_error(block=True)
    assert be._force_two_pass
    be.check_async_error(block=True)    # reported once, then clear
    # the process is on the two-pass kernels now, whatever the spin limit: same call, right bytes
    s, si, am = make_meta(scale=4.0)
    q = be.cast_to_fp8_intime(xd, s, am[0:1], si, be.DT_E4M3)
    om = oracle_meta(scale=4.0)
    want = ocast.cast_to_fp8(x, om, fp8.E4M3, in_time=True)
    assert torch.equal(q.cpu(), want)
    assert same_float(am[0], om['amax'][0]) and same_float(s, om['scale']) and same_float(si, om['scale_inv'])
    be.check_async_error(block=True)


def test_expired_wait_is_seen_by_the_check_that_never_synchronises(be):
    x = torch.randn(2 * 1024 * 1024, device='cuda')
    s, si, am = make_meta()
    be.check_async_error(block=False)    # requests copies of the (clean) error words
    torch.cuda.synchronize()
    be.check_async_error(block=False)
    be.set_spin_limit(0)
    be.cast_to_fp8_intime(x, s, am[0:1], si, be.DT_E5M2)
    be.set_spin_limit(1 << 20)
    torch.cuda.synchronize()
    seen = False
    for _ in range(3):    # the first call may still hold a copy requested before the failure
        try:
            be.check_async_error(block=False)
        except be.WaitExpiredError:
            seen = True
            break
        torch.cuda.synchronize()
    assert seen and be._force_two_pass


def test_expired_wait_of_the_fused_gemm_cast_is_reported(be):
    lib = be.load()
    g = torch.Generator(device='cuda').manual_seed(5)
    a = torch.randint(0, 120, (512, 256), dtype=torch.uint8, device='cuda', generator=g)
    b = torch.randint(0, 120, (768, 256), dtype=torch.uint8, device='cuda', generator=g)
    one = torch.ones((), device='cuda')
    s, si, am = make_meta(scale=2.0)
    be.set_spin_limit(0)
    q = be.fp8_gemm_cast(a, be.DT_E4M3, one, b, be.DT_E4M3, one, torch.bfloat16, be.DT_E4M3, s, am[0:1], si)
    torch.cuda.synchronize()
    assert q is not None and torch.isnan(am[0]).item() and s.item() == 2.0
    ws = be.workspace(a.device)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.msamp_check_async_error(ws.data_ptr(), stream) == be.ERR_TIMEOUT
    assert b'gave up waiting' in lib.msamp_last_error()
    assert lib.msamp_check_async_error(ws.data_ptr(), stream) == 0
    # with waiting restored the fused call gives what the two steps give
    be.set_spin_limit(1 << 20)
    s1, si1, am1 = make_meta(scale=2.0)
    q1 = be.fp8_gemm_cast(a, be.DT_E4M3, one, b, be.DT_E4M3, one, torch.bfloat16, be.DT_E4M3, s1, am1[0:1], si1)
    d = torch.empty(768, 512, dtype=torch.bfloat16, device='cuda')
    be.fp8_gemm(a, be.DT_E4M3, one, b, be.DT_E4M3, one, d)
    s2, si2, am2 = make_meta(scale=2.0)
    q2 = be.cast_to_fp8_intime(d, s2, am2[0:1], si2, be.DT_E4M3, two_pass=True)
    assert q1 is not None and torch.equal(q1, q2) and same_float(am1, am2) and same_float(s1, s2)
    assert lib.msamp_check_async_error(ws.data_ptr(), stream) == 0


def test_waiting_kernels_follow_the_stream_that_is_in_use(be):
    """The one-pass kernels are kept to one stream per device at a time, but a stream that has gone idle does not
    keep them: after a warm-up on a side stream the main stream gets them back (seen through the spin limit of zero,
    which only a one-pass kernel reacts to)."""
    x = torch.randn(2 * 1024 * 1024, device='cuda')

    def one_pass_ran():
        s, si, am = make_meta(scale=4.0)
        be.set_spin_limit(0)
        try:
            be.cast_to_fp8_intime(x, s, am[0:1], si, be.DT_E4M3)
            torch.cuda.synchronize()
        finally:
            be.set_spin_limit(1 << 20)
        gave_up = bool(torch.isnan(am[0]).item())
        if gave_up:
            with pytest.raises(be.WaitExpiredError):
                be.check_async_error(block=True)
            be._force_two_pass = False
        return gave_up

    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        assert one_pass_ran()        # the side stream takes the device over from the idle main stream
    assert one_pass_ran()            # and the main stream takes it back once the side stream is idle
    with torch.cuda.stream(side):
        # while the main stream is busy the side stream is refused and takes the two-pass kernels: right bytes, no NaN
        big = torch.randn(64 * 1024 * 1024, device='cuda')
        torch.cuda.current_stream().wait_stream(torch.cuda.default_stream())
    s0, si0, am0 = make_meta()
    for _ in range(40):
        be.cast_to_fp8_intime(big, s0, am0[0:1], si0, be.DT_E4M3)    # main stream: busy for a few milliseconds
    with torch.cuda.stream(side):
        s, si, am = make_meta(scale=4.0)
        be.set_spin_limit(0)
        try:
            be.cast_to_fp8_intime(x, s, am[0:1], si, be.DT_E4M3)
        finally:
            be.set_spin_limit(1 << 20)
        side.synchronize()
        assert not torch.isnan(am[0]).item()
    torch.cuda.synchronize()
    be.check_async_error(block=True)
