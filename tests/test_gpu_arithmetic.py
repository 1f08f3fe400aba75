"""GPU parity of Arithmetic.add_to_fp8 against the oracle, bit for bit, and the reference's own test
(tests/operators/test_arithmetic.py:25-42) on this implementation."""

import itertools

import pytest
import torch

import msamp    # noqa: F401
from msamp.common.dtype import Dtypes
from msamp.common.tensor import ScalingMeta
from msamp.nn import model_state
from msamp.operators.arithmetic import Arithmetic
from oracle import arithmetic as oarith, cast as ocast, fp8
from tests.gpu_util import FMT, same_float

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh_state():
    model_state.clear()
    ScalingMeta.in_time_scaling = True
    yield


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize('fp8_dt', [5, 6])
@pytest.mark.parametrize('n', [1, 5, 4096, 100003, 1 << 21])
def test_add_to_fp8_against_oracle(dtype, fp8_dt, n):
    g = torch.Generator().manual_seed(n + fp8_dt)
    x = (torch.randn(n, generator=g) * 3).to(dtype)
    om = ocast.new_meta()
    q = ocast.cast_to_fp8(x, om, FMT[fp8_dt], in_time=True)
    qd = q.cuda()
    meta = ScalingMeta(Dtypes.kfloat8_e4m3 if fp8_dt == 5 else Dtypes.kfloat8_e5m2, scale=om['scale'].clone().cuda(),
                       scale_inv=om['scale_inv'].clone().cuda(), amax=om['amax'].clone().cuda())
    for step in range(4):
        other = (torch.randn(n, generator=g) * (0.1 if step % 2 else 10.0)).to(dtype)
        q = oarith.add_to_fp8(q, om, FMT[fp8_dt], other)
        Arithmetic.add_to_fp8(qd, meta, other.cuda())
        assert torch.equal(qd.cpu(), q), step
        assert same_float(meta.scale, om['scale']) and same_float(meta.scale_inv, om['scale_inv'])
        assert same_float(meta.amax[0], om['amax'][0])


def test_add_to_fp8_as_the_reference_tests_it():
    torch.manual_seed(100)
    sizes = [1024, 3072]
    for i, j, dtype, qtype in itertools.product(sizes, sizes, [torch.float16, torch.bfloat16, torch.float32],
                                                [Dtypes.kfloat8_e4m3, Dtypes.kfloat8_e5m2]):
        input1 = torch.rand((i, j), dtype=dtype, device='cuda')
        t1 = input1.cast(qtype)
        t2 = input1.cast(qtype)
        for _ in range(3):
            input2 = torch.rand((i, j), dtype=dtype, device='cuda')
            Arithmetic.add_to_fp8(t1.value, t1.meta, input2)
            t2.copy_((t2.to(dtype) + input2).cast(qtype, meta=t2.meta))
            assert torch.equal(t1.value, t2.value)
            assert torch.equal(t1.meta.scale, t2.meta.scale) and torch.equal(t1.meta.scale_inv, t2.meta.scale_inv)
            assert torch.equal(t1.meta.amax, t2.meta.amax)


def test_add_to_fp8_misaligned_nan_and_errors():
    flat = torch.zeros(1001, dtype=torch.uint8, device='cuda')
    view = flat[1:]
    meta = ScalingMeta(Dtypes.kfloat8_e4m3)
    other = torch.arange(1000, dtype=torch.float32, device='cuda') - 500
    Arithmetic.add_to_fp8(view, meta, other)
    om = ocast.new_meta()
    want = oarith.add_to_fp8(torch.zeros(1000, dtype=torch.uint8), om, fp8.E4M3, other.cpu())
    assert torch.equal(view.cpu(), want) and meta.amax[0].item() == 500.0 and flat[0].item() == 0
    other[7] = float('nan')
    Arithmetic.add_to_fp8(view, meta, other)
    assert torch.isnan(meta.amax[0]).item() and view[7].item() & 0x7F == 0x7F
    with pytest.raises(ValueError):
        Arithmetic.add_to_fp8(view.cpu(), meta, other)
    with pytest.raises(ValueError):
        Arithmetic.add_to_fp8(torch.zeros(4, device='cuda'), meta, other[:4])
    with pytest.raises(ValueError):
        Arithmetic.add_to_fp8(view, ScalingMeta(Dtypes.kfloat16), other)
