"""GPU tests of the msamp API surface on the HIP kernels: the reference's own test ideas
(tests/common/tensor, tests/nn, tests/optim, tests/test_initialize.py) on this implementation."""

import copy
import itertools
from functools import partial

import pytest
import torch

import msamp
from msamp.common.dtype import Dtypes
from msamp.common.tensor import ScalingMeta, ScalingTensor, TypeCast
from msamp.nn import FP8Linear, LinearReplacer, ScalingParameter, model_state
from msamp.optim import DSAdam, LBAdam, LBAdamW, LBAdamWBase
from oracle import cast as ocast, fp8, gemm as ogemm
from tests.gpu_util import rel_fro, same_float

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh_state():
    model_state.clear()
    ScalingMeta.in_time_scaling = True
    yield
    model_state.clear()


def test_cast_fp8_and_fp16_round_trip():
    torch.manual_seed(100)
    x16 = torch.rand((4, 4), dtype=torch.float16, device='cuda')
    meta = ScalingMeta(Dtypes.kfloat8_e4m3)
    q = TypeCast.cast_to_fp8(x16, meta)
    assert q.dtype == torch.uint8 and q.shape == x16.shape
    assert torch.allclose(x16, TypeCast.cast_from_fp8(q, meta, Dtypes.kfloat16), 0, 0.1)
    x32 = torch.rand((4, 4), device='cuda')
    meta = ScalingMeta(Dtypes.kfloat16)
    h = TypeCast.cast_to_fp16(x32, meta)
    assert h.dtype == torch.float16
    assert torch.allclose(x32, TypeCast.cast_from_fp16(h, meta, Dtypes.kfloat32), 0, 1e-3)
    with pytest.raises(ValueError):
        TypeCast.cast_from_fp8(x16, meta, Dtypes.kfloat32)


def test_scaling_tensor_casts_and_scale_ops():
    torch.manual_seed(0)
    x = torch.randn(64, 48, device='cuda') * 1e-3
    st = x.cast(Dtypes.kfloat16)
    assert st.dtype == torch.float16 and st.qtype == Dtypes.kfloat16
    assert torch.allclose(st.float(), x, rtol=2e-3, atol=0)
    # scaled fp16 -> E4M3 reuses the stored amax: compare with the oracle's recipe bit for bit
    q = st.cast(Dtypes.kfloat8_e4m3)
    old = {'scale': st.meta.scale.cpu(), 'scale_inv': st.meta.scale_inv.cpu(), 'amax': st.meta.amax.cpu()}
    want_q, want_meta = ocast.scaled_fp16_to_fp8(st.value.cpu(), old, fp8.E4M3)
    assert torch.equal(q.value.cpu(), want_q)
    assert same_float(q.meta.scale, want_meta['scale']) and same_float(q.meta.scale_inv, want_meta['scale_inv'])
    assert same_float(q.meta.amax, want_meta['amax'])
    assert torch.allclose(q.float(), x, rtol=0.07, atol=1e-6)
    # a tiny value survives fp16 -> E4M3 through the scale
    tiny = torch.tensor([2.0**-17], device='cuda').cast(Dtypes.kfloat16).cast(Dtypes.kfloat8_e4m3)
    assert tiny.float().item() == 2.0**-17
    # mul_/div_ act on scale_inv only
    before = q.value.clone()
    q.mul_(2.0)
    assert torch.equal(q.value, before) and torch.allclose(q.float(), 2 * x, rtol=0.07, atol=1e-6)
    q.div_(torch.tensor(2.0, device='cuda'))
    assert torch.allclose(q.float(), x, rtol=0.07, atol=1e-6)
    # fused cast+transpose equals cast then transpose
    a, at = x.fused_cast_transpose(Dtypes.kfloat8_e4m3)
    b = x.cast(Dtypes.kfloat8_e4m3)
    assert torch.equal(a.value, b.value) and torch.equal(at.value, b.fp8_transpose().value)
    assert torch.equal(at.value, b.value.t().contiguous())
    # non-finite input shows in amax
    bad = torch.tensor([1.0, float('nan')], device='cuda').cast(Dtypes.kfloat8_e4m3)
    assert bad.has_inf_or_nan() and not b.has_inf_or_nan()
    assert b.half().dtype == torch.float16 and b.bfloat16().dtype == torch.bfloat16 and b.to(torch.float32).dtype == torch.float32


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
def test_fp8linear_against_nn_linear(dtype):
    torch.manual_seed(1000)
    lin = torch.nn.Linear(32, 16).cuda().to(dtype)
    ref = copy.deepcopy(lin)
    model = LinearReplacer.replace(lin, Dtypes.kfloat16)
    assert isinstance(model, FP8Linear) and isinstance(model.weight, ScalingParameter)
    x = torch.randn(8, 4, 32, device='cuda', dtype=dtype, requires_grad=True)
    x2 = x.detach().clone().requires_grad_(True)
    y, y2 = model(x), ref(x2)
    assert y.dtype == dtype and y.shape == y2.shape
    assert torch.allclose(y.float(), y2.float(), 0, 0.1)
    y.sum().backward()
    y2.sum().backward()
    assert torch.allclose(x.grad.float(), x2.grad.float(), 0, 0.1)
    assert torch.equal(model.bias.grad, ref.bias.grad)
    assert isinstance(model.weight.grad, ScalingTensor) and model.weight.grad.qtype == Dtypes.kfloat8_e4m3
    assert torch.allclose(model.weight.grad.float(), ref.weight.grad.float(), 0.07, 0.5)    # FP8 inputs, E4M3 storage


def test_fp8linear_autocast_and_grad_accumulation():
    torch.manual_seed(3)
    lin = torch.nn.Linear(16, 16).cuda()
    model = LinearReplacer.replace(copy.deepcopy(lin), Dtypes.kfloat16)
    x = torch.randn(8, 16, device='cuda')
    with torch.autocast('cuda', dtype=torch.bfloat16):
        assert model(x).dtype == torch.bfloat16
    full = LinearReplacer.replace(copy.deepcopy(lin), Dtypes.kfloat16)
    full(x).sum().backward()
    for part in x.chunk(2):
        model(part).sum().backward()
    assert torch.allclose(model.weight.grad.float(), full.weight.grad.float(), 0.14, 0.5)


def test_flattened_metas_are_checked():
    model = LinearReplacer.replace(torch.nn.Linear(8, 8).cuda(), Dtypes.kfloat16)
    x = torch.randn(4, 8, device='cuda')
    model(x)
    model.scaling_metas['input'].scale = torch.ones((), device='cuda')
    with pytest.raises(RuntimeError):
        model(x)


def test_fp8linear_step_against_oracle_pipeline():
    """x, W, dy -> casts (in-time warm-up), three GEMMs: y and dx against the oracle's casts + fp32-class GEMM."""
    torch.manual_seed(5)
    tokens, d_in, d_out = 256, 128, 192
    lin = torch.nn.Linear(d_in, d_out, bias=False).cuda().bfloat16()
    w_ref = lin.weight.detach().cpu()
    model = LinearReplacer.replace(lin, Dtypes.kbfloat16)
    x = torch.randn(tokens, d_in, device='cuda', dtype=torch.bfloat16, requires_grad=True)
    dy = (torch.randn(tokens, d_out, device='cuda') * 1e-3).bfloat16()
    y = model(x)
    y.backward(dy)
    xm, wm, gm = ocast.new_meta(), ocast.new_meta(), ocast.new_meta()
    xq = ocast.cast_to_fp8(x.detach().cpu(), xm, fp8.E4M3, in_time=True)
    wq = ocast.cast_to_fp8(w_ref, wm, fp8.E4M3, in_time=True)
    gq = ocast.cast_to_fp8(dy.cpu(), gm, fp8.E5M2, in_time=True)
    y_want = ogemm.fp8_gemm(wq, wm['scale_inv'], fp8.E4M3, xq, xm['scale_inv'], fp8.E4M3)
    dx_want = ogemm.fp8_gemm(wq.t().contiguous(), wm['scale_inv'], fp8.E4M3, gq, gm['scale_inv'], fp8.E5M2)
    dw_want = ogemm.fp8_gemm(xq.t().contiguous(), xm['scale_inv'], fp8.E4M3, gq.t().contiguous(), gm['scale_inv'], fp8.E5M2)
    assert rel_fro(y.float(), y_want) < 1e-2 and rel_fro(x.grad.float(), dx_want) < 1e-2
    assert rel_fro(model.weight.grad.float(), dw_want) < 0.05    # E4M3 storage of the weight gradient
    metas = model.scaling_metas
    assert same_float(metas['input'].amax[0], xm['amax'][0]) and same_float(metas['input'].scale, xm['scale'])
    assert same_float(metas['ograd'].amax[0], gm['amax'][0]) and same_float(metas['ograd'].scale, gm['scale'])


def _code_rank(q):
    """FP8 codes (sign-magnitude bytes) as integers ordered like the values they stand for."""
    q = q.to(torch.int16)
    return torch.where(q >= 128, 127 - q, q)


def test_full_size_fp8linear_step_with_delayed_scaling_against_oracle_pipeline():
    """x[8192, 4096], W[4096, 4096] in bfloat16: 17 steps fill the 16-deep amax windows of `input` and `ograd`, so the
    18th step -- on new data of another magnitude -- quantizes with the scale the window holds (delayed scaling, reference
    msamp/common/tensor/cast.py:31-44 and msamp/optim/optimizer.py:91-108).  That step through the module API against
    the oracle's casts, window updates and GEMMs: metas to the bit, y and dx within the GEMM bar, the FP8 weight
    gradient within one code (values next to zero: within 2**-7 of the scaled range)."""
    from oracle import scaling as oscaling
    torch.manual_seed(21)
    tokens, d_in, d_out, window = 8192, 4096, 4096, 16
    lin = torch.nn.Linear(d_in, d_out, bias=False).cuda().bfloat16()
    w_ref = lin.weight.detach().cpu()
    model = LinearReplacer.replace(lin, Dtypes.kbfloat16)
    opt = LBAdamW(model.parameters(), lr=0.0)    # drives the window update only
    assert model.scaling_metas['input'].window_size == window
    x1 = torch.randn(tokens, d_in, device='cuda', dtype=torch.bfloat16)
    dy1 = (torch.randn(tokens, d_out, device='cuda') * 1e-3).bfloat16()
    for _ in range(17):
        model(x1).backward(dy1)
        model.weight.grad = None
        opt._update_scaling_factors()
    assert not model.scaling_metas['input'].is_in_time_scaling() and not model.scaling_metas['ograd'].is_in_time_scaling()
    # new data, 1.4 times larger: some of it saturates under the window's scale, in the kernel as in the oracle
    x2 = (torch.randn(tokens, d_in, device='cuda') * 1.4).bfloat16().requires_grad_()
    dy2 = (torch.randn(tokens, d_out, device='cuda') * 1.4e-3).bfloat16()
    y = model(x2)
    y.backward(dy2)

    def warmed_meta(first, fmt):
        scales, amaxs, counters = torch.ones(1), torch.zeros(1, window), torch.zeros(1, dtype=torch.int32)
        a1 = first.detach().abs().max().float().cpu()
        for _ in range(17):
            amaxs[0, 0] = torch.maximum(amaxs[0, 0], a1)
            oscaling.update_scaling_factors(scales, amaxs, counters, fp8.FP_MAX[fmt], 0)
        assert int(counters[0]) == 17
        return {'scale': scales[0].clone(), 'scale_inv': torch.reciprocal(scales[0]), 'amax': amaxs[0].clone()}

    xm, gm = warmed_meta(x1, fp8.E4M3), warmed_meta(dy1, fp8.E5M2)
    wm, dwm = ocast.new_meta(), ocast.new_meta()
    xq = ocast.cast_to_fp8(x2.detach().cpu(), xm, fp8.E4M3, in_time=False)
    gq = ocast.cast_to_fp8(dy2.cpu(), gm, fp8.E5M2, in_time=False)
    wq = ocast.cast_to_fp8(w_ref, wm, fp8.E4M3, in_time=True)
    metas = model.scaling_metas
    for name, om in (('input', xm), ('ograd', gm)):
        assert same_float(metas[name].scale, om['scale']) and same_float(metas[name].scale_inv, om['scale_inv'])
        assert same_float(metas[name].amax[0], om['amax'][0]) and int(metas[name].amax_counter) == 17
    y_want = ogemm.fp8_gemm(wq, wm['scale_inv'], fp8.E4M3, xq, xm['scale_inv'], fp8.E4M3)
    assert rel_fro(y.float().cpu(), y_want) < 1e-2
    del y_want
    dx_want = ogemm.fp8_gemm(wq.t().contiguous(), wm['scale_inv'], fp8.E4M3, gq, gm['scale_inv'], fp8.E5M2)
    assert rel_fro(x2.grad.float().cpu(), dx_want) < 1e-2
    del dx_want
    dw_want = ogemm.fp8_gemm(xq.t().contiguous(), xm['scale_inv'], fp8.E4M3, gq.t().contiguous(), gm['scale_inv'], fp8.E5M2,
                             out_dtype=torch.bfloat16)
    dwq_want = ocast.cast_to_fp8(dw_want, dwm, fp8.E4M3, in_time=True, sync=True)
    grad = model.weight.grad
    assert isinstance(grad, ScalingTensor) and grad.qtype == Dtypes.kfloat8_e4m3
    assert same_float(grad.meta.scale, dwm['scale'])
    distance = (_code_rank(grad.value.cpu()) - _code_rank(dwq_want)).abs()
    # Within one code wherever codes are at least 2**-6 apart (|scaled value| >= 2**-3; the tensor's amax is scaled to
    # 224 .. 448).  Closer to zero the codes are as fine as 2**-9 -- 8e-6 of the amax -- and the GEMM's own error spans
    # more than one of them: there the values agree to 2**-7.
    want_val, got_val = fp8.decode(dwq_want, fp8.E4M3), fp8.decode(grad.value.cpu(), fp8.E4M3)
    coarse = want_val.abs() >= 2.0**-3
    assert int(distance[coarse].max()) <= 1 and float((got_val - want_val)[~coarse].abs().max()) <= 2.0**-7
    assert float((distance != 0).float().mean()) < 0.005


def test_fp8linear_bias_rides_in_the_forward_gemm():
    """The bias is added in the epilogue of the forward GEMM (one rounding): against the oracle with the bias, within
    one ulp (of the larger of the bare and the biased output) of the reference's two steps (GEMM rounded, then + bias rounded), and the bias gradient is the
    column sum of dy exactly as autograd forms it for `out + bias`."""
    torch.manual_seed(11)
    tokens, d_in, d_out = 512, 256, 384
    lin = torch.nn.Linear(d_in, d_out, bias=True).cuda()
    w_ref, b_ref = lin.weight.detach().cpu(), lin.bias.detach().clone()
    model = LinearReplacer.replace(lin, Dtypes.kfloat16)
    x = torch.randn(tokens, d_in, device='cuda', dtype=torch.bfloat16, requires_grad=True)
    dy = torch.randn(tokens, d_out, device='cuda').bfloat16()
    y = model(x)
    y.backward(dy)
    assert y.dtype == torch.bfloat16 and model.bias.grad.dtype == torch.float32
    assert torch.equal(model.bias.grad, dy.sum(0).to(torch.float32))
    y0 = torch.nn.functional.linear(x.detach(), model.weight, None)    # the same GEMM without the bias
    two_step = (y0 + b_ref.bfloat16().view(1, -1)).float()
    # the two-step result carries the rounding of the bare GEMM output as well: one ulp of the largest of the three
    ulp = torch.maximum(torch.maximum(two_step.abs(), y.detach().float().abs()), y0.float().abs()) * 2.0**-7
    assert ((y.detach().float() - two_step).abs() <= ulp).all()
    assert not torch.equal(y.detach(), y0)
    xm, wm = ocast.new_meta(), ocast.new_meta()
    xq = ocast.cast_to_fp8(x.detach().cpu(), xm, fp8.E4M3, in_time=True)
    w16 = ocast.cast_to_fp16(w_ref, wm, in_time=True)
    wq, wm8 = ocast.scaled_fp16_to_fp8(w16, wm, fp8.E4M3)
    want = ogemm.fp8_gemm(wq, wm8['scale_inv'], fp8.E4M3, xq, xm['scale_inv'], fp8.E4M3, bias=b_ref.cpu().bfloat16().float())
    assert rel_fro(y.detach().float(), want) < 1e-2


def _check_optimizer_step(torch_cls, lb_cls, diff=3e-4):
    x = torch.randn(4, 4, device='cuda')
    linear = torch.nn.Linear(4, 4).cuda()
    wd, steps = 1e-3, 4
    m1 = copy.deepcopy(linear)
    o1 = torch_cls(m1.parameters(), weight_decay=wd)
    for _ in range(steps):
        m1(x).sum().backward()
        o1.step()
        o1.zero_grad()
    model_state.clear()
    m2 = LinearReplacer.replace(copy.deepcopy(linear), Dtypes.kfloat16)
    o2 = lb_cls(m2.parameters(), weight_decay=wd)
    for _ in range(steps):
        m2(x).sum().backward()
        o2.all_reduce_grads(m2)
        o2.step()
        o2.zero_grad()
    assert torch.allclose(m1.weight, m2.weight.float(), 0, diff)
    assert torch.allclose(m1.bias, m2.bias.float(), 0, diff)


def test_optimizers_track_torch_adamw():
    torch.manual_seed(100)
    dtypes = [torch.uint8, torch.float16]
    pairs = list(itertools.product(dtypes, dtypes)) + [(torch.float32, torch.float32)]
    for m_dt, v_dt in pairs:
        kw = dict(exp_avg_dtype=m_dt, exp_avg_sq_dtype=v_dt)
        _check_optimizer_step(torch.optim.AdamW, partial(LBAdamWBase, **kw))
        _check_optimizer_step(torch.optim.AdamW, partial(LBAdamW, **kw))
        _check_optimizer_step(torch.optim.AdamW, partial(DSAdam, **kw))
        _check_optimizer_step(torch.optim.Adam, partial(LBAdam, **kw))


def test_fused_adamw_only_for_weights_under_in_time_scaling(monkeypatch):
    """The fused kernel rescales the weight from its new amax; with in-time scaling off the reference keeps the stored
    scale (msamp/optim/adamw.py:174 through msamp/common/tensor/cast.py:31-44), so such weights take the per-tensor path."""
    torch.manual_seed(7)
    linear = torch.nn.Linear(64, 32, bias=False).cuda()
    with torch.no_grad():
        # amax 0.1: the float16 payload's scale is 2**19 and the step below stays inside float16 under the kept scale
        linear.weight.clamp_(-0.1, 0.1)
        linear.weight[0, 0] = 0.1
    x = torch.randn(16, 64, device='cuda')
    results = {}
    for in_time in (True, False):
        model_state.clear()
        model = LinearReplacer.replace(copy.deepcopy(linear), Dtypes.kfloat16)
        opt = LBAdamW(model.parameters(), lr=0.01)
        calls = []
        fused_step = LBAdamW._fused_step
        monkeypatch.setattr(LBAdamW, '_fused_step', lambda self, idx, *a, **k: (calls.append(len(idx)), fused_step(self, idx, *a, **k)))
        model(x).sum().backward()
        opt.all_reduce_grads(model)
        scale_before = model.weight.meta.scale.clone()
        with ScalingMeta.in_time_scaling_context(in_time):
            opt.step()
        monkeypatch.undo()
        results[in_time] = (calls, scale_before, model.weight.meta.scale.clone(), model.weight.float())
    calls, before, after, w_fused = results[True]
    assert calls == [1]
    calls, before, after, w_staged = results[False]
    assert calls == [] and torch.equal(before, after)
    # same update either way, up to the coarser grid of the kept scale
    assert torch.allclose(w_fused, w_staged, rtol=0, atol=float(w_fused.abs().max()) * 2e-3)


def test_one_pass_adamw_matches_the_in_place_step():
    """LBAdamW(one_pass='double') takes the fused step in one pass into spare buffers and swaps memory afterwards;
    one_pass='shift' takes it inside arenas of its own, writing a little further along each time: same weights, moments
    and metas as the default in-place step after every step, with the payload tensors staying the objects they were
    while their addresses alternate between two places."""
    torch.manual_seed(13)
    lin = torch.nn.Sequential(torch.nn.Linear(256, 512, bias=False), torch.nn.Linear(512, 128, bias=False),
                              torch.nn.Linear(128, 70, bias=False)).cuda()
    x = torch.randn(64, 256, device='cuda')
    runs = {}
    for mode in (None, 'double', 'shift'):
        model_state.clear()
        model = LinearReplacer.replace(copy.deepcopy(lin), Dtypes.kfloat8_e4m3)
        opt = LBAdamW(model.parameters(), lr=1e-2, one_pass=mode)
        values = [p.value for p in model.parameters()]
        addresses = []
        history = []
        for step in range(6):
            model(x * (1 + step)).square().mean().backward()
            opt.all_reduce_grads(model)
            opt.step()
            opt.zero_grad()
            addresses.append([p.value.data_ptr() for p in model.parameters()])
            history.append([(p.value.clone(), p.meta.scale.clone(), opt.state[p]['exp_avg'].value.clone(),
                             opt.state[p]['exp_avg'].meta.scale.clone(), opt.state[p]['exp_avg_sq'].value.clone(),
                             opt.state[p]['exp_avg_sq'].meta.scale.clone()) for p in model.parameters()])
        assert all(p.value is v for p, v in zip(model.parameters(), values))
        if mode is None:
            assert all(a == addresses[0] for a in addresses)
            assert opt.extra_bytes() == 0
        else:
            assert addresses[0] != addresses[1] and addresses[0] == addresses[2] and addresses[1] == addresses[3]
            assert opt.extra_bytes() > 0
        runs[mode] = history
    for mode in ('double', 'shift'):
        for a, b in zip(runs[None], runs[mode]):
            for pa, pb in zip(a, b):
                assert all(torch.equal(ta, tb) for ta, tb in zip(pa, pb)), mode
    from msamp import _backend
    _backend.check_async_error(block=True)


def test_shifting_adamw_survives_a_replaced_state_and_a_state_dict_round_trip():
    """one_pass='shift' keeps the payloads in its own arenas; when something puts other tensors in their place
    (load_state_dict does) the optimizer adopts them again, and training goes on as it does in place."""
    torch.manual_seed(14)
    lin = torch.nn.Sequential(torch.nn.Linear(64, 96, bias=False), torch.nn.Linear(96, 32, bias=False)).cuda()
    x = torch.randn(32, 64, device='cuda')

    def run(mode):
        model_state.clear()
        model = LinearReplacer.replace(copy.deepcopy(lin), Dtypes.kfloat8_e4m3)
        opt = LBAdamW(model.parameters(), lr=1e-2, one_pass=mode)
        out = []
        for step in range(5):
            model(x * (1 + step)).square().mean().backward()
            opt.all_reduce_grads(model)
            opt.step()
            opt.zero_grad()
            if step == 2:
                saved = copy.deepcopy(opt.state_dict())
                opt.load_state_dict(saved)
            out.append([(p.value.clone(), opt.state[p]['exp_avg'].value.clone(), opt.state[p]['exp_avg_sq'].value.clone())
                        for p in model.parameters()])
        return out

    for a, b in zip(run(None), run('shift')):
        for pa, pb in zip(a, b):
            assert all(torch.equal(ta, tb) for ta, tb in zip(pa, pb))


def test_captured_forward_and_backward_see_the_weights_of_eager_steps():
    """The default optimizer step leaves every payload where it was, so a graph captured of forward and backward keeps
    reading the current weights while the optimizer steps eagerly between replays."""
    torch.manual_seed(15)
    lin = torch.nn.Linear(128, 256, bias=False).cuda().bfloat16()

    def build():
        model_state.clear()
        model = LinearReplacer.replace(copy.deepcopy(lin), Dtypes.kfloat8_e4m3)
        return model, LBAdamW(model.parameters(), lr=1e-2)

    xs = [torch.randn(256, 128, device='cuda').bfloat16() * (1 + i % 3) for i in range(6)]
    dy = (torch.randn(256, 256, device='cuda') * 1e-2).bfloat16()
    # eager reference
    model, opt = build()
    want = []
    for x in xs:
        y = model(x)
        y.backward(dy)
        opt.all_reduce_grads(model)
        opt.step()
        opt.zero_grad()
        want.append((y.detach().clone(), model.weight.value.clone()))
    # forward and backward from a graph, the step eager
    model, opt = build()
    x = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        model(x).backward(dy)
        model.weight.grad = None
    torch.cuda.current_stream().wait_stream(side)
    model_state.clear()
    model, opt = build()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = model(x)
        y.backward(dy)
    grad = model.weight.grad
    for i, xi in enumerate(xs):
        x.copy_(xi)
        graph.replay()
        model.weight.grad = grad
        model_state.ready_to_scale_tensor = True
        opt.all_reduce_grads(model)
        opt.step()
        torch.cuda.synchronize()
        assert torch.equal(y, want[i][0]), i
        assert torch.equal(model.weight.value, want[i][1]), i


@pytest.mark.parametrize('bias', [False, True])
def test_optimizer_step_under_capture_after_an_eager_step(bias):
    """A fused step can be captured once an eager step has built the device tables: the gradients made under capture live
    elsewhere, their addresses reach the table through a pinned copy that the graph holds.  (Bias correction is
    computed on the host from the step count, so a captured step repeats the one it was captured with: off here.)
    With a bias the step has a second launch, the one for parameters kept in high precision, with a table of its own."""
    torch.manual_seed(16)
    lin = torch.nn.Linear(128, 256, bias=bias).cuda().bfloat16()
    xs = [torch.randn(256, 128, device='cuda').bfloat16() * (1 + i % 3) for i in range(5)]
    dy = (torch.randn(256, 256, device='cuda') * 1e-2).bfloat16()

    def build():
        model_state.clear()
        model = LinearReplacer.replace(copy.deepcopy(lin), Dtypes.kfloat8_e4m3)
        return model, LBAdamW(model.parameters(), lr=1e-2, bias_correction=False)

    model, opt = build()
    want = []
    for x in xs:
        model(x).backward(dy)
        opt.all_reduce_grads(model)
        opt.step()
        opt.zero_grad()
        want.append((model.weight.value.clone(), opt.state[model.weight]['exp_avg'].value.clone(),
                     model.bias.detach().clone() if bias else None))
    model, opt = build()
    x = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        model(x).backward(dy)
        opt.all_reduce_grads(model)
        opt.step()
        model.weight.grad = None
        if bias:
            model.bias.grad = None
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert torch.equal(model.weight.value, want[0][0])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        model(x).backward(dy)
        model_state.ready_to_scale_tensor = True
        opt.step()
        model.weight.grad = None
        if bias:
            model.bias.grad = None
    for i in range(1, len(xs)):
        x.copy_(xs[i])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(model.weight.value, want[i][0]), i
        assert torch.equal(opt.state[model.weight]['exp_avg'].value, want[i][1]), i
        assert not bias or torch.equal(model.bias, want[i][2]), i
        assert torch.isfinite(xs[i].float().sum()).item()    # eager work between replays


def test_historical_window_quantization():
    model = LinearReplacer.replace(torch.nn.Linear(4, 8).cuda(), Dtypes.kfloat16)
    opt = LBAdamW(model.parameters())
    window = []
    for i in list(range(17)) * 6:
        x = torch.full((1, 4), float(i), device='cuda')
        window = (window + [i])[-16:]
        y = model(x)
        assert model.scaling_metas['input'].amax.max().item() == max(window)
        y.sum().backward()
        opt.all_reduce_grads(model)
        opt.step()
    assert model.scaling_metas['input'].amax_counter.item() == 17 * 6
    assert not model.scaling_metas['input'].is_in_time_scaling()


def _linear_step_record(model, opt, x, dy):
    metas = model.scaling_metas
    return dict(
        dx=x.grad.clone(), dw=model.weight.grad.value.clone(), dw_scale_inv=model.weight.grad.meta.scale_inv.clone(),
        metas={k: (m.scale.clone(), m.scale_inv.clone(), m.amax.clone(), m.amax_counter.clone()) for k, m in metas.items()}
    )


def test_training_step_replays_from_a_graph():
    """Nothing in forward + backward + window update waits for the GPU or decides on the host, so one captured graph
    serves the warm-up (in-time scaling) and the steady state (delayed scaling) alike: 24 steps with changing inputs,
    every replay against the eager run, bit for bit, with eager work in between."""
    tokens, d_in, d_out, steps = 256, 128, 192, 24
    torch.manual_seed(3)
    w0 = (torch.randn(d_out, d_in) * 0.05).bfloat16()
    xs = [(torch.randn(tokens, d_in) * (1 + (i % 5))).bfloat16().cuda() for i in range(steps)]
    dys = [(torch.randn(tokens, d_out) * 1e-3 * (1 + (i % 3))).bfloat16().cuda() for i in range(steps)]

    def build():
        model_state.clear()
        lin = torch.nn.Linear(d_in, d_out, bias=False).cuda().bfloat16()
        with torch.no_grad():
            lin.weight.copy_(w0)
        model = LinearReplacer.replace(lin, Dtypes.kbfloat16)
        return model, LBAdamW(model.parameters())

    # eager
    model, opt = build()
    want = []
    for i in range(steps):
        x = xs[i].clone().requires_grad_(True)
        y = model(x)
        y.backward(dys[i])
        opt._update_scaling_factors()
        rec = _linear_step_record(model, opt, x, dys[i])
        rec['y'] = y.detach().clone()
        want.append(rec)
        model.weight.grad = None

    # graph: three eager steps on a side stream (allocator warm-up), then capture the fourth and replay the rest
    model, opt = build()
    x = xs[0].clone().requires_grad_(True)
    dy = dys[0].clone()
    n_eager = 3
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for i in range(n_eager):
            with torch.no_grad():
                x.copy_(xs[i])
                dy.copy_(dys[i])
            y = model(x)
            y.backward(dy)
            opt._update_scaling_factors()
            x.grad = None
            model.weight.grad = None
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.no_grad():
        x.copy_(xs[n_eager])
        dy.copy_(dys[n_eager])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = model(x)
        y.backward(dy)
        model_state.ready_to_scale_tensor = True
        opt._update_scaling_factors()
    for i in range(n_eager, steps):
        with torch.no_grad():
            x.copy_(xs[i])
            dy.copy_(dys[i])
        graph.replay()
        got = _linear_step_record(model, opt, x, dy)
        torch.cuda.synchronize()
        w = want[i]
        assert torch.equal(y, w['y']) and torch.equal(got['dx'], w['dx']), i
        assert torch.equal(got['dw'], w['dw']) and same_float(got['dw_scale_inv'], w['dw_scale_inv']), i
        for k in w['metas']:
            for a, b in zip(got['metas'][k], w['metas'][k]):
                assert same_float(a.float(), b.float()), (i, k)
        # eager work between replays
        assert torch.isfinite((xs[i].float() @ w0.float().cuda().t()).sum()).item()
    assert model.scaling_metas['input'].amax_counter.item() == steps


def test_backward_without_transposed_copies_matches_the_explicit_path(monkeypatch):
    """At shapes the kernel reads K-major operands for, the backward pass skips dy^T, W^T and x^T; gradients and
    metas must equal, bit for bit, what the path with the three explicit transposes gives."""
    from msamp.operators.gemm import Gemm
    tokens, d_in, d_out = 512, 256, 768
    torch.manual_seed(9)
    w0 = (torch.randn(d_out, d_in) * 0.05).bfloat16()
    x0 = torch.randn(tokens, d_in).bfloat16().cuda()
    dy = (torch.randn(tokens, d_out) * 1e-3).bfloat16().cuda()
    assert Gemm.kmajor_supported(d_in, tokens, d_out, True, False) and Gemm.kmajor_supported(d_in, d_out, tokens, True, True)

    def run(accumulate_twice):
        model_state.clear()
        lin = torch.nn.Linear(d_in, d_out, bias=False).cuda().bfloat16()
        with torch.no_grad():
            lin.weight.copy_(w0)
        model = LinearReplacer.replace(lin, Dtypes.kbfloat16)
        x = x0.clone().requires_grad_(True)
        for _ in range(2 if accumulate_twice else 1):    # the second pass accumulates into the FP8 weight gradient
            model(x).backward(dy)
        g = model.weight.grad
        return x.grad.clone(), g.value.clone(), g.meta.scale_inv.clone(), {k: m.amax.clone() for k, m in model.scaling_metas.items()}

    for twice in (False, True):
        fast = run(twice)
        with monkeypatch.context() as mp:
            mp.setattr(Gemm, 'kmajor_supported', classmethod(lambda cls, *a, **k: False))
            slow = run(twice)
        assert torch.equal(fast[0], slow[0]) and torch.equal(fast[1], slow[1]) and same_float(fast[2], slow[2])
        assert all(same_float(fast[3][k], slow[3][k]) for k in fast[3])


def test_optimizer_state_dict_round_trip():
    torch.manual_seed(7)
    x = torch.randn(4, 4, device='cuda')
    linear = torch.nn.Linear(4, 4).cuda()
    m1 = LinearReplacer.replace(copy.deepcopy(linear), Dtypes.kfloat16)
    o1 = LBAdamW(m1.parameters())
    for _ in range(2):
        m1(x).sum().backward()
        o1.step()
        o1.zero_grad()
    sd = o1.state_dict()
    assert set(sd) == {'state', 'param_groups'} and set(sd['state']) == {0, 1}
    st = sd['state'][0]
    assert st['step'] == 2 and isinstance(st['exp_avg'], ScalingTensor) and st['exp_avg'].dtype == torch.uint8
    assert isinstance(st['exp_avg_sq'], ScalingTensor) and st['exp_avg_sq'].dtype == torch.float16
    m2 = LinearReplacer.replace(copy.deepcopy(linear), Dtypes.kfloat16)    # re-flattens m1's metas too
    m2.weight.copy_(m1.weight)
    m2.bias.data.copy_(m1.bias.data)
    o2 = LBAdamW(m2.parameters())
    o2.load_state_dict(copy.deepcopy(sd))
    # metas of the two models must see the same history for the runs to stay equal
    for k in ('input', 'wgrad', 'ograd'):
        m2.scaling_metas[k].copy_(m1.scaling_metas[k])
    for m, o in ((m1, o1), (m2, o2)):
        m(x).sum().backward()
        o.step()
    assert torch.equal(m1.weight.value, m2.weight.value)
    assert torch.equal(o1.state[m1.weight]['exp_avg'].value, o2.state[m2.weight]['exp_avg'].value)


@pytest.mark.parametrize('opt_level', ['O1', 'O2'])
def test_initialize_and_train(opt_level):
    torch.manual_seed(11)
    model = torch.nn.Sequential(torch.nn.Linear(32, 64), torch.nn.ReLU(), torch.nn.Linear(64, 16)).cuda()
    model[2].use_fp32_linear = False
    opt = torch.optim.AdamW(model.parameters(), lr=1e-2, weight_decay=0.01)
    model, opt = msamp.initialize(model, opt, opt_level=opt_level)
    assert isinstance(opt, LBAdamW) and all(isinstance(m, FP8Linear) for m in (model[0], model[2]))
    assert opt.exp_avg_dtype == (torch.uint8 if opt_level == 'O2' else torch.float32)
    assert [type(p) for p in opt.param_groups[0]['params']] == [ScalingParameter, torch.nn.Parameter] * 2
    x = torch.randn(64, 32, device='cuda')
    target = torch.randn(64, 16, device='cuda')
    losses = []
    for _ in range(30):
        loss = torch.nn.functional.mse_loss(model(x), target)
        loss.backward()
        msamp.clip_grad_norm_(model.parameters(), 10.0)
        opt.step()
        opt.zero_grad()
        losses.append(loss.item())
    assert losses[-1] < 0.7 * losses[0]
    st = opt.state[model[0].weight]
    if opt_level == 'O2':
        assert st['exp_avg'].dtype == torch.uint8 and st['exp_avg_sq'].dtype == torch.float16
    model_state.clear()
    lin = torch.nn.Linear(4, 4).cuda()
    _, adam_opt = msamp.initialize(lin, torch.optim.Adam(lin.parameters()), opt_level=opt_level)
    assert isinstance(adam_opt, LBAdam) and adam_opt.use_adam


def test_grad_scaler_unscale_with_scaling_tensor_grads():
    model = LinearReplacer.replace(torch.nn.Linear(8, 8).cuda(), Dtypes.kfloat16)
    x = torch.randn(4, 8, device='cuda')
    (model(x).sum() * 128.0).backward()
    g = model.weight.grad
    before = g.float().clone()
    found = torch.zeros(1, device='cuda')
    torch._amp_foreach_non_finite_check_and_unscale_([g, model.bias.grad], found, torch.tensor(1 / 128.0, device='cuda'))
    assert found.item() == 0 and torch.allclose(g.float(), before / 128.0)
    g.meta.amax[0] = float('inf')
    torch._amp_foreach_non_finite_check_and_unscale_([g], found, torch.tensor(1.0, device='cuda'))
    assert found.item() == 1


def test_empty_inputs_are_accepted_everywhere():
    """Zero elements through every entry point: nothing is written but the meta, which comes out as for a tensor of
    zeros (amax 0, the scale in force kept, scale_inv = 1 / scale).  The reference raises here (`max()` of an empty
    tensor); a library must not fault."""
    from msamp import _backend as be
    from tests.gpu_util import make_meta
    dev = 'cuda'
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        x = torch.zeros(0, dtype=dtype, device=dev)
        for fp8_dt in (5, 6):
            s, si, am = make_meta(scale=4.0)
            am[0] = 3.0
            assert be.cast_to_fp8(x, s, am[0:1], si, fp8_dt).numel() == 0
            assert am[0].item() == 3.0 and s.item() == 4.0 and si.item() == 0.25
            for two_pass in (False, True):
                s, si, am = make_meta(scale=4.0)
                am[0] = 3.0
                assert be.cast_to_fp8_intime(x, s, am[0:1], si, fp8_dt, two_pass=two_pass).numel() == 0
                assert am[0].item() == 0.0 and s.item() == 4.0 and si.item() == 0.25
            for counter in (0, 99):
                s, si, am = make_meta(scale=4.0)
                cnt = torch.full((), counter, dtype=torch.int32, device=dev)
                assert be.cast_to_fp8_gated(x, s, am[0:1], si, fp8_dt, cnt, 16).numel() == 0
                assert s.item() == 4.0 and si.item() == 0.25
            for shape in ((0, 64), (64, 0), (0, 0)):
                s, si, am = make_meta(scale=4.0)
                q, qt = be.cast_transpose(x.view(shape), s, am[0:1], si, fp8_dt)
                assert q.shape == shape and qt.shape == shape[::-1]
                q, qt = be.cast_transpose(x.view(shape), s, am[0:1], si, fp8_dt, in_time=True)
                assert q.shape == shape and s.item() == 4.0
        cell = torch.full((1, ), 7.0, device=dev)
        be.amax(x, cell)
        assert cell.item() == 0.0
        assert be.scale_cast(x, torch.ones((), device=dev), torch.float16).numel() == 0
    q0 = torch.zeros(0, dtype=torch.uint8, device=dev)
    assert be.cast_from_fp8(q0, torch.ones((), device=dev), 5, torch.float32).numel() == 0
    assert be.fp8_transpose(q0.view(0, 16)).shape == (16, 0)
    s, si, am = make_meta(scale=4.0)
    be.add_to_fp8(q0, 5, s, si, am[0:1], torch.zeros(0, device=dev))
    be.scale_update(torch.zeros(0, device=dev), torch.zeros(0, 16, device=dev), 448.0, 0, want_mask=False)
    # GEMM: no rows or no columns -> nothing to do; no reduction length is an error, as is a ragged one
    one = torch.ones((), device=dev)
    a = torch.zeros(0, 32, dtype=torch.uint8, device=dev)
    b = torch.zeros(8, 32, dtype=torch.uint8, device=dev)
    be.fp8_gemm(a, 5, one, b, 5, one, torch.empty(8, 0, device=dev))
    be.fp8_gemm(b, 5, one, a, 5, one, torch.empty(0, 8, device=dev))
    with pytest.raises(Exception):
        be.fp8_gemm(torch.zeros(8, 0, dtype=torch.uint8, device=dev), 5, one, torch.zeros(8, 0, dtype=torch.uint8, device=dev), 5, one,
                    torch.empty(8, 8, device=dev))
    # fused AdamW: no tensors at all
    be.adamw_fused(torch.zeros(0, be.ADAMW_DESC_WORDS, dtype=torch.int64, device=dev), 0,
                   torch.zeros(0, 2, dtype=torch.int32, device=dev), 0, 5, 6, 1e-3, 0.9, 0.95, 1e-8, 0.1, 1, True, False, False, True)


@pytest.mark.parametrize('optimizer, kw', [
    (LBAdamW, dict()),
    (LBAdamW, dict(weight_decay=0.0, maximize=True)),
    (LBAdamW, dict(tensor_scale=False, bias_correction=False)),
    (LBAdam, dict(weight_decay=0.05)),
])
def test_small_plain_parameters_take_one_launch_with_the_bits_of_the_two_stages(monkeypatch, optimizer, kw):
    """Parameters kept in float32 / float16 / bfloat16 with E4M3 and scaled-float16 moments (biases, norm weights) go
    through both stages of the reference recipe (msamp/optim/adamw.py:148-199) in one launch for all of them, larger
    ones (an embedding) in three launches chunk by chunk: same parameter, moment payloads and metas, bit for bit, as the
    two stages taken tensor by tensor, over several steps whose gradients change size by orders of magnitude (so the
    moment scales move)."""
    shapes = [(1, ), (70, ), (4099, ), (3, 1000), (LBAdamW._PLAIN_LIMIT, ), (LBAdamW._PLAIN_LIMIT + 1, ), (3, 349_527), (1 << 20, )]
    dtypes = [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
              (torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32)]    # (the last: a bf16 module's bias)
    runs = {}
    for fused in (True, False):
        gen = torch.Generator(device='cuda').manual_seed(31)
        params = []
        for p_dt, g_dt in dtypes:
            for shape in shapes:
                params.append((torch.nn.Parameter((torch.randn(shape, device='cuda', generator=gen) * 0.3).to(p_dt)), g_dt))
                if g_dt != p_dt:
                    params[-1][0].grad_dtype = g_dt
        # a large one that is not aligned for four elements keeps the two stages tensor by tensor
        base = torch.randn(LBAdamW._PLAIN_LIMIT + 10, device='cuda', generator=gen)
        params.append((torch.nn.Parameter(base[1:]), torch.float32))
        opt = optimizer([p for p, _ in params], lr=3e-3, **kw)
        calls = []
        if fused:
            plain_step = LBAdamW._plain_step
            monkeypatch.setattr(LBAdamW, '_plain_step', lambda self, idx, *a, **k: (calls.append(len(idx)), plain_step(self, idx, *a, **k)))
        else:
            monkeypatch.setattr(LBAdamW, '_plain_fusable', classmethod(lambda cls, *a: False))
        history = []
        for step, size in enumerate((1.0, 1e-3, 40.0, 1e-6, 0.0, 2.0)):
            for p, g_dt in params:
                p.grad = (torch.randn(p.shape, device='cuda', generator=gen) * size).to(g_dt)
            opt.step()
            history.append([(p.detach().clone(), ) + tuple(t.clone() for name in ('exp_avg', 'exp_avg_sq')
                                                           for t in (opt.state[p][name].value, opt.state[p][name].meta.scale,
                                                                     opt.state[p][name].meta.scale_inv, opt.state[p][name].meta.amax))
                            for p, _ in params])
        monkeypatch.undo()
        if fused:
            # per pair of types one call with the five shapes that a workgroup takes whole and one with the three larger ones
            assert calls == [5, 3] * len(dtypes) * 6
        runs[fused] = history
    for step, (a, b) in enumerate(zip(runs[True], runs[False])):
        for t, (x, y) in enumerate(zip(a, b)):
            for which, (u, v) in enumerate(zip(x, y)):
                assert same_float(u, v) if u.is_floating_point() else torch.equal(u, v), (step, t, which)
    # the moment scales did move
    assert len({float(h[1][2]) for h in runs[True]}) > (1 if kw.get('tensor_scale', True) else 0)


def test_plain_parameter_step_follows_gradients_that_move():
    """The descriptor table of the one-launch step is kept from step to step; a gradient at a new address (grads set to
    None between steps) is found again."""
    torch.manual_seed(5)
    p = torch.nn.Parameter(torch.randn(300, device='cuda'))
    q = torch.nn.Parameter(p.detach().clone())
    opt_p, opt_q = LBAdamW([p], lr=1e-2), LBAdamW([q], lr=1e-2)
    keep = []
    for step in range(4):
        g = torch.randn(300, device='cuda')
        keep.append(g)    # (held, so that the next gradient gets another address)
        p.grad = g.clone()
        if q.grad is None:
            q.grad = torch.empty_like(g)
        q.grad.copy_(g)
        opt_p.step()
        opt_q.step()
        p.grad = None
        assert torch.equal(p, q)


@pytest.mark.parametrize('optimizer, kw', [
    (LBAdamW, dict()),
    (LBAdamW, dict(weight_decay=0.0, maximize=True)),
    (LBAdamW, dict(bias_correction=False, betas=(0.8, 0.95), eps=1e-6)),
    (LBAdam, dict(weight_decay=0.05)),
])
def test_float32_moment_step_in_one_kernel_has_the_bits_of_the_chain(monkeypatch, optimizer, kw):
    """With float32 exp_avg / exp_avg_sq the reference's step is a chain of element-wise torch calls
    (msamp/optim/adamw.py:200-232); the one-pass kernel that stands in for it leaves the same parameter and moments, bit
    for bit, over several steps: float32 / bfloat16 / float16 parameters, gradients of another type, a parameter that
    is a misaligned view (no vector loads), and a scaled-float16 ScalingTensor weight that is requantized after the step."""
    shapes = [(1, ), (70, ), (4099, ), (1 << 20, ), (3, 349_527)]
    dtypes = [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
              (torch.float32, torch.bfloat16)]
    runs = {}
    for fused in (True, False):
        gen = torch.Generator(device='cuda').manual_seed(77)
        params = []
        for p_dt, g_dt in dtypes:
            for shape in shapes:
                params.append((torch.nn.Parameter((torch.randn(shape, device='cuda', generator=gen) * 0.3).to(p_dt)), g_dt))
                if g_dt != p_dt:
                    params[-1][0].grad_dtype = g_dt
        base = torch.randn(5001, device='cuda', generator=gen)
        params.append((torch.nn.Parameter(base[1:]), torch.float32))    # 4 bytes past a 16-byte boundary
        weight = torch.nn.Parameter(torch.randn(64, 48, device='cuda', generator=gen) * 0.05)
        scaled = ScalingParameter(weight.detach().cast(Dtypes.kfloat16))
        opt = optimizer([p for p, _ in params] + [scaled], lr=3e-3, exp_avg_dtype=torch.float32, exp_avg_sq_dtype=torch.float32,
                        **kw)
        calls = []
        f32_step = LBAdamW._f32_step
        if fused:
            monkeypatch.setattr(LBAdamW, '_f32_step', lambda self, *a, **k: (calls.append(1), f32_step(self, *a, **k))[1])
        else:
            monkeypatch.setattr(LBAdamW, '_f32_step', lambda self, *a, **k: False)
        history = []
        for step, size in enumerate((1.0, 1e-3, 40.0, 0.0, 2.0)):
            for p, g_dt in params:
                p.grad = (torch.randn(p.shape, device='cuda', generator=gen) * size).to(g_dt)
            scaled.grad = (torch.randn(64, 48, device='cuda', generator=gen) * size).cast(Dtypes.kfloat8_e4m3)
            opt.step()
            history.append([(p.detach().clone(), opt.state[p]['exp_avg'].clone(), opt.state[p]['exp_avg_sq'].clone())
                            for p, _ in params] +
                           [(scaled.value.clone(), scaled.meta.scale.clone(), opt.state[scaled]['exp_avg'].clone(),
                             opt.state[scaled]['exp_avg_sq'].clone())])
        monkeypatch.undo()
        assert len(calls) == (5 * (len(params) + 1) if fused else 0)
        runs[fused] = history
    for step, (a, b) in enumerate(zip(runs[True], runs[False])):
        for t, (x, y) in enumerate(zip(a, b)):
            for which, (u, v) in enumerate(zip(x, y)):
                assert same_float(u, v), (step, t, which, (u.float() - v.float()).abs().max().item())
