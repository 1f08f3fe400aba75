"""GPU parity of the FP8 AdamW kernels against the CPU oracle: quantized weights and moments within
one code (1 FP8 ulp) after a step -- in practice bit-equal -- and metas bit-exact."""

import numpy as np
import pytest
import torch

from oracle import adamw as oadam, cast as ocast, fp8
from tests.gpu_util import same_float

pytestmark = pytest.mark.gpu

HYPER = dict(lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)


@pytest.fixture(scope='module')
def be():
    from msamp import _backend
    _backend.load()
    return _backend


def _quant(x, fmt):
    meta = ocast.new_meta()
    return ocast.cast_to_fp8(x, meta, fmt, in_time=True), meta


def _inputs(n, seed, w_fmt, g_fmt, zero_state=False):
    g = torch.Generator().manual_seed(seed)
    wf = 0.02 * torch.randn(n, generator=g)
    if w_fmt == 'f16':
        wm = ocast.new_meta()
        w = ocast.cast_to_fp16(wf, wm, in_time=True)
    else:
        w, wm = _quant(wf, w_fmt)
    gq, gm = _quant(1e-3 * torch.randn(n, generator=g), g_fmt)
    mf = torch.zeros(n) if zero_state else (1e-4 * torch.randn(n, generator=g)).abs()
    vf = torch.zeros(n) if zero_state else (1e-4 * torch.randn(n, generator=g)).abs()
    m, mm = _quant(mf, fp8.E4M3)
    vm = ocast.new_meta()
    v = ocast.cast_to_fp16(vf, vm, in_time=True)
    return dict(w=w, wm=wm, g=gq, gm=gm, m=m, mm=mm, v=v, vm=vm)


def _dev_meta(meta):
    return [meta['scale'].clone().cuda().reshape(()), meta['scale_inv'].clone().cuda().reshape(()), meta['amax'].clone().cuda()]


def _code_distance(a, b):
    """Distance in code steps between two FP8 payloads (sign-magnitude order)."""
    def key(t):
        t = t.to(torch.int32)
        return torch.where(t >= 128, -(t - 128), t)
    return (key(a.cpu()) - key(b.cpu())).abs()


def _fused(be, tensors, w_dt, g_dt, step, **kw):
    """Run msamp_adamw_fp8_fused on a list of tensor dicts; returns device copies of everything."""
    dev = []
    rows = []
    for t in tensors:
        d = dict(w=t['w'].cuda(), g=t['g'].cuda(), m=t['m'].cuda(), v=t['v'].cuda(), wm=_dev_meta(t['wm']),
                 gsi=t['gm']['scale_inv'].clone().cuda().reshape(()), mm=_dev_meta(t['mm']), vm=_dev_meta(t['vm']))
        dev.append(d)
        rows.append((d['w'].data_ptr(), d['g'].data_ptr(), d['m'].data_ptr(), d['v'].data_ptr(),
                     d['wm'][0].data_ptr(), d['wm'][1].data_ptr(), d['wm'][2].data_ptr(), d['gsi'].data_ptr(),
                     d['mm'][0].data_ptr(), d['mm'][1].data_ptr(), d['mm'][2].data_ptr(),
                     d['vm'][0].data_ptr(), d['vm'][1].data_ptr(), d['vm'][2].data_ptr(), d['w'].numel(), 0, 0, 0, 0))
    desc = torch.from_numpy(np.asarray(rows, dtype=np.int64)).cuda()
    chunks = [(t['w'].numel() + be.ADAMW_CHUNK - 1) // be.ADAMW_CHUNK for t in tensors]
    bm = np.stack([np.repeat(np.arange(len(tensors), dtype=np.int32), chunks),
                   np.concatenate([np.arange(c, dtype=np.int32) for c in chunks])], axis=1).copy()
    block_map = torch.from_numpy(bm).cuda()
    hyper = dict(HYPER)
    hyper.update(kw)
    if hyper.get('speculative'):
        # one pass into separate buffers: afterwards the inputs are untouched and the outputs hold the new state
        before = [(d['w'].clone(), d['m'].clone(), d['v'].clone()) for d in dev]
        outs = [(torch.full_like(d['w'], 0x55), torch.full_like(d['m'], 0x55), torch.full_like(d['v'], 0x55)) for d in dev]
        table = torch.tensor([[o[0].data_ptr(), o[1].data_ptr(), o[2].data_ptr(), 0] for o in outs], dtype=torch.int64).cuda()
        redo = torch.full((len(dev), ), -1, dtype=torch.int32, device='cuda')
        be.adamw_fused_speculative(desc, table, redo, len(tensors), block_map, block_map.shape[0], w_dt, g_dt, hyper['lr'],
                                   hyper['beta1'], hyper['beta2'], hyper['eps'], hyper['weight_decay'], step,
                                   hyper.get('bias_correction', True), hyper.get('adam_mode', False),
                                   hyper.get('maximize', False), hyper.get('tensor_scale', True))
        torch.cuda.synchronize()
        for d, b, o, r in zip(dev, before, outs, redo.tolist()):
            assert torch.equal(d['w'], b[0]) and torch.equal(d['m'], b[1]) and torch.equal(d['v'].view(torch.int16), b[2].view(torch.int16))
            d['w'], d['m'], d['v'] = o
            d['redo'] = r
        assert (desc[:, 15].cpu() == 0).all()
        return dev
    be.adamw_fused(desc, len(tensors), block_map, block_map.shape[0], w_dt, g_dt, hyper['lr'], hyper['beta1'], hyper['beta2'],
                   hyper['eps'], hyper['weight_decay'], step, hyper.get('bias_correction', True), hyper.get('adam_mode', False),
                   hyper.get('maximize', False), hyper.get('tensor_scale', True), blocks_per_tensor=chunks,
                   group_blocks=hyper.get('group_blocks'))
    torch.cuda.synchronize()
    # the scratch words of the descriptors are left zeroed
    assert (desc[:, 15].cpu() == 0).all()
    return dev


def _check(dev, t, w_fmt, g_fmt, step, **kw):
    hyper = dict(HYPER)
    hyper.update(kw)
    (w2, wm2, m2, mm2, v2, vm2), _ = oadam.step_tensor(
        t['w'], t['wm'], w_fmt, t['g'], t['gm']['scale_inv'], g_fmt, t['m'], t['mm'], t['v'], t['vm'], step=step, **hyper
    )
    for got, want, name in ((dev['wm'], wm2, 'w'), (dev['mm'], mm2, 'm'), (dev['vm'], vm2, 'v')):
        assert same_float(got[0], want['scale']), name
        assert same_float(got[1], want['scale_inv']), name
        assert same_float(got[2][0], want['amax'][0]), name
    if w_fmt == 'f16':
        dw = (dev['w'].cpu().view(torch.int16).int() - w2.view(torch.int16).int()).abs()
    else:
        dw = _code_distance(dev['w'], w2)
    dm = _code_distance(dev['m'], m2)
    dv = (dev['v'].cpu().view(torch.int16).int() - v2.view(torch.int16).int()).abs()
    assert dw.max().item() <= 1 and dm.max().item() <= 1 and dv.max().item() <= 1
    # and almost all of them are bit-equal
    for d in (dw, dm, dv):
        assert (d != 0).float().mean().item() < 1e-3


@pytest.mark.parametrize('w_fmt,w_dt,g_fmt,g_dt', [(fp8.E4M3, 5, fp8.E5M2, 6), ('f16', 3, fp8.E4M3, 5), (fp8.E5M2, 6, fp8.E4M3, 5)])
@pytest.mark.parametrize('step,zero_state', [(1, True), (2, False)])
def test_fused_step_multi_tensor(be, w_fmt, w_dt, g_fmt, g_dt, step, zero_state):
    sizes = [16384 * 4, 16384 * 2 + 777, 5, 4096 * 1024]
    tensors = [_inputs(n, 100 + i, w_fmt, g_fmt, zero_state) for i, n in enumerate(sizes)]
    dev = _fused(be, tensors, w_dt, g_dt, step)
    for d, t in zip(dev, tensors):
        _check(d, t, w_fmt, g_fmt, step)


@pytest.mark.parametrize('kw', [dict(adam_mode=True), dict(maximize=True), dict(bias_correction=False), dict(weight_decay=0.0),
                                dict(tensor_scale=False)])
def test_fused_step_variants(be, kw):
    t = _inputs(16384 * 3 + 100, 7, fp8.E4M3, fp8.E5M2)
    dev = _fused(be, [t], 5, 6, 3, **kw)
    _check(dev[0], t, fp8.E4M3, fp8.E5M2, 3, **kw)


def test_fused_step_maximum_comes_from_the_update_term(be):
    """The amax pass bounds 16 elements at a time by max|p| + step * max|m'| / (sqrt(min v') / sbc2 + eps); here the
    largest |p'| belongs to elements with a small weight and a large update (zero second moment, largest first
    moment), spread over lanes that otherwise hold small values."""
    n = 16384 * 6 + 48
    t = _inputs(n, 55, fp8.E4M3, fp8.E5M2)
    for idx in (5, 16384 * 2 + 17, n - 3):
        t['v'][idx] = 0.0
        t['m'][idx] = 0x7E if idx != 5 else 0xFE    # +-448 / scale
        t['g'][idx] = 0
        t['w'][idx] = 0x01                           # smallest positive weight code
    for kw in (dict(lr=0.5), dict(lr=0.5, eps=0.0), dict()):
        dev = _fused(be, [t], 5, 6, 2, **kw)
        _check(dev[0], t, fp8.E4M3, fp8.E5M2, 2, **kw)


def test_fused_step_nan_state_reaches_the_weight_amax(be):
    """A NaN second moment makes that element's new weight NaN: the weight amax must say so (NaN), the scale stays,
    and every other weight is what the oracle gives."""
    n = 16384 * 3
    t = _inputs(n, 56, fp8.E4M3, fp8.E5M2)
    bad = 16384 + 4321
    t['v'].view(torch.int16)[bad] = 0x7E00
    dev = _fused(be, [t], 5, 6, 2)[0]
    (w2, wm2, _, _, _, _), _ = oadam.step_tensor(t['w'], t['wm'], fp8.E4M3, t['g'], t['gm']['scale_inv'], fp8.E5M2, t['m'], t['mm'],
                                                 t['v'], t['vm'], step=2, **HYPER)
    assert torch.isnan(dev['wm'][2][0]).item() and torch.isnan(wm2['amax'][0]).item()
    assert same_float(dev['wm'][0], wm2['scale']) and same_float(dev['wm'][0], t['wm']['scale'])
    d = _code_distance(dev['w'], w2)
    d[bad] = 0    # the sign of a NaN is not defined
    assert d.max().item() <= 1 and dev['w'][bad].item() & 0x7F == 0x7F and w2[bad].item() & 0x7F == 0x7F


def test_fused_step_grouping_does_not_change_results(be):
    sizes = [16384 * 3, 16384 * 5 + 9, 100, 16384 * 2]
    tensors = [_inputs(n, 300 + i, fp8.E4M3, fp8.E5M2) for i, n in enumerate(sizes)]
    ref = _fused(be, tensors, 5, 6, 2, group_blocks=0)
    for gb in (1, 4, 6, 1000):
        got = _fused(be, tensors, 5, 6, 2, group_blocks=gb)
        for a, b in zip(ref, got):
            assert torch.equal(a['w'], b['w']) and torch.equal(a['m'], b['m']) and torch.equal(a['v'], b['v'])
            assert all(torch.equal(x, y) for x, y in zip(a['wm'] + a['mm'] + a['vm'], b['wm'] + b['mm'] + b['vm']))


def test_config3_full_size_every_tensor_matches(be):
    """1.0e9 parameters as 238 tensors of [4096, 1024] and a tail of 1 755 648 elements, one fused step.  Every full
    tensor holds the same bytes, so all of them must come out identical to the first, which is checked against the
    oracle; the tail (a prefix of the same bytes, its own metas) is checked against the oracle too."""
    per, total = 4096 * 1024, 1_000_000_000
    n_full, tail = total // per, total % per
    base = _inputs(per, 77, fp8.E4M3, fp8.E5M2)
    last = {k: (v[:tail].clone() if isinstance(v, torch.Tensor) else {kk: vv.clone() for kk, vv in v.items()})
            for k, v in base.items()}
    tensors = [base] * n_full + [last]
    dev = _fused(be, tensors, 5, 6, 2)
    _check(dev[0], base, fp8.E4M3, fp8.E5M2, 2)
    _check(dev[-1], last, fp8.E4M3, fp8.E5M2, 2)
    first = dev[0]
    for d in dev[1:n_full]:
        assert torch.equal(d['w'], first['w']) and torch.equal(d['m'], first['m']) and torch.equal(d['v'], first['v'])
        assert all(torch.equal(x, y) for x, y in zip(d['wm'] + d['mm'] + d['vm'], first['wm'] + first['mm'] + first['vm']))


def test_fused_step_sparse_gradient_and_zero_state(be):
    """Nine gradients in ten are exactly zero and the moments start at zero: for those elements m' = v' = 0 and the
    first pass' bound has to come from eps alone (the reciprocal square root of zero is infinite)."""
    n = 16384 * 5 + 321
    t = _inputs(n, 91, fp8.E4M3, fp8.E5M2, zero_state=True)
    g = torch.Generator().manual_seed(92)
    t['g'][torch.rand(n, generator=g) < 0.9] = 0
    t['g'][7] = 0x80    # a negative zero as well
    for step, kw in ((1, dict()), (1, dict(adam_mode=True)), (3, dict(maximize=True))):
        dev = _fused(be, [t], 5, 6, step, **kw)
        _check(dev[0], t, fp8.E4M3, fp8.E5M2, step, **kw)


def _same_state(a, b):
    bits = lambda t: t.view(torch.int32) if t.dtype == torch.float32 else (t.view(torch.int16) if t.dtype == torch.float16 else t)
    return all(torch.equal(bits(x), bits(y)) for x, y in zip([a['w'], a['m'], a['v']] + a['wm'] + a['mm'] + a['vm'],
                                                             [b['w'], b['m'], b['v']] + b['wm'] + b['mm'] + b['vm']))


def _next_inputs(t, dev, seed, g_fmt, grad_std=1e-3):
    """The state a fused step left on the device as the input of the next step, with a fresh gradient."""
    meta = lambda m: dict(scale=m[0].cpu().reshape(()), scale_inv=m[1].cpu().reshape(()), amax=m[2].cpu())
    gq, gm = _quant(grad_std * torch.randn(t['w'].numel(), generator=torch.Generator().manual_seed(seed)), g_fmt)
    return dict(w=dev['w'].cpu(), wm=meta(dev['wm']), g=gq, gm=gm, m=dev['m'].cpu(), mm=meta(dev['mm']), v=dev['v'].cpu(),
                vm=meta(dev['vm']))


@pytest.mark.parametrize('w_fmt,w_dt,g_fmt,g_dt', [(fp8.E4M3, 5, fp8.E5M2, 6), ('f16', 3, fp8.E4M3, 5), (fp8.E5M2, 6, fp8.E4M3, 5)])
def test_speculative_step_equals_the_in_place_step(be, w_fmt, w_dt, g_fmt, g_dt):
    """Four steps in a row, each taken both ways from the same state: the one-pass step into separate buffers leaves the
    bits of the two-pass step, whether its guess (the scales in force) holds or not.  The first step starts from zero
    moments with scale 1, so every guess is wrong; later steps with gradients of the same size keep their scales; a
    gradient sixteen times larger moves the moment scales of that step."""
    sizes = [16384 * 4, 16384 * 2 + 777, 5, 4096 * 1024, 16384]
    tensors = [_inputs(n, 400 + i, w_fmt, g_fmt, zero_state=True) for i, n in enumerate(sizes)]
    hits = misses = 0
    for step in range(1, 5):
        plain = _fused(be, tensors, w_dt, g_dt, step)
        spec = _fused(be, tensors, w_dt, g_dt, step, speculative=True)
        for a, b, t in zip(plain, spec, tensors):
            assert _same_state(a, b), (step, t['w'].numel())
            assert b['redo'] in (0, 1)
            moved = not (same_float(a['wm'][0], t['wm']['scale']) and same_float(a['mm'][0], t['mm']['scale']) and
                         same_float(a['vm'][0], t['vm']['scale']))
            assert b['redo'] == int(moved)
            hits += 1 - b['redo']
            misses += b['redo']
        _check(spec[3], tensors[3], w_fmt, g_fmt, step)
        tensors = [_next_inputs(t, d, 500 + 10 * step + i, g_fmt, grad_std=1.6e-2 if step == 3 else 1e-3)
                   for i, (t, d) in enumerate(zip(tensors, plain))]
    assert hits >= 3 and misses >= len(sizes)


@pytest.mark.parametrize('kw', [dict(adam_mode=True), dict(maximize=True), dict(bias_correction=False), dict(weight_decay=0.0),
                                dict(tensor_scale=False), dict(lr=0.5, eps=0.0)])
def test_speculative_step_variants(be, kw):
    t = _inputs(16384 * 3 + 100, 7, fp8.E4M3, fp8.E5M2)
    for step in (2, 3):
        plain = _fused(be, [t], 5, 6, step, **kw)[0]
        spec = _fused(be, [t], 5, 6, step, speculative=True, **kw)[0]
        assert _same_state(plain, spec)
        _check(spec, t, fp8.E4M3, fp8.E5M2, step, **kw)
        t = _next_inputs(t, plain, 60 + step, fp8.E5M2)


def test_speculative_step_special_values(be):
    """A NaN second moment (NaN weight amax, scale kept), zero gradients on zero state, and the largest |p'| coming from
    the update term: same bits as the in-place step in each case."""
    n = 16384 * 3
    t = _inputs(n, 56, fp8.E4M3, fp8.E5M2)
    t['v'].view(torch.int16)[16384 + 4321] = 0x7E00
    plain, spec = _fused(be, [t], 5, 6, 2)[0], _fused(be, [t], 5, 6, 2, speculative=True)[0]
    assert torch.isnan(spec['wm'][2][0]).item() and _same_state(plain, spec)
    t = _inputs(16384 * 5 + 321, 91, fp8.E4M3, fp8.E5M2, zero_state=True)
    t['g'][torch.rand(t['g'].numel(), generator=torch.Generator().manual_seed(92)) < 0.9] = 0
    for step, kw in ((1, dict()), (1, dict(adam_mode=True))):
        assert _same_state(_fused(be, [t], 5, 6, step, **kw)[0], _fused(be, [t], 5, 6, step, speculative=True, **kw)[0])
    n = 16384 * 6 + 48
    t = _inputs(n, 55, fp8.E4M3, fp8.E5M2)
    for idx in (5, 16384 * 2 + 17, n - 3):
        t['v'][idx] = 0.0
        t['m'][idx] = 0x7E if idx != 5 else 0xFE
        t['g'][idx] = 0
        t['w'][idx] = 0x01
    for kw in (dict(lr=0.5), dict(lr=0.5, eps=0.0), dict()):
        spec = _fused(be, [t], 5, 6, 2, speculative=True, **kw)[0]
        assert _same_state(_fused(be, [t], 5, 6, 2, **kw)[0], spec)
        _check(spec, t, fp8.E4M3, fp8.E5M2, 2, **kw)


def _fused_shift(be, tensors, w_dt, g_dt, step, slack, up, check_clean=True, **kw):
    """msamp_adamw_fp8_fused_shift on a list of tensor dicts: the payloads are laid out back to back, padded to whole
    chunks, in three arenas with `slack` chunks of room (below the data when the step moves down, above it when it moves
    up); returns device copies of everything, the new payloads read from where the step put them."""
    ch = be.ADAMW_CHUNK
    chunks = [(t['w'].numel() + ch - 1) // ch for t in tensors]
    pos = np.concatenate([[0], np.cumsum(chunks)]).tolist()
    total = pos[-1]
    wsz = 2 if w_dt == 3 else 1
    arenas = {k: torch.full(((total + slack) * ch * sz, ), 0x55, dtype=torch.uint8, device='cuda')
              for k, sz in (('w', wsz), ('m', 1), ('v', 2))}
    size = dict(w=wsz, m=1, v=2)
    src, dst = (0, slack) if up else (slack, 0)

    def view(kind, t_idx, off, like):
        first = (pos[t_idx] + off) * ch * size[kind]
        return arenas[kind][first:first + like.numel() * size[kind]].view(like.dtype)

    dev, rows = [], []
    for i, t in enumerate(tensors):
        d = dict(g=t['g'].cuda(), wm=_dev_meta(t['wm']), gsi=t['gm']['scale_inv'].clone().cuda().reshape(()),
                 mm=_dev_meta(t['mm']), vm=_dev_meta(t['vm']))
        for kind in 'wmv':
            d[kind] = view(kind, i, src, t[kind])
            d[kind].copy_(t[kind])
        dev.append(d)
        rows.append((d['w'].data_ptr(), d['g'].data_ptr(), d['m'].data_ptr(), d['v'].data_ptr(),
                     d['wm'][0].data_ptr(), d['wm'][1].data_ptr(), d['wm'][2].data_ptr(), d['gsi'].data_ptr(),
                     d['mm'][0].data_ptr(), d['mm'][1].data_ptr(), d['mm'][2].data_ptr(),
                     d['vm'][0].data_ptr(), d['vm'][1].data_ptr(), d['vm'][2].data_ptr(), d['w'].numel(), 0, 0, 0, 0))
    desc = torch.from_numpy(np.asarray(rows, dtype=np.int64)).cuda()
    bm = np.stack([np.repeat(np.arange(len(tensors), dtype=np.int32), chunks),
                   np.concatenate([np.arange(c, dtype=np.int32) for c in chunks])], axis=1).copy()
    block_map = torch.from_numpy(bm).cuda()
    hyper = dict(HYPER)
    hyper.update(kw)
    redo = torch.full((len(dev), ), -1, dtype=torch.int32, device='cuda')
    sync = torch.zeros(be.adamw_shift_sync_bytes(len(dev), total), dtype=torch.uint8, device='cuda')
    be.adamw_fused_shift(desc, redo, sync, len(tensors), block_map, total, (slack if up else -slack) * ch, w_dt, g_dt, hyper['lr'],
                         hyper['beta1'], hyper['beta2'], hyper['eps'], hyper['weight_decay'], step,
                         hyper.get('bias_correction', True), hyper.get('adam_mode', False), hyper.get('maximize', False),
                         hyper.get('tensor_scale', True))
    torch.cuda.synchronize()
    for i, (d, t, r) in enumerate(zip(dev, tensors, redo.tolist())):
        for kind in 'wmv':
            d[kind] = view(kind, i, dst, t[kind]).clone()
        d['redo'] = r
    if check_clean:    # accumulators and counters of the descriptors are left zeroed
        assert (desc[:, 15].cpu() == 0).all() and (desc[:, 16].cpu() & 0xffffffff == 0).all()
    return dev


@pytest.mark.parametrize('w_fmt,w_dt,g_fmt,g_dt', [(fp8.E4M3, 5, fp8.E5M2, 6), ('f16', 3, fp8.E4M3, 5), (fp8.E5M2, 6, fp8.E4M3, 5)])
@pytest.mark.parametrize('slack', [256, 300, 4096])
def test_shifting_step_equals_the_in_place_step(be, w_fmt, w_dt, g_fmt, g_dt, slack):
    """The one-pass step inside shifting arenas against the two-pass step in place, four steps in a row from the same
    states, the direction alternating.  The first step starts from zero moments with scale 1, so every guess is wrong and
    every tensor takes its second round: with little room (256 chunks, exactly the largest tensor: the workgroups that
    overwrite a chunk meet tensors that have only just finished) those rounds are taken by the workgroups that follow,
    with 300 partly by them and partly by the closing launch, with more room than data (4096) by the closing launch
    alone.  Later steps keep their scales; a gradient sixteen times larger moves them again."""
    sizes = [16384 * 4, 16384 * 2 + 777, 5, 4096 * 1024, 16384]
    tensors = [_inputs(n, 400 + i, w_fmt, g_fmt, zero_state=True) for i, n in enumerate(sizes)]
    hits = misses = 0
    for step in range(1, 5):
        plain = _fused(be, tensors, w_dt, g_dt, step)
        moved = _fused_shift(be, tensors, w_dt, g_dt, step, slack, up=step % 2 == 0)
        for a, b, t in zip(plain, moved, tensors):
            assert _same_state(a, b), (step, t['w'].numel())
            changed = not (same_float(a['wm'][0], t['wm']['scale']) and same_float(a['mm'][0], t['mm']['scale']) and
                           same_float(a['vm'][0], t['vm']['scale']))
            assert b['redo'] == int(changed)
            hits += 1 - b['redo']
            misses += b['redo']
        tensors = [_next_inputs(t, d, 500 + 10 * step + i, g_fmt, grad_std=1.6e-2 if step == 3 else 1e-3)
                   for i, (t, d) in enumerate(zip(tensors, plain))]
    assert hits >= 3 and misses >= len(sizes)
    be.check_async_error(block=True)


@pytest.mark.parametrize('kw', [dict(adam_mode=True), dict(maximize=True), dict(bias_correction=False), dict(weight_decay=0.0),
                                dict(tensor_scale=False), dict(lr=0.5, eps=0.0)])
def test_shifting_step_variants(be, kw):
    t = [_inputs(16384 * 3 + 100, 7, fp8.E4M3, fp8.E5M2), _inputs(16384 * 2, 8, fp8.E4M3, fp8.E5M2)]
    for step in (2, 3):
        plain = _fused(be, t, 5, 6, step, **kw)
        moved = _fused_shift(be, t, 5, 6, step, 4, up=step == 3, **kw)
        assert all(_same_state(a, b) for a, b in zip(plain, moved))
        t = [_next_inputs(ti, pi, 60 + step + 7 * i, fp8.E5M2) for i, (ti, pi) in enumerate(zip(t, plain))]
    be.check_async_error(block=True)


def test_shifting_step_many_tensors_little_room(be):
    """Forty tensors of eight to forty chunks and room for 48 chunks: every workgroup from the 49th on overwrites a
    chunk whose tensor finished moments ago, and in the first step also does that chunk again."""
    sizes = [16384 * (8 + (7 * i) % 33) - (i % 3) * 1000 for i in range(40)]
    tensors = [_inputs(n, 900 + i, fp8.E4M3, fp8.E5M2, zero_state=i % 2 == 0) for i, n in enumerate(sizes)]
    for step in (1, 2, 3):
        plain = _fused(be, tensors, 5, 6, step)
        moved = _fused_shift(be, tensors, 5, 6, step, 48, up=step == 2)
        assert all(_same_state(a, b) for a, b in zip(plain, moved)), step
        tensors = [_next_inputs(t, d, 950 + 50 * step + i, fp8.E5M2) for i, (t, d) in enumerate(zip(tensors, plain))]
    be.check_async_error(block=True)


def test_config3_full_size_shifting_step_matches(be):
    """1.0e9 parameters as 238 tensors of [4096, 1024] and a tail, 61 036 chunks, with the room the optimizer gives them
    (2816 chunks): one shifting step up and one down from the same state, every tensor compared with the in-place
    step on the same bytes (all full tensors hold the same bytes, so one in-place result serves them all)."""
    per, total = 4096 * 1024, 1_000_000_000
    n_full, tail = total // per, total % per
    base = _inputs(per, 77, fp8.E4M3, fp8.E5M2)
    last = {k: (v[:tail].clone() if isinstance(v, torch.Tensor) else {kk: vv.clone() for kk, vv in v.items()})
            for k, v in base.items()}
    want_full, want_tail = _fused(be, [base, last], 5, 6, 2)
    tensors = [base] * n_full + [last]
    for up in (True, False):
        moved = _fused_shift(be, tensors, 5, 6, 2, 2816, up=up)
        assert _same_state(want_tail, moved[-1])
        for i, d in enumerate(moved[:n_full]):
            assert _same_state(want_full, d), (up, i)
        del moved
    be.check_async_error(block=True)


def _rescaled(t, w=0, g=0, m=0, v=0, g_factor=1.0):
    """The same payloads read through other factors: every scale times 2^k (scale_inv divided), the gradient's scale_inv
    times g_factor on top.  Dequantized values change, codes do not."""
    out = {k: (x.clone() if isinstance(x, torch.Tensor) else {kk: vv.clone() for kk, vv in x.items()}) for k, x in t.items()}
    for key, k in (('wm', w), ('gm', g), ('mm', m), ('vm', v)):
        out[key]['scale'] = out[key]['scale'] * 2.0 ** k
        out[key]['scale_inv'] = out[key]['scale_inv'] * 2.0 ** -k
    out['gm']['scale_inv'] = out['gm']['scale_inv'] * g_factor
    return out


@pytest.mark.parametrize('shifts', [dict(w=28, g=10, m=25, v=20), dict(w=-25, g=-38, m=-27, v=-28), dict(w=45), dict(g=-70),
                                    dict(m=60, v=-60), dict(g_factor=0.3), dict(g_factor=-1.0), dict(g=12, g_factor=1.0 + 2.0 ** -23)])
def test_one_pass_steps_fold_their_factors_only_where_that_is_exact(be, shifts):
    """The one-pass kernels fold the four dequantization factors into the update's coefficients when all of them are
    powers of two between 2^-40 and 2^40, and take the plain chain otherwise.  Payloads read through factors well inside
    that range, at its edges, beyond it, and through a gradient factor that is no power of two (or negative): both
    one-pass forms against the in-place step, which never folds, bit for bit."""
    sizes = [16384 * 2, 16384 + 4001, 16384 * 5]
    tensors = [_rescaled(_inputs(n, 1200 + i, fp8.E4M3, fp8.E5M2), **shifts) for i, n in enumerate(sizes)]
    for step in (2, 3):
        plain = _fused(be, tensors, 5, 6, step)
        moved = _fused_shift(be, tensors, 5, 6, step, 8, up=step == 3)
        spec = _fused(be, tensors, 5, 6, step, speculative=True)
        for a, b, c in zip(plain, moved, spec):
            assert _same_state(a, b) and _same_state(a, c), (step, shifts)
        tensors = [_next_inputs(t, d, 1300 + 10 * step + i, fp8.E5M2) for i, (t, d) in enumerate(zip(tensors, plain))]
    be.check_async_error(block=True)


def test_shifting_step_refuses_a_tensor_longer_than_the_room(be):
    """A tensor of 256 chunks with room for 255: some workgroup would have to overwrite a chunk of its own tensor.  The
    kernel flags the layout in the sticky error word, leaves those chunks alone and runs to its end."""
    tensors = [_inputs(16384 * 2, 31, fp8.E4M3, fp8.E5M2), _inputs(4096 * 1024, 32, fp8.E4M3, fp8.E5M2)]
    be.check_async_error(block=True)
    saved = be._force_two_pass
    try:
        _fused_shift(be, tensors, 5, 6, 2, 255, up=False, check_clean=False)
        with pytest.raises(be.WaitExpiredError):
            be.check_async_error(block=True)
    finally:
        be._force_two_pass = saved
    be.check_async_error(block=True)


def test_fused_step_is_deterministic(be):
    t = _inputs(16384 * 9, 21, fp8.E4M3, fp8.E5M2)
    a = _fused(be, [t], 5, 6, 2)[0]
    b = _fused(be, [t], 5, 6, 2)[0]
    assert torch.equal(a['w'], b['w']) and torch.equal(a['m'], b['m']) and torch.equal(a['v'], b['v'])


def test_stage1_stage2_entry_points(be):
    n = 100003
    t = _inputs(n, 33, fp8.E4M3, fp8.E5M2)
    p0 = fp8.decode(t['w'], fp8.E4M3) * t['wm']['scale_inv']
    g0 = fp8.decode(t['g'], fp8.E5M2) * t['gm']['scale_inv']
    inv_m, inv_v = (1.0 / t['mm']['scale']).item(), (1.0 / t['vm']['scale']).item()
    hyper = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8)
    p_want, am_want, av_want = oadam.stage1(p0, g0, t['m'], inv_m, t['v'], inv_v, step=4, **hyper)
    p, g, m, v = p0.cuda(), g0.cuda(), t['m'].cuda(), t['v'].cuda()
    am, av = torch.zeros(1, device='cuda'), torch.zeros(1, device='cuda')
    be.adamw_stage1(p, g, m, 5, inv_m, am, 0.9, v, 3, inv_v, av, 0.999, 1e-8, 4, 1e-3, True)
    assert torch.equal(p.cpu(), p_want) and am.item() == am_want.item() and av.item() == av_want.item()
    m_want, v_want = oadam.stage2(g0, t['m'], inv_m, 4096.0, t['v'], inv_v, 2.0**20, beta1=0.9, beta2=0.999)
    be.adamw_stage2(g, m, 5, inv_m, 4096.0, 0.9, v, 3, inv_v, 2.0**20, 0.999)
    assert torch.equal(m.cpu(), m_want) and torch.equal(v.cpu(), v_want)


@pytest.mark.parametrize('kw', [dict(), dict(adam_mode=True), dict(maximize=True, weight_decay=0.0), dict(bias_correction=False, eps=1e-6),
                                dict(adam_mode=True, maximize=True, beta1=0.8, beta2=0.999)])
@pytest.mark.parametrize('grad_dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_float32_moment_step_matches_the_oracle_to_the_bit(be, kw, grad_dtype):
    """msamp_adamw_f32 against oracle.adamw.float32_step (the chain of msamp/optim/adamw.py:200-232 with the roundings it
    has on a GPU): parameter and both moments bit-equal over three steps, on a size with a ragged tail and, offset by
    one element, without vector loads; gradients of eight orders of magnitude, some zero, one infinite."""
    hyper = dict(HYPER)
    hyper.update(kw)
    n = 3 * 65536 + 37
    rng = np.random.default_rng(41)
    for offset in (0, 1):
        p = (rng.standard_normal(n) * 0.3).astype(np.float32)
        m = np.zeros(n, np.float32)
        v = np.zeros(n, np.float32)
        dev = [torch.from_numpy(np.concatenate([np.zeros(offset, np.float32), t])).cuda()[offset:] for t in (p, m, v)]
        for step in (1, 2, 3):
            g = (rng.standard_normal(n) * 10.0 ** rng.uniform(-6, 2, n)).astype(np.float32)
            g[::97] = 0.0
            if step == 2:
                g[1234] = np.inf
            g_dev = torch.from_numpy(np.concatenate([np.zeros(offset, np.float32), g])).cuda().to(grad_dtype)[offset:].contiguous()
            g = g_dev.float().cpu().numpy()
            with np.errstate(all='ignore'):
                p, m, v = oadam.float32_step(p, g, m, v, step=step, **hyper)
            be.adamw_f32(dev[0], g_dev, dev[1], dev[2], hyper['lr'], hyper['beta1'], hyper['beta2'], hyper['eps'],
                         hyper['weight_decay'], step, hyper.get('bias_correction', True), hyper.get('adam_mode', False),
                         hyper.get('maximize', False))
            torch.cuda.synchronize()
            for got, want, name in zip(dev, (p, m, v), 'pmv'):
                assert same_float(got, torch.from_numpy(want)), (offset, step, name)
