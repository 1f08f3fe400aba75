"""GPU parity of the FP8 GEMM: within 1e-2 relative Frobenius error of an fp32-class matmul on the
dequantized operands (the bar for this path); fp32 output is held to 1e-3
(the FP8 MFMA aligns the 64 products of a K block to a common exponent with a finite number of bits,
so heavily cancelling sums are not exact to float32)."""

import json
import os

import pytest
import torch

from oracle import fp8, gemm as ogemm
from tests.gpu_util import FMT, rel_fro, same_float

pytestmark = pytest.mark.gpu

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), 'golden', 'reference_kats.json')))
TOL_F32, TOL_16 = 1e-3, 1e-2


@pytest.fixture(scope='module')
def be():
    from msamp import _backend
    _backend.load()
    return _backend


@pytest.fixture
def large_tiles_only(be):
    """Problems small enough for the GEMM with 128 x 128 tiles decline the fused GEMM + cast (the two steps are faster
    there); with the small tile switched off the fused forms take them, which keeps these small cases on the fused path."""
    be.set_small_tile_limit(0)
    yield
    be.set_small_tile_limit(128)


def _rand_fp8(shape, fp8_dt, seed, spread=1.0):
    """Random FP8 payload (finite codes) built by quantizing N(0, spread) on the CPU."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g) * spread
    return fp8.encode(x, FMT[fp8_dt])


def _run(be, a, a_dt, a_si, b, b_dt, b_si, out_dtype=torch.float32, accumulate=False, bias=None, out=None):
    n, m = b.shape[0], a.shape[0]
    if out is None:
        out = torch.empty(n, m, dtype=out_dtype, device='cuda')
    be.fp8_gemm(a.cuda(), a_dt, torch.tensor(a_si, device='cuda'), b.cuda(), b_dt, torch.tensor(b_si, device='cuda'), out,
                accumulate, None if bias is None else bias.cuda())
    return out


def test_reference_ones_case_through_api():
    import msamp    # noqa: F401
    from msamp.common.dtype import Dtypes
    from msamp.operators.gemm import Gemm
    k = GOLDEN['gemm_ones']
    ta = torch.ones(k['a_shape'], device='cuda')
    tb = torch.ones(k['b_shape'], device='cuda')
    sa, sb = ta.cast(Dtypes.kfloat8_e4m3), tb.cast(Dtypes.kfloat8_e4m3)
    out = Gemm.fp8_gemm(sa, sb, Dtypes.kfloat32)
    assert list(out.shape) == k['out_shape'] and out.equal(torch.matmul(tb, ta.t())) and (out == k['value']).all()
    out = torch.ones(k['out_shape'], device='cuda')
    out = Gemm.fp8_gemm(sa, sb, Dtypes.kfloat32, out=out)
    assert (out == k['value']).all()


@pytest.mark.parametrize('a_dt,b_dt', [(5, 5), (5, 6), (6, 5), (6, 6)])
@pytest.mark.parametrize('m,n,k', [(32, 32, 64), (128, 128, 128), (256, 256, 256), (300, 200, 384), (1, 1, 16), (33, 65, 48),
                                   (512, 384, 1040), (129, 257, 144)])
def test_random_against_oracle(be, a_dt, b_dt, m, n, k):
    a = _rand_fp8((m, k), a_dt, 1000 + m + k)
    b = _rand_fp8((n, k), b_dt, 2000 + n + k)
    a_si, b_si = 0.125, 2.0
    want = ogemm.fp8_gemm(a, torch.tensor(a_si), FMT[a_dt], b, torch.tensor(b_si), FMT[b_dt])
    got = _run(be, a, a_dt, a_si, b, b_dt, b_si)
    assert rel_fro(got, want) < TOL_F32
    got16 = _run(be, a, a_dt, a_si, b, b_dt, b_si, out_dtype=torch.bfloat16)
    assert rel_fro(got16.float(), want) < TOL_16


def test_orientation_probe(be):
    """One-hot rows: out[n, m] must pair row n of b with row m of a."""
    m, n, k = 70, 40, 64
    a = torch.zeros(m, k)
    b = torch.zeros(n, k)
    for i in range(m):
        a[i, i % k] = 1.0 + (i % 7)
    for j in range(n):
        b[j, (3 * j) % k] = 1.0 + (j % 5)
    aq, bq = fp8.encode(a, fp8.E4M3), fp8.encode(b, fp8.E4M3)
    got = _run(be, aq, 5, 1.0, bq, 5, 1.0).cpu()
    assert torch.equal(got, b @ a.t())


@pytest.mark.parametrize('out_dtype', [torch.float32, torch.float16, torch.bfloat16])
def test_accumulate_and_bias(be, out_dtype):
    m, n, k = 192, 136, 256
    a, b = _rand_fp8((m, k), 5, 1), _rand_fp8((n, k), 6, 2, spread=0.01)
    g = torch.Generator().manual_seed(3)
    prev = torch.randn(n, m, generator=g).to(out_dtype)
    bias = torch.randn(m, generator=g).to(out_dtype)
    want = ogemm.fp8_gemm(a, torch.tensor(0.5), fp8.E4M3, b, torch.tensor(4.0), fp8.E5M2, out=prev.float(), bias=bias.float())
    got = _run(be, a, 5, 0.5, b, 6, 4.0, accumulate=True, bias=bias, out=prev.cuda().clone())
    assert rel_fro(got.float(), want) < (TOL_F32 if out_dtype == torch.float32 else TOL_16)


@pytest.mark.parametrize('m,n,k', [(4096, 2048, 256), (4100, 2056, 384), (3001, 2999, 128), (4101, 1031, 256)])
@pytest.mark.parametrize('out_dtype', [torch.bfloat16, torch.float32, torch.float16])
def test_large_tiles_ragged_edges_accumulate_bias(be, m, n, k, out_dtype):
    """Shapes big enough for the 256x256 direct-to-LDS kernel, with ragged right/bottom edges,
    odd row lengths (no 16-byte row stores), bias and accumulation."""
    a, b = _rand_fp8((m, k), 5, 5), _rand_fp8((n, k), 6, 6, spread=0.05)
    tol = TOL_F32 if out_dtype == torch.float32 else TOL_16
    want = ogemm.fp8_gemm(a, torch.tensor(0.25), fp8.E4M3, b, torch.tensor(8.0), fp8.E5M2)
    got = _run(be, a, 5, 0.25, b, 6, 8.0, out_dtype=out_dtype)
    assert rel_fro(got.float(), want) < tol
    g = torch.Generator().manual_seed(9)
    prev = torch.randn(n, m, generator=g).to(out_dtype)
    bias = torch.randn(m, generator=g).to(out_dtype)
    want2 = want + prev.float() + bias.float().view(1, -1)
    got2 = _run(be, a, 5, 0.25, b, 6, 8.0, accumulate=True, bias=bias, out=prev.cuda().clone())
    assert rel_fro(got2.float(), want2) < tol
    # untouched memory around the output: write into the middle of a larger buffer
    buf = torch.full((n + 2, m), 7.0, dtype=out_dtype, device='cuda')
    _run(be, a, 5, 0.25, b, 6, 8.0, out=buf[1:n + 1])
    assert (buf[0] == 7).all() and (buf[n + 1] == 7).all() and torch.equal(buf[1:n + 1], got)


@pytest.mark.parametrize('a_dt,b_dt', [(5, 5), (5, 6), (6, 5)])
@pytest.mark.parametrize('m,n,k', [(256, 256, 256), (512, 768, 384), (1024, 300, 256), (4096, 4096, 512), (256, 512, 640)])
@pytest.mark.parametrize('out_dtype', [torch.float32, torch.bfloat16])
def test_kmajor_operands_match_transposed_copies(be, a_dt, b_dt, m, n, k, out_dtype):
    """Operands handed over as [K, rows] must give exactly what the row-major kernel gives on their transposed
    copies (same products, same order): `a` alone K-major for any n, both K-major when n is a multiple of 256;
    with bias and accumulation as well."""
    a = _rand_fp8((m, k), a_dt, 11 * m + k).cuda()
    b = _rand_fp8((n, k), b_dt, 13 * n + k, spread=0.5).cuda()
    a_t, b_t = a.t().contiguous(), b.t().contiguous()
    sa, sb = torch.tensor(0.25, device='cuda'), torch.tensor(2.0, device='cuda')
    same = torch.equal

    want = be.fp8_gemm(a, a_dt, sa, b, b_dt, sb, torch.empty(n, m, dtype=out_dtype, device='cuda'))
    got = be.fp8_gemm(a_t, a_dt, sa, b, b_dt, sb, torch.empty(n, m, dtype=out_dtype, device='cuda'), a_kmajor=True)
    assert same(got, want)
    assert be.gemm_kmajor_supported(m, n, k, True, True) == (n % 256 == 0)
    if n % 256 == 0:
        got_both = be.fp8_gemm(a_t, a_dt, sa, b_t, b_dt, sb, torch.empty(n, m, dtype=out_dtype, device='cuda'), a_kmajor=True,
                               b_kmajor=True)
        assert torch.equal(got_both, got)    # one kernel, two layouts: always to the bit
        assert same(got_both, want)
        bias = torch.randn(m, device='cuda').to(out_dtype)
        base = torch.randn(n, m, device='cuda').to(out_dtype)
        want2 = be.fp8_gemm(a, a_dt, sa, b, b_dt, sb, base.clone(), accumulate=True, bias=bias)
        got2 = be.fp8_gemm(a_t, a_dt, sa, b_t, b_dt, sb, base.clone(), accumulate=True, bias=bias, a_kmajor=True, b_kmajor=True)
        assert same(got2, want2)


def test_kmajor_rejects_unsupported_shapes(be):
    a = _rand_fp8((128, 100), 5, 1).cuda()    # [K=128, M=100]: M is not a multiple of 256
    b = _rand_fp8((64, 128), 5, 2).cuda()
    one = torch.ones((), device='cuda')
    with pytest.raises(RuntimeError):
        be.fp8_gemm(a, 5, one, b, 5, one, torch.empty(64, 100, device='cuda'), a_kmajor=True)
    assert not be.gemm_kmajor_supported(100, 64, 128, True, False)
    assert not be.gemm_kmajor_supported(256, 256, 256, False, True)
    assert not be.gemm_kmajor_supported(256, 256, 128, True, True)    # a single 128-byte slice of K: not for this kernel
    assert be.gemm_kmajor_supported(256, 256, 256, True, True)


def test_k_not_multiple_of_16_is_padded_by_the_operator():
    import msamp    # noqa: F401
    from msamp.common.dtype import Dtypes
    from msamp.operators.gemm import Gemm
    g = torch.Generator().manual_seed(4)
    ta, tb = torch.randn(5, 7, generator=g).cuda(), torch.randn(3, 7, generator=g).cuda()
    sa, sb = ta.cast(Dtypes.kfloat8_e4m3), tb.cast(Dtypes.kfloat8_e5m2)
    out = Gemm.fp8_gemm(sa, sb, Dtypes.kfloat32)
    want = sb.float() @ sa.float().t()
    assert out.shape == (3, 5) and rel_fro(out, want) < TOL_F32


def test_operands_at_odd_offsets_of_a_flat_buffer(be):
    """A payload that is a view one byte into a flat buffer: the operator copies it to an aligned allocation and gives
    the bits of the aligned call; the C entry point itself names the alignment in its error."""
    import msamp    # noqa: F401
    from msamp.common.dtype import Dtypes
    from msamp.common.tensor import ScalingTensor
    from msamp.operators.gemm import Gemm
    g = torch.Generator().manual_seed(11)
    for (m, n, k), kmajor in [((48, 40, 64), False), ((256, 512, 256), True), ((256, 256, 384), False)]:
        sa = (torch.randn(m, k, generator=g).cuda()).cast(Dtypes.kfloat8_e4m3)
        sb = (torch.randn(n, k, generator=g).cuda()).cast(Dtypes.kfloat8_e5m2)
        want = Gemm.fp8_gemm(sa, sb, Dtypes.kbfloat16)
        want_q = Gemm.fp8_gemm(sa, sb, Dtypes.kfloat32).cast(Dtypes.kfloat8_e4m3)

        def shifted(t, transposed=False):
            payload = t.value.t().contiguous() if transposed else t.value
            flat = torch.empty(payload.numel() + 1, dtype=torch.uint8, device='cuda')
            view = flat[1:].view(payload.shape)
            view.copy_(payload)
            assert view.data_ptr() % 16 == 1 and view.is_contiguous()
            return ScalingTensor(view, t.meta)

        ua, ub = shifted(sa, kmajor), shifted(sb)
        got = Gemm.fp8_gemm(ua, ub, Dtypes.kbfloat16, a_kmajor=kmajor)
        assert torch.equal(got, want)
        if m % 256 == 0 and n % 256 == 0 and not kmajor:
            from msamp.common.tensor import ScalingMeta
            meta = ScalingMeta(Dtypes.kfloat8_e4m3, window_size=1)
            fused = Gemm.fp8_gemm_cast(shifted(sa), ub, Dtypes.kfloat32, meta)
            assert fused is not None and torch.equal(fused.value, want_q.value)
        with pytest.raises(RuntimeError, match='aligned'):
            out = torch.empty(n, m, dtype=torch.bfloat16, device='cuda')
            be.fp8_gemm(shifted(sa).value, 5, sa.meta.scale_inv, ub.value, 6, sb.meta.scale_inv, out)


def test_bad_arguments_raise(be):
    a = torch.zeros(16, 24, dtype=torch.uint8, device='cuda')
    si = torch.ones((), device='cuda')
    with pytest.raises(RuntimeError):
        be.fp8_gemm(a, 5, si, a, 5, si, torch.empty(16, 16, device='cuda'))    # K % 16 != 0
    with pytest.raises(ValueError):
        be.fp8_gemm(a, 5, si, a, 5, si, torch.empty(8, 16, device='cuda'))    # wrong output shape


def test_config2_fp8linear_shapes_sampled(be):
    """The three GEMMs of one FP8Linear step at x[8192,4096], W[4096,4096]: forward, dgrad, wgrad.
    Checked on a sample of output rows/columns against the oracle, plus linearity in the scale."""
    tokens, d_in, d_out = 8192, 4096, 4096
    x = _rand_fp8((tokens, d_in), 5, 11)
    w = _rand_fp8((d_out, d_in), 5, 12, spread=0.02 * 64)
    dy = _rand_fp8((tokens, d_out), 6, 13)
    xs, ws, dys = 1 / 64., 1 / 4096., 2.0**-16
    rows = torch.tensor([0, 1, 255, 256, 4095, 4096, 8191])
    cols = torch.tensor([0, 31, 32, 1000, 4095])
    # forward: y[tokens, d_out] = x W^T  -> a = W, b = x
    y = _run(be, w, 5, ws, x, 5, xs, out_dtype=torch.bfloat16)
    want = ogemm.fp8_gemm(w[cols], torch.tensor(ws), fp8.E4M3, x[rows], torch.tensor(xs), fp8.E4M3)
    assert rel_fro(y[rows.cuda()][:, cols.cuda()].float(), want) < TOL_16
    # dgrad: dx[tokens, d_in] = dy W -> a = W^T[d_in, d_out], b = dy
    wt = w.t().contiguous()
    dx = _run(be, wt, 5, ws, dy, 6, dys, out_dtype=torch.bfloat16)
    want = ogemm.fp8_gemm(wt[cols], torch.tensor(ws), fp8.E4M3, dy[rows], torch.tensor(dys), fp8.E5M2)
    assert rel_fro(dx[rows.cuda()][:, cols.cuda()].float(), want) < TOL_16
    # wgrad: dW[d_out, d_in] = dy^T x -> a = x^T[d_in, tokens], b = dy^T[d_out, tokens]
    xt, dyt = x.t().contiguous(), dy.t().contiguous()
    dw = _run(be, xt, 5, xs, dyt, 6, dys, out_dtype=torch.float32)
    r2 = torch.tensor([0, 1, 2047, 4095])
    want = ogemm.fp8_gemm(xt[cols], torch.tensor(xs), fp8.E4M3, dyt[r2], torch.tensor(dys), fp8.E5M2)
    assert rel_fro(dw[r2.cuda()][:, cols.cuda()], want) < TOL_F32
    dw2 = _run(be, xt, 5, 2 * xs, dyt, 6, dys, out_dtype=torch.float32)
    assert torch.equal(dw2, 2 * dw)


def _gpu_codes(shape, fp8_dt, seed):
    """Random finite FP8 payload made on the GPU (magnitude codes below the top binade, random sign)."""
    g = torch.Generator(device='cuda').manual_seed(seed)
    top = 0x70 if fp8_dt == 5 else 0x74
    mag = torch.randint(0, top, shape, generator=g, device='cuda', dtype=torch.uint8)
    sign = torch.randint(0, 2, shape, generator=g, device='cuda', dtype=torch.uint8) << 7
    return mag | sign


@pytest.mark.parametrize('tokens,d_out,d_in', [(16384, 11008, 4096), (16384, 4096, 11008), (16384, 12288, 4096),
                                               (16384, 4096, 4096), (16384, 8192, 28672), (16384, 10240, 8192),
                                               (16384, 28672, 8192), (16384, 8192, 8192)])
def test_llama_layer_shapes_sampled(be, tokens, d_out, d_in):
    """Forward, dgrad and wgrad of the Llama-7B / 70B projection shapes (K up to 28672), operands handed over the way
    the layer holds them (dgrad and wgrad read K-major operands in place).  Sampled rows and columns against the
    oracle; exact linearity in the output factor over the whole matrix."""
    x = _gpu_codes((tokens, d_in), 5, 1)
    w = _gpu_codes((d_out, d_in), 5, 2)
    dy = _gpu_codes((tokens, d_out), 6, 3)
    xs, ws, dys = 2.0**-7, 2.0**-9, 2.0**-14
    one = lambda v: torch.tensor(v, device='cuda')
    rows = torch.tensor([0, 255, 256, 8191, tokens - 1])
    cols = torch.tensor([0, 31, 257, d_out - 1])
    cin = torch.tensor([0, 129, 4000, d_in - 1])
    cpu = lambda t, idx, dim=0: t.index_select(dim, idx.cuda()).cpu()
    # forward y[tokens, d_out] = x W^T
    y = torch.empty(tokens, d_out, dtype=torch.bfloat16, device='cuda')
    be.fp8_gemm(w, 5, one(ws), x, 5, one(xs), y)
    want = ogemm.fp8_gemm(cpu(w, cols), torch.tensor(ws), fp8.E4M3, cpu(x, rows), torch.tensor(xs), fp8.E4M3)
    assert rel_fro(y[rows.cuda()][:, cols.cuda()].float(), want) < TOL_16
    y2 = torch.empty_like(y)
    be.fp8_gemm(w, 5, one(2 * ws), x, 5, one(xs), y2)
    assert torch.equal(y2, 2 * y)
    del y, y2
    # dgrad dx[tokens, d_in] = dy W: a = W^T, handed over as W (K-major)
    assert be.gemm_kmajor_supported(d_in, tokens, d_out, True, False)
    dx = torch.empty(tokens, d_in, dtype=torch.bfloat16, device='cuda')
    be.fp8_gemm(w, 5, one(ws), dy, 6, one(dys), dx, a_kmajor=True)
    want = ogemm.fp8_gemm(cpu(w, cin, 1).t().contiguous(), torch.tensor(ws), fp8.E4M3, cpu(dy, rows), torch.tensor(dys), fp8.E5M2)
    assert rel_fro(dx[rows.cuda()][:, cin.cuda()].float(), want) < TOL_16
    del dx
    # wgrad dW[d_out, d_in] = dy^T x: a = x^T, b = dy^T, handed over as x and dy (both K-major)
    assert be.gemm_kmajor_supported(d_in, d_out, tokens, True, True)
    dw = torch.empty(d_out, d_in, dtype=torch.float32, device='cuda')
    be.fp8_gemm(x, 5, one(xs), dy, 6, one(dys), dw, a_kmajor=True, b_kmajor=True)
    want = ogemm.fp8_gemm(cpu(x, cin, 1).t().contiguous(), torch.tensor(xs), fp8.E4M3, cpu(dy, cols, 1).t().contiguous(),
                          torch.tensor(dys), fp8.E5M2)
    assert rel_fro(dw[cols.cuda()][:, cin.cuda()], want) < TOL_F32


def _strip(n):
    """One index per block of 256 (one per tile of the kernel), at an offset that moves through the tile: whole rows and
    columns of the output at these indices pass through every tile, every wave quadrant and every 16-row block."""
    return torch.tensor([min(256 * i + (37 * i + 5) % 256, n - 1) for i in range((n + 255) // 256)])


@pytest.mark.parametrize('tokens,d_out,d_in', [(16384, 11008, 4096), (16384, 4096, 11008), (16384, 12288, 4096),
                                               (16384, 4096, 4096), (16384, 8192, 28672), (16384, 10240, 8192),
                                               (16384, 28672, 8192), (16384, 8192, 8192)])
def test_llama_layer_shapes_whole_rows_and_columns(be, tokens, d_out, d_in):
    """The same 24 GEMMs, each checked on whole output rows and whole output columns -- one row through every row of
    tiles, one column through every column of tiles, so every tile and each of its four wave quadrants is crossed --
    against a float32 matmul on the CPU of the operands as torch's own float8 types decode them."""
    x = _gpu_codes((tokens, d_in), 5, 11)
    w = _gpu_codes((d_out, d_in), 5, 12)
    dy = _gpu_codes((tokens, d_out), 6, 13)
    xs, ws, dys = 2.0**-7, 2.0**-9, 2.0**-14
    one = lambda v: torch.tensor(v, device='cuda')
    xf = (x.view(torch.float8_e4m3fn).float() * xs).cpu()
    wf = (w.view(torch.float8_e4m3fn).float() * ws).cpu()
    dyf = (dy.view(torch.float8_e5m2).float() * dys).cpu()
    rt, ro, ri = _strip(tokens), _strip(d_out), _strip(d_in)

    def check(out, want_rows, r, want_cols, c, tol):
        assert rel_fro(out[r.cuda()].float().cpu(), want_rows) < tol
        assert rel_fro(out[:, c.cuda()].float().cpu(), want_cols) < tol
        # and nothing in the strips is far off on its own (a slip confined to a few elements hides in a norm)
        scale = want_rows.abs().max().item()
        assert (out[r.cuda()].float().cpu() - want_rows).abs().max().item() < 0.05 * scale

    y = torch.empty(tokens, d_out, dtype=torch.bfloat16, device='cuda')
    be.fp8_gemm(w, 5, one(ws), x, 5, one(xs), y)
    check(y, xf[rt] @ wf.t(), rt, xf @ wf[ro].t(), ro, TOL_16)
    del y
    dx = torch.empty(tokens, d_in, dtype=torch.bfloat16, device='cuda')
    be.fp8_gemm(w, 5, one(ws), dy, 6, one(dys), dx, a_kmajor=True)
    check(dx, dyf[rt] @ wf, rt, dyf @ wf[:, ri], ri, TOL_16)
    del dx
    dw = torch.empty(d_out, d_in, dtype=torch.float32, device='cuda')
    be.fp8_gemm(x, 5, one(xs), dy, 6, one(dys), dw, a_kmajor=True, b_kmajor=True)
    check(dw, dyf[:, ro].t() @ xf, ro, dyf.t() @ xf[:, ri], ri, TOL_F32)


def test_operand_beyond_4_gib(be):
    """An operand of 70 016 x 65 536 bytes (4.6 GB): its 32-bit byte offsets would wrap, so the library has to route
    it to the kernel with 64-bit addressing.  Rows below and above the 4 GiB mark against the oracle."""
    m, n, k = 256, 70016, 65536
    a = _gpu_codes((m, k), 5, 21)
    b = _gpu_codes((n, k), 5, 22)
    one = lambda v: torch.tensor(v, device='cuda')
    out = torch.empty(n, m, dtype=torch.float32, device='cuda')
    be.fp8_gemm(a, 5, one(2.0**-8), b, 5, one(2.0**-8), out)
    rows = torch.tensor([0, 65535, 65536, 65537, n - 1])
    want = ogemm.fp8_gemm(a.cpu(), torch.tensor(2.0**-8), fp8.E4M3, b[rows.cuda()].cpu(), torch.tensor(2.0**-8), fp8.E4M3)
    assert rel_fro(out[rows.cuda()], want) < TOL_F32


def _two_steps(be, a, a_dt, sa, b, b_dt, sb, hp, nan_to_inf, kmajor, old_scale=1.0):
    """The unfused path: GEMM into an hp buffer, then the in-time cast of that buffer."""
    k, m = a.shape if kmajor else a.shape[::-1]
    n = b.shape[1] if kmajor else b.shape[0]
    d = be.fp8_gemm(a, a_dt, sa, b, b_dt, sb, torch.empty(n, m, dtype=hp, device='cuda'), a_kmajor=kmajor, b_kmajor=kmajor)
    s, si, am = torch.full((), old_scale, device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')
    q = be.cast_to_fp8_intime(d, s, am, si, 5, nan_to_inf=nan_to_inf)
    return q, s, si, am


@pytest.mark.parametrize('a_dt,b_dt', [(5, 6), (5, 5), (6, 6)])
@pytest.mark.parametrize('m,n,k', [(256, 256, 256), (1024, 512, 384), (4096, 4096, 512), (2048, 8192, 256), (512, 256, 640)])
@pytest.mark.parametrize('hp', [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize('kmajor', [True, False])
def test_gemm_with_fused_cast_matches_the_two_steps(be, large_tiles_only, a_dt, b_dt, m, n, k, hp, kmajor):
    """GEMM + in-time cast in one launch: payload, amax, scale and scale_inv must equal, bit for bit, what the GEMM
    into an hp buffer followed by the in-time cast of that buffer gives (the weight-gradient path of FP8Linear)."""
    a = _rand_fp8((m, k), a_dt, 3 * m + k).cuda()
    b = _rand_fp8((n, k), b_dt, 5 * n + k, spread=0.5).cuda()
    if kmajor:
        a, b = a.t().contiguous(), b.t().contiguous()
    sa, sb = torch.tensor(0.125, device='cuda'), torch.tensor(0.5, device='cuda')
    want_q, want_s, want_si, want_am = _two_steps(be, a, a_dt, sa, b, b_dt, sb, hp, True, kmajor)
    s, si, am = torch.ones((), device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')
    got = be.fp8_gemm_cast(a, a_dt, sa, b, b_dt, sb, hp, 5, s, am, si, nan_to_inf=True, a_kmajor=kmajor, b_kmajor=kmajor)
    assert got is not None, 'the fused kernel should take this problem'
    assert torch.equal(got, want_q)
    assert same_float(am, want_am) and same_float(s, want_s) and same_float(si, want_si)
    assert float(want_am) > 0


@pytest.mark.parametrize('nan_to_inf', [True, False])
@pytest.mark.parametrize('poison', ['nan', 'inf', 'zero'])
def test_gemm_with_fused_cast_special_values(be, nan_to_inf, poison):
    """A NaN or Inf in the product (E5M2 operands carry them) reaches amax as through the two steps, the scale falls
    back to the old one; an all-zero product leaves amax 0 and the old scale."""
    m, n, k = 512, 256, 256
    a = _rand_fp8((k, m), 6, 1).cuda()    # both operands K-major, as the backward pass has them
    b = _rand_fp8((k, n), 6, 2).cuda()
    if poison == 'nan':
        a[7, 5] = 0x7f
    elif poison == 'inf':
        a[7, 5] = 0x7c
    else:
        a.zero_()
    one = torch.ones((), device='cuda')
    want_q, want_s, want_si, want_am = _two_steps(be, a, 6, one, b, 6, one, torch.bfloat16, nan_to_inf, True, old_scale=4.0)
    s, si, am = torch.full((), 4.0, device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')
    got = be.fp8_gemm_cast(a, 6, one, b, 6, one, torch.bfloat16, 5, s, am, si, nan_to_inf=nan_to_inf, a_kmajor=True, b_kmajor=True)
    assert got is not None
    assert torch.equal(got, want_q)
    assert same_float(am, want_am) and same_float(s, want_s) and same_float(si, want_si)


def test_gemm_with_fused_cast_declines_what_it_cannot_take(be):
    """Ragged shapes, mixed layouts, more tiles than compute units without speculation: None, and nothing written."""
    one = torch.ones((), device='cuda')

    def call(m, n, k, **kw):
        a = _rand_fp8((k, m) if kw.get('a_kmajor') else (m, k), 5, 1).cuda()
        b = _rand_fp8((k, n) if kw.get('b_kmajor') else (n, k), 5, 2).cuda()
        s, si, am = torch.full((), 2.0, device='cuda'), torch.full((), 3.0, device='cuda'), torch.full((1,), 5.0, device='cuda')
        got = be.fp8_gemm_cast(a, 5, one, b, 5, one, torch.bfloat16, kw.pop('q_dt', 5), s, am, si, **kw)
        return got, float(s), float(si), float(am)

    assert call(300, 256, 256) == (None, 2.0, 3.0, 5.0)
    assert call(256, 256, 272) == (None, 2.0, 3.0, 5.0)
    assert call(256, 256, 128) == (None, 2.0, 3.0, 5.0)    # a single slice of K
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    side = 256 * (int(cus ** 0.5) + 1)
    assert call(side, side, 256, speculate=False) == (None, 2.0, 3.0, 5.0)    # more tiles than compute units wait for nobody
    assert call(256, 256, 256, q_dt=6) == (None, 2.0, 3.0, 5.0)
    assert call(256, 256, 256, a_kmajor=True) == (None, 2.0, 3.0, 5.0)    # mixed layouts
    for layout in (dict(), dict(a_kmajor=True, b_kmajor=True)):
        got, *_ = call(256, 256, 256, **layout)
        assert got is not None
    # small enough for the 128 x 128 tiles (K of four slices and more, few large tiles): the two steps are faster
    assert call(512, 256, 640) == (None, 2.0, 3.0, 5.0)
    assert call(2048, 2048, 1024, a_kmajor=True, b_kmajor=True) == (None, 2.0, 3.0, 5.0)
    try:
        be.set_small_tile_limit(0)
        got, *_ = call(512, 256, 640)
        assert got is not None
    finally:
        be.set_small_tile_limit(128)


def _spec_case(be, a, a_dt, sa, b, b_dt, sb, hp, kmajor, meta, old=None):
    """One call of the speculative form on `meta` = (scale, scale_inv, amax) against the two steps from the same meta
    values; returns the codes.  `old`: previous gradient to accumulate into."""
    k, m = a.shape if kmajor else a.shape[::-1]
    n = b.shape[1] if kmajor else b.shape[0]
    s, si, am = meta
    s2, si2, am2 = s.clone(), si.clone(), am.clone()
    d2 = old.clone() if old is not None else torch.empty(n, m, dtype=hp, device='cuda')
    be.fp8_gemm(a, a_dt, sa, b, b_dt, sb, d2, accumulate=old is not None, a_kmajor=kmajor, b_kmajor=kmajor)
    want = be.cast_to_fp8_intime(d2, s2, am2, si2, 5, nan_to_inf=True, two_pass=True, speculate=False)
    d = old.clone() if old is not None else torch.full((n, m), float('nan'), dtype=hp, device='cuda')
    got = be.fp8_gemm_cast(a, a_dt, sa, b, b_dt, sb, hp, 5, s, am, si, nan_to_inf=True, a_kmajor=kmajor, b_kmajor=kmajor,
                           hp_out=d, accumulate=old is not None)
    assert got is not None, 'the speculative form should take this problem'
    assert torch.equal(d.view(torch.int16), d2.view(torch.int16)), 'the stored product differs from the plain GEMM'
    assert torch.equal(got, want)
    assert same_float(am, am2) and same_float(s, s2) and same_float(si, si2)
    return got


@pytest.mark.parametrize('a_dt,b_dt', [(5, 6), (5, 5)])
@pytest.mark.parametrize('m,n,k', [(4352, 4096, 256), (4096, 11008, 384), (8192, 28672, 256), (512, 256, 640)])
@pytest.mark.parametrize('hp', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('kmajor', [True, False])
def test_gemm_with_speculative_cast_matches_the_two_steps(be, large_tiles_only, a_dt, b_dt, m, n, k, hp, kmajor):
    """More output tiles than compute units (272, 688 and 3584 tiles; the small case is sent the same way by keeping
    the waiting kernels off): the GEMM stores the product and, beside it, the codes for the scale the meta holds.  A
    fresh meta (scale 1: the rule moves it, the product is cast again), the same operands again (the scale stands:
    nothing is read back), operands four times larger (the scale moves again), then accumulation into the previous
    product: codes, amax, scale, scale_inv and the stored product equal the two steps, bit for bit, every time."""
    a = _gpu_codes((k, m) if kmajor else (m, k), a_dt, 3 * m + k)
    b = _gpu_codes((k, n) if kmajor else (n, k), b_dt, 5 * n + k)
    # (the codes are uniformly random, E5M2 ones reach 14336: factors that keep the float16 products finite)
    sa, sb = (torch.tensor(v, device='cuda') for v in ((0.125, 0.5) if hp == torch.bfloat16 else (2.0 ** -12, 2.0 ** -10)))
    meta = (torch.ones((), device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda'))
    small = (m // 256) * (n // 256) <= torch.cuda.get_device_properties(0).multi_processor_count
    saved = be._force_two_pass
    be._force_two_pass = be._force_two_pass or small
    try:
        _spec_case(be, a, a_dt, sa, b, b_dt, sb, hp, kmajor, meta)
        first_scale = meta[0].clone()
        assert float(first_scale) != 1.0
        _spec_case(be, a, a_dt, sa, b, b_dt, sb, hp, kmajor, meta)
        assert same_float(meta[0], first_scale)
        _spec_case(be, a, a_dt, sa * 4, b, b_dt, sb, hp, kmajor, meta)
        assert float(meta[0]) == float(first_scale) / 4
        g = torch.Generator(device='cuda').manual_seed(m + n)
        old = (torch.randn(n, m, device='cuda', generator=g) * float(meta[2][0]) * 0.3).to(hp)
        _spec_case(be, a, a_dt, sa * 4, b, b_dt, sb, hp, kmajor, meta, old=old)
    finally:
        be._force_two_pass = saved


@pytest.mark.parametrize('poison', ['nan', 'inf', 'zero'])
def test_gemm_with_speculative_cast_special_values(be, poison):
    """A NaN or an Inf in the product, or an all-zero product, through the speculative form (272 tiles)."""
    m, n, k = 4352, 4096, 256
    a = _gpu_codes((k, m), 6, 1)
    b = _gpu_codes((k, n), 6, 2)
    if poison == 'nan':
        a[7, 5] = 0x7f
    elif poison == 'inf':
        a[7, 5] = 0x7c
    else:
        a.zero_()
    one = torch.ones((), device='cuda')
    meta = (torch.full((), 4.0, device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda'))
    _spec_case(be, a, 6, one, b, 6, one, torch.bfloat16, True, meta)
    _spec_case(be, a, 6, one, b, 6, one, torch.bfloat16, True, meta)


def test_gemm_with_speculative_cast_replays_from_a_graph(be):
    """The speculative form waits for nobody and takes its decisions on the GPU, so it can be captured: replays over
    operands whose scale stands and whose scale moves, each against the eager two steps, with eager work in between."""
    m, n, k = 4352, 4096, 256
    a = _gpu_codes((k, m), 5, 11)
    b = _gpu_codes((k, n), 6, 12)
    sb = torch.tensor(0.5, device='cuda')
    sa = torch.tensor(0.125, device='cuda')
    s, si, am = torch.ones((), device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')
    d = torch.empty(n, m, dtype=torch.bfloat16, device='cuda')
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        be.fp8_gemm_cast(a, 5, sa, b, 6, sb, torch.bfloat16, 5, s, am, si, nan_to_inf=True, a_kmajor=True, b_kmajor=True, hp_out=d)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        q = be.fp8_gemm_cast(a, 5, sa, b, 6, sb, torch.bfloat16, 5, s, am, si, nan_to_inf=True, a_kmajor=True, b_kmajor=True, hp_out=d)
    assert q is not None
    for factor in (0.125, 0.125, 1.0, 1.0, 0.03125, 0.125):
        sa.fill_(factor)
        s0, si0, am0 = s.clone(), si.clone(), am.clone()
        graph.replay()
        d2 = be.fp8_gemm(a, 5, sa, b, 6, sb, torch.empty_like(d), a_kmajor=True, b_kmajor=True)
        want = be.cast_to_fp8_intime(d2, s0, am0, si0, 5, nan_to_inf=True, two_pass=True, speculate=False)
        torch.cuda.synchronize()
        assert torch.equal(q, want) and torch.equal(d.view(torch.int16), d2.view(torch.int16)), factor
        assert same_float(am, am0) and same_float(s, s0) and same_float(si, si0), factor


def test_fp8linear_weight_gradient_uses_the_fused_kernel_and_matches(be, large_tiles_only):
    """FP8Linear backward: the weight gradient from the fused launch equals the one from the two steps."""
    import msamp
    from msamp import _backend
    from msamp.nn import LinearReplacer
    from msamp.common.dtype import Dtypes
    torch.manual_seed(3)
    lin = torch.nn.Linear(512, 256, bias=False).cuda().bfloat16()
    model = LinearReplacer.replace(lin, Dtypes.kfloat16)
    x = torch.randn(1024, 512, device='cuda', dtype=torch.bfloat16)
    dy = torch.randn(1024, 256, device='cuda', dtype=torch.bfloat16)

    def grad(fused):
        saved = _backend.fp8_gemm_cast
        calls = []
        if fused:
            def spy(*a, **kw):
                out = saved(*a, **kw)
                calls.append(out is not None)
                return out
            _backend.fp8_gemm_cast = spy
        else:
            _backend.fp8_gemm_cast = lambda *a, **kw: None
        try:
            for p in model.parameters():
                p.grad = None
            model(x).backward(dy)
        finally:
            _backend.fp8_gemm_cast = saved
        g = model.weight.grad
        return g.value.clone(), g.meta.scale.clone(), g.meta.scale_inv.clone(), g.meta.amax.clone(), calls

    q1, s1, si1, am1, calls = grad(True)
    assert calls == [True]
    q0, s0, si0, am0, _ = grad(False)
    assert torch.equal(q1, q0) and same_float(s1, s0) and same_float(si1, si0) and same_float(am1, am0)


def test_gemm_with_fused_cast_many_random_cases(be, large_tiles_only):
    """A sweep over seeds, scales, layouts and output types, with few tiles (where the unfused row-major GEMM runs the
    generic kernel) and many: every case equal to the two steps, to the bit."""
    cases = 0
    for it in range(12):
        for (m, n, k), kmajor in (((1024, 768, 384), True), ((256, 256, 1024), False), ((3072, 3072, 256), False),
                                  ((4096, 1024, 384), False)):
            hp = (torch.bfloat16, torch.float32, torch.float16)[it % 3]
            a_dt, b_dt = ((5, 6), (6, 5), (5, 5), (6, 6))[it % 4]
            a = _gpu_codes((k, m) if kmajor else (m, k), a_dt, 100 * it + m)
            b = _gpu_codes((k, n) if kmajor else (n, k), b_dt, 200 * it + n)
            sa = torch.tensor(2.0 ** -(it % 7), device='cuda')
            sb = torch.tensor(2.0 ** -(it % 5 + 3), device='cuda')
            want_q, want_s, want_si, want_am = _two_steps(be, a, a_dt, sa, b, b_dt, sb, hp, True, kmajor)
            s, si, am = torch.ones((), device='cuda'), torch.ones((), device='cuda'), torch.zeros(1, device='cuda')
            got = be.fp8_gemm_cast(a, a_dt, sa, b, b_dt, sb, hp, 5, s, am, si, nan_to_inf=True, a_kmajor=kmajor, b_kmajor=kmajor)
            assert got is not None, (it, m, n, k, kmajor)
            assert torch.equal(got, want_q), (it, m, n, k, kmajor, hp)
            assert same_float(am, want_am) and same_float(s, want_s) and same_float(si, want_si), (it, m, n, k, kmajor, hp)
            cases += 1
    assert cases == 48


@pytest.mark.parametrize('m,n,k', [(256, 256, 256), (300, 200, 384), (1024, 768, 1024), (2048, 2048, 4096)])
@pytest.mark.parametrize('out_dtype', [torch.float32, torch.bfloat16])
def test_generic_and_direct_to_lds_kernels_agree_to_the_bit(be, m, n, k, out_dtype):
    """K a multiple of 128 goes to the direct-to-LDS kernel; the same operands with 16 zero bytes appended to every row
    (K + 16) go to the generic kernel.  The zeros add nothing, and both kernels add up the 128-byte blocks of K in
    ascending order, so the outputs must be equal bit for bit (which makes results independent of the dispatch)."""
    a, b = _gpu_codes((m, k), 5, 3 * m + k), _gpu_codes((n, k), 6, 7 * n + k)
    sa, sb = torch.tensor(0.5, device='cuda'), torch.tensor(0.25, device='cuda')
    want = be.fp8_gemm(a, 5, sa, b, 6, sb, torch.empty(n, m, dtype=out_dtype, device='cuda'))
    a2, b2 = torch.nn.functional.pad(a, (0, 16)).contiguous(), torch.nn.functional.pad(b, (0, 16)).contiguous()
    got = be.fp8_gemm(a2, 5, sa, b2, 6, sb, torch.empty(n, m, dtype=out_dtype, device='cuda'))
    assert torch.equal(got, want)


@pytest.mark.parametrize('m,n,k', [(4396, 4616, 384), (4352, 4608, 640), (8192, 4352, 256)])
@pytest.mark.parametrize('out_dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('mode', ['plain', 'bias_and_sum'])
def test_several_rounds_of_tiles_agree_with_the_generic_kernel(be, m, n, k, out_dtype, mode):
    """More 256 x 256 tiles than compute units (several rounds of workgroups, whole tiles and tiles on the ragged edges
    mixed), every output type, with and without bias and sum: the direct-to-LDS kernel compared bit for bit with the
    generic kernel (the same operands with 16 zero bytes appended to every row)."""
    a, b = _gpu_codes((m, k), 5, 5 * m + k), _gpu_codes((n, k), 6, 11 * n + k)
    sa, sb = torch.tensor(0.5, device='cuda'), torch.tensor(0.125, device='cuda')
    a2, b2 = torch.nn.functional.pad(a, (0, 16)).contiguous(), torch.nn.functional.pad(b, (0, 16)).contiguous()
    g = torch.Generator(device='cuda').manual_seed(m + n)
    bias = prev = None
    if mode == 'bias_and_sum':
        bias = torch.randn(m, device='cuda', generator=g).to(out_dtype)
        prev = torch.randn(n, m, device='cuda', generator=g).to(out_dtype)
    outs = []
    for x, y in ((a, b), (a2, b2)):
        out = prev.clone() if prev is not None else torch.full((n, m), float('nan'), dtype=out_dtype, device='cuda')
        outs.append(be.fp8_gemm(x, 5, sa, y, 6, sb, out, accumulate=prev is not None, bias=bias))
    assert torch.equal(outs[0].view(torch.int32 if out_dtype == torch.float32 else torch.int16),
                       outs[1].view(torch.int32 if out_dtype == torch.float32 else torch.int16))
    assert not bool(outs[0].isnan().any())


@pytest.mark.parametrize('m,n,k', [(2048, 2048, 4096), (4096, 1024, 4096), (1024, 768, 1024), (2056, 1100, 512), (300, 200, 640),
                                   (128, 128, 512), (1031, 1999, 1152), (1, 1, 512), (33, 65, 1024), (7, 513, 768)])
@pytest.mark.parametrize('out_dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('mode', ['plain', 'bias_and_sum'])
def test_small_and_large_tiles_agree_to_the_bit(be, m, n, k, out_dtype, mode):
    """Problems with few 256 x 256 tiles run 128 x 128 tiles (four stages, fragments read a slice ahead).  The same
    problem through both, the limit set to take the one and then the other: every output equal bit for bit, on whole
    and ragged tiles, rows that 16-byte stores do not fit, all output types, with and without bias and sum."""
    for a_dt, b_dt in ((5, 5), (5, 6), (6, 5)):
        a, b = _gpu_codes((m, k), a_dt, 5 * m + k + a_dt), _gpu_codes((n, k), b_dt, 11 * n + k + b_dt)
        sa, sb = torch.tensor(0.5, device='cuda'), torch.tensor(0.125, device='cuda')
        g = torch.Generator(device='cuda').manual_seed(m + n)
        bias = prev = None
        if mode == 'bias_and_sum':
            bias = torch.randn(m, device='cuda', generator=g).to(out_dtype)
            prev = torch.randn(n, m, device='cuda', generator=g).to(out_dtype)
        outs = []
        try:
            for limit in (1 << 20, 0):
                be.set_small_tile_limit(limit)
                buf = torch.full((n + 2, m), 7.0, dtype=out_dtype, device='cuda')
                out = buf[1:n + 1]
                if prev is not None:
                    out.copy_(prev)
                else:
                    out.fill_(float('nan'))
                be.fp8_gemm(a, a_dt, sa, b, b_dt, sb, out, accumulate=prev is not None, bias=bias)
                assert bool((buf[0] == 7).all()) and bool((buf[n + 1] == 7).all())
                outs.append(out.clone())
        finally:
            be.set_small_tile_limit(128)
        view = torch.int32 if out_dtype == torch.float32 else torch.int16
        assert torch.equal(outs[0].view(view), outs[1].view(view)), (a_dt, b_dt)
        assert not bool(outs[0].isnan().any())


@pytest.mark.parametrize('m,n,k', [(2048, 2048, 1024), (1024, 512, 640), (256, 256, 512), (2048, 1024, 4096), (512, 3072, 1152)])
@pytest.mark.parametrize('out_dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('both', [False, True])
def test_small_tiles_read_kmajor_operands_like_the_large_tile(be, m, n, k, out_dtype, both):
    """The backward GEMMs of a small layer hand their operands over K-major ([K, rows]).  The kernel with 128 x 128
    tiles reads them in place as the large one does (k-rows of 128 bytes in LDS, transposing reads): both kernels on
    the same operands, equal bit for bit, and equal to the row-major call on the transposed copies."""
    for a_dt, b_dt in ((5, 6), (5, 5), (6, 6)):
        a, b = _gpu_codes((m, k), a_dt, 3 * m + k + a_dt), _gpu_codes((n, k), b_dt, 7 * n + k + b_dt)
        sa, sb = torch.tensor(0.25, device='cuda'), torch.tensor(2.0, device='cuda')
        a_t, b_t = a.t().contiguous(), b.t().contiguous()
        outs = []
        try:
            for limit in (1 << 20, 0):
                be.set_small_tile_limit(limit)
                out = torch.full((n, m), float('nan'), dtype=out_dtype, device='cuda')
                be.fp8_gemm(a_t, a_dt, sa, b_t if both else b, b_dt, sb, out, a_kmajor=True, b_kmajor=both)
                outs.append(out)
            be.set_small_tile_limit(1 << 20)
            outs.append(be.fp8_gemm(a, a_dt, sa, b, b_dt, sb, torch.full((n, m), float('nan'), dtype=out_dtype, device='cuda')))
        finally:
            be.set_small_tile_limit(128)
        view = torch.int32 if out_dtype == torch.float32 else torch.int16
        assert torch.equal(outs[0].view(view), outs[1].view(view)), (a_dt, b_dt)
        assert torch.equal(outs[0].view(view), outs[2].view(view)), (a_dt, b_dt)
        assert not bool(outs[0].isnan().any())


def test_random_small_ragged_problems_with_bias_and_accumulation(be):
    """Random shapes up to 700 x 700 with K both a multiple of 128 (direct-to-LDS kernel, whose 256 x 256 tiles are
    mostly padding here) and not (generic kernel), every output type, with and without bias and accumulation."""
    import random
    rng = random.Random(4)
    for it in range(32):
        m, n = rng.randint(1, 700), rng.randint(1, 700)
        k = rng.choice([128, 256, 384, 1024, 16, 48, 144, 1040])
        a_dt, b_dt = rng.choice([(5, 5), (5, 6), (6, 5), (6, 6)])
        a = _rand_fp8((m, k), a_dt, 10 * it + 1)
        b = _rand_fp8((n, k), b_dt, 10 * it + 2, spread=0.5)
        a_si, b_si = 2.0 ** rng.randint(-6, 3), 2.0 ** rng.randint(-6, 3)
        ref = ogemm.fp8_gemm(a, torch.tensor(a_si), FMT[a_dt], b, torch.tensor(b_si), FMT[b_dt])
        od = rng.choice([torch.float32, torch.bfloat16, torch.float16])
        mode = rng.choice(['plain', 'bias', 'acc', 'both'])
        bias = torch.randn(m).to(od) if mode in ('bias', 'both') else None
        base = torch.randn(n, m).to(od) if mode in ('acc', 'both') else None
        if bias is not None:
            ref = ref + bias.float()
        if base is not None:
            ref = ref + base.float()
        got = _run(be, a, a_dt, a_si, b, b_dt, b_si, out_dtype=od, accumulate=base is not None, bias=bias,
                   out=None if base is None else base.clone().cuda())
        assert rel_fro(got.float(), ref) < (TOL_F32 if od == torch.float32 else TOL_16), (it, m, n, k, od, mode)


@pytest.mark.parametrize('nr,nc,k,a_kmajor,b_kmajor', [
    (28672, 8192, 16384, True, True),      # tile columns grouped, the XCD patch turned for X
    (8192, 28672, 16384, True, True),      # tile rows grouped, the patch turned for Y
    (8192, 28672, 16384, True, False),     # the same with only Y K-major
    (9216, 28672, 16384, True, False),     # the same with a last group of four tile rows
    (8192, 12288, 16384, False, False),    # row-major: the patch as it was
    (16384, 4096, 4096, False, False),     # tall, everything cached: rows grouped
    (4096, 16384, 4096, False, False),     # wide: columns grouped
    (28928, 8448, 256, False, False),      # 113 x 33 tiles: a count that 8 does not divide
    (1280, 2304, 256, True, True),         # 5 x 9 tiles, fewer than one round
])
def test_every_tile_is_written_whatever_the_walk(be, nr, nc, k, a_kmajor, b_kmajor):
    """The tile walk (groups of tile rows or columns, XCD-contiguous ids, the patch of an XCD turned or not) is chosen
    from the shape and the operand layouts.  Operands that are constant along K make the whole output predictable,
    D[r, c] = K * x[r] * y[c] with powers of two (exact in bf16), so a tile that the walk skipped, or wrote twice with
    another tile's data, shows."""
    g = torch.Generator(device='cuda').manual_seed(nr + nc)
    # E4M3 codes of 2^-2 .. 2^1: exponent field 5 .. 8, mantissa 0
    ex = torch.randint(5, 9, (nr, ), device='cuda', generator=g, dtype=torch.int32)
    ey = torch.randint(5, 9, (nc, ), device='cuda', generator=g, dtype=torch.int32)
    xs = (ex << 3).to(torch.uint8)
    ys = (ey << 3).to(torch.uint8)
    x = xs.view(1, nr).expand(k, nr).contiguous() if b_kmajor else xs.view(nr, 1).expand(nr, k).contiguous()
    y = ys.view(1, nc).expand(k, nc).contiguous() if a_kmajor else ys.view(nc, 1).expand(nc, k).contiguous()
    out = torch.full((nr, nc), float('nan'), dtype=torch.bfloat16, device='cuda')
    one = torch.ones((), device='cuda')
    want = (float(k) * torch.exp2((ex - 7).float()).view(nr, 1) * torch.exp2((ey - 7).float()).view(1, nc)).to(torch.bfloat16)
    lib = be.load()
    # the walk the rules pick, then each of the four registered by hand (what the timing at first use may choose)
    be.tune_gemm_walks(False)
    try:
        for walk in (-1, 0, 1, 2, 3, 4, 7):    # (4..7: the split waits too; they apply to row-major operands only)
            assert lib.msamp_fp8_gemm_set_walk(nc, nr, k, int(a_kmajor), int(b_kmajor), walk) == 0
            assert lib.msamp_fp8_gemm_get_walk(nc, nr, k, int(a_kmajor), int(b_kmajor)) == walk
            out.fill_(float('nan'))
            be.fp8_gemm(y, 5, one, x, 5, one, out, a_kmajor=a_kmajor, b_kmajor=b_kmajor)
            bad = (out != want) | out.isnan()
            assert not bool(bad.any()), f'walk {walk}: {int(bad.sum())} wrong outputs, first at {bad.nonzero()[0].tolist()}'
    finally:
        lib.msamp_fp8_gemm_set_walk(nc, nr, k, int(a_kmajor), int(b_kmajor), -1)
        be.tune_gemm_walks(True)


@pytest.mark.parametrize('n, m, k', [(1024, 768, 256), (2048, 1280, 384), (1536, 2048, 1152), (4096, 2048, 4096), (2304, 1792, 640),
                                     (8192, 4096, 24576 + 128)])
def test_split_waits_change_no_bit(be, large_tiles_only, n, m, k):
    """With both operands row-major the K loop can await a slice's tile loads in two parts (bit 2 of a registered walk; by
    rule from K = 24576 on): random codes, even and odd slice counts down to two and three, ragged edges, bias and sum
    -- the same bits as the plain form and as the generic kernel."""
    g = torch.Generator(device='cuda').manual_seed(n + m + k)
    a = torch.randint(0, 0x7f, (m, k), device='cuda', dtype=torch.uint8, generator=g)
    b = torch.randint(0, 0x7f, (n - 3, k), device='cuda', dtype=torch.uint8, generator=g)    # a ragged last tile row
    a_si = torch.tensor(0.37, device='cuda')
    b_si = torch.tensor(1.9, device='cuda')
    bias = torch.randn(m, device='cuda', generator=g).bfloat16()
    lib = be.load()
    be.tune_gemm_walks(False)
    outs = {}
    try:
        for walk in (0, 4, 1, 5, 6, 7, -1):
            assert lib.msamp_fp8_gemm_set_walk(m, n - 3, k, 0, 0, walk) == 0
            plain = be.fp8_gemm(a, 5, a_si, b, 6, b_si, torch.full((n - 3, m), float('nan'), dtype=torch.bfloat16, device='cuda'))
            summed = be.fp8_gemm(a, 5, a_si, b, 6, b_si, plain.clone(), accumulate=True, bias=bias)
            outs[walk] = (plain, summed)
    finally:
        lib.msamp_fp8_gemm_set_walk(m, n - 3, k, 0, 0, -1)
        be.tune_gemm_walks(True)
    for walk, (plain, summed) in outs.items():
        assert torch.equal(plain.view(torch.int16), outs[0][0].view(torch.int16)), walk
        assert torch.equal(summed.view(torch.int16), outs[0][1].view(torch.int16)), walk
    if k <= 4096:
        # the generic kernel (K made unfit for the direct-to-LDS kernel by 16 columns of zero codes)
        pad = lambda t: torch.cat([t, torch.zeros(t.shape[0], 16, dtype=torch.uint8, device='cuda')], dim=1)    # noqa: E731
        generic = be.fp8_gemm(pad(a), 5, a_si, pad(b), 6, b_si, torch.empty(n - 3, m, dtype=torch.bfloat16, device='cuda'))
        assert torch.equal(generic.view(torch.int16), outs[0][0].view(torch.int16))


def test_walk_timed_at_first_use_changes_no_bit(be):
    """A problem with two rounds of tiles or more has its tile walks timed the first time it is seen (the call computes
    the product some forty times over); whatever walk comes out, the product is the one of the rules' walk, bit for bit,
    in that call and in the following ones, also through the entry point that casts on to E4M3; a problem met first
    under stream capture, or a small one, is left to the rules."""
    torch.manual_seed(21)
    n, m, k = 8192, 4096, 1024    # 32 x 16 = 512 tiles
    a = torch.randint(0, 0x78, (m, k), device='cuda', dtype=torch.uint8)
    b = torch.randint(0, 0x78, (n, k), device='cuda', dtype=torch.uint8)
    one = torch.ones((), device='cuda')
    be.forget_gemm_walks()
    be.tune_gemm_walks(False)
    want = be.fp8_gemm(a, 5, one, b, 5, one, torch.empty(n, m, dtype=torch.bfloat16, device='cuda'))
    assert be.load().msamp_fp8_gemm_get_walk(m, n, k, 0, 0) == -1
    be.tune_gemm_walks(True)
    try:
        first = be.fp8_gemm(a, 5, one, b, 5, one, torch.full((n, m), float('nan'), dtype=torch.bfloat16, device='cuda'))
        assert (m, n, k, False, False) in be._walk_seen
        assert be.load().msamp_fp8_gemm_get_walk(m, n, k, 0, 0) in range(-1, 8)
        second = be.fp8_gemm(a, 5, one, b, 5, one, torch.full((n, m), float('nan'), dtype=torch.bfloat16, device='cuda'))
        assert torch.equal(first, want) and torch.equal(second, want)
        # adding into an output never times (the timed launches would add forty times)
        acc = want.clone()
        be.forget_gemm_walks()
        be.fp8_gemm(a, 5, one, b, 5, one, acc, accumulate=True)
        assert not be._walk_seen
        assert torch.equal(acc, (want.float() * 2).to(torch.bfloat16))
        # the weight-gradient form: timed on a scratch product, then the fused call
        at, bt = a.t().contiguous(), b.t().contiguous()
        metas = [(torch.ones((), device='cuda'), torch.zeros(1, device='cuda'), torch.ones((), device='cuda')) for _ in range(2)]
        be.tune_gemm_walks(False)
        q0 = be.fp8_gemm_cast(at, 5, one, bt, 5, one, torch.bfloat16, 5, *metas[0], a_kmajor=True, b_kmajor=True)
        be.tune_gemm_walks(True)
        q1 = be.fp8_gemm_cast(at, 5, one, bt, 5, one, torch.bfloat16, 5, *metas[1], a_kmajor=True, b_kmajor=True)
        assert (m, n, k, True, True) in be._walk_seen
        assert q0 is not None and torch.equal(q0, q1) and all(torch.equal(u, v) for u, v in zip(metas[0], metas[1]))
        # under capture nothing is timed and the problem stays unseen
        be.forget_gemm_walks()
        out = torch.empty(n, m, dtype=torch.bfloat16, device='cuda')
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            be.tune_gemm_walks(False)
            be.fp8_gemm(a, 5, one, b, 5, one, out)    # (allocator and library warm-up on the side stream)
            be.tune_gemm_walks(True)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            be.fp8_gemm(a, 5, one, b, 5, one, out)
        assert not be._walk_seen
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
    finally:
        be.forget_gemm_walks()
        be.tune_gemm_walks(True)
