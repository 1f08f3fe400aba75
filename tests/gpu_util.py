"""Helpers shared by the GPU parity tests."""

import torch

from oracle import cast as ocast, fp8

FMT = {5: fp8.E4M3, 6: fp8.E5M2}


def make_meta(dev='cuda', window=1, scale=1.0):
    """Device-side triple (scale, scale_inv, amax) as the C ABI wants them."""
    return (torch.full((), scale, device=dev), torch.ones((), device=dev), torch.zeros(window, device=dev))


def oracle_meta(window=1, scale=1.0):
    m = ocast.new_meta(window)
    m['scale'] = torch.tensor(scale)
    return m


def c1_input(seed=0, n_rows=4096, n_cols=4096):
    """fp32 N(0,1) with 0.1% of the entries (uniformly chosen) multiplied by 100."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n_rows, n_cols, generator=g)
    n = x.numel()
    idx = torch.randperm(n, generator=g)[:n // 1000]
    x.view(-1)[idx] *= 100
    return x


def same_float(a, b):
    """Bit equality of two float32 scalars/tensors, NaN equal to NaN."""
    a, b = a.detach().cpu().float(), b.detach().cpu().float()
    return torch.equal(torch.nan_to_num(a, nan=12345.0), torch.nan_to_num(b, nan=12345.0)) and \
        torch.equal(torch.isnan(a), torch.isnan(b))


def rel_fro(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).norm() / want.norm().clamp_min(1e-30)).item()
