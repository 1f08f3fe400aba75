"""Power-of-two scaling rule and the delayed-scaling amax window.  Test infrastructure only."""

import numpy as np
import torch


def _log2_f32(x):
    """Correctly rounded float32 log2 (float64 log2 narrowed once).  The reference evaluates
    torch.log2 in float32 on its device; libraries differ from one another by an ulp on a few
    inputs (torch's own CPU vector path does on large tensors), which can move the floor only for
    fp_max/amax within a few ulps below a power of two.  The correctly rounded value is the
    library-independent reading, and is what the HIP kernel computes.  parity unpinned for those
    boundary inputs: only a run of the reference on its own device could pin them."""
    shape = x.shape
    a = x.detach().to(torch.float32).reshape(-1).numpy().astype(np.float64)
    with np.errstate(divide='ignore', invalid='ignore'):
        r = np.log2(a).astype(np.float32)
    return torch.from_numpy(r).reshape(shape)


def compute_scaling_factor(amax, scale, fp_max, margin=0):
    """New scale from amax; follows msamp/common/tensor/meta.py:51-56 in float32.

    exp = floor(log2(fp_max/amax)) - margin; sf = round(2**|exp|); keep ``scale`` where
    amax is not > 0 or not finite; invert where exp < 0.  `fp_max / amax` with a Python float on
    the left is evaluated by torch (eagerly and under TorchScript) as reciprocal(amax) * fp_max.
    """
    amax = amax.to(torch.float32)
    scale = scale.to(torch.float32)
    exp = torch.floor(_log2_f32(fp_max / amax)) - margin
    sf = torch.round(torch.pow(2, torch.abs(exp)))
    sf = torch.where(amax > 0.0, sf, scale)
    sf = torch.where(torch.isfinite(amax), sf, scale)
    sf = torch.where(exp < 0, 1 / sf, sf)
    return sf


def update_scaling_factors(scales, amaxs, counters, fp_max, margin=0):
    """One optimizer-step update of flattened metas; follows msamp/optim/optimizer.py:91-108.

    scales (n,), amaxs (n, window), counters (n,) are modified in place.
    """
    bad = ~torch.isfinite(amaxs[:, 0])
    amaxs[bad, 0] = 0
    sf = compute_scaling_factor(amaxs.max(1).values, scales, fp_max, margin)
    amaxs.copy_(amaxs.roll(1, dims=1))
    amaxs[:, 0] = 0
    counters += 1
    counters[bad] = 0
    scales.copy_(sf)
    return bad
