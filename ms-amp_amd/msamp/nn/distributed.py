"""The compute side of the FP8 gradient reducer (msamp/nn/distributed.py:124-193).

The reference's reducer, once every gradient of a bucket has arrived, (2) takes each gradient's amax and
MAX-reduces them over the ranks, (3) derives pow-2 scales times 1/sqrt(world size), (4) quantizes the
gradients to E4M3 into one flat buffer and (5) SUM-reduces that buffer.  This module does (2) to (4) for a
whole bucket in four launches; the collectives are left to the caller (this build runs on one GPU).
"""

import math

import torch

from msamp import _backend
from msamp.common.dtype import Dtypes
from msamp.common.tensor import ScalingMeta, ScalingTensor


class GradientBucket:
    """A flat FP8 buffer for a fixed list of gradient sizes, and the tables to fill it.

    `quantize(grads, world_size)` returns one ScalingTensor per gradient, each a view of the buffer with
    its own meta, already divided by the world size the way the reducer leaves it (distributed.py:192),
    so that a SUM all-reduce of `flat` (times the dequantization) yields the average.
    """
    def __init__(self, numels, device='cuda', qtype=Dtypes.kfloat8_e4m3, speculate=True):
        if not Dtypes.is_fp8_qtype(qtype):
            raise TypeError('the bucket holds FP8 gradients')
        self.speculate = speculate    # write the codes during the amax pass, with the scales of the round before
        self.numels = [int(n) for n in numels]
        self.qtype = qtype
        self.flat = torch.zeros(sum(self.numels), dtype=torch.uint8, device=device)
        self.metas = [ScalingMeta(qtype) for _ in self.numels]
        self._views, offset = [], 0
        for n in self.numels:
            self._views.append(self.flat.narrow(0, offset, n))
            offset += n
        self._tables = None
        self._wrapped = None

    def _get_tables(self, grads):
        sig = tuple(g.data_ptr() for g in grads)
        if self._tables is None or self._tables[0] != sig:
            items, block_map = _backend.bucket_tables(
                grads, self._views, [m.amax for m in self.metas], [m.scale for m in self.metas],
                [m.scale_inv for m in self.metas]
            )
            self._tables = (sig, items, block_map)
        return self._tables[1], self._tables[2]

    @torch.no_grad()
    def quantize(self, grads, world_size=1, reduce_amax=None):
        """grads: contiguous CUDA tensors of one dtype (fp32 / fp16 / bf16) with the bucket's sizes.
        reduce_amax(list of 1-element amax tensors): the MAX all-reduce over the ranks, if there are any."""
        if len(grads) != len(self.numels) or any(g.numel() != n for g, n in zip(grads, self.numels)):
            raise ValueError('gradients do not match the sizes of the bucket')
        if not grads:
            return []
        dtype = grads[0].dtype
        if any(g.dtype != dtype or not g.is_cuda or not g.is_contiguous() for g in grads):
            raise ValueError('gradients must be contiguous CUDA tensors of one dtype')
        items, block_map = self._get_tables(grads)
        in_dt = _backend._dt(grads[0])
        # The amax pass already writes the codes, with the scales of the round before; the second call then only redoes
        # the gradients whose scale came out different (same bytes either way).
        _backend.bucket_amax(items, block_map, in_dt, nan_to_inf=True,
                             speculate_fp8_dt=int(self.qtype) if self.speculate else None)
        if reduce_amax is not None:
            reduce_amax([m.amax[0:1] for m in self.metas])
        # the division of each finished tensor by the world size (a division of its scale_inv) rides along
        _backend.bucket_cast(items, block_map, in_dt, int(self.qtype), 1.0 / math.sqrt(world_size), float(world_size))
        # the wrappers of the flat buffer's parts are the same from call to call while the shapes are
        shapes = tuple(g.shape for g in grads)
        if self._wrapped is None or self._wrapped[0] != shapes:
            self._wrapped = (shapes, [ScalingTensor(view.view(g.shape), meta) for g, view, meta in zip(grads, self._views, self.metas)])
        return list(self._wrapped[1])
