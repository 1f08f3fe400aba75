"""TypeCast: torch.Tensor <-> quantized payloads (msamp/common/tensor/cast.py:14-136)."""

import torch
import torch.distributed as dist

from msamp import _backend
from msamp.common.dtype import Dtypes, Floating


def _world_size():
    return dist.get_world_size() if dist.is_available() and dist.is_initialized() else 1


class TypeCast:
    """Static cast helpers; every arithmetic step runs in the HIP library."""
    @staticmethod
    def _sync_amax(meta):
        """sync=True: NaN/+Inf amax -> +Inf, all-reduce(MAX) over the meta's group (cast.py:37-44)."""
        meta.amax[0:1].nan_to_num_(nan=torch.inf, posinf=torch.inf)
        if _world_size() > 1:
            dist.all_reduce(meta.amax[0], op=dist.ReduceOp.MAX, group=meta.group)
            return meta.amax[0].clone()
        return None

    @staticmethod
    def cast_to_fp8(input, meta, sync=False, fuse_transpose=False):
        """Quantize to FP8 (uint8 payload) with meta.qtype, updating meta.

        In-time scaling (window 1 or warm-up): amax[0] = max|x|, scale from it, then quantize --
        one fused library call.  Otherwise quantize with the stored scale and fold max|x| into
        amax[0].  scale_inv = 1/scale either way.  With fuse_transpose the transposed payload of
        the 2-D input is produced in the same pass and a pair is returned.
        """
        if not (input.is_cuda and input.is_contiguous()):
            raise ValueError('The input tensor is not in cuda memory or contiguous.')
        if not meta.scale.is_cuda:
            raise ValueError('The meta.scale is not in cuda memory.')
        if input.dtype in (torch.uint8, torch.int8):
            raise ValueError('The input tensor is already quantized.')
        fp8_dt = int(meta.qtype)
        amax0 = meta.amax[0:1]
        mode = meta.scaling_mode()
        if mode == 'gated':
            if not sync:
                if fuse_transpose:
                    if input.dim() != 2:
                        raise ValueError('fuse_transpose needs a 2-D input.')
                    return _backend.cast_transpose_gated(
                        input, meta.scale, amax0, meta.scale_inv, fp8_dt, meta.amax_counter, meta.window_size
                    )
                return _backend.cast_to_fp8_gated(
                    input, meta.scale, amax0, meta.scale_inv, fp8_dt, meta.amax_counter, meta.window_size
                )
            mode = 'in_time' if bool(meta.is_warmup()) else 'delayed'    # sync=True: decide on the host
        in_time = mode == 'in_time'
        fused_in_time = in_time and not (sync and _world_size() > 1)
        sync_amax = None
        if not fused_in_time:
            if in_time:
                _backend.amax(input, amax0)
            if sync:
                sync_amax = TypeCast._sync_amax(meta)
            if in_time or sync:
                meta.reset_scaling_factor()
        if fuse_transpose:
            if input.dim() != 2:
                raise ValueError('fuse_transpose needs a 2-D input.')
            if fused_in_time:
                out = _backend.cast_transpose(input, meta.scale, amax0, meta.scale_inv, fp8_dt, in_time=True, nan_to_inf=sync)
            else:
                out = _backend.cast_transpose(input, meta.scale, amax0, meta.scale_inv, fp8_dt)
        elif fused_in_time:
            out = _backend.cast_to_fp8_intime(input, meta.scale, amax0, meta.scale_inv, fp8_dt, nan_to_inf=sync)
        else:
            out = _backend.cast_to_fp8(input, meta.scale, amax0, meta.scale_inv, fp8_dt)
        if sync_amax is not None:
            meta.amax[0].copy_(sync_amax)
        return out

    @staticmethod
    def cast_to_fp16(input, meta, sync=False):
        """Scaled 16-bit (or 32-bit) payload: (input * scale).to(dtype of meta.qtype)."""
        in_time = meta.is_in_time_scaling()
        if in_time or sync:
            _backend.amax(input.contiguous(), meta.amax[0:1])
        if sync:
            TypeCast._sync_amax(meta)
        if in_time or sync:
            meta.reset_scaling_factor()
        meta.scale_inv.copy_(torch.reciprocal(meta.scale))
        return _backend.scale_cast(input.contiguous(), meta.scale, Dtypes.get_dtype_from_qtype(meta.qtype))

    @staticmethod
    def cast_from_fp8(input, meta, otype):
        """Dequantize an FP8 payload: otype(float(q) * scale_inv)."""
        if not (input.is_cuda and input.is_contiguous()):
            raise ValueError('The input tensor is not in cuda memory or contiguous.')
        if input.dtype != torch.uint8:
            raise ValueError('The dtype of input tensor is not torch.uint8.')
        return _backend.cast_from_fp8(input, meta.scale_inv, int(meta.qtype), Dtypes.get_dtype_from_qtype(otype))

    @staticmethod
    def cast_from_fp16(input, meta, otype):
        """Unscale a 16/32-bit payload: (input * scale_inv).to(otype)."""
        return _backend.scale_cast(input.contiguous(), meta.scale_inv, Dtypes.get_dtype_from_qtype(otype))

    cast_from_fp32 = cast_from_fp16


__all__ = ['TypeCast', 'Floating']
