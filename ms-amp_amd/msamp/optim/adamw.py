"""LBAdamW: the FP8 AdamW step on HIP kernels (msamp/optim/adamw.py:19-235).

Quantized-state parameters whose weight, gradient and both moments are ScalingTensors of the
supported formats take one fused multi-tensor call (three launches for the whole group); everything
else follows the reference's two-stage recipe tensor by tensor.
"""

import math

import numpy as np
import torch

from msamp import _backend
from msamp.common.dtype import Dtypes, Floating
from msamp.common.tensor import ScalingMeta, ScalingTensor
from msamp.optim.adamw_base import LBAdamWBase

_FUSED_WEIGHT_QTYPES = (Dtypes.kfloat8_e4m3, Dtypes.kfloat8_e5m2, Dtypes.kfloat16)


class LBAdamW(LBAdamWBase):
    """AdamW with low-bit moments (default: E4M3 exp_avg, scaled-fp16 exp_avg_sq)."""
    def __init__(self, params, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2,
                 amsgrad=False, *, maximize=False, exp_avg_dtype=torch.uint8, exp_avg_sq_dtype=torch.float16,
                 tensor_scale=True, double_buffer=True):
        """double_buffer (not in the reference): the fused step writes the new weight and moment payloads into a second
        set of buffers (4 more bytes per parameter) and swaps the two sets afterwards, which lets it read every tensor
        once instead of twice; the values are the same bit for bit.  The payload tensors (`.value`) remain the same
        objects, but their memory alternates between two addresses: pass False when something holds those addresses
        (a captured graph of the forward pass, views taken of `.value`).  Payloads that are themselves views of other
        storage (a flat buffer) and steps taken under stream capture keep the in-place step."""
        self.tensor_scale = tensor_scale
        self.double_buffer = double_buffer
        self._fused_cache = {}
        self._spare = {}    # id(parameter) -> [weight, exp_avg, exp_avg_sq] payload buffers not in use right now
        super().__init__(
            params, lr=lr, bias_correction=bias_correction, betas=betas, eps=eps, weight_decay=weight_decay,
            amsgrad=False, maximize=maximize, exp_avg_dtype=exp_avg_dtype, exp_avg_sq_dtype=exp_avg_sq_dtype
        )

    # ---- fused multi-tensor path ------------------------------------------------------------
    @staticmethod
    def _fusable(p, g, m, v):
        if not all(isinstance(t, ScalingTensor) for t in (p, g, m, v)):
            return False
        if p.qtype not in _FUSED_WEIGHT_QTYPES or not Dtypes.is_fp8_qtype(g.qtype):
            return False
        if m.qtype != Dtypes.kfloat8_e4m3 or v.qtype != Dtypes.kfloat16:
            return False
        # The fused kernel always derives the weight's new scale from the amax of the updated weight.  The per-tensor
        # recipe re-quantizes through param.cast(), which does that only under in-time scaling (reference
        # msamp/optim/adamw.py:172-174 with msamp/common/tensor/cast.py:31-44); a weight meta in any other mode takes
        # the per-tensor path.
        if p.meta.scaling_mode() != 'in_time':
            return False
        tensors = (p.value, g.value, m.value, v.value)
        if not all(t.is_cuda and t.is_contiguous() and t.numel() == p.value.numel() for t in tensors):
            return False
        return all(t.data_ptr() % 16 == 0 for t in tensors)

    def _fused_tables(self, key, params, grads, exp_avgs, exp_avg_sqs):
        """Device descriptor table + block map for a list of tensors, cached while no pointer changes."""
        rows = []
        for p, g, m, v in zip(params, grads, exp_avgs, exp_avg_sqs):
            rows.append((
                p.value.data_ptr(), g.value.data_ptr(), m.value.data_ptr(), v.value.data_ptr(),
                p.meta.scale.data_ptr(), p.meta.scale_inv.data_ptr(), p.meta.amax.data_ptr(),
                g.meta.scale_inv.data_ptr(),
                m.meta.scale.data_ptr(), m.meta.scale_inv.data_ptr(), m.meta.amax.data_ptr(),
                v.meta.scale.data_ptr(), v.meta.scale_inv.data_ptr(), v.meta.amax.data_ptr(),
                p.value.numel(), 0, 0, 0, 0,
            ))
        sig = tuple(rows)
        cached = self._fused_cache.get(key)
        if cached is not None and cached[0] == sig:
            return cached[1], cached[2], cached[3], cached[4]
        device = params[0].value.device
        desc = torch.from_numpy(np.asarray(rows, dtype=np.int64).reshape(len(rows), _backend.ADAMW_DESC_WORDS)).to(device)
        chunks = [(p.value.numel() + _backend.ADAMW_CHUNK - 1) // _backend.ADAMW_CHUNK for p in params]
        tensor_idx = np.repeat(np.arange(len(params), dtype=np.int32), chunks)
        chunk_idx = np.concatenate([np.arange(c, dtype=np.int32) for c in chunks]) if chunks else np.zeros(0, np.int32)
        block_map = torch.from_numpy(np.stack([tensor_idx, chunk_idx], axis=1).copy()).to(device)
        self._fused_cache[key] = (sig, desc, block_map, int(block_map.shape[0]), chunks)
        return desc, block_map, int(block_map.shape[0]), chunks

    def _fused_step(self, idx, params, grads, exp_avgs, exp_avg_sqs, step, *, beta1, beta2, lr, weight_decay, eps,
                    maximize):
        ps, gs = [params[i] for i in idx], [grads[i] for i in idx]
        ms, vs = [exp_avgs[i] for i in idx], [exp_avg_sqs[i] for i in idx]
        wq, gq = ps[0].qtype, gs[0].qtype
        if self.double_buffer and self._can_swap(ps, ms, vs):
            # the payload pointers alternate between two sets from step to step: one cached table per set
            key = (int(wq), int(gq), id(ps[0]), ps[0].value.data_ptr())
            desc, block_map, n_blocks, _ = self._fused_tables(key, ps, gs, ms, vs)
            spares = [self._spare_buffers(p, m, v) for p, m, v in zip(ps, ms, vs)]
            outputs, redo = self._output_tables(key, spares)
            _backend.adamw_fused_speculative(
                desc, outputs, redo, len(ps), block_map, n_blocks, int(wq), int(gq), lr, beta1, beta2, eps, weight_decay, step,
                self.bias_correction, self.use_adam, maximize, self.tensor_scale
            )
            # the payload tensors stay the objects they were and trade their memory with the spares
            for p, m, v, spare in zip(ps, ms, vs, spares):
                for i, t in enumerate((p.value, m.value, v.value)):
                    old = t.data
                    t.data = spare[i]
                    spare[i] = old
            return
        key = (int(wq), int(gq), id(ps[0]))
        desc, block_map, n_blocks, chunks = self._fused_tables(key, ps, gs, ms, vs)
        _backend.adamw_fused(
            desc, len(ps), block_map, n_blocks, int(wq), int(gq), lr, beta1, beta2, eps, weight_decay, step,
            self.bias_correction, self.use_adam, maximize, self.tensor_scale, blocks_per_tensor=chunks
        )

    @staticmethod
    def _can_swap(ps, ms, vs):
        """Swapping payload tensors is safe when nothing else aliases them and no graph is recording their addresses."""
        if torch.cuda.is_current_stream_capturing():
            return False
        return all(t.value._base is None for group in (ps, ms, vs) for t in group)

    def _spare_buffers(self, p, m, v):
        spare = self._spare.get(id(p))
        current = (p.value, m.value, v.value)
        if spare is None or any(s.shape != c.shape or s.dtype != c.dtype or s.device != c.device for s, c in zip(spare, current)):
            spare = [torch.empty_like(c) for c in current]
            self._spare[id(p)] = spare
        return spare

    def _output_tables(self, key, spares):
        rows = tuple((s[0].data_ptr(), s[1].data_ptr(), s[2].data_ptr(), 0) for s in spares)
        cached = self._fused_cache.get(('out', ) + key)
        if cached is not None and cached[0] == rows:
            return cached[1], cached[2]
        device = spares[0][0].device
        outputs = torch.from_numpy(np.asarray(rows, dtype=np.int64).reshape(len(rows), _backend.ADAMW_BUFFER_WORDS)).to(device)
        redo = torch.zeros(len(rows), dtype=torch.int32, device=device)
        self._fused_cache[('out', ) + key] = (rows, outputs, redo)
        return outputs, redo

    # ---- per-tensor path (reference recipe) -----------------------------------------------
    def _staged_step(self, idx, params, grads, exp_avgs, exp_avg_sqs, state_steps, *, beta1, beta2, lr, weight_decay,
                     eps, maximize):
        if not idx:
            return
        inv_m = [(1.0 / exp_avgs[i].meta.scale).item() for i in idx]
        inv_v = [(1.0 / exp_avg_sqs[i].meta.scale).item() for i in idx]
        for i in idx:
            exp_avgs[i].meta.amax.zero_()
            exp_avg_sqs[i].meta.amax.zero_()
        for j, i in enumerate(idx):
            param = params[i].float()
            grad = grads[i].float() if not maximize else -grads[i].float()
            if weight_decay != 0:
                if self.use_adam:
                    grad = grad.add(param, alpha=weight_decay)
                else:
                    param.mul_(1 - lr * weight_decay)
            param, grad = param.contiguous(), grad.contiguous()
            m, v = exp_avgs[i], exp_avg_sqs[i]
            _backend.adamw_stage1(
                param, grad, m.value, _backend.state_dt(m.value, int(m.qtype)), inv_m[j], m.meta.amax, beta1, v.value,
                _backend.state_dt(v.value, int(v.qtype)), inv_v[j], v.meta.amax, beta2, eps, state_steps[i], lr,
                self.bias_correction
            )
            if isinstance(params[i], ScalingTensor):
                params[i].copy_(param.cast(params[i].qtype, meta=params[i].meta))
            elif param.data_ptr() != params[i].data_ptr():
                params[i].copy_(param)
        if self.tensor_scale:
            amaxs = torch.cat([exp_avgs[i].meta.amax[0:1] for i in idx])
            sq_amaxs = torch.cat([exp_avg_sqs[i].meta.amax[0:1] for i in idx])
            ones = amaxs.new_ones((1, ))
            new_m = ScalingMeta.compute_scaling_factor(amaxs, ones, Floating.fp_maxs[exp_avgs[idx[0]].dtype], 0).tolist()
            new_v = ScalingMeta.compute_scaling_factor(sq_amaxs, ones, Floating.fp_maxs[exp_avg_sqs[idx[0]].dtype], 0).tolist()
        else:
            new_m = new_v = [1.0] * len(idx)
        for j, i in enumerate(idx):
            # as in the reference, stage 2 sees the gradient without the Adam-mode L2 term
            grad = grads[i].float() if not maximize else -grads[i].float()
            m, v = exp_avgs[i], exp_avg_sqs[i]
            m.meta.scale.fill_(new_m[j])
            m.meta.scale_inv.fill_(1.0 / new_m[j])
            v.meta.scale.fill_(new_v[j])
            v.meta.scale_inv.fill_(1.0 / new_v[j])
            _backend.adamw_stage2(
                grad.contiguous(), m.value, _backend.state_dt(m.value, int(m.qtype)), inv_m[j], new_m[j], beta1, v.value,
                _backend.state_dt(v.value, int(v.qtype)), inv_v[j], new_v[j], beta2
            )

    def adamw_fn(self, params, grads, exp_avgs, exp_avg_sqs, max_exp_avg_sqs, state_steps, *, amsgrad, beta1, beta2, lr,
                 weight_decay, eps, maximize):
        if amsgrad:
            raise ValueError('Only amsgrad=False is supported for now.')
        if len(exp_avgs) > 0 and exp_avgs[0].dtype != torch.float32:
            fused = {}
            staged = []
            for i in range(len(params)):
                if self._fusable(params[i], grads[i], exp_avgs[i], exp_avg_sqs[i]):
                    fused.setdefault((int(params[i].qtype), int(grads[i].qtype), state_steps[i]), []).append(i)
                else:
                    staged.append(i)
            hyper = dict(beta1=beta1, beta2=beta2, lr=lr, weight_decay=weight_decay, eps=eps, maximize=maximize)
            for (_, _, step), idx in fused.items():
                self._fused_step(idx, params, grads, exp_avgs, exp_avg_sqs, step, **hyper)
            self._staged_step(staged, params, grads, exp_avgs, exp_avg_sqs, state_steps, **hyper)
            return
        # float32 moments: whole-tensor float32 update, then requantize the parameter if it is low-bit
        for i, p in enumerate(params):
            param = p.float()
            grad = grads[i].float() if not maximize else -grads[i].float()
            exp_avg, exp_avg_sq = exp_avgs[i], exp_avg_sqs[i]
            if weight_decay != 0:
                if self.use_adam:
                    grad = grad.add(param, alpha=weight_decay)
                else:
                    param.mul_(1 - lr * weight_decay)
            bc1 = 1 - beta1**state_steps[i] if self.bias_correction else 1.0
            bc2 = 1 - beta2**state_steps[i] if self.bias_correction else 1.0
            exp_avg.mul_(beta1).add_(grad, alpha=1 - beta1)
            exp_avg_sq.mul_(beta2).add_(torch.square(grad), alpha=1 - beta2)
            denom = (exp_avg_sq.sqrt() / math.sqrt(bc2)).add_(eps)
            param.add_(exp_avg / denom, alpha=-(lr / bc1))
            if isinstance(p, ScalingTensor):
                p.copy_(param.cast(p.qtype, meta=p.meta))
            elif param.data_ptr() != p.data_ptr():
                p.copy_(param)
