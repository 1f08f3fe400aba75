"""LBAdamW: the FP8 AdamW step on HIP kernels (msamp/optim/adamw.py:19-235).

Quantized-state parameters whose weight, gradient and both moments are ScalingTensors of the
supported formats take one fused multi-tensor call (three launches for the whole group); small parameters
kept in high precision (biases, norm weights) with quantized moments take one launch for all of them;
everything else follows the reference's two-stage recipe tensor by tensor.
"""

import math

import numpy as np
import torch

from msamp import _backend
from msamp.common.dtype import Dtypes, Floating
from msamp.common.tensor import ScalingMeta, ScalingTensor
from msamp.optim.adamw_base import LBAdamWBase

_FUSED_WEIGHT_QTYPES = (Dtypes.kfloat8_e4m3, Dtypes.kfloat8_e5m2, Dtypes.kfloat16)


class _FusedPlan:
    """What one group of fusable parameters needs from step to step: the device tables of the fused kernels and, for
    the one-pass forms, where the payloads live."""
    def __init__(self):
        self.params = ()           # ids of the parameters, in order
        self.static_sig = None     # addresses that only a rebuild changes (metas of weight and moments)
        self.sig = None            # addresses that may change between steps (payloads, gradient, its scale_inv)
        self.desc = None           # [n, ADAMW_DESC_WORDS] int64 on the device (one per phase for the moving forms)
        self.block_map = None
        self.n_blocks = 0
        self.chunks = None
        self.stage = None          # pinned staging rows for the columns that change
        # shifting arenas
        self.arenas = None         # {'w','m','v'}: uint8 tensors
        self.views = None          # [phase][tensor] -> (w, m, v) views
        self.phase = 0             # 0: payloads at the top (the room below), 1: at the bottom
        self.slack = 0
        self.widths = (1, 1, 2)    # bytes per element of the weight, exp_avg and exp_avg_sq payloads
        self.redo = None
        self.sync = None
        # two sets of buffers
        self.spare = None
        self.outputs = None


class LBAdamW(LBAdamWBase):
    """AdamW with low-bit moments (default: E4M3 exp_avg, scaled-fp16 exp_avg_sq)."""
    def __init__(self, params, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2,
                 amsgrad=False, *, maximize=False, exp_avg_dtype=torch.uint8, exp_avg_sq_dtype=torch.float16,
                 tensor_scale=True, one_pass=None, double_buffer=False):
        """one_pass (not in the reference) selects how the fused step gets at its data; the values are the same bit for
        bit in every form:

        None (default): in place, as the reference's optimizer works: every payload keeps its address; the step reads
            every tensor twice (the scales of the new values are only known after a full pass), 14 bytes of memory
            traffic per parameter.
        'shift': the optimizer moves the payloads of weights and moments into three arenas of its own, with a little
            room at one end (a few thousand 16 Ki-element chunks: about 0.3 bytes per parameter for a billion
            parameters), and every step writes the new payloads that much further along, alternately down and up.
            The step then reads every tensor once (9 bytes per parameter).  The payload tensors (`.value`) remain the
            same objects, but their memory alternates between two addresses from step to step.
        'double': the step writes into a second set of payload buffers (4 more bytes per parameter) and the two sets
            trade places; one pass as well, and the addresses alternate as well.

        Pass None when something holds the payload addresses across steps (a captured graph of the forward pass, views
        taken of `.value`).  Steps taken under stream capture, and payloads that are views of somebody else's storage,
        keep the in-place step whatever is asked for.  `double_buffer=True` is the older spelling of one_pass='double'."""
        if double_buffer and one_pass is None:
            one_pass = 'double'
        if one_pass not in (None, 'shift', 'double'):
            raise ValueError("one_pass must be None, 'shift' or 'double'")
        self.tensor_scale = tensor_scale
        self.one_pass = one_pass
        self._plans = {}
        self._groups = None
        super().__init__(
            params, lr=lr, bias_correction=bias_correction, betas=betas, eps=eps, weight_decay=weight_decay,
            amsgrad=False, maximize=maximize, exp_avg_dtype=exp_avg_dtype, exp_avg_sq_dtype=exp_avg_sq_dtype
        )

    @property
    def double_buffer(self):
        return self.one_pass == 'double'

    def extra_bytes(self):
        """Device memory the one-pass forms hold beyond the payloads themselves (the room in the arenas, the second
        set of buffers)."""
        total = 0
        for plan in self._plans.values():
            if plan.arenas is not None:
                total += sum(plan.slack * _backend.ADAMW_CHUNK * width for width in plan.widths)
            if plan.spare is not None:
                total += sum(t.numel() * t.element_size() for trio in plan.spare for t in trio)
        return total

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

    # columns of a descriptor row that may change between steps: weight, grad, exp_avg, exp_avg_sq payloads and the
    # gradient's scale_inv
    _MOVING = (0, 1, 2, 3, 7)

    @staticmethod
    def _moving_sig(ps, gs, ms, vs):
        return ([p.value.data_ptr() for p in ps], [g.value.data_ptr() for g in gs], [m.value.data_ptr() for m in ms],
                [v.value.data_ptr() for v in vs], [g.meta.scale_inv.data_ptr() for g in gs])

    @staticmethod
    def _static_rows(ps, ms, vs):
        return [(p.meta.scale.data_ptr(), p.meta.scale_inv.data_ptr(), p.meta.amax.data_ptr(), 0,
                 m.meta.scale.data_ptr(), m.meta.scale_inv.data_ptr(), m.meta.amax.data_ptr(),
                 v.meta.scale.data_ptr(), v.meta.scale_inv.data_ptr(), v.meta.amax.data_ptr(), p.value.numel(), 0, 0, 0, 0)
                for p, m, v in zip(ps, ms, vs)]

    def _plan_for(self, key, ps, ms, vs):
        """The cached plan of this group if it still describes these parameters, else a fresh one (tables not built)."""
        ids = tuple(id(p) for p in ps)
        plan = self._plans.get(key)
        if plan is not None and plan.params == ids:
            return plan
        plan = _FusedPlan()
        plan.params = ids
        plan.chunks = [(p.value.numel() + _backend.ADAMW_CHUNK - 1) // _backend.ADAMW_CHUNK for p in ps]
        device = ps[0].value.device
        tensor_idx = np.repeat(np.arange(len(ps), dtype=np.int32), plan.chunks)
        chunk_idx = np.concatenate([np.arange(c, dtype=np.int32) for c in plan.chunks]) if plan.chunks else np.zeros(0, np.int32)
        plan.block_map = torch.from_numpy(np.stack([tensor_idx, chunk_idx], axis=1).copy()).to(device)
        plan.n_blocks = int(plan.block_map.shape[0])
        self._plans[key] = plan
        return plan

    def _table(self, plan, slot, ps, gs, ms, vs, sig=None):
        """Device descriptor table `slot` of the plan, brought up to date: built in full the first time (and again when
        a meta tensor has been replaced), afterwards only the columns whose addresses changed since the last step
        are sent again."""
        sig = sig or self._moving_sig(ps, gs, ms, vs)
        metas = [id(t) for p, m, v in zip(ps, ms, vs) for t in (p.meta.scale, m.meta.scale, v.meta.scale)]
        if plan.desc is None or plan.static_sig != metas:
            plan.desc, plan.sig, plan.stage, plan.static_sig = {}, {}, {}, metas
        desc = plan.desc.get(slot)
        capturing = torch.cuda.is_current_stream_capturing()
        if desc is None:
            if capturing:
                raise RuntimeError('LBAdamW: the first fused step of a parameter group builds device tables and cannot be '
                                   'captured; take a step outside the capture first (two with one_pass set).')
            rows = np.zeros((len(ps), _backend.ADAMW_DESC_WORDS), dtype=np.int64)
            rows[:, 4:19] = np.asarray(self._static_rows(ps, ms, vs), dtype=np.int64)
            for col, values in zip(self._MOVING, sig):
                rows[:, col] = values
            # a pinned copy of the rows stays with the table: what a captured step sends its new addresses through
            stage = torch.from_numpy(rows).pin_memory()
            plan.desc[slot] = torch.empty_like(stage, device=ps[0].value.device)
            plan.desc[slot].copy_(stage)
            plan.stage[slot] = stage
            plan.sig[slot] = sig
            return plan.desc[slot]
        old = plan.sig[slot]
        if old != sig:
            if capturing:
                # (gradients made under capture come from the graph's own memory) the whole table again, from pinned
                # memory: one copy the graph can hold.  The scratch words of the rows are zero between calls anyway.
                stage = plan.stage[slot]
                for col, values in zip(self._MOVING, sig):
                    stage[:, col] = torch.tensor(values, dtype=torch.int64)
                desc.copy_(stage, non_blocking=True)
            else:
                for col, values, before in zip(self._MOVING, sig, old):
                    if values != before:
                        desc[:, col] = torch.tensor(values, dtype=torch.int64).to(desc.device)
            plan.sig[slot] = sig
        return desc

    def _fused_step(self, idx, params, grads, exp_avgs, exp_avg_sqs, step, *, beta1, beta2, lr, weight_decay, eps,
                    maximize):
        ps, gs = [params[i] for i in idx], [grads[i] for i in idx]
        ms, vs = [exp_avgs[i] for i in idx], [exp_avg_sqs[i] for i in idx]
        wq, gq = int(ps[0].qtype), int(gs[0].qtype)
        key = (wq, gq, id(ps[0]))
        plan = self._plan_for(key, ps, ms, vs)
        if any(g.value.data_ptr() % 16 or not g.value.is_contiguous() for g in gs):
            # a gradient the fused kernels do not take (the grouping is kept from an earlier step): this step tensor by tensor
            self._groups = None
            self._staged_step(idx, params, grads, exp_avgs, exp_avg_sqs, [step] * len(params), beta1=beta1, beta2=beta2, lr=lr,
                              weight_decay=weight_decay, eps=eps, maximize=maximize)
            return
        hyper = (lr, beta1, beta2, eps, weight_decay, step, self.bias_correction, self.use_adam, maximize, self.tensor_scale)
        capturing = torch.cuda.is_current_stream_capturing()
        if self.one_pass == 'shift' and not capturing and self._shift_step(plan, ps, gs, ms, vs, wq, gq, hyper):
            return
        if self.one_pass == 'double' and not capturing and self._can_swap(ps, ms, vs):
            self._double_step(plan, ps, gs, ms, vs, wq, gq, hyper)
            return
        # in place, with the table of wherever the payloads are now (a moving form that has run leaves them at one of its
        # two places, and the table it keeps for that place holds the right addresses)
        if self.one_pass == 'shift' and plan.arenas is not None:
            slot = ('shift', plan.phase)
        elif self.one_pass == 'double' and plan.spare is not None:
            slot = ('double', ps[0].value.data_ptr())
        else:
            slot = ('in_place', ps[0].value.data_ptr())
        desc = self._table(plan, slot, ps, gs, ms, vs)
        _backend.adamw_fused(desc, len(ps), plan.block_map, plan.n_blocks, wq, gq, *hyper, blocks_per_tensor=plan.chunks)

    # ---- one pass between two sets of buffers -----------------------------------------------
    def _double_step(self, plan, ps, gs, ms, vs, wq, gq, hyper):
        current = [(p.value, m.value, v.value) for p, m, v in zip(ps, ms, vs)]
        if plan.spare is None or any(s.shape != c.shape or s.dtype != c.dtype or s.device != c.device
                                     for trio, cur in zip(plan.spare, current) for s, c in zip(trio, cur)):
            plan.spare = [[torch.empty_like(c) for c in cur] for cur in current]
            plan.outputs = {}
        slot = ('double', ps[0].value.data_ptr())
        desc = self._table(plan, slot, ps, gs, ms, vs)
        out_sig = [tuple(t.data_ptr() for t in trio) for trio in plan.spare]
        cached = plan.outputs.get(slot)
        if cached is None or cached[0] != out_sig:
            rows = np.asarray([sig + (0, ) for sig in out_sig], dtype=np.int64).reshape(len(ps), _backend.ADAMW_BUFFER_WORDS)
            cached = (out_sig, torch.from_numpy(rows).to(desc.device))
            plan.outputs[slot] = cached
        if plan.redo is None:
            plan.redo = torch.zeros(len(ps), dtype=torch.int32, device=desc.device)
        _backend.adamw_fused_speculative(desc, cached[1], plan.redo, len(ps), plan.block_map, plan.n_blocks, wq, gq, *hyper)
        # the payload tensors stay the objects they were and trade their memory with the spares
        for cur, trio in zip(current, plan.spare):
            for i, t in enumerate(cur):
                old = t.data
                t.data = trio[i]
                trio[i] = old

    @staticmethod
    def _can_swap(ps, ms, vs):
        """Swapping payload tensors is safe when nothing else aliases them."""
        return all(t.value._base is None for group in (ps, ms, vs) for t in group)

    # ---- one pass inside shifting arenas -----------------------------------------------------
    # room beyond the largest tensor: what the chip keeps in flight (about a thousand chunks) twice over, plus the lead
    # with which a tensor's outcome is decided before its first chunk is written over
    _SHIFT_MARGIN = 2560

    def _adopt(self, plan, ps, ms, vs):
        """Move the payloads into arenas of the optimizer's own (once; again if somebody replaced a payload)."""
        ch = _backend.ADAMW_CHUNK
        total = sum(plan.chunks)
        biggest = max(plan.chunks)
        plan.slack = biggest + min(self._SHIFT_MARGIN, max(total // 4, 1))
        device = ps[0].value.device
        plan.widths = (ps[0].value.element_size(), 1, 2)
        try:
            arenas = [torch.empty((total + plan.slack) * ch * width, dtype=torch.uint8, device=device) for width in plan.widths]
        except torch.cuda.OutOfMemoryError:
            return False
        pos = np.concatenate([[0], np.cumsum(plan.chunks)]).tolist()
        plan.views = [[], []]
        for i, (p, m, v) in enumerate(zip(ps, ms, vs)):
            for phase, off in ((0, plan.slack), (1, 0)):
                trio = []
                for arena, width, t in zip(arenas, plan.widths, (p.value, m.value, v.value)):
                    first = (pos[i] + off) * ch * width
                    trio.append(arena[first:first + t.numel() * width].view(t.dtype).view(t.shape))
                plan.views[phase].append(trio)
            # one tensor at a time, so that at most one payload exists twice while the arenas fill
            for t, view in zip((p.value, m.value, v.value), plan.views[0][i]):
                view.copy_(t)
                t.data = view
        plan.arenas = arenas
        plan.phase = 0
        plan.redo = torch.zeros(len(ps), dtype=torch.int32, device=device)
        plan.sync = torch.zeros(_backend.adamw_shift_sync_bytes(len(ps), total), dtype=torch.uint8, device=device)
        plan.desc = None
        return True

    def _shift_step(self, plan, ps, gs, ms, vs, wq, gq, hyper):
        """The step inside the arenas; False if this group cannot be taken that way (the caller then goes in place)."""
        sig = self._moving_sig(ps, gs, ms, vs)
        if plan.arenas is not None:
            home = plan.views[plan.phase]
            if any(w != trio[0].data_ptr() or m != trio[1].data_ptr() or v != trio[2].data_ptr()
                   for w, m, v, trio in zip(sig[0], sig[2], sig[3], home)):
                plan.arenas = None    # somebody put other tensors in place of the payloads (load_state_dict, .data): adopt again
        if plan.arenas is None:
            if not self._can_swap(ps, ms, vs) or len({p.value.element_size() for p in ps}) != 1:
                return False
            if not self._adopt(plan, ps, ms, vs):
                return False
            sig = self._moving_sig(ps, gs, ms, vs)
        desc = self._table(plan, ('shift', plan.phase), ps, gs, ms, vs, sig)
        shift = (-plan.slack if plan.phase == 0 else plan.slack) * _backend.ADAMW_CHUNK
        _backend.adamw_fused_shift(desc, plan.redo, plan.sync, len(ps), plan.block_map, plan.n_blocks, shift, wq, gq, *hyper)
        plan.phase = 1 - plan.phase
        # the payload tensors stay the objects they were; their memory is now the other place in the arena
        for p, m, v, trio in zip(ps, ms, vs, plan.views[plan.phase]):
            p.value.data = trio[0]
            m.value.data = trio[1]
            v.value.data = trio[2]
        return True

    # ---- parameters kept in high precision: one launch for all of them ---------------------
    _PLAIN_DTYPES = (torch.float32, torch.float16, torch.bfloat16)
    _PLAIN_LIMIT = 1 << 16    # elements up to which one workgroup takes a whole parameter (biases, norm weights, ...)

    @classmethod
    def _plain_fusable(cls, p, g, m, v):
        if isinstance(p, ScalingTensor) or isinstance(g, ScalingTensor) or not torch.is_tensor(p) or not torch.is_tensor(g):
            return False
        if not (isinstance(m, ScalingTensor) and isinstance(v, ScalingTensor)):
            return False
        if p.dtype not in cls._PLAIN_DTYPES or g.dtype not in cls._PLAIN_DTYPES:
            return False
        if m.qtype != Dtypes.kfloat8_e4m3 or v.qtype != Dtypes.kfloat16 or v.value.dtype != torch.float16:
            return False
        if p.numel() == 0 or m.meta.amax.numel() != 1 or v.meta.amax.numel() != 1:
            return False
        tensors = (p, g, m.value, v.value)
        if not all(t.is_cuda and t.is_contiguous() and t.numel() == p.numel() for t in tensors):
            return False
        # larger ones go chunk by chunk, four elements at a time
        return p.numel() <= cls._PLAIN_LIMIT or all(t.data_ptr() % 16 == 0 for t in tensors)

    def _plain_step(self, idx, params, grads, exp_avgs, exp_avg_sqs, step, *, beta1, beta2, lr, weight_decay, eps, maximize):
        """Both stages of the reference recipe (msamp/optim/adamw.py:148-199) for all plain parameters of one type in
        one launch (small ones) or three (the others, chunk by chunk), nothing read back by the host."""
        ps, gs = [params[i] for i in idx], [grads[i] for i in idx]
        ms, vs = [exp_avgs[i] for i in idx], [exp_avg_sqs[i] for i in idx]
        chunked = ps[0].numel() > self._PLAIN_LIMIT
        payloads = [t for quad in zip(ps, gs, (m.value for m in ms), (v.value for v in vs)) for t in quad]
        # (gradients are new tensors every step, and a parameter's storage may have been replaced)
        if any(not g.is_contiguous() or g.numel() != p.numel() for p, g in zip(ps, gs)) or \
                (chunked and any(t.data_ptr() % 16 for t in payloads)) or any(not t.is_contiguous() for t in payloads):
            self._groups = None    # (the grouping is kept from an earlier step) this step tensor by tensor
            self._staged_step(idx, params, grads, exp_avgs, exp_avg_sqs, [step] * len(params), beta1=beta1, beta2=beta2, lr=lr,
                              weight_decay=weight_decay, eps=eps, maximize=maximize)
            return
        key = ('plain', ps[0].dtype, gs[0].dtype, chunked, id(ps[0]))
        plan = self._plans.get(key)
        ids = tuple(id(p) for p in ps)
        if plan is None or plan.params != ids:
            plan = _FusedPlan()
            plan.params = ids
            if chunked:
                plan.chunks = [(p.numel() + _backend.ADAMW_CHUNK - 1) // _backend.ADAMW_CHUNK for p in ps]
                tensor_idx = np.repeat(np.arange(len(ps), dtype=np.int32), plan.chunks)
                chunk_idx = np.concatenate([np.arange(c, dtype=np.int32) for c in plan.chunks])
                plan.block_map = torch.from_numpy(np.stack([tensor_idx, chunk_idx], axis=1).copy()).to(ps[0].device)
                plan.n_blocks = int(plan.block_map.shape[0])
            self._plans[key] = plan
        static = [id(t) for m, v in zip(ms, vs) for t in (m.meta.scale, m.meta.scale_inv, m.meta.amax, v.meta.scale,
                                                           v.meta.scale_inv, v.meta.amax)]
        sig = ([p.data_ptr() for p in ps], [g.data_ptr() for g in gs], [m.value.data_ptr() for m in ms],
               [v.value.data_ptr() for v in vs])
        if plan.desc is None or plan.static_sig != static:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError('LBAdamW: the first step of a parameter group builds device tables and cannot be captured; '
                                   'take a step outside the capture first.')
            rows = np.zeros((len(ps), _backend.ADAMW_DESC_WORDS), dtype=np.int64)
            for col, values in enumerate(sig):
                rows[:, col] = values
            for r, (m, v) in enumerate(zip(ms, vs)):
                rows[r, 8:14] = (m.meta.scale.data_ptr(), m.meta.scale_inv.data_ptr(), m.meta.amax.data_ptr(),
                                 v.meta.scale.data_ptr(), v.meta.scale_inv.data_ptr(), v.meta.amax.data_ptr())
                rows[r, 14] = ps[r].numel()
            # a pinned copy of the rows stays with the table: what a captured step sends its new addresses through
            plan.stage = torch.from_numpy(rows).pin_memory()
            plan.desc = plan.stage.to(ps[0].device)
            plan.static_sig, plan.sig = static, sig
        elif plan.sig != sig:
            if torch.cuda.is_current_stream_capturing():
                # (gradients made under capture come from the graph's own memory) the whole table again, from pinned
                # memory: one copy that the graph can hold
                for col, values in enumerate(sig):
                    plan.stage[:, col] = torch.tensor(values, dtype=torch.int64)
                plan.desc.copy_(plan.stage, non_blocking=True)
            else:
                for col, (values, before) in enumerate(zip(sig, plan.sig)):
                    if values != before:
                        plan.desc[:, col] = torch.tensor(values, dtype=torch.int64).to(plan.desc.device)
            plan.sig = sig
        _backend.adamw_plain_fused(plan.desc, len(ps), _backend.hp_dt(ps[0]), _backend.hp_dt(gs[0]), lr, beta1, beta2, eps,
                                   weight_decay, step, self.bias_correction, self.use_adam, maximize, self.tensor_scale,
                                   block_map=plan.block_map, n_blocks=plan.n_blocks)

    # ---- float32 moments ---------------------------------------------------------------------
    def _f32_step(self, p, g, exp_avg, exp_avg_sq, step, *, beta1, beta2, lr, weight_decay, eps, maximize):
        """The chain of element-wise calls of the reference's float32 branch (msamp/optim/adamw.py:200-232) as one kernel,
        same bits; False where the kernel does not apply (the chain below then runs as written)."""
        moments = (exp_avg, exp_avg_sq)
        if any(isinstance(t, ScalingTensor) or t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous()
               for t in moments):
            return False
        param = p.float()
        grad = g.float() if isinstance(g, ScalingTensor) or g.dtype not in self._PLAIN_DTYPES else g
        if not (param.is_cuda and grad.is_cuda) or any(t.numel() != param.numel() for t in (grad, ) + moments):
            return False
        param, grad = param.contiguous(), grad.contiguous()
        _backend.adamw_f32(param, grad, exp_avg, exp_avg_sq, lr, beta1, beta2, eps, weight_decay, step, self.bias_correction,
                           self.use_adam, maximize)
        if isinstance(p, ScalingTensor):
            p.copy_(param.cast(p.qtype, meta=p.meta))
        elif param.data_ptr() != p.data_ptr():
            p.copy_(param)
        return True

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
            # Which parameters take the fused call is looked into once per set of parameters, states, gradient formats and
            # step counts (the look costs more host time than everything else in a step); what may change from step to
            # step without showing here -- where a gradient's payload lies -- is checked in _fused_step.
            key = (tuple(map(id, params)), tuple(map(id, exp_avgs)), tuple(map(id, exp_avg_sqs)),
                   tuple(g.qtype if isinstance(g, ScalingTensor) else g.dtype for g in grads),
                   tuple(n - state_steps[0] for n in state_steps), ScalingMeta.in_time_scaling)
            if self._groups is not None and self._groups[0] == key:
                fused, plain, staged = self._groups[1:]
            else:
                fused, plain = {}, {}
                staged = []
                for i in range(len(params)):
                    if self._fusable(params[i], grads[i], exp_avgs[i], exp_avg_sqs[i]):
                        fused.setdefault((int(params[i].qtype), int(grads[i].qtype), state_steps[i]), []).append(i)
                    elif self._plain_fusable(params[i], grads[i], exp_avgs[i], exp_avg_sqs[i]):
                        plain.setdefault((params[i].dtype, grads[i].dtype, state_steps[i],
                                          params[i].numel() > self._PLAIN_LIMIT), []).append(i)
                    else:
                        staged.append(i)
                self._groups = (key, fused, plain, staged)
            hyper = dict(beta1=beta1, beta2=beta2, lr=lr, weight_decay=weight_decay, eps=eps, maximize=maximize)
            for idx in fused.values():    # (one call per weight format, gradient format and step count)
                self._fused_step(idx, params, grads, exp_avgs, exp_avg_sqs, state_steps[idx[0]], **hyper)
            for idx in plain.values():    # (one call per parameter type, gradient type and step count)
                self._plain_step(idx, params, grads, exp_avgs, exp_avg_sqs, state_steps[idx[0]], **hyper)
            self._staged_step(staged, params, grads, exp_avgs, exp_avg_sqs, state_steps, **hyper)
            return
        # float32 moments: whole-tensor float32 update, then requantize the parameter if it is low-bit
        for i, p in enumerate(params):
            if self._f32_step(p, grads[i], exp_avgs[i], exp_avg_sqs[i], state_steps[i], beta1=beta1, beta2=beta2, lr=lr,
                              weight_decay=weight_decay, eps=eps, maximize=maximize):
                continue
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
