"""ModelState: every FP8 layer's input/wgrad/ograd metas flattened into contiguous tensors so one
kernel updates all of them per optimizer step (msamp/nn/state.py:12-194)."""

from collections import OrderedDict

import torch

from msamp.common.dtype import Dtypes


class ModelState:
    """Process-wide registry of the flattened scaling metas."""
    def __init__(self):
        self._ready_to_scale_tensor = False
        self._flattened_scaling_metas = None
        self._local_scaling_metas = OrderedDict()
        self._use_fp8_ddp = False

    @property
    def ready_to_scale_tensor(self):
        return self._ready_to_scale_tensor

    @ready_to_scale_tensor.setter
    def ready_to_scale_tensor(self, value):
        self._ready_to_scale_tensor = value

    @property
    def flattened_scaling_metas(self):
        return self._flattened_scaling_metas

    @flattened_scaling_metas.setter
    def flattened_scaling_metas(self, value):
        self._flattened_scaling_metas = value

    @property
    def local_scaling_metas(self):
        return self._local_scaling_metas

    @property
    def use_fp8_ddp(self):
        return self._use_fp8_ddp

    @use_fp8_ddp.setter
    def use_fp8_ddp(self, value):
        self._use_fp8_ddp = value

    def clear(self):
        """Forget every registered model (metas stay locked; meant for tests and re-initialisation)."""
        self.__init__()

    @staticmethod
    def _check_in_mem(inner, outer):
        """Raise RuntimeError unless `inner`'s storage range lies inside `outer`'s."""
        p1, p2 = inner.data_ptr(), outer.data_ptr()
        s1 = Dtypes.dtype_to_size[inner.dtype] * inner.numel()
        s2 = Dtypes.dtype_to_size[outer.dtype] * outer.numel()
        if not (p2 <= p1 and p1 + s1 <= p2 + s2):
            raise RuntimeError(f'Memory ({p1}, {p1 + s1}) not in ({p2}, {p2 + s2})')

    @staticmethod
    def _flat_tensors(tensors):
        """Concatenate into one buffer and re-point every tensor at its slice of that buffer."""
        flat = torch.cat([t.reshape(-1) for t in tensors])
        offset = 0
        for t in tensors:
            n = t.numel()
            t.data = flat[offset:offset + n].view(t.shape)
            offset += n
        return flat

    @classmethod
    def _flatten_scaling_metas(cls, metas):
        n = len(metas)
        window_size = metas[0].window_size
        if any(m.window_size != window_size for m in metas):
            raise RuntimeError('All metas must have the same window_size.')
        qtype = metas[0].qtype
        if any(m.qtype != qtype for m in metas):
            raise RuntimeError('All metas must have the same qtype.')
        scales = cls._flat_tensors([m.scale for m in metas])
        scales_inv = cls._flat_tensors([m.scale_inv for m in metas])
        amaxs = cls._flat_tensors([m.amax for m in metas])
        amax_counters = cls._flat_tensors([m.amax_counter for m in metas])
        for m in metas:
            m.locked = True
        return dict(
            qtype=qtype, scales=scales, scales_inv=scales_inv, amaxs=amaxs.view(n, window_size), amax_counters=amax_counters
        )

    def check_metas_in_flat(self, scaling_metas):
        """RuntimeError if any tensor of these metas no longer aliases the flattened buffers."""
        if self._flattened_scaling_metas is None:
            return
        for key, meta in scaling_metas.items():
            flat = self._flattened_scaling_metas[key]
            ModelState._check_in_mem(meta.scale, flat['scales'])
            ModelState._check_in_mem(meta.scale_inv, flat['scales_inv'])
            ModelState._check_in_mem(meta.amax, flat['amaxs'])
            ModelState._check_in_mem(meta.amax_counter, flat['amax_counters'])

    def register_scaling_metas(self, model, group=None):
        """Collect `scaling_metas` of every module of `model` and (re)flatten all registered ones."""
        for name, module in model.named_modules():
            if getattr(module, 'scaling_metas', None) is not None:
                key, i = name, 2
                while key in self._local_scaling_metas:
                    key = f'{name}_{i}'
                    i += 1
                self._local_scaling_metas[key] = module.scaling_metas
        metas = list(self._local_scaling_metas.values())
        if not metas:
            return
        self._flattened_scaling_metas = {
            key: ModelState._flatten_scaling_metas([m[key] for m in metas])
            for key in metas[0].keys()
        }
        for per_module in metas:
            for m in per_module.values():
                m.group = group
        for per_module in metas:
            self.check_metas_in_flat(per_module)


model_state = ModelState()
