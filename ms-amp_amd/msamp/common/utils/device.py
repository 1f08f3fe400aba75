"""Device capability probe (msamp/common/utils/device.py:12-22 checks for 'h100'; here: gfx950)."""

import torch


class Device:
    """Static device queries."""
    @staticmethod
    def arch_name():
        if not torch.cuda.is_available():
            return ''
        props = torch.cuda.get_device_properties(torch.cuda.current_device())
        return getattr(props, 'gcnArchName', '') or props.name

    @staticmethod
    def is_fp8_supported():
        """True on CDNA4 (gfx950: OCP FP8 converters and the K=64/128 FP8 MFMA)."""
        return 'gfx950' in Device.arch_name().lower()
