"""Utilities: device probe, logger, the native-kernel wrapper."""

from msamp.common.utils.device import Device
from msamp.common.utils.logging import logger
from msamp.common.utils.transformer_engine_wrapper import TransformerEngineWrapper, PaddingTensor

__all__ = ['Device', 'logger', 'TransformerEngineWrapper', 'PaddingTensor']
