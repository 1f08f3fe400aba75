"""dtype package: QType, Dtypes, Floating."""

from msamp.common.dtype.dtypes import QType, Dtypes
from msamp.common.dtype.floating import Floating

__all__ = ['QType', 'Dtypes', 'Floating']
