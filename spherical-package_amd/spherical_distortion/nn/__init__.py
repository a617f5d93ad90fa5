from .modules import (MappedConvolution, MappedTransposedConvolution, MappedMaxPool,  # noqa: F401
                      Resample, Unresample)
from ..layer_utils import InterpolationType  # noqa: F401
