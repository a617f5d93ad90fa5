from .modules import (MappedConvolution, MappedTransposedConvolution, MappedMaxPool,  # noqa: F401
                      MappedMaxUnpool,
                      MappedAvgPool, MappedAvgUnpool, Resample, Unresample, UVResample)
from ..layer_utils import InterpolationType  # noqa: F401
