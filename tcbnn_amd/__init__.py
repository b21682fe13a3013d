"""MI355X (gfx950) binarized-network inference path: Python host mirror of the reference's
layer API over the C ABI of libtcbnn_hip.so (see include/tcbnn_hip.h)."""
from . import _lib  # noqa: F401  (raises if the HIP library is not built)
from . import data  # noqa: F401  (host-only dataset readers and the accuracy check)
from ._lib import TcbnnError, VARIANTS, lib  # noqa: F401
from .layers import (ArrayWeights, Conv128LayerParam, Fc128LayerParam, In128LayerParam,  # noqa: F401
                     InConv128LayerParam, Out128LayerParam, TextWeightFile)
from .nets import Network, SPECS, synthetic_input, synthetic_weights  # noqa: F401
