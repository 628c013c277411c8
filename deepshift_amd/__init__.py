"""MI355X (gfx950) implementation of DeepShift's shift-kernel inference path.

Module layout mirrors the reference's ``deepshift`` package: ``kernels`` (dispatch to the HIP
library), ``utils`` (fixed-point / power-of-two helpers, weight packing), ``ste``, ``modules``
(``LinearShift``, ``Conv2dShift``), ``modules_q`` (``LinearShiftQ``, ``Conv2dShiftQ``) and
``convert`` (``convert_to_shift``, ``round_shift_weights``).
"""
from . import kernels, utils, ste, modules, modules_q, convert  # noqa: F401
from .modules import LinearShift, Conv2dShift  # noqa: F401
from .modules_q import LinearShiftQ, Conv2dShiftQ  # noqa: F401
from .convert import convert_to_shift, round_shift_weights, count_layer_type  # noqa: F401

__version__ = "0.1.0"
