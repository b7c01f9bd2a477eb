"""MI355X-native ternary BitLinear (int8 activations x int2-packed weights).

The compute path is the HIP library built by ``python -m bitnet_amd.build``;
this package is the thin host side that mirrors the reference operator
interface (gpu/model.py:18-85, gpu/pack_weight.py, gpu/convert_checkpoint.py).
"""
from ._lib import BitLinearLibraryError, load_library  # noqa: F401
from .pack_weight import convert_weight_int2_to_int8, convert_weight_int8_to_int2  # noqa: F401


def __getattr__(name):
    # torch-dependent host mirror is imported lazily so that the ABI checks
    # (load_library) work without initialising torch
    if name in (
        "bitnet_int8xint2_linear", "bitnet_int8xint2_linear_seg", "bitnet_int8xint2_acc",
        "quant_input", "BitLinearKernel", "BitLinear",
    ):
        from . import bitlinear

        return getattr(bitlinear, name)
    raise AttributeError(name)
