"""MI355X (gfx950) W8A8 linear backend for VolvoxAI packages.

The product is the C-ABI library ``lib/libvxhip_w8a8.so`` (header:
``include/vxhip_w8a8.h``) plus the C backend provider in ``provider/``.  This
Python package is a thin ctypes binding over that ABI, used by the tests and the
benchmark; PyTorch appears only as the owner of device buffers and streams.
"""
from ._lib import library, library_path, build_library, LibraryMissing  # noqa: F401
from .w8a8 import (  # noqa: F401
    DTYPE_I8, DTYPE_U8, Context, QLinear, PackedLinear, qlinear_i8u8,
    packed_linear_f32, quantize_typed_f32_i8u8, dequantize_typed_i8u8_f32,
    requantize_linear_i8u8, requantize_forward, kernel_variants, force_variant,
    ROW_OP_NONE, ROW_OP_RMSNORM, ROW_OP_SWIGLU,
)
