"""MI355X-native MXFP6 block-scaled GEMM behind the reference's `tk_kernel.dispatch_micro` operator."""
from . import tk_kernel  # noqa: F401
from .tk_kernel import E2M3, E3M2, LAYOUT_ROW, LAYOUT_TILE, dispatch_micro, pack_weights, quantize, scale_width, tile_operand, tile_scales, unpack_weights  # noqa: F401
