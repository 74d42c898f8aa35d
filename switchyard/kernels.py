"""`switchyard.kernels` on MI355X: every public name of the reference's module
(switchyard/kernels.py:12-93) bound to the gfx950 implementation in switchyard_amd.kernels."""

from switchyard_amd.kernels import (GEMM_MAX_ROWS, GEMV_MAX_ROWS, experts, ext, ffn, moe_layer, pick, route,  # noqa: F401
                                    tile_offsets)

__all__ = ["ext", "tile_offsets", "route", "GEMV_MAX_ROWS", "GEMM_MAX_ROWS", "pick", "ffn", "experts", "moe_layer"]
