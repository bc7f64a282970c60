"""FlashMoBA for AMD Instinct MI355X (gfx950): the reference's Python API over hand-written HIP kernels."""
__version__ = "2.0.0+mi355x"

from flash_moba.flash_moba_interface import (  # noqa: F401
    flash_topk_varlen_func,
    flash_moba_attn_varlen_func,
    flash_moba_varlen_func,
)
