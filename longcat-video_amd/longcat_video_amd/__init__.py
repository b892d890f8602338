"""MI355X (gfx950) block-sparse attention engine behind the LongCat-Video
``longcat_video/block_sparse_attention`` call surface.

``flash_attn_bsa_3d`` is the drop-in for the reference operator
(longcat_video/block_sparse_attention/bsa_interface.py:612); everything below it
runs in hand-written HIP kernels reached through a C-ABI shared library.
There is no CPU or eager fallback: if the library is missing, importing the
operator modules raises.
"""
from .block_sparse_attention.bsa_interface import (  # noqa: F401
    flash_attn_bsa,
    flash_attn_bsa_3d,
)

__all__ = ["flash_attn_bsa", "flash_attn_bsa_3d"]
