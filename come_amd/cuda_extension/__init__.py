"""Drop-in for the reference's ``src/cuda_extension`` package
(``src/cuda_extension/__init__.py:1-23``): same public names, HIP kernels underneath."""

from .flash_attn import (
    flash_attn_varlen_qkvpacked_func,
    flash_attn_varlen_qkvpacked_func_w_perkey_bias,
    infer_flash_attn_varlen_max_seqlen,
)
from .co_me import co_me_cuext

__all__ = [
    "co_me_cuext",
    "flash_attn_varlen_qkvpacked_func",
    "flash_attn_varlen_qkvpacked_func_w_perkey_bias",
    "infer_flash_attn_varlen_max_seqlen",
]
