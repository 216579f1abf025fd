"""flash_attn_npu_3 for MI355X (gfx950): the third-generation call surface of
MinghuasLab/flash-attention-npu for the KV-cache path (reference flash_attn_npu_3/__init__.py:19-24;
no torch_npu import, no device-name gate), over the same gfx950 kernels as flash_attn_npu."""
__version__ = "0.3.0+mi355x"

from .flash_attn_npu_interface import (  # noqa: F401
    flash_attn_func,
    flash_attn_varlen_func,
    flash_attn_with_kvcache,
    get_scheduler_metadata,
)

__all__ = ["flash_attn_func", "flash_attn_varlen_func", "flash_attn_with_kvcache", "get_scheduler_metadata"]
