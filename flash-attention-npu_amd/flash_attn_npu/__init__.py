"""flash_attn_npu for MI355X (gfx950): the paged KV-cache attention forward of
MinghuasLab/flash-attention-npu behind the same public names
(reference flash_attn_npu/__init__.py:12-21; no torch_npu import, no device-name gate)."""
__version__ = "0.3.0+mi355x"

from .flash_attn_npu_interface import (  # noqa: F401
    flash_attn_func,
    flash_attn_kvpacked_func,
    flash_attn_qkvpacked_func,
    flash_attn_varlen_func,
    flash_attn_varlen_kvpacked_func,
    flash_attn_varlen_qkvpacked_func,
    flash_attn_with_kvcache,
)

__all__ = ["flash_attn_func", "flash_attn_kvpacked_func", "flash_attn_qkvpacked_func", "flash_attn_varlen_func",
           "flash_attn_varlen_kvpacked_func", "flash_attn_varlen_qkvpacked_func", "flash_attn_with_kvcache"]
