"""Drop-in `flash_attn` package whose forward path runs on hand-written gfx950 (MI355X) kernels."""
__version__ = "2.3.3+mi355x.0"

from flash_attn.flash_attn_interface import (  # noqa: F401
    flash_attn_func,
    flash_attn_kvpacked_func,
    flash_attn_qkvpacked_func,
    flash_attn_varlen_func,
    flash_attn_varlen_kvpacked_func,
    flash_attn_varlen_qkvpacked_func,
    flash_attn_with_kvcache,
)
