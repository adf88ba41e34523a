__version__ = "0.0.1"

from flash_attn_v100.flash_attn_interface import (
    flash_attn_func,
)
