"""Flash STU's inference path on MI355X: the reference's public names
(flash_stu/__init__.py:1-15) backed by libflashstu_hip.so."""
from .blocks.block import FlashSTUBlock
from .config import FlashSTUConfig
from .model import FlashSTU
from .modules.attention import Attention
from .modules.stu import STU
from .utils.stu_utils import convolve, get_spectral_filters

__all__ = ["FlashSTU", "FlashSTUConfig", "FlashSTUBlock", "STU", "Attention", "get_spectral_filters", "convolve"]
