from .block import FlashSTUBlock

__all__ = ["FlashSTUBlock"]
