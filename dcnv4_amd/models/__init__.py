from .flash_intern_image import FlashInternImage, flash_intern_image

__all__ = ["FlashInternImage", "flash_intern_image"]
