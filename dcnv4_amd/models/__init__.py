from .flash_intern_image import FlashInternImage, FlashInternImageBackbone, flash_intern_image

__all__ = ["FlashInternImage", "FlashInternImageBackbone", "flash_intern_image"]
