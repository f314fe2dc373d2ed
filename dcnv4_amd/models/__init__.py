from .checkpoint import check_state_dict, load_checkpoint, offset_mask_features, reference_schema, unwrap_checkpoint
from .flash_intern_image import FlashInternImage, FlashInternImageBackbone, flash_intern_image

__all__ = ["FlashInternImage", "FlashInternImageBackbone", "flash_intern_image", "reference_schema", "check_state_dict",
           "load_checkpoint", "unwrap_checkpoint", "offset_mask_features"]
