"""MI355X-native DCNv4 and flash deformable attention operators behind the reference's Python
surface (DCNv4_op/DCNv4/__init__.py:1-2): ``DCNv4Function``, ``FlashDeformAttnFunction``,
``DCNv4``, ``FlashDeformAttn`` and the ``ext`` module of four raw operator functions.
Importing the package loads libdcnv4_gfx950.so and fails if it has not been built.
"""
from . import ext
from .functions import DCNv4Function, FlashDeformAttnFunction
from .modules import DCNv4, FlashDeformAttn

__all__ = ["ext", "DCNv4Function", "FlashDeformAttnFunction", "DCNv4", "FlashDeformAttn"]
