"""Import alias: ``import DCNv4`` / ``from DCNv4 import ext`` resolve to :mod:`dcnv4_amd`, so code written
against the reference package (DCNv4_op/DCNv4/__init__.py:1-2) runs unchanged."""
import sys

import dcnv4_amd
from dcnv4_amd import DCNv4, DCNv4Function, FlashDeformAttn, FlashDeformAttnFunction, ext, functions, modules

sys.modules[__name__ + ".ext"] = ext
sys.modules[__name__ + ".functions"] = functions
sys.modules[__name__ + ".modules"] = modules

__all__ = ["ext", "DCNv4Function", "FlashDeformAttnFunction", "DCNv4", "FlashDeformAttn"]
