"""Quantizer registry: the names the reference's CLI and model constructors use
(src/models/quantization/quantizers/__init__.py:59-100) for the MXFP4 path."""
from .base import BaseQuantizer, NoQuantizer
from .mxfp4 import (AlbertTsengQuantizer, AlignedAlbertTsengQuantizer, QuestMXFP4Quantizer,
                    mxfp4_forward_kernel_wrapper)

QUANTIZER_CLASSES = {
    "NoQuantizer": NoQuantizer,
    "QuestMXFP4Quantizer": QuestMXFP4Quantizer,
    "AlbertTsengQuantizer": AlbertTsengQuantizer,
    "AlignedAlbertTsengQuantizer": AlignedAlbertTsengQuantizer,
}

__all__ = ["BaseQuantizer", "NoQuantizer", "QuestMXFP4Quantizer",
           "AlbertTsengQuantizer", "AlignedAlbertTsengQuantizer", "mxfp4_forward_kernel_wrapper",
           "QUANTIZER_CLASSES"]
