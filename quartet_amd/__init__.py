"""MI355X-native implementation of Quartet's MXFP4 quantized-linear hot path.

Public surface mirrors the reference's ``models.quantization`` package:
``QuantizedLinear``, ``QUANTIZER_CLASSES``, ``BACKWARD_SCHEMES`` and the quantizer / scheme classes.
"""
from .backward import BACKWARD_SCHEMES, EW_EtX_Scheme, QEQWtt_QEtQXtt_Scheme, QEW_QEtX_Scheme
from .linear import (QuantizedLinear, QuartetLinearFn, enable_packed_weight_cache, invalidate_packed_weights,
                     set_device_seed_base)
from .quantizers import (QUANTIZER_CLASSES, AlbertTsengQuantizer, AlignedAlbertTsengQuantizer, BaseQuantizer,
                         NoQuantizer, QuestMXFP4Quantizer, mxfp4_forward_kernel_wrapper)

__all__ = ["QuantizedLinear", "QuartetLinearFn", "QUANTIZER_CLASSES", "BACKWARD_SCHEMES", "BaseQuantizer",
           "NoQuantizer", "QuestMXFP4Quantizer", "AlbertTsengQuantizer", "AlignedAlbertTsengQuantizer",
           "EW_EtX_Scheme", "QEW_QEtX_Scheme", "QEQWtt_QEtQXtt_Scheme", "mxfp4_forward_kernel_wrapper", "enable_packed_weight_cache", "invalidate_packed_weights", "set_device_seed_base"]
