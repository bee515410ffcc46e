"""Quantization facade: config-driven codec calls, sizing, error feedback."""
from lowbit_comm_amd.exceptions import CCDLUnavailableError

from .codec import dequantize_tensor, quantize_tensor
from .error_feedback import ErrorFeedbackState
from .quantizer import Quantizer
from .sizing import QuantizationSizeEstimate, estimate_payload_size, estimate_quantized_size

__all__ = [
    "CCDLUnavailableError", "ErrorFeedbackState", "QuantizationSizeEstimate", "Quantizer", "dequantize_tensor",
    "estimate_payload_size", "estimate_quantized_size", "quantize_tensor",
]
