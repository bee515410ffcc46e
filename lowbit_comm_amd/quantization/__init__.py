"""Config-driven codec calls, payload sizing and error feedback: the names the reference's
``ccdl_comm.quantization`` package exports, bound here to this build's modules."""
from lowbit_comm_amd.exceptions import CCDLUnavailableError
from lowbit_comm_amd.quantization import codec as _codec
from lowbit_comm_amd.quantization import error_feedback as _error_feedback
from lowbit_comm_amd.quantization import quantizer as _quantizer
from lowbit_comm_amd.quantization import sizing as _sizing

quantize_tensor = _codec.quantize_tensor
dequantize_tensor = _codec.dequantize_tensor
ErrorFeedbackState = _error_feedback.ErrorFeedbackState
Quantizer = _quantizer.Quantizer
QuantizationSizeEstimate = _sizing.QuantizationSizeEstimate
estimate_quantized_size = _sizing.estimate_quantized_size
estimate_payload_size = _sizing.estimate_payload_size      # size of a fused [codes || scales] payload

__all__ = sorted(name for name, value in dict(globals()).items()
                 if not name.startswith("_") and getattr(value, "__module__", "").startswith("lowbit_comm_amd"))
