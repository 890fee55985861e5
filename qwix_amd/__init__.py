"""qwix_amd: MI355X-native quantize + quantized dot_general path with Qwix's public surface."""
from qwix_amd.core.qarray import (HowToQuantize, Int4Tensor, QArray, calibrate, compute_scale_zero_point, dequantize,
                                  quantize_api as quantize, quantize_with_scale_zero_point)
from qwix_amd.core.dot_general import dot_general

__all__ = ['HowToQuantize', 'Int4Tensor', 'QArray', 'calibrate', 'compute_scale_zero_point', 'dequantize',
           'quantize', 'quantize_with_scale_zero_point', 'dot_general']
