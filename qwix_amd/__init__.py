"""qwix_amd: MI355X-native quantize + quantized dot_general path behind Qwix's public surface."""
from qwix_amd.core.qarray import (HowToQuantize, Int4Tensor, QArray, calibrate, compute_scale_zero_point, dequantize,
                                  quantize_api as quantize, quantize_with_scale_zero_point)
from qwix_amd.core.dot_general import dot_general
from qwix_amd.core.einsum import einsum
from qwix_amd.core.dot import dot
from qwix_amd.core.ragged_dot import RaggedDotDimensionNumbers, ragged_dot, ragged_dot_general
from qwix_amd.qconfig import QuantizationProvider, QuantizationRule
from qwix_amd.providers.ptq import BoxedParamProvider, PtqProvider, WithAux, quantize_params
from qwix_amd.model import quantize_model
from qwix_amd.utils.checkpoint_util import process_prequantized_params, restore_quantization_rules

__all__ = ['HowToQuantize', 'Int4Tensor', 'QArray', 'calibrate', 'compute_scale_zero_point', 'dequantize', 'quantize',
           'quantize_with_scale_zero_point', 'dot_general', 'einsum', 'dot', 'RaggedDotDimensionNumbers', 'ragged_dot', 'ragged_dot_general', 'QuantizationProvider', 'QuantizationRule',
           'BoxedParamProvider', 'PtqProvider', 'WithAux', 'quantize_params', 'quantize_model', 'process_prequantized_params',
           'restore_quantization_rules']
