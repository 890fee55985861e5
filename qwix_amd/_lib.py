"""ctypes binding of libqwix_hip.so (the C ABI declared in include/qwix_hip.h).

There is no fallback: if the shared library is missing, importing the kernels raises.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libqwix_hip.so')

OK = 0
F32, BF16, I32 = 0, 1, 2
INT8, INT4, E4M3 = 0, 1, 2
ABSMAX, MINMAX = 0, 1
LAYOUT_NATURAL, LAYOUT_REDUCE_MINOR = 0, 1

_c = ctypes
_vp, _i64, _int, _f32, _sz = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_float, _c.c_size_t

# name -> (restype, argtypes); mirrors include/qwix_hip.h one to one.
SIGNATURES = {
    'qwix_hip_abi_version': (_int, []),
    'qwix_hip_last_error': (_c.c_char_p, []),
    'qwix_hip_quantize_workspace_bytes': (_sz, [_i64, _i64, _i64, _i64, _int]),
    'qwix_hip_quantize': (_int, [_vp, _int, _i64, _i64, _i64, _i64, _int, _int, _f32, _int, _vp, _vp, _vp, _vp, _sz, _vp]),
    'qwix_hip_quantize_static_max_bytes': (_sz, []),
    'qwix_hip_quantize_static': (_int, [_vp, _int, _i64, _i64, _i64, _i64, _int, _int, _f32, _int, _vp, _vp, _vp, _vp]),
    'qwix_hip_calibrate': (_int, [_vp, _int, _i64, _i64, _i64, _i64, _int, _f32, _vp, _vp, _vp, _sz, _vp]),
    'qwix_hip_calibrate_rms': (_int, [_vp, _int, _c.POINTER(_i64), _i64, _i64, _f32, _vp, _vp]),
    'qwix_hip_compute_scale_zero_point': (_int, [_vp, _vp, _int, _i64, _int, _int, _vp, _vp, _vp]),
    'qwix_hip_quantize_with_scale': (_int, [_vp, _int, _i64, _i64, _i64, _i64, _int, _vp, _vp, _int, _vp, _vp]),
    'qwix_hip_quantize_with_scale_noise': (_int, [_vp, _int, _i64, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp, _vp]),
    'qwix_hip_quantize_generic': (_int, [_vp, _int, _c.POINTER(_i64), _i64, _i64, _int, _int, _f32, _vp, _vp, _vp, _vp]),
    'qwix_hip_dequantize': (_int, [_vp, _int, _int, _i64, _i64, _i64, _i64, _vp, _vp, _int, _vp, _vp]),
    'qwix_hip_dequantize_generic': (_int, [_vp, _int, _c.POINTER(_i64), _i64, _i64, _vp, _vp, _int, _vp, _vp]),
    'qwix_hip_transpose_q': (_int, [_vp, _int, _i64, _i64, _vp, _vp]),
    'qwix_hip_qgemm': (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _i64, _vp, _int, _vp, _int, _int, _vp, _int, _i64, _vp]),
    'qwix_hip_qgemm_workspace_bytes': (_sz, [_i64, _i64, _i64]),
    'qwix_hip_qgemm_ws': (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _i64, _vp, _int, _vp, _int, _int, _vp, _int, _i64, _vp, _sz, _vp]),
    'qwix_hip_qgemm_zp': (_int, [_vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _int, _vp, _int, _vp, _vp, _vp, _int, _i64, _vp]),
    'qwix_hip_qgemm_ragged': (_int, [_vp, _i64, _vp, _i64, _i64, _int, _i64, _i64, _i64, _vp, _i64, _vp, _int, _vp, _int, _i64, _int, _vp, _int, _i64, _vp]),
    'qwix_hip_qgemm_batched': (_int, [_vp, _i64, _i64, _vp, _i64, _i64, _int, _i64, _i64, _i64, _i64, _vp, _int, _i64, _vp, _int, _i64, _int, _vp, _int, _i64, _i64, _vp]),
    'qwix_hip_qgemm_fused_act': (_int, [_vp, _int, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _int, _vp, _int, _i64, _vp]),
    'qwix_hip_qgemm_dynamic_act_workspace_bytes': (_sz, [_i64, _i64, _i64, _int]),
    'qwix_hip_qgemm_dynamic_act': (_int, [_vp, _int, _i64, _vp, _i64, _int, _i64, _i64, _i64, _vp, _int, _int, _vp, _int, _i64, _vp, _sz, _vp]),
    'qwix_hip_qgemm_hadamard_act_workspace_bytes': (_sz, [_i64, _i64, _i64, _int]),
    'qwix_hip_qgemm_hadamard_act': (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _f32, _i64, _vp, _i64, _int, _i64, _vp, _int, _vp, _int, _i64, _vp, _sz, _vp]),
    'qwix_hip_ksum_i8': (_int, [_vp, _i64, _i64, _i64, _vp, _vp]),
    'qwix_hip_qgemm_grouped': (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _i64, _i64, _vp, _int, _i64, _vp, _int, _vp, _int, _i64, _int, _vp, _vp]),
    'qwix_hip_qgemm_grouped_workspace_bytes': (_sz, [_i64, _i64, _i64, _i64, _int]),
    'qwix_hip_qgemm_grouped_ws': (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _i64, _i64, _vp, _int, _i64, _vp, _int, _vp, _int, _i64, _int, _vp, _vp, _sz, _vp]),
    'qwix_hip_qgemm_grouped_zp': (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _i64, _i64, _vp, _int, _i64, _vp, _int, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _int, _i64, _int, _vp, _vp]),
    'qwix_hip_ksum_groups': (_int, [_vp, _int, _i64, _i64, _i64, _i64, _vp, _vp]),
    'qwix_hip_gemm_bf16': (_int, [_vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _int, _i64, _vp]),
    'qwix_hip_gemm_bf16_wq': (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _i64, _i64, _vp, _int, _vp, _vp, _int, _i64, _vp]),
    'qwix_hip_gemm_bf16_wq_workspace_bytes': (_sz, [_i64, _i64, _i64, _i64]),
    'qwix_hip_gemm_bf16_wq_ws': (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _i64, _i64, _vp, _int, _vp, _vp, _int, _i64, _vp, _sz, _vp]),
    'qwix_hip_dequantize_rm': (_int, [_vp, _int, _i64, _i64, _i64, _i64, _vp, _vp, _int, _vp, _int, _vp]),
    'qwix_hip_gemv_wq': (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _i64, _i64, _vp, _int, _vp, _int, _i64, _vp]),
    'qwix_hip_gemv_wq_zp': (_int, [_vp, _i64, _vp, _i64, _int, _i64, _i64, _i64, _i64, _vp, _int, _vp, _vp, _int, _i64, _vp]),
    'qwix_hip_fwht': (_int, [_vp, _int, _i64, _i64, _vp, _vp, _f32, _vp, _vp]),
    'qwix_hip_fwht_quantize': (_int, [_vp, _int, _i64, _i64, _vp, _vp, _f32, _i64, _int, _vp, _vp, _vp]),
    'qwix_hip_mfma_ceiling_ops': (_c.c_double, [_i64]),
    'qwix_hip_mfma_ceiling': (_int, [_vp, _sz, _vp, _sz, _int, _i64, _vp, _vp]),
}

_lib = None


class QwixHipError(RuntimeError):
  pass


def load() -> ctypes.CDLL:
  """Opens the shared library and declares every prototype."""
  global _lib
  if _lib is not None:
    return _lib
  if not os.path.exists(LIB_PATH):
    raise QwixHipError(
        f'{LIB_PATH} is missing: build it with `python qwix_amd/csrc/build.py` '
        '(there is no CPU or eager fallback for these ops).'
    )
  lib = ctypes.CDLL(LIB_PATH)
  for name, (res, args) in SIGNATURES.items():
    fn = getattr(lib, name)
    fn.restype = res
    fn.argtypes = args
  _lib = lib
  return lib


def call(name: str, *args) -> None:
  """Calls an int-returning entry point and raises with the library's message on error."""
  lib = load()
  status = getattr(lib, name)(*args)
  if status != OK:
    msg = lib.qwix_hip_last_error().decode('utf-8', 'replace')
    kind = {1: ValueError, 2: NotImplementedError}.get(status, QwixHipError)
    raise kind(f'{name}: {msg}')


def ptr(t) -> int | None:
  return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def stream_of(t: torch.Tensor) -> int:
  """The current HIP stream of the tensor's device, as the handle the C ABI takes."""
  if not t.is_cuda:
    raise QwixHipError('qwix_amd kernels need tensors on a HIP device (got a CPU tensor); there is no CPU path.')
  if _raw_stream is not None:  # an order of magnitude cheaper than building a torch.cuda.Stream object
    return _raw_stream(t.device.index)
  return torch.cuda.current_stream(t.device).cuda_stream


def float_tag(dtype: torch.dtype) -> int:
  if dtype == torch.float32:
    return F32
  if dtype == torch.bfloat16:
    return BF16
  raise NotImplementedError(f'float dtype {dtype} is not supported by the HIP kernels (f32, bf16 only)')
