#!/usr/bin/env python3
"""Benchmark of the quantize + quantized-dot hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extra] [--no-cpu-baseline]

A "step" is one pass of the hot path over one batch of synthetic input that is already resident
in HBM.  The default workload is the dynamic-range w8a8 int8 prefill GEMM at 4096^3 (the shape the
metric "int8 qdot TOPS + % MFMA peak" is quoted on): per step the bf16 activations are quantized
per token to int8 on the fly and multiplied with the pre-quantized int8 weight on the matrix
cores, with the per-token x per-channel scale epilogue fused, bf16 out.  All launches go through
the C ABI of libqwix_hip.so with preallocated buffers.

Prints ONE JSON line.  `roofline` describes the dominant kernel (the MFMA GEMM): achieved =
2*M*N*K / mean kernel time.  The kernel time comes from a second timed region of the same length in
which only that kernel is launched, back to back, between two events on the launch stream: a pair of
events around every single launch inside the step loop adds about 3 us of its own to a 10 us kernel.
`cpu_baseline` times the NumPy oracle of the same step on a bounded sample on the host cores; it is
a reported baseline, not a target.  `extra` carries the other workloads of the metric (quantize
GB/s, fp8 GEMM, weight-only GEMV, Hadamard-rotated GEMM), each with its own roofline fraction.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_TOPS = 5000.0   # MI355X dense int8 / fp8 matrix peak, TOP/s (TFLOP/s for fp8)
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E peak, GB/s


SPIN_UP_S = 0.5           # minimum duration of the untimed warm-up


def _events(n):
  import torch
  return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


class Workload:
  """setup() allocates everything; step(i) enqueues step number i; kernel(i) enqueues only the dominant
  kernel of that step on inputs a step has already produced; describe() gives the static numbers."""

  name = ''
  dtype = ''
  metric = ''
  unit = ''
  bound = 'mfma'

  def setup(self, dev): ...
  def step(self, i=0): ...
  def kernel(self, i=0): ...
  def work_per_step(self) -> float: ...      # ops (mfma) or bytes (hbm) of the whole step's headline figure
  def kernel_work(self) -> float: ...        # algorithmic ops / bytes of ONE launch of the dominant kernel


def _lib():
  from qwix_amd import _lib as L
  L.load()
  return L


class QdotW8A8(Workload):
  """activation quantize (per token) + MFMA GEMM with fused scale epilogue, one library call per step
  (qwix_hip_qgemm_dynamic_act: the quantize kernel and the GEMM back to back on a caller workspace); qtype int8 or e4m3."""

  bound = 'mfma'

  def __init__(self, name, M, K, N, qtype):
    self.name, self.M, self.K, self.N, self.qtype = name, M, K, N, qtype
    self.dtype = 'int8' if qtype == 'int8' else 'f8e4m3'
    self.metric = ('int8' if qtype == 'int8' else 'fp8') + ' qdot TOPS (dynamic-range w8a8, activation quantize included)'
    self.unit = 'TOPS'
    self.kernel_name = 'qgemm_pp_kernel' if ((M + 255) // 256) * ((N + 255) // 256) >= 192 and K >= 256 else 'qgemm_dma_kernel'

  def setup(self, dev):
    import torch
    from qwix_amd.core import qarray
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(3000 + self.M)
    self.x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
    w = (torch.randn(self.K, self.N, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
    # PTQ: the weight is quantized once, per output channel, into the K-contiguous layout.
    wq = qarray.quantize(w, qarray.HowToQuantize(qtype=self.qtype, channelwise_axes=[1]))
    del w
    self.wq = wq
    self.b = wq.qvalue.permute(1, 0)          # (N, K) contiguous
    assert self.b.is_contiguous()
    self.sb = wq.scale.reshape(-1).contiguous()
    self.xq = torch.empty(self.M, self.K, dtype=wq.qvalue.dtype, device=dev)
    self.sa = torch.empty(self.M, dtype=torch.bfloat16, device=dev)
    self.out = torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev)
    self.qt = L.INT8 if self.qtype == 'int8' else L.E4M3
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L
    # the step is one library call (quantize + GEMM on a caller workspace); the GEMM alone, for the roofline figure,
    # runs on activations quantized once here
    nws = int(L.load().qwix_hip_qgemm_dynamic_act_workspace_bytes(self.M, self.N, self.K, L.BF16))
    self.ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=dev)
    L.call('qwix_hip_quantize', self.x.data_ptr(), L.BF16, self.M, self.K, 1, self.K, self.qt, L.ABSMAX, 0.0,
           L.LAYOUT_NATURAL, self.xq.data_ptr(), self.sa.data_ptr(), None, None, 0, self.stream)

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_qgemm_dynamic_act', self.x.data_ptr(), L.BF16, self.K, self.b.data_ptr(), self.K, self.qt, self.M,
           self.N, self.K, self.sb.data_ptr(), L.BF16, L.BF16, self.out.data_ptr(), L.BF16, self.N, self.ws.data_ptr(),
           self.ws.numel(), self.stream)

  def kernel(self, i=0):
    L = self.L
    L.call('qwix_hip_qgemm', self.xq.data_ptr(), self.K, self.b.data_ptr(), self.K, self.qt, self.M, self.N, self.K,
           self.sa.data_ptr(), L.BF16, self.sb.data_ptr(), L.BF16, L.BF16, self.out.data_ptr(), L.BF16, self.N,
           self.stream)

  def work_per_step(self):
    return 2.0 * self.M * self.N * self.K

  def kernel_work(self):
    return 2.0 * self.M * self.N * self.K

  def describe(self):
    return {'workload': self.name, 'M': self.M, 'K': self.K, 'N': self.N,
            'activation': 'bf16 N(0,1), per-token absmax -> ' + self.qtype + ' each step',
            'weight': 'bf16 N(0,0.02) per-output-channel ' + self.qtype + ' (pre-quantized)', 'out': 'bf16'}

  def cpu_baseline(self, budget_rows=4096, repeats=3):
    """The oracle's version of one step on the first `budget_rows` tokens (best of `repeats`)."""
    import numpy as np
    from oracle import qwix_oracle as O
    rows = min(budget_rows, self.M)
    x = self.x[:rows].to('cpu').float().numpy()
    wq = self.wq
    wv = wq.qvalue.to('cpu')
    if self.qtype == 'int8':
      wnp = wv.numpy()
    else:
      import torch
      wnp = wv.contiguous().view(torch.uint8).numpy()
    owq = O.QArray(np.ascontiguousarray(wnp), O.FArr(wq.scale.to('cpu').float().numpy(), O.BF16), None, self.qtype)
    how = O.HowToQuantize(qtype=self.qtype, channelwise_axes=[0])
    dn = (((1,), (0,)), ((), ()))
    dt = float('inf')
    for _ in range(repeats):
      t0 = time.perf_counter()
      xq = O.quantize(O.FArr(x, O.BF16), how)
      O.dot_general(xq, owq, dn)
      dt = min(dt, time.perf_counter() - t0)
    ops = 2.0 * rows * self.N * self.K
    return {'value': round(ops / dt / 1e12, 5), 'unit': 'TOPS', 'cores': _blas_threads(), 'kind': 'port',
            'sample': f'first {rows} of {self.M} tokens against the full ({self.K},{self.N}) weight: oracle quantize + '
                      f'dot_general (float64 BLAS accumulate), best of {repeats}: {dt:.2f} s'}


class QuantizeRows(Workload):
  bound = 'hbm'

  def __init__(self, name, M, K, qtype):
    self.name, self.M, self.K, self.qtype = name, M, K, qtype
    self.dtype = 'bf16->' + qtype
    self.metric = 'quantize GB/s (per-token absmax, bf16 -> ' + qtype + ')'
    self.unit = 'GB/s'
    self.kernel_name = 'rows_kernel'

  def setup(self, dev):
    import torch
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(7)
    self.x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
    qb = self.K // 2 if self.qtype == 'int4' else self.K
    self.q = torch.empty(self.M, qb, dtype=torch.uint8, device=dev)
    self.s = torch.empty(self.M, dtype=torch.bfloat16, device=dev)
    self.qt = {'int8': L.INT8, 'int4': L.INT4, 'float8_e4m3fn': L.E4M3}[self.qtype]
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_quantize', self.x.data_ptr(), L.BF16, self.M, self.K, 1, self.K, self.qt, L.ABSMAX, 0.0,
           L.LAYOUT_NATURAL, self.q.data_ptr(), self.s.data_ptr(), None, None, 0, self.stream)

  kernel = step

  def work_per_step(self):
    return self.M * self.K * 2.0 + self.q.numel() + self.M * 2.0

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'M': self.M, 'K': self.K}


class QuantizeWeight(Workload):
  """PTQ of a (K, N) weight: per-output-channel absmax (reduction along the strided axis), written in the
  K-contiguous layout the GEMM reads."""

  bound = 'hbm'

  def __init__(self, name, K, N, qtype, group=None):
    self.name, self.K, self.N, self.qtype, self.group = name, K, N, qtype, group
    self.dtype = 'bf16->' + qtype
    self.metric = 'weight quantize GB/s (per-channel absmax along K, bf16 -> ' + qtype + ')'
    self.unit = 'GB/s'
    self.kernel_name = 'cols_quantize_kernel'

  def setup(self, dev):
    import torch
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(9)
    self.w = (torch.randn(self.K, self.N, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
    tile = self.group or self.K
    qb = self.K // 2 if self.qtype == 'int4' else self.K
    self.q = torch.empty(self.N, qb, dtype=torch.uint8, device=dev)
    self.s = torch.empty(self.K // tile, self.N, dtype=torch.bfloat16, device=dev)
    self.qt = {'int8': L.INT8, 'int4': L.INT4, 'float8_e4m3fn': L.E4M3}[self.qtype]
    self.tile = tile
    n = L.load().qwix_hip_quantize_workspace_bytes(1, self.K, self.N, tile, L.ABSMAX)
    self.ws = torch.empty(max(int(n), 16), dtype=torch.uint8, device=dev)
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_quantize', self.w.data_ptr(), L.BF16, 1, self.K, self.N, self.tile, self.qt, L.ABSMAX, 0.0,
           L.LAYOUT_REDUCE_MINOR, self.q.data_ptr(), self.s.data_ptr(), None, self.ws.data_ptr(), self.ws.numel(),
           self.stream)

  kernel = step

  def work_per_step(self):
    return self.K * self.N * 2.0 + self.q.numel() + self.s.numel() * 2.0

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'K': self.K, 'N': self.N, 'group': self.group}


class FwhtQuantize(Workload):
  """C5 activations: Walsh-Hadamard rotation along K fused with per-token int8 quantization."""

  bound = 'hbm'

  def __init__(self, name, M, K):
    self.name, self.M, self.K = name, M, K
    self.dtype = 'bf16->int8'
    self.metric = 'Hadamard rotate + quantize GB/s (per-token absmax, bf16 -> int8)'
    self.unit = 'GB/s'
    self.kernel_name = 'fwht_mfma_kernel' if K == 8192 else 'fwht_reg_kernel'

  def setup(self, dev):
    import torch
    from qwix_amd.contrib import hadamard_rot as hr
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(5001)
    self.x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
    self.signs = hr.random_signs(g, self.K, torch.bfloat16, dev)
    self.q = torch.empty(self.M, self.K, dtype=torch.int8, device=dev)
    self.s = torch.empty(self.M, dtype=torch.bfloat16, device=dev)
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_fwht_quantize', self.x.data_ptr(), L.BF16, self.M, self.K, self.signs.data_ptr(), None, 1.0, self.K,
           L.INT8, self.q.data_ptr(), self.s.data_ptr(), self.stream)

  kernel = step

  def work_per_step(self):
    return self.M * self.K * 3.0 + self.M * 2.0

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'M': self.M, 'K': self.K}


class PlainCopy(Workload):
  """A device-to-device copy of known size: the yardstick the HBM counters are scaled by."""

  bound = 'hbm'

  def __init__(self, name, nbytes):
    self.name, self.nbytes = name, nbytes
    self.dtype = 'u8'
    self.metric = 'plain copy GB/s (read + write)'
    self.unit = 'GB/s'
    self.kernel_name = 'torch copy_'

  def setup(self, dev):
    import torch
    self.src = torch.randint(0, 255, (self.nbytes,), dtype=torch.uint8, device=dev)
    self.dst = torch.empty_like(self.src)

  def step(self, i=0):
    self.dst.copy_(self.src)

  kernel = step

  def work_per_step(self):
    return 2.0 * self.nbytes

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'bytes_read': self.nbytes, 'bytes_written': self.nbytes}


class GemvW4(Workload):
  bound = 'hbm'

  def __init__(self, name, M, K, N, group, qtype='int4'):
    self.name, self.M, self.K, self.N, self.group, self.qtype = name, M, K, N, group, qtype
    self.dtype = 'bf16 x ' + qtype
    self.metric = f'weight-only {qtype} g128 GEMV GB/s'
    self.unit = 'GB/s'
    self.kernel_name = 'gemv_wq_kernel'
    self.wbytes = 0.5 if qtype == 'int4' else 1.0

  def setup(self, dev):
    import torch
    from qwix_amd.core import qarray
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(2000)
    self.x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
    w = (torch.randn(self.K, self.N, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
    wq = qarray.quantize_api(w, self.qtype, channelwise_axes=[1], tiled_axes={0: self.group}, scale_dtype=torch.float32)
    b = wq.qvalue.permute(1, 0)
    b = b.data if self.qtype == 'int4' else b.contiguous()
    assert b.is_contiguous()
    s = wq.scale.contiguous()
    # A decoder walks through a different weight matrix per layer: rotate over enough copies that a
    # launch finds none of its weights in the 256 MB last-level cache.
    self.copies = max(1, -(-(640 << 20) // (b.numel() * b.element_size())))
    self.b = [b] + [b.clone() for _ in range(self.copies - 1)]
    self.s = [s] + [s.clone() for _ in range(self.copies - 1)]
    self.out = torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev)
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    c = i % self.copies
    L.call('qwix_hip_gemv_wq', self.x.data_ptr(), self.K, self.b[c].data_ptr(), int(self.K * self.wbytes),
           L.INT4 if self.qtype == 'int4' else L.INT8, self.M, self.N,
           self.K, self.group, self.s[c].data_ptr(), L.F32, self.out.data_ptr(), L.BF16, self.N, self.stream)

  kernel = step

  def work_per_step(self):
    return self.K * self.N * self.wbytes + (self.K // self.group) * self.N * 4.0 + self.M * self.K * 2.0 + self.M * self.N * 2.0

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'M': self.M, 'K': self.K, 'N': self.N, 'group': self.group,
            'weight_copies_rotated': self.copies}


class WeightOnlyPrefill(Workload):
  """Weight-only int4 g128 at prefill size on the bf16 matrix cores (f32 accumulate, bf16 out).  Above 1024 rows
  the int4 weight is dequantized into a K-contiguous bf16 array per step and multiplied from there; up to 1024
  rows one kernel dequantizes it slab by slab inside its workgroups (the operator's own choice of path)."""

  bound = 'mfma'
  peak_tops = 2500.0   # dense bf16 MFMA peak, TFLOP/s

  def __init__(self, name, M, K, N, group):
    self.name, self.M, self.K, self.N, self.group = name, M, K, N, group
    self.dtype = 'bf16 x int4'
    self.metric = 'weight-only int4 g128 prefill TFLOP/s (weight dequantize included)'
    self.unit = 'TFLOP/s'
    self.fused = M <= 1024
    # 256 x 256 tiles (ping-pong kernel) once they fill most of the chip, 128 x 128 tiles below
    self.kernel_name = ('wgemm_wq_kernel' if self.fused else
                        'qgemm_pp_kernel' if -(-M // 256) * -(-N // 256) >= 192 else 'qgemm_dma_kernel')

  def setup(self, dev):
    import torch
    from qwix_amd.core import qarray
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(2100)
    self.x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
    w = (torch.randn(self.K, self.N, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
    wq = qarray.quantize_api(w, 'int4', channelwise_axes=[1], tiled_axes={0: self.group}, scale_dtype=torch.float32)
    self.b = wq.qvalue.permute(1, 0).data
    assert self.b.is_contiguous()
    self.s = wq.scale.contiguous()
    self.w = torch.empty(self.N, self.K, dtype=torch.bfloat16, device=dev)
    self.out = torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev)
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L
    # few tiles (the down projection's N 4096): K in ranges, f32 partials in a workspace, as the operator calls it
    self.nws = int(L.load().qwix_hip_gemm_bf16_wq_workspace_bytes(self.M, self.N, self.K, self.group)) if self.fused else 0
    self.ws = torch.empty(max(self.nws, 16), dtype=torch.uint8, device=dev)

  def step(self, i=0):
    L = self.L
    if not self.fused:
      L.call('qwix_hip_dequantize_rm', self.b.data_ptr(), L.INT4, 1, self.K, self.N, self.group, self.s.data_ptr(), None,
             L.F32, self.w.data_ptr(), L.BF16, self.stream)
    self.kernel(i)

  def kernel(self, i=0):
    L = self.L
    if self.fused:
      L.call('qwix_hip_gemm_bf16_wq_ws', self.x.data_ptr(), self.K, self.b.data_ptr(), self.b.stride(0), L.INT4, self.M,
             self.N, self.K, self.group, self.s.data_ptr(), L.F32, None, self.out.data_ptr(), L.BF16, self.N,
             self.ws.data_ptr() if self.nws else None, self.nws, self.stream)
      return
    L.call('qwix_hip_gemm_bf16', self.x.data_ptr(), self.K, self.w.data_ptr(), self.K, self.M, self.N, self.K,
           self.out.data_ptr(), L.BF16, self.N, self.stream)

  def work_per_step(self):
    return 2.0 * self.M * self.N * self.K

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'M': self.M, 'K': self.K, 'N': self.N, 'group': self.group}


class QdotDecode(Workload):
  """Dynamic-range w8a8 at decode size: per-token int8 quantize of a few tokens + the quantized GEMM that
  streams the int8 weight once (HBM-bound): the skinny kernel up to 16 tokens, the 64-row tile above."""

  bound = 'hbm'
  graph_ok = False

  def __init__(self, name, M, K, N, kernel_name='qgemm_skinny_kernel'):
    self.name, self.M, self.K, self.N = name, M, K, N
    self.dtype = 'int8'
    self.metric = 'w8a8 int8 decode GB/s (activation quantize included)'
    self.unit = 'GB/s'
    self.kernel_name = kernel_name

  def setup(self, dev):
    import torch
    from qwix_amd.core import qarray
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(2100)
    self.x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
    w = (torch.randn(self.K, self.N, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
    wq = qarray.quantize(w, qarray.HowToQuantize(qtype='int8', channelwise_axes=[1]))
    b = wq.qvalue.permute(1, 0)
    assert b.is_contiguous()
    self.copies = max(1, -(-(640 << 20) // (b.numel())))   # rotate: every launch reads its weight from HBM
    self.b = [b] + [b.clone() for _ in range(self.copies - 1)]
    self.sb = wq.scale.reshape(-1).contiguous()
    self.xq = torch.empty(self.M, self.K, dtype=torch.int8, device=dev)
    self.sa = torch.empty(self.M, dtype=torch.bfloat16, device=dev)
    self.out = torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev)
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_quantize', self.x.data_ptr(), L.BF16, self.M, self.K, 1, self.K, L.INT8, L.ABSMAX, 0.0,
           L.LAYOUT_NATURAL, self.xq.data_ptr(), self.sa.data_ptr(), None, None, 0, self.stream)
    self.kernel(i)

  def kernel(self, i=0):
    L = self.L
    L.call('qwix_hip_qgemm', self.xq.data_ptr(), self.K, self.b[i % self.copies].data_ptr(), self.K, L.INT8, self.M,
           self.N, self.K, self.sa.data_ptr(), L.BF16, self.sb.data_ptr(), L.BF16, L.BF16, self.out.data_ptr(), L.BF16,
           self.N, self.stream)

  def work_per_step(self):
    return self.K * self.N + self.N * 2.0 + self.M * self.K * 3.0 + self.M * self.N * 2.0

  def kernel_work(self):
    return self.K * self.N + self.N * 2.0 + self.M * self.K * 1.0 + self.M * self.N * 2.0

  def describe(self):
    return {'workload': self.name, 'M': self.M, 'K': self.K, 'N': self.N, 'weight_copies_rotated': self.copies}


class QdotDecodeFused(QdotDecode):
  """The same decode step in one launch: the per-token quantization of the activations happens inside the
  skinny GEMM (every workgroup re-derives the row scales from the bf16 activations it reads from L2)."""

  def __init__(self, name, M, K, N):
    super().__init__(name, M, K, N)
    self.metric = 'w8a8 int8 decode GB/s (activation quantize fused into the GEMM launch)'
    self.kernel_name = 'qgemm_skinny_fused_kernel'

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_qgemm_fused_act', self.x.data_ptr(), L.BF16, self.K, self.b[i % self.copies].data_ptr(), self.K,
           self.M, self.N, self.K, self.sb.data_ptr(), L.BF16, self.out.data_ptr(), L.BF16, self.N, self.stream)

  kernel = step

  def work_per_step(self):
    return self.K * self.N + self.N * 2.0 + self.M * self.K * 2.0 + self.M * self.N * 2.0

  kernel_work = work_per_step


class HadamardQdot(Workload):
  """C5: FWHT + per-token int8 quantize of the activations each step, then int8 x int4 g128 grouped GEMM
  against the offline-rotated weight."""

  bound = 'mfma'

  def __init__(self, name, M, K, N):
    self.name, self.M, self.K, self.N = name, M, K, N
    self.dtype = 'int8 x int4'
    self.metric = 'Hadamard-rotated a8w4 g128 qdot TOPS (FWHT + activation quantize included)'
    self.unit = 'TOPS'
    self.kernel_name = 'qgemm_grouped_dma_kernel'

  def setup(self, dev):
    import torch
    from qwix_amd.contrib import hadamard_rot as hr
    from qwix_amd.core import qarray
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(5000)
    x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32)
    idx = torch.randperm(self.K, generator=g)[: -(-self.K // 100)]
    x[:, idx] *= 50.0
    self.x = x.to(torch.bfloat16).to(dev)
    w = (torch.randn(self.K, self.N, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
    self.signs = hr.random_signs(g, self.K, torch.bfloat16, dev)
    wq = hr.rotate_and_quantize(w, 0, qarray.HowToQuantize(qtype='int4', channelwise_axes=[1], tiled_axes={0: 128}),
                                pre_sign=self.signs, out_scale=1.0 / self.K)
    del w
    self.b = wq.qvalue.permute(1, 0).data
    assert self.b.is_contiguous()
    self.sb = wq.scale.contiguous()
    self.xq = torch.empty(self.M, self.K, dtype=torch.int8, device=dev)
    self.sa = torch.empty(self.M, dtype=torch.bfloat16, device=dev)
    self.out = torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev)
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L
    # few tiles: K in ranges with f32 partial sums in a workspace, as the operator calls it (0 bytes: not split)
    self.nws = int(L.load().qwix_hip_qgemm_grouped_workspace_bytes(self.M, self.N, self.K, 128, L.INT4))
    self.ws = torch.empty(max(self.nws, 16), dtype=torch.uint8, device=dev)

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_fwht_quantize', self.x.data_ptr(), L.BF16, self.M, self.K, self.signs.data_ptr(), None, 1.0, self.K,
           L.INT8, self.xq.data_ptr(), self.sa.data_ptr(), self.stream)
    self.kernel(i)

  def kernel(self, i=0):
    L = self.L
    L.call('qwix_hip_qgemm_grouped_ws', self.xq.data_ptr(), self.K, self.b.data_ptr(), self.K // 2, L.INT4, self.M, self.N,
           self.K, 128, self.sa.data_ptr(), L.BF16, 1, self.sb.data_ptr(), L.BF16, self.out.data_ptr(), L.BF16, self.N, 0,
           None, self.ws.data_ptr() if self.nws else None, self.nws, self.stream)

  def work_per_step(self):
    return 2.0 * self.M * self.N * self.K

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'M': self.M, 'K': self.K, 'N': self.N, 'group': 128}


class HadamardQdotDecode(HadamardQdot):
  """C5 at a decode batch: the weight (int4 values + group scales) is streamed once per step, so the step is HBM-bound;
  the figure is bytes of weights, scales, activations and outputs per second."""

  bound = 'hbm'

  def __init__(self, name, M, K, N):
    super().__init__(name, M, K, N)
    self.metric = 'Hadamard-rotated a8w4 g128 decode GB/s (FWHT + activation quantize included)'
    self.unit = 'GB/s'
    self.kernel_name = 'qgemm_grouped_decode_kernel'

  def work_per_step(self):
    return self.K * self.N / 2 + (self.K // 128) * self.N * 2 + self.M * self.K * 2 + self.M * self.N * 2

  def kernel_work(self):
    return self.K * self.N / 2 + (self.K // 128) * self.N * 2 + self.M * self.K + self.M * self.N * 2

  def cpu_baseline(self, *a, **k):
    return None


class QdotSubChannel(Workload):
  """Sub-channel w8a8: per-token, per-group activation quantize each step (groups of `group` along K), then the
  sub-channel GEMM against a weight with one scale per group and output channel; qtype int8 or e4m3."""

  bound = 'mfma'

  def __init__(self, name, M, K, N, group, qtype):
    self.name, self.M, self.K, self.N, self.group, self.qtype = name, M, K, N, group, qtype
    self.dtype = 'int8' if qtype == 'int8' else 'f8e4m3'
    self.metric = self.dtype + ' sub-channel qdot TOPS (group %d on both operands, activation quantize included)' % group
    self.unit = 'TOPS'
    self.kernel_name = 'qgemm_grouped_dma_kernel'

  def setup(self, dev):
    import torch
    from qwix_amd.core import qarray
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(3100 + self.M)
    self.x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
    w = (torch.randn(self.K, self.N, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
    wq = qarray.quantize(w, qarray.HowToQuantize(qtype=self.qtype, channelwise_axes=[1], tiled_axes={0: self.group}))
    del w
    self.b = wq.qvalue.permute(1, 0)
    assert self.b.is_contiguous()
    self.sb = wq.scale.contiguous()           # (K / group, N)
    self.ga = self.K // self.group
    self.xq = torch.empty(self.M, self.K, dtype=wq.qvalue.dtype, device=dev)
    self.sa = torch.empty(self.M, self.ga, dtype=torch.bfloat16, device=dev)
    self.out = torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev)
    self.qt = L.INT8 if self.qtype == 'int8' else L.E4M3
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_quantize', self.x.data_ptr(), L.BF16, self.M, self.K, 1, self.group, self.qt, L.ABSMAX, 0.0,
           L.LAYOUT_NATURAL, self.xq.data_ptr(), self.sa.data_ptr(), None, None, 0, self.stream)
    self.kernel(i)

  def kernel(self, i=0):
    L = self.L
    L.call('qwix_hip_qgemm_grouped', self.xq.data_ptr(), self.K, self.b.data_ptr(), self.K, self.qt, self.M, self.N,
           self.K, self.group, self.sa.data_ptr(), L.BF16, self.ga, self.sb.data_ptr(), L.BF16, self.out.data_ptr(),
           L.BF16, self.N, 0, None, self.stream)

  def work_per_step(self):
    return 2.0 * self.M * self.N * self.K

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'M': self.M, 'K': self.K, 'N': self.N, 'group': self.group, 'qtype': self.qtype}


class RaggedQdot(Workload):
  """Mixture-of-experts matmul: the tokens are sorted by expert (uneven groups, sizes in device memory);
  per-token int8 activation quantize + one ragged MFMA GEMM against G per-channel int8 expert weights."""

  bound = 'mfma'

  def __init__(self, name, M, K, N, G, qtype='int8'):
    self.name, self.M, self.K, self.N, self.G, self.qtype = name, M, K, N, G, qtype
    self.dtype = 'int8' if qtype == 'int8' else 'f8e4m3'
    self.metric = self.dtype + ' ragged qdot TOPS (w8a8 mixture-of-experts matmul, activation quantize included)'
    self.unit = 'TOPS'
    big = M // G >= 768 and ((M + 255) // 256) * ((N + 255) // 256) >= 192 and K >= 256
    self.kernel_name = 'qgemm_ragged_pp_kernel' if big else 'qgemm_ragged_dma_kernel'
    # Few tokens per expert: the operations per byte of expert weights fall below the machine balance
    # (peak MFMA rate / peak HBM rate), and the roofline that bounds the kernel is the memory one.
    if 2.0 * M * N * K / self.kernel_bytes() < PEAK_MFMA_TOPS * 1e12 / (PEAK_HBM_GBS * 1e9):
      self.roofline_bound = 'hbm'

  def kernel_bytes(self):
    """Every expert's weights and scales once, the quantized activations in, the bf16 results out."""
    return float(self.G * self.N * self.K + self.G * self.N * 2 + self.M * self.K + self.M * 2 + self.M * self.N * 2)

  def roofline_work(self):
    switched = self.bound == 'mfma' and getattr(self, 'roofline_bound', self.bound) == 'hbm'
    return self.kernel_bytes() if switched else self.kernel_work()

  def setup(self, dev):
    import numpy as np
    import torch
    from qwix_amd.core import qarray
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(5000 + self.G)
    self.x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
    # expert weights, quantized once per (expert, output channel) and kept K-contiguous: (G, N, K)
    self.b = torch.empty(self.G, self.N, self.K, dtype=torch.int8 if self.qtype == 'int8' else torch.float8_e4m3fn, device=dev)
    self.sb = torch.empty(self.G, self.N, dtype=torch.bfloat16, device=dev)
    for e in range(self.G):
      w = (torch.randn(self.K, self.N, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
      wq = qarray.quantize(w, qarray.HowToQuantize(qtype=self.qtype, channelwise_axes=[1]))
      self.b[e].copy_(wq.qvalue.permute(1, 0))
      self.sb[e].copy_(wq.scale.reshape(-1))
    # uneven routing: sizes drawn around M / G, every token assigned
    r = np.random.Generator(np.random.PCG64(17)).dirichlet(np.full(self.G, 8.0))
    sizes = np.floor(r * self.M).astype(np.int64)
    sizes[-1] += self.M - sizes.sum()
    self.sizes_host = sizes.tolist()
    self.sizes = torch.tensor(self.sizes_host, dtype=torch.int32, device=dev)
    self.xq = torch.empty(self.M, self.K, dtype=self.b.dtype, device=dev)
    self.sa = torch.empty(self.M, dtype=torch.bfloat16, device=dev)
    self.out = torch.empty(self.M, self.N, dtype=torch.bfloat16, device=dev)
    self.qt = L.INT8 if self.qtype == 'int8' else L.E4M3
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_quantize', self.x.data_ptr(), L.BF16, self.M, self.K, 1, self.K, self.qt, L.ABSMAX, 0.0,
           L.LAYOUT_NATURAL, self.xq.data_ptr(), self.sa.data_ptr(), None, None, 0, self.stream)
    self.kernel(i)

  def kernel(self, i=0):
    L = self.L
    L.call('qwix_hip_qgemm_ragged', self.xq.data_ptr(), self.K, self.b.data_ptr(), self.K, self.N * self.K, self.qt,
           self.M, self.N, self.K, self.sizes.data_ptr(), self.G, self.sa.data_ptr(), L.BF16, self.sb.data_ptr(),
           L.BF16, self.N, L.BF16, self.out.data_ptr(), L.BF16, self.N, self.stream)

  def work_per_step(self):
    return 2.0 * self.M * self.N * self.K

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'tokens': self.M, 'K': self.K, 'N': self.N, 'experts': self.G,
            'group_sizes': f'uneven, {min(self.sizes_host)}..{max(self.sizes_host)} rows (device memory)',
            'weight': 'per-expert per-output-channel ' + self.qtype + ' (pre-quantized)', 'out': 'bf16'}


class RaggedDecode(RaggedQdot):
  """Mixture-of-experts decode: a few tokens per expert, so the step is bound by reading every expert's
  weight once; reported as the bytes of weights (+ activations, outputs) per second."""

  bound = 'hbm'

  def __init__(self, name, M, K, N, G):
    super().__init__(name, M, K, N, G, 'int8')
    self.metric = 'ragged qdot GB/s (w8a8 mixture-of-experts decode, weight streaming, activation quantize included)'
    self.unit = 'GB/s'
    self.kernel_name = 'qgemm_ragged_skinny_kernel'

  def work_per_step(self):
    return float(self.G * self.N * self.K + self.M * self.K * 3 + self.M * self.N * 2 + self.G * self.N * 2)

  def kernel_work(self):
    return float(self.G * self.N * self.K + self.M * self.K + self.M * self.N * 2 + self.G * self.N * 2)


class QuantizeStatic(Workload):
  """Static-range activation quantization: the scale was computed offline, one read and one write."""

  bound = 'hbm'

  def __init__(self, name, M, K):
    self.name, self.M, self.K = name, M, K
    self.dtype = 'bf16->int8'
    self.metric = 'quantize GB/s (static range, per-tensor scale, bf16 -> int8)'
    self.unit = 'GB/s'
    self.kernel_name = 'rows_kernel'

  def setup(self, dev):
    import torch
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(11)
    self.x = torch.randn(self.M, self.K, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
    self.scale = (self.x.abs().max().float() / 127.5).to(torch.bfloat16).reshape(1)
    self.q = torch.empty(self.M, self.K, dtype=torch.int8, device=dev)
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    # one scale for the whole array: outer = 1, every element in one reduce group
    L.call('qwix_hip_quantize_with_scale', self.x.data_ptr(), L.BF16, 1, self.M * self.K, 1, self.M * self.K, L.INT8,
           self.scale.data_ptr(), None, L.LAYOUT_NATURAL, self.q.data_ptr(), self.stream)

  kernel = step

  def work_per_step(self):
    return float(self.M * self.K * 3)

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'M': self.M, 'K': self.K, 'scale': 'per-tensor, precomputed'}


class QuantizeBlocks(Workload):
  """PTQ of a (K, N) weight with one scale per 128 x 128 block (tiles on both axes), natural layout."""

  bound = 'hbm'

  def __init__(self, name, K, N, qtype, block=128):
    self.name, self.K, self.N, self.qtype, self.block = name, K, N, qtype, block
    self.dtype = 'bf16->' + qtype
    self.metric = 'weight quantize GB/s (absmax per %dx%d block, bf16 -> %s)' % (block, block, qtype)
    self.unit = 'GB/s'
    self.kernel_name = 'blocks_kernel'

  def setup(self, dev):
    import ctypes
    import torch
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(13)
    self.w = (torch.randn(self.K, self.N, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
    self.q = torch.empty(self.K, self.N, dtype=torch.uint8, device=dev)
    self.s = torch.empty(self.K // self.block, self.N // self.block, dtype=torch.bfloat16, device=dev)
    self.qt = {'int8': L.INT8, 'float8_e4m3fn': L.E4M3}[self.qtype]
    self.dims = (ctypes.c_int64 * 5)(1, self.K, 1, self.N, 1)
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_quantize_generic', self.w.data_ptr(), L.BF16, self.dims, self.block, self.block, self.qt,
           L.ABSMAX, 0.0, self.q.data_ptr(), self.s.data_ptr(), None, self.stream)

  kernel = step

  def work_per_step(self):
    return self.K * self.N * 3.0 + self.s.numel() * 2.0

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'K': self.K, 'N': self.N, 'block': self.block, 'qtype': self.qtype}


class QdotZeroPoint(QdotW8A8):
  """w8a8 with an asymmetric (minmax) int8 activation: quantize with zero point, K-sums of the weight rows,
  GEMM with the zero-point correction in the epilogue."""

  def __init__(self, name, M, K, N):
    super().__init__(name, M, K, N, 'int8')
    self.metric = 'int8 qdot TOPS (asymmetric activation, zero-point correction, activation quantize included)'

  def setup(self, dev):
    import torch
    super().setup(dev)
    self.x = (self.x.float() + 0.5).to(torch.bfloat16)  # a shifted distribution, as minmax is meant for
    self.zp = torch.empty(self.M, dtype=torch.int8, device=dev)
    self.zu = torch.empty(self.M, dtype=torch.int32, device=dev)
    self.zv = torch.empty(self.N, dtype=torch.int32, device=dev)
    L = self.L
    L.call('qwix_hip_ksum_i8', self.b.data_ptr(), self.K, self.N, self.K, self.zv.data_ptr(), self.stream)  # weights: once

  def step(self, i=0):
    L = self.L
    L.call('qwix_hip_quantize', self.x.data_ptr(), L.BF16, self.M, self.K, 1, self.K, self.qt, L.MINMAX, 0.0,
           L.LAYOUT_NATURAL, self.xq.data_ptr(), self.sa.data_ptr(), self.zp.data_ptr(), None, 0, self.stream)
    self.zu.copy_(self.zp)  # int8 -> int32 zero points (M values)
    self.kernel(i)

  def kernel(self, i=0):
    L = self.L
    L.call('qwix_hip_qgemm_zp', self.xq.data_ptr(), self.K, self.b.data_ptr(), self.K, self.M, self.N, self.K,
           self.sa.data_ptr(), L.BF16, self.sb.data_ptr(), L.BF16, self.zu.data_ptr(), self.zv.data_ptr(),
           self.out.data_ptr(), L.BF16, self.N, self.stream)

  def cpu_baseline(self, *a, **k):
    return None


class QdotBatched(Workload):
  """Batch axes of dot_general in one launch: 'bqd,bkd->bqk' with int8 operands (attention scores).  With
  d = 128 the output write dominates: an HBM-bound contraction."""

  bound = 'hbm'

  def __init__(self, name, B, Q, Kv, D):
    self.name, self.B, self.Q, self.Kv, self.D = name, B, Q, Kv, D
    self.dtype = 'int8'
    self.metric = 'batched int8 qdot GB/s (bqd,bkd->bqk, bf16 out)'
    self.unit = 'GB/s'
    self.kernel_name = 'qgemm_batched_dma_kernel'

  def setup(self, dev):
    import torch
    L = _lib()
    g = torch.Generator(device='cpu').manual_seed(21)
    B, Q, Kv, D = self.B, self.Q, self.Kv, self.D
    self.a = torch.randint(-127, 128, (B, Q, D), generator=g, dtype=torch.int8).to(dev)
    self.b = torch.randint(-127, 128, (B, Kv, D), generator=g, dtype=torch.int8).to(dev)
    self.sa = (torch.rand(B, Q, generator=g) * 0.01 + 0.001).to(torch.bfloat16).to(dev)
    self.sb = (torch.rand(B, Kv, generator=g) * 0.01 + 0.001).to(torch.bfloat16).to(dev)
    self.out = torch.empty(B, Q, Kv, dtype=torch.bfloat16, device=dev)
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    L = self.L
    B, Q, Kv, D = self.B, self.Q, self.Kv, self.D
    L.call('qwix_hip_qgemm_batched', self.a.data_ptr(), D, Q * D, self.b.data_ptr(), D, Kv * D, L.INT8, B, Q, Kv, D,
           self.sa.data_ptr(), L.BF16, Q, self.sb.data_ptr(), L.BF16, Kv, 0, self.out.data_ptr(), L.BF16, Kv, Q * Kv,
           self.stream)

  kernel = step

  def work_per_step(self):
    B, Q, Kv, D = self.B, self.Q, self.Kv, self.D
    return float(B * (Q * D + Kv * D + 2 * (Q + Kv) + 2 * Q * Kv))

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'batch': self.B, 'q': self.Q, 'k': self.Kv, 'd': self.D,
            'ops': 2.0 * self.B * self.Q * self.Kv * self.D}


class PtqMlpGraph(Workload):
  """The reference's own example configuration (MLP 1024 -> 4096 -> 1024 on 256 tokens, int8 weights and
  activations) through the provider surface: four small kernels per forward, launch-bound.  The forward is
  captured once into a HIP graph and replayed; the eager time of the same forward is reported beside it."""

  bound = 'mfma'

  def __init__(self, name):
    self.name = name
    self.dtype = 'int8'
    self.metric = 'PTQ MLP forward TOPS (int8 w8a8 through the provider, HIP graph replay)'
    self.unit = 'TOPS'
    self.kernel_name = 'graph'
    self.ops = 2.0 * 2 * 256 * 1024 * 4096

  def setup(self, dev):
    import torch
    import qwix_amd
    from qwix_amd import nn
    model = nn.MLP(4096, 1024)
    g = torch.Generator().manual_seed(1001)
    params = model.init(g, 1024, torch.float32, dev)
    self.x = torch.rand(256, 1024, generator=g, dtype=torch.float32).to(dev)
    rules = [qwix_amd.QuantizationRule(module_path='.*', weight_qtype='int8', act_qtype='int8')]
    self.model = qwix_amd.quantize_model(model, qwix_amd.PtqProvider(rules))
    self.qparams = qwix_amd.quantize_params(params, self.model.init(params, self.x))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
      for _ in range(3):
        self.model.apply(self.qparams, self.x)
    torch.cuda.current_stream().wait_stream(side)
    self.graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(self.graph):
      self.out = self.model.apply(self.qparams, self.x)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(200):
      self.model.apply(self.qparams, self.x)
    torch.cuda.synchronize()
    self.eager_us = (time.perf_counter() - t0) / 200 * 1e6

  def step(self, i=0):
    self.graph.replay()

  kernel = step

  def work_per_step(self):
    return self.ops

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'tokens': 256, 'layers': '1024 -> 4096 -> 1024', 'weights': 'int8 per channel',
            'activations': 'int8 per token, quantized on the fly', 'eager_us_per_forward': round(self.eager_us, 1)}


class MfmaCeiling(Workload):
  """What the matrix cores sustain with given operand bytes and no memory traffic: MFMAs back to back on register
  operands (`qwix_hip_mfma_ceiling`), every launch about 10 ms.  `data`: 'zeros'; 'gauss30' (int8 N(0, 30^2) bytes, the
  same bytes read as e4m3 for fp8); 'operands' (the quantized activations and weights of the 4096^2 w8a8 workload of
  that type: per-token / per-channel absmax of bf16 N(0,1) and N(0,0.02))."""

  bound = 'mfma'
  ITERS = 10000

  def __init__(self, name, qtype, data):
    self.name, self.qtype, self.data = name, qtype, data
    self.dtype = 'int8' if qtype == 'int8' else 'f8e4m3'
    self.metric = ('int8' if qtype == 'int8' else 'fp8') + ' MFMA rate on register operands (no memory traffic): ' + data
    self.unit = 'TOPS'
    self.kernel_name = 'mfma_ceiling_kernel'

  def setup(self, dev):
    import torch
    from qwix_amd.core import qarray
    L = _lib()
    n = 1 << 24
    g = torch.Generator(device='cpu').manual_seed(77)
    if self.data == 'zeros':
      self.a = torch.zeros(n, dtype=torch.uint8, device=dev)
      self.b = torch.zeros(n, dtype=torch.uint8, device=dev)
    elif self.data == 'gauss30':
      mk = lambda: torch.randn(n, generator=g).mul_(30.0).round_().clamp_(-126, 126).to(torch.int8).view(torch.uint8).to(dev)
      self.a, self.b = mk(), mk()
    else:
      x = torch.randn(4096, 4096, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
      w = (torch.randn(4096, 4096, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16).to(dev)
      xq = qarray.quantize(x, qarray.HowToQuantize(qtype=self.qtype, channelwise_axes=[0]))
      wq = qarray.quantize(w, qarray.HowToQuantize(qtype=self.qtype, channelwise_axes=[1]))
      self.a = xq.qvalue.contiguous().view(torch.uint8).reshape(-1)
      self.b = wq.qvalue.permute(1, 0).contiguous().view(torch.uint8).reshape(-1)
    self.sink = torch.zeros(1, dtype=torch.int32, device=dev)
    self.qt = L.INT8 if self.qtype == 'int8' else L.E4M3
    self.ops = float(L.load().qwix_hip_mfma_ceiling_ops(self.ITERS))
    self.stream = torch.cuda.current_stream().cuda_stream
    self.L = L

  def step(self, i=0):
    self.L.call('qwix_hip_mfma_ceiling', self.a.data_ptr(), self.a.numel(), self.b.data_ptr(), self.b.numel(), self.qt,
                self.ITERS, self.sink.data_ptr(), self.stream)

  kernel = step

  def work_per_step(self):
    return self.ops

  kernel_work = work_per_step

  def describe(self):
    return {'workload': self.name, 'operand_bytes': self.data, 'iterations': self.ITERS, 'workgroups': 256, 'wavefronts_per_workgroup': 8}


WORKLOADS = {
    'quantize_act_8192': lambda: QuantizeRows('quantize_act_8192', 8192, 8192, 'int8'),
    'c3_int8_w8a8_4096': lambda: QdotW8A8('c3_int8_w8a8_4096', 4096, 4096, 4096, 'int8'),
    'c4_fp8_w8a8_ffn': lambda: QdotW8A8('c4_fp8_w8a8_ffn', 8192, 8192, 28672, 'float8_e4m3fn'),
    'c3_fp8_w8a8_4096': lambda: QdotW8A8('c3_fp8_w8a8_4096', 4096, 4096, 4096, 'float8_e4m3fn'),
    'c3_int8_w8a8_8192': lambda: QdotW8A8('c3_int8_w8a8_8192', 8192, 8192, 8192, 'int8'),
    'quantize_act_4096': lambda: QuantizeRows('quantize_act_4096', 4096, 4096, 'int8'),
    'quantize_act_8192_fp8': lambda: QuantizeRows('quantize_act_8192_fp8', 8192, 8192, 'float8_e4m3fn'),
    'w8a8_decode_m16': lambda: QdotDecode('w8a8_decode_m16', 16, 4096, 14336),
    'w8a8_decode_m64': lambda: QdotDecode('w8a8_decode_m64', 64, 4096, 14336, 'qgemm_dma_kernel'),
    'w8a8_decode_m64_k8192': lambda: QdotDecode('w8a8_decode_m64_k8192', 64, 8192, 28672, 'qgemm_mid_kernel'),
    'w8a8_decode_m16_k2048': lambda: QdotDecode('w8a8_decode_m16_k2048', 16, 2048, 8192),
    'w8a8_decode_m16_k2048_fused': lambda: QdotDecodeFused('w8a8_decode_m16_k2048_fused', 16, 2048, 8192),
    'c2_gemv_w4_m1': lambda: GemvW4('c2_gemv_w4_m1', 1, 4096, 14336, 128),
    'c2_gemv_w4_m16': lambda: GemvW4('c2_gemv_w4_m16', 16, 4096, 14336, 128),
    'c2_gemv_w4_m32': lambda: GemvW4('c2_gemv_w4_m32', 32, 4096, 14336, 128),
    'w8a16_gemv_m1': lambda: GemvW4('w8a16_gemv_m1', 1, 4096, 14336, 128, 'int8'),
    'w8a16_gemv_m16': lambda: GemvW4('w8a16_gemv_m16', 16, 4096, 14336, 128, 'int8'),
    'c2_w4a16_prefill_m2048': lambda: WeightOnlyPrefill('c2_w4a16_prefill_m2048', 2048, 4096, 14336, 128),
    'c2_w4a16_prefill_m512': lambda: WeightOnlyPrefill('c2_w4a16_prefill_m512', 512, 4096, 14336, 128),
    'c2_w4a16_prefill_m128': lambda: WeightOnlyPrefill('c2_w4a16_prefill_m128', 128, 4096, 14336, 128),
    'c2_w4a16_prefill_m128_down': lambda: WeightOnlyPrefill('c2_w4a16_prefill_m128_down', 128, 14336, 4096, 128),
    'c4_quantize_weight_fp8': lambda: QuantizeWeight('c4_quantize_weight_fp8', 8192, 28672, 'float8_e4m3fn'),
    'c5_quantize_weight_int4_g128': lambda: QuantizeWeight('c5_quantize_weight_int4_g128', 8192, 8192, 'int4', 128),
    'c3_quantize_weight_int8': lambda: QuantizeWeight('c3_quantize_weight_int8', 4096, 4096, 'int8'),
    'c5_fwht_quantize_act': lambda: FwhtQuantize('c5_fwht_quantize_act', 2048, 8192),
    'fwht_quantize_8192x8192': lambda: FwhtQuantize('fwht_quantize_8192x8192', 8192, 8192),
    'plain_copy_1g': lambda: PlainCopy('plain_copy_1g', 1 << 30),
    'moe_ragged_int8_8x1024': lambda: RaggedQdot('moe_ragged_int8_8x1024', 8192, 4096, 14336, 8),
    'moe_ragged_int8_64x128': lambda: RaggedQdot('moe_ragged_int8_64x128', 8192, 2048, 4096, 64),
    'moe_decode_int8_64x4': lambda: RaggedDecode('moe_decode_int8_64x4', 256, 2048, 4096, 64),
    'moe_ragged_fp8_8x1024': lambda: RaggedQdot('moe_ragged_fp8_8x1024', 8192, 4096, 14336, 8, 'float8_e4m3fn'),
    'quantize_weight_fp8_block128': lambda: QuantizeBlocks('quantize_weight_fp8_block128', 4096, 14336, 'float8_e4m3fn'),
    'srq_quantize_act_4096': lambda: QuantizeStatic('srq_quantize_act_4096', 4096, 4096),
    'zp_int8_w8a8_4096': lambda: QdotZeroPoint('zp_int8_w8a8_4096', 4096, 4096, 4096),
    'batched_qk_int8_32x2048': lambda: QdotBatched('batched_qk_int8_32x2048', 32, 2048, 2048, 128),
    'c1_ptq_mlp_graph': lambda: PtqMlpGraph('c1_ptq_mlp_graph'),
    'c5_hadamard_a8w4': lambda: HadamardQdot('c5_hadamard_a8w4', 2048, 8192, 8192),
    'c5_hadamard_a8w4_m128': lambda: HadamardQdot('c5_hadamard_a8w4_m128', 128, 8192, 8192),
    'c5_hadamard_a8w4_decode_m16': lambda: HadamardQdotDecode('c5_hadamard_a8w4_decode_m16', 16, 8192, 8192),
    'int8_subchannel_g128_4096': lambda: QdotSubChannel('int8_subchannel_g128_4096', 4096, 4096, 4096, 128, 'int8'),
    'fp8_subchannel_g128_4096': lambda: QdotSubChannel('fp8_subchannel_g128_4096', 4096, 4096, 4096, 128, 'float8_e4m3fn'),
    'mfma_ceiling_int8_zeros': lambda: MfmaCeiling('mfma_ceiling_int8_zeros', 'int8', 'zeros'),
    'mfma_ceiling_int8_gauss30': lambda: MfmaCeiling('mfma_ceiling_int8_gauss30', 'int8', 'gauss30'),
    'mfma_ceiling_int8_operands': lambda: MfmaCeiling('mfma_ceiling_int8_operands', 'int8', 'operands'),
    'mfma_ceiling_fp8_zeros': lambda: MfmaCeiling('mfma_ceiling_fp8_zeros', 'float8_e4m3fn', 'zeros'),
    'mfma_ceiling_fp8_gauss30': lambda: MfmaCeiling('mfma_ceiling_fp8_gauss30', 'float8_e4m3fn', 'gauss30'),
    'mfma_ceiling_fp8_operands': lambda: MfmaCeiling('mfma_ceiling_fp8_operands', 'float8_e4m3fn', 'operands'),
}
# The measured matrix-core ceilings: run first, so that every MFMA-bound line can carry `frac_of_ceiling`.
CEILINGS = {'int8': 'mfma_ceiling_int8_operands', 'f8e4m3': 'mfma_ceiling_fp8_operands'}
CEILING_EXTRA = ['mfma_ceiling_int8_zeros', 'mfma_ceiling_int8_gauss30', 'mfma_ceiling_int8_operands',
                 'mfma_ceiling_fp8_zeros', 'mfma_ceiling_fp8_gauss30', 'mfma_ceiling_fp8_operands']
DEFAULT = 'c3_int8_w8a8_4096'
EXTRA = ['quantize_act_4096', 'quantize_act_8192', 'quantize_act_8192_fp8', 'c4_quantize_weight_fp8', 'c5_quantize_weight_int4_g128', 'c3_int8_w8a8_8192', 'c4_fp8_w8a8_ffn', 'c2_gemv_w4_m1', 'c2_gemv_w4_m16', 'c2_gemv_w4_m32', 'w8a16_gemv_m1', 'w8a16_gemv_m16', 'c2_w4a16_prefill_m2048', 'c2_w4a16_prefill_m512', 'c2_w4a16_prefill_m128', 'c2_w4a16_prefill_m128_down', 'w8a8_decode_m16', 'w8a8_decode_m64', 'w8a8_decode_m64_k8192', 'w8a8_decode_m16_k2048', 'w8a8_decode_m16_k2048_fused',
         'c5_hadamard_a8w4', 'c5_hadamard_a8w4_m128', 'c5_hadamard_a8w4_decode_m16', 'c5_fwht_quantize_act', 'fwht_quantize_8192x8192', 'int8_subchannel_g128_4096', 'fp8_subchannel_g128_4096', 'moe_ragged_int8_8x1024',
         'moe_ragged_int8_64x128', 'moe_decode_int8_64x4', 'quantize_weight_fp8_block128', 'srq_quantize_act_4096', 'zp_int8_w8a8_4096', 'batched_qk_int8_32x2048', 'c1_ptq_mlp_graph']


def _blas_threads() -> int:
  try:
    from threadpoolctl import threadpool_info
    n = [p.get('num_threads', 0) for p in threadpool_info() if p.get('user_api') == 'blas']
    if n:
      return int(max(n))
  except Exception:
    pass
  return int(os.environ.get('OMP_NUM_THREADS', os.cpu_count() or 1))


REPEATS = 7               # the timed region (exactly `steps` steps) is repeated; the median is reported


def run(wl: Workload, steps: int, warmup: int, spin_up: float = None, repeats: int = REPEATS):
  """Returns (seconds per step, seconds per launch of the dominant kernel, timing summary).

  Both figures are medians over `repeats` repetitions of a timed region of exactly `steps` steps, each
  bracketed by a device synchronisation on both sides: a single region of 50 x 80 us is 4 ms, short enough
  for one clock excursion to decide it."""
  import torch
  dev = torch.device('cuda:0')
  wl.setup(dev)
  # Untimed warm-up: the requested steps, and at least SPIN_UP_S seconds of them -- the first few hundred
  # milliseconds of GPU work after process start run at a lower clock than steady state.
  t_start = time.perf_counter()
  i = 0
  spin_up = SPIN_UP_S if spin_up is None else spin_up
  while i < warmup or time.perf_counter() - t_start < spin_up:
    wl.step(i)
    i += 1
    if i % 16 == 0:
      torch.cuda.synchronize()
  torch.cuda.synchronize()
  step_t = []
  for _ in range(repeats):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
      wl.step(i)
    torch.cuda.synchronize()
    step_t.append((time.perf_counter() - t0) / steps)
  # the dominant kernel alone, on the inputs the last step left behind
  e0, e1 = _events(2)
  for i in range(min(warmup, 3)):
    wl.kernel(i)
  kern_t = []
  for _ in range(repeats):
    torch.cuda.synchronize()
    e0.record()
    for i in range(steps):
      wl.kernel(i)
    e1.record()
    torch.cuda.synchronize()
    kern_t.append(e0.elapsed_time(e1) * 1e-3 / steps)
  med = lambda v: sorted(v)[len(v) // 2]
  timing = {'repeats': repeats, 'step_ms_min': round(min(step_t) * 1e3, 5), 'step_ms_median': round(med(step_t) * 1e3, 5),
            'step_ms_max': round(max(step_t) * 1e3, 5), 'kernel_us_min': round(min(kern_t) * 1e6, 3),
            'kernel_us_median': round(med(kern_t) * 1e6, 3)}
  return med(step_t), med(kern_t), timing


def summarize(wl: Workload, step_s: float, kern_s: float, ceilings: dict = None) -> dict:
  scale = 1e12 if wl.bound == 'mfma' else 1e9
  value = wl.work_per_step() / step_s / scale
  # the roofline that bounds the dominant kernel need not be the one the metric's unit suggests
  rb = getattr(wl, 'roofline_bound', wl.bound)
  peak = getattr(wl, 'peak_tops', PEAK_MFMA_TOPS) if rb == 'mfma' else PEAK_HBM_GBS
  work = wl.roofline_work() if hasattr(wl, 'roofline_work') else wl.kernel_work()
  achieved = work / kern_s / (1e12 if rb == 'mfma' else 1e9)
  roof = {'bound': rb, 'kernel': wl.kernel_name, 'achieved': round(achieved, 2), 'peak': peak,
          'unit': 'TFLOP/s' if rb == 'mfma' else 'GB/s', 'frac': round(achieved / peak, 4),
          'traffic': _traffic(wl.name), **_mfma_util(wl.name)}
  # `frac` stays priced against the nominal peak; `frac_of_ceiling` is the same rate against what the matrix cores
  # sustained in this very run on register operands of this workload's kind (see MfmaCeiling), no memory traffic.
  if rb == 'mfma' and peak == PEAK_MFMA_TOPS and not isinstance(wl, MfmaCeiling):
    c = (ceilings or {}).get(_ceiling_dtype(wl))
    roof['ceiling'] = c
    roof['frac_of_ceiling'] = round(achieved / c, 4) if c else None
  return {'value': round(value, 2), 'unit': wl.unit, 'ms_per_step': round(step_s * 1e3, 5), 'roofline': roof}


def _ceiling_dtype(wl) -> str:
  """The operand type whose matrix-core ceiling prices this workload: int4 weights are widened to int8 in registers
  and multiplied by the int8 instruction."""
  return 'int8' if wl.dtype.startswith('int8') else wl.dtype


def measure_ceilings(dtypes, spin_up) -> tuple:
  """Runs the matrix-core ceiling workloads; returns ({dtype: TOPS on the benchmark's operand bytes}, {name: line})."""
  import torch
  ceilings, lines = {}, {}
  prefixes = tuple(CEILINGS[d].rsplit('_', 1)[0] + '_' for d in dtypes)   # all operand kinds of the wanted types
  names = [n for n in CEILING_EXTRA if n.startswith(prefixes)]
  for name in names:
    w = WORKLOADS[name]()
    s, km, _ = run(w, 3, 1, min(spin_up, 0.2), 3)
    r = summarize(w, s, km)
    lines[name] = {'metric': w.metric, 'value': r['value'], 'unit': r['unit'], 'ms_per_step': r['ms_per_step'],
                   'roofline': r['roofline']}
    for d, n in CEILINGS.items():
      if n == name:
        ceilings[d] = r['roofline']['achieved']
    del w
    torch.cuda.empty_cache()
  return ceilings, lines


def _traffic(name: str):
  """HBM bytes per launch of the dominant kernel, from committed rocprofv3 --pmc measurements."""
  p = os.path.join(ROOT, 'profiles', 'hbm_traffic.json')
  if os.path.exists(p):
    try:
      return json.load(open(p)).get(name)
    except Exception:
      return None
  return None


def _mfma_util(name: str) -> dict:
  """Matrix-core utilisation of the dominant kernel from committed rocprofv3 --pmc measurements
  (SQ_VALU_MFMA_BUSY_CYCLES / SQ_BUSY_CYCLES and friends; profiles/mfma_util.json), {} when not measured."""
  p = os.path.join(ROOT, 'profiles', 'mfma_util.json')
  if os.path.exists(p):
    try:
      v = json.load(open(p)).get(name)
      return {'mfma_util': v} if v is not None else {}
    except Exception:
      return {}
  return {}


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument('--gpus', type=int, default=1)
  ap.add_argument('--steps', type=int, default=50)
  ap.add_argument('--warmup', type=int, default=5)
  ap.add_argument('--workload', default=DEFAULT, choices=sorted(WORKLOADS))
  ap.add_argument('--repeats', type=int, default=REPEATS,
                  help='repetitions of the timed region of --steps steps; the median is reported')
  ap.add_argument('--no-extra', action='store_true', help='skip the other workloads of the metric')
  ap.add_argument('--no-cpu-baseline', action='store_true')
  ap.add_argument('--no-ceiling', action='store_true',
                  help='skip the matrix-core ceiling measurement that roofline.frac_of_ceiling is priced against')
  ap.add_argument('--spin-up', type=float, default=SPIN_UP_S,
                  help='minimum seconds of untimed warm-up (profiling runs shorten it to keep traces small)')
  args = ap.parse_args()
  if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
    print('bench.py: this build runs on ONE GPU only (no collectives, no sharding); re-run with --gpus 1. '
          'The reported value is the single GPU throughput.', file=sys.stderr)
    sys.exit(2)
  import torch
  if not torch.cuda.is_available():
    print('bench.py: no GPU visible; the hot path has no CPU fallback.', file=sys.stderr)
    sys.exit(2)

  wl = WORKLOADS[args.workload]()
  extra_on = not args.no_extra and args.workload == DEFAULT
  ceilings, ceiling_lines = {}, {}
  if not args.no_ceiling and not isinstance(wl, MfmaCeiling):
    want = sorted(CEILINGS) if extra_on else [d for d in CEILINGS if d == _ceiling_dtype(wl) and getattr(wl, 'roofline_bound', wl.bound) == 'mfma']
    if want:
      ceilings, ceiling_lines = measure_ceilings(want, args.spin_up)
  step_s, kmean, timing = run(wl, args.steps, args.warmup, args.spin_up, args.repeats)
  res = summarize(wl, step_s, kmean, ceilings)
  line = {
      'metric': wl.metric, 'value': res['value'], 'unit': res['unit'], 'n_gpus': 1, 'steps': args.steps,
      'warmup': args.warmup, 'ms_per_step': res['ms_per_step'], 'higher_is_better': True, 'scaling': 'weak',
      'vs_baseline': None, 'dtype': wl.dtype, 'data': 'synthetic', 'config': wl.describe(),
      'roofline': res['roofline'], 'timing': timing,
  }
  if not args.no_cpu_baseline and hasattr(wl, 'cpu_baseline'):
    line['cpu_baseline'] = wl.cpu_baseline()
  else:
    line['cpu_baseline'] = None
  if extra_on:
    extra = dict(ceiling_lines)
    for name in EXTRA:
      w = WORKLOADS[name]()
      n = max(5, min(args.steps, 20))
      s, km, _ = run(w, n, 3, args.spin_up, min(args.repeats, 5))
      r = summarize(w, s, km, ceilings)
      extra[name] = {'metric': w.metric, 'value': r['value'], 'unit': r['unit'], 'ms_per_step': r['ms_per_step'],
                     'roofline': r['roofline']}
      del w
      torch.cuda.empty_cache()
    line['extra'] = extra
  print(json.dumps(line))


if __name__ == '__main__':
  main()
