

def test_contraction_to_a_scalar():
  """Operands without free or batch axes contract to a 0-d result (bf16 rounding and reshapes keep the shape ())."""
  x = O.FArr(O.round_to_bf16(np.arange(32, dtype=np.float32) / 7), O.BF16)
  w = O.FArr(O.round_to_bf16(np.arange(32, dtype=np.float32)[::-1] / 9), O.BF16)
  how = O.HowToQuantize(qtype='int8', channelwise_axes=[])
  xq, wq = O.quantize(x, how), O.quantize(w, how)
  out = O.dot_general(xq, wq, (((0,), (0,)), ((), ())))
  assert out.v.shape == () and out.dtype == O.BF16
  acc = int(xq.qvalue.astype(np.int64) @ wq.qvalue.astype(np.int64))
  want = O.round_to_bf16(O.round_to_bf16(O.round_to_bf16(np.float32(acc)) * xq.scale.v.reshape(())) * wq.scale.v.reshape(()))
  assert float(out.v) == float(want)
