"""The two int8 KV quantisers of the reference, op for op (test infrastructure).

Each op below is one eager torch-CPU op, so every intermediate is rounded to
the working dtype exactly where the reference rounds it.

`compute_dtype` and `scale_heads` are the two knobs the HIP kernels expose on
top of the reference-literal behaviour:
  * compute_dtype=None  -> work in the input dtype (reference literal);
    torch.float32       -> upcast first, so scale and quotient are fp32.
  * scale_heads=1       -> one scale per token over all heads (reference
    literal, reduce axes (-3, -1)); scale_heads=H -> one scale per head.
"""

import torch

EPS = 1e-5  # quantize.py:21


def _reduce_axes(scale_heads: int, n_heads: int):
  if scale_heads == 1:
    return (-3, -1)
  if scale_heads == n_heads:
    return (-1,)
  raise ValueError(f"scale_heads must be 1 or {n_heads}, got {scale_heads}")


def quantize_decode(val, scale_heads: int = 1, compute_dtype=None):
  """Int8KVCacheGenerate.quantize, cache_manager.py:532-537.

  val is (batch, heads, seqlen, dim).  absmax over (heads, dim), true division
  by 127, true division of the values by the scale, truncating int8 cast.  No
  clamp, no epsilon.  An all-zero token divides 0 by 0; the cast of that NaN is
  backend-defined in the reference, and is defined as code 0 here.
  """
  x = val if compute_dtype is None else val.to(compute_dtype)
  axes = _reduce_axes(scale_heads, x.shape[-3])
  scale = torch.amax(x.abs(), dim=axes, keepdim=True)
  scale = scale / 127
  ratio = x / scale
  ratio = torch.where(torch.isnan(ratio), torch.zeros_like(ratio), ratio)
  return ratio.to(torch.int8), scale


def quantize_insert(w, scale_heads: int = 1, compute_dtype=None):
  """quantize_tensor(w, (-3, -1)), symmetric 8 bit, quantize.py:58-75.

  Called on the prefill K/V at engine.py:429-432.  absmax, clamp to EPS,
  divide by 127, multiply the values by the reciprocal, round half to even,
  clamp to [-128, 127].  Returns (codes, scales); the reference's third
  return value (zero point) is None on this path.
  """
  x = w if compute_dtype is None else w.to(compute_dtype)
  axes = _reduce_axes(scale_heads, x.shape[-3])
  max_val = x.abs().amax(dim=axes, keepdim=True)
  max_val = max_val.clamp(min=EPS)
  scales = max_val / 127
  codes = torch.clamp(torch.round(x * (1.0 / scales) + 0), -128, 127)
  return codes.to(torch.int8), scales


def dequantize(codes, scale):
  """dequantize_tensor, quantize.py:78-83 (symmetric branch)."""
  return codes * scale
