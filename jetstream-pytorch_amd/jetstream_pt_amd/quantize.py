"""int8 KV quantisation entry points on the device.

`quantize_kv` is the one-token decode quantiser of Int8KVCacheGenerate
(reference: cache_manager.py:532-537) or, with rounding="rne", the symmetric
int8 branch of quantize_tensor over axes (-3, -1) (reference:
quantize.py:58-75), both run by the fused HIP kernel without touching a cache.
"""

import torch

from . import _ffi


def _rounding_code(rounding):
  if rounding == "trunc":
    return _ffi.ROUND_TRUNC
  if rounding == "rne":
    return _ffi.ROUND_RNE
  raise ValueError(f"rounding must be 'trunc' or 'rne', got {rounding!r}")


def quantize_kv(xk, xv, *, rounding="trunc", scale_heads=1, scale_dtype=None, freqs_cis=None):
  """Quantises one token per slot: xk, xv (batch, heads, 1, dim).

  Returns (k_codes, v_codes, k_scale, v_scale); codes int8 of the input
  shape, scales (batch, scale_heads, 1, 1) in `scale_dtype` (default: the
  input dtype).  With `freqs_cis` (the step's rotary factors, (batch, 1,
  dim / 2) complex64) xk is taken unrotated and apply_rotary_emb
  (jetstream_pt/layers.py:368-379) is applied to it in the same launch.
  """
  _ffi.dev(xk, "xk"), _ffi.dev(xv, "xv")
  b, h, t, d = xk.shape
  if t != 1 or xv.shape != xk.shape:
    raise ValueError(f"expected matching (batch, heads, 1, dim) tensors, got {tuple(xk.shape)} and {tuple(xv.shape)}")
  sdt = scale_dtype or xk.dtype
  kq = torch.empty_like(xk, dtype=torch.int8)
  vq = torch.empty_like(xv, dtype=torch.int8)
  ks = torch.empty((b, scale_heads, 1, 1), dtype=sdt, device=xk.device)
  vs = torch.empty((b, scale_heads, 1, 1), dtype=sdt, device=xk.device)
  args = _ffi.QuantAppendArgs(
      new_k=_ffi.ptr(xk), new_v=_ffi.ptr(xv), out_k=_ffi.ptr(kq), out_v=_ffi.ptr(vq),
      out_k_scale=_ffi.ptr(ks), out_v_scale=_ffi.ptr(vs), pos_count=b, batch=b, heads=h,
      seq=1, dim=d, in_dtype=_ffi.dtype_code(xk.dtype), scale_dtype=_ffi.dtype_code(sdt),
      scale_heads=scale_heads, rounding=_rounding_code(rounding))
  rope = None
  if freqs_cis is not None:
    rope = _ffi.rope_factors(freqs_cis, b, d)
    args.rope = _ffi.ptr(rope)
  _ffi.check(_ffi.lib.jpt_kv_append_quant_i8(args, _ffi.stream()))
  del rope
  return kq, vq, ks, vs
