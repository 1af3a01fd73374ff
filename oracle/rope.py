"""Rotary embedding of the step's keys, restated (test infrastructure).

Follows apply_rotary_emb / reshape_for_broadcast, jetstream_pt/layers.py:349-379:
x (batch, seqlen, heads, dim) is viewed as complex pairs (2i, 2i+1), multiplied
by freqs_cis (batch, seqlen, dim / 2) complex64 broadcast over heads, all in
float32, and cast back to the dtype of x.

`rotate` spells the complex product out with real float32 ops, one rounding per
op and no fused multiply-add: re = a*c - b*d, im = a*d + b*c.  That op order is
the canonical one the HIP kernels follow bit for bit.  Pinned by
tests/test_oracle_rope.py: against torch's own complex product (the literal
reference text), against angles whose rotation is known in closed form, and by
norm preservation.
"""

import torch


def apply_rotary_emb_literal(xq, xk, freqs_cis):
  """The reference text, run on torch-CPU (layers.py:368-379)."""
  xq_ = torch.view_as_complex(xq.float().reshape(*xq.shape[:-1], -1, 2))
  xk_ = torch.view_as_complex(xk.float().reshape(*xk.shape[:-1], -1, 2))
  shape = [d if i == 1 or i == xq_.ndim - 1 else 1 for i, d in enumerate(xq_.shape)]
  shape[0] = xq_.shape[0]
  f = freqs_cis.view(*shape)  # reshape_for_broadcast, layers.py:349-365
  xq_out = torch.view_as_real(xq_ * f).flatten(3)
  xk_out = torch.view_as_real(xk_ * f).flatten(3)
  return xq_out.type_as(xq), xk_out.type_as(xk)


def rotate(x, freqs_cis):
  """x (batch, seqlen, heads, dim) -> same shape and dtype, rotated."""
  a, b = x.float()[..., 0::2], x.float()[..., 1::2]
  c = torch.view_as_real(freqs_cis)[..., 0].unsqueeze(2)  # (batch, seqlen, 1, dim/2)
  d = torch.view_as_real(freqs_cis)[..., 1].unsqueeze(2)
  re = (a * c) - (b * d)
  im = (a * d) + (b * c)
  return torch.stack((re, im), dim=-1).flatten(3).to(x.dtype)


def precompute_freqs_cis(dim, end, theta=10000.0):
  """third_party/llama/model_exportable.py:199-211 without rope scaling."""
  freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: (dim // 2)].float() / dim))
  t = torch.arange(end, dtype=torch.float32)
  freqs = torch.outer(t, freqs)
  return torch.polar(torch.ones_like(freqs), freqs)
