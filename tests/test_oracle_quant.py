"""Pins oracle.quant (both int8 KV quantisers) to bit-level closed forms that
do not use torch's bf16 arithmetic: bf16 rounding is redone here on the raw
bits, divisions are done in float64 and rounded once to float32 (exact for
float32 operands by the double-rounding theorem, 53 >= 2*24+2)."""

import numpy as np
import pytest
import torch

from oracle import quant


def bf16_round(x32):
  """float32 -> nearest-even bf16, returned as float32 (numpy, bit level)."""
  u = np.asarray(x32, dtype=np.float32).view(np.uint32).astype(np.uint64)
  u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
  return u.astype(np.uint32).view(np.float32)


def f32_div(a, b):
  return (np.asarray(a, dtype=np.float64) / np.asarray(b, dtype=np.float64)).astype(np.float32)


def closed_form_decode(x32, bf16):
  """x32: (B, H, 1, D) float32 holding bf16-representable values."""
  r = bf16_round if bf16 else (lambda v: np.asarray(v, dtype=np.float32))
  a = np.abs(x32).max(axis=(1, 3), keepdims=True)
  s = r(f32_div(a, 127.0))
  q = r(f32_div(x32, s))
  return np.trunc(q).astype(np.int8), s


def closed_form_insert(x32, bf16):
  r = bf16_round if bf16 else (lambda v: np.asarray(v, dtype=np.float32))
  eps = r(np.float32(1e-5))
  a = np.maximum(np.abs(x32).max(axis=(1, 3), keepdims=True), eps)
  s = r(f32_div(a, 127.0))
  inv = r(f32_div(1.0, s))
  q = r((np.asarray(x32, dtype=np.float64) * np.asarray(inv, dtype=np.float64)).astype(np.float32))
  return np.clip(np.rint(q), -128, 127).astype(np.int8), s  # rint = half to even


def rand_tokens(seed, dtype, shape=(64, 4, 1, 32)):
  g = torch.Generator().manual_seed(seed)
  x = torch.randn(shape, generator=g) * torch.logspace(-6, 3, shape[0]).reshape(-1, 1, 1, 1)
  return x.to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_decode_quantiser_closed_form(dtype):
  x = rand_tokens(11, dtype)
  codes, scale = quant.quantize_decode(x)
  want_c, want_s = closed_form_decode(x.float().numpy(), dtype == torch.bfloat16)
  assert scale.dtype == dtype and scale.shape == (64, 1, 1, 1)
  assert np.array_equal(scale.float().numpy(), want_s)
  assert np.array_equal(codes.numpy(), want_c)
  assert int(codes.abs().max()) <= 127


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_insert_quantiser_closed_form(dtype):
  x = rand_tokens(12, dtype)
  x[3] = 0  # all-zero token exercises the epsilon clamp
  codes, scale = quant.quantize_insert(x)
  want_c, want_s = closed_form_insert(x.float().numpy(), dtype == torch.bfloat16)
  assert np.array_equal(scale.float().numpy(), want_s)
  assert np.array_equal(codes.numpy(), want_c)
  assert torch.count_nonzero(codes[3]) == 0


def test_fp32_scale_mode_is_upcast_first():
  x = rand_tokens(13, torch.bfloat16)
  c, s = quant.quantize_decode(x, compute_dtype=torch.float32)
  wc, ws = closed_form_decode(x.float().numpy(), bf16=False)
  assert s.dtype == torch.float32
  assert np.array_equal(c.numpy(), wc) and np.array_equal(s.numpy(), ws)


def test_per_head_scales():
  x = rand_tokens(14, torch.bfloat16, (8, 4, 1, 16))
  c, s = quant.quantize_decode(x, scale_heads=4)
  assert s.shape == (8, 4, 1, 1)
  for h in range(4):
    ch, sh = quant.quantize_decode(x[:, h:h + 1])
    assert torch.equal(c[:, h:h + 1], ch) and torch.equal(s[:, h:h + 1], sh)


def test_exhaustive_bf16_against_fixed_scale():
  """All finite bf16 values that do not exceed the token's absmax, one token."""
  bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
  allv = bits.view(torch.bfloat16)
  amax = torch.tensor(3.140625, dtype=torch.bfloat16)
  keep = torch.isfinite(allv.float()) & (allv.float().abs() <= amax.float())
  x = allv[keep].reshape(1, 1, 1, -1)
  assert x.abs().max() == amax
  c, s = quant.quantize_decode(x)
  wc, ws = closed_form_decode(x.float().numpy(), True)
  assert np.array_equal(c.numpy(), wc) and np.array_equal(s.float().numpy(), ws)
  c2, s2 = quant.quantize_insert(x)
  wc2, _ = closed_form_insert(x.float().numpy(), True)
  assert np.array_equal(c2.numpy(), wc2)
  # properties: sign kept, reconstruction within one step
  xf = x.float()
  assert torch.all((c.float() * xf) >= 0)
  assert torch.all((c.float() * s.float() - xf).abs() <= s.float() * 1.0001)


def test_rounding_modes_differ_as_documented():
  """Truncation vs half-to-even on hand-built ratios (scale 1: absmax 127)."""
  vals = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 0.999, 126.5, -126.5, 3.75]
  x = torch.tensor(vals).reshape(1, 1, 1, -1)
  ct, st = quant.quantize_decode(x)
  ci, si = quant.quantize_insert(x)
  assert st.item() == 1.0 and si.item() == 1.0
  assert ct.flatten().tolist() == [127, 0, 1, 2, 0, -1, -2, 0, 126, -126, 3]
  assert ci.flatten().tolist() == [127, 0, 2, 2, 0, -2, -2, 1, 126, -126, 4]


def test_insert_clamps_at_127():
  # bf16: absmax 1.0 -> s = bf16(1/127) = 0.007873535; inv = bf16(127.0078) = 127
  # so the largest ratio is 127; craft a case where the product rounds to 128
  x = torch.tensor([0.0247, 0.0247 * 0.999], dtype=torch.bfloat16).reshape(1, 1, 1, 2)
  c, _ = quant.quantize_insert(x)
  assert int(c.max()) <= 127 and int(c.min()) >= -128
