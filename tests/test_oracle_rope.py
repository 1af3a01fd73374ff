"""Pins oracle.rope (layers.py:349-379)."""
import math

import torch

from oracle import rope as orope


def _inputs(dtype, seed=0, b=3, t=2, h=4, d=128):
  g = torch.Generator().manual_seed(seed)
  x = (torch.randn((b, t, h, d), generator=g) * 3).to(dtype)
  pos = torch.randint(0, 4096, (b, t), generator=g)
  table = orope.precompute_freqs_cis(d, 4096)
  return x, table[pos]  # (b, t, d/2) complex64


def test_spelled_out_product_equals_the_reference_text():
  for dtype in (torch.bfloat16, torch.float32):
    x, f = _inputs(dtype)
    lit_q, lit_k = orope.apply_rotary_emb_literal(x, x[:, :, :2], f)
    got = orope.rotate(x, f)
    if dtype == torch.float32:
      # torch's vectorised complex product may round differently in the last place
      assert torch.allclose(got, lit_q, rtol=0, atol=2e-6 * float(x.abs().max()))
    else:
      diff = (got.float() - lit_q.float()).abs()
      ulp = torch.maximum(lit_q.float().abs(), torch.tensor(1e-30)) * 2.0 ** -7
      assert torch.all(diff <= ulp) and (diff > 0).float().mean() < 1e-3
    assert torch.equal(orope.rotate(x[:, :, :2], f), got[:, :, :2])
    assert lit_k.shape == x[:, :, :2].shape


def test_known_angles_and_norm():
  x = torch.arange(1, 9, dtype=torch.float32).reshape(1, 1, 1, 8)
  zero = torch.polar(torch.ones(1, 1, 4), torch.zeros(1, 1, 4))
  assert torch.equal(orope.rotate(x, zero), x)
  quarter = torch.complex(torch.zeros(1, 1, 4), torch.ones(1, 1, 4))  # exactly i
  assert orope.rotate(x, quarter).flatten().tolist() == [-2, 1, -4, 3, -6, 5, -8, 7]
  half = torch.complex(-torch.ones(1, 1, 4), torch.zeros(1, 1, 4))
  assert torch.equal(orope.rotate(x, half), -x)
  y, f = _inputs(torch.float32, seed=5)
  r = orope.rotate(y, f)
  n0 = (y[..., 0::2] ** 2 + y[..., 1::2] ** 2)
  n1 = (r[..., 0::2] ** 2 + r[..., 1::2] ** 2)
  assert torch.allclose(n0, n1, rtol=1e-5)
  # position 0 of the llama table is the identity; the first frequency is one radian per position
  t = orope.precompute_freqs_cis(128, 8)
  assert torch.equal(t[0], torch.ones(64, dtype=torch.complex64))
  assert math.isclose(float(t[1, 0].real), math.cos(1.0), rel_tol=1e-6)
  assert math.isclose(float(t[3, 0].imag), math.sin(3.0), rel_tol=1e-6)
