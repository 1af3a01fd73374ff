"""Pins oracle.attention / oracle.attn_layers to the float64 closed form, to
algebraic identities, and to the one saved paged-attention vector the
reference holds."""

import math

import pytest
import torch

from oracle import Env, quant
from oracle import attention as A
from oracle.attn_layers import AttentionKernel, Int8KVAttentionKernel
from oracle.kv_cache import Int8KVCacheGenerate, KVCacheGenerate


def rnd(g, shape, dtype=torch.bfloat16, scale=1.0):
  return (torch.randn(shape, generator=g) * scale).to(dtype)


def make_int8(g, b, h, s, d):
  k = torch.randint(-127, 128, (b, h, s, d), generator=g, dtype=torch.int8)
  v = torch.randint(-127, 128, (b, h, s, d), generator=g, dtype=torch.int8)
  ks = (torch.rand((b, 1, s, 1), generator=g) * 0.045 + 0.005).to(torch.bfloat16)
  vs = (torch.rand((b, 1, s, 1), generator=g) * 0.045 + 0.005).to(torch.bfloat16)
  return k, v, ks, vs


def test_closed_form_hand_case():
  """Two keys, scores ln(3) apart -> weights 3/4 and 1/4."""
  q = torch.tensor([[[[math.sqrt(2.0) * math.log(3.0), 0.0]]]], dtype=torch.float64)
  k = torch.tensor([[[[1.0, 0.0], [0.0, 1.0]]]], dtype=torch.float64)
  v = torch.tensor([[[[4.0, 0.0], [0.0, 8.0]]]], dtype=torch.float64)
  o, m, l = A.closed_form(q, k, v)
  assert torch.allclose(o, torch.tensor([[[[3.0, 2.0]]]], dtype=torch.float64))
  assert math.isclose(m.item(), math.log(3.0)) and math.isclose(l.item(), 4.0 / 3.0)


@pytest.mark.parametrize("hq,hkv", [(4, 4), (8, 2)])
@pytest.mark.parametrize("quantized", [False, True])
def test_ragged_equals_closed_form(hq, hkv, quantized):
  g = torch.Generator().manual_seed(21)
  b, s, d, bk = 5, 64, 16, 16
  end = torch.tensor([0, 1, 16, 37, 64])
  q = rnd(g, (b, hq, 1, d))
  if quantized:
    k, v, ks, vs = make_int8(g, b, hkv, s, d)
  else:
    k, v, ks, vs = rnd(g, (b, hkv, s, d)), rnd(g, (b, hkv, s, d)), None, None
  o, (m, l) = A.ragged_mha(q, k, v, 0, None, end, None, None, ks, vs, bk=bk)
  rep = hq // hkv
  assert o.shape == (b, hkv, rep, d) and m.shape == (b, hkv, rep)
  wo, wm, wl = A.closed_form(q, k, v, lengths=end, k_scale=ks, v_scale=vs)
  o4, (m4, l4) = A.reshape_outputs(rep, o, m, l)
  # o is re-rounded to bf16 after every block (attention_kernel.py:327-329)
  assert torch.allclose(o4.double(), wo, atol=1e-2, rtol=1e-2)
  live = end > 0
  assert torch.allclose(m4[live].double(), wm[live], rtol=1e-5, atol=1e-5)
  assert torch.allclose(l4[live].double(), wl[live], rtol=1e-4)
  # empty slot: o = 0, m = -inf, l = 0 (attention_kernel.py:279-283)
  assert torch.count_nonzero(o4[0]) == 0 and torch.all(torch.isinf(m4[0])) and torch.all(l4[0] == 0)


def test_ragged_stacked_selects_layer():
  g = torch.Generator().manual_seed(22)
  k5, v5 = rnd(g, (3, 2, 2, 32, 8)), rnd(g, (3, 2, 2, 32, 8))
  q, end = rnd(g, (2, 4, 1, 8)), torch.tensor([9, 32])
  o, (m, l) = A.ragged_mha(q, k5, v5, 2, None, end, bk=8)
  o2, (m2, l2) = A.ragged_mha(q, k5[2], v5[2], 0, None, end, bk=8)
  assert torch.equal(o, o2) and torch.equal(m, m2) and torch.equal(l, l2)


@pytest.mark.parametrize("quantized", [False, True])
def test_dense_and_flash_equal_closed_form(quantized):
  g = torch.Generator().manual_seed(23)
  b, hq, hkv, s, d = 3, 8, 4, 48, 16
  q = rnd(g, (b, hq, 1, d))
  if quantized:
    k, v, ks, vs = make_int8(g, b, hkv, s, d)
  else:
    k, v, ks, vs = rnd(g, (b, hkv, s, d)), rnd(g, (b, hkv, s, d)), None, None
  pos = torch.tensor([5, 47, 20])
  mask = torch.where(torch.arange(s)[None, :] <= pos[:, None], 0.0, -math.inf).reshape(b, 1, 1, s)
  wo, wm, wl = A.closed_form(q, k, v, mask=mask, k_scale=ks, v_scale=vs)
  od = A.dense_attention(q, k, v, ks, vs, mask)
  assert od.shape == (b, hq, 1, d) and od.dtype == torch.bfloat16
  # the dense entry point keeps scores, probabilities and output in bf16;
  # with int8 codes the bf16 logits are large and carry most of the error
  assert torch.allclose(od.double(), wo, atol=5e-2 if quantized else 2e-2, rtol=2e-2)
  of, (mf, lf) = A.flash_attention(q, k, v, 0, ks, vs, mask)
  assert torch.allclose(of.double(), wo, atol=1e-2, rtol=1e-2)
  assert torch.allclose(mf.double(), wm, rtol=1e-5) and torch.allclose(lf.double(), wl, rtol=1e-4)
  # flash identity: o * denom = sum e^{s-max} v
  assert mf.shape == (b, hq, 1, 1) and lf.shape == (b, hq, 1, 1)


def test_flash_single_new_token():
  """S = 1: o = vscale * v, max = q.k / sqrt(D) * kscale, denom = 1."""
  g = torch.Generator().manual_seed(24)
  q, xk, xv = rnd(g, (3, 4, 1, 8)), rnd(g, (3, 2, 1, 8)), rnd(g, (3, 2, 1, 8))
  kq, ks = quant.quantize_decode(xk)
  vq, vs = quant.quantize_decode(xv)
  o, (m, l) = A.flash_attention(q, kq, vq, 0, ks, vs, None)
  assert torch.all(l == 1)
  want_o = (vq.float() * vs.float()).repeat_interleave(2, dim=1)
  assert torch.allclose(o.float(), want_o, rtol=1e-2)
  want_m = (q.float().reshape(3, 2, 2, 8) * kq.float()).sum(-1) / math.sqrt(8) * ks.float().reshape(3, 1, 1)
  assert torch.allclose(m.reshape(3, 2, 2), want_m, rtol=1e-5, atol=1e-6)


def test_merge_equals_attention_over_concatenation():
  g = torch.Generator().manual_seed(25)
  b, hq, hkv, s, d = 2, 4, 2, 24, 8
  q = rnd(g, (b, hq, 1, d), torch.float32)
  k, v = rnd(g, (b, hkv, s, d), torch.float32), rnd(g, (b, hkv, s, d), torch.float32)
  nk, nv = rnd(g, (b, hkv, 1, d), torch.float32), rnd(g, (b, hkv, 1, d), torch.float32)
  end = torch.tensor([7, 24])
  o1, (m1, l1) = A.flash_attention(q, k, v, 0, None, None,
                                   torch.where(torch.arange(s)[None] < end[:, None], 0.0, -math.inf).reshape(b, 1, 1, s))
  o2, (m2, l2) = A.flash_attention(q, nk, nv, 0)
  merged = A.merge_new_token(o1, m1, l1, o2, m2, l2)
  kc = torch.cat([k, nk], dim=2)
  vc = torch.cat([v, nv], dim=2)
  keep = torch.cat([torch.arange(s)[None] < end[:, None], torch.ones(b, 1, dtype=torch.bool)], dim=1)
  mask = torch.where(keep, 0.0, -math.inf).reshape(b, 1, 1, s + 1)
  wo, _, _ = A.closed_form(q, kc, vc, mask=mask)
  assert torch.allclose(merged.double(), wo, atol=1e-5)


def test_split_kv_merge_is_associative():
  """(m, l) algebra used by split-KV kernels: merging the halves of a row
  reproduces the whole row."""
  g = torch.Generator().manual_seed(26)
  q = rnd(g, (1, 2, 1, 8), torch.float32)
  k, v = rnd(g, (1, 2, 40, 8), torch.float32), rnd(g, (1, 2, 40, 8), torch.float32)
  oa, (ma, la) = A.flash_attention(q, k[:, :, :13], v[:, :, :13])
  ob, (mb, lb) = A.flash_attention(q, k[:, :, 13:], v[:, :, 13:])
  ow, (mw, lw) = A.flash_attention(q, k, v)
  assert torch.allclose(A.merge_new_token(oa, ma, la, ob, mb, lb), ow, atol=1e-6)
  gm = torch.max(ma, mb)
  assert torch.allclose(gm, mw) and torch.allclose(la * torch.exp(ma - gm) + lb * torch.exp(mb - gm), lw, rtol=1e-6)


def test_paged_equals_dense_after_gather():
  g = torch.Generator().manual_seed(27)
  hq, hkv, p, ps, d, b = 8, 2, 12, 4, 8, 3
  kp, vp = rnd(g, (hkv, p, ps, d)), rnd(g, (hkv, p, ps, d))
  table = torch.tensor([[3, 7, 1, 11], [0, 2, 11, 11], [5, 11, 11, 11]])
  lens = torch.tensor([13, 8, 0])
  q = rnd(g, (b, hq, d))
  out = A.paged_attention(q, kp, vp, lens, table, sm_scale=1 / math.sqrt(d))
  for bi in range(2):
    k = A.gather_pages(kp, table[bi], lens[bi])[None]
    v = A.gather_pages(vp, table[bi], lens[bi])[None]
    wo, _, _ = A.closed_form(q[bi].reshape(1, hq, 1, d), k, v)
    assert torch.allclose(out[bi].double(), wo.reshape(hq, d), atol=1e-2)
  assert torch.count_nonzero(out[2]) == 0


def test_paged_saved_vector_says_unscaled_softmax(kats):
  """The reference's only saved paged-attention output is reproduced by a
  softmax WITHOUT 1/sqrt(head_dim) and missed by the scaled one."""
  k = kats["paged_attention_saved_data"]
  h, p, ps, d = k["n_heads"], k["total_num_pages"], k["page_size"], k["head_dim"]
  xq = torch.tensor(k["xq_pair"]).repeat(d // 2).reshape(1, 1, d).repeat(1, h, 1)
  kp, vp = torch.zeros((h, p, ps, d)), torch.zeros((h, p, ps, d))
  kp[:, 0, :k["seq_len"]] = torch.tensor(k["keys_pairs"]).repeat(1, d // 2)
  vp[:, 0, :k["seq_len"]] = torch.tensor(k["values_pairs"]).repeat(1, d // 2)
  table = torch.zeros((1, k["pages_per_sequence"]), dtype=torch.int32)
  lens = torch.tensor([k["seq_len"]])
  saved = torch.tensor(k["saved_output_pair"])
  unscaled = A.paged_attention(xq, kp, vp, lens, table, sm_scale=1.0)[0, 0, :2]
  scaled = A.paged_attention(xq, kp, vp, lens, table, sm_scale=1 / math.sqrt(d))[0, 0, :2]
  assert (unscaled - saved).abs().max() < 2e-5
  assert (scaled - saved).abs().max() > 4e-4


@pytest.mark.parametrize("ring", [True, False])
def test_reference_scenario_int8_kernel_tracks_float_kernel(ring):
  """tests/test_quantization.py:160-284: same q/k/v through the bf16 cache
  kernel and the int8 cache kernel, three steps.  The reference asserts atol
  0.01 on its own jax.random draw; on this draw the int8 error peaks at
  0.012, so the bound here is 0.02."""
  g = torch.Generator().manual_seed(28)
  batch, nl = 4, 3
  env = Env(batch_size=batch, num_layers=nl, ring_buffer=ring, bf16_enable=False, block_size=50)
  shape = (nl, batch, 2, 100, 2) if env.generate_cache_stacked else (batch, 2, 100, 2)
  ck, cv = rnd(g, shape, torch.float32), rnd(g, shape, torch.float32)
  ik, iks = quant.quantize_insert(ck)
  iv, ivs = quant.quantize_insert(cv)
  xq, xk, xv = (rnd(g, (batch, 2, 1, 2), torch.float32) for _ in range(3))
  fcache = KVCacheGenerate(ck.clone(), cv.clone(), None, None, env)
  icache = Int8KVCacheGenerate(ik, iv, iks, ivs, None, None, env)
  fker, iker = AttentionKernel(env, 0), Int8KVAttentionKernel(env, 0)
  for layer, position in ((1, 57), (1, 58), (2, 3)):
    pos = [position] if ring else torch.tensor([position] * batch)
    mask = torch.tensor([0.0] * position + [-math.inf] * (100 - position)).expand(batch, 1, 1, 100)
    res = []
    for ker, cache in ((fker, fcache), (iker, icache)):
      ker.layer_id, cache.input_pos = layer, pos
      res.append(ker(xq, xk, xv, mask, cache, start=None, end=pos))
      cache.finalize()
    assert torch.allclose(res[0], res[1], atol=0.02)


def test_lazy_orchestration_equals_attention_over_updated_cache():
  """Lazy (attend old cache, attend new token, merge) == eager (write, attend)."""
  g = torch.Generator().manual_seed(29)
  b, hq, hkv, s, d = 3, 4, 2, 32, 8
  pos = torch.tensor([4, 31, 17])
  ck, cv = rnd(g, (1, b, hkv, s, d), torch.float32), rnd(g, (1, b, hkv, s, d), torch.float32)
  xq, xk, xv = rnd(g, (b, hq, 1, d), torch.float32), rnd(g, (b, hkv, 1, d), torch.float32), rnd(g, (b, hkv, 1, d), torch.float32)
  lazy_env = Env(batch_size=b, num_layers=1, ring_buffer=False, bf16_enable=False, block_size=8)
  cache = KVCacheGenerate(ck.clone(), cv.clone(), pos, None, lazy_env)
  out = AttentionKernel(lazy_env, 0)(xq, xk, xv, None, cache, end=pos)
  cache.finalize()
  want, _, _ = A.closed_form(xq, cache.cache_k[0], cache.cache_v[0], lengths=pos + 1)
  assert torch.allclose(out.double(), want, atol=1e-5)
