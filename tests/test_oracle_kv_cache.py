"""Pins oracle.kv_cache to brute-force loops: every mode of update()/finalize()
must touch exactly one line per (layer, slot, head) and nothing else."""

import itertools

import pytest
import torch

from oracle import Env, quant
from oracle.kv_cache import Int8KVCacheGenerate, KVCacheGenerate

B, H, S, D, L = 4, 2, 16, 4, 3


def env_for(ring, lazy, stacked, new_stacked):
  return Env(batch_size=B, num_layers=L, ring_buffer=ring, testing=True,
             lazy_cache_update=lazy, generate_cache_stacked=stacked,
             new_cache_stacked=new_stacked)


MODES = [
    ("ring_eager", dict(ring=True, lazy=False, stacked=False, new_stacked=False)),
    ("ring_lazy", dict(ring=True, lazy=True, stacked=False, new_stacked=False)),
    ("eager", dict(ring=False, lazy=False, stacked=False, new_stacked=False)),
    ("eager_stacked", dict(ring=False, lazy=False, stacked=True, new_stacked=False)),
    ("lazy_unstacked", dict(ring=False, lazy=True, stacked=False, new_stacked=False)),
    ("lazy_stacked_newlist", dict(ring=False, lazy=True, stacked=True, new_stacked=False)),
    ("lazy_stacked", dict(ring=False, lazy=True, stacked=True, new_stacked=True)),
]


def rnd(g, shape, dtype=torch.bfloat16):
  return torch.randn(shape, generator=g).to(dtype)


@pytest.mark.parametrize("name,mode", MODES)
def test_bf16_cache_modes(name, mode):
  g = torch.Generator().manual_seed(5)
  env = env_for(**mode)
  shape = (L, B, H, S, D) if mode["stacked"] else (B, H, S, D)
  ck, cv = rnd(g, shape), rnd(g, shape)
  want_k, want_v = ck.clone(), cv.clone()
  pos = [9] if mode["ring"] else [3, 0, 15, 7]
  cache = KVCacheGenerate(ck, cv, torch.tensor(pos), None, env)
  layers = range(L) if mode["stacked"] else [0]
  for layer in layers:
    k, v = rnd(g, (B, H, 1, D)), rnd(g, (B, H, 1, D))
    rk, rv = cache.update(k, v, layer)
    assert rk.shape == (B, H, S, D) and rv.shape == (B, H, S, D)
    for b, h in itertools.product(range(B), range(H)):
      p = pos[0] if mode["ring"] else pos[b]
      tgt_k = want_k[layer] if mode["stacked"] else want_k
      tgt_v = want_v[layer] if mode["stacked"] else want_v
      tgt_k[b, h, p] = k[b, h, 0]
      tgt_v[b, h, p] = v[b, h, 0]
    if not mode["lazy"]:
      full_k = want_k[layer] if mode["stacked"] else want_k
      assert torch.equal(rk, full_k)
  if mode["lazy"]:
    assert not torch.equal(cache.cache_k, want_k)  # nothing written before finalize
  cache.finalize()
  assert torch.equal(cache.cache_k, want_k) and torch.equal(cache.cache_v, want_v)


@pytest.mark.parametrize("name,mode", MODES)
@pytest.mark.parametrize("variant", [dict(), dict(rounding="rne", scale_heads=H, scale_dtype=torch.float32)])
def test_int8_cache_modes(name, mode, variant):
  if name == "eager_stacked":
    pytest.skip("the reference's int8 eager branch indexes a 4-D cache only (cache_manager.py:566-571)")
  g = torch.Generator().manual_seed(6)
  env = env_for(**mode)
  shape = (L, B, H, S, D) if mode["stacked"] else (B, H, S, D)
  cache = Int8KVCacheGenerate.empty(shape, None, env, **variant)
  hs = variant.get("scale_heads", 1)
  assert cache.k_scaler.shape == ((L, B, hs, S, 1) if mode["stacked"] else (B, hs, S, 1))
  assert torch.all(cache.k_scaler == 1) and torch.count_nonzero(cache.cache_k) == 0
  want = [t.clone() for t in (cache.cache_k, cache.cache_v, cache.k_scaler, cache.v_scaler)]
  pos = [9] if mode["ring"] else [3, 0, 15, 7]
  cache.input_pos = torch.tensor(pos)
  qfn = quant.quantize_insert if variant else quant.quantize_decode
  layers = range(L) if mode["stacked"] else [0]
  for layer in layers:
    k, v = rnd(g, (B, H, 1, D)), rnd(g, (B, H, 1, D))
    ret = cache.update(k, v, layer)
    assert len(ret) == 8
    qk, sk = qfn(k, hs, variant.get("scale_dtype"))
    qv, sv = qfn(v, hs, variant.get("scale_dtype"))
    assert torch.equal(ret[2], qk) and torch.equal(ret[6], sk)
    assert torch.equal(ret[3], qv) and torch.equal(ret[7], sv)
    skip_scales = mode["ring"] and mode["lazy"]  # reference finalize writes codes only
    for b in range(B):
      p = pos[0] if mode["ring"] else pos[b]
      tgt = [w[layer] if mode["stacked"] else w for w in want]
      tgt[0][b, :, p] = qk[b, :, 0]
      tgt[1][b, :, p] = qv[b, :, 0]
      if not skip_scales:
        tgt[2][b, :, p] = sk[b, :, 0]
        tgt[3][b, :, p] = sv[b, :, 0]
  cache.finalize()
  got = (cache.cache_k, cache.cache_v, cache.k_scaler, cache.v_scaler)
  for a, w in zip(got, want):
    assert torch.equal(a, w)


def test_reference_scenario_update_finalize_dequant():
  """tests/test_quantization.py:72-153: (layer 1, pos 57), (1, 58), (2, 3);
  codes * scale reproduces the input within 0.1, ring and left-aligned."""
  for ring in (True, False):
    env = Env(batch_size=4, num_layers=3, ring_buffer=ring)
    shape = (3, 4, 2, 100, 2) if env.generate_cache_stacked else (4, 2, 100, 2)
    cache = Int8KVCacheGenerate.empty(shape, None, env)
    g = torch.Generator().manual_seed(1)
    k, v = rnd(g, (4, 2, 1, 2)), rnd(g, (4, 2, 1, 2))
    for layer, pos in ((1, 57), (1, 58), (2, 3)):
      cache.input_pos = [pos] if ring else torch.tensor([pos] * 4)
      cache.update(k, v, layer)
      cache.finalize()
      nk = cache.cache_k * cache.k_scaler
      nv = cache.cache_v * cache.v_scaler
      if env.generate_cache_stacked:
        nk, nv = nk[layer], nv[layer]
      assert torch.allclose(k.float(), nk[:, :, pos:pos + 1].float(), atol=0.1)
      assert torch.allclose(v.float(), nv[:, :, pos:pos + 1].float(), atol=0.1)


def test_prefill_cache_pretends_to_be_quantised():
  """cache_manager.py:42-69: KVCachePrefill keeps K/V as they are; with
  kv_quantize it returns the 8-tuple Int8KVAttentionKernel unpacks
  (layers.py:677-686), scalers = bf16 ones (B, 1, T, 1), nothing quantised -
  so attention through it equals attention over the unquantised K/V."""
  from oracle import attention as A
  from oracle.attn_layers import AttentionKernel, Int8KVAttentionKernel
  from oracle.kv_cache import KVCachePrefill
  g = torch.Generator().manual_seed(11)
  t, h, d = 12, 2, 8
  k, v, q = rnd(g, (1, h, t, d)), rnd(g, (1, h, t, d)), rnd(g, (1, h, t, d))
  plain = KVCachePrefill()
  assert plain.update(k, v) == (k, v) and plain.state() == (k, v)
  cache = KVCachePrefill(kv_quantize=True)
  ret = cache.update(k, v, 3)
  assert len(ret) == 8 and ret[0] is k and ret[1] is v
  assert [ret[i] for i in (2, 3, 6, 7)] == [None] * 4
  for ones in ret[4:6]:
    assert ones.shape == (1, 1, t, 1) and ones.dtype == torch.bfloat16 and bool((ones == 1).all())
  assert cache.state() == (k, v) and cache.finalize() is None
  env = Env(batch_size=1, num_layers=1, ring_buffer=False)
  mask = torch.full((t, t), float("-inf")).triu(1).reshape(1, 1, t, t)
  quantised_path = Int8KVAttentionKernel(env, 0)(q, k, v, mask, KVCachePrefill(kv_quantize=True))
  plain_path = AttentionKernel(env, 0)(q, k, v, mask, KVCachePrefill())
  assert torch.equal(quantised_path, plain_path)  # multiplying by bf16 ones changes no bit
  exact, _, _ = A.closed_form(q, k, v, mask=mask)
  assert (quantised_path.double() - exact).abs().max() < 5e-2
