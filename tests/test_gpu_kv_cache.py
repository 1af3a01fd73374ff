"""GPU parity: cache update()/finalize() through the C ABI against the CPU
oracle on the same seeded inputs.  Bit-exact for every cache byte, code and
scale (integer/byte work: no tolerance)."""

import itertools

import pytest
import torch

from oracle import Env as OEnv
from oracle import kv_cache as okv
from oracle import quant as oquant

pytestmark = pytest.mark.gpu

B, H, S, D, L = 4, 2, 16, 8, 3
DEV = "cuda"

MODES = [
    ("ring_eager", dict(ring_buffer=True, lazy_cache_update=False, generate_cache_stacked=False, new_cache_stacked=False)),
    ("ring_lazy", dict(ring_buffer=True, lazy_cache_update=True, generate_cache_stacked=False, new_cache_stacked=False)),
    ("eager", dict(ring_buffer=False, lazy_cache_update=False, generate_cache_stacked=False, new_cache_stacked=False)),
    ("eager_stacked", dict(ring_buffer=False, lazy_cache_update=False, generate_cache_stacked=True, new_cache_stacked=False)),
    ("lazy_unstacked", dict(ring_buffer=False, lazy_cache_update=True, generate_cache_stacked=False, new_cache_stacked=False)),
    ("lazy_stacked_newlist", dict(ring_buffer=False, lazy_cache_update=True, generate_cache_stacked=True, new_cache_stacked=False)),
    ("lazy_stacked", dict(ring_buffer=False, lazy_cache_update=True, generate_cache_stacked=True, new_cache_stacked=True)),
]


def envs(flags, bf16=True, batch=B, layers=L):
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData
  o = OEnv(batch_size=batch, num_layers=layers, testing=True, bf16_enable=bf16, **flags)
  g = JetEngineEnvironment(JetEngineEnvironmentData(
      batch_size=batch, num_layers=layers, testing=True, bf16_enable=bf16, **flags))
  for f in ("lazy_cache_update", "generate_cache_stacked", "new_cache_stacked", "ring_buffer"):
    assert getattr(o, f) == getattr(g, f)
  return o, g


def rnd(g, shape, dtype):
  mag = torch.logspace(-3, 2, shape[0]).reshape(-1, *([1] * (len(shape) - 1)))
  return (torch.randn(shape, generator=g) * mag).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("name,flags", MODES)
def test_float_cache_modes(name, flags, dtype):
  from jetstream_pt_amd import cache_manager as cm
  g = torch.Generator().manual_seed(100)
  oenv, genv = envs(flags, bf16=dtype == torch.bfloat16)
  stacked = flags["generate_cache_stacked"]
  shape = (L, B, H, S, D) if stacked else (B, H, S, D)
  ck, cv = rnd(g, shape, dtype), rnd(g, shape, dtype)
  pos = [9] if flags["ring_buffer"] else [3, 0, 15, 7]
  ocache = okv.KVCacheGenerate(ck.clone(), cv.clone(), torch.tensor(pos), None, oenv)
  gcache = cm.KVCacheGenerate(ck.to(DEV), cv.to(DEV), torch.tensor(pos, device=DEV), None, genv)
  for layer in (range(L) if stacked else [0]):
    k, v = rnd(g, (B, H, 1, D), dtype), rnd(g, (B, H, 1, D), dtype)
    ok, ov = ocache.update(k, v, layer)
    gk, gv = gcache.update(k.to(DEV), v.to(DEV), layer)
    assert torch.equal(gk.cpu(), ok) and torch.equal(gv.cpu(), ov), f"update() return, layer {layer}"
  ocache.finalize()
  gcache.finalize()
  assert torch.equal(gcache.cache_k.cpu(), ocache.cache_k)
  assert torch.equal(gcache.cache_v.cpu(), ocache.cache_v)


VARIANTS = [
    dict(),  # reference literal: truncation, one bf16 scale per token
    dict(rounding="rne"),
    dict(scale_heads=H, scale_dtype=torch.float32),
    dict(rounding="rne", scale_heads=H, scale_dtype=torch.float32),
    dict(scale_dtype=torch.float32),
]


@pytest.mark.parametrize("variant", VARIANTS, ids=lambda v: "-".join(f"{k}={v[k]}" for k in v) or "literal")
# every mode the reference's int8 cache has: its eager update indexes a 4-D cache
# (cache_manager.py:566-571), so there is no eager mode over a stacked one
@pytest.mark.parametrize("name,flags", [m for m in MODES if m[0] != "eager_stacked"])
def test_int8_cache_modes(name, flags, variant):
  from jetstream_pt_amd import cache_manager as cm
  g = torch.Generator().manual_seed(101)
  oenv, genv = envs(flags)
  stacked = flags["generate_cache_stacked"]
  shape = (L, B, H, S, D) if stacked else (B, H, S, D)
  ocache = okv.Int8KVCacheGenerate.empty(shape, None, oenv, **variant)
  gcache = cm.Int8KVCacheGenerate.empty(shape, DEV, genv, **variant)
  pos = [9] if flags["ring_buffer"] else [3, 0, 15, 7]
  ocache.input_pos = torch.tensor(pos)
  gcache.input_pos = torch.tensor(pos, device=DEV)
  for layer in (range(L) if stacked else [0]):
    k, v = rnd(g, (B, H, 1, D), torch.bfloat16), rnd(g, (B, H, 1, D), torch.bfloat16)
    oret = ocache.update(k, v, layer)
    gret = gcache.update(k.to(DEV), v.to(DEV), layer)
    assert len(gret) == 8
    for i in (2, 3, 6, 7):  # k_quant, v_quant, kscale, vscale
      assert gret[i].dtype == oret[i].dtype and gret[i].shape == oret[i].shape
      assert torch.equal(gret[i].cpu(), oret[i]), f"update() return {i}, layer {layer}"
  ocache.finalize()
  gcache.finalize()
  for name_ in ("cache_k", "cache_v", "k_scaler", "v_scaler"):
    a, w = getattr(gcache, name_).cpu(), getattr(ocache, name_)
    assert a.dtype == w.dtype and torch.equal(a, w), name_


@pytest.mark.parametrize("rounding,ofn", [("trunc", oquant.quantize_decode), ("rne", oquant.quantize_insert)])
@pytest.mark.parametrize("in_dtype,scale_dtype", [(torch.bfloat16, None), (torch.bfloat16, torch.float32), (torch.float32, None)])
@pytest.mark.parametrize("heads", [8, 16, 32, 5])
def test_quantiser_wide_dynamic_range(heads, rounding, ofn, in_dtype, scale_dtype):
  """256 tokens spanning 1e-6 .. 1e3 in magnitude, heads x 128 (1024, 2048 and
  4096 elements a token take the register-resident kernel, 640 the generic one)."""
  from jetstream_pt_amd.quantize import quantize_kv
  g = torch.Generator().manual_seed(102)
  x = (torch.randn((256, heads, 1, 128), generator=g) * torch.logspace(-6, 3, 256).reshape(-1, 1, 1, 1)).to(in_dtype)
  y = (torch.randn((256, heads, 1, 128), generator=g) * 3).to(in_dtype)
  for hs in (1, heads):
    kq, vq, ks, vs = quantize_kv(x.to(DEV), y.to(DEV), rounding=rounding, scale_heads=hs, scale_dtype=scale_dtype)
    for got_c, got_s, src in ((kq, ks, x), (vq, vs, y)):
      wc, ws = ofn(src, hs, scale_dtype)
      assert got_s.dtype == ws.dtype and torch.equal(got_s.cpu(), ws)
      assert torch.equal(got_c.cpu(), wc)


def test_quantiser_exhaustive_bf16():
  """Every finite bf16 value not above the absmax, both rounding modes."""
  from jetstream_pt_amd.quantize import quantize_kv
  bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
  allv = bits.view(torch.bfloat16)
  for amax in (3.140625, 0.0247, 1.0, 250.0):
    a = torch.tensor(amax, dtype=torch.bfloat16)
    keep = torch.isfinite(allv.float()) & (allv.float().abs() <= a.float())
    vals = allv[keep]
    n = vals.numel() // 128 * 128
    x = vals[:n].reshape(1, n // 128, 1, 128).clone()
    x[0, 0, 0, 0] = a
    for rounding, ofn in (("trunc", oquant.quantize_decode), ("rne", oquant.quantize_insert)):
      wc, ws = ofn(x)
      kq, _, ks, _ = quantize_kv(x.to(DEV), x.to(DEV), rounding=rounding)
      assert torch.equal(ks.cpu(), ws) and torch.equal(kq.cpu(), wc), (amax, rounding)


def test_all_zero_token_is_defined():
  from jetstream_pt_amd.quantize import quantize_kv
  x = torch.zeros((2, 2, 1, 8), dtype=torch.bfloat16)
  x[1] = 1.0
  kq, _, ks, _ = quantize_kv(x.to(DEV), x.to(DEV))
  assert torch.count_nonzero(kq[0]) == 0 and ks[0].item() == 0.0
  wc, ws = oquant.quantize_decode(x)
  assert torch.equal(kq.cpu(), wc) and torch.equal(ks.cpu(), ws)


def test_untouched_bytes_and_idempotence():
  """Only line pos[b] of each (slot, head) changes; rewriting the same token
  changes nothing."""
  from jetstream_pt_amd import cache_manager as cm
  g = torch.Generator().manual_seed(103)
  _, genv = envs(dict(ring_buffer=False, lazy_cache_update=False, generate_cache_stacked=False, new_cache_stacked=False), batch=8)
  ck = torch.randn((8, 4, 64, 128), generator=g).to(torch.bfloat16)
  pos = torch.randint(0, 64, (8,), generator=g)
  cache = cm.KVCacheGenerate(ck.to(DEV), ck.to(DEV).clone(), pos.to(DEV), None, genv)
  k = torch.randn((8, 4, 1, 128), generator=g).to(torch.bfloat16)
  cache.update(k.to(DEV), k.to(DEV), 0)
  after = cache.cache_k.cpu()
  changed = (after != ck).any(dim=-1)
  want = torch.zeros_like(changed)
  for b, h in itertools.product(range(8), range(4)):
    want[b, h, pos[b]] = True
  assert torch.equal(changed | want, want)
  cache.update(k.to(DEV), k.to(DEV), 0)
  assert torch.equal(cache.cache_k.cpu(), after)


def test_reference_scenario_update_finalize_dequant():
  """tests/test_quantization.py:72-153 through the GPU classes."""
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData
  for ring in (True, False):
    env = JetEngineEnvironment(JetEngineEnvironmentData(batch_size=4, num_layers=3, ring_buffer=ring))
    shape = (3, 4, 2, 100, 2) if env.generate_cache_stacked else (4, 2, 100, 2)
    cache = cm.Int8KVCacheGenerate.empty(shape, DEV, env)
    g = torch.Generator().manual_seed(1)
    k = torch.randn((4, 2, 1, 2), generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn((4, 2, 1, 2), generator=g).to(torch.bfloat16).to(DEV)
    for layer, pos in ((1, 57), (1, 58), (2, 3)):
      cache.input_pos = [pos] if ring else torch.tensor([pos] * 4)
      cache.update(k, v, layer)
      cache.finalize()
      nk, nv = cache.cache_k * cache.k_scaler, cache.cache_v * cache.v_scaler
      if env.generate_cache_stacked:
        nk, nv = nk[layer], nv[layer]
      assert torch.allclose(k.float(), nk[:, :, pos:pos + 1].float(), atol=0.1)
      assert torch.allclose(v.float(), nv[:, :, pos:pos + 1].float(), atol=0.1)
