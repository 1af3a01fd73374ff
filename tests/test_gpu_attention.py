"""GPU parity: decode attention through the C ABI against the float64 closed
form and the CPU restatement of the reference's kernels.

Tolerances (floating point): outputs max-abs 1e-2 against the float64 closed
form where |expected| < 2; from 2 on the half-ulp by which a bf16 output may
differ from the unrounded closed form, 2^-8 |expected|, takes 0.0078 or more of
that and is added (conftest.attention_bound); row max and softmax denominator
rtol 1e-3.  The largest error every check saw is recorded (tests/conftest.py)."""

import math
import os

import numpy as np
import pytest
import torch

from conftest import attention_bound, record_parity
from oracle import Env as OEnv
from oracle import attention as OA
from oracle import kv_cache as okv
from oracle.attn_layers import AttentionKernel as OAttn
from oracle.attn_layers import Int8KVAttentionKernel as OInt8Attn

pytestmark = pytest.mark.gpu
DEV = "cuda"
OUT_ATOL, STAT_RTOL = 1e-2, 1e-3


def rnd(g, shape, dtype=torch.bfloat16):
  return torch.randn(shape, generator=g).to(dtype)


def int8_cache(g, b, h, s, d, hs=1, sdt=torch.float32):
  k = torch.randint(-127, 128, (b, h, s, d), generator=g, dtype=torch.int8)
  v = torch.randint(-127, 128, (b, h, s, d), generator=g, dtype=torch.int8)
  ks = (torch.rand((b, hs, s, 1), generator=g) * 0.045 + 0.005).to(sdt)
  vs = (torch.rand((b, hs, s, 1), generator=g) * 0.045 + 0.005).to(sdt)
  return k, v, ks, vs


def check_out(got, want, what=""):
  got, want = got.double().cpu(), want.double()
  test = os.environ.get("PYTEST_CURRENT_TEST", "attention").split("::")[-1].split(" ")[0]
  err = record_parity(f"attention/{test}", got, want)
  bound = attention_bound(want)
  assert torch.all(err <= bound), f"{what}: max err {err.max():.4g} (bound {OUT_ATOL})"


def check_vs_reference_arithmetic(got, want, what, roundings=1, vmax=None):
  """Against the oracle's restatement of the reference's own arithmetic, whose
  result is itself rounded to bf16 (once per block of the ragged recurrence,
  attention_kernel.py:327-329, and once more by the new-token merge): each such
  rounding moves it by up to half a bf16 ulp of a value no larger than the
  largest dequantised value row `vmax` (|expected| stands in when vmax is not
  given and every rounding is of the final value).  On top of check_out's bound."""
  got, want = got.double().cpu(), want.double()
  test = os.environ.get("PYTEST_CURRENT_TEST", "attention").split("::")[-1].split(" ")[0]
  err = record_parity(f"attention_vs_reference_arithmetic/{test}", got, want)
  theirs = roundings * 2.0 ** -8 * (want.abs() if vmax is None else vmax)
  bound = attention_bound(want) + theirs
  assert torch.all(err <= bound), f"{what}: max err {err.max():.4g}"


def check_stats(m, l, wm, wl, live):
  m, l = m.double().cpu().reshape(wm.shape), l.double().cpu().reshape(wl.shape)
  assert torch.allclose(m[live], wm[live], rtol=STAT_RTOL, atol=1e-4)
  assert torch.allclose(l[live], wl[live], rtol=STAT_RTOL)
  dead = ~live
  if dead.any():
    assert torch.all(torch.isinf(m[dead]) & (m[dead] < 0)) and torch.all(l[dead] == 0)


def to_dev(*xs):
  return [None if x is None else x.to(DEV) for x in xs]


LENGTH_SETS = {
    "edges": [0, 1, 31, 32, 33, 127, 128, 129],
    "long": [4096, 3000, 17, 2049],
}


@pytest.mark.parametrize("lens_name", list(LENGTH_SETS))
@pytest.mark.parametrize("hq,hkv", [(32, 8), (8, 8), (16, 1)])
@pytest.mark.parametrize("kind", ["int8_f32", "int8_bf16_perhead", "bf16"])
def test_ragged_fast_kernel_vs_closed_form(kind, hq, hkv, lens_name):
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(300)
  lens = LENGTH_SETS[lens_name]
  b, d = len(lens), 128
  s = 4096 if lens_name == "long" else 256
  if lens_name == "long":
    hq, hkv = hq // min(hkv, 4) if hkv >= 4 else hq, max(1, hkv // 4)
  end = torch.tensor(lens, dtype=torch.int32)
  q = rnd(g, (b, hq, 1, d))
  if kind == "bf16":
    k, v, ks, vs = rnd(g, (b, hkv, s, d)), rnd(g, (b, hkv, s, d)), None, None
  elif kind == "int8_f32":
    k, v, ks, vs = int8_cache(g, b, hkv, s, d)
  else:
    k, v, ks, vs = int8_cache(g, b, hkv, s, d, hs=hkv, sdt=torch.bfloat16)
  wo, wm, wl = OA.closed_form(q, k, v, lengths=end, k_scale=ks, v_scale=vs)
  gq, gk, gv, gks, gvs, gend = to_dev(q, k, v, ks, vs, end)
  o, (m, l) = ak.ragged_mha(gq, gk, gv, 0, None, gend, None, None, gks, gvs)
  rep = hq // hkv
  assert o.shape == (b, hkv, rep, d) and m.shape == (b, hkv, rep) and o.dtype == torch.bfloat16
  check_out(o.reshape(b, hq, 1, d), wo, "fast")
  live = (end > 0).reshape(b, 1, 1, 1).expand(b, hq, 1, 1)
  check_stats(m, l, wm, wl, live)
  # the shape-generic kernel must agree too (second implementation)
  o2, m2, l2 = ak._attend("ragged", gq, gk, gv, lengths=gend, k_scaler=gks, v_scaler=gvs,
                          want_stats=True, force_generic=True)
  check_out(o2, wo, "generic")
  check_stats(m2, l2, wm, wl, live)
  # and both track the restatement of the reference's blockwise kernel
  ro, (rm, rl) = OA.ragged_mha(q, k, v, 0, None, end, None, None, ks, vs, bk=min(512, s))
  vmax = float(v.float().abs().max()) * (float(vs.float().max()) if vs is not None else 1.0)
  check_vs_reference_arithmetic(o.reshape(b, hq, 1, d), OA.reshape_outputs(rep, ro)[0], "vs reference recurrence",
                                roundings=(max(lens) + 511) // 512, vmax=vmax)


@pytest.mark.parametrize("kind", ["int8", "bf16"])
def test_ragged_very_large_batch(kind):
  """1100 slots x 32 KV heads: more work items per worker than the kernel keeps
  listed in LDS, so the later ones are fetched as they are reached."""
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(312)
  rng = np.random.default_rng(312)
  b, hq, hkv, s, d = 1100, 32, 32, 128, 128
  lens = rng.integers(0, s + 1, b).astype(np.int32)
  lens[:8] = [0, 1, 31, 32, 33, s, s - 1, 2]
  end = torch.from_numpy(lens)
  q = rnd(g, (b, hq, 1, d))
  if kind == "int8":
    k, v, ks, vs = int8_cache(g, b, hkv, s, d)
  else:
    k, v, ks, vs = rnd(g, (b, hkv, s, d)), rnd(g, (b, hkv, s, d)), None, None
  wo, wm, wl = OA.closed_form(q, k, v, lengths=end, k_scale=ks, v_scale=vs)
  gq, gk, gv, gks, gvs, gend = to_dev(q, k, v, ks, vs, end)
  o, (m, l) = ak.ragged_mha(gq, gk, gv, 0, None, gend, None, None, gks, gvs)
  check_out(o.reshape(b, hq, 1, d), wo, "very large batch")
  check_stats(m, l, wm, wl, (end > 0).reshape(b, 1, 1, 1).expand(b, hq, 1, 1))


def test_ragged_stacked_cache_selects_layer_and_reuses_plan():
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(301)
  nl, b, hq, hkv, s, d = 3, 5, 8, 2, 512, 128
  end = torch.tensor([512, 77, 0, 300, 1], dtype=torch.int32)
  q = rnd(g, (b, hq, 1, d))
  k = torch.randint(-127, 128, (nl, b, hkv, s, d), generator=g, dtype=torch.int8)
  v = torch.randint(-127, 128, (nl, b, hkv, s, d), generator=g, dtype=torch.int8)
  ks = (torch.rand((nl, b, 1, s, 1), generator=g) * 0.045 + 0.005).to(torch.bfloat16)
  vs = (torch.rand((nl, b, 1, s, 1), generator=g) * 0.045 + 0.005).to(torch.bfloat16)
  gq, gk, gv, gks, gvs, gend = to_dev(q, k, v, ks, vs, end)
  plan, _ = ak.precompute_ragged_block_indices(gend, b, hq, hkv, s)
  kern = ak.RaggedAttentionKernel(OEnv(block_size=512))
  for layer in (2, 0, 1, 2):
    wo, wm, wl = OA.closed_form(q, k[layer], v[layer], lengths=end, k_scale=ks[layer], v_scale=vs[layer])
    o, (m, l) = kern(gq, gk, gv, layer, None, plan.lengths, plan, None, gks, gvs)
    check_out(o.reshape(b, hq, 1, d), wo, f"layer {layer} (planned)")
    o2, _ = kern(gq, gk, gv, layer, None, gend, None, None, gks, gvs)
    assert torch.equal(o, o2), "a reused plan must not change the result"


@pytest.mark.parametrize("shape", [dict(b=3, hq=4, hkv=2, s=48, d=16, t=1), dict(b=2, hq=2, hkv=2, s=100, d=2, t=1),
                                   dict(b=2, hq=4, hkv=4, s=40, d=64, t=5), dict(b=8, hq=32, hkv=32, s=1024, d=128, t=1)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_dense_and_flash_with_mask(shape, dtype):
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(302)
  b, hq, hkv, s, d, t = (shape[x] for x in ("b", "hq", "hkv", "s", "d", "t"))
  q, k, v = rnd(g, (b, hq, t, d), dtype), rnd(g, (b, hkv, s, d), dtype), rnd(g, (b, hkv, s, d), dtype)
  pos = torch.randint(0, s, (b,), generator=g)
  mask = torch.where(torch.arange(s)[None, :] <= pos[:, None], 0.0, -math.inf).reshape(b, 1, 1, s)
  wo, wm, wl = OA.closed_form(q, k, v, mask=mask)
  gq, gk, gv, gmask = to_dev(q, k, v, mask)
  o = ak.dense_attention(gq, gk, gv, None, None, gmask)
  assert o.shape == (b, hq, t, d) and o.dtype == dtype
  check_out(o, wo, "dense")
  of, (mf, lf) = ak.flash_attention(gq, gk, gv, 0, None, None, gmask)
  assert mf.shape == (b, hq, t, 1) and lf.shape == (b, hq, t, 1)
  check_out(of, wo, "flash")
  check_stats(mf, lf, wm, wl, torch.ones_like(wm, dtype=torch.bool))
  # the reference's own dense arithmetic (activation-dtype scores) stays within its noise
  ref = OA.dense_attention(q, k, v, None, None, mask)
  assert (o.cpu().double() - ref.double()).abs().max() < (5e-2 if dtype == torch.bfloat16 else 1e-4)


def test_dense_int8_with_scalers():
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(303)
  b, hq, hkv, s, d = 4, 8, 4, 256, 128
  q = rnd(g, (b, hq, 1, d))
  k, v, ks, vs = int8_cache(g, b, hkv, s, d, sdt=torch.bfloat16)
  pos = torch.tensor([0, 255, 100, 31])
  mask = torch.where(torch.arange(s)[None, :] <= pos[:, None], 0.0, -math.inf).reshape(b, 1, 1, s)
  wo, _, _ = OA.closed_form(q, k, v, mask=mask, k_scale=ks, v_scale=vs)
  o = ak.dense_attention(*to_dev(q, k, v, ks, vs, mask))
  check_out(o, wo, "dense int8")


def test_flash_single_new_token_identity():
  """S = 1: o = vscale * v, max = q.k / sqrt(D) * kscale, denom = 1."""
  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd.quantize import quantize_kv
  g = torch.Generator().manual_seed(304)
  q, xk, xv = rnd(g, (3, 8, 1, 128)), rnd(g, (3, 2, 1, 128)), rnd(g, (3, 2, 1, 128))
  gq, gk, gv = to_dev(q, xk, xv)
  kq, vq, ks, vs = quantize_kv(gk, gv)
  o, (m, l) = ak.flash_attention(gq, kq, vq, 0, ks, vs, None)
  assert torch.all(l == 1)
  want_o = (vq.float() * vs.float()).repeat_interleave(4, dim=1).cpu()
  check_out(o, want_o, "new token")
  want_m = (q.float().reshape(3, 2, 4, 128) * kq.cpu().float()).sum(-1) / math.sqrt(128) * ks.cpu().float().reshape(3, 1, 1)
  assert torch.allclose(m.cpu().reshape(3, 2, 4), want_m, rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("quantized", [False, True])
def test_fused_new_token_equals_unfused_and_concatenation(quantized):
  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd.quantize import quantize_kv
  g = torch.Generator().manual_seed(305)
  b, hq, hkv, s, d = 6, 16, 4, 1024, 128
  end = torch.tensor([0, 5, 128, 700, 1024, 333], dtype=torch.int32)
  q, xk, xv = rnd(g, (b, hq, 1, d)), rnd(g, (b, hkv, 1, d)), rnd(g, (b, hkv, 1, d))
  if quantized:
    k, v, ks, vs = int8_cache(g, b, hkv, s, d, sdt=torch.bfloat16)
  else:
    k, v, ks, vs = rnd(g, (b, hkv, s, d)), rnd(g, (b, hkv, s, d)), None, None
  gq, gk, gv, gks, gvs, gend, gxk, gxv = to_dev(q, k, v, ks, vs, end, xk, xv)
  if quantized:
    nk, nv, nks, nvs = quantize_kv(gxk, gxv)
    new = dict(new_key=nk, new_value=nv, new_k_scaler=nks, new_v_scaler=nvs)
    ck, cv = nk.cpu(), nv.cpu()
    cks, cvs = nks.cpu(), nvs.cpu()
  else:
    new = dict(new_key=gxk, new_value=gxv)
    ck, cv, cks, cvs = xk, xv, None, None
  fused, _ = ak.ragged_mha(gq, gk, gv, 0, None, gend, None, None, gks, gvs, **new)
  o1, (m1, l1) = ak.ragged_mha(gq, gk, gv, 0, None, gend, None, None, gks, gvs)
  o2, (m2, l2) = ak.flash_attention(gq, new["new_key"], new["new_value"], 0,
                                    new.get("new_k_scaler"), new.get("new_v_scaler"), None)
  unfused = ak.lse_merge(o1.reshape(b, hq, 1, d), m1.reshape(b, hq, 1, 1), l1.reshape(b, hq, 1, 1), o2, m2, l2)
  # the unfused result went through three bf16 roundings (both partial outputs and the merge)
  check_vs_reference_arithmetic(fused.reshape(b, hq, 1, d), unfused.cpu(), "fused vs unfused", roundings=3)
  # closed form over the cache with the new token appended at position end[b]
  kc, vc = torch.cat([k, torch.zeros_like(k[:, :, :1])], 2), torch.cat([v, torch.zeros_like(v[:, :, :1])], 2)
  for bi in range(b):
    kc[bi, :, end[bi]], vc[bi, :, end[bi]] = ck[bi, :, 0], cv[bi, :, 0]
  ksc = vsc = None
  if quantized:
    ksc, vsc = torch.cat([ks, ks[:, :, :1]], 2).clone(), torch.cat([vs, vs[:, :, :1]], 2).clone()
    for bi in range(b):
      ksc[bi, :, end[bi]], vsc[bi, :, end[bi]] = cks[bi, :, 0], cvs[bi, :, 0]
  wo, _, _ = OA.closed_form(q, kc, vc, lengths=end + 1, k_scale=ksc, v_scale=vsc)
  check_out(fused.reshape(b, hq, 1, d), wo, "fused vs closed form")


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (16, 4, 128), (8, 1, 128), (16, 16, 128), (32, 32, 128), (4, 2, 64)])
@pytest.mark.parametrize("sdt,per_head", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("rounding", ["trunc", "rne"])
def test_attention_launch_quantises_the_new_token(rounding, sdt, per_head, hq, hkv, d):
  """new_key_raw: the attention launch does the quantiser's work too.  Codes
  and scales must be the separate quantiser's bit for bit (which the oracle
  pins), the output that of attending those codes.  Head_dim 64 takes the
  library's quantise-first route."""
  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd.quantize import quantize_kv
  from oracle import quant as oq
  g = torch.Generator().manual_seed(311)
  b, s = 7, 512
  end = torch.tensor([0, 5, 128, 400, 512, 333, 31], dtype=torch.int32)
  hs = hkv if per_head else 1
  q, xk, xv = rnd(g, (b, hq, 1, d)), rnd(g, (b, hkv, 1, d)), rnd(g, (b, hkv, 1, d))
  xk[2] = 0                      # an all-zero token: scale 0 (trunc) or eps/127 (rne), codes 0
  xv[3, 0, 0, :5] = 300.0        # a dominant element
  k, v, ks, vs = int8_cache(g, b, hkv, s, d, hs=hs, sdt=sdt)
  gq, gk, gv, gks, gvs, gend, gxk, gxv = to_dev(q, k, v, ks, vs, end, xk, xv)
  wk, wv, wks, wvs = quantize_kv(gxk, gxv, rounding=rounding, scale_heads=hs, scale_dtype=sdt)
  cdt = None if sdt == torch.bfloat16 else sdt
  ok_, oks = (oq.quantize_decode if rounding == "trunc" else oq.quantize_insert)(xk, hs, cdt)
  assert torch.equal(wk.cpu(), ok_) and torch.equal(wks.cpu().reshape(-1), oks.to(sdt).reshape(-1))
  want, (wm, wl) = ak.ragged_mha(gq, gk, gv, 0, None, gend, None, None, gks, gvs, new_key=wk, new_value=wv,
                                 new_k_scaler=wks, new_v_scaler=wvs)
  nk, nv = torch.full_like(wk, 77), torch.full_like(wv, 77)
  nks, nvs = torch.full_like(wks, -1.0), torch.full_like(wvs, -1.0)
  got, (m, l) = ak.ragged_mha(gq, gk, gv, 0, None, gend, None, None, gks, gvs, new_key=nk, new_value=nv,
                              new_k_scaler=nks, new_v_scaler=nvs, new_key_raw=gxk, new_value_raw=gxv,
                              new_rounding=rounding)
  assert torch.equal(nk, wk) and torch.equal(nv, wv), "codes"
  assert torch.equal(nks, wks) and torch.equal(nvs, wvs), "scales"
  if hkv <= 16 or d != 128:
    assert torch.equal(got, want) and torch.equal(m, wm) and torch.equal(l, wl)
  else:
    # more than 16 KV heads: the raw token takes two tiles, so the cache tiles fall to
    # other consumers than in the launch that is given the codes - another summation order
    check_out(got.reshape(b, hq, 1, d), want.reshape(b, hq, 1, d).float().cpu(), "32 KV heads")
    assert torch.allclose(m, wm, rtol=STAT_RTOL, atol=1e-4) and torch.allclose(l, wl, rtol=STAT_RTOL)


@pytest.mark.parametrize("kind", ["bf16", "int8", "tiny_f32"])
def test_paged_equals_dense_after_gather(kind):
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(306)
  rng = np.random.default_rng(306)
  if kind == "tiny_f32":
    hq, hkv, p, ps, d, mp = 8, 2, 24, 4, 8, 6
    lens = [13, 8, 0, 24, 1]
  else:
    hq, hkv, p, ps, d, mp = 16, 4, 64, 64, 128, 8
    lens = [500, 64, 0, 65, 1, 512]
  b = len(lens)
  table = torch.full((b, mp), p - 1, dtype=torch.int32)
  perm = rng.permutation(p)
  at = 0
  for bi, n in enumerate(lens):
    need = -(-n // ps)
    table[bi, :need] = torch.from_numpy(perm[at:at + need].astype(np.int32))
    at += need
  seq = torch.tensor(lens, dtype=torch.int32)
  ksp = vsp = None
  if kind == "int8":
    kp = torch.randint(-127, 128, (hkv, p, ps, d), generator=g, dtype=torch.int8)
    vp = torch.randint(-127, 128, (hkv, p, ps, d), generator=g, dtype=torch.int8)
    ksp = torch.rand((1, p, ps), generator=g) * 0.045 + 0.005
    vsp = torch.rand((1, p, ps), generator=g) * 0.045 + 0.005
    q = rnd(g, (b, hq, d))
  else:
    dt = torch.float32 if kind == "tiny_f32" else torch.bfloat16
    kp, vp, q = rnd(g, (hkv, p, ps, d), dt), rnd(g, (hkv, p, ps, d), dt), rnd(g, (b, hq, d), dt)
  for sm in (1.0, 1 / math.sqrt(d)):
    want = OA.paged_attention(q.float(), kp, vp, seq, table, sm_scale=sm, k_scale_pages=ksp, v_scale_pages=vsp)
    got = ak.call_paged_attention(None, *to_dev(q, kp, vp), seq.numpy(), table.numpy(), sm_scale=sm,
                                  k_scaler=None if ksp is None else ksp.to(DEV),
                                  v_scaler=None if vsp is None else vsp.to(DEV))
    assert got.shape == (b, hq, d)
    check_out(got, want, f"paged sm_scale={sm}")


def test_paged_saved_vector_of_the_reference(kats):
  """The reference's one saved paged output (unused by its assertions) is met
  by the default sm_scale = 1 and missed with 1/sqrt(head_dim)."""
  from jetstream_pt_amd import attention_kernel as ak
  k = kats["paged_attention_saved_data"]
  h, p, ps, d = k["n_heads"], k["total_num_pages"], k["page_size"], k["head_dim"]
  xq = torch.tensor(k["xq_pair"]).repeat(d // 2).reshape(1, 1, d).repeat(1, h, 1).to(torch.bfloat16)
  kp, vp = torch.zeros((h, p, ps, d)), torch.zeros((h, p, ps, d))
  kp[:, 0, :k["seq_len"]] = torch.tensor(k["keys_pairs"]).repeat(1, d // 2)
  vp[:, 0, :k["seq_len"]] = torch.tensor(k["values_pairs"]).repeat(1, d // 2)
  table = np.zeros((1, k["pages_per_sequence"]), dtype=np.int32)
  lens = np.array([k["seq_len"]], dtype=np.int32)
  saved = torch.tensor(k["saved_output_pair"])
  gq, gk, gv = to_dev(xq, kp.to(torch.bfloat16), vp.to(torch.bfloat16))
  out = ak.call_paged_attention(None, gq, gk, gv, lens, table)[0, 0, :2].float().cpu()
  assert (out - saved).abs().max() < 5e-5
  scaled = ak.call_paged_attention(None, gq, gk, gv, lens, table, sm_scale=1 / math.sqrt(d))[0, 0, :2].float().cpu()
  assert (scaled - saved).abs().max() > 3e-4


def _envs(ring, bf16, batch, layers, block=512):
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData
  o = OEnv(batch_size=batch, num_layers=layers, ring_buffer=ring, bf16_enable=bf16, block_size=block)
  g = JetEngineEnvironment(JetEngineEnvironmentData(batch_size=batch, num_layers=layers, ring_buffer=ring,
                                                    bf16_enable=bf16, block_size=block))
  return o, g


@pytest.mark.parametrize("ring", [True, False])
@pytest.mark.parametrize("fuse", [True, False])
def test_orchestration_reference_scenario(ring, fuse):
  """tests/test_quantization.py:160-284 through the GPU classes, checked
  against the oracle's orchestration on the same inputs: float cache kernel
  and int8 cache kernel, three steps at (layer 1, pos 57), (1, 58), (2, 3)."""
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import layers
  from oracle import quant as oquant
  g = torch.Generator().manual_seed(307)
  batch, nl = 4, 3
  oenv, genv = _envs(ring, False, batch, nl, block=50)
  shape = (nl, batch, 2, 100, 2) if oenv.generate_cache_stacked else (batch, 2, 100, 2)
  ck, cv = rnd(g, shape, torch.float32), rnd(g, shape, torch.float32)
  ik, iks = oquant.quantize_insert(ck)
  iv, ivs = oquant.quantize_insert(cv)
  xq, xk, xv = (rnd(g, (batch, 2, 1, 2), torch.float32) for _ in range(3))
  of = okv.KVCacheGenerate(ck.clone(), cv.clone(), None, None, oenv)
  oi = okv.Int8KVCacheGenerate(ik.clone(), iv.clone(), iks.clone(), ivs.clone(), None, None, oenv)
  gf = cm.KVCacheGenerate(ck.to(DEV), cv.to(DEV), None, None, genv)
  gi = cm.Int8KVCacheGenerate(*to_dev(ik, iv, iks, ivs), None, None, genv)
  okers = (OAttn(oenv, 0), OInt8Attn(oenv, 0))
  gkers = (layers.AttentionKernel(genv, 0, fuse_new_token=fuse), layers.Int8KVAttentionKernel(genv, 0, fuse_new_token=fuse))
  gq, gxk, gxv = to_dev(xq, xk, xv)
  for layer, position in ((1, 57), (1, 58), (2, 3)):
    pos = [position] if ring else torch.tensor([position] * batch)
    mask = torch.tensor([0.0] * position + [-math.inf] * (100 - position)).expand(batch, 1, 1, 100)
    for oker, gker, ocache, gcache in zip(okers, gkers, (of, oi), (gf, gi)):
      oker.layer_id = gker.layer_id = layer
      ocache.input_pos = pos
      gcache.input_pos = pos if ring else pos.to(DEV)
      want = oker(xq, xk, xv, mask, ocache, start=None, end=pos)
      got = gker(gq, gxk, gxv, mask.to(DEV), gcache, start=None,
                 end=None if ring else pos.to(DEV).to(torch.int32))
      ocache.finalize()
      gcache.finalize()
      check_out(got, want, f"layer {layer} pos {position} {type(gker).__name__}")
    # cache state stays bit-exact step after step
    assert torch.equal(gf.cache_k.cpu(), of.cache_k) and torch.equal(gi.cache_k.cpu(), oi.cache_k)
    assert torch.equal(gi.k_scaler.cpu(), oi.k_scaler) and torch.equal(gi.v_scaler.cpu(), oi.v_scaler)


def test_orchestration_llama3_shaped_lazy_int8():
  """Production left-aligned mode at head_dim 128, GQA 32/8: stacked int8
  cache, lazy update, ragged attention with the fused new token; outputs vs
  closed form over the finalized cache, cache state vs the oracle."""
  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import layers
  g = torch.Generator().manual_seed(308)
  b, nl, hq, hkv, s, d = 6, 2, 32, 8, 512, 128
  oenv, genv = _envs(False, True, b, nl)
  shape = (nl, b, hkv, s, d)
  ocache = okv.Int8KVCacheGenerate.empty(shape, None, oenv)
  ocache.cache_k.copy_(torch.randint(-127, 128, shape, generator=g, dtype=torch.int8))
  ocache.cache_v.copy_(torch.randint(-127, 128, shape, generator=g, dtype=torch.int8))
  ocache.k_scaler.copy_((torch.rand(ocache.k_scaler.shape, generator=g) * 0.045 + 0.005).to(torch.bfloat16))
  ocache.v_scaler.copy_((torch.rand(ocache.v_scaler.shape, generator=g) * 0.045 + 0.005).to(torch.bfloat16))
  gcache = cm.Int8KVCacheGenerate(*to_dev(ocache.cache_k, ocache.cache_v, ocache.k_scaler, ocache.v_scaler),
                                  None, None, genv)
  pos = torch.tensor([0, 1, 130, 511, 300, 64], dtype=torch.int32)
  ocache.input_pos, gcache.input_pos = pos, pos.to(DEV)
  plan, _ = ak.precompute_ragged_block_indices(pos.to(DEV), b, hq, hkv, s)
  outs, qs = [], []
  for layer in range(nl):
    xq, xk, xv = rnd(g, (b, hq, 1, d)), rnd(g, (b, hkv, 1, d)), rnd(g, (b, hkv, 1, d))
    want = OInt8Attn(oenv, layer)(xq, xk, xv, None, ocache, start=None, end=pos)
    got = layers.Int8KVAttentionKernel(genv, layer)(*to_dev(xq, xk, xv), None, gcache, start=None,
                                                     end=plan.lengths, ragged_batch_index=plan)
    check_vs_reference_arithmetic(got, want, f"layer {layer} vs oracle orchestration", roundings=3, vmax=127 * 0.05)
    outs.append(got), qs.append(xq)
  ocache.finalize()
  gcache.finalize()
  for name in ("cache_k", "cache_v", "k_scaler", "v_scaler"):
    assert torch.equal(getattr(gcache, name).cpu(), getattr(ocache, name)), name
  for layer in range(nl):
    wo, _, _ = OA.closed_form(qs[layer], ocache.cache_k[layer], ocache.cache_v[layer], lengths=pos + 1,
                              k_scale=ocache.k_scaler[layer], v_scale=ocache.v_scaler[layer])
    check_out(outs[layer], wo, f"layer {layer} vs closed form over the finalized cache")


def test_paged_orchestration_end_to_end():
  """Insert prompts, then decode steps of fill_new_pages / indices / paged
  append / paged attention, checked per step against dense attention over
  the oracle's gathered pages."""
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import layers
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData
  from jetstream_pt_amd.page_attention_manager import PageAttentionManager
  g = torch.Generator().manual_seed(309)
  rng = np.random.default_rng(309)
  b, hq, hkv, p, ps, d, mp = 6, 16, 4, 96, 64, 128, 8
  env = JetEngineEnvironment(JetEngineEnvironmentData(batch_size=b, paged_attention_total_num_pages=p,
                                                      paged_attention_page_size=ps))
  pam = PageAttentionManager(b, p, ps, mp, free_list_order=rng.permutation(p).astype(np.int32))
  cache = cm.PageKVCacheGenerate.empty((hkv, p, ps, d), DEV, env)
  pk, pv = cache.state()
  lens = np.array([63, 0, 64, 200, 1, 127], dtype=np.int32)
  for slot, n in enumerate(lens):
    if n:
      k, v = rnd(g, (1, hkv, int(n), d)), rnd(g, (1, hkv, int(n), d))
      _, idx = pam.reserve_pages_insert(slot, int(n))
      pam.insert_prefill_cache([(k.to(DEV), v.to(DEV))], [(pk, pv)], idx)
  sm = 1 / math.sqrt(d)
  kern = layers.AttentionKernel(env, 0, sm_scale_paged=sm)
  for step in range(3):
    pam.fill_new_pages(lens)
    pti = pam.get_page_token_indices(lens)
    xq, xk, xv = rnd(g, (b, hq, 1, d)), rnd(g, (b, hkv, 1, d)), rnd(g, (b, hkv, 1, d))
    obj = cm.PageKVCacheGenerate(pk, pv, pam, pti, None, env=env)
    out = kern(*to_dev(xq, xk, xv), None, obj)
    assert out.shape == (b, hq, 1, d)
    want = OA.paged_attention(xq.squeeze(2).float(), pk.cpu(), pv.cpu(), pam.lengths, pam.page_indices, sm_scale=sm)
    check_out(out.squeeze(2), want, f"step {step}")
    # the appended row is the step's token
    for j in range(pti.shape[1]):
      page, tok, slot = (int(x) for x in pti[:, j])
      assert torch.equal(pk[:, page, tok % ps].cpu(), xk[slot, :, 0])
    lens = np.where(lens == 0, 0, lens + 1).astype(np.int32)


def test_ragged_mqa_single_head_entry_points():
  """ragged_mqa / ragged_mqa_reference (reference attention_kernel.py:122, :342):
  one KV head, q (B, T, D), k/v (B, S, D) or stacked with `layer`; same numbers
  as the head's slice of ragged_mha; shard_kv_heads hands the function back."""
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(320)
  nl, b, t, s, d = 2, 4, 4, 256, 128
  end = torch.tensor([256, 3, 0, 130], dtype=torch.int32)
  q = rnd(g, (b, t, d))
  k = torch.randint(-127, 128, (nl, b, s, d), generator=g, dtype=torch.int8)
  v = torch.randint(-127, 128, (nl, b, s, d), generator=g, dtype=torch.int8)
  ks = (torch.rand((nl, b, 1, s), generator=g) * 0.045 + 0.005).to(torch.bfloat16)
  vs = (torch.rand((nl, b, 1, s), generator=g) * 0.045 + 0.005).to(torch.bfloat16)
  gq, gk, gv, gks, gvs, gend = to_dev(q, k, v, ks, vs, end)
  for fn in (ak.ragged_mqa, ak.ragged_mqa_reference):
    for layer in range(nl):
      wo, wm, wl = OA.closed_form(q.unsqueeze(1), k[layer].unsqueeze(1), v[layer].unsqueeze(1),
                                  lengths=end, k_scale=ks[layer].unsqueeze(-1), v_scale=vs[layer].unsqueeze(-1))
      o, (m, l) = fn(gq, gk, gv, layer, None, gend, None, None, gks, gvs, quantized=True)
      assert o.shape == (b, t, d) and m.shape == (b, t) and l.shape == (b, t)
      check_out(o.unsqueeze(1), wo, f"{fn.__name__} layer {layer}")
      live = (end > 0).reshape(b, 1, 1, 1).expand(b, 1, t, 1)
      check_stats(m, l, wm, wl, live)
    # unstacked, no scalers (bf16 cache)
    kb, vb = rnd(g, (b, s, d)), rnd(g, (b, s, d))
    wo, _, _ = OA.closed_form(q.unsqueeze(1), kb.unsqueeze(1), vb.unsqueeze(1), lengths=end)
    o, _ = fn(gq, kb.to(DEV), vb.to(DEV), 0, None, gend)
    check_out(o.unsqueeze(1), wo, f"{fn.__name__} bf16")
  assert ak.shard_kv_heads(ak.call_paged_attention, None, "x") is ak.call_paged_attention
  assert ak.check_status() == ak.STATUS_SLOT_FULL  # no launch gave up; slot 0 sits at the cache's capacity


@pytest.mark.parametrize("hq,hkv", [(4, 4), (8, 2)])
def test_prefill_through_the_int8_kernel_with_pretend_quantised_cache(hq, hkv):
  """KVCachePrefill(kv_quantize=True) (reference cache_manager.py:55-58): update()
  returns the 8-tuple with bf16 ones as scalers and Int8KVAttentionKernel
  unpacks it (layers.py:677-698) for a prefill-shaped call, T > 1 with a causal
  mask; checked against the oracle's classes on the same inputs and against the
  closed form.  Such a call uses the shape-generic kernel: it must not create
  a split-KV workspace (they are sized by the query rows)."""
  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import layers
  g = torch.Generator().manual_seed(321)
  t, d = 40, 128
  oenv, genv = _envs(False, True, 1, 1)
  xq, xk, xv = rnd(g, (1, hq, t, d)), rnd(g, (1, hkv, t, d)), rnd(g, (1, hkv, t, d))
  mask = torch.full((t, t), -math.inf).triu(1).reshape(1, 1, t, t)
  ocache, gcache = okv.KVCachePrefill(kv_quantize=True), cm.KVCachePrefill(kv_quantize=True)
  gq, gk, gv, gmask = to_dev(xq, xk, xv, mask)
  ret = gcache.update(gk, gv)
  assert len(ret) == 8 and ret[2] is None and ret[3] is None and ret[6] is None and ret[7] is None
  assert ret[0] is gk and ret[1] is gv
  for ones in ret[4:6]:
    assert ones.shape == (1, 1, t, 1) and ones.dtype == torch.bfloat16 and bool((ones == 1).all())
  n_dense, n_shared = len(ak._dense_workspaces), len(ak._workspaces)
  torch.cuda.synchronize()
  before = torch.cuda.memory_allocated()
  got = layers.Int8KVAttentionKernel(genv, 0)(gq, gk, gv, gmask, gcache)
  torch.cuda.synchronize()
  assert (len(ak._dense_workspaces), len(ak._workspaces)) == (n_dense, n_shared)
  assert torch.cuda.memory_allocated() - before <= 4 * got.numel() * got.element_size() + (1 << 20)
  assert got.shape == (1, hq, t, d)
  assert gcache.state()[0] is gk and gcache.state()[1] is gv
  exact, _, _ = OA.closed_form(xq, xk, xv, mask=mask.repeat(1, 1, hq // hkv, 1))  # rows: (q head of the group, t)
  check_out(got, exact, "prefill closed form")
  if hq == hkv:
    # the reference's own arithmetic (bf16 scores, dense_attention :605-625; its mask
    # only broadcasts over folded query heads when there is one per KV head)
    want = OInt8Attn(oenv, 0)(xq, xk, xv, mask, ocache)
    assert (got.cpu().double() - want.double()).abs().max() < 5e-2


def test_long_prefill_shaped_dense_call_allocates_no_workspace():
  """dense_attention with T = 1024 query rows: before the fix a 1.4 GiB
  zero-filled workspace was built (and cached) for a kernel that never used it."""
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(322)
  t, hq, hkv, d = 1024, 32, 8, 128
  q, k, v = (rnd(g, (1, h, t, d)).to(DEV) for h in (hq, hkv, hkv))
  from jetstream_pt_amd import _ffi
  a = _ffi.AttnArgs(batch=1, q_heads=hq, kv_heads=hkv, q_rows=t, seq=t)
  assert _ffi.lib.jpt_attn_workspace_bytes(a) == _ffi.ATTN_WS_STATE_BYTES
  n_dense = len(ak._dense_workspaces)
  torch.cuda.synchronize()
  torch.cuda.reset_peak_memory_stats()
  before = torch.cuda.memory_allocated()
  o = ak.dense_attention(q, k, v)
  torch.cuda.synchronize()
  assert torch.cuda.max_memory_allocated() - before <= 2 * o.numel() * o.element_size() + (1 << 20)
  assert len(ak._dense_workspaces) == n_dense
  rows = torch.tensor([0, 1, 500, 1023])
  want, _, _ = OA.closed_form(q[:, :, rows].cpu(), k.cpu(), v.cpu())
  check_out(o[:, :, rows], want, "rows of a long prefill-shaped call")
