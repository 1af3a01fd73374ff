"""GPU parity on randomly drawn shapes: the attention entry points against the
float64 closed form, and the paged attention launch that appends the token
against the separate append launch.  Seeds are fixed; every case prints its
parameters before it runs.

Tolerances: outputs max-abs 1e-2 (plus the bf16 output's own half-ulp where
|expected| >= 2: conftest.attention_bound, the same function every attention
test uses), row max / denominator rtol 1e-3; pages, codes and scales bit for bit."""

import math

import numpy as np
import pytest
import torch

from conftest import attention_close
from oracle import attention as OA

pytestmark = pytest.mark.gpu
DEV = "cuda"


_close = attention_close


def _dev(*xs):
  return [None if x is None else x.to(DEV) for x in xs]


@pytest.mark.parametrize("block", range(4))
def test_random_ragged_dense_paged_attention(block):
  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd.quantize import quantize_kv
  for it in range(12):
    seed = 7000 + 100 * block + it
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    hq, hkv = [(32, 8), (8, 8), (16, 1), (64, 8), (32, 32), (8, 2), (16, 16), (4, 1), (12, 4)][rng.integers(9)]
    b, d = int(rng.integers(1, 41)), 128
    s = int(rng.choice([128, 256, 1024, 4096]))
    kind = ["int8_f32", "int8_bf16_perhead", "bf16", "int8_f32_perhead"][rng.integers(4)]
    mode = int(rng.integers(4))
    if mode == 0:
      lens = rng.integers(0, s + 1, b)
    elif mode == 1:
      lens = rng.choice([0, 1, 31, 32, 33, 127, 128, 129, s - 1, s], b)
    elif mode == 2:
      lens = np.minimum(s, rng.lognormal(math.log(max(s // 8, 2)), 1.0, b).astype(np.int64))
    else:
      lens = np.full(b, s if rng.integers(2) else int(rng.integers(0, s + 1)))
    new_tok = bool(rng.integers(2))
    raw = new_tok and kind.startswith("int8") and bool(rng.integers(2))
    lens = np.minimum(lens, s - 1 if new_tok else s).astype(np.int32)
    desc = f"seed {seed} hq {hq} hkv {hkv} b {b} s {s} {kind} lens-mode {mode} new {new_tok} raw {raw}"
    print(desc, flush=True)
    end = torch.from_numpy(lens)
    q = torch.randn((b, hq, 1, d), generator=g).to(torch.bfloat16)
    hs = hkv if "perhead" in kind else 1
    sdt = torch.bfloat16 if "bf16" in kind else torch.float32
    if kind == "bf16":
      k = torch.randn((b, hkv, s, d), generator=g).to(torch.bfloat16)
      v = torch.randn((b, hkv, s, d), generator=g).to(torch.bfloat16)
      ks = vs = None
    else:
      k = torch.randint(-127, 128, (b, hkv, s, d), generator=g, dtype=torch.int8)
      v = torch.randint(-127, 128, (b, hkv, s, d), generator=g, dtype=torch.int8)
      ks = (torch.rand((b, hs, s, 1), generator=g) * 0.045 + 0.005).to(sdt)
      vs = (torch.rand((b, hs, s, 1), generator=g) * 0.045 + 0.005).to(sdt)
    gq, gk, gv, gks, gvs, gend = _dev(q, k, v, ks, vs, end)
    kw = {}
    k2, v2, ks2, vs2, end2 = k, v, ks, vs, end
    if new_tok:
      xk = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16)
      xv = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16)
      gxk, gxv = _dev(xk, xv)
      if kind == "bf16":
        nk, nv, nks, nvs = gxk, gxv, None, None
      else:
        nk, nv, nks, nvs = quantize_kv(gxk, gxv, rounding="trunc", scale_heads=hs, scale_dtype=sdt)
      # expected: the token appended at position len
      k2, v2 = k.clone(), v.clone()
      idx, ar = torch.from_numpy(lens.astype(np.int64)), torch.arange(b)
      k2[ar, :, idx] = nk.cpu()[:, :, 0]
      v2[ar, :, idx] = nv.cpu()[:, :, 0]
      if ks is not None:
        ks2, vs2 = ks.clone(), vs.clone()
        ks2[ar, :, idx, 0] = nks.cpu().reshape(b, hs)
        vs2[ar, :, idx, 0] = nvs.cpu().reshape(b, hs)
      end2 = end + 1
      if raw:
        ok, ov = torch.full_like(nk, 77), torch.full_like(nv, 77)
        oks, ovs = torch.full_like(nks, -1.0), torch.full_like(nvs, -1.0)
        kw = dict(new_key=ok, new_value=ov, new_k_scaler=oks, new_v_scaler=ovs, new_key_raw=gxk,
                  new_value_raw=gxv, new_rounding="trunc")
      else:
        kw = dict(new_key=nk, new_value=nv, new_k_scaler=nks, new_v_scaler=nvs)
    wo, wm, wl = OA.closed_form(q, k2, v2, lengths=end2, k_scale=ks2, v_scale=vs2)
    o, (m, l) = ak.ragged_mha(gq, gk, gv, 0, None, gend, None, None, gks, gvs, **kw)
    assert _close(o, wo), "ragged " + desc
    live = end2 > 0
    assert torch.allclose(m.double().cpu().reshape(b, hq)[live], wm.double().reshape(b, hq)[live], rtol=1e-3, atol=1e-4), desc
    assert torch.allclose(l.double().cpu().reshape(b, hq)[live], wl.double().reshape(b, hq)[live], rtol=1e-3), desc
    if raw:
      assert torch.equal(ok, nk) and torch.equal(ov, nv) and torch.equal(oks, nks) and torch.equal(ovs, nvs), "codes " + desc
    if not new_tok and s <= 1024 and (lens > 0).all():
      # the same lengths as an additive 0 / -inf mask through the dense and flash entry points
      mask = torch.full((b, 1, 1, s), float("-inf"))
      for bi in range(b):
        mask[bi, :, :, :int(lens[bi])] = 0
      fo, _ = ak.flash_attention(gq, gk, gv, 0, k_scaler=gks, v_scaler=gvs, mask=mask.to(DEV))
      assert _close(fo, wo), "flash " + desc
      do = ak.dense_attention(gq, gk, gv, k_scaler=gks, v_scaler=gvs, mask=mask.to(DEV))
      assert _close(do, wo), "dense " + desc
    if kind in ("int8_f32", "bf16") and not new_tok and s <= 1024:
      # the same cache cut into pages in random order
      ps = int(rng.choice([32, 64, 128]))
      mp = s // ps
      need = [-(-int(n) // ps) for n in lens]
      pages = sum(need) + 3
      perm = rng.permutation(pages)
      table = np.full((b, mp), pages - 1, dtype=np.int32)
      kp = torch.zeros((hkv, pages, ps, d), dtype=k.dtype)
      vp = torch.zeros_like(kp)
      ksp = vsp = None
      if ks is not None:
        ksp, vsp = torch.full((1, pages, ps), 0.01), torch.full((1, pages, ps), 0.01)
      at = 0
      for bi in range(b):
        for j in range(need[bi]):
          pg = int(perm[at])
          at += 1
          table[bi, j] = pg
          kp[:, pg] = k[bi, :, j * ps:(j + 1) * ps]
          vp[:, pg] = v[bi, :, j * ps:(j + 1) * ps]
          if ks is not None:
            ksp[0, pg] = ks[bi, 0, j * ps:(j + 1) * ps, 0]
            vsp[0, pg] = vs[bi, 0, j * ps:(j + 1) * ps, 0]
      got = ak.call_paged_attention(None, gq.squeeze(2), kp.to(DEV), vp.to(DEV), lens, table, sm_scale=1 / math.sqrt(d),
                                    k_scaler=None if ksp is None else ksp.to(DEV),
                                    v_scaler=None if vsp is None else vsp.to(DEV))
      assert _close(got, wo), "paged " + desc


@pytest.mark.parametrize("block", range(3))
def test_random_paged_attention_that_appends(block):
  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData
  from jetstream_pt_amd.quantize import quantize_kv
  for it in range(25):
    seed = 9000 + 100 * block + it
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    hkv = int(rng.choice([1, 2, 4, 8, 16, 32]))
    rep = min(int(rng.choice([1, 2, 4, 8])), 64 // hkv)
    hq = hkv * rep
    ps, mp, b, d = int(rng.choice([32, 64, 128])), int(rng.integers(1, 9)), int(rng.integers(1, 33)), 128
    kind = ["bf16", "int8_codes", "int8_raw", "int8_raw_perhead_bf16"][rng.integers(4)]
    cap = mp * ps
    lens = rng.integers(0, cap + 1, b).astype(np.int32)
    for j, special in enumerate([0, cap, ps, ps - 1][:b]):
      lens[j] = special  # an inactive slot, a full one, a page boundary, the row before it
    need = [min(mp, int(n) // ps + 1) if n else 0 for n in lens]  # the page of position n is there already
    pages = sum(need) + 2
    perm = rng.permutation(pages - 1).astype(np.int32)  # the last page is the table's filler
    table = np.full((b, mp), pages - 1, dtype=np.int32)
    at = 0
    for bi in range(b):
      table[bi, :need[bi]] = perm[at:at + need[bi]]
      at += need[bi]
    desc = f"seed {seed} hq {hq} hkv {hkv} b {b} ps {ps} mp {mp} {kind}"
    print(desc, flush=True)
    int8, per_head = kind != "bf16", kind.endswith("perhead_bf16")
    sdt, hs = (torch.bfloat16, hkv) if per_head else (torch.float32, 1)
    if int8:
      kp = torch.randint(-127, 128, (hkv, pages, ps, d), generator=g, dtype=torch.int8)
      vp = torch.randint(-127, 128, (hkv, pages, ps, d), generator=g, dtype=torch.int8)
      ksp = (torch.rand((hs, pages, ps), generator=g) * 0.045 + 0.005).to(sdt)
      vsp = (torch.rand((hs, pages, ps), generator=g) * 0.045 + 0.005).to(sdt)
    else:
      kp = torch.randn((hkv, pages, ps, d), generator=g).to(torch.bfloat16)
      vp = torch.randn((hkv, pages, ps, d), generator=g).to(torch.bfloat16)
      ksp = vsp = None
    q = torch.randn((b, hq, d), generator=g).to(torch.bfloat16)
    xk = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16)
    xv = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16)
    gq, gxk, gxv = _dev(q, xk, xv)
    glens, gtable = torch.from_numpy(lens).to(DEV), torch.from_numpy(table).to(DEV)
    act = (lens > 0) & (lens < cap)
    active = np.nonzero(act)[0]
    idx = np.stack([table[active, lens[active] // ps], np.arange(len(active)) * ps + lens[active] % ps,
                    active]).astype(np.int32)
    clone = lambda t: None if t is None else t.clone().to(DEV)
    wk, wv, wks, wvs = clone(kp), clone(vp), clone(ksp), clone(vsp)
    env = JetEngineEnvironment(JetEngineEnvironmentData(paged_attention_total_num_pages=pages,
                                                        paged_attention_page_size=ps))
    if len(active):  # the separate append launch, then attention over the longer slots
      ref = cm.Int8PageKVCacheGenerate(wk, wv, wks, wvs, None, idx, env=env) if int8 \
          else cm.PageKVCacheGenerate(wk, wv, None, idx, env=env)
      ref.update(gxk, gxv, 0)
    after = np.where(act, lens + 1, lens).astype(np.int32)
    want = OA.paged_attention(q.float(), wk.cpu(), wv.cpu(), torch.from_numpy(after), torch.from_numpy(table),
                              sm_scale=1.0, k_scale_pages=None if wks is None else wks.cpu().float(),
                              v_scale_pages=None if wvs is None else wvs.cpu().float())
    fk, fv, fks, fvs = clone(kp), clone(vp), clone(ksp), clone(vsp)
    if kind == "bf16":
      append = dict(new_key=gxk, new_value=gxv)
    elif kind == "int8_codes":
      ck, cv, cks, cvs = quantize_kv(gxk, gxv, rounding="trunc", scale_heads=hs, scale_dtype=sdt)
      append = dict(new_key=ck, new_value=cv, new_k_scaler=cks, new_v_scaler=cvs)
    else:
      append = dict(new_key=torch.empty((b, hkv, 1, d), dtype=torch.int8, device=DEV),
                    new_value=torch.empty((b, hkv, 1, d), dtype=torch.int8, device=DEV),
                    new_k_scaler=torch.empty((b, hs), dtype=sdt, device=DEV),
                    new_v_scaler=torch.empty((b, hs), dtype=sdt, device=DEV),
                    new_key_raw=gxk, new_value_raw=gxv, new_rounding="trunc")
    got = ak.call_paged_attention(None, gq, fk, fv, glens, gtable, sm_scale=1.0, k_scaler=fks, v_scaler=fvs,
                                  append=append)
    assert torch.equal(fk, wk) and torch.equal(fv, wv), "pages " + desc
    if int8:
      assert torch.equal(fks, wks) and torch.equal(fvs, wvs), "scale pages " + desc
    live = torch.from_numpy(act)
    if live.any():
      assert _close(got.float()[live], want.float()[live]), "outputs " + desc
