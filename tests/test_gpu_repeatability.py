"""GPU: the single-launch decode attention gives the same bits every time, and
its cross-workgroup protocols survive what the host can throw at them.

Slots cut in two are folded by the two groups of waves of one workgroup through
LDS; slots cut in three or more park float32 partials in memory, count their
arrival, and are folded by whichever worker's producer wave asks the hand-out
counter first.  Who folds is decided by timing; WHAT is folded, and in which
order, is not - so every launch on the same inputs must produce bit-identical
outputs, row maxima and denominators.  Each case is launched REPEATS times and
compared with its first launch; the first difference stops the test.

Also here: the hand-out counters hold whatever an earlier launch left in them
(tested with values near 2^32 and inside the cycle), and jpt_attn_status puts
the counters of a workspace back after a launch that gave up (the condition is
written into the state block by the host: no kernel misbehaves in any test).
"""

import ctypes
import math

import numpy as np
import pytest
import torch

from conftest import attention_close
from oracle import attention as OA

pytestmark = pytest.mark.gpu
DEV = "cuda"
REPEATS = 200

# words of the workspace's state block (csrc/attn_plan.h)
STATUS, N_ENTRIES, N_MERGES, ARRIVALS_AT, ARRIVALS_COUNT, HAND_OUT, HAND_OUT_STRIDE, HAND_OUT_COUNTERS = 0, 2, 3, 4, 5, 16, 16, 8


def _state(ws):
  return ws.buf[:4096].view(torch.int32)


def _int8_cache(g, b, hkv, s, d, hs=1, sdt=torch.float32):
  k = torch.randint(-127, 128, (b, hkv, s, d), generator=g, dtype=torch.int8)
  v = torch.randint(-127, 128, (b, hkv, s, d), generator=g, dtype=torch.int8)
  ks = (torch.rand((b, hs, s, 1), generator=g) * 0.045 + 0.005).to(sdt)
  vs = (torch.rand((b, hs, s, 1), generator=g) * 0.045 + 0.005).to(sdt)
  return k, v, ks, vs


def _repeat(launch, what):
  """launch() -> tuple of tensors; REPEATS launches, all equal to the first, bit for bit."""
  from jetstream_pt_amd import attention_kernel as ak
  first = [t.clone() for t in launch()]
  torch.cuda.synchronize()
  for i in range(1, REPEATS):
    again = launch()
    for j, (x, y) in enumerate(zip(first, again)):
      # NaN-proof and exact: compare the bits
      same = torch.equal(x.view(torch.int16 if x.element_size() == 2 else torch.int32 if x.element_size() == 4 else torch.int8),
                         y.view(torch.int16 if y.element_size() == 2 else torch.int32 if y.element_size() == 4 else torch.int8))
      assert same, f"{what}: launch {i} differs from launch 0 in output {j}"
  assert ak.check_status() & ~ak.STATUS_SLOT_FULL == 0
  return first


@pytest.mark.parametrize("kind", ["int8_f32", "int8_bf16_perhead", "bf16"])
def test_ragged_launch_is_bit_repeatable(kind):
  """32/8 heads; whole slots, slots cut in two (paired through LDS) and slots cut in
  3..16 (partials, arrival counters, merge hand-out) in one launch, with the step's
  token fused (raw bf16 for the int8 caches: the launch quantises it)."""
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(41)
  b, hq, hkv, s, d = 12, 32, 8, 4096, 128
  lens = torch.tensor([4095, 100, 200, 3000, 700, 0, 1500, 2500, 31, 513, 300, 450], dtype=torch.int32)
  q = torch.randn((b, hq, 1, d), generator=g).to(torch.bfloat16)
  xk = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16)
  xv = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16)
  hs = hkv if "perhead" in kind else 1
  sdt = torch.bfloat16 if "bf16_" in kind else torch.float32
  if kind == "bf16":
    k = torch.randn((b, hkv, s, d), generator=g).to(torch.bfloat16)
    v = torch.randn((b, hkv, s, d), generator=g).to(torch.bfloat16)
    gks = gvs = None
    kw = dict(new_key=xk.to(DEV), new_value=xv.to(DEV))
  else:
    k, v, ks, vs = _int8_cache(g, b, hkv, s, d, hs, sdt)
    gks, gvs = ks.to(DEV), vs.to(DEV)
    kw = dict(new_key=torch.zeros((b, hkv, 1, d), dtype=torch.int8, device=DEV),
              new_value=torch.zeros((b, hkv, 1, d), dtype=torch.int8, device=DEV),
              new_k_scaler=torch.zeros((b, hs), dtype=sdt, device=DEV),
              new_v_scaler=torch.zeros((b, hs), dtype=sdt, device=DEV),
              new_key_raw=xk.to(DEV), new_value_raw=xv.to(DEV), new_rounding="trunc")
  gq, gk, gv, glens = q.to(DEV), k.to(DEV), v.to(DEV), lens.to(DEV)
  plan, _ = ak.precompute_ragged_block_indices(glens, b, hq, hkv, s)
  st = _state(plan.workspace).cpu()
  assert st[N_MERGES] >= 4, "the case must have slots cut in three or more"

  def launch():
    o, (m, l) = ak.ragged_mha(gq, gk, gv, 0, None, plan.lengths, plan, None, gks, gvs, **kw)
    outs = [o, m, l]
    if kind != "bf16":
      outs += [kw["new_key"], kw["new_value"], kw["new_k_scaler"], kw["new_v_scaler"]]
    return outs

  first = _repeat(launch, kind)
  # ... and the bits are the right ones
  k2, v2 = k.clone(), v.clone()
  ar, idx = torch.arange(b), lens.long()
  if kind == "bf16":
    k2[ar, :, idx], v2[ar, :, idx] = xk[:, :, 0], xv[:, :, 0]
    ks2 = vs2 = None
  else:
    k2[ar, :, idx], v2[ar, :, idx] = first[3].cpu()[:, :, 0], first[4].cpu()[:, :, 0]
    ks2, vs2 = ks.clone(), vs.clone()
    ks2[ar, :, idx, 0], vs2[ar, :, idx, 0] = first[5].cpu().reshape(b, hs), first[6].cpu().reshape(b, hs)
  wo, _, _ = OA.closed_form(q, k2, v2, lengths=lens + 1, k_scale=ks2, v_scale=vs2)
  assert attention_close(first[0], wo)


def test_dense_launches_are_bit_repeatable():
  """No lengths: every slot is cut alike.  1024 positions a slot at 32 KV heads are cut
  in two (all pairs, the mask's tile path); 8192 positions at 8 KV heads in ten."""
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(42)
  for b, hq, hkv, s, masked in ((8, 32, 32, 1024, True), (8, 32, 8, 8192, False)):
    d = 128
    q = torch.randn((b, hq, 1, d), generator=g).to(torch.bfloat16)
    k = torch.randn((b, hkv, s, d), generator=g).to(torch.bfloat16)
    v = torch.randn((b, hkv, s, d), generator=g).to(torch.bfloat16)
    mask = None
    lens = torch.full((b,), s, dtype=torch.int32)
    if masked:
      lens = torch.randint(1, s + 1, (b,), generator=g, dtype=torch.int32)
      mask = torch.full((b, 1, 1, s), float("-inf"))
      for bi in range(b):
        mask[bi, :, :, :int(lens[bi])] = 0
    gq, gk, gv, gmask = q.to(DEV), k.to(DEV), v.to(DEV), None if mask is None else mask.to(DEV)

    def launch():
      o, (m, l) = ak.flash_attention(gq, gk, gv, 0, mask=gmask)
      return [o, m, l]

    first = _repeat(launch, f"dense {hq}/{hkv} x {s}")
    wo, _, _ = OA.closed_form(q, k, v, lengths=lens)
    assert attention_close(first[0], wo)


@pytest.mark.parametrize("kind", ["bf16", "int8"])
def test_paged_launch_is_bit_repeatable(kind):
  """64/8 heads (eight query rows a KV head), pages of 64 in random order; slots of one
  page up to 40 pages, so the launch has whole slots, pairs and merges."""
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(43)
  rng = np.random.default_rng(43)
  hq, hkv, ps, d, mp = 64, 8, 64, 128, 40
  lens = np.array([2560, 64, 100, 1900, 700, 1, 1500, 2000, 333, 1024], dtype=np.int32)
  b = len(lens)
  need = [-(-int(n) // ps) for n in lens]
  pages = sum(need) + 5
  perm = rng.permutation(pages)
  table = np.full((b, mp), pages - 1, dtype=np.int32)
  at = 0
  for bi in range(b):
    table[bi, :need[bi]] = perm[at:at + need[bi]]
    at += need[bi]
  q = torch.randn((b, hq, d), generator=g).to(torch.bfloat16)
  ksp = vsp = None
  if kind == "int8":
    kp = torch.randint(-127, 128, (hkv, pages, ps, d), generator=g, dtype=torch.int8)
    vp = torch.randint(-127, 128, (hkv, pages, ps, d), generator=g, dtype=torch.int8)
    ksp = torch.rand((1, pages, ps), generator=g) * 0.045 + 0.005
    vsp = torch.rand((1, pages, ps), generator=g) * 0.045 + 0.005
  else:
    kp = torch.randn((hkv, pages, ps, d), generator=g).to(torch.bfloat16)
    vp = torch.randn((hkv, pages, ps, d), generator=g).to(torch.bfloat16)
  gq, gk, gv = q.to(DEV), kp.to(DEV), vp.to(DEV)
  gks, gvs = (None, None) if ksp is None else (ksp.to(DEV), vsp.to(DEV))
  glens, gtable = torch.from_numpy(lens).to(DEV), torch.from_numpy(table).to(DEV)
  sm = 1 / math.sqrt(d)

  def launch():
    return [ak.call_paged_attention(None, gq, gk, gv, glens, gtable, sm_scale=sm, k_scaler=gks, v_scaler=gvs)]

  first = _repeat(launch, f"paged {kind}")
  want = OA.paged_attention(q.float(), kp, vp, torch.from_numpy(lens), torch.from_numpy(table), sm_scale=sm,
                            k_scale_pages=ksp, v_scale_pages=vsp)
  assert attention_close(first[0], want)


@pytest.mark.parametrize("found", [2 ** 32 - 3, 2 ** 31 + 5, 1, 7, 70, 71, 72, 1000])
def test_merge_hand_out_counter_takes_any_start(found):
  """A dense plan is made once per shape and reused for the life of the process: its
  hand-out counters are never reset between launches.  Whatever a launch finds in
  them - here written by the host: values near 2^32, values inside the cycle of a
  launch's asks, values just outside it - every merge is done exactly once: the
  output equals the one of a freshly planned launch bit for bit, and no wave gives up."""
  from jetstream_pt_amd import attention_kernel as ak
  g = torch.Generator().manual_seed(44)
  b, hq, hkv, s, d = 8, 32, 8, 8192, 128  # every slot is cut in ten: 64 merges, eight a counter
  q = torch.randn((b, hq, 1, d), generator=g).to(torch.bfloat16)
  k, v, ks, vs = _int8_cache(g, b, hkv, s, d)
  gq, gk, gv, gks, gvs = q.to(DEV), k.to(DEV), v.to(DEV), ks.to(DEV), vs.to(DEV)
  want, (wm, wl) = ak.flash_attention(gq, gk, gv, 0, k_scaler=gks, v_scaler=gvs)
  key = next(kk for kk in ak._dense_workspaces if kk[2:] == (b, hq, hkv, 1, s))
  ws = ak._dense_workspaces[key]
  st = _state(ws)
  assert int(st[N_MERGES]) == b, "every slot must be cut in three or more"
  torch.cuda.synchronize()
  for c in range(HAND_OUT_COUNTERS):
    assert int(st[HAND_OUT + c * HAND_OUT_STRIDE]) == 0, "a complete launch leaves its counters where it found them"
  for launch in range(3):  # the first finds `found`, the next ones what that launch left
    if launch == 0:
      value = found if found < 2 ** 31 else found - 2 ** 32
      for c in range(HAND_OUT_COUNTERS):
        st[HAND_OUT + c * HAND_OUT_STRIDE] = value
    got, (m, l) = ak.flash_attention(gq, gk, gv, 0, k_scaler=gks, v_scaler=gvs)
    assert torch.equal(got, want) and torch.equal(m, wm) and torch.equal(l, wl), f"launch {launch} after {found}"
  assert ak.check_status() == 0
  wo, _, _ = OA.closed_form(q, k, v, lengths=torch.full((b,), s, dtype=torch.int32), k_scale=ks, v_scale=vs)
  assert attention_close(want, wo)
  for c in range(HAND_OUT_COUNTERS):  # put back, for whoever uses this shape's plan next
    st[HAND_OUT + c * HAND_OUT_STRIDE] = 0


def test_status_call_resets_the_counters_after_a_launch_that_gave_up():
  """What a launch that gave up leaves behind - arrival counts without their merge,
  hand-out counters mid-cycle - must not reach the next launch on the plan.  The
  host writes that state (no kernel gives up here): jpt_attn_status reports the bit
  once, clears the counters, and the plan works again."""
  from jetstream_pt_amd import _ffi, attention_kernel as ak
  g = torch.Generator().manual_seed(45)
  b, hq, hkv, s, d = 6, 32, 8, 4096, 128
  lens = torch.tensor([4000, 3000, 100, 2000, 800, 4096], dtype=torch.int32)
  q = torch.randn((b, hq, 1, d), generator=g).to(torch.bfloat16)
  k, v, ks, vs = _int8_cache(g, b, hkv, s, d)
  gq, gk, gv, gks, gvs, glens = q.to(DEV), k.to(DEV), v.to(DEV), ks.to(DEV), vs.to(DEV), lens.to(DEV)
  plan, _ = ak.precompute_ragged_block_indices(glens, b, hq, hkv, s)
  want, (wm, wl) = ak.ragged_mha(gq, gk, gv, 0, None, plan.lengths, plan, None, gks, gvs)
  torch.cuda.synchronize()
  st = _state(plan.workspace)
  assert int(st[N_MERGES]) >= 3
  at, count = int(st[ARRIVALS_AT]), int(st[ARRIVALS_COUNT])
  assert count == b * hkv and at * 4 >= 65536
  arrivals = plan.workspace.buf.view(torch.int32)[at:at + count]
  assert int(arrivals.abs().max()) == 0, "a complete launch leaves every arrival counter at zero"
  arrivals.fill_(2)
  for c in range(HAND_OUT_COUNTERS):
    st[HAND_OUT + c * HAND_OUT_STRIDE] = 3
  st[STATUS] = ak.STATUS_GAVE_UP | ak.STATUS_SLOT_FULL
  with pytest.raises(RuntimeError):
    ak.check_status(plan)
  torch.cuda.synchronize()
  assert int(arrivals.abs().max()) == 0 and int(st[STATUS]) == 0
  assert all(int(st[HAND_OUT + c * HAND_OUT_STRIDE]) == 0 for c in range(HAND_OUT_COUNTERS))
  got, (m, l) = ak.ragged_mha(gq, gk, gv, 0, None, plan.lengths, plan, None, gks, gvs)
  assert torch.equal(got, want) and torch.equal(m, wm) and torch.equal(l, wl)
  word = ctypes.c_int32(-1)
  _ffi.check(_ffi.lib.jpt_attn_status(_ffi.ptr(plan.workspace.buf), _ffi.stream(), ctypes.byref(word)))
  assert word.value == 0
