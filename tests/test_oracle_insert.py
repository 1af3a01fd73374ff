"""Pins the oracle's restatement of the engine's prefill -> decode insert
(engine.py:371-626) by brute force on small shapes and by hand-worked cases."""

import torch

from oracle import Env
from oracle import insert as oins
from oracle import quant as oquant


def _state(env, batch, heads, seq, dim, layers, quantized, seed=0):
  g = torch.Generator().manual_seed(seed)
  dt = torch.int8 if quantized else torch.bfloat16
  def cache():
    if quantized:
      return torch.randint(-127, 128, (batch, heads, seq, dim), generator=g, dtype=torch.int8)
    return torch.randn((batch, heads, seq, dim), generator=g).to(dt)
  def scale():
    return torch.rand((batch, 1, seq, 1), generator=g).to(torch.bfloat16)
  if env.generate_cache_stacked:
    caches = [(torch.stack([cache() for _ in range(layers)]), torch.stack([cache() for _ in range(layers)]))]
    scales = [(torch.stack([scale() for _ in range(layers)]), torch.stack([scale() for _ in range(layers)]))]
  else:
    caches = [(cache(), cache()) for _ in range(layers)]
    scales = [(scale(), scale()) for _ in range(layers)]
  return dict(caches=caches, cache_scales=scales if quantized else None,
              mask=torch.zeros((batch, seq)), start=torch.zeros(batch, dtype=torch.int32),
              input_pos=torch.zeros(batch, dtype=torch.int32), lens=torch.zeros(batch, dtype=torch.int32))


def _clone(state):
  c = lambda x: x.clone()
  out = dict(state)
  out["caches"] = [(c(k), c(v)) for k, v in state["caches"]]
  if state["cache_scales"] is not None:
    out["cache_scales"] = [(c(k), c(v)) for k, v in state["cache_scales"]]
  for f in ("mask", "start", "input_pos", "lens"):
    out[f] = c(state[f])
  return out


def _layer(state, env, idx):
  if env.generate_cache_stacked:
    return state["caches"][0][0][idx], state["caches"][0][1][idx]
  return state["caches"][idx]


def _brute_rows(before, after, new, slot, positions):
  """Every element of `after` equals `before` except rows `positions` of `slot`,
  which hold the prompt's rows in order."""
  b, h, s, d = before.shape
  expect = before.clone()
  for t, p in enumerate(positions):
    for hh in range(h):
      expect[slot, hh, p, :] = new[hh, t, :]
  assert torch.equal(after, expect)


def test_no_wrap_left_aligned_float_writes_from_zero():
  env = Env(batch_size=3, num_layers=2, cache_len=16, ring_buffer=False)  # stacked
  st = _state(env, 3, 2, 16, 4, 2, quantized=False)
  before = _clone(st)
  g = torch.Generator().manual_seed(1)
  prefix = [(torch.randn((1, 2, 8, 4), generator=g).to(torch.bfloat16),
             torch.randn((1, 2, 8, 4), generator=g).to(torch.bfloat16)) for _ in range(2)]
  oins.insert(env, prefix, 5, st, slot=1)
  for idx in range(2):
    for which in (0, 1):
      _brute_rows(_layer(before, env, idx)[which], _layer(st, env, idx)[which], prefix[idx][which][0], 1, range(0, 8))
  # mask: positions [0, 5) open, the rest -inf; start 0; input_pos 5; lens 1
  assert st["mask"][1].tolist() == [0.0] * 5 + [float("-inf")] * 11
  assert st["mask"][0].tolist() == [0.0] * 16
  assert (st["start"][1], st["input_pos"][1], st["lens"][1]) == (0, 5, 1)


def test_ring_no_wrap_and_wrap_positions():
  env = Env(batch_size=2, num_layers=1, cache_len=16, ring_buffer=True)
  g = torch.Generator().manual_seed(2)
  prefix = [(torch.randn((1, 2, 8, 4), generator=g).to(torch.bfloat16),
             torch.randn((1, 2, 8, 4), generator=g).to(torch.bfloat16))]
  # current_position 12, prompt of 6 (padded 8): start 6, end 14 < 16 -> no wrap, rows 6..13
  st = _state(env, 2, 2, 16, 4, 1, quantized=False)
  before = _clone(st)
  oins.insert(env, prefix, 6, st, slot=0, current_position=12)
  _brute_rows(before["caches"][0][0], st["caches"][0][0], prefix[0][0][0], 0, range(6, 14))
  assert st["mask"][0].tolist() == [float("-inf")] * 6 + [0.0] * 6 + [float("-inf")] * 4
  assert int(st["start"][0]) == 6
  # current_position 3, prompt of 6 (padded 8): start -3 -> wrap: rows 13,14,15,0,1,2,3,4
  st = _state(env, 2, 2, 16, 4, 1, quantized=False)
  before = _clone(st)
  oins.insert(env, prefix, 6, st, slot=1, current_position=3)
  _brute_rows(before["caches"][0][1], st["caches"][0][1], prefix[0][1][0], 1, [13, 14, 15, 0, 1, 2, 3, 4])
  open_pos = {13, 14, 15, 0, 1, 2}
  assert st["mask"][1].tolist() == [0.0 if i in open_pos else float("-inf") for i in range(16)]
  assert int(st["start"][1]) == 13 and int(st["input_pos"][1]) == 6
  # end_insert == seq also takes the wrap path (strict <): start 8, rows 8..15
  st = _state(env, 2, 2, 16, 4, 1, quantized=False)
  before = _clone(st)
  oins.insert(env, prefix, 8, st, slot=0, current_position=16)
  _brute_rows(before["caches"][0][0], st["caches"][0][0], prefix[0][0][0], 0, range(8, 16))


def test_quantised_insert_matches_per_token_quantiser_and_untouched_rows():
  for ring, pos_kw, rows in ((False, {}, list(range(0, 8))), (True, dict(current_position=3), [13, 14, 15, 0, 1, 2, 3, 4])):
    env = Env(batch_size=2, num_layers=2, cache_len=16, ring_buffer=ring)
    st = _state(env, 2, 2, 16, 4, 2, quantized=True)
    before = _clone(st)
    g = torch.Generator().manual_seed(3)
    prefix = [(torch.randn((1, 2, 8, 4), generator=g).to(torch.bfloat16) * 3,
               torch.randn((1, 2, 8, 4), generator=g).to(torch.bfloat16)) for _ in range(2)]
    oins.insert(env, prefix, 6, st, slot=1, **pos_kw)
    for idx in range(2):
      for which in (0, 1):
        new = prefix[idx][which]
        codes = torch.empty((2, 8, 4), dtype=torch.int8)
        scales = torch.empty(8, dtype=torch.bfloat16)
        for t in range(8):  # one token at a time: (1, H, 1, D)
          c, s = oquant.quantize_insert(new[:, :, t:t + 1, :])
          codes[:, t, :] = c[0, :, 0, :]
          scales[t] = s.reshape(())
        if env.generate_cache_stacked:
          cache_b, cache_a = before["caches"][0][which][idx], st["caches"][0][which][idx]
          sc_b, sc_a = before["cache_scales"][0][which][idx], st["cache_scales"][0][which][idx]
        else:
          cache_b, cache_a = before["caches"][idx][which], st["caches"][idx][which]
          sc_b, sc_a = before["cache_scales"][idx][which], st["cache_scales"][idx][which]
        _brute_rows(cache_b, cache_a, codes, 1, rows)
        expect = sc_b.clone()
        for t, p in enumerate(rows):
          expect[1, 0, p, 0] = scales[t]
        assert torch.equal(sc_a, expect)


def test_insert_quantiser_dequantises_within_half_a_step():
  g = torch.Generator().manual_seed(4)
  x = (torch.randn((1, 4, 16, 8), generator=g) * 2).to(torch.bfloat16)
  codes, scales = oquant.quantize_insert(x)
  err = (codes.float() * scales.float() - x.float()).abs()
  # half a quantisation step plus the bf16 rounding of the reciprocal and product
  assert torch.all(err <= scales.float() * 0.5 + x.float().abs() * 2 ** -7 + 1e-6)
  assert int(codes.abs().max()) <= 127 + 1
