"""Prefill -> decode insert, restated from the reference engine (test infrastructure).

Follows jetstream_pt/engine.py: `_insert_no_wrap` (:371-488), `_insert_wrap`
(:491-581) and the dispatch in `insert` (:606-626).  Tensors are torch-CPU and
updated in place; the DecodeState fields the reference rebuilds (tokens aside)
are passed in as a dict: caches, cache_scales, mask, start, input_pos, lens.
"""

import torch

from . import quant


def _quantize(new_entry, compute_dtype=None):
  """quantize_tensor over (heads, dim) per token: engine.py:429-432 (axes -3, -1
  on (1, H, T, D)) and :548-551 (axes 1, 2 on (T, H, D)) are the same reduction.
  compute_dtype None works in the prompt's dtype, as the reference does; the
  HIP path works in the scalers' dtype, which is the same unless float32
  scalers are asked for."""
  return quant.quantize_insert(new_entry, compute_dtype=compute_dtype)


def insert_no_wrap(env, prefix_caches, prefix_seq_len, state, slot, current_position=0, compute_dtype=None):
  """engine.py:371-488."""
  seq = env.cache_sequence_length
  cur = current_position if env.ring_buffer else prefix_seq_len  # :380-383
  pos = cur - prefix_seq_len  # :385
  x = torch.arange(seq)
  state["mask"][slot] = torch.where((x < cur) & (x >= pos), 0.0, float("-inf"))  # :388-391
  state["start"][slot] = pos % seq  # :392-394
  state["input_pos"][slot] = prefix_seq_len  # :395
  caches, scales = state["caches"], state.get("cache_scales")
  quantized = scales is not None
  stacked = env.generate_cache_stacked
  for idx, (newk, newv) in enumerate(prefix_caches):
    t = newk.shape[2]
    if stacked:
      ck, cv = caches[0][0][idx], caches[0][1][idx]  # update_index [idx, slot, 0, pos, 0], :410, :461
    else:
      ck, cv = caches[idx]  # update_index [slot, 0, pos, 0], :421, :470
    if not quantized:
      ck[slot, :, pos:pos + t, :] = newk[0]  # dynamic_update_slice, :401-405
      cv[slot, :, pos:pos + t, :] = newv[0]
    else:
      sk, sv = (scales[0][0][idx], scales[0][1][idx]) if stacked else scales[idx]
      for c, s, new in ((ck, sk, newk), (cv, sv, newv)):
        vals, sc = _quantize(new, compute_dtype)  # (1, H, T, D), (1, 1, T, 1)
        c[slot, :, pos:pos + t, :] = vals[0]  # :443-447
        s[slot, :, pos:pos + t, :] = sc[0].to(s.dtype)  # :436-440
  state["lens"][slot] = 1  # :477
  return state


def insert_wrap(env, prefix_caches, prefix_seq_len, state, slot, current_position, compute_dtype=None):
  """engine.py:491-581 (ring buffer only; caches are never stacked there)."""
  seq = env.cache_sequence_length
  start_insert = (current_position - prefix_seq_len) % seq  # :498-500
  t = prefix_caches[0][0].shape[2]
  update_indexes = (torch.arange(t) + start_insert) % seq  # :502-505
  x = torch.arange(seq)
  if current_position > start_insert:  # :508-519
    cond = (x >= start_insert) & (x < current_position)
  else:
    cond = (x >= start_insert) | (x < current_position)
  state["mask"][slot] = torch.where(cond, 0.0, float("-inf"))  # :521-522
  state["start"][slot] = start_insert  # :523
  state["input_pos"][slot] = prefix_seq_len  # :524
  caches, scales = state["caches"], state.get("cache_scales")
  for idx, (newk, newv) in enumerate(prefix_caches):
    ck, cv = caches[idx]
    if scales is None:
      ck[slot][:, update_indexes, :] = newk[0]  # cache.at[slot, :, update_indexes, :].set, :536-538
      cv[slot][:, update_indexes, :] = newv[0]
    else:
      sk, sv = scales[idx]
      for c, s, new in ((ck, sk, newk), (cv, sv, newv)):
        entry = new[0].transpose(0, 1)  # (T, H, D), :547
        vals, sc = _quantize(entry.unsqueeze(0).transpose(1, 2), compute_dtype)  # same reduction as axes (1, 2) on (T, H, D)
        c[slot][:, update_indexes, :] = vals[0]  # :556
        s[slot][:, update_indexes, :] = sc[0].to(s.dtype)  # :552
  state["lens"][slot] = 1  # :570
  return state


def insert(env, prefix_caches, prefix_seq_len, state, slot, current_position=0, compute_dtype=None):
  """engine.py:606-626."""
  if env.ring_buffer:
    start_insert = current_position - prefix_seq_len
    end_insert = start_insert + prefix_caches[0][0].shape[2]  # padded length
    if start_insert >= 0 and end_insert < env.cache_sequence_length:
      return insert_no_wrap(env, prefix_caches, prefix_seq_len, state, slot, current_position, compute_dtype)
    return insert_wrap(env, prefix_caches, prefix_seq_len, state, slot, current_position, compute_dtype)
  return insert_no_wrap(env, prefix_caches, prefix_seq_len, state, slot, current_position, compute_dtype)
