"""Prefill -> decode insert of one prompt into one batch slot.

Mirrors the cache and bookkeeping part of the reference engine's insert
(jetstream_pt/engine.py): `_insert_no_wrap` (:371-488), `_insert_wrap`
(:491-581), `insert` (:606-626) and, for int8 pages, the paged insert
(:583-604 with page_attention_manager.py:83-142).  Caches are updated in
place by one kernel launch for all layers (K and V together; per-layer
tensors travel as a pointer table); with a quantised
cache the prompt is quantised per token over (heads, dim) by the reference's
insert quantiser (quantize.py:58-75: round half to even, clamp, eps 1e-5) in
the prompt's dtype.
"""

import torch

from . import _ffi


def _rounding_code(rounding):
  return {"trunc": _ffi.ROUND_TRUNC, "rne": _ffi.ROUND_RNE}[rounding]


def _layer_views(cache, layer, n_layers):
  """(k, v) of `layer`, given a stacked (L, B, H, S, D) pair or a list of
  per-layer (k, v) pairs."""
  if isinstance(cache, (list, tuple)) and isinstance(cache[0], (list, tuple)):
    if len(cache) == 1 and cache[0][0].dim() == 5:  # reference: [(stacked_k, stacked_v)]
      return cache[0][0][layer], cache[0][1][layer]
    return cache[layer]
  k, v = cache
  return (k[layer], v[layer]) if k.dim() == 5 else (k, v)


def insert_prefix_caches(prefix_caches, caches, cache_scales, slot, start, *, rounding="rne"):
  """Writes the prompt's per-layer (key, value) pairs - each (1, heads, T, D) -
  into slot `slot` of the decode caches at positions (start + t) mod S.

  caches: list of per-layer (k, v) tensors (B, H, S, D), or [(k, v)] with
  stacked (L, B, H, S, D) tensors (the reference's two DecodeState layouts).
  cache_scales: None for float caches; else the scalers in the same layout,
  each (B, Hs, S, 1) / (L, B, Hs, S, 1).  int8 caches are quantised into;
  float caches take a copy (cast to the cache dtype first).
  """
  n_layers = len(prefix_caches)
  layers, keep, common, shape = [], [], None, None
  for layer, (newk, newv) in enumerate(prefix_caches):
    k, v = _layer_views(caches, layer, n_layers)
    k, v = _ffi.dev(k, "cache_k"), _ffi.dev(v, "cache_v")
    batch, heads, seq, dim = k.shape
    if newk.dim() == 4:
      newk, newv = newk[0], newv[0]
    tokens = newk.shape[1]
    quant = k.dtype == torch.int8 and newk.dtype != torch.int8
    if not quant and newk.dtype != k.dtype:
      newk, newv = newk.to(k.dtype), newv.to(v.dtype)
    newk, newv = _ffi.dev(newk.contiguous(), "prefix key"), _ffi.dev(newv.contiguous(), "prefix value")
    if newk.shape != (heads, tokens, dim):
      raise ValueError(f"prefix key {tuple(newk.shape)} does not match cache {tuple(k.shape)}")
    ks = vs = None
    if quant:
      ks, vs = _layer_views(cache_scales, layer, n_layers)
      ks, vs = _ffi.dev(ks, "k_scaler"), _ffi.dev(vs, "v_scaler")
    this = (tuple(k.shape), k.dtype, tuple(newk.shape), newk.dtype, None if ks is None else (ks.dtype, tuple(ks.shape)))
    if shape is not None and this != shape:
      raise ValueError("the layers of one insert must agree in shape and dtype")
    shape = this
    if common is None:
      common = _ffi.PrefillInsertArgs(
          tokens=tokens, heads=heads, dim=dim, slot=int(slot), batch=batch, seq=seq,
          start=int(start), in_dtype=_ffi.dtype_code(newk.dtype), dst_dtype=_ffi.dtype_code(k.dtype))
      if quant:
        common.scale_dtype, common.scale_heads = _ffi.dtype_code(ks.dtype), ks.shape[1]
        common.rounding = _rounding_code(rounding)
    layers.append((_ffi.ptr(newk), _ffi.ptr(newv), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(ks), _ffi.ptr(vs)))
    keep += [newk, newv]
  if layers:
    _launch_layers(common, layers, keep)


def _launch_layers(common, layers, keep):
  """One launch for all the layers of `layers` (lists of six pointers)."""
  table = (_ffi.InsertLayer * len(layers))(*[_ffi.InsertLayer(*l) for l in layers])
  _ffi.check(_ffi.lib.jpt_prefill_insert_layers(common, table, len(layers), _ffi.stream()))
  del keep


def insert_prefix_pages_int8(prefix_caches, decode_caches, scale_pages, page_ids, *, rounding="rne"):
  """int8 pages: per layer, quantises the prompt (1, heads, T, D) per token and
  writes token t to page page_ids[t // ps], row t % ps; the rest of the last
  page is zero-filled (as insert_prefill_cache does for float pages).
  decode_caches / scale_pages: per-layer lists of (k, v) pairs."""
  ids = _ffi.as_i32(page_ids, decode_caches[0][0].device)
  layers, keep, common, shape = [], [ids], None, None
  for (newk, newv), (pk, pv), (ks, vs) in zip(prefix_caches, decode_caches, scale_pages):
    pk, pv = _ffi.dev(pk, "pages_k"), _ffi.dev(pv, "pages_v")
    ks, vs = _ffi.dev(ks, "k_scale_pages"), _ffi.dev(vs, "v_scale_pages")
    heads, total, ps, dim = pk.shape
    if newk.dim() == 4:
      newk, newv = newk[0], newv[0]
    newk, newv = _ffi.dev(newk.contiguous(), "prefix key"), _ffi.dev(newv.contiguous(), "prefix value")
    this = (tuple(pk.shape), tuple(newk.shape), newk.dtype, ks.dtype, tuple(ks.shape))
    if shape is not None and this != shape:
      raise ValueError("the layers of one insert must agree in shape and dtype")
    shape = this
    if common is None:
      common = _ffi.PrefillInsertArgs(
          page_ids=_ffi.ptr(ids), n_pages=ids.numel(), tokens=newk.shape[1], heads=heads, dim=dim,
          total_pages=total, page_size=ps, in_dtype=_ffi.dtype_code(newk.dtype), dst_dtype=_ffi.I8,
          scale_dtype=_ffi.dtype_code(ks.dtype), scale_heads=ks.shape[0], rounding=_rounding_code(rounding))
    layers.append((_ffi.ptr(newk), _ffi.ptr(newv), _ffi.ptr(pk), _ffi.ptr(pv), _ffi.ptr(ks), _ffi.ptr(vs)))
    keep += [newk, newv]
  if layers:
    _launch_layers(common, layers, keep)


def insert_prefix_pages_copy(prefix_caches, decode_caches, page_ids):
  """Float pages, all layers in one launch: token t of every layer's prompt
  (1, heads, T, D) goes to page page_ids[t // ps], row t % ps, the rest of the
  last page is zero-filled (insert_prefill_cache, page_attention_manager.py:
  83-142).  Needs head_dim % 4 == 0 and layers of one shape and dtype; returns
  False, having done nothing, when that does not hold."""
  ids = _ffi.as_i32(page_ids, decode_caches[0][0].device)
  layers, keep, common, shape = [], [ids], None, None
  for (newk, newv), (pk, pv) in zip(prefix_caches, decode_caches):
    if not (pk.is_cuda and pk.is_contiguous() and pv.is_contiguous()) or pk.dtype not in (torch.bfloat16, torch.float32):
      return False
    heads, total, ps, dim = pk.shape
    newk, newv = newk.to(pk.dtype).contiguous(), newv.to(pv.dtype).contiguous()
    this = (tuple(pk.shape), pk.dtype, tuple(newk.shape))
    if dim % 4 != 0 or newk.dim() != 4 or newk.shape[0] != 1 or newk.shape[1] != heads or newk.shape[3] != dim \
        or (shape is not None and this != shape) or not newk.is_cuda:
      return False
    shape = this
    if common is None:
      common = _ffi.PrefillInsertArgs(
          page_ids=_ffi.ptr(ids), n_pages=ids.numel(), tokens=newk.shape[2], heads=heads, dim=dim,
          total_pages=total, page_size=ps, in_dtype=_ffi.dtype_code(pk.dtype), dst_dtype=_ffi.dtype_code(pk.dtype))
    layers.append((_ffi.ptr(newk), _ffi.ptr(newv), _ffi.ptr(pk), _ffi.ptr(pv), None, None))
    keep += [newk, newv]
  if layers:
    _launch_layers(common, layers, keep)
  return True


def insert_prefix_pages_int8_stacked(prefix_k, prefix_v, pages_k, pages_v, k_scale_pages, v_scale_pages,
                                     page_ids, *, rounding="rne"):
  """All layers of one prompt in one launch: prefix_k/v (L, heads, T, D),
  pages (L, heads, P, ps, D) int8, scale pages (L, Hs, P, ps)."""
  pk, pv = _ffi.dev(pages_k, "pages_k"), _ffi.dev(pages_v, "pages_v")
  ks, vs = _ffi.dev(k_scale_pages, "k_scale_pages"), _ffi.dev(v_scale_pages, "v_scale_pages")
  newk, newv = prefix_k, prefix_v
  # the first T rows of a longer buffer are taken as they are (no copy)
  if not (newk.is_cuda and newk.stride(3) == 1 and newk.stride(2) == newk.shape[3] and
          newk.stride() == newv.stride()):
    newk, newv = _ffi.dev(newk.contiguous(), "prefix key"), _ffi.dev(newv.contiguous(), "prefix value")
  layers, heads, total, ps, dim = pk.shape
  if newk.shape[0] != layers or newk.shape[1] != heads or newk.shape[3] != dim:
    raise ValueError(f"prefix {tuple(newk.shape)} does not match pages {tuple(pk.shape)}")
  ids = _ffi.as_i32(page_ids, pk.device)
  a = _ffi.PrefillInsertArgs(
      src_k=_ffi.ptr(newk), src_v=_ffi.ptr(newv), dst_k=_ffi.ptr(pk), dst_v=_ffi.ptr(pv),
      k_scale=_ffi.ptr(ks), v_scale=_ffi.ptr(vs), page_ids=_ffi.ptr(ids), n_pages=ids.numel(),
      tokens=newk.shape[2], heads=heads, dim=dim, total_pages=total, page_size=ps,
      in_dtype=_ffi.dtype_code(newk.dtype), dst_dtype=_ffi.I8, scale_dtype=_ffi.dtype_code(ks.dtype),
      scale_heads=ks.shape[1], rounding=_rounding_code(rounding), n_layers=layers,
      src_layer_stride=newk.stride(0), dst_layer_stride=pk.stride(0), scale_layer_stride=ks.stride(0),
      src_head_stride=newk.stride(1))
  _ffi.check(_ffi.lib.jpt_prefill_insert(a, _ffi.stream()))


def insert_prompts_pages_int8_stacked(prefixes, pages_k, pages_v, k_scale_pages, v_scale_pages, page_ids, *,
                                      rounding="rne"):
  """Several prompts at once, all layers, one launch: prefixes is a list of
  (prefix_k, prefix_v) pairs, each (L, heads, T_i, D); page_ids a list of
  int32 device tensors (prompt i's pages, e.g. rows of the device allocator's
  table).  Same result as insert_prefix_pages_int8_stacked once a prompt."""
  pk, pv = _ffi.dev(pages_k, "pages_k"), _ffi.dev(pages_v, "pages_v")
  ks, vs = _ffi.dev(k_scale_pages, "k_scale_pages"), _ffi.dev(v_scale_pages, "v_scale_pages")
  layers, heads, total, ps, dim = pk.shape
  recs, keep = [], []
  for (newk, newv), ids in zip(prefixes, page_ids):
    if not (newk.is_cuda and newk.stride(3) == 1 and newk.stride(2) == newk.shape[3] and
            newk.stride() == newv.stride()):
      newk, newv = _ffi.dev(newk.contiguous(), "prefix key"), _ffi.dev(newv.contiguous(), "prefix value")
    if newk.shape[0] != layers or newk.shape[1] != heads or newk.shape[3] != dim or newk.dtype != prefixes[0][0].dtype:
      raise ValueError(f"prefix {tuple(newk.shape)} does not match pages {tuple(pk.shape)}")
    ids = _ffi.as_i32(ids, pk.device)
    recs.append(_ffi.InsertPrompt(_ffi.ptr(newk), _ffi.ptr(newv), _ffi.ptr(ids), newk.stride(1), newk.stride(0),
                                  newk.shape[2], ids.numel()))
    keep += [newk, newv, ids]
  if not recs:
    return
  a = _ffi.PrefillInsertArgs(
      dst_k=_ffi.ptr(pk), dst_v=_ffi.ptr(pv), k_scale=_ffi.ptr(ks), v_scale=_ffi.ptr(vs), heads=heads, dim=dim,
      total_pages=total, page_size=ps, in_dtype=_ffi.dtype_code(prefixes[0][0].dtype), dst_dtype=_ffi.I8,
      scale_dtype=_ffi.dtype_code(ks.dtype), scale_heads=ks.shape[1], rounding=_rounding_code(rounding),
      n_layers=layers, dst_layer_stride=pk.stride(0), scale_layer_stride=ks.stride(0))
  table = (_ffi.InsertPrompt * len(recs))(*recs)
  _ffi.check(_ffi.lib.jpt_prefill_insert_prompts(a, table, len(recs), _ffi.stream()))
  del keep


def insert(env, prefix_caches, prefix_seq_len, caches, cache_scales, slot, *, current_position=0,
           mask=None, start=None, input_pos=None, lens=None):
  """The reference's Engine.insert for dense caches: picks no-wrap or wrap as
  engine.py:606-626 does, writes the caches (and scalers), and updates the
  slot's row of the bookkeeping tensors that are given, in place:
  mask (B, S) additive, start (B,), input_pos (B,), lens (B,).
  Returns the first cache position written."""
  seq = env.cache_sequence_length
  padded = prefix_caches[0][0].shape[-2]
  if env.ring_buffer:
    start_insert = current_position - prefix_seq_len
    end_insert = start_insert + padded
    wrap = not (start_insert >= 0 and end_insert < seq)
    cur = current_position
  else:
    wrap, cur = False, prefix_seq_len
  if not wrap:
    pos = cur - prefix_seq_len
    insert_prefix_caches(prefix_caches, caches, cache_scales, slot, pos)
    first = pos % seq
    if mask is not None:
      x = torch.arange(seq, device=mask.device)
      mask[slot] = torch.where((x < cur) & (x >= pos), 0.0, float("-inf")).to(mask.dtype)
  else:
    first = (current_position - prefix_seq_len) % seq
    insert_prefix_caches(prefix_caches, caches, cache_scales, slot, first)
    if mask is not None:
      x = torch.arange(seq, device=mask.device)
      cond = ((x >= first) & (x < current_position)) if current_position > first else \
          ((x >= first) | (x < current_position))
      mask[slot] = torch.where(cond, 0.0, float("-inf")).to(mask.dtype)
  if start is not None:
    start[slot] = first
  if input_pos is not None:
    input_pos[slot] = prefix_seq_len
  if lens is not None:
    lens[slot] = 1
  return first
