"""Decode-time KV cache objects, restated on torch-CPU (test infrastructure).

Follows jetstream_pt/cache_manager.py branch by branch.  Tensors are plain
torch CPU tensors updated in place (the reference rebinds a functional
jax.Array inside the same wrapper, cache_manager.py:255-261, which callers
observe as in-place mutation).

Where the reference's two write primitives differ on an out-of-range
position (scatter drops it, dynamic_update_slice clamps it) the behaviour is
undefined here: positions must satisfy 0 <= pos < cache length.
"""

import torch

from . import quant


def _positions(pos, n):
  p = torch.as_tensor(pos, dtype=torch.int64).reshape(-1)
  assert p.numel() == n, f"expected {n} positions, got {p.numel()}"
  return p


class KVCachePrefill:
  """cache_manager.py:42-69: remembers K/V; pretends to be quantised."""

  def __init__(self, kv_quantize=False, stacked=False):
    self.kv_quantize = kv_quantize
    self.cache_k = None
    self.cache_v = None
    self.stacked = stacked

  def update(self, key, value, layer_id=0):
    self.cache_k, self.cache_v = key, value
    if self.kv_quantize:  # cache_manager.py:55-58
      bsz, _, seq, _ = key.shape
      ones = torch.ones((bsz, 1, seq, 1), dtype=torch.bfloat16)
      return key, value, None, None, ones, ones, None, None
    return key, value

  def state(self):
    return self.cache_k, self.cache_v

  def finalize(self):
    return


def _write_line_per_slot(cache, new, pos):
  """update_single_cache_line, cache_manager.py:154-173 / :479-501.

  cache (..., B, H, S, D) and new (..., B, H, 1, D) share their leading dims;
  slot b's single line goes to sequence index pos[b].
  """
  b = cache.shape[-4]
  for bb, pp in enumerate(_positions(pos, b).tolist()):
    cache[..., bb, :, pp : pp + 1, :] = new[..., bb, :, :, :]


class KVCacheGenerate:
  """cache_manager.py:93-313 (bf16/f32 cache)."""

  def __init__(self, cache_k, cache_v, position, sharding=None, env=None):
    self.cache_k, self.cache_v = cache_k, cache_v
    self.input_pos = position
    self.sharding = sharding
    self.env = env
    self.stacked = env.generate_cache_stacked
    self.new_ks = self.new_vs = None
    if env.lazy_cache_update:  # cache_manager.py:120-134
      if env.generate_cache_stacked:
        if env.new_cache_stacked:
          layer, batch, heads, _, dim = cache_k.shape
          shape = (layer, batch, heads, 1, dim)
          self.new_ks = torch.zeros(shape, dtype=env.default_type)
          self.new_vs = torch.zeros(shape, dtype=env.default_type)
        else:
          self.new_ks, self.new_vs = [], []
      else:
        assert not env.new_cache_stacked

  def update(self, key, value, layer_id: int = 0):
    env = self.env
    if env.lazy_cache_update:  # cache_manager.py:230-248
      if env.new_cache_stacked:
        assert env.generate_cache_stacked
        self.new_ks[layer_id, ...] = key
        self.new_vs[layer_id, ...] = value
        return self.cache_k[layer_id], self.cache_v[layer_id]
      if env.generate_cache_stacked:
        self.new_ks.append(key)
        self.new_vs.append(value)
        return self.cache_k[layer_id], self.cache_v[layer_id]
      self.new_ks, self.new_vs = key, value
      return self.cache_k, self.cache_v

    if env.ring_buffer:  # cache_manager.py:250-262
      assert not env.new_cache_stacked and not env.generate_cache_stacked
      pos = _positions(self.input_pos, 1)
      self.cache_k[..., pos, :] = key
      self.cache_v[..., pos, :] = value
      return self.cache_k, self.cache_v

    batch = torch.arange(env.batch_size)
    pos = _positions(self.input_pos, env.batch_size)
    if env.generate_cache_stacked:  # cache_manager.py:265-278
      self.cache_k[layer_id, batch, :, pos, :] = key.squeeze(2)
      self.cache_v[layer_id, batch, :, pos, :] = value.squeeze(2)
      return self.cache_k[layer_id], self.cache_v[layer_id]
    # cache_manager.py:280-293
    self.cache_k[batch, :, pos, :] = key.squeeze(2)
    self.cache_v[batch, :, pos, :] = value.squeeze(2)
    return self.cache_k, self.cache_v

  def finalize(self):
    env = self.env
    if not env.lazy_cache_update:
      return
    if env.ring_buffer:  # cache_manager.py:180-189
      pos = _positions(self.input_pos, 1)
      self.cache_k[..., pos, :] = self.new_ks
      self.cache_v[..., pos, :] = self.new_vs
      return
    if env.generate_cache_stacked and not env.new_cache_stacked:
      # cache_manager.py:203-215
      batch = torch.arange(env.batch_size)
      pos = _positions(self.input_pos, env.batch_size)
      _, b, head, _, dim = self.cache_k.shape
      for i in range(env.num_layers):
        self.cache_k[i, batch, :, pos, :] = self.new_ks[i].reshape(b, head, dim)
        self.cache_v[i, batch, :, pos, :] = self.new_vs[i].reshape(b, head, dim)
      return
    # cache_manager.py:193-201 and :216-225
    _write_line_per_slot(self.cache_k, self.new_ks, self.input_pos)
    _write_line_per_slot(self.cache_v, self.new_vs, self.input_pos)

  def state(self):
    return self.cache_k, self.cache_v

  @classmethod
  def empty(cls, shape, device, env):
    """cache_manager.py:299-313 (the non-testing, zero-filled branch)."""
    dtype = torch.bfloat16 if env.bf16_enable else torch.float32
    return cls(
        torch.zeros(shape, dtype=dtype), torch.zeros(shape, dtype=dtype), 0,
        device, env=env,
    )


class Int8KVCacheGenerate:
  """cache_manager.py:337-657 (int8 codes + per-token scales).

  `rounding`, `scale_heads`, `scale_dtype` select the quantiser variant; the
  defaults are the reference-literal ones (truncating Q_decode, one scale per
  token over all heads, scale in the activation dtype).
  """

  def __init__(
      self, cache_k, cache_v, cache_k_scaler, cache_v_scaler, input_pos,
      sharding=None, env=None, *, rounding="trunc", scale_heads=1,
      scale_dtype=None,
  ):
    self.cache_k, self.cache_v = cache_k, cache_v
    self.k_scaler, self.v_scaler = cache_k_scaler, cache_v_scaler
    self.input_pos = input_pos
    self.sharding = sharding
    self.env = env
    self.stacked = env.generate_cache_stacked
    self.rounding, self.scale_heads = rounding, scale_heads
    self.scale_dtype = scale_dtype
    self.new_ks = self.new_vs = None
    self.new_k_scaler = self.new_v_scaler = None
    if env.lazy_cache_update:  # cache_manager.py:368-394
      if env.generate_cache_stacked:
        layer, batch, heads, _, dim = cache_k.shape
        if env.new_cache_stacked:
          sdt = scale_dtype or env.default_type
          self.new_ks = torch.zeros((layer, batch, heads, 1, dim), dtype=torch.int8)
          self.new_vs = torch.zeros((layer, batch, heads, 1, dim), dtype=torch.int8)
          self.new_k_scaler = torch.zeros((layer, batch, scale_heads, 1, 1), dtype=sdt)
          self.new_v_scaler = torch.zeros((layer, batch, scale_heads, 1, 1), dtype=sdt)
        else:
          self.new_ks, self.new_vs = [], []
          self.new_k_scaler, self.new_v_scaler = [], []
      else:
        assert not env.new_cache_stacked

  def quantize(self, val):
    fn = quant.quantize_decode if self.rounding == "trunc" else quant.quantize_insert
    return fn(val, self.scale_heads, self.scale_dtype)

  def update(self, xk, xv, layer_id: int = 0):
    env = self.env
    k_quant, kscale = self.quantize(xk)  # cache_manager.py:541-542
    v_quant, vscale = self.quantize(xv)
    if env.lazy_cache_update:  # cache_manager.py:544-560
      if env.new_cache_stacked:
        self.new_ks[layer_id, ...] = k_quant
        self.new_vs[layer_id, ...] = v_quant
        self.new_k_scaler[layer_id, ...] = kscale
        self.new_v_scaler[layer_id, ...] = vscale
      elif env.generate_cache_stacked:
        self.new_ks.append(k_quant)
        self.new_vs.append(v_quant)
        self.new_k_scaler.append(kscale)
        self.new_v_scaler.append(vscale)
      else:
        self.new_ks, self.new_vs = k_quant, v_quant
        self.new_k_scaler, self.new_v_scaler = kscale, vscale
    elif env.ring_buffer:  # cache_manager.py:561-565
      pos = _positions(self.input_pos, 1)
      self.cache_k[:, :, pos, :] = k_quant
      self.cache_v[:, :, pos, :] = v_quant
      self.k_scaler[:, :, pos, :] = kscale
      self.v_scaler[:, :, pos, :] = vscale
    else:  # cache_manager.py:566-571
      batch = torch.arange(env.batch_size)
      pos = _positions(self.input_pos, env.batch_size)
      self.cache_k[batch, :, pos, :] = k_quant.squeeze(2)
      self.cache_v[batch, :, pos, :] = v_quant.squeeze(2)
      self.k_scaler[batch, :, pos, :] = kscale.squeeze(2)
      self.v_scaler[batch, :, pos, :] = vscale.squeeze(2)
    return (
        self.cache_k, self.cache_v, k_quant, v_quant,
        self.k_scaler, self.v_scaler, kscale, vscale,
    )

  def finalize(self):
    env = self.env
    if not env.lazy_cache_update:
      return
    if env.ring_buffer:
      # cache_manager.py:588-597: codes only; the scalers are NOT written.
      pos = _positions(self.input_pos, 1)
      self.cache_k[..., pos, :] = self.new_ks
      self.cache_v[..., pos, :] = self.new_vs
      return
    if env.generate_cache_stacked and not env.new_cache_stacked:
      # cache_manager.py:444-477: per slot, per layer
      b = self.cache_k.shape[-4]
      pos = _positions(self.input_pos, b).tolist()
      pairs = (
          (self.cache_k, self.new_ks), (self.cache_v, self.new_vs),
          (self.k_scaler, self.new_k_scaler), (self.v_scaler, self.new_v_scaler),
      )
      for bb, pp in enumerate(pos):
        for layer in range(env.num_layers):
          for dst, src in pairs:
            dst[layer, bb, :, pp : pp + 1, :] = src[layer][bb]
      return
    # cache_manager.py:478-501 (stacked+stacked, or fully unstacked)
    _write_line_per_slot(self.cache_k, self.new_ks, self.input_pos)
    _write_line_per_slot(self.cache_v, self.new_vs, self.input_pos)
    _write_line_per_slot(self.k_scaler, self.new_k_scaler, self.input_pos)
    _write_line_per_slot(self.v_scaler, self.new_v_scaler, self.input_pos)

  def state(self):
    return self.cache_k, self.cache_v

  def scalers(self):
    return self.k_scaler, self.v_scaler

  @classmethod
  def empty(cls, shape, device, env, *, rounding="trunc", scale_heads=1,
            scale_dtype=None):
    """cache_manager.py:513-530: zero codes, scalers of ONES."""
    cache_k = torch.zeros(shape, dtype=torch.int8)
    cache_v = torch.zeros(shape, dtype=torch.int8)
    if env.generate_cache_stacked:
      s_shape = (shape[0], shape[1], scale_heads, shape[3], 1)
    else:
      s_shape = (shape[0], scale_heads, shape[2], 1)
    sdt = scale_dtype or torch.bfloat16
    return cls(
        cache_k, cache_v, torch.ones(s_shape, dtype=sdt),
        torch.ones(s_shape, dtype=sdt), 0, device, env=env, rounding=rounding,
        scale_heads=scale_heads, scale_dtype=scale_dtype,
    )


class PageKVCacheGenerate:
  """cache_manager.py:660-724 (paged bf16/f32 cache (heads, pages, ps, dim))."""

  def __init__(self, cache_k, cache_v, page_attention_manager,
               page_token_indices, sharding=None, env=None):
    self.cache_k, self.cache_v = cache_k, cache_v
    self.page_attention_manager = page_attention_manager
    self.page_token_indices = page_token_indices
    self.sharding = sharding
    self.env = env
    self.stacked = False

  def update(self, key, value, layer_id=0):
    """cache_manager.py:681-706, the literal gather / set / scatter."""
    idx = torch.as_tensor(self.page_token_indices, dtype=torch.int64)

    def _update(cache, x):
      x = x.squeeze(2).permute(1, 0, 2)  # (heads, batch, dim)
      x = x[:, idx[2], :]
      head, _, page_size, dim = cache.shape
      selected = cache[:, idx[0], :, :].reshape(head, -1, dim)
      selected[:, idx[1], :] = x
      cache[:, idx[0], :, :] = selected.reshape(head, -1, page_size, dim)

    _update(self.cache_k, key)
    _update(self.cache_v, value)
    return self.cache_k, self.cache_v

  def state(self):
    return self.cache_k, self.cache_v

  def finalize(self):
    return

  @classmethod
  def empty(cls, shape, device, env):
    dtype = torch.bfloat16 if env.bf16_enable else torch.float32
    return cls(
        torch.zeros(shape, dtype=dtype), torch.zeros(shape, dtype=dtype), None,
        None, device, env=env,
    )
