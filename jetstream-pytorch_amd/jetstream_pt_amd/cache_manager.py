"""Decode-time KV cache objects writing through the HIP kernels.

Same classes, constructor arguments, attributes and update()/finalize()/
state()/scalers()/empty() contract as the reference module
(jetstream_pt/cache_manager.py): KVCachePrefill (:42), KVCacheGenerate (:93),
Int8KVCacheGenerate (:337), PageKVCacheGenerate (:660).  Caches are torch
tensors on the ROCm device and are updated in place; update() returns the
same tensors (or the layer's view of a stacked cache) the reference returns.

Every per-slot write is one kernel launch for K and V together (and both
scalers, and all layers in finalize), where the reference issues one scatter
or one dynamic_update_slice per slot, per layer, per tensor.

Keyword-only additions on Int8KVCacheGenerate, defaults reference-literal:
  rounding     "trunc" (the decode quantiser, :532-537) or "rne"
               (quantize_tensor's round-half-even + clamp, quantize.py:58-75)
  scale_heads  1 (one scale per token over all heads) or kv_heads
  scale_dtype  None = activation dtype, or torch.float32
"""

import torch

from . import _ffi
from .page_attention_manager import DeviceTokenIndices, PageAttentionManager
from .quantize import _rounding_code


# pylint: disable-next=all
class CacheInterface:
  """Kv cache interface: update(key, value[, layer_id]) with key/value shaped
  (batch, heads, seqlen, head_dim) returns the full cache after the update."""

  def update(self, key, value):
    raise NotImplementedError


class KVCachePrefill:
  """Prefill-time stand-in: remembers K/V (reference :42-69)."""

  def __init__(self, kv_quantize=False, stacked=False):
    self.kv_quantize = kv_quantize
    self.cache_k = None
    self.cache_v = None
    self.stacked = stacked

  def update(self, key, value, layer_id=0):
    self.cache_k = key
    self.cache_v = value
    if self.kv_quantize:  # pretend to be quantized
      bsz, _, seq, _ = key.shape
      ones = torch.ones((bsz, 1, seq, 1), dtype=torch.bfloat16, device=key.device)
      return key, value, None, None, ones, ones, None, None
    return key, value

  def state(self):
    return self.cache_k, self.cache_v

  def finalize(self):
    return


def _scatter_lines(pairs, pos, pos_count, n_layers, batch, seq):
  """pairs: [(dst (L?, B, H, S, X), src (L?, B, H, 1, X))]; one launch."""
  arr = (_ffi.LineTensor * len(pairs))()
  for i, (dst, src) in enumerate(pairs):
    _ffi.dev(dst, "cache"), _ffi.dev(src, "new line")
    if src.dtype != dst.dtype:
      raise ValueError(f"line dtype {src.dtype} does not match cache dtype {dst.dtype}")
    arr[i] = _ffi.LineTensor(_ffi.ptr(dst), _ffi.ptr(src), dst.shape[-3],
                             dst.shape[-1] * dst.element_size())
  _ffi.check(_ffi.lib.jpt_kv_scatter_lines(
      arr, len(pairs), _ffi.ptr(pos), pos_count, n_layers, batch, seq, _ffi.stream()))


class KVCacheGenerate:
  """bf16 / f32 decode cache (reference :93-313)."""

  # pylint: disable=too-many-instance-attributes
  def __init__(self, cache_k: torch.Tensor, cache_v: torch.Tensor, position, sharding=None,
               env=None):
    self.cache_k = cache_k
    self.cache_v = cache_v
    self.input_pos = position
    self.sharding = sharding
    self.env = env
    self.new_ks = None
    self.new_vs = None
    self.stacked = env.generate_cache_stacked
    self.batch = torch.arange(env.batch_size)
    if env.lazy_cache_update:
      if env.generate_cache_stacked:
        if env.new_cache_stacked:
          layer, batch, heads, _, dim = cache_k.shape
          shape = (layer, batch, heads, 1, dim)
          self.new_ks = torch.zeros(shape, dtype=cache_k.dtype, device=cache_k.device)
          self.new_vs = torch.zeros(shape, dtype=cache_k.dtype, device=cache_k.device)
        else:
          self.new_ks, self.new_vs = [], []
      else:  # when generate cache is not stacked, new cache cannot stack
        assert not env.new_cache_stacked

  def _pos(self, count):
    return _ffi.as_i32(self.input_pos, self.cache_k.device, count)

  def _write(self, cache_k, cache_v, new_k, new_v, ring):
    """cache (L?, B, H, S, D) <- new (L?, B, H, 1, D) at the stored position(s)."""
    n_layers = cache_k.shape[0] if cache_k.dim() == 5 else 1
    batch, seq = cache_k.shape[-4], cache_k.shape[-2]
    count = 1 if ring else batch
    _scatter_lines([(cache_k, new_k.to(cache_k.dtype).contiguous()),
                    (cache_v, new_v.to(cache_v.dtype).contiguous())],
                   self._pos(count), count, n_layers, batch, seq)

  def update(self, key, value, layer_id: int = 0):
    """Update kv cache"""
    env = self.env
    if env.lazy_cache_update:
      if env.new_cache_stacked:
        assert env.generate_cache_stacked, "When new cache stacked, must have generate_cache_stacked!"
        self.new_ks[layer_id, ...] = key
        self.new_vs[layer_id, ...] = value
        return self.cache_k[layer_id], self.cache_v[layer_id]
      if env.generate_cache_stacked:
        self.new_ks.append(key)
        self.new_vs.append(value)
        return self.cache_k[layer_id], self.cache_v[layer_id]
      self.new_ks = key
      self.new_vs = value
      return self.cache_k, self.cache_v

    if env.ring_buffer:
      assert not env.new_cache_stacked and not env.generate_cache_stacked, \
          "Ring buffer doesn't support stacked cache."
      self._write(self.cache_k, self.cache_v, key, value, ring=True)
      return self.cache_k, self.cache_v

    if env.generate_cache_stacked:
      layer_k, layer_v = self.cache_k[layer_id], self.cache_v[layer_id]
      self._write(layer_k, layer_v, key, value, ring=False)
      return layer_k, layer_v

    self._write(self.cache_k, self.cache_v, key, value, ring=False)
    return self.cache_k, self.cache_v

  def finalize(self):
    """Applies the lazily stashed lines of every layer in one launch."""
    env = self.env
    if not env.lazy_cache_update:
      return
    new_ks, new_vs = self.new_ks, self.new_vs
    if isinstance(new_ks, list):  # cache stacked, new lines kept per layer
      new_ks, new_vs = torch.stack(new_ks), torch.stack(new_vs)
      self.new_ks, self.new_vs = [], []
    self._write(self.cache_k, self.cache_v, new_ks, new_vs, ring=env.ring_buffer)

  def state(self):
    return self.cache_k, self.cache_v

  @classmethod
  def empty(cls, shape, device, env):
    """Create empty kv caches"""
    dtype = torch.bfloat16 if env.bf16_enable else torch.float32
    device = device if isinstance(device, (str, torch.device)) else "cuda"
    k = torch.zeros(shape, dtype=dtype, device=device)
    v = torch.zeros(shape, dtype=dtype, device=device)
    return cls(k, v, 0, None, env=env)


class Int8KVCacheGenerate:
  """int8 codes + per-token scales (reference :337-657)."""

  # pylint: disable=too-many-instance-attributes
  def __init__(self, cache_k, cache_v, cache_k_scaler, cache_v_scaler, input_pos,
               sharding=None, env=None, *, rounding="trunc", scale_heads=None,
               scale_dtype=None):
    self.cache_k = cache_k
    self.cache_v = cache_v
    self.k_scaler = cache_k_scaler
    self.v_scaler = cache_v_scaler
    self.input_pos = input_pos
    self.sharding = sharding
    self.env = env
    self.stacked = env.generate_cache_stacked
    self.batch = torch.arange(env.batch_size)
    self.rounding = rounding
    self.scale_heads = cache_k_scaler.shape[-3] if scale_heads is None else scale_heads
    self.scale_dtype = cache_k_scaler.dtype if scale_dtype is None else scale_dtype
    if self.scale_dtype != cache_k_scaler.dtype:
      raise ValueError("scale_dtype must match the scaler tensors")
    self.new_ks = self.new_vs = None
    self.new_k_scaler = self.new_v_scaler = None
    dev = cache_k.device
    if env.lazy_cache_update:
      if env.generate_cache_stacked:
        layer, batch, heads, _, dim = cache_k.shape
        if env.new_cache_stacked:
          self.new_ks = torch.zeros((layer, batch, heads, 1, dim), dtype=torch.int8, device=dev)
          self.new_vs = torch.zeros((layer, batch, heads, 1, dim), dtype=torch.int8, device=dev)
          sshape = (layer, batch, self.scale_heads, 1, 1)
          self.new_k_scaler = torch.zeros(sshape, dtype=self.scale_dtype, device=dev)
          self.new_v_scaler = torch.zeros(sshape, dtype=self.scale_dtype, device=dev)
        else:
          self.new_ks, self.new_vs, self.new_k_scaler, self.new_v_scaler = [], [], [], []
      else:  # when generate cache is not stacked, new cache cannot stack
        assert not env.new_cache_stacked

  def _pos(self, count):
    return _ffi.as_i32(self.input_pos, self.cache_k.device, count)

  def _quantize_into(self, xk, xv, out, cache=None, ring=False, freqs_cis=None):
    """Runs the fused quantiser.  out = (k_codes, v_codes, k_scale, v_scale)
    destinations shaped (B, H, 1, D) / (B, Hs, 1, 1); cache = optional
    (cache_k, cache_v, k_scaler, v_scaler) 4-D views to scatter into."""
    xk, xv = _ffi.dev(xk.contiguous(), "xk"), _ffi.dev(xv.contiguous(), "xv")
    b, h, t, d = xk.shape
    if t != 1:
      raise ValueError("the decode cache takes one token per update")
    a = _ffi.QuantAppendArgs(
        new_k=_ffi.ptr(xk), new_v=_ffi.ptr(xv), batch=b, heads=h, dim=d, seq=1, pos_count=b,
        in_dtype=_ffi.dtype_code(xk.dtype), scale_dtype=_ffi.dtype_code(self.scale_dtype),
        scale_heads=self.scale_heads, rounding=_rounding_code(self.rounding))
    for t_ in out:
      _ffi.dev(t_, "quantiser output")
    a.out_k, a.out_v, a.out_k_scale, a.out_v_scale = (_ffi.ptr(t_) for t_ in out)
    rope = None
    if freqs_cis is not None:  # xk is unrotated: the launch rotates it first
      rope = _ffi.rope_factors(freqs_cis, b, d)
      a.rope = _ffi.ptr(rope)
    pos = None
    if cache is not None:
      for t_ in cache:
        _ffi.dev(t_, "cache")
      a.cache_k, a.cache_v, a.k_scale, a.v_scale = (_ffi.ptr(t_) for t_ in cache)
      a.seq = cache[0].shape[-2]
      a.pos_count = 1 if ring else b
      pos = self._pos(a.pos_count)
      a.pos = _ffi.ptr(pos)
    _ffi.check(_ffi.lib.jpt_kv_append_quant_i8(a, _ffi.stream()))

  def quantize(self, val):
    """Quantize value: (batch, heads, 1, dim) -> (codes, scale)."""
    from .quantize import quantize_kv
    kq, _, ks, _ = quantize_kv(val, val, rounding=self.rounding, scale_heads=self.scale_heads,
                               scale_dtype=self.scale_dtype)
    return kq, ks

  def update(self, xk, xv, layer_id: int = 0, *, defer_quantize=False, freqs_cis=None):
    """Update kv cache.

    freqs_cis: the step's rotary factors when xk has NOT been through
    apply_rotary_emb yet; the quantiser launch then rotates it first.

    defer_quantize (lazy mode only): return the tensors the codes and scales of
    this token WILL live in without launching the quantiser; the caller hands
    them to ragged_mha together with xk/xv as new_key_raw/new_value_raw and the
    attention launch fills them."""
    env = self.env
    b, h, _, d = xk.shape
    dev = xk.device
    if defer_quantize and not env.lazy_cache_update:
      raise ValueError("defer_quantize needs lazy_cache_update")
    stash = env.lazy_cache_update and env.new_cache_stacked
    if stash:  # quantise straight into this layer's stash rows
      out = (self.new_ks[layer_id], self.new_vs[layer_id],
             self.new_k_scaler[layer_id], self.new_v_scaler[layer_id])
    else:
      out = (torch.empty((b, h, 1, d), dtype=torch.int8, device=dev),
             torch.empty((b, h, 1, d), dtype=torch.int8, device=dev),
             torch.empty((b, self.scale_heads, 1, 1), dtype=self.scale_dtype, device=dev),
             torch.empty((b, self.scale_heads, 1, 1), dtype=self.scale_dtype, device=dev))
    if env.lazy_cache_update:
      if not defer_quantize:
        self._quantize_into(xk, xv, out, freqs_cis=freqs_cis)
      if not env.new_cache_stacked:
        if env.generate_cache_stacked:
          self.new_ks.append(out[0])
          self.new_vs.append(out[1])
          self.new_k_scaler.append(out[2])
          self.new_v_scaler.append(out[3])
        else:
          self.new_ks, self.new_vs, self.new_k_scaler, self.new_v_scaler = out
    else:
      if self.cache_k.dim() == 5:  # eager + stacked: this layer's view (the reference has no such branch)
        cache = (self.cache_k[layer_id], self.cache_v[layer_id],
                 self.k_scaler[layer_id], self.v_scaler[layer_id])
      else:
        cache = (self.cache_k, self.cache_v, self.k_scaler, self.v_scaler)
      self._quantize_into(xk, xv, out, cache, ring=env.ring_buffer, freqs_cis=freqs_cis)
    k_quant, v_quant, kscale, vscale = out
    return (self.cache_k, self.cache_v, k_quant, v_quant, self.k_scaler, self.v_scaler,
            kscale, vscale)

  def finalize(self):
    """Applies the stashed codes and scales of every layer in one launch."""
    env = self.env
    if not env.lazy_cache_update:
      return
    new = [self.new_ks, self.new_vs, self.new_k_scaler, self.new_v_scaler]
    if isinstance(self.new_ks, list):
      new = [torch.stack(x) for x in new]
      self.new_ks, self.new_vs, self.new_k_scaler, self.new_v_scaler = [], [], [], []
    pairs = [(self.cache_k, new[0]), (self.cache_v, new[1])]
    if not env.ring_buffer:
      # the reference's ring-buffer finalize writes the codes only (:588-597)
      pairs += [(self.k_scaler, new[2].to(self.k_scaler.dtype)),
                (self.v_scaler, new[3].to(self.v_scaler.dtype))]
    n_layers = self.cache_k.shape[0] if self.cache_k.dim() == 5 else 1
    batch, seq = self.cache_k.shape[-4], self.cache_k.shape[-2]
    count = 1 if env.ring_buffer else batch
    _scatter_lines([(dst, src.contiguous()) for dst, src in pairs], self._pos(count), count,
                   n_layers, batch, seq)

  def state(self):
    return self.cache_k, self.cache_v

  def scalers(self):
    return self.k_scaler, self.v_scaler

  @classmethod
  # pylint: disable-next=all
  def empty(cls, shape, device, env, *, rounding="trunc", scale_heads=1, scale_dtype=None):
    """Zero codes and scalers of ONES, as the reference creates them (:513-530)."""
    device = device if isinstance(device, (str, torch.device)) else "cuda"
    cache_k = torch.zeros(shape, dtype=torch.int8, device=device)
    cache_v = torch.zeros(shape, dtype=torch.int8, device=device)
    if env.generate_cache_stacked:
      s_shape = (shape[0], shape[1], scale_heads, shape[3], 1)
    else:
      s_shape = (shape[0], scale_heads, shape[2], 1)
    sdt = scale_dtype or torch.bfloat16
    kscaler = torch.ones(s_shape, dtype=sdt, device=device)
    vscaler = torch.ones(s_shape, dtype=sdt, device=device)
    return cls(cache_k, cache_v, kscaler, vscaler, 0, None, env=env, rounding=rounding,
               scale_heads=scale_heads, scale_dtype=sdt)


class PageKVCacheGenerate:
  """Paged cache (heads, total_pages, page_size, dim) (reference :660-724).

  update() writes one row per active slot straight into its page; the
  reference gathers every active page, patches it and scatters it back.
  """

  def __init__(self, cache_k: torch.Tensor, cache_v: torch.Tensor,
               page_attention_manager: PageAttentionManager, page_token_indices, sharding=None,
               env=None):
    self.cache_k = cache_k
    self.cache_v = cache_v
    self.page_attention_manager = page_attention_manager
    self.page_token_indices = page_token_indices
    self.sharding = sharding
    self.env = env
    self.stacked = False

  def update(self, key, value, layer_id=0, *, defer_append=False):
    """Update kv cache.  defer_append: write nothing - the attention launch
    appends the token itself (call_paged_attention(append=...))."""
    if defer_append:
      return self.cache_k, self.cache_v
    pk, pv = _ffi.dev(self.cache_k, "cache_k"), _ffi.dev(self.cache_v, "cache_v")
    heads, total, ps, dim = pk.shape
    key = _ffi.dev(key.to(pk.dtype).contiguous(), "key")
    value = _ffi.dev(value.to(pv.dtype).contiguous(), "value")
    idx = self.page_token_indices
    if isinstance(idx, DeviceTokenIndices):  # column count stays on the device
      _ffi.check(_ffi.lib.jpt_paged_append_dev(
          _ffi.ptr(pk), _ffi.ptr(pv), _ffi.ptr(key), _ffi.ptr(value), _ffi.ptr(idx.indices), idx.stride,
          _ffi.ptr(idx.n_active), key.shape[0], heads, total, ps, dim * pk.element_size(), _ffi.stream()))
      return self.cache_k, self.cache_v
    if not (isinstance(idx, torch.Tensor) and idx.is_cuda and idx.dtype == torch.int32):
      idx = _ffi.as_i32(idx, pk.device).reshape(3, -1)
      self.page_token_indices = idx
    idx = idx.contiguous()
    _ffi.check(_ffi.lib.jpt_paged_append(
        _ffi.ptr(pk), _ffi.ptr(pv), _ffi.ptr(key), _ffi.ptr(value), _ffi.ptr(idx), idx.shape[1],
        key.shape[0], heads, total, ps, dim * pk.element_size(), _ffi.stream()))
    return self.cache_k, self.cache_v

  def state(self):
    return self.cache_k, self.cache_v

  def finalize(self):
    return

  @classmethod
  def empty(cls, shape, device, env):
    """Create empty kv caches"""
    dtype = torch.bfloat16 if env.bf16_enable else torch.float32
    device = device if isinstance(device, (str, torch.device)) else "cuda"
    k = torch.zeros(shape, dtype=dtype, device=device)
    v = torch.zeros(shape, dtype=dtype, device=device)
    return cls(k, v, None, None, None, env=env)


class Int8PageKVCacheGenerate:
  """int8 paged cache: codes (heads, total_pages, page_size, dim) and scale
  pages (scale_heads, total_pages, page_size).  The reference has no such
  class (its paged cache is bf16/f32 only); this composes its decode
  quantiser with its paged row write.  update() returns
  (cache_k, cache_v, k_scale_pages, v_scale_pages)."""

  def __init__(self, cache_k, cache_v, k_scale_pages, v_scale_pages, page_attention_manager,
               page_token_indices, sharding=None, env=None, *, rounding="trunc"):
    self.cache_k, self.cache_v = cache_k, cache_v
    self.k_scaler, self.v_scaler = k_scale_pages, v_scale_pages
    self.page_attention_manager = page_attention_manager
    self.page_token_indices = page_token_indices
    self.sharding = sharding
    self.env = env
    self.stacked = False
    self.rounding = rounding

  def update(self, key, value, layer_id=0, *, freqs_cis=None, defer_append=False):
    """freqs_cis: rotary factors of the step when `key` is still unrotated.
    defer_append: write nothing - the attention launch quantises and appends
    the token itself (call_paged_attention(append=...))."""
    if defer_append:
      return self.cache_k, self.cache_v, self.k_scaler, self.v_scaler
    pk, pv = _ffi.dev(self.cache_k, "cache_k"), _ffi.dev(self.cache_v, "cache_v")
    ks, vs = _ffi.dev(self.k_scaler, "k_scale_pages"), _ffi.dev(self.v_scaler, "v_scale_pages")
    heads, total, ps, dim = pk.shape
    key, value = _ffi.dev(key.contiguous(), "key"), _ffi.dev(value.contiguous(), "value")
    idx = self.page_token_indices
    n_dev, stride = None, 0
    if isinstance(idx, DeviceTokenIndices):  # column count stays on the device
      n_dev, stride, idx = idx.n_active, idx.stride, idx.indices
    elif not (isinstance(idx, torch.Tensor) and idx.is_cuda and idx.dtype == torch.int32):
      idx = _ffi.as_i32(idx, pk.device).reshape(3, -1)
      self.page_token_indices = idx
    idx = idx.contiguous()
    a = _ffi.PagedQuantAppendArgs(
        new_k=_ffi.ptr(key), new_v=_ffi.ptr(value), pages_k=_ffi.ptr(pk), pages_v=_ffi.ptr(pv),
        k_scale_pages=_ffi.ptr(ks), v_scale_pages=_ffi.ptr(vs), indices=_ffi.ptr(idx),
        n_active_dev=_ffi.ptr(n_dev), indices_stride=stride,
        n_active=idx.shape[1], batch=key.shape[0], heads=heads, total_pages=total, page_size=ps,
        dim=dim, in_dtype=_ffi.dtype_code(key.dtype), scale_dtype=_ffi.dtype_code(ks.dtype),
        scale_heads=ks.shape[0], rounding=_rounding_code(self.rounding))
    rope = None
    if freqs_cis is not None:
      rope = _ffi.rope_factors(freqs_cis, key.shape[0], dim)
      a.rope = _ffi.ptr(rope)
    _ffi.check(_ffi.lib.jpt_paged_append_quant_i8(a, _ffi.stream()))
    del rope
    return self.cache_k, self.cache_v, self.k_scaler, self.v_scaler

  def state(self):
    return self.cache_k, self.cache_v

  def scalers(self):
    return self.k_scaler, self.v_scaler

  def finalize(self):
    return

  @classmethod
  def empty(cls, shape, device, env, *, scale_heads=1, scale_dtype=torch.float32, rounding="trunc"):
    device = device if isinstance(device, (str, torch.device)) else "cuda"
    heads, total, ps, _ = shape
    return cls(torch.zeros(shape, dtype=torch.int8, device=device),
               torch.zeros(shape, dtype=torch.int8, device=device),
               torch.ones((scale_heads, total, ps), dtype=scale_dtype, device=device),
               torch.ones((scale_heads, total, ps), dtype=scale_dtype, device=device),
               None, None, None, env=env, rounding=rounding)
