"""Decode-step attention orchestration: cache update, attention, new-token merge.

AttentionKernel and Int8KVAttentionKernel keep the reference's constructor and
call signature (jetstream_pt/layers.py:382-550, :553-718): cache.update(), then
attention over the returned cache by the implementation the mode flags pick
(ragged / flash / paged / dense), then - in lazy-update mode - the step's own
token attended separately and merged by log-sum-exp.

With `fuse_new_token` (default) the ragged path hands the new token to the
attention launch itself, which merges it in its epilogue; the unfused sequence
(second flash_attention call + lse_merge) stays available and is what the
other lazy combinations use.  With `fuse_quantize` (default) the int8 kernel
also leaves the token's quantisation to that launch: cache.update() only names
the stash rows, and the attention kernel writes codes and scales into them.
Only this attention part of the reference's layers.py is provided;
projections, RoPE and norms are outside the KV path.
"""

import torch

from . import _ffi
from . import attention_kernel as ak
from .scopes import scoped
from .cache_manager import Int8KVCacheGenerate


def apply_rotary_emb(xq, xk, freqs_cis):
  """The reference's apply_rotary_emb (jetstream_pt/layers.py:368-379) as one small
  launch per tensor: xq, xk (bs, seqlen, heads, dim), freqs_cis (bs, seqlen,
  dim / 2) complex64.  Either tensor may be None (e.g. xk, when the KV append
  rotates the key itself); returns (xq_out, xk_out)."""
  outs = []
  for x in (xq, xk):
    if x is None:
      outs.append(None)
      continue
    x = _ffi.dev(x.contiguous(), "x")
    bs, seqlen, heads, dim = x.shape
    f = _ffi.rope_factors(freqs_cis, bs * seqlen, dim)
    out = torch.empty_like(x)
    _ffi.check(_ffi.lib.jpt_rope(_ffi.ptr(out), _ffi.ptr(x), _ffi.ptr(f), bs * seqlen, heads, dim,
                                 _ffi.dtype_code(x.dtype), _ffi.stream()))
    outs.append(out)
  return tuple(outs)


class AttentionKernel:

  def __init__(self, env, layer_id, *, sm_scale_paged=1.0, fuse_new_token=True):
    self.env = env
    self.layer_id = layer_id
    self.sm_scale_paged = sm_scale_paged
    self.fuse_new_token = fuse_new_token
    self.dense_attention = ak.dense_attention
    self.flash_attention = ak.flash_attention
    self.page_attention = ak.call_paged_attention
    self.ragged_attention_orig = ak.RaggedAttentionKernel(env)
    self.ragged_attention_new = ak.RaggedAttentionKernel(env)

  def _attend(self, xq, keys, values, k_scaler, v_scaler, local_mask, cache, start, end,
              ragged_batch_index, ragged_block_index, new_token=None):
    env = self.env
    bsz, num_heads, seqlen, head_dim = xq.shape
    local_max = local_denom = None
    if env.ragged_mha and seqlen == 1 and keys.shape[-2] > 1:
      impl = self.ragged_attention_new if keys.dim() == 4 else self.ragged_attention_orig
      local_output, (local_max, local_denom) = impl(
          xq, keys, values, self.layer_id, start, end, ragged_batch_index, ragged_block_index,
          k_scaler, v_scaler, **(new_token or {}))
    elif env.flash_attention and seqlen == 1:
      local_output, (local_max, local_denom) = self.flash_attention(
          xq=xq, keys=keys, values=values, layer=self.layer_id, k_scaler=k_scaler,
          v_scaler=v_scaler, mask=local_mask)
    elif env.page_attention and seqlen == 1 and hasattr(cache, "page_attention_manager"):
      pam = cache.page_attention_manager
      lengths, page_indices = pam.device_tables(xq.device)
      if new_token is not None:  # the launch appends the token: lengths before the step
        lengths = pam.step_lens
      # one split plan per decode step, shared by the layers
      plan = ak.paged_decode_plan(pam, lengths, bsz, num_heads, keys.shape[0], keys.shape[2],
                                  page_indices.shape[1])
      local_output = self.page_attention(
          env, torch.squeeze(xq, 2), keys, values, lengths, page_indices,
          sm_scale=self.sm_scale_paged, k_scaler=k_scaler, v_scaler=v_scaler, plan=plan,
          append=new_token)
    else:
      local_output = self.dense_attention(
          xq=xq, keys=keys, values=values, k_scaler=k_scaler, v_scaler=v_scaler, mask=local_mask)
    local_output = local_output.reshape(bsz, num_heads, seqlen, head_dim)
    if local_max is not None:
      local_max = local_max.reshape(bsz, num_heads, seqlen, 1)
      local_denom = local_denom.reshape(bsz, num_heads, seqlen, 1)
    return local_output, (local_max, local_denom)

  def _will_append_in_launch(self, xq, cache, keys):
    """Paged cache, one token per slot, the device-resident allocator (its
    lengths before the step stay on the device) and the streaming kernel's
    shapes: the attention launch appends the step's token to the pages itself."""
    pam = getattr(cache, "page_attention_manager", None)
    return (self.fuse_new_token and self.env.page_attention and xq.shape[2] == 1
            and getattr(pam, "step_lens", None) is not None and xq.dtype == torch.bfloat16
            and xq.shape[3] == 128 and keys.dim() == 4 and keys.shape[2] % 32 == 0
            and not (self.env.ragged_mha or self.env.flash_attention))

  def _will_fuse(self, seqlen, keys):
    env = self.env
    return (self.fuse_new_token and env.lazy_cache_update and seqlen == 1 and env.ragged_mha
            and keys.shape[-2] > 1)

  def __call__(self, xq, xk, xv, mask, cache, start=None, end=None, ragged_batch_index=None,
               ragged_block_index=None):
    """xq (batch, heads, seqlen, head_dim); xk, xv (batch, kv_heads, seqlen, head_dim);
    mask additive 0/-inf or None; cache a CacheInterface object."""
    seqlen = xq.shape[2]
    args = (cache, start, end, ragged_batch_index, ragged_block_index)
    if hasattr(cache, "page_attention_manager") and self._will_append_in_launch(xq, cache, cache.cache_k):
      keys, values = scoped("attn_insert_cache", cache.update, xk, xv, self.layer_id, defer_append=True)
      new = dict(new_key=xk.to(keys.dtype).contiguous(), new_value=xv.to(keys.dtype).contiguous())
      return scoped("attn_qkv+attn_new_qkv+attn_global", self._attend, xq, keys, values, None, None, mask, *args, new_token=new)[0]
    orig_keys, orig_values = scoped("attn_insert_cache", cache.update, xk, xv, self.layer_id)
    if self._will_fuse(seqlen, orig_keys):
      dt = orig_keys.dtype
      new = dict(new_key=xk.to(dt).contiguous(), new_value=xv.to(dt).contiguous())
      return scoped("attn_qkv+attn_new_qkv+attn_global", self._attend, xq, orig_keys, orig_values, None, None, mask, *args, new_token=new)[0]
    existing_output, (existing_max, existing_denom) = scoped(
        "attn_qkv", self._attend, xq, orig_keys, orig_values, None, None, mask, *args)
    if not self.env.lazy_cache_update or seqlen > 1:
      return existing_output
    new_output, (new_max, new_denom) = scoped("attn_new_qkv", self._attend, xq, xk, xv, None, None, None, *args)
    return scoped("attn_global", ak.lse_merge, existing_output, existing_max, existing_denom, new_output,
                  new_max, new_denom)


class Int8KVAttentionKernel(AttentionKernel):

  def __init__(self, env, layer_id, *, sm_scale_paged=1.0, fuse_new_token=True, fuse_quantize=True):
    super().__init__(env, layer_id, sm_scale_paged=sm_scale_paged, fuse_new_token=fuse_new_token)
    self.fuse_quantize = fuse_quantize and fuse_new_token

  def __call__(self, xq, xk, xv, mask, cache, start=None, end=None, ragged_batch_index=None,
               ragged_block_index=None, *, freqs_cis=None):
    """freqs_cis (keyword, optional): the step's rotary factors when xk has NOT been
    through apply_rotary_emb; the launch that quantises the key rotates it first
    (xq must come rotated).  One token per slot only."""
    seqlen = xq.shape[2]
    if freqs_cis is not None and (xk.shape[2] != 1 or not hasattr(cache, "rounding")):
      # no quantiser launch to fold the rotation into: rotate here
      xk = apply_rotary_emb(None, xk.transpose(1, 2), freqs_cis)[1].transpose(1, 2)
      freqs_cis = None
    rope_kw = {} if freqs_cis is None else {"freqs_cis": freqs_cis}
    args = (cache, start, end, ragged_batch_index, ragged_block_index)
    if (hasattr(cache, "page_attention_manager") and hasattr(cache, "rounding")
        and self._will_append_in_launch(xq, cache, cache.cache_k) and xk.dtype == torch.bfloat16):
      # int8 pages: the attention launch quantises the token, writes codes and
      # scales into its page and attends it
      keys, values, k_scaler, v_scaler = scoped("attn_insert_cache", cache.update, xk, xv, self.layer_id, defer_append=True)
      bsz, hkv, _, dim = xk.shape
      hs = k_scaler.shape[0]
      new = dict(new_key=torch.empty((bsz, hkv, 1, dim), dtype=torch.int8, device=xk.device),
                 new_value=torch.empty((bsz, hkv, 1, dim), dtype=torch.int8, device=xk.device),
                 new_k_scaler=torch.empty((bsz, hs), dtype=k_scaler.dtype, device=xk.device),
                 new_v_scaler=torch.empty((bsz, hs), dtype=k_scaler.dtype, device=xk.device),
                 new_key_raw=xk.contiguous(), new_value_raw=xv.contiguous(), new_rounding=cache.rounding,
                 new_key_rope=freqs_cis)
      return scoped("attn_qkv+attn_new_qkv+attn_global", self._attend, xq, keys, values, k_scaler, v_scaler, mask, *args, new_token=new)[0]
    # the ragged launch can quantise the token itself (one launch less)
    fuse_quant = (self.fuse_quantize and isinstance(cache, Int8KVCacheGenerate)
                  and self._will_fuse(seqlen, cache.cache_k) and xk.dtype == torch.bfloat16
                  and xk.is_contiguous() and xv.is_contiguous())
    ret = scoped("attn_insert_cache", cache.update, xk, xv, self.layer_id, defer_quantize=True) if fuse_quant \
        else scoped("attn_insert_cache", cache.update, xk, xv, self.layer_id, **rope_kw)
    if len(ret) == 4:  # int8 pages: (codes k, codes v, scale pages k, scale pages v)
      orig_keys, orig_values, k_scaler, v_scaler = ret
      new_key = new_value = new_k_scaler = new_v_scaler = None
    else:
      (orig_keys, orig_values, new_key, new_value, k_scaler, v_scaler, new_k_scaler,
       new_v_scaler) = ret
    if new_key is not None and self._will_fuse(seqlen, orig_keys):
      new = dict(new_key=new_key, new_value=new_value, new_k_scaler=new_k_scaler,
                 new_v_scaler=new_v_scaler)
      if fuse_quant:
        new.update(new_key_raw=xk, new_value_raw=xv, new_rounding=cache.rounding, new_key_rope=freqs_cis)
      return scoped("attn_qkv+attn_new_qkv+attn_global", self._attend, xq, orig_keys, orig_values, k_scaler,
                    v_scaler, mask, *args, new_token=new)[0]
    existing_output, (existing_max, existing_denom) = scoped(
        "attn_qkv", self._attend, xq, orig_keys, orig_values, k_scaler, v_scaler, mask, *args)
    if not self.env.lazy_cache_update or seqlen > 1:
      return existing_output
    # over the QUANTISED new token, as the reference does (layers.py:704-706)
    new_output, (new_max, new_denom) = scoped(
        "attn_new_qkv", self._attend, xq, new_key, new_value, new_k_scaler, new_v_scaler, None, *args)
    return scoped("attn_global", ak.lse_merge, existing_output, existing_max, existing_denom, new_output,
                  new_max, new_denom)
