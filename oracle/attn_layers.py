"""Decode-step orchestration of the attention call (test infrastructure).

Follows jetstream_pt/layers.py:416-550 (AttentionKernel) and :586-718
(Int8KVAttentionKernel): cache.update, attention over the returned cache with
the implementation the mode flags select, and - in lazy mode - a second
attention over the single new token merged by log-sum-exp.

The reference pads a single query row to two rows on some branches
(layers.py:449-457, :619-623) and slices the padding off again; the padding
row never influences row 0, so it is not restated.
"""


from . import attention as A


class AttentionKernel:

  def __init__(self, env, layer_id, sm_scale_paged=1.0):
    self.env, self.layer_id = env, layer_id
    self.sm_scale_paged = sm_scale_paged

  def _attend(self, xq, keys, values, k_scaler, v_scaler, mask, cache, end):
    env = self.env
    bsz, num_heads, seqlen, head_dim = xq.shape
    local_max = local_denom = None
    if env.ragged_mha and seqlen == 1 and keys.shape[-2] > 1:
      out, (local_max, local_denom) = A.ragged_mha(
          xq, keys, values, self.layer_id, None, end, None, None, k_scaler,
          v_scaler, bk=env.block_size,
      )
    elif env.flash_attention and seqlen == 1:
      out, (local_max, local_denom) = A.flash_attention(
          xq, keys, values, self.layer_id, k_scaler, v_scaler, mask,
      )
    elif env.page_attention and seqlen == 1 and k_scaler is None:
      pam = cache.page_attention_manager
      out = A.paged_attention(
          xq.squeeze(2), keys, values, pam.lengths, pam.page_indices,
          sm_scale=self.sm_scale_paged,
      )
    else:
      out = A.dense_attention(xq, keys, values, k_scaler, v_scaler, mask)
    out = out.reshape(bsz, num_heads, seqlen, head_dim)
    if local_max is not None:
      local_max = local_max.reshape(bsz, num_heads, seqlen, 1)
      local_denom = local_denom.reshape(bsz, num_heads, seqlen, 1)
    return out, (local_max, local_denom)

  def __call__(self, xq, xk, xv, mask, cache, start=None, end=None,
               ragged_batch_index=None, ragged_block_index=None):
    seqlen = xq.shape[2]
    keys, values = cache.update(xk, xv, self.layer_id)  # layers.py:521
    out, (mx, den) = self._attend(xq, keys, values, None, None, mask, cache, end)
    if not self.env.lazy_cache_update or seqlen > 1:  # layers.py:530
      return out
    new_out, (new_mx, new_den) = self._attend(
        xq, xk, xv, None, None, None, cache, end)  # layers.py:535
    return A.merge_new_token(out, mx, den, new_out, new_mx, new_den)


class Int8KVAttentionKernel(AttentionKernel):

  def __call__(self, xq, xk, xv, mask, cache, start=None, end=None,
               ragged_batch_index=None, ragged_block_index=None):
    seqlen = xq.shape[2]
    (keys, values, new_key, new_value, k_scaler, v_scaler, new_k_scaler,
     new_v_scaler) = cache.update(xk, xv, self.layer_id)  # layers.py:677-686
    out, (mx, den) = self._attend(
        xq, keys, values, k_scaler, v_scaler, mask, cache, end)
    if not self.env.lazy_cache_update or seqlen > 1:  # layers.py:698
      return out
    # layers.py:704-706: over the QUANTISED new token
    new_out, (new_mx, new_den) = self._attend(
        xq, new_key, new_value, new_k_scaler, new_v_scaler, None, cache, end)
    return A.merge_new_token(out, mx, den, new_out, new_mx, new_den)
