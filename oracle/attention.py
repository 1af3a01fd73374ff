"""Decode attention entry points, restated on torch-CPU (test infrastructure).

Follows jetstream_pt/attention_kernel.py (ragged, dense, flash, paged) and the
merge in jetstream_pt/layers.py:539-548.  `closed_form` is the float64
textbook masked softmax attention every other function here is pinned to.
"""

import math

import numpy as np
import torch

DEFAULT_MASK_VALUE = -0.7 * float(np.finfo(np.dtype("float32")).max)  # attention_kernel.py:18


def reshape_heads(xq, keys):
  """attention_kernel.py:583-590: fold the q heads of one KV head into rows."""
  bq, hq, tq, dq = xq.shape
  rep = hq // keys.shape[-3]
  if rep > 1:
    xq = xq.reshape(bq, keys.shape[-3], rep * tq, dq)
  return xq, rep


def reshape_outputs(rep, o, m=None, d=None):
  """attention_kernel.py:593-602."""
  bq, hqo, tqo, dq = o.shape
  tq, hq = tqo // rep, hqo * rep
  o = o.reshape(bq, hq, tq, dq)
  if m is not None and d is not None:
    m = m.reshape(bq, hq, tq, 1)
    d = d.reshape(bq, hq, tq, 1)
  return o, (m, d)


def _ragged_one_head(q, k, v, end, k_scale, v_scale, bk, normalize_var, quantized):
  """ragged_mqa_kernel_reference over its (b, i) grid, attention_kernel.py:255-329.

  q (B, T, D); k, v (B, S, D); k_scale, v_scale (B, 1, S); end (B,).
  Returns o (B, T, D) in q's dtype, m, l (B, T) float32.
  """
  bsz, t, d = q.shape
  seq = k.shape[-2]
  o = torch.zeros_like(q)
  m = torch.full((bsz, t), -math.inf, dtype=torch.float32)
  l = torch.zeros((bsz, t), dtype=torch.float32)
  for b in range(bsz):
    length = int(end[b])
    qf = q[b].float()
    for i in range(seq // bk):
      if not i * bk < length:  # :289
        continue
      blk = slice(i * bk, (i + 1) * bk)
      kf, vf = k[b, blk].float(), v[b, blk].float()
      qk = qf @ kf.T  # :296
      if normalize_var:
        qk = qk / math.sqrt(d)  # :300-301
      if quantized:
        qk = qk * k_scale[b, :, blk].float()  # :303-304
      pos = i * bk + torch.arange(bk)
      mask_add = torch.where(pos < length, 0.0, DEFAULT_MASK_VALUE).float()
      qk = qk + mask_add[None, :]  # :306-307
      m_curr = qk.max(dim=-1).values
      s_curr = torch.exp(qk - m_curr[:, None])
      l_curr = s_curr.sum(dim=-1)
      if quantized:
        s_curr = s_curr * v_scale[b, :, blk].float()  # :314-315
      o_curr_times_l_curr = s_curr @ vf
      m_prev, l_prev = m[b].clone(), l[b].clone()
      m_next = torch.maximum(m_prev, m_curr)
      alpha = torch.exp(m_prev - m_next)
      beta = torch.exp(m_curr - m_next)
      l_next = alpha * l_prev + beta * l_curr
      l_next_safe = torch.where(l_next == 0.0, torch.ones_like(l_next), l_next)
      m[b], l[b] = m_next, l_next_safe
      o[b] = (
          (l_prev * alpha)[:, None] * o[b].float()
          + beta[:, None] * o_curr_times_l_curr
      ).div(l_next_safe[:, None]).to(o.dtype)  # :327-329
  return o, m, l


def ragged_mha(q, k, v, layer, start, end, ragged_batch_index=None,
               ragged_block_index=None, k_scaler=None, v_scaler=None, bk=512,
               normalize_var=True):
  """attention_kernel.py:480-580: GQA fold, then one head at a time.

  q (B, Hq, T, D); k, v (B, Hkv, S, D) or stacked (L, B, Hkv, S, D) with the
  layer picked by `layer` (:386-396); scalers (B, 1, S, 1) / (L, B, 1, S, 1).
  start and the two ragged index tables are dead inputs on this live path.
  Returns o (B, Hkv, rep*T, D), (m, l) each (B, Hkv, rep*T).
  """
  del start, ragged_batch_index, ragged_block_index
  bk = min(bk, k.shape[-2])
  q, _ = reshape_heads(q, k)
  if k.ndim == 5:
    k, v = k[layer], v[layer]
    if k_scaler is not None:
      k_scaler, v_scaler = k_scaler[layer], v_scaler[layer]
  quantized = k_scaler is not None
  bq, hkv = q.shape[0], k.shape[-3]
  tk = k.shape[-2]
  if quantized:
    k_scale, v_scale = k_scaler.squeeze(-1), v_scaler.squeeze(-1)
  else:
    k_scale = v_scale = torch.ones((bq, 1, tk), dtype=torch.bfloat16)

  def head_scale(s, h):  # one scale row per KV head, or one shared by all heads
    return s[:, h:h + 1] if s.shape[1] > 1 else s

  outs = [
      _ragged_one_head(q[:, h], k[:, h], v[:, h], end, head_scale(k_scale, h),
                       head_scale(v_scale, h), bk, normalize_var, quantized)
      for h in range(hkv)
  ]
  o = torch.stack([x[0] for x in outs], dim=1)
  m = torch.stack([x[1] for x in outs], dim=1)
  l = torch.stack([x[2] for x in outs], dim=1)
  return o, (m, l)


def _scale_view(scaler, bsz, seq):
  """(B, Hs, S, 1) -> broadcastable (B, Hs, 1, S); the reference only has Hs=1
  and writes reshape(bsz, 1, 1, S) (attention_kernel.py:613)."""
  return scaler.reshape(bsz, -1, 1, seq)


def dense_attention(xq, keys, values, k_scaler=None, v_scaler=None, mask=None):
  """attention_kernel.py:605-633, in the input dtype like the reference."""
  xq, rep = reshape_heads(xq, keys)
  bsz, _, _, head_dim = xq.shape
  if not keys.is_floating_point():
    # int8 codes: the reference's einsum runs on jnp arrays, whose type
    # promotion lifts the codes to the activation dtype (exact, |code| <= 128)
    keys, values = keys.to(xq.dtype), values.to(xq.dtype)
  scores = torch.einsum("ikjl,ikml->ikjm", xq, keys) / math.sqrt(head_dim)
  if k_scaler is not None:
    scores = scores * _scale_view(k_scaler, bsz, keys.shape[2])
  if mask is not None:
    scores = scores + mask
  scores = torch.softmax(scores.float(), dim=-1).type_as(xq)
  if v_scaler is not None:
    scores = scores * _scale_view(v_scaler, bsz, keys.shape[2])
  output = torch.einsum("ikjm,ikml->ikjl", scores, values)
  return reshape_outputs(rep, output)[0]


def flash_attention(xq, keys, values, layer=0, k_scaler=None, v_scaler=None,
                    mask=None, normalize_var=True):
  """attention_kernel.py:636-710: returns o and (max, denominator)."""
  xq, rep = reshape_heads(xq, keys)
  if keys.ndim == 5:  # :647-651
    keys, values = keys[layer], values[layer]
    k_scaler = k_scaler[layer] if k_scaler is not None else None
    v_scaler = v_scaler[layer] if v_scaler is not None else None
  bsz, seq = keys.shape[0], keys.shape[-2]
  logits = torch.einsum("bhqd,bhkd->bhqk", xq.float(), keys.float())
  if normalize_var:
    logits = logits / math.sqrt(keys.shape[-1])
  if k_scaler is not None:
    logits = logits * _scale_view(k_scaler, bsz, seq)
  if mask is not None:
    logits = logits + mask
  logits_max = logits.max(dim=-1, keepdim=True).values
  unnormalized = torch.exp(logits - logits_max)
  denominator = unnormalized.sum(dim=-1, keepdim=True)
  if v_scaler is not None:  # :676-679, after the sum
    unnormalized = unnormalized * _scale_view(v_scaler, bsz, seq)
  o = torch.einsum("bhqk,bhkd->bhqd", unnormalized.type_as(xq),
                   values.to(xq.dtype)) / denominator
  return reshape_outputs(rep, o, logits_max, denominator)


def gather_pages(pages, page_row, length):
  """PageAttentionManager._compress_cache, page_attention_manager.py:195-200."""
  head, _, _, dim = pages.shape
  idx = torch.as_tensor(np.asarray(page_row), dtype=torch.int64)
  return pages[:, idx, :, :].reshape(head, -1, dim)[:, :int(length), :]


def paged_attention(xq, k_pages, v_pages, seq_lens, page_indices, sm_scale=1.0,
                    k_scale_pages=None, v_scale_pages=None):
  """What call_paged_attention computes (attention_kernel.py:789-808).

  The arithmetic lives in JAX's external TPU kernel; this restates the
  reference's own in-repo equivalence instead (tests/test_attention_kernal.py
  :159-189: gather the slot's pages, mask to the length, dense softmax
  attention), in float64.  q (B, Hq, D); pages (Hkv, P, ps, D); optional
  scale pages (Hs, P, ps) for int8 pages.  Returns (B, Hq, D) in q's dtype.
  """
  bsz, hq, d = xq.shape
  hkv = k_pages.shape[0]
  out = torch.zeros((bsz, hq, d), dtype=torch.float64)
  for b in range(bsz):
    n = int(seq_lens[b])
    if n == 0:
      continue
    k = gather_pages(k_pages, page_indices[b], n).double()
    v = gather_pages(v_pages, page_indices[b], n).double()
    if k_scale_pages is not None:
      ks = gather_pages(k_scale_pages.unsqueeze(-1), page_indices[b], n).double()
      vs = gather_pages(v_scale_pages.unsqueeze(-1), page_indices[b], n).double()
      k, v = k * ks, v * vs
    q = xq[b].double().reshape(hkv, hq // hkv, d)
    p = torch.softmax(torch.einsum("hrd,htd->hrt", q, k) * sm_scale, dim=-1)
    out[b] = torch.einsum("hrt,htd->hrd", p, v).reshape(hq, d)
  return out.to(xq.dtype)


def merge_new_token(existing_output, existing_max, existing_denom, new_output,
                    new_max, new_denom):
  """layers.py:539-548 / :708-717: log-sum-exp merge of two partial results."""
  global_max = torch.max(existing_max, new_max)
  alpha = torch.exp(existing_max - global_max)
  beta = torch.exp(new_max - global_max)
  global_denom = alpha * existing_denom + beta * new_denom
  return (
      existing_denom * alpha * existing_output + beta * new_output * new_denom
  ) / global_denom


def closed_form(q, k, v, lengths=None, mask=None, k_scale=None, v_scale=None,
                sm_scale=None):
  """Float64 textbook attention: softmax(q k^T * sm_scale + mask) v.

  q (B, Hq, T, D); k, v (B, Hkv, S, D) (codes if scales are given, which are
  (B, Hs, S, 1)); `lengths` (B,) keeps positions < length.  Returns o
  (B, Hq, T, D) float64 plus the row max and the softmax denominator
  relative to it, both (B, Hq, T, 1); an empty row gives o = 0, max = -inf,
  denominator = 0.
  """
  bsz, hq, t, d = q.shape
  hkv, seq = k.shape[1], k.shape[2]
  rep = hq // hkv
  kd, vd = k.double(), v.double()
  if k_scale is not None:
    kd = kd * k_scale.double()
    vd = vd * v_scale.double()
  qd = q.double().reshape(bsz, hkv, rep * t, d)
  s = torch.einsum("bhrd,bhsd->bhrs", qd, kd)
  s = s * (1.0 / math.sqrt(d) if sm_scale is None else sm_scale)
  if mask is not None:
    s = s + mask.double()
  if lengths is not None:
    keep = torch.arange(seq)[None, :] < torch.as_tensor(lengths).reshape(-1, 1)
    s = s.masked_fill(~keep[:, None, None, :], -math.inf)
  mx = s.max(dim=-1, keepdim=True).values
  safe = torch.where(torch.isinf(mx), torch.zeros_like(mx), mx)
  e = torch.exp(s - safe)
  den = e.sum(dim=-1, keepdim=True)
  o = torch.einsum("bhrs,bhsd->bhrd", e, vd) / torch.where(den == 0, torch.ones_like(den), den)
  shape = (bsz, hq, t)
  return o.reshape(*shape, d), mx.reshape(*shape, 1), den.reshape(*shape, 1)
