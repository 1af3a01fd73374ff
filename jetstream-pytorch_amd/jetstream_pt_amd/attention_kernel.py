"""Decode attention entry points backed by the HIP kernels.

Same names and argument order as the reference module
(jetstream_pt/attention_kernel.py): dense_attention (:628), flash_attention
(:688), ragged_mqa (:122), ragged_mqa_reference (:342), ragged_mha (:480),
RaggedAttentionKernel (:713), shard_kv_heads (:762), call_paged_attention
(:789), reshape_heads / reshape_outputs (:583-602).  Tensors are torch tensors
on the ROCm device; sharding arguments are accepted and ignored (one GPU).

Additions, all keyword-only or optional:
  * `sm_scale` on call_paged_attention.  The reference hands an unscaled q to
    JAX's external kernel; the only saved output the reference holds is
    reproduced by a softmax without 1/sqrt(head_dim), so 1.0 is the default.
  * `new_key` / `new_value` (+ scalers) on ragged_mha: the step's own token is
    attended as one more position inside the same launch, which is what the
    reference's lazy-update path does with a second flash_attention call and a
    log-sum-exp merge (layers.py:534-550).
  * `new_key_raw` / `new_value_raw` on ragged_mha (int8 cache): the step's
    token before quantisation.  The attention launch then quantises it too
    (Int8KVCacheGenerate.quantize, cache_manager.py:532-537) and WRITES
    `new_key` / `new_value` and their scalers, saving the separate launch.
    With `new_key_rope` (the step's freqs_cis) the key is taken unrotated and
    apply_rotary_emb (layers.py:368-379) is applied to it there as well.
  * `precompute_ragged_block_indices` returns a DecodePlan; pass it where the
    reference passes its `ragged_batch_index` table and every layer of the
    decode step reuses one split plan instead of re-planning per layer.
"""

import collections
import ctypes
import math
import weakref

import torch

from . import _ffi
from .quantize import _rounding_code


# ---- workspace and split plans ----------------------------------------------------


_live_workspaces = weakref.WeakSet()  # every workspace still in use, for check_status()


class _Workspace:
  """Device scratch for the split-KV kernel; the leading state block stays zero."""

  def __init__(self, nbytes, device):
    self.buf = torch.zeros(nbytes, dtype=torch.uint8, device=device)
    _live_workspaces.add(self)

  @property
  def nbytes(self):
    return self.buf.numel()


_workspaces = {}
_dense_workspaces = collections.OrderedDict()  # most recently used last
_MAX_DENSE_WORKSPACES = 8
_FAST_MAX_ROWS = 16  # query rows per KV head (rep * T) the streaming kernel takes


def _streaming_kernel_may_run(rows, dim, q_dtype, kv_dtype):
  """Whether the library's streaming kernel can take this shape at all; other
  shapes go to its shape-generic kernel, which uses no workspace and no plan."""
  return (rows <= _FAST_MAX_ROWS and dim == 128 and q_dtype == torch.bfloat16
          and kv_dtype in (torch.int8, torch.bfloat16))


STATUS_GAVE_UP, STATUS_SLOT_FULL, STATUS_PLAN_OVERFLOW = 1, 2, 4


def check_status(plan=None):
  """Raises RuntimeError if a streaming-kernel launch gave up since the last
  check (a bounded in-kernel wait ran out: its outputs, and those of every
  launch on that workspace since, are not to be used), or if a plan did not fit
  its array.  Looks at `plan`'s workspace, or at every workspace still alive
  (the shared ones and those of every DecodePlan).
  Synchronises the current stream; the record is cleared by the check, and
  after a launch that gave up the library puts the plan's counters back, so
  the plan can be used again.  Call it where the decode loop synchronises
  anyway - where the step's ResultTokens (engine.py:828-834) are copied to the
  host - not inside a captured step.
  Returns the remaining status bits: STATUS_SLOT_FULL says that a planned step
  saw a slot at cache capacity, whose new token (if the step carries one) was
  attended but not stored."""
  if plan is not None:
    spaces = [plan.workspace]
  else:
    spaces = list(_live_workspaces)
  bad = 0
  for ws in spaces:
    word = ctypes.c_int32(0)
    _ffi.check(_ffi.lib.jpt_attn_status(_ffi.ptr(ws.buf), _ffi.stream(), ctypes.byref(word)))
    bad |= word.value
  if bad & STATUS_GAVE_UP:
    raise RuntimeError("a decode attention launch gave up on a bounded wait inside the kernel; "
                       "its outputs (and any token it was to quantise or append) are not valid")
  if bad & STATUS_PLAN_OVERFLOW:
    raise RuntimeError("a decode attention plan had more entries than its array holds; "
                       "the outputs of launches on that plan are not valid")
  return bad & ~(STATUS_GAVE_UP | STATUS_PLAN_OVERFLOW)


def _shared_workspace(nbytes, device):
  # one per (device, stream): calls that share a workspace must not overlap
  key = (torch.device(device), torch.cuda.current_stream(device).cuda_stream)
  ws = _workspaces.get(key)
  if ws is None or ws.nbytes < nbytes:
    ws = _Workspace(nbytes, device)
    _workspaces[key] = ws
  return ws


class DecodePlan:
  """The split of a decode step's per-slot lengths into workgroup chunks,
  computed once and reused by every layer of the step."""

  def __init__(self, lengths, batch, q_heads, kv_heads, q_rows=1, *, seq=None,
               page_size=None, max_pages=None):
    self.lengths = _ffi.dev(lengths, "lengths")
    self.paged = page_size is not None
    self.key = (batch, q_heads, kv_heads, q_rows, seq, page_size, max_pages)
    args = _ffi.AttnArgs(
        lengths=_ffi.ptr(lengths), batch=batch, q_heads=q_heads, kv_heads=kv_heads,
        q_rows=q_rows, seq=seq or 0, page_size=page_size or 0, max_pages=max_pages or 0)
    nbytes = _ffi.lib.jpt_attn_workspace_bytes(args)
    self.workspace = _Workspace(nbytes, lengths.device)
    args.workspace = _ffi.ptr(self.workspace.buf)
    args.workspace_bytes = nbytes
    self._args = args
    self.replan()

  def replan(self):
    """Plans again for the current contents of `lengths` (same tensor, same workspace)."""
    _ffi.check(_ffi.lib.jpt_attn_plan(self._args, int(self.paged), _ffi.stream()))


def paged_decode_plan(pam, lengths, batch, q_heads, kv_heads, page_size, max_pages):
  """The split plan of a paged decode step, planned once per change of the page
  manager's tables and shared by every layer's call_paged_attention (the paged
  counterpart of precompute_ragged_block_indices).  Kept on the manager."""
  key = (batch, q_heads, kv_heads, 1, None, page_size, max_pages)
  version = getattr(pam, "_version", None)
  plan = getattr(pam, "_decode_plan", None)
  if plan is None or plan.key != key or plan.lengths.data_ptr() != lengths.data_ptr():
    plan = DecodePlan(lengths, batch, q_heads, kv_heads, page_size=page_size, max_pages=max_pages)
    pam._decode_plan = plan
  elif version is None or version != pam._decode_plan_version:
    plan.replan()
  pam._decode_plan_version = version
  return plan


def precompute_ragged_block_indices(end, batch, q_heads, kv_heads, seq, q_rows=1):
  """Per-step planning for ragged_mha.

  Stands where the reference's precompute_ragged_block_indices stands
  (engine.py:674-729): called once per decode step, its result is handed to
  every layer's ragged attention call.  Returns (plan, None) so it unpacks
  like the reference's (ragged_batch_index, ragged_block_index).
  """
  end = _ffi.as_i32(end, end.device if isinstance(end, torch.Tensor) else "cuda", batch)
  return DecodePlan(end, batch, q_heads, kv_heads, q_rows, seq=seq), None


# ---- the one launcher behind every entry point ---------------------------------------


def _scale_tensor(s, paged):
  """Dense scalers (B, Hs, S, 1) or (B, Hs, S); scale pages (Hs, P, ps).
  Returns the contiguous tensor and Hs."""
  if not paged and s.dim() == 4:
    s = s.squeeze(-1)
  if s.dim() != 3:
    raise ValueError(f"scaler has shape {tuple(s.shape)}")
  return _ffi.dev(s, "scaler"), s.shape[0 if paged else 1]


def _attend(mode, xq, keys, values, *, lengths=None, page_table=None, mask=None,
            k_scaler=None, v_scaler=None, sm_scale=None, new_key=None,
            new_value=None, new_k_scaler=None, new_v_scaler=None, new_key_raw=None,
            new_value_raw=None, new_rounding="trunc", new_key_rope=None, new_to_pages=False,
            want_stats=False, plan=None, force_generic=False):
  """xq (B, Hq, T, D); keys/values (B, Hkv, S, D) or pages (Hkv, P, ps, D).
  Returns (o (B, Hq, T, D), max (B, Hq, T) | None, denom (B, Hq, T) | None)."""
  xq = _ffi.dev(xq, "xq")
  keys, values = _ffi.dev(keys, "keys"), _ffi.dev(values, "values")
  b, hq, t, d = xq.shape
  device = xq.device
  a = _ffi.AttnArgs()
  a.q, a.k, a.v = _ffi.ptr(xq), _ffi.ptr(keys), _ffi.ptr(values)
  a.batch, a.q_heads, a.q_rows, a.dim = b, hq, t, d
  a.q_dtype = _ffi.dtype_code(xq.dtype)
  a.kv_dtype = _ffi.dtype_code(keys.dtype)
  if keys.shape != values.shape or keys.dtype != values.dtype:
    raise ValueError("keys and values must agree in shape and dtype")
  keep = [xq, keys, values]  # tensors the enqueued kernel reads
  if mode == "paged":
    hkv, total, ps, dk = keys.shape
    a.kv_heads, a.total_pages, a.page_size = hkv, total, ps
    page_table = _ffi.dev(page_table, "page_indices")
    if page_table.dtype != torch.int32 or page_table.shape[0] != b:
      raise ValueError("page_indices must be int32 (batch, max_pages)")
    a.max_pages = page_table.shape[1]
    a.page_table = _ffi.ptr(page_table)
    keep.append(page_table)
  else:
    if keys.dim() != 4 or keys.shape[0] != b:
      raise ValueError(f"keys {tuple(keys.shape)} do not match xq {tuple(xq.shape)}")
    _, hkv, s, dk = keys.shape
    a.kv_heads, a.seq = hkv, s
  if dk != d:
    raise ValueError(f"head_dim mismatch: q {d}, keys {dk}")
  if lengths is not None:
    lengths = _ffi.as_i32(lengths, device, b)
    a.lengths = _ffi.ptr(lengths)
    keep.append(lengths)
  if k_scaler is not None:
    ks, hs = _scale_tensor(k_scaler, mode == "paged")
    vs, _ = _scale_tensor(v_scaler, mode == "paged")
    if ks.dtype != vs.dtype or ks.shape != vs.shape:
      raise ValueError("k_scaler and v_scaler must agree in shape and dtype")
    a.k_scale, a.v_scale = _ffi.ptr(ks), _ffi.ptr(vs)
    a.scale_dtype, a.scale_heads = _ffi.dtype_code(ks.dtype), hs
    keep += [ks, vs]
  if mask is not None:
    s = keys.shape[2]
    mask = _ffi.dev(mask, "mask") if mask.is_contiguous() else mask
    m4 = mask
    while m4.dim() < 4:
      m4 = m4.unsqueeze(0)
    if m4.shape[-1] != s or m4.stride(-1) != 1:
      m4 = m4.expand(*m4.shape[:-1], s).contiguous()
    m4 = m4.expand(b, hq, t, s)
    if m4.dtype not in (torch.float32, torch.bfloat16):
      m4 = m4.float()
    a.mask = _ffi.ptr(m4)
    a.mask_dtype = _ffi.dtype_code(m4.dtype)
    a.mask_stride_b, a.mask_stride_h, a.mask_stride_t = m4.stride(0), m4.stride(1), m4.stride(2)
    keep.append(m4)
  if new_key is not None:
    nk, nv = _ffi.dev(new_key, "new_key"), _ffi.dev(new_value, "new_value")
    if nk.shape != (b, hkv, 1, d) or nk.dtype != keys.dtype:
      raise ValueError("new_key must be (batch, kv_heads, 1, dim) in the cache dtype")
    a.new_k, a.new_v = _ffi.ptr(nk), _ffi.ptr(nv)
    keep += [nk, nv]
    if new_k_scaler is not None:
      nks = _ffi.dev(new_k_scaler, "new_k_scaler").to(ks.dtype)
      nvs = _ffi.dev(new_v_scaler, "new_v_scaler").to(ks.dtype)
      a.new_k_scale, a.new_v_scale = _ffi.ptr(nks), _ffi.ptr(nvs)
      keep += [nks, nvs]
    if new_key_raw is not None:
      # the launch quantises the token itself: new_key/new_value and their
      # scalers are written, so they must be the caller's own tensors
      rk, rv = _ffi.dev(new_key_raw, "new_key_raw"), _ffi.dev(new_value_raw, "new_value_raw")
      if rk.shape != (b, hkv, 1, d) or rk.dtype != torch.bfloat16 or rv.shape != rk.shape \
          or rv.dtype != rk.dtype or not (rk.is_contiguous() and rv.is_contiguous()):
        raise ValueError("new_key_raw/new_value_raw must be contiguous bf16 (batch, kv_heads, 1, dim)")
      if new_k_scaler is None or nks is not new_k_scaler or nvs is not new_v_scaler \
          or nk is not new_key or nv is not new_value:
        raise ValueError("with new_key_raw, new_key/new_value and their scalers are outputs: "
                         "contiguous device tensors in the cache's dtypes")
      a.new_k_raw, a.new_v_raw = _ffi.ptr(rk), _ffi.ptr(rv)
      a.new_rounding = _rounding_code(new_rounding)
      keep += [rk, rv]
      if new_key_rope is not None:  # new_key_raw is unrotated
        rope = _ffi.rope_factors(new_key_rope, b, d, "new_key_rope")
        a.new_k_rope = _ffi.ptr(rope)
        keep.append(rope)
    elif new_key_rope is not None:
      raise ValueError("new_key_rope goes with new_key_raw (the launch that quantises the token rotates it)")
  if new_to_pages:
    if mode != "paged" or new_key is None:
      raise ValueError("new_to_pages goes with paged attention and a new token")
    a.new_to_pages = 1
  a.sm_scale = 1.0 / math.sqrt(d) if sm_scale is None else float(sm_scale)
  a.force_generic = int(force_generic)

  out = torch.empty_like(xq)
  a.out = _ffi.ptr(out)
  omax = oden = None
  if want_stats:
    omax = torch.empty((b, hq, t), dtype=torch.float32, device=device)
    oden = torch.empty((b, hq, t), dtype=torch.float32, device=device)
    a.out_max, a.out_denom = _ffi.ptr(omax), _ffi.ptr(oden)

  ws = None
  if not _streaming_kernel_may_run(hq // hkv * t, d, xq.dtype, keys.dtype) or force_generic:
    pass  # prefill-shaped and other calls of the generic kernel: no workspace, no plan
  elif plan is not None and plan.key == (b, hq, hkv, t, a.seq or None, a.page_size or None,
                                         a.max_pages or None) and lengths is not None \
      and plan.lengths.data_ptr() == lengths.data_ptr():
    ws, a.reuse_plan = plan.workspace, 1
  elif lengths is None and mode == "dense":
    # every slot attends all `seq` positions: the split depends on the shape
    # only, so it is planned once per (stream, shape) into a workspace of its
    # own; the least recently used of these is dropped when there are too many
    key = (torch.device(device), torch.cuda.current_stream(device).cuda_stream, b, hq, hkv, t, a.seq)
    ws = _dense_workspaces.get(key)
    if ws is None:
      ws = _Workspace(_ffi.lib.jpt_attn_workspace_bytes(a), device)
      pa = _ffi.AttnArgs(batch=b, q_heads=hq, kv_heads=hkv, q_rows=t, seq=a.seq,
                         workspace=_ffi.ptr(ws.buf), workspace_bytes=ws.nbytes)
      if _ffi.lib.jpt_attn_plan(pa, 0, _ffi.stream()) == _ffi.OK:
        _dense_workspaces[key] = ws
        a.reuse_plan = 1
        while len(_dense_workspaces) > _MAX_DENSE_WORKSPACES:
          _dense_workspaces.popitem(last=False)
    else:
      _dense_workspaces.move_to_end(key)
      a.reuse_plan = 1
  else:
    ws = _shared_workspace(_ffi.lib.jpt_attn_workspace_bytes(a), device)
  if ws is not None:
    a.workspace, a.workspace_bytes = _ffi.ptr(ws.buf), ws.nbytes

  fn = {"ragged": _ffi.lib.jpt_attn_ragged, "dense": _ffi.lib.jpt_attn_dense,
        "paged": _ffi.lib.jpt_attn_paged}[mode]
  _ffi.check(fn(a, _ffi.stream()))
  del keep
  return out, omax, oden


# ---- reference-named entry points ----------------------------------------------------


def reshape_heads(xq, keys):
  """Folds the q heads that share a KV head into rows (reference :583-590)."""
  bq, hq, tq, dq = xq.shape
  hkv = keys.shape[-3]
  rep = hq // hkv
  if rep > 1:
    xq = xq.reshape(bq, hkv, rep * tq, dq)
  return xq, rep


def reshape_outputs(rep, o, m=None, d=None):
  """Unfolds what reshape_heads folded (reference :593-602)."""
  bq, hqo, tqo, dq = o.shape
  tq, hq = tqo // rep, hqo * rep
  o = o.reshape(bq, hq, tq, dq)
  if m is not None and d is not None:
    m = m.reshape(bq, hq, tq, 1)
    d = d.reshape(bq, hq, tq, 1)
  return o, (m, d)


def _pick_layer(keys, values, layer, k_scaler, v_scaler):
  if keys.dim() == 5:
    keys, values = keys[layer], values[layer]
    if k_scaler is not None and k_scaler.dim() == 5:
      k_scaler, v_scaler = k_scaler[layer], v_scaler[layer]
  return keys, values, k_scaler, v_scaler


def dense_attention(xq, keys, values, k_scaler=None, v_scaler=None, mask=None):
  """softmax(q k^T / sqrt(d) * k_scaler + mask) * v_scaler @ v over every
  cache position; returns o (B, Hq, T, D).  Scores are kept in float32, where
  the reference keeps them in the activation dtype."""
  out, _, _ = _attend("dense", xq, keys, values, mask=mask, k_scaler=k_scaler, v_scaler=v_scaler)
  return out


def flash_attention(xq, keys, values, layer, k_scaler=None, v_scaler=None, mask=None,
                    normalize_var=True):
  """Same attention, also returning the row max and the softmax denominator:
  o (B, Hq, T, D), (max, denom) each (B, Hq, T, 1)."""
  keys, values, k_scaler, v_scaler = _pick_layer(keys, values, layer, k_scaler, v_scaler)
  sm = None if normalize_var else 1.0
  out, mx, den = _attend("dense", xq, keys, values, mask=mask, k_scaler=k_scaler,
                         v_scaler=v_scaler, sm_scale=sm, want_stats=True)
  return out, (mx.unsqueeze(-1), den.unsqueeze(-1))


def ragged_mha(q, k, v, layer, start, end, ragged_batch_index=None,
               ragged_block_index=None, k_scaler=None, v_scaler=None, bk=512,
               mask_value=None, normalize_var=True, q_shard_axis=0,
               kv_shard_axis=0, testing=False, *, new_key=None, new_value=None,
               new_k_scaler=None, new_v_scaler=None, new_key_raw=None, new_value_raw=None,
               new_rounding="trunc", new_key_rope=None):
  """Left-aligned ragged attention: slot b attends positions < end[b].

  Returns what the reference returns: o folded to (B, Hkv, rep*T, D) and
  (m, l) each (B, Hkv, rep*T).  `start`, `bk`, `mask_value` and the shard
  axes are accepted for signature compatibility; `ragged_batch_index` may
  carry a DecodePlan (see precompute_ragged_block_indices).
  """
  del start, ragged_block_index, bk, mask_value, q_shard_axis, kv_shard_axis, testing
  k, v, k_scaler, v_scaler = _pick_layer(k, v, layer, k_scaler, v_scaler)
  plan = ragged_batch_index if isinstance(ragged_batch_index, DecodePlan) else None
  out, mx, den = _attend(
      "ragged", q, k, v, lengths=end, k_scaler=k_scaler, v_scaler=v_scaler,
      sm_scale=None if normalize_var else 1.0, new_key=new_key, new_value=new_value,
      new_k_scaler=new_k_scaler, new_v_scaler=new_v_scaler, new_key_raw=new_key_raw,
      new_value_raw=new_value_raw, new_rounding=new_rounding, new_key_rope=new_key_rope,
      want_stats=True, plan=plan)
  bq, hq, tq, dq = q.shape
  hkv = k.shape[-3]
  rows = hq // hkv * tq
  return out.reshape(bq, hkv, rows, dq), (mx.reshape(bq, hkv, rows), den.reshape(bq, hkv, rows))


def ragged_mqa_reference(q, k, v, layer, start, end, ragged_batch_index=None,
                         ragged_block_index=None, k_scaler=None, v_scaler=None, bk=512,
                         mask_value=None, normalize_var=True, testing=False, quantized=False):
  """The reference's per-KV-head entry point (attention_kernel.py:342-466), which its
  ragged_mha vmaps over the heads: q (B, T, D); k, v (B, S, D), or stacked
  (L, B, S, D) with `layer` picking one; scalers (B, 1, S) / (L, B, 1, S) or None.
  Returns o (B, T, D) in q's dtype and (m, l), each (B, T) float32.  Here it is
  ragged_mha on a single head (the launch covers all heads at once, so callers
  with several heads should call ragged_mha)."""
  del quantized  # told by the scalers
  if k.dim() == 4:  # stacked
    k, v = k[layer], v[layer]
    if k_scaler is not None and k_scaler.dim() == 4:
      k_scaler, v_scaler = k_scaler[layer], v_scaler[layer]
  if q.dim() != 3 or k.dim() != 3:
    raise ValueError(f"ragged_mqa takes q (B, T, D) and k (B, S, D); got {tuple(q.shape)}, {tuple(k.shape)}")
  out, (m, l) = ragged_mha(q.unsqueeze(1), k.unsqueeze(1), v.unsqueeze(1), 0, start, end,
                           ragged_batch_index, ragged_block_index, k_scaler, v_scaler, bk=bk,
                           mask_value=mask_value, normalize_var=normalize_var, testing=testing)
  return out.squeeze(1), (m.squeeze(1), l.squeeze(1))


# The reference's Pallas variant of the same function (attention_kernel.py:122-252);
# one implementation serves both names here.
ragged_mqa = ragged_mqa_reference


def shard_kv_heads(paged_attention_impl, mesh=None, kv_head_mesh_axis_name=None):
  """The reference wraps its paged kernel in a shard_map over the KV heads of a
  device mesh (attention_kernel.py:762-786).  On one GPU every head is local:
  the function comes back as it is."""
  del mesh, kv_head_mesh_axis_name
  return paged_attention_impl


class RaggedAttentionKernel:
  """Callable with the reference's constructor and call signature (:713-759)."""

  def __init__(self, env, input_specs=None, output_specs=None, q_shard_axis=0, kv_shard_axis=0):
    self.env = env

  def __call__(self, xq, keys, values, layer, start, end, ragged_batch_index=None,
               ragged_block_index=None, k_scaler=None, v_scaler=None, **new_token):
    return ragged_mha(xq, keys, values, layer, start, end, ragged_batch_index,
                      ragged_block_index, k_scaler, v_scaler, bk=self.env.block_size,
                      **new_token)


def call_paged_attention(env, xq, keys, values, seq_lens, page_indices, *, sm_scale=1.0,
                         k_scaler=None, v_scaler=None, plan=None, append=None):
  """Paged decode attention: xq (B, Hq, D), pages (Hkv, P, ps, D), seq_lens
  (B,), page_indices (B, max_pages); returns (B, Hq, D).  seq_lens and
  page_indices may be numpy arrays (as PageAttentionManager holds them) or
  int32 device tensors.  With int8 pages pass scale pages (Hs, P, ps).

  append: None, or the step's own token as a dict of the new-token keywords of
  ragged_mha (new_key/new_value in the pages' dtype with their scalers, or
  new_key_raw/new_value_raw bf16 plus output tensors).  The launch then also
  appends the token to the pages (PageKVCacheGenerate.update's scatter,
  cache_manager.py:663-724) and attends it: seq_lens are the lengths BEFORE the
  step, slots of length 0 are inactive, and the page of position seq_lens[b]
  must already be in page_indices."""
  del env
  device = xq.device
  if not isinstance(page_indices, torch.Tensor):
    import numpy as np
    page_indices = torch.from_numpy(np.ascontiguousarray(page_indices, dtype=np.int32)).to(device)
  extra = {} if append is None else dict(append, new_to_pages=True)
  out, _, _ = _attend("paged", xq.unsqueeze(2), keys, values, lengths=seq_lens,
                      page_table=page_indices, k_scaler=k_scaler, v_scaler=v_scaler,
                      sm_scale=sm_scale, plan=plan, **extra)
  return out.squeeze(2)


def lse_merge(existing_output, existing_max, existing_denom, new_output, new_max, new_denom):
  """out = (l1 a o1 + b o2 l2) / (a l1 + b l2) with a = exp(m1 - g),
  b = exp(m2 - g), g = max(m1, m2) (reference: layers.py:539-548)."""
  o1, o2 = _ffi.dev(existing_output, "existing_output"), _ffi.dev(new_output.contiguous(), "new_output")
  dim = o1.shape[-1]
  rows = o1.numel() // dim
  f = lambda x: _ffi.dev(x.to(torch.float32).reshape(-1).contiguous(), "stat")
  m1, l1, m2, l2 = f(existing_max), f(existing_denom), f(new_max), f(new_denom)
  if o2.dtype != o1.dtype:
    o2 = o2.to(o1.dtype)
  out = torch.empty_like(o1)
  _ffi.check(_ffi.lib.jpt_lse_merge(
      _ffi.ptr(out), _ffi.ptr(o1), _ffi.ptr(m1), _ffi.ptr(l1), _ffi.ptr(o2), _ffi.ptr(m2),
      _ffi.ptr(l2), rows, dim, _ffi.dtype_code(o1.dtype), _ffi.stream()))
  return out
