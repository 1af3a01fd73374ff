"""ctypes binding of libjpt_mi355.so (the C ABI declared in include/jpt_mi355.h).

There is no fallback: if the library is missing, importing this module raises,
and every op needs its tensors on the ROCm device.
"""

import ctypes
import os
import queue

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("JPT_MI355_LIB") or os.path.join(_HERE, "libjpt_mi355.so")

if not os.path.exists(LIB_PATH):
  raise ImportError(
      f"{LIB_PATH} is missing: build it with `python jetstream-pytorch_amd/build_lib.py` "
      "(hipcc, gfx950). jetstream_pt_amd has no CPU or PyTorch fallback."
  )

lib = ctypes.CDLL(LIB_PATH)

OK, E_BADARG, E_NOPAGES, E_PAGE_OVERFLOW, E_HIP = 0, -1, -2, -3, -4
BF16, F32, I8 = 0, 1, 2
ROUND_TRUNC, ROUND_RNE = 0, 1
ATTN_WS_STATE_BYTES = 65536
ATTN_STATIC_SCRATCH_BYTES = 8 << 20
MAX_LINE_TENSORS = 4

_c = ctypes
_vp, _i32, _i64, _f32 = _c.c_void_p, _c.c_int32, _c.c_int64, _c.c_float
_i32p = _c.POINTER(_c.c_int32)


class LineTensor(_c.Structure):
  _fields_ = [("dst", _vp), ("src", _vp), ("heads", _i32), ("row_bytes", _i32)]


class QuantAppendArgs(_c.Structure):
  _fields_ = [
      ("new_k", _vp), ("new_v", _vp), ("cache_k", _vp), ("cache_v", _vp),
      ("k_scale", _vp), ("v_scale", _vp), ("out_k", _vp), ("out_v", _vp),
      ("out_k_scale", _vp), ("out_v_scale", _vp), ("pos", _vp),
      ("pos_count", _i32), ("batch", _i32), ("heads", _i32), ("seq", _i32),
      ("dim", _i32), ("in_dtype", _i32), ("scale_dtype", _i32),
      ("scale_heads", _i32), ("rounding", _i32), ("rope", _vp),
  ]


class PagedQuantAppendArgs(_c.Structure):
  _fields_ = [
      ("new_k", _vp), ("new_v", _vp), ("pages_k", _vp), ("pages_v", _vp),
      ("k_scale_pages", _vp), ("v_scale_pages", _vp), ("indices", _vp),
      ("n_active", _i32), ("batch", _i32), ("heads", _i32),
      ("total_pages", _i32), ("page_size", _i32), ("dim", _i32),
      ("in_dtype", _i32), ("scale_dtype", _i32), ("scale_heads", _i32),
      ("rounding", _i32), ("n_active_dev", _vp), ("indices_stride", _i32),
      ("rope", _vp),
  ]


class Dpam(_c.Structure):
  _fields_ = [
      ("state", _vp), ("ring", _vp), ("page_indices", _vp), ("lengths", _vp),
      ("n_alloc", _vp), ("update_indices", _vp), ("batch", _i32),
      ("total_pages", _i32), ("page_size", _i32), ("max_pages", _i32),
  ]


DPAM_NOPAGES, DPAM_OVERFLOW, DPAM_BADARG = 1, 2, 4


class PrefillInsertArgs(_c.Structure):
  _fields_ = [
      ("src_k", _vp), ("src_v", _vp), ("dst_k", _vp), ("dst_v", _vp),
      ("k_scale", _vp), ("v_scale", _vp), ("page_ids", _vp), ("n_pages", _i32),
      ("tokens", _i32), ("heads", _i32), ("dim", _i32), ("slot", _i32),
      ("batch", _i32), ("seq", _i32), ("start", _i32), ("total_pages", _i32),
      ("page_size", _i32), ("in_dtype", _i32), ("dst_dtype", _i32),
      ("scale_dtype", _i32), ("scale_heads", _i32), ("rounding", _i32),
      ("n_layers", _i32), ("src_layer_stride", _i64), ("dst_layer_stride", _i64),
      ("scale_layer_stride", _i64), ("src_head_stride", _i64),
  ]


class InsertLayer(_c.Structure):
  _fields_ = [("src_k", _vp), ("src_v", _vp), ("dst_k", _vp), ("dst_v", _vp),
              ("k_scale", _vp), ("v_scale", _vp)]


class InsertPrompt(_c.Structure):
  _fields_ = [("src_k", _vp), ("src_v", _vp), ("page_ids", _vp), ("src_head_stride", _i64),
              ("src_layer_stride", _i64), ("tokens", _i32), ("n_pages", _i32)]


class AttnArgs(_c.Structure):
  _fields_ = [
      ("q", _vp), ("k", _vp), ("v", _vp), ("k_scale", _vp), ("v_scale", _vp),
      ("lengths", _vp), ("page_table", _vp), ("mask", _vp), ("new_k", _vp),
      ("new_v", _vp), ("new_k_scale", _vp), ("new_v_scale", _vp), ("out", _vp),
      ("out_max", _vp), ("out_denom", _vp), ("workspace", _vp),
      ("workspace_bytes", _i64), ("mask_stride_b", _i64),
      ("mask_stride_h", _i64), ("mask_stride_t", _i64), ("batch", _i32),
      ("q_heads", _i32), ("kv_heads", _i32), ("q_rows", _i32), ("dim", _i32),
      ("seq", _i32), ("total_pages", _i32), ("page_size", _i32),
      ("max_pages", _i32), ("q_dtype", _i32), ("kv_dtype", _i32),
      ("scale_dtype", _i32), ("scale_heads", _i32), ("mask_dtype", _i32),
      ("sm_scale", _f32), ("force_generic", _i32), ("reuse_plan", _i32),
      ("new_k_raw", _vp), ("new_v_raw", _vp), ("new_rounding", _i32),
      ("new_k_rope", _vp), ("new_to_pages", _i32),
  ]


def _sig(name, restype, *argtypes):
  fn = getattr(lib, name)
  fn.restype = restype
  fn.argtypes = list(argtypes)
  return fn


_sig("jpt_version", _i32)
_sig("jpt_last_error", _c.c_char_p)
_sig("jpt_kv_scatter_lines", _i32, _c.POINTER(LineTensor), _i32, _vp, _i32, _i32, _i32, _i32, _vp)
_sig("jpt_kv_append_quant_i8", _i32, _c.POINTER(QuantAppendArgs), _vp)
_sig("jpt_rope", _i32, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp)
_sig("jpt_paged_insert", _i32, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp)
_sig("jpt_paged_append", _i32, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp)
_sig("jpt_paged_append_dev", _i32, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _i32, _i32, _i32, _vp)
_sig("jpt_paged_gather", _i32, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp)
_sig("jpt_paged_append_quant_i8", _i32, _c.POINTER(PagedQuantAppendArgs), _vp)
_sig("jpt_prefill_insert", _i32, _c.POINTER(PrefillInsertArgs), _vp)
_sig("jpt_prefill_insert_layers", _i32, _c.POINTER(PrefillInsertArgs), _c.POINTER(InsertLayer), _i32, _vp)
_sig("jpt_prefill_insert_prompts", _i32, _c.POINTER(PrefillInsertArgs), _c.POINTER(InsertPrompt), _i32, _vp)
_sig("jpt_attn_workspace_bytes", _i64, _c.POINTER(AttnArgs))
_sig("jpt_attn_plan", _i32, _c.POINTER(AttnArgs), _i32, _vp)
_sig("jpt_attn_ragged", _i32, _c.POINTER(AttnArgs), _vp)
_sig("jpt_attn_dense", _i32, _c.POINTER(AttnArgs), _vp)
_sig("jpt_attn_paged", _i32, _c.POINTER(AttnArgs), _vp)
_sig("jpt_attn_status", _i32, _vp, _vp, _i32p)
_sig("jpt_attn_ragged_static", _i32, _c.POINTER(AttnArgs), _vp)
_sig("jpt_lse_merge", _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _vp)
_sig("jpt_pam_create", _i32, _i32, _i32, _i32, _i32, _i32p, _c.POINTER(_vp))
_sig("jpt_pam_destroy", None, _vp)
_sig("jpt_pam_tables", _i32, _vp, _c.POINTER(_i32p), _c.POINTER(_i32p))
_sig("jpt_pam_reserve_insert", _i32, _vp, _i32, _i32, _i32p)
_sig("jpt_pam_reserve_decode", _i32, _vp, _i32, _i32)
_sig("jpt_pam_fill_new_pages", _i32, _vp, _i32p)
_sig("jpt_pam_page_token_indices", _i32, _vp, _i32p, _i32p, _i32p)
_sig("jpt_pam_free", _i32, _vp, _i32)
_sig("jpt_pam_free_count", _i32, _vp, _i32p)
_sig("jpt_dpam_init", _i32, _c.POINTER(Dpam), _vp, _vp)
_sig("jpt_dpam_reserve_insert", _i32, _c.POINTER(Dpam), _vp, _vp, _i32, _i32, _i32, _vp)
_sig("jpt_dpam_free", _i32, _c.POINTER(Dpam), _vp, _i32, _i32, _vp)
_sig("jpt_dpam_decode_step", _i32, _c.POINTER(Dpam), _vp, _vp)
_sig("jpt_decode_advance", _i32, _vp, _i32, _i64, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp)
_sig("jpt_ragged_block_indices", _i32, _vp, _vp, _i32, _i32, _i32, _vp, _vp, _vp)

EXPORTS = (
    "jpt_version", "jpt_last_error", "jpt_kv_scatter_lines",
    "jpt_kv_append_quant_i8", "jpt_paged_insert", "jpt_paged_append",
    "jpt_paged_gather", "jpt_paged_append_quant_i8", "jpt_prefill_insert",
    "jpt_attn_workspace_bytes", "jpt_attn_plan", "jpt_attn_ragged", "jpt_attn_dense",
    "jpt_attn_paged", "jpt_lse_merge", "jpt_pam_create", "jpt_pam_destroy",
    "jpt_pam_tables", "jpt_pam_reserve_insert", "jpt_pam_reserve_decode",
    "jpt_pam_fill_new_pages", "jpt_pam_page_token_indices", "jpt_pam_free",
    "jpt_pam_free_count", "jpt_paged_append_dev", "jpt_dpam_init", "jpt_dpam_reserve_insert",
    "jpt_dpam_free", "jpt_dpam_decode_step", "jpt_decode_advance", "jpt_rope",
    "jpt_ragged_block_indices", "jpt_prefill_insert_layers", "jpt_prefill_insert_prompts",
    "jpt_attn_status", "jpt_attn_ragged_static",
)


def check(status):
  """Maps a status code to the exception type the reference raises."""
  if status == OK:
    return
  msg = lib.jpt_last_error().decode("utf-8", "replace")
  if status == E_NOPAGES:
    raise queue.Empty(msg)
  if status == E_PAGE_OVERFLOW:
    raise IndexError(msg)
  if status == E_BADARG:
    raise ValueError(msg)
  raise RuntimeError(f"jpt_mi355 status {status}: {msg}")


_DTYPES = {torch.bfloat16: BF16, torch.float32: F32, torch.int8: I8}


def dtype_code(dtype):
  try:
    return _DTYPES[dtype]
  except KeyError:
    raise ValueError(f"unsupported dtype {dtype}") from None


def dev(t, name="tensor"):
  """Checks that `t` is a contiguous tensor on the ROCm device."""
  if not isinstance(t, torch.Tensor):
    raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
  if not t.is_cuda:
    raise RuntimeError(
        f"{name} is on {t.device}: jetstream_pt_amd runs on the ROCm device only")
  if not t.is_contiguous():
    raise ValueError(f"{name} must be contiguous (shape {tuple(t.shape)}, strides {t.stride()})")
  return t


def rope_factors(freqs_cis, rows, dim, name="freqs_cis"):
  """The step's rotary factors as a contiguous float32 (rows, dim / 2, 2) device
  tensor of (cos, sin): accepts the reference's complex64 freqs_cis
  (rows[, 1], dim / 2) - viewed, not copied - or that real layout itself."""
  f = freqs_cis
  if not isinstance(f, torch.Tensor) or not f.is_cuda:
    raise RuntimeError(f"{name} must be a tensor on the ROCm device")
  if f.is_complex():
    if f.dtype != torch.complex64:
      raise ValueError(f"{name} must be complex64")
    f = torch.view_as_real(f)
  if f.dtype != torch.float32 or f.numel() != rows * dim or f.shape[-1] != 2:
    raise ValueError(f"{name} must hold (cos, sin) float32 pairs for {rows} rows of {dim // 2} pairs, "
                     f"got {tuple(freqs_cis.shape)} {freqs_cis.dtype}")
  return f.reshape(rows, dim // 2, 2).contiguous()


def ptr(t):
  return None if t is None else _vp(t.data_ptr())


def stream():
  return _vp(torch.cuda.current_stream().cuda_stream)


def as_i32(x, device, n=None):
  """Positions / lengths as an int32 device tensor (accepts lists, numpy, any int dtype)."""
  if isinstance(x, torch.Tensor):
    t = x.to(device=device, dtype=torch.int32).reshape(-1)
  else:
    import numpy as np
    t = torch.from_numpy(np.ascontiguousarray(np.asarray(x, dtype=np.int32).reshape(-1))).to(device)
  if n is not None and t.numel() != n:
    raise ValueError(f"expected {n} entries, got {t.numel()}")
  return t.contiguous()
