"""The C-ABI library loads without a GPU and exports every function the public
header declares; no compute entry point is called here."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "jpt_mi355.h")


def declared_functions():
  text = open(HEADER).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\b(jpt_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
  from jetstream_pt_amd import _ffi
  names = declared_functions()
  assert len(names) >= 20
  lib = ctypes.CDLL(_ffi.LIB_PATH)
  missing = [n for n in names if not hasattr(lib, n)]
  assert not missing, f"declared in the header but not exported: {missing}"
  assert sorted(_ffi.EXPORTS) == names


def test_version_and_error_channel():
  from jetstream_pt_amd import _ffi
  assert _ffi.lib.jpt_version() == 1
  # argument validation happens before any device work
  assert _ffi.lib.jpt_attn_ragged(None, None) == _ffi.E_BADARG
  assert b"NULL" in _ffi.lib.jpt_last_error()
  with pytest.raises(ValueError):
    _ffi.check(_ffi.lib.jpt_kv_append_quant_i8(None, None))


def test_ops_refuse_cpu_tensors():
  import torch
  from jetstream_pt_amd import attention_kernel as ak
  q = torch.zeros((1, 2, 1, 8))
  with pytest.raises(RuntimeError, match="ROCm device only"):
    ak.dense_attention(q, q, q)
