"""The named ranges of the path (scopes.py) carry the reference's scope names
and cost nothing when switched off."""
import importlib
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "jetstream-pytorch_amd"))


def test_scoped_is_a_plain_call_when_off(monkeypatch):
  monkeypatch.delenv("JPT_SCOPES", raising=False)
  try:
    scopes = importlib.import_module("jetstream_pt_amd.scopes")
  except (ImportError, OSError):  # the package refuses to import without its library
    import pytest
    pytest.skip("library not built")
  scopes = importlib.reload(scopes)
  assert not scopes.ENABLED
  assert scopes.scoped("attn_global", lambda a, b=1: a + b, 2, b=3) == 5
  with scopes.scope("attn_qkv"):
    pass
