"""Named ranges around the path's steps, under the names of the reference's
`jax.named_scope` blocks (layers.py:520-539, 676-708; attention_kernel.py:140,
560), so that a rocprofv3 `--marker-trace` / torch profiler timeline of a decode
step reads like the reference's.  Off unless JPT_SCOPES=1 (a range is two host
calls per step of the path; ranges mark host time, the launches are
asynchronous).
"""
import contextlib
import os

import torch

ENABLED = os.environ.get("JPT_SCOPES", "0") == "1"


@contextlib.contextmanager
def scope(name):
  if not ENABLED:
    yield
    return
  torch.cuda.nvtx.range_push(name)  # roctx on ROCm builds of torch
  try:
    yield
  finally:
    torch.cuda.nvtx.range_pop()


def scoped(name, fn, *args, **kwargs):
  with scope(name):
    return fn(*args, **kwargs)
