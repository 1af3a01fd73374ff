import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "jetstream-pytorch_amd")):
  if p not in sys.path:
    sys.path.insert(0, p)


def pytest_configure(config):
  config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def kats():
  with open(os.path.join(ROOT, "tests", "golden", "reference_kats.json")) as f:
    return json.load(f)


# Largest absolute attention-output error each GPU parity check saw, with the
# largest magnitude of the expected values beside it; written as
# parity_max_abs.json into the run's output folder at the end of a GPU session
# (the measured errors the documentation quotes come from there).
PARITY_ERRORS = {}


def record_parity(name, got, want):
  """Returns the element-wise |got - want| (float64 CPU tensors in, or
  anything .double() takes) and remembers its maximum under `name`."""
  err = (got - want).abs()
  if err.numel():
    prev = PARITY_ERRORS.get(name, (0.0, 0.0))
    PARITY_ERRORS[name] = (max(prev[0], float(err.max())), max(prev[1], float(want.abs().max())))
  return err


# Tolerance of every attention-output check on the GPU: max-abs 1e-2 against the
# unrounded expectation.  The output is bf16, and a bf16 number differs from the
# value it stands for by up to half an ulp: 2^-8 = 0.0039 for |x| in [1, 2),
# 0.0078 in [2, 4), 0.0156 in [4, 8).  Below SMALL = 2 the bound is 1e-2 and
# nothing else.  From 2 on the output's own rounding leaves 0.002 of the 1e-2 to
# the arithmetic (measured over random caches: 0.0112 in [2, 2.56) with bf16
# probabilities, 0.0090 with int8 codes), and from 2.56 on it exceeds 1e-2 alone:
# there the half ulp, at most 2^-8 |expected|, is added to the bound.
# `rounded_want`: the expectation is itself a bf16 output (another kernel's), off
# by half an ulp of its own: two such numbers differ by a whole ulp, 2^-7 |x|,
# which is 0.0078 in [1, 2) and above 1e-2 from 2 on.
ATTN_ATOL, ATTN_HALF_ULP, ATTN_SMALL = 1e-2, 2.0 ** -8, 2.0


def attention_bound(want, rounded_want=False):
  import torch
  w = want.abs()
  n = 2 if rounded_want else 1
  return torch.where(w < ATTN_SMALL, torch.full_like(w, ATTN_ATOL), ATTN_ATOL + n * ATTN_HALF_ULP * w)


def attention_close(got, want, rounded_want=False):
  """True if every element of `got` is finite and within attention_bound of `want`."""
  import torch
  got, want = got.double().cpu().reshape(want.shape), want.double().cpu()
  err, bound = (got - want).abs(), attention_bound(want, rounded_want)
  ok = bool(torch.isfinite(got).all() and torch.all(err <= bound))
  if not ok and err.numel():
    worst = int(torch.argmax(torch.nan_to_num(err - bound, nan=float("inf"))))
    print(f"attention_close: |got - want| = {float(err.flatten()[worst]):.5g} at want = {float(want.flatten()[worst]):.5g} "
          f"(bound {float(bound.flatten()[worst]):.5g}); {int((err > bound).sum())} of {err.numel()} outside", flush=True)
  return ok


def pytest_sessionfinish(session, exitstatus):
  if not PARITY_ERRORS:
    return
  out = os.path.join(ROOT, "gpurun_out")
  try:
    os.makedirs(out, exist_ok=True)
    with open(os.path.join(out, "parity_max_abs.json"), "w") as f:
      json.dump({k: {"max_abs_err": v[0], "max_abs_expected": v[1]} for k, v in sorted(PARITY_ERRORS.items())},
                f, indent=1)
  except OSError:
    pass


@pytest.fixture(autouse=True)
def no_attention_launch_gave_up(request):
  """After every GPU test: no streaming-kernel launch may have given up on one
  of its bounded waits (the status word of every workspace still alive is read
  and cleared; check_status raises if one did)."""
  yield
  if request.node.get_closest_marker("gpu") is None:
    return
  ak = sys.modules.get("jetstream_pt_amd.attention_kernel")
  if ak is not None:
    ak.check_status()
