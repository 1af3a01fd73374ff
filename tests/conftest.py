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
# largest magnitude of the expected values beside it; written under gpurun_out/
# at the end of a GPU session (the figures DESIGN.md quotes come from there).
PARITY_ERRORS = {}


def record_parity(name, got, want):
  """Returns the element-wise |got - want| (float64 CPU tensors in, or
  anything .double() takes) and remembers its maximum under `name`."""
  err = (got - want).abs()
  if err.numel():
    prev = PARITY_ERRORS.get(name, (0.0, 0.0))
    PARITY_ERRORS[name] = (max(prev[0], float(err.max())), max(prev[1], float(want.abs().max())))
  return err


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
