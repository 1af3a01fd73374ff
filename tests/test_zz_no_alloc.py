"""The allocation-free entry point, jpt_attn_ragged_static, through the C ABI:
same outputs as jpt_attn_ragged (bit for bit: the same kernels on the same
plan), on two calls in a row, the second with a smaller input; nothing is
allocated by the call.  Collected last: it shares one device array with every
other user of that entry point in the process."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(g, b, hq, hkv, s, lens):
  d = 128
  q = torch.randn((b, hq, 1, d), generator=g).to(torch.bfloat16).to(DEV)
  k = torch.randint(-127, 128, (b, hkv, s, d), generator=g, dtype=torch.int8).to(DEV)
  v = torch.randint(-127, 128, (b, hkv, s, d), generator=g, dtype=torch.int8).to(DEV)
  ks = (torch.rand((b, 1, s), generator=g) * 0.045 + 0.005).to(DEV)
  vs = (torch.rand((b, 1, s), generator=g) * 0.045 + 0.005).to(DEV)
  xk = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16).to(DEV)
  xv = torch.randn((b, hkv, 1, d), generator=g).to(torch.bfloat16).to(DEV)
  end = torch.tensor(lens, dtype=torch.int32, device=DEV)
  return q, k, v, ks, vs, xk, xv, end


def _outputs(case):
  q, k = case[0], case[1]
  b, hq, _, d = q.shape
  hkv = k.shape[1]
  out = torch.empty_like(q)
  omax = torch.empty((b, hq, 1), dtype=torch.float32, device=DEV)
  oden = torch.empty_like(omax)
  nk = torch.empty((b, hkv, 1, d), dtype=torch.int8, device=DEV)
  nv = torch.empty_like(nk)
  nks = torch.empty((b, 1), dtype=torch.float32, device=DEV)
  nvs = torch.empty_like(nks)
  return out, omax, oden, nk, nv, nks, nvs


def _run(fn, case, workspace, outputs=None):
  """One launch that quantises and attends the step's token too (every kind of
  scratch use: plan, partials of split slots, status word).  Returns every
  tensor the launch writes (`outputs`, or new ones)."""
  from jetstream_pt_amd import _ffi
  q, k, v, ks, vs, xk, xv, end = case
  b, hq, _, d = q.shape
  hkv, s = k.shape[1], k.shape[2]
  out, omax, oden, nk, nv, nks, nvs = outputs if outputs is not None else _outputs(case)
  a = _ffi.AttnArgs(
      q=_ffi.ptr(q), k=_ffi.ptr(k), v=_ffi.ptr(v), k_scale=_ffi.ptr(ks), v_scale=_ffi.ptr(vs),
      lengths=_ffi.ptr(end), new_k=_ffi.ptr(nk), new_v=_ffi.ptr(nv), new_k_scale=_ffi.ptr(nks),
      new_v_scale=_ffi.ptr(nvs), new_k_raw=_ffi.ptr(xk), new_v_raw=_ffi.ptr(xv), out=_ffi.ptr(out),
      out_max=_ffi.ptr(omax), out_denom=_ffi.ptr(oden), batch=b, q_heads=hq, kv_heads=hkv, q_rows=1, dim=d,
      seq=s, q_dtype=_ffi.BF16, kv_dtype=_ffi.I8, scale_dtype=_ffi.F32, scale_heads=1,
      sm_scale=1.0 / d ** 0.5, new_rounding=_ffi.ROUND_TRUNC)
  if workspace is not None:
    a.workspace, a.workspace_bytes = _ffi.ptr(workspace), workspace.numel()
  _ffi.check(fn(a, _ffi.stream()))
  return out, omax, oden, nk, nv, nks, nvs


def test_static_scratch_entry_point_matches_and_allocates_nothing():
  from jetstream_pt_amd import _ffi
  g = torch.Generator().manual_seed(900)
  # first a batch with slots long enough to be split into several chunks (partials in the
  # scratch), then a smaller one with other lengths: the array still holds the first call's
  # plan and partials when the second starts
  cases = [_case(g, 24, 32, 8, 4096, [4096, 3000, 1, 0, 17, 2049] * 4),
           _case(g, 5, 8, 2, 512, [512, 33, 0, 100, 7])]
  for case in cases:
    q, k = case[0], case[1]
    sizes = _ffi.AttnArgs(batch=q.shape[0], q_heads=q.shape[1], kv_heads=k.shape[1], q_rows=1, seq=k.shape[2])
    nbytes = _ffi.lib.jpt_attn_workspace_bytes(sizes)
    assert nbytes <= _ffi.ATTN_STATIC_SCRATCH_BYTES
    ws = torch.zeros(nbytes, dtype=torch.uint8, device=DEV)
    want = _run(_ffi.lib.jpt_attn_ragged, case, ws)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    # the outputs below are torch's; the call itself must not add to them
    got = _run(_ffi.lib.jpt_attn_ragged_static, case, None)
    torch.cuda.synchronize()
    outputs = sum(t.numel() * t.element_size() for t in got)
    assert torch.cuda.max_memory_allocated() - before <= outputs + 8 * 512  # torch rounds each tensor up
    for name, x, y in zip("out max denom new_k new_v new_k_scale new_v_scale".split(), got, want):
      assert torch.equal(x, y), name
    # torch's counters above see torch's allocator only.  The device's own: with the outputs
    # allocated beforehand, a call (not the process's first, which loads what the runtime loads
    # once) leaves the device's free memory exactly where it was.
    outputs = _outputs(case)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    again = _run(_ffi.lib.jpt_attn_ragged_static, case, None, outputs)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed during the call"
    for name, x, y in zip("out max denom new_k new_v new_k_scale new_v_scale".split(), again, want):
      assert torch.equal(x, y), name
    word = ctypes.c_int32(-1)
    _ffi.check(_ffi.lib.jpt_attn_status(None, _ffi.stream(), ctypes.byref(word)))
    assert word.value & 1 == 0  # no wave gave up; bit 2 only says a slot was at capacity


def test_static_scratch_entry_point_refuses_what_does_not_fit():
  from jetstream_pt_amd import _ffi
  a = _ffi.AttnArgs(batch=4096, q_heads=128, kv_heads=8, q_rows=1, seq=1024, dim=128)
  assert _ffi.lib.jpt_attn_workspace_bytes(a) > _ffi.ATTN_STATIC_SCRATCH_BYTES
  with pytest.raises(ValueError, match="workspace of"):
    _ffi.check(_ffi.lib.jpt_attn_ragged_static(a, _ffi.stream()))
