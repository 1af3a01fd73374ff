"""GPU parity: the prefill -> decode insert through the C ABI against the CPU
oracle (engine.py:371-626 restated) on the same seeded inputs.  Cache bytes,
codes, scales and bookkeeping are compared bit for bit."""

import pytest
import torch

from oracle import Env as OEnv
from oracle import insert as oins
from oracle import quant as oquant

pytestmark = pytest.mark.gpu
DEV = "cuda"


def make_state(stacked, batch, heads, seq, dim, layers, quantized, scale_dtype=torch.bfloat16, seed=0):
  g = torch.Generator().manual_seed(seed)
  def cache():
    if quantized:
      return torch.randint(-127, 128, (batch, heads, seq, dim), generator=g, dtype=torch.int8)
    return torch.randn((batch, heads, seq, dim), generator=g).to(torch.bfloat16)
  def scale():
    return torch.rand((batch, 1, seq, 1), generator=g).to(scale_dtype)
  if stacked:
    caches = [(torch.stack([cache() for _ in range(layers)]), torch.stack([cache() for _ in range(layers)]))]
    scales = [(torch.stack([scale() for _ in range(layers)]), torch.stack([scale() for _ in range(layers)]))]
  else:
    caches = [(cache(), cache()) for _ in range(layers)]
    scales = [(scale(), scale()) for _ in range(layers)]
  return dict(caches=caches, cache_scales=scales if quantized else None,
              mask=torch.zeros((batch, seq)), start=torch.zeros(batch, dtype=torch.int32),
              input_pos=torch.zeros(batch, dtype=torch.int32), lens=torch.zeros(batch, dtype=torch.int32))


def to_dev(state):
  mv = lambda pairs: None if pairs is None else [(k.to(DEV), v.to(DEV)) for k, v in pairs]
  return dict(caches=mv(state["caches"]), cache_scales=mv(state["cache_scales"]),
              mask=state["mask"].to(DEV), start=state["start"].to(DEV),
              input_pos=state["input_pos"].to(DEV), lens=state["lens"].to(DEV))


def assert_same(dev_state, cpu_state):
  for name in ("caches", "cache_scales"):
    if cpu_state[name] is None:
      continue
    for (dk, dv), (ck, cv) in zip(dev_state[name], cpu_state[name]):
      assert torch.equal(dk.cpu(), ck), name
      assert torch.equal(dv.cpu(), cv), name
  for name in ("mask", "start", "input_pos", "lens"):
    assert torch.equal(dev_state[name].cpu(), cpu_state[name]), name


def run_both(ring, quantized, shape, prompt, seq_len, slot, current_position=0, scale_dtype=torch.bfloat16,
             prefix_dtype=torch.bfloat16):
  from jetstream_pt_amd import insert as gins
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData
  batch, heads, seq, dim, layers = shape
  oenv = OEnv(batch_size=batch, num_layers=layers, cache_len=seq, ring_buffer=ring)
  genv = JetEngineEnvironment(JetEngineEnvironmentData(
      batch_size=batch, num_layers=layers, cache_sequence_length=seq, ring_buffer=ring))
  cpu = make_state(oenv.generate_cache_stacked, batch, heads, seq, dim, layers, quantized, scale_dtype)
  dev = to_dev(cpu)
  g = torch.Generator().manual_seed(11)
  mag = torch.logspace(-2, 1.5, prompt).reshape(1, 1, prompt, 1)
  prefix = [((torch.randn((1, heads, prompt, dim), generator=g) * mag).to(prefix_dtype),
             (torch.randn((1, heads, prompt, dim), generator=g) * mag).to(prefix_dtype)) for _ in range(layers)]
  # the HIP quantiser works in the scalers' dtype (the prompt's dtype unless float32 scalers are used)
  compute = torch.float32 if (quantized and scale_dtype == torch.float32) else None
  oins.insert(oenv, prefix, seq_len, cpu, slot, current_position, compute_dtype=compute)
  gins.insert(genv, [(k.to(DEV), v.to(DEV)) for k, v in prefix], seq_len, dev["caches"], dev["cache_scales"], slot,
              current_position=current_position, mask=dev["mask"], start=dev["start"],
              input_pos=dev["input_pos"], lens=dev["lens"])
  torch.cuda.synchronize()
  assert_same(dev, cpu)


@pytest.mark.parametrize("quantized", [False, True])
def test_left_aligned_stacked_insert(quantized):
  run_both(False, quantized, (3, 2, 32, 8, 2), prompt=16, seq_len=11, slot=2)


@pytest.mark.parametrize("quantized", [False, True])
@pytest.mark.parametrize("current_position,seq_len,prompt", [(24, 10, 16), (3, 6, 8), (16, 8, 8), (31, 20, 24)])
def test_ring_insert_wrap_and_no_wrap(quantized, current_position, seq_len, prompt):
  run_both(True, quantized, (2, 2, 32, 8, 2), prompt=prompt, seq_len=seq_len, slot=1,
           current_position=current_position)


def test_llama3_shaped_quantised_insert_fp32_scales():
  # 8 KV heads x 128, prompt padded to 1024, float32 scalers (the kernel's vector path)
  run_both(False, True, (4, 8, 2048, 128, 2), prompt=1024, seq_len=1000, slot=3, scale_dtype=torch.float32)


@pytest.mark.parametrize("ring,current_position,seq_len,prompt", [(False, 0, 37, 40), (True, 250, 61, 64), (True, 3, 5, 8)])
def test_llama3_shaped_quantised_insert_bf16_scales_ragged_counts(ring, current_position, seq_len, prompt):
  # token counts that are not multiples of the four tokens a workgroup takes, ring wrap included
  run_both(ring, True, (3, 8, 256, 128, 2), prompt=prompt, seq_len=seq_len, slot=1, current_position=current_position)


def test_float32_prefix_into_float32_quantiser():
  run_both(False, True, (2, 4, 64, 16, 1), prompt=32, seq_len=30, slot=0, scale_dtype=torch.float32,
           prefix_dtype=torch.float32)


@pytest.mark.parametrize("tokens", [1, 64, 100, 130])
def test_int8_paged_insert_equals_quantise_then_page_layout(tokens):
  from jetstream_pt_amd import insert as gins
  heads, total, ps, dim, layers = 4, 24, 64, 32, 2
  n_pages = (tokens + ps - 1) // ps
  g = torch.Generator().manual_seed(tokens)
  page_ids = torch.randperm(total, generator=g)[:n_pages].to(torch.int32)
  pools = [(torch.randint(-127, 128, (heads, total, ps, dim), generator=g, dtype=torch.int8),
            torch.randint(-127, 128, (heads, total, ps, dim), generator=g, dtype=torch.int8)) for _ in range(layers)]
  scale_pages = [(torch.rand((1, total, ps), generator=g), torch.rand((1, total, ps), generator=g)) for _ in range(layers)]
  prefix = [((torch.randn((1, heads, tokens, dim), generator=g) * 2).to(torch.bfloat16),
             torch.randn((1, heads, tokens, dim), generator=g).to(torch.bfloat16)) for _ in range(layers)]
  dpools = [(k.to(DEV), v.to(DEV)) for k, v in pools]
  dscales = [(k.to(DEV), v.to(DEV)) for k, v in scale_pages]
  gins.insert_prefix_pages_int8([(k.to(DEV), v.to(DEV)) for k, v in prefix], dpools, dscales, page_ids)
  torch.cuda.synchronize()
  for layer in range(layers):
    for which in (0, 1):
      codes, scales = oquant.quantize_insert(prefix[layer][which].float())  # float32 scales: quantiser in float32
      want = pools[layer][which].clone()
      want_s = scale_pages[layer][which].clone()
      padded = torch.zeros((heads, n_pages * ps, dim), dtype=torch.int8)
      padded[:, :tokens, :] = codes[0]
      want[:, page_ids.long(), :, :] = padded.reshape(heads, n_pages, ps, dim)
      flat = want_s[0, page_ids.long(), :].reshape(-1)
      flat[:tokens] = scales.reshape(-1)
      want_s[0, page_ids.long(), :] = flat.reshape(n_pages, ps)
      assert torch.equal(dpools[layer][which].cpu(), want)
      assert torch.equal(dscales[layer][which].cpu(), want_s)


def test_int8_paged_insert_all_layers_in_one_launch():
  from jetstream_pt_amd import insert as gins
  layers, heads, total, ps, dim, tokens = 3, 8, 16, 64, 128, 150
  g = torch.Generator().manual_seed(5)
  page_ids = torch.tensor([9, 2, 14], dtype=torch.int32)
  pk = torch.randint(-127, 128, (layers, heads, total, ps, dim), generator=g, dtype=torch.int8)
  pv = torch.randint(-127, 128, (layers, heads, total, ps, dim), generator=g, dtype=torch.int8)
  sk, sv = torch.rand((layers, 1, total, ps), generator=g), torch.rand((layers, 1, total, ps), generator=g)
  nk = torch.randn((layers, heads, tokens, dim), generator=g).to(torch.bfloat16)
  nv = torch.randn((layers, heads, tokens, dim), generator=g).to(torch.bfloat16)
  one = [(pk.to(DEV), pv.to(DEV)), (sk.to(DEV), sv.to(DEV))]
  per = [[(pk[l].to(DEV), pv[l].to(DEV)) for l in range(layers)], [(sk[l].to(DEV), sv[l].to(DEV)) for l in range(layers)]]
  # the prompt is the head of a longer buffer: strided rows, no copy
  longk = torch.cat([nk, torch.ones((layers, heads, 40, dim), dtype=nk.dtype)], dim=2).to(DEV)
  longv = torch.cat([nv, torch.ones((layers, heads, 40, dim), dtype=nv.dtype)], dim=2).to(DEV)
  gins.insert_prefix_pages_int8_stacked(longk[:, :, :tokens], longv[:, :, :tokens], one[0][0], one[0][1],
                                        one[1][0], one[1][1], page_ids)
  gins.insert_prefix_pages_int8([(nk[l:l + 1].to(DEV), nv[l:l + 1].to(DEV)) for l in range(layers)], per[0], per[1], page_ids)
  torch.cuda.synchronize()
  for l in range(layers):
    assert torch.equal(one[0][0][l], per[0][l][0]) and torch.equal(one[0][1][l], per[0][l][1])
    assert torch.equal(one[1][0][l], per[1][l][0]) and torch.equal(one[1][1][l], per[1][l][1])
  assert not torch.equal(one[0][0].cpu(), pk)


@pytest.mark.parametrize("block", range(3))
def test_random_dense_inserts(block):
  """Randomly drawn insert shapes - stacked and per-layer caches, ring wrap,
  copy and both quantiser kernels (heads * dim == 1024 takes the wide one),
  one to five layers in one launch - bit for bit against the oracle."""
  import numpy as np
  for it in range(10):
    seed = 500 + 100 * block + it
    rng = np.random.default_rng(seed)
    heads, dim = [(8, 128), (4, 256), (16, 64), (2, 8), (3, 16), (32, 32), (1, 128)][rng.integers(7)]
    seq = int(rng.choice([32, 64, 256, 1024]))
    batch, layers = int(rng.integers(1, 5)), int(rng.integers(1, 6))
    ring = bool(rng.integers(2))
    quantized = bool(rng.integers(2))
    prompt = int(rng.choice([p for p in (8, 16, 24, 40, 64, 128) if p <= seq]))
    seq_len = int(rng.integers(1, prompt + 1))
    slot = int(rng.integers(batch))
    current_position = int(rng.integers(seq)) if ring else 0
    scale_dtype = torch.float32 if (quantized and rng.integers(2)) else torch.bfloat16
    print(f"seed {seed} ring {ring} quantized {quantized} batch {batch} heads {heads} seq {seq} dim {dim} "
          f"layers {layers} prompt {prompt} seq_len {seq_len} slot {slot} pos {current_position} {scale_dtype}", flush=True)
    run_both(ring, quantized, (batch, heads, seq, dim, layers), prompt=prompt, seq_len=seq_len, slot=slot,
             current_position=current_position, scale_dtype=scale_dtype)


@pytest.mark.parametrize("heads,dim", [(8, 128), (2, 8)])
def test_int8_paged_insert_of_several_prompts_in_one_launch(heads, dim):
  """Prompts of different lengths into one stacked pool with one call: the
  pool must equal prompt-by-prompt inserts bit for bit.  (8, 128) takes the
  one-launch kernel, (2, 8) the library's prompt-by-prompt route."""
  import numpy as np
  from jetstream_pt_amd import insert as gins
  layers, total, ps = 3, 40, 32
  g = torch.Generator().manual_seed(9)
  rng = np.random.default_rng(9)
  pk = torch.randint(-127, 128, (layers, heads, total, ps, dim), generator=g, dtype=torch.int8)
  pv = torch.randint(-127, 128, (layers, heads, total, ps, dim), generator=g, dtype=torch.int8)
  sk, sv = torch.rand((layers, 1, total, ps), generator=g), torch.rand((layers, 1, total, ps), generator=g)
  lens = [1, 33, 64, 100, 7, 160]
  perm = rng.permutation(total).astype(np.int32)
  buf_k = torch.randn((layers, heads, 200, dim), generator=g).to(torch.bfloat16).to(DEV)  # one long buffer, prompts are its heads
  buf_v = torch.randn((layers, heads, 200, dim), generator=g).to(torch.bfloat16).to(DEV)
  prefixes, ids, at = [], [], 0
  for n in lens:
    need = -(-n // ps)
    ids.append(torch.from_numpy(perm[at:at + need].copy()).to(DEV))
    at += need
    prefixes.append((buf_k[:, :, :n], buf_v[:, :, :n]))
  many = [t.to(DEV) for t in (pk, pv, sk, sv)]
  one = [t.to(DEV) for t in (pk, pv, sk, sv)]
  gins.insert_prompts_pages_int8_stacked(prefixes, *many, ids)
  for (k, v), i in zip(prefixes, ids):
    gins.insert_prefix_pages_int8_stacked(k, v, *one, i)
  torch.cuda.synchronize()
  for a, b in zip(many, one):
    assert torch.equal(a, b)
  assert not torch.equal(many[0].cpu(), pk)
