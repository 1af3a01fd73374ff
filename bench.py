"""Benchmark of the decode-time KV-cache hot path on one MI355X.

Headline workload (BASELINE.json configs[2], `--workload c3`, the default):
ragged GQA decode attention for one Llama-3-8B layer - batch 128, 32 q heads /
8 KV heads, head_dim 128, cache length 8192, int8 KV codes with fp32 per-token
scales, per-slot lengths log-normal (median 400, sigma 1) clipped to [16, 8192].

A step is one layer-step of the production left-aligned mode: fused int8
quantise + stash of the new token, then ragged attention over the cache with
the new token merged in the same launch.  Steps rotate over the 32 layers of
a stacked cache (64 GiB of codes), so every step streams cold data; once per
32 steps the per-step split plan is recomputed and finalize() scatters the 32
stashed tokens into the cache (both inside the timed region).

Timing: a pass over the layers (plan, every layer's step, finalize) is
captured once in a HIP graph and replayed at least 50 times, each replay
between its own pair of events on the stream the work runs on; `ms_per_step`
is the MEDIAN replay divided by the layers in it, `min_us_per_layer` the
fastest, `repeats` the number of replays (`steps`/`warmup` echo the command
line: enough whole passes are run to cover them).

Prints one JSON line.  `value` is algorithmic bytes of the layer-step divided
by its time; `roofline` is the attention launch alone (a separate timed loop
of attention launches only); `cpu_baseline` times the CPU oracle's
restatement of the reference path on the host cores.

The other configurations of BASELINE.json are parity-test cases; the default run
times them after the headline, the same way, and adds them to the same JSON line
as `other_workloads` (layer-step and attention launch of each; the headline
fields stay C3's); `--workload c1|c2|c4|c5` times one of them alone (same JSON
shape, no cpu_baseline):
  c1  dense bf16 eager update + dense attention, B=8, 32 heads, S=1024
  c2  int8 MHA decode step, B=96, 32 heads, S=2048, lengths U[128, 2048] (a slot at
      2048 is full: it is attended, its new token is attended too but not stored)
  c4  paged bf16, B=256, 64 q / 8 kv heads, 32768 pages of 64, page
      allocation every decode step, paged attention that appends the token
  c5  paged int8, 32 layers, B=256, 32 q / 8 kv heads, 16384 pages of 64 per
      layer; every decode step frees 16 slots and inserts 16 new prompts;
      a slot that has reached max_cache_len (4096) retires before the step
"""

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "jetstream-pytorch_amd")):
  if _p not in sys.path:
    sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0
D = 128
B, HQ, HKV, S, LAYERS = 128, 32, 8, 8192, 32  # the headline workload
SEED = 3
PROBE_COPY_BYTES = 1 << 30
# HBM bytes of one attention launch on the headline workload, from hardware
# counters (FETCH_SIZE + WRITE_SIZE, each calibrated on a 1 GiB copy; see
# --probe-traffic): a recorded measurement, kept in the summary of the counter
# runs under profiles/ and read from there.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "attn_decode_c3_int8_hbm_traffic_pmc.txt")
MIN_REPEATS = 50


def measured_attn_traffic_bytes():
  """The `traffic_bytes_per_launch:` line of the counter summary, or None."""
  try:
    with open(TRAFFIC_SUMMARY) as f:
      for line in f:
        if line.startswith("traffic_bytes_per_launch:"):
          return int(line.split(":")[1].split()[0])
  except (OSError, ValueError):
    pass
  return None
DEV = "cuda:0"


def seeded_lengths(torch, batch=B, median=400.0, lo=16, hi=S, seed=SEED):
  g = torch.Generator().manual_seed(seed)
  z = torch.randn(batch, generator=g, dtype=torch.float64)
  return torch.clamp(torch.round(torch.exp(math.log(median) + z)), lo, hi).to(torch.int32)


def uniform_lengths(torch, batch, lo, hi, seed):
  g = torch.Generator().manual_seed(seed)
  return torch.randint(lo, hi + 1, (batch,), generator=g, dtype=torch.int32)


def dense_attn_bytes(total, batch, hq, hkv, e_kv, scales, new_token, e_scale=4):
  """Algorithmic bytes of one attention launch over `total` attended
  positions: K and V of those positions, their per-token scales (shared by all
  heads), q in and o out (bf16), the lengths, and the new token if fused."""
  kv = total * hkv * D * 2 * e_kv
  sc = total * e_scale * 2 if scales else 0
  qo = batch * hq * D * 2 * 2
  new = (batch * hkv * D * 2 * e_kv + (batch * e_scale * 2 if scales else 0)) if new_token else 0
  return kv + sc + qo + new + batch * 4


def attn_bytes(lengths):
  """The headline workload's attention launch."""
  return dense_attn_bytes(int(lengths.sum()), B, HQ, HKV, 1, True, True)


# ---- workloads -------------------------------------------------------------------
# A builder returns a dict: step(i) and attn_only(i) enqueue layer-step i;
# step_bytes / attn_bytes are algorithmic bytes per layer-step / attention launch;
# graph says whether a pass over the layers may be captured in a HIP graph.


def build_dense_int8(torch, nl, batch, hq, hkv, seq, lengths, name):
  """Left-aligned production mode (lazy update, stacked int8 cache, ragged
  attention with the new token fused): the shape of c2 and c3."""
  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import layers
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData

  env = JetEngineEnvironment(JetEngineEnvironmentData(batch_size=batch, num_layers=nl, ring_buffer=False))
  torch.manual_seed(SEED)  # the cache contents below come from the device's default generator
  cache = cm.Int8KVCacheGenerate.empty((nl, batch, hkv, seq, D), DEV, env, scale_heads=1,
                                       scale_dtype=torch.float32)
  for l in range(nl):  # codes uniform [-127, 127], scales U(0.005, 0.05)
    cache.cache_k[l].random_(-127, 128)
    cache.cache_v[l].random_(-127, 128)
    cache.k_scaler[l].uniform_(0.005, 0.05)
    cache.v_scaler[l].uniform_(0.005, 0.05)
  g = torch.Generator(device=DEV).manual_seed(SEED)
  xq = torch.randn((batch, hq, 1, D), generator=g, device=DEV).to(torch.bfloat16)
  xk = torch.randn((batch, hkv, 1, D), generator=g, device=DEV).to(torch.bfloat16)
  xv = torch.randn((batch, hkv, 1, D), generator=g, device=DEV).to(torch.bfloat16)
  pos = lengths.to(DEV)
  cache.input_pos = pos
  kernels = [layers.Int8KVAttentionKernel(env, l) for l in range(nl)]
  state = {"plan": None}

  def step(i):
    l = i % nl
    if l == 0:
      state["plan"], _ = ak.precompute_ragged_block_indices(pos, batch, hq, hkv, seq)
    plan = state["plan"]
    out = kernels[l](xq, xk, xv, None, cache, start=None, end=plan.lengths, ragged_batch_index=plan)
    if l == nl - 1:
      cache.finalize()
    return out

  plan, _ = ak.precompute_ragged_block_indices(pos, batch, hq, hkv, seq)
  new = dict(new_key=cache.new_ks[0], new_value=cache.new_vs[0],
             new_k_scaler=cache.new_k_scaler[0], new_v_scaler=cache.new_v_scaler[0],
             new_key_raw=xk, new_value_raw=xv)  # the launch quantises the token too, as in step()

  def attn_only(i):
    return ak.ragged_mha(xq, cache.cache_k, cache.cache_v, i % nl, None, plan.lengths, plan, None,
                         cache.k_scaler, cache.v_scaler, **new)

  total = int(lengths.sum())
  append = batch * hkv * D * (2 + 1) * 2 + batch * 4 * 2           # bf16 in, codes + fp32 scales out
  ab = dense_attn_bytes(total, batch, hq, hkv, 1, True, True)
  finalize = (batch * hkv * D + batch * 4) * 2 * 2                # per layer: stash read, cache written
  return dict(step=step, attn_only=attn_only, step_bytes=ab + append + finalize, attn_bytes=ab, graph=True,
              cache=cache, lengths=lengths, xq=xq, xk=xk, xv=xv, env=env,
              config={"workload": name, "batch": batch, "q_heads": hq, "kv_heads": hkv, "head_dim": D,
                      "max_cache_len": seq, "layers_rotated": nl, "cached_tokens": total,
                      "kv": "int8 codes + fp32 per-token scales"},
              kernel="attn_decode_kernel<int8> (one launch: chunks, then the merges of split slots)")


def build_c3(torch, args):
  lengths = seeded_lengths(torch)
  w = build_dense_int8(torch, args.layers or LAYERS, B, HQ, HKV, S, lengths,
                       "C3 ragged GQA int8 decode layer-step: KV quantise+stash, ragged attention with "
                       "fused new token, finalize amortised over the layers")
  w["config"]["lengths"] = "log-normal(median 400, sigma 1) in [16, 8192], seed 3"
  return w


def build_c2(torch, args):
  lengths = uniform_lengths(torch, 96, 128, 2048, seed=2)
  if getattr(args, "full_slot", False):  # parity tests: the edge of the range, whatever the draw holds
    lengths[0] = 2048
  w = build_dense_int8(torch, args.layers or 32, 96, 32, 32, 2048, lengths,
                       "C2 int8 MHA decode layer-step: KV quantise+stash, ragged attention with fused new "
                       "token, finalize amortised over the layers")
  w["config"]["lengths"] = "uniform [128, 2048], seed 2"
  return w


def build_c1(torch, args):
  """Dense bf16 eager per-slot update + dense attention over the whole cache
  with an additive mask."""
  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import layers
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData

  nl, batch, heads, seq = args.layers or 32, 8, 32, 1024
  env = JetEngineEnvironment(JetEngineEnvironmentData(
      batch_size=batch, num_layers=nl, cache_sequence_length=seq, testing=True, ring_buffer=False,
      lazy_cache_update=False, ragged_mha=False, flash_attention=False, generate_cache_stacked=False,
      new_cache_stacked=False))
  g = torch.Generator().manual_seed(1)
  pos = torch.randint(0, seq, (batch,), generator=g, dtype=torch.int32)
  gd = torch.Generator(device=DEV).manual_seed(1)
  caches = []
  x = torch.arange(seq).reshape(1, 1, seq, 1)
  live = (x < pos.reshape(batch, 1, 1, 1)).to(DEV)
  for _ in range(nl):
    k = torch.randn((batch, heads, seq, D), generator=gd, device=DEV).to(torch.bfloat16) * live
    v = torch.randn((batch, heads, seq, D), generator=gd, device=DEV).to(torch.bfloat16) * live
    caches.append(cm.KVCacheGenerate(k, v, pos.to(DEV), None, env=env))
  xq = torch.randn((batch, heads, 1, D), generator=gd, device=DEV).to(torch.bfloat16)
  xk = torch.randn((batch, heads, 1, D), generator=gd, device=DEV).to(torch.bfloat16)
  xv = torch.randn((batch, heads, 1, D), generator=gd, device=DEV).to(torch.bfloat16)
  mask = torch.where(torch.arange(seq).reshape(1, 1, 1, seq) <= pos.reshape(batch, 1, 1, 1), 0.0,
                     float("-inf")).to(DEV)
  kernels = [layers.AttentionKernel(env, l) for l in range(nl)]

  def step(i):
    l = i % nl
    return kernels[l](xq, xk, xv, mask, caches[l])

  def attn_only(i):
    c = caches[i % nl]
    return ak.dense_attention(xq, c.cache_k, c.cache_v, mask=mask)

  ab = batch * heads * seq * D * 2 * 2 + batch * seq * 4 + batch * heads * D * 2 * 2
  append = batch * heads * D * 2 * 2 * 2
  return dict(step=step, attn_only=attn_only, step_bytes=ab + append, attn_bytes=ab, graph=True,
              caches=caches, pos=pos, mask=mask, xq=xq, xk=xk, xv=xv, env=env,
              config={"workload": "C1 dense bf16 eager layer-step: per-slot KV line write, dense attention over "
                                  "all 1024 positions with an additive mask",
                      "batch": batch, "q_heads": heads, "kv_heads": heads, "head_dim": D,
                      "max_cache_len": seq, "layers_rotated": nl, "kv": "bf16"},
              kernel="attn_decode_kernel<bf16, mask> (one launch: chunks, then the merges of split slots)")


def build_paged(torch, args, int8):
  """c4 (bf16 pages) / c5 (int8 pages, prompt churn): page allocation once per
  decode step, then per layer a paged append and a paged attention (one launch
  with the device allocator: the attention launch appends the token).  By default
  the allocator, its tables and the per-slot lengths live on the device and a
  decode step is replayed from one HIP graph (allocation, token indices, all
  layers, position advance); prompt churn is enqueued between replays.
  args.host_alloc keeps the allocator on the host as the reference does
  (lengths pulled every step, tables uploaded), which cannot be captured."""
  import numpy as np

  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import decode_state
  from jetstream_pt_amd import insert as gins
  from jetstream_pt_amd import layers
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData
  from jetstream_pt_amd.page_attention_manager import DevicePageAttentionManager, PageAttentionManager

  host_alloc = bool(getattr(args, "host_alloc", False))
  log_on = bool(getattr(args, "log", host_alloc))  # index arrays kept for the parity tests
  if int8:
    nl, batch, hq, hkv, ps, total, max_pages, seed = args.layers or 32, 256, 32, 8, 64, 16384, 64, 5
    lengths = seeded_lengths(torch, batch, 600.0, 16, 4096, seed).numpy().astype(np.int32)
  else:
    nl, batch, hq, hkv, ps, total, max_pages, seed = args.layers or 4, 256, 64, 8, 64, 32768, 128, 4
    lengths = uniform_lengths(torch, batch, 32, 2048, seed).numpy().astype(np.int32)
  env = JetEngineEnvironment(JetEngineEnvironmentData(
      batch_size=batch, num_layers=nl, paged_attention_total_num_pages=total, paged_attention_page_size=ps))
  rng = np.random.default_rng(seed)
  torch.manual_seed(seed)  # pool contents come from the device's default generator
  order = rng.permutation(total).astype(np.int32)
  if host_alloc:
    pam = PageAttentionManager(batch, total, ps, max_pages, free_list_order=order)
    for slot in range(batch):
      pam.reserve_pages_insert(slot, int(lengths[slot]))
  else:
    pam = DevicePageAttentionManager(batch, total, ps, max_pages, device=DEV, free_list_order=order)
    pam.reserve_pages_insert_many(np.arange(batch, dtype=np.int32), lengths)
  dlens = torch.from_numpy(lengths.copy()).to(DEV)  # the engine's per-slot lengths, device copy
  e_kv = 1 if int8 else 2
  kdt = torch.int8 if int8 else torch.bfloat16
  pools_k = torch.empty((nl, hkv, total, ps, D), dtype=kdt, device=DEV)
  pools_v = torch.empty_like(pools_k)
  for l in range(nl):
    if int8:
      pools_k[l].random_(-127, 128)
      pools_v[l].random_(-127, 128)
    else:
      pools_k[l].normal_()
      pools_v[l].normal_()
  sk = sv = None
  if int8:
    sk = torch.empty((nl, 1, total, ps), device=DEV).uniform_(0.005, 0.05)
    sv = torch.empty((nl, 1, total, ps), device=DEV).uniform_(0.005, 0.05)
  gd = torch.Generator(device=DEV).manual_seed(seed)
  xq = torch.randn((batch, hq, 1, D), generator=gd, device=DEV).to(torch.bfloat16)
  xk = torch.randn((batch, hkv, 1, D), generator=gd, device=DEV).to(torch.bfloat16)
  xv = torch.randn((batch, hkv, 1, D), generator=gd, device=DEV).to(torch.bfloat16)
  prompt_k = prompt_v = None
  if int8:
    caches = [cm.Int8PageKVCacheGenerate(pools_k[l], pools_v[l], sk[l], sv[l], pam, None, env=env) for l in range(nl)]
    kernels = [layers.Int8KVAttentionKernel(env, l) for l in range(nl)]
    # Every prompt of a decode step comes from a buffer of its own (16 x (K + V) x 64 MiB = 2 GiB a
    # step at 32 layers), so that the insert reads HBM: slices of one buffer would sit in the
    # 256 MB memory-side cache from the second prompt on.
    prompt_k = torch.randn((16, nl, hkv, 1024, D), generator=gd, device=DEV).to(torch.bfloat16)
    prompt_v = torch.randn((16, nl, hkv, 1024, D), generator=gd, device=DEV).to(torch.bfloat16)
  else:
    caches = [cm.PageKVCacheGenerate(pools_k[l], pools_v[l], pam, None, env=env) for l in range(nl)]
    kernels = [layers.AttentionKernel(env, l) for l in range(nl)]
  state = {"lens": lengths.copy(), "decode_steps": 0, "attended": 0, "pages": 0, "inserted": 0, "log": [],
           "prompts_used": 0}
  churn = 16 if int8 else 0

  # Requests of a decode step go to the device through pinned staging buffers that exist
  # before the timed loop (allocating pinned memory waits for the device): row 0 the slots to
  # free, row 1 their new lengths (0 for a slot that retires), as int32 for the allocator and as
  # int64 for torch's index_copy_.  A ring of them, each with the event of its last upload, so
  # that the host can run passes ahead of the device.
  ring_n = 64
  stage = stage_dev = None
  if not host_alloc:
    stage = [(torch.empty((2, batch), dtype=torch.int32).pin_memory(), torch.empty((batch,), dtype=torch.int64).pin_memory())
             for _ in range(ring_n)]
    stage_dev = [(torch.empty((2, batch), dtype=torch.int32, device=DEV), torch.empty((batch,), dtype=torch.int64, device=DEV))
                 for _ in range(ring_n)]
  uploaded = [None] * ring_n
  passes_run = [0]

  def upload(slots, new_lens):
    """slots and their new lengths (numpy int32) -> device views (slots, lens, slots as int64)."""
    j = passes_run[0] % ring_n
    passes_run[0] += 1
    if uploaded[j] is not None:
      uploaded[j].synchronize()
    n = len(slots)
    (h32, h64), (d32, d64) = stage[j], stage_dev[j]
    h32[0, :n] = torch.from_numpy(slots)
    h32[1, :n] = torch.from_numpy(new_lens)
    h64[:n] = h32[0, :n]
    d32.copy_(h32, non_blocking=True)
    d64.copy_(h64, non_blocking=True)
    uploaded[j] = torch.cuda.Event()
    uploaded[j].record()
    return d32[0, :n], d32[1, :n], d64[:n]

  def before_pass():
    """What the engine does once per decode step before the layers run: new
    prompts take over some slots, then (host allocator only) pages for the
    step are reserved and the tables uploaded.  Also the byte accounting."""
    lens = state["lens"]
    full = np.nonzero(lens >= max_pages * ps)[0].astype(np.int32)
    # a slot at max_cache_len cannot take another token: its request is over, the slot retires
    if len(full) and host_alloc:
      for slot in full:
        pam.free_pages_resource(int(slot))
    if len(full) and host_alloc:
      state["log"].append(("free_many", full.copy()))
    lens[full] = 0
    slots = ns = np.zeros((0,), dtype=np.int32)
    if churn:
      slots = rng.choice(batch, churn, replace=False).astype(np.int32)
      ns = np.array([int(rng.integers(64, 1025)) for _ in slots], dtype=np.int32)
    if host_alloc:
      for slot, n in zip(slots, ns):
        pam.free_pages_resource(int(slot))
        _, ids = pam.reserve_pages_insert(int(slot), int(n))
        ids = np.array(ids, dtype=np.int32)
        j = state["prompts_used"] % 16
        state["prompts_used"] += 1
        gins.insert_prefix_pages_int8_stacked(prompt_k[j, :, :, :n], prompt_v[j, :, :, :n], pools_k, pools_v, sk, sv, ids)
        state["log"].append(("insert", int(slot), int(n), ids, j))
    elif len(full) or len(slots):
      # one upload, one free (retired slots and the slots the new prompts take over), one
      # reservation, one update of the engine's lengths, and all of the step's prompts in one
      # insert launch; page ids are views of the device table (no copy)
      retire = np.setdiff1d(full, slots).astype(np.int32)
      dfree, dnew, dfree64 = upload(np.concatenate([retire, slots]), np.concatenate([np.zeros_like(retire), ns]))
      pam.free_pages_resource_many(dfree)
      if len(slots):
        pam.reserve_pages_insert_many(dfree[len(retire):], dnew[len(retire):])
      dlens.index_copy_(0, dfree64, dnew)
      if len(slots):
        gins.insert_prompts_pages_int8_stacked(
            [(prompt_k[j, :, :, :n], prompt_v[j, :, :, :n]) for j, n in enumerate(ns)], pools_k, pools_v, sk, sv,
            [pam.page_indices[int(slot), : (int(n) + ps - 1) // ps] for slot, n in zip(slots, ns)])
      if log_on:
        state["log"].append(("free_many", np.concatenate([retire, slots])))
      if log_on and len(slots):
        state["log"].append(("insert_many", slots.copy(), ns.copy(),
                             [pam.page_indices[int(s), : (int(n) + ps - 1) // ps].cpu().numpy() for s, n in zip(slots, ns)],
                             list(range(len(ns)))))
    if len(slots):
      lens[slots] = ns
      state["inserted"] += int(ns.sum())
    if host_alloc:
      pam.fill_new_pages(lens)
      idx_host = pam.get_page_token_indices(lens)
      idx = torch.from_numpy(idx_host).to(DEV)
      state["log"].append(("decode", lens.copy(), idx_host))
      for c in caches:
        c.page_token_indices = idx
    elif log_on:
      state["log"].append(("decode", lens.copy(), None))
    lens += (lens > 0)
    state["decode_steps"] += 1
    state["attended"] += int(lens.sum())
    state["pages"] += int(((lens + ps - 1) // ps).sum())

  def step(i):
    l = i % nl
    if l == 0 and not host_alloc:  # allocation and token indices for the step, on the device
      idx = pam.decode_step(dlens)
      for c in caches:
        c.page_token_indices = idx
      if log_on:  # parity tests only: pulls the index array to the host
        kind, lens_before, _ = state["log"][-1]
        state["log"][-1] = (kind, lens_before, idx.to_host())
    out = kernels[l](xq, xk, xv, None, caches[l])
    if l == nl - 1 and not host_alloc:
      decode_state.advance(dlens)
    return out

  def attn_only(i):
    l = i % nl
    lens_d, table = pam.device_tables(DEV)
    plan = ak.paged_decode_plan(pam, lens_d, batch, hq, hkv, ps, max_pages)  # once per table change, as in step()
    return ak.call_paged_attention(env, xq.squeeze(2), pools_k[l], pools_v[l], lens_d, table,
                                   k_scaler=sk[l] if int8 else None, v_scaler=sv[l] if int8 else None, plan=plan)

  def bytes_now():
    """Average algorithmic bytes per layer-step / attention launch over the
    decode steps run so far (lengths grow by one per step)."""
    n = max(state["decode_steps"], 1)
    att, pages = state["attended"] / n, state["pages"] / n
    ab = att * hkv * D * 2 * e_kv + (att * 4 * 2 if int8 else 0) + batch * hq * D * 2 * 2 + pages * 4 + batch * 4
    append = batch * hkv * D * (2 * 2 + 2 * e_kv) + (batch * 4 * 2 if int8 else 0)
    ins = state["inserted"] / n * (hkv * D * 2 * (2 + 1) + 4 * 2) if int8 else 0   # per layer
    return ab + append + ins, ab

  where = "host page allocation (lengths pulled, tables uploaded)" if host_alloc else \
      "page allocation, token indices and position advance on the device"
  per_layer = "paged append + paged attention" if host_alloc else "one paged attention launch that also appends the token"
  name = ("C5 paged int8 layer-step: per decode step 16 slots freed and 16 prompts quantised into pages (all "
          f"layers), {where}; per layer {'quantised ' if host_alloc else ''}{per_layer}" if int8 else
          f"C4 paged bf16 layer-step: {where} once per decode step; per layer {per_layer}")
  return dict(step=step, before_pass=before_pass, attn_only=attn_only, bytes_now=bytes_now, graph=not host_alloc,
              pam=pam, pools=(pools_k, pools_v), dlens=dlens,
              scale_pages=(sk, sv), caches=caches, state=state, xq=xq, xk=xk, xv=xv, env=env,
              prompts=(prompt_k, prompt_v), initial_lengths=lengths,
              config={"workload": name, "batch": batch, "q_heads": hq, "kv_heads": hkv, "head_dim": D,
                      "page_size": ps, "total_pages": total, "max_pages_per_seq": max_pages, "layers_rotated": nl,
                      "kv": "int8 pages + fp32 scale pages" if int8 else "bf16 pages"},
              kernel=("attn_decode_kernel<int8, paged>" if int8 else "attn_decode_kernel<bf16, paged>") +
                     " (one launch: chunks, then the merges of split slots)")


def build_c4(torch, args):
  return build_paged(torch, args, False)


def build_c5(torch, args):
  return build_paged(torch, args, True)


WORKLOADS = {"c1": build_c1, "c2": build_c2, "c3": build_c3, "c4": build_c4, "c5": build_c5}


def run_gpu(args):
  import torch

  torch.cuda.set_device(0)
  w = WORKLOADS[args.workload](torch, args)
  nl = w["config"]["layers_rotated"]
  use_graph = w["graph"] and not args.no_graph

  def timed(fn, steps, warmup, before=None):
    """fn(i) enqueues step i.  A whole pass over the layers is replayed from one
    captured HIP graph where the workload allows (what a serving loop does with
    a launch-bound decode step), otherwise launched from Python.  before(),
    when given, is the eager per-pass work ahead of layer 0 (it is inside the
    timed region).  Every pass is timed by its own pair of events; returns
    (median, min, mean over the whole region) in ms per step and the passes."""
    before = before or (lambda: None)
    warmup = (max(warmup, nl) + nl - 1) // nl * nl  # whole passes
    for i in range(warmup):
      if i % nl == 0:
        before()
      fn(i)
    torch.cuda.synchronize()
    graph = None
    if use_graph:
      graph = torch.cuda.CUDAGraph()
      with torch.cuda.graph(graph):
        for i in range(nl):
          fn(i)
      before()
      graph.replay()
      torch.cuda.synchronize()
    passes = max((steps + nl - 1) // nl, MIN_REPEATS)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(passes + 1)]
    marks[0].record()
    for r in range(passes):
      before()
      if graph is not None:
        graph.replay()
      else:
        for i in range(nl):
          fn(i)
      marks[r + 1].record()
    torch.cuda.synchronize()
    each = sorted(marks[r].elapsed_time(marks[r + 1]) / nl for r in range(passes))
    whole = marks[0].elapsed_time(marks[passes]) / (passes * nl)
    return each[len(each) // 2], each[0], whole, passes

  ms_per_step, ms_min, ms_mean, passes = timed(w["step"], args.steps, args.warmup, w.get("before_pass"))
  if "bytes_now" in w:
    w["step_bytes"], w["attn_bytes"] = w["bytes_now"]()
  attn_ms, attn_min, _, _ = timed(w["attn_only"], args.steps, args.warmup)
  w.update(ms_per_step=ms_per_step, ms_min=ms_min, ms_mean=ms_mean, repeats=passes, attn_ms=attn_ms,
           attn_min=attn_min, launch="hip graph of one pass over the layers" if use_graph else "python")
  return w


def run_traffic_probe(args):
  """Work for a hardware-counter run (rocprofv3 --pmc FETCH_SIZE or WRITE_SIZE):
  a few attention launches of the headline workload next to plain copies of a
  buffer of known size, whose counter reading calibrates the counter's unit."""
  import torch

  from jetstream_pt_amd import attention_kernel as ak

  torch.cuda.set_device(0)
  if args.workload != "c3":
    # the workload's own attention launch (c4: bf16 pages), eight times, each next to a calibration copy
    w = WORKLOADS[args.workload](torch, args)
    if "before_pass" in w:
      w["before_pass"]()
    w["step"](0)  # the step's page allocation and plan
    src = torch.empty(PROBE_COPY_BYTES // 4, dtype=torch.float32, device=DEV).normal_()
    dst = torch.empty_like(src)
    for i in range(8):
      w["attn_only"](i)
      dst.copy_(src)
    torch.cuda.synchronize()
    launch_bytes = w["bytes_now"]()[1] if "bytes_now" in w else w["attn_bytes"]
    print(json.dumps({"probe": "traffic", "workload": args.workload, "attention_launches": 8, "copies": 8,
                      "copy_bytes_read": PROBE_COPY_BYTES, "copy_bytes_written": PROBE_COPY_BYTES,
                      "attn_algorithmic_bytes": int(launch_bytes)}))
    return
  nl = 4
  lengths = seeded_lengths(torch).to(DEV)
  k = torch.empty((nl, B, HKV, S, D), dtype=torch.int8, device=DEV)
  v = torch.empty_like(k)
  for l in range(nl):
    k[l].random_(-127, 128)
    v[l].random_(-127, 128)
  ks = torch.empty((nl, B, 1, S, 1), device=DEV).uniform_(0.005, 0.05)
  vs = torch.empty_like(ks).uniform_(0.005, 0.05)
  g = torch.Generator(device=DEV).manual_seed(SEED)
  xq = torch.randn((B, HQ, 1, D), generator=g, device=DEV).to(torch.bfloat16)
  xk = torch.randn((B, HKV, 1, D), generator=g, device=DEV).to(torch.bfloat16)
  xv = torch.randn((B, HKV, 1, D), generator=g, device=DEV).to(torch.bfloat16)
  nk = torch.empty((B, HKV, 1, D), dtype=torch.int8, device=DEV)  # written by the launch
  nv = torch.empty_like(nk)
  nks = torch.empty((B, 1, 1, 1), device=DEV)
  nvs = torch.empty_like(nks)
  plan, _ = ak.precompute_ragged_block_indices(lengths, B, HQ, HKV, S)
  src = torch.empty(PROBE_COPY_BYTES // 4, dtype=torch.float32, device=DEV).normal_()
  dst = torch.empty_like(src)
  for i in range(8):
    ak.ragged_mha(xq, k, v, i % nl, None, plan.lengths, plan, None, ks, vs, new_key=nk, new_value=nv,
                  new_k_scaler=nks, new_v_scaler=nvs, new_key_raw=xk, new_value_raw=xv)
    dst.copy_(src)
  torch.cuda.synchronize()
  print(json.dumps({"probe": "traffic", "attention_launches": 8, "copies": 8,
                    "copy_bytes_read": PROBE_COPY_BYTES, "copy_bytes_written": PROBE_COPY_BYTES,
                    "attn_algorithmic_bytes": attn_bytes(lengths.cpu())}))


def run_cpu_baseline(budget_s=20.0):
  """The oracle (CPU restatement of the reference path) on one layer of the
  headline workload: Int8KVCacheGenerate.update + ragged_mha + new-token flash
  attention + merge, on the host cores."""
  import torch

  from oracle import Env as OEnv
  from oracle import kv_cache as okv
  from oracle.attn_layers import Int8KVAttentionKernel as OInt8Attn

  cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1))
  torch.set_num_threads(cores)
  lengths = seeded_lengths(torch)
  g = torch.Generator().manual_seed(SEED)
  oenv = OEnv(batch_size=B, num_layers=1, ring_buffer=False)
  shape = (1, B, HKV, S, D)
  cache = okv.Int8KVCacheGenerate.empty(shape, None, oenv, scale_dtype=torch.float32)
  cache.cache_k.random_(-127, 128, generator=g)
  cache.cache_v.random_(-127, 128, generator=g)
  cache.k_scaler.uniform_(0.005, 0.05, generator=g)
  cache.v_scaler.uniform_(0.005, 0.05, generator=g)
  cache.input_pos = lengths
  xq = torch.randn((B, HQ, 1, D), generator=g).to(torch.bfloat16)
  xk = torch.randn((B, HKV, 1, D), generator=g).to(torch.bfloat16)
  xv = torch.randn((B, HKV, 1, D), generator=g).to(torch.bfloat16)
  kern = OInt8Attn(oenv, 0)
  kern(xq, xk, xv, None, cache, start=None, end=lengths)  # warm-up
  times = []
  t_end = time.perf_counter() + budget_s
  while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 50):
    t0 = time.perf_counter()
    kern(xq, xk, xv, None, cache, start=None, end=lengths)
    times.append(time.perf_counter() - t0)
  times.sort()
  med = times[len(times) // 2]
  nbytes = attn_bytes(lengths) + B * HKV * D * (2 + 1) * 2 + B * 4 * 2
  return dict(value=round(nbytes / med / 1e9, 3), unit="GB/s", cores=cores, kind="port",
              sample=f"one full layer-step (all {B} slots, {int(lengths.sum())} cached tokens), "
                     f"median of {len(times)} runs, {med * 1e3:.1f} ms each")


T0 = time.perf_counter()


def progress(what):
  """A line on stderr per phase: a long run must show that it is alive."""
  print(f"[bench {time.perf_counter() - T0:6.1f} s] {what}", file=sys.stderr, flush=True)


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=640)
  ap.add_argument("--warmup", type=int, default=64)
  ap.add_argument("--layers", type=int, default=0, help="cache layers to rotate over (0 = the workload's own)")
  ap.add_argument("--workload", choices=sorted(WORKLOADS), default="c3")
  ap.add_argument("--no-cpu-baseline", action="store_true")
  ap.add_argument("--no-graph", action="store_true", help="launch every step from Python")
  ap.add_argument("--no-other-workloads", action="store_true",
                  help="c3: skip the timing of c1, c2, c4 and c5 that follows the headline")
  ap.add_argument("--first-use-memory", action="store_true",
                  help="time the workload on its first allocation only (no free-and-allocate-again pass)")
  ap.add_argument("--host-alloc", action="store_true",
                  help="c4/c5: page allocator on the host as in the reference (no graph capture)")
  ap.add_argument("--probe-traffic", action="store_true",
                  help="run a few attention launches and calibration copies for a counter run")
  args = ap.parse_args()
  if args.gpus != 1:
    sys.exit("bench.py measures one GPU: the path is built and measured on a single MI355X "
             "(--gpus must be 1)")
  if args.probe_traffic:
    run_traffic_probe(args)
    return
  progress(f"{args.workload}: building and timing")
  r = run_gpu(args)
  first_use = None
  if not args.first_use_memory:
    # HBM handed out for the first time after the device comes up streams more
    # slowly on this pool than memory that has been allocated before (C3: 48.4
    # against 45.1 us per layer-step, the same kernels, the same virtual
    # addresses).  A serving process on a node that has been up for a while
    # sits in the second state: the workload is built once on first-use memory
    # (reported as first_use_memory), freed, and built again for `value`.
    import gc

    import torch
    first_use = {"us_per_layer": round(r["ms_per_step"] * 1e3, 2),
                 "GB_per_s": round(r["step_bytes"] / (r["ms_per_step"] * 1e-3) / 1e9, 1),
                 "attention_us_per_launch": round(r["attn_ms"] * 1e3, 2)}
    del r
    gc.collect()
    torch.cuda.empty_cache()
    progress(f"{args.workload}: built again on memory that has been used before")
    r = run_gpu(args)
  gbps = r["step_bytes"] / (r["ms_per_step"] * 1e-3) / 1e9
  attn_gbps = r["attn_bytes"] / (r["attn_ms"] * 1e-3) / 1e9
  headline = args.workload == "c3"
  cfg = dict(r["config"])
  cfg["launch"] = r["launch"]
  model_layers = cfg["layers_rotated"] if args.workload == "c5" else LAYERS
  line = {
      "metric": "decode-attn HBM GB/s (% of 8 TB/s) + us/layer, Llama-3-8B GQA int8 B=128",
      "value": round(gbps, 1),
      "unit": "GB/s",
      "n_gpus": 1,
      "steps": args.steps,
      "warmup": args.warmup,
      "ms_per_step": round(r["ms_per_step"], 5),
      "higher_is_better": True,
      "scaling": "weak",
      "vs_baseline": None,
      "dtype": "bf16",
      "data": "synthetic",
      "config": cfg,
      "us_per_layer": round(r["ms_per_step"] * 1e3, 2),
      "min_us_per_layer": round(r["ms_min"] * 1e3, 2),
      "mean_us_per_layer": round(r["ms_mean"] * 1e3, 2),
      "repeats": r["repeats"],
      "timing": f"median of {r['repeats']} passes over {cfg['layers_rotated']} layers, each pass between its own events",
      "pct_of_hbm_peak": round(100 * gbps / HBM_PEAK_GBPS, 1),
      "tokens_per_s": round(cfg["batch"] / (r["ms_per_step"] * 1e-3 * model_layers), 1),
      "roofline": {
          "bound": "hbm", "kernel": r["kernel"],
          "achieved": round(attn_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
          "frac": round(attn_gbps / HBM_PEAK_GBPS, 4),
          "traffic": measured_attn_traffic_bytes() if headline and cfg["layers_rotated"] == LAYERS else None,
          "us_per_launch": round(r["attn_ms"] * 1e3, 2), "min_us_per_launch": round(r["attn_min"] * 1e3, 2),
          "algorithmic_bytes": int(r["attn_bytes"]),
      },
  }
  if first_use is not None:
    cfg["memory"] = "synthetic cache allocated, freed and allocated again before timing; first_use_memory = the same run on the first allocation"
    line["first_use_memory"] = first_use
  if headline and not args.no_other_workloads and not args.layers:
    # The other four configurations of BASELINE.json, timed the same way in the same run, one
    # after another (each is built, timed and freed before the next): for the record, the
    # headline fields above are C3's alone.
    import copy
    import gc

    import torch
    del r
    others = {}
    for name in ("c1", "c2", "c4", "c5"):
      gc.collect()
      torch.cuda.empty_cache()
      a2 = copy.copy(args)
      a2.workload = name
      progress(f"{name}: building and timing")
      o = run_gpu(a2)
      o_gbps = o["step_bytes"] / (o["ms_per_step"] * 1e-3) / 1e9
      o_attn = o["attn_bytes"] / (o["attn_ms"] * 1e-3) / 1e9
      others[name] = {
          "workload": o["config"]["workload"], "layers_rotated": o["config"]["layers_rotated"],
          "us_per_layer": round(o["ms_per_step"] * 1e3, 2), "min_us_per_layer": round(o["ms_min"] * 1e3, 2),
          "mean_us_per_layer": round(o["ms_mean"] * 1e3, 2), "repeats": o["repeats"],
          "GB_per_s": round(o_gbps, 1), "pct_of_hbm_peak": round(100 * o_gbps / HBM_PEAK_GBPS, 1),
          "layer_step_bytes": int(o["step_bytes"]),
          "attention": {"kernel": o["kernel"], "us_per_launch": round(o["attn_ms"] * 1e3, 2),
                        "min_us_per_launch": round(o["attn_min"] * 1e3, 2), "GB_per_s": round(o_attn, 1),
                        "frac": round(o_attn / HBM_PEAK_GBPS, 4), "algorithmic_bytes": int(o["attn_bytes"])},
      }
      del o
    line["other_workloads"] = others
  if headline and not args.no_cpu_baseline:
    progress("cpu baseline")
    line["cpu_baseline"] = run_cpu_baseline()
  progress("done")
  print(json.dumps(line))


if __name__ == "__main__":
  main()
