"""Benchmark of the decode-time KV-cache hot path on one MI355X.

Workload (BASELINE.json configs[2], the headline): ragged GQA decode
attention for one Llama-3-8B layer - batch 128, 32 q heads / 8 KV heads,
head_dim 128, cache length 8192, int8 KV codes with fp32 per-token scales,
per-slot lengths log-normal (median 400, sigma 1) clipped to [16, 8192].

A step is one layer-step of the production left-aligned mode: fused int8
quantise + stash of the new token, then ragged attention over the cache with
the new token merged in the same launch.  Steps rotate over the 32 layers of
a stacked cache (64 GiB of codes), so every step streams cold data; once per
32 steps the per-step split plan is recomputed and finalize() scatters the 32
stashed tokens into the cache (both inside the timed region).

Prints one JSON line.  `value` is algorithmic bytes of the layer-step divided
by its time; `roofline` is the attention kernel alone (a separate timed loop
of attention launches only); `cpu_baseline` times the CPU oracle's
restatement of the reference path on the host cores.
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
B, HQ, HKV, D, S, LAYERS = 128, 32, 8, 128, 8192, 32
SEED = 3
PROBE_COPY_BYTES = 1 << 30
# HBM bytes of one attention launch (decode kernel + merge kernel) on this
# workload, from hardware counters (FETCH_SIZE + WRITE_SIZE, each calibrated on a
# 1 GiB copy; see --probe-traffic).  A recorded measurement, not computed here.
MEASURED_ATTN_TRAFFIC_BYTES = 163_210_000


def seeded_lengths(torch):
  g = torch.Generator().manual_seed(SEED)
  z = torch.randn(B, generator=g, dtype=torch.float64)
  return torch.clamp(torch.round(torch.exp(math.log(400.0) + z)), 16, S).to(torch.int32)


def attn_bytes(lengths):
  """Algorithmic bytes of one attention launch: int8 K and V codes of the
  attended positions, their fp32 scales (one per token, shared by all heads),
  q in and o out (bf16), the lengths, and the new token's codes and scales."""
  total = int(lengths.sum())
  kv = total * HKV * D * 2
  scales = total * 4 * 2
  qo = B * HQ * D * 2 * 2
  new_tok = B * HKV * D * 2 + B * 4 * 2
  return kv + scales + qo + new_tok + B * 4


def append_bytes():
  """Quantise + stash: bf16 K and V in, int8 codes and fp32 scales out."""
  return B * HKV * D * (2 + 1) * 2 + B * 4 * 2


def finalize_bytes_per_layer():
  """finalize(): per layer, codes and scales read from the stash and written
  into the cache."""
  return (B * HKV * D + B * 4) * 2 * 2


def run_gpu(args):
  import torch

  from jetstream_pt_amd import attention_kernel as ak
  from jetstream_pt_amd import cache_manager as cm
  from jetstream_pt_amd import layers
  from jetstream_pt_amd.environment import JetEngineEnvironment, JetEngineEnvironmentData

  dev = "cuda:0"
  torch.cuda.set_device(0)
  lengths = seeded_lengths(torch)
  nl = args.layers
  env = JetEngineEnvironment(JetEngineEnvironmentData(batch_size=B, num_layers=nl, ring_buffer=False))
  shape = (nl, B, HKV, S, D)
  cache = cm.Int8KVCacheGenerate.empty(shape, dev, env, scale_heads=1, scale_dtype=torch.float32)
  for l in range(nl):  # codes uniform [-127, 127], scales U(0.005, 0.05)
    cache.cache_k[l].random_(-127, 128)
    cache.cache_v[l].random_(-127, 128)
    cache.k_scaler[l].uniform_(0.005, 0.05)
    cache.v_scaler[l].uniform_(0.005, 0.05)
  g = torch.Generator(device=dev).manual_seed(SEED)
  xq = torch.randn((B, HQ, 1, D), generator=g, device=dev).to(torch.bfloat16)
  xk = torch.randn((B, HKV, 1, D), generator=g, device=dev).to(torch.bfloat16)
  xv = torch.randn((B, HKV, 1, D), generator=g, device=dev).to(torch.bfloat16)
  pos = lengths.to(dev)
  cache.input_pos = pos
  kernels = [layers.Int8KVAttentionKernel(env, l) for l in range(nl)]
  state = {"plan": None}

  def layer_step(i):
    l = i % nl
    if l == 0:
      state["plan"], _ = ak.precompute_ragged_block_indices(pos, B, HQ, HKV, S)
    plan = state["plan"]
    out = kernels[l](xq, xk, xv, None, cache, start=None, end=plan.lengths, ragged_batch_index=plan)
    if l == nl - 1:
      cache.finalize()
    return out

  def timed(fn, steps, warmup):
    """fn(i) enqueues step i.  Whole passes over the layers are replayed from
    one captured HIP graph (what a serving loop does with a launch-bound
    decode step); a remainder of steps runs eagerly."""
    for i in range(max(warmup, nl)):
      fn(i)
    torch.cuda.synchronize()
    graph = None
    if not args.no_graph and steps >= nl:
      graph = torch.cuda.CUDAGraph()
      with torch.cuda.graph(graph):
        for i in range(nl):
          fn(i)
      graph.replay()
      torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    done = 0
    if graph is not None:
      for _ in range(steps // nl):
        graph.replay()
      done = steps // nl * nl
    for i in range(done, steps):
      fn(i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps

  ms_per_step = timed(layer_step, args.steps, args.warmup)

  # one attention launch alone (decode kernel + partial-merge kernel), same inputs
  plan, _ = ak.precompute_ragged_block_indices(pos, B, HQ, HKV, S)
  new = dict(new_key=cache.new_ks[0], new_value=cache.new_vs[0],
             new_k_scaler=cache.new_k_scaler[0], new_v_scaler=cache.new_v_scaler[0])
  def attn_only(i):
    return ak.ragged_mha(xq, cache.cache_k, cache.cache_v, i % nl, None, plan.lengths, plan, None,
                         cache.k_scaler, cache.v_scaler, **new)
  attn_ms = timed(attn_only, args.steps, args.warmup)

  step_bytes = attn_bytes(lengths) + append_bytes() + finalize_bytes_per_layer()
  return dict(ms_per_step=ms_per_step, attn_ms=attn_ms, step_bytes=step_bytes,
              attn_bytes=attn_bytes(lengths), total_tokens=int(lengths.sum()))


def run_traffic_probe(args):
  """Work for a hardware-counter run (rocprofv3 --pmc FETCH_SIZE or WRITE_SIZE):
  a few attention launches of the headline workload next to plain copies of a
  buffer of known size, whose counter reading calibrates the counter's unit."""
  import torch

  from jetstream_pt_amd import attention_kernel as ak

  dev = "cuda:0"
  torch.cuda.set_device(0)
  nl = 4
  lengths = seeded_lengths(torch).to(dev)
  k = torch.empty((nl, B, HKV, S, D), dtype=torch.int8, device=dev)
  v = torch.empty_like(k)
  for l in range(nl):
    k[l].random_(-127, 128)
    v[l].random_(-127, 128)
  ks = torch.empty((nl, B, 1, S, 1), device=dev).uniform_(0.005, 0.05)
  vs = torch.empty_like(ks).uniform_(0.005, 0.05)
  g = torch.Generator(device=dev).manual_seed(SEED)
  xq = torch.randn((B, HQ, 1, D), generator=g, device=dev).to(torch.bfloat16)
  nk = torch.empty((B, HKV, 1, D), dtype=torch.int8, device=dev).random_(-127, 128)
  nv = torch.empty_like(nk).random_(-127, 128)
  nks = torch.empty((B, 1, 1, 1), device=dev).uniform_(0.005, 0.05)
  nvs = torch.empty_like(nks).uniform_(0.005, 0.05)
  plan, _ = ak.precompute_ragged_block_indices(lengths, B, HQ, HKV, S)
  src = torch.empty(PROBE_COPY_BYTES // 4, dtype=torch.float32, device=dev).normal_()
  dst = torch.empty_like(src)
  for i in range(8):
    ak.ragged_mha(xq, k, v, i % nl, None, plan.lengths, plan, None, ks, vs, new_key=nk, new_value=nv,
                  new_k_scaler=nks, new_v_scaler=nvs)
    dst.copy_(src)
  torch.cuda.synchronize()
  print(json.dumps({"probe": "traffic", "attention_launches": 8, "copies": 8,
                    "copy_bytes_read": PROBE_COPY_BYTES, "copy_bytes_written": PROBE_COPY_BYTES,
                    "attn_algorithmic_bytes": attn_bytes(lengths.cpu())}))


def run_cpu_baseline(budget_s=20.0):
  """The oracle (CPU restatement of the reference path) on one layer of the
  same workload: Int8KVCacheGenerate.update + ragged_mha + new-token flash
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
  nbytes = attn_bytes(lengths) + append_bytes()
  return dict(value=round(nbytes / med / 1e9, 3), unit="GB/s", cores=cores, kind="port",
              sample=f"one full layer-step (all {B} slots, {int(lengths.sum())} cached tokens), "
                     f"median of {len(times)} runs, {med * 1e3:.1f} ms each")


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=640)
  ap.add_argument("--warmup", type=int, default=64)
  ap.add_argument("--layers", type=int, default=LAYERS)
  ap.add_argument("--no-cpu-baseline", action="store_true")
  ap.add_argument("--no-graph", action="store_true", help="launch every step from Python")
  ap.add_argument("--probe-traffic", action="store_true",
                  help="run a few attention launches and calibration copies for a counter run")
  args = ap.parse_args()
  if args.gpus != 1:
    sys.exit("bench.py measures one GPU: the path is built and measured on a single MI355X "
             "(--gpus must be 1)")
  if args.probe_traffic:
    run_traffic_probe(args)
    return
  r = run_gpu(args)
  gbps = r["step_bytes"] / (r["ms_per_step"] * 1e-3) / 1e9
  attn_gbps = r["attn_bytes"] / (r["attn_ms"] * 1e-3) / 1e9
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
      "config": {
          "workload": "C3 ragged GQA int8 decode layer-step: KV quantise+stash, ragged attention "
                      "with fused new token, finalize amortised over 32 layers",
          "batch": B, "q_heads": HQ, "kv_heads": HKV, "head_dim": D, "max_cache_len": S,
          "layers_rotated": args.layers, "cached_tokens": r["total_tokens"],
          "launch": "python" if args.no_graph else "hip graph of one pass over the layers",
          "kv": "int8 codes + fp32 per-token scales", "lengths": "log-normal(median 400, sigma 1) in [16, 8192], seed 3",
      },
      "us_per_layer": round(r["ms_per_step"] * 1e3, 2),
      "pct_of_hbm_peak": round(100 * gbps / HBM_PEAK_GBPS, 1),
      "tokens_per_s": round(B / (r["ms_per_step"] * 1e-3 * LAYERS), 1),
      "roofline": {
          "bound": "hbm", "kernel": "attn_decode_kernel<int8> + attn_merge_kernel (one attention launch)",
          "achieved": round(attn_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
          "frac": round(attn_gbps / HBM_PEAK_GBPS, 4),
          "traffic": MEASURED_ATTN_TRAFFIC_BYTES if args.layers == LAYERS else None,
          "us_per_launch": round(r["attn_ms"] * 1e3, 2), "algorithmic_bytes": r["attn_bytes"],
      },
  }
  if not args.no_cpu_baseline:
    line["cpu_baseline"] = run_cpu_baseline()
  print(json.dumps(line))


if __name__ == "__main__":
  main()
