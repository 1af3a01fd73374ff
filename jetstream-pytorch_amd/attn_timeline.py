"""When the workers of the decode-attention launch start, stream and end.

Runs the headline workload's attention launch (C3: batch 128, 32 q / 8 kv heads,
int8 cache of 8192 positions, log-normal lengths, the step's token quantised and
attended in the launch) on the development twin of the library,
libjpt_mi355_timeline.so (build_lib.py builds it beside the product's), whose
kernel leaves per-wave clock readings in the workspace's state block, and prints
a summary: first load, first tile consumed, the producers' last tile, the
groups' ends, and a least-squares fit of a bin's end time on its tiles and items
(a bin = the eight workers that take the heads of one plan entry).

  python jetstream-pytorch_amd/attn_timeline.py [--case c3|<positions per slot>|uniform:LO:HI] [--batch B] [--unfused]

Times are in microseconds from the first wave's start, on the constant 100 MHz
clock; the kernel's duration by the host's clock is about 1.8 us longer than the
last wave's end (launch and completion).  Development aid: the product library
is not involved, and nothing of the package imports this file.
"""

import argparse
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
for _p in (ROOT, HERE):
  if _p not in sys.path:
    sys.path.insert(0, _p)
os.environ["JPT_MI355_LIB"] = os.path.join(HERE, "jetstream_pt_amd", "libjpt_mi355_timeline.so")

import numpy as np  # noqa: E402
import torch  # noqa: E402

import bench  # noqa: E402
from jetstream_pt_amd import attention_kernel as ak  # noqa: E402


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--case", default="c3", help="c3; a number: every slot that many positions long; "
                  "uniform:LO:HI: lengths drawn uniformly from [LO, HI] (seed 4)")
  ap.add_argument("--batch", type=int, default=0, help="slots (default: the headline workload's 128)")
  ap.add_argument("--unfused", action="store_true", help="attention over the cache only, no new token")
  ap.add_argument("--reps", type=int, default=3)
  args = ap.parse_args()
  dev = "cuda"
  b, hq, hkv, s, d, nl = args.batch or bench.B, bench.HQ, bench.HKV, bench.S, bench.D, 8
  if b > bench.B:
    s, nl = s * bench.B // b, 4  # the same bytes of cache
  torch.manual_seed(3)
  k = torch.empty((nl, b, hkv, s, d), dtype=torch.int8, device=dev)
  v = torch.empty_like(k)
  for l in range(nl):
    k[l].random_(-127, 128)
    v[l].random_(-127, 128)
  ks = torch.empty((nl, b, 1, s, 1), device=dev).uniform_(0.005, 0.05)
  vs = torch.empty_like(ks).uniform_(0.005, 0.05)
  q = torch.randn((b, hq, 1, d), device=dev).to(torch.bfloat16)
  xk = torch.randn((b, hkv, 1, d), device=dev).to(torch.bfloat16)
  xv = torch.randn((b, hkv, 1, d), device=dev).to(torch.bfloat16)
  nk = torch.zeros((b, hkv, 1, d), dtype=torch.int8, device=dev)
  nv = torch.zeros_like(nk)
  nks = torch.zeros((b, 1, 1, 1), device=dev)
  nvs = torch.zeros_like(nks)
  if args.case == "c3":
    lengths = bench.seeded_lengths(torch, b)
  elif args.case.startswith("uniform:"):
    lo, hi = (int(x) for x in args.case.split(":")[1:])
    lengths = bench.uniform_lengths(torch, b, lo, min(hi, s - 1), 4)
  else:
    lengths = torch.full((b,), int(args.case))
  lengths = lengths.to(dev).to(torch.int32)
  plan, _ = ak.precompute_ragged_block_indices(lengths, b, hq, hkv, s)
  new = {} if args.unfused else dict(new_key=nk, new_value=nv, new_k_scaler=nks, new_v_scaler=nvs,
                                     new_key_raw=xk, new_value_raw=xv)

  def launch(i):
    return ak.ragged_mha(q, k, v, i % nl, None, plan.lengths, plan, None, ks, vs, **new)

  print(f"case {args.case}, {'cache only' if args.unfused else 'token quantised and attended in the launch'}; "
        f"{int(lengths.sum())} cached positions; one line block per launch sampled")
  for rep in range(args.reps):
    for i in range(16):
      launch(i)
    torch.cuda.synchronize()
    raw = plan.workspace.buf[1024:1024 + 2048 * 16].view(torch.int32).cpu().numpy().astype(np.int64)
    tr = raw.reshape(256, 2, 4, 4) & 0xffffffff  # [workgroup, group, producer | consumers, record]
    t0 = tr[..., 0].min()
    us = lambda x: (x - t0) / 100.0
    prod, cons = tr[:, :, 0, :], tr[:, :, 1:, :]
    gend = us(cons[..., 2]).max(axis=2)  # a group ends with its last consumer
    tiles = prod[..., 3] & 0xffff
    items = cons[:, :, 0, 3] >> 16
    print(f"== launch sample {rep}")
    print("  waves start by %.2f; producers' first load: median %.2f, last %.2f; consumers' first tile: median %.2f"
          % (us(tr[..., 0]).max(), np.median(us(prod[..., 1])), us(prod[..., 1]).max(), np.median(us(cons[..., 1]))))
    print("  producers' last tile landed: median %.2f, p90 %.2f, last %.2f"
          % tuple(np.percentile(us(prod[..., 2]), [50, 90, 100])))
    print("  groups end: p1 %.1f  p10 %.1f  median %.1f  p90 %.1f  p99 %.1f  last %.1f"
          % tuple(np.percentile(gend, [1, 10, 50, 90, 99, 100])))
    print("  from a group's last tile landing to its end: mean %.2f; spread of its consumers' ends: mean %.2f"
          % ((gend - us(prod[..., 2])).mean(), (us(cons[..., 2]).max(axis=2) - us(cons[..., 2]).min(axis=2)).mean()))
    for n in sorted(set(items.flatten())):
      m = items == n
      print(f"  workers with {n} items: {m.sum():3d}, tiles {tiles[m].mean():.1f} ({tiles[m].min()}..{tiles[m].max()}), "
            f"end mean {gend[m].mean():.2f}, last {gend[m].max():.2f}")
    worker = np.arange(512)
    blk, grp = worker % 256, worker // 256
    bins = (worker >> 6) * 8 + (worker & 7)
    ge, tl, it = gend[blk, grp], tiles[blk, grp], items[blk, grp]
    bm = np.array([ge[bins == x].mean() for x in range(64)])
    bt = np.array([tl[bins == x].mean() for x in range(64)])
    bi = np.array([it[bins == x].mean() for x in range(64)])
    within = np.array([ge[bins == x].max() - ge[bins == x].min() for x in range(64)])
    a = np.stack([bt, bi, np.ones(64)], 1)
    coef = np.linalg.lstsq(a, bm, rcond=None)[0]
    print("  bins: mean end %.2f, std of the bins' means %.2f, spread inside a bin (mean) %.2f"
          % (bm.mean(), bm.std(), within.mean()))
    print("  fit over the 64 bins: end = %.3f * tiles + %.2f * items + %.2f, residual std %.2f"
          % (coef[0], coef[1], coef[2], (bm - a @ coef).std()))
    xcd = np.arange(256) % 8
    print("  per XCD, mean end: " + " ".join("%.1f" % gend[xcd == x].mean() for x in range(8)))
    print("  per XCD, producers' first load: " + " ".join("%.2f" % us(prod[..., 1])[xcd == x].mean() for x in range(8))
          + "; last tile landed: " + " ".join("%.1f" % us(prod[..., 2])[xcd == x].mean() for x in range(8)))


if __name__ == "__main__":
  main()
