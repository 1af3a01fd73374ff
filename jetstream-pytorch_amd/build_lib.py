"""Builds libjpt_mi355.so (HIP kernels + host allocator + C ABI) for gfx950.

Usage: python build_lib.py            (from anywhere)
The library lands next to the Python package that loads it, so that it
travels with the source tree.
"""

import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
OUT_DIR = os.path.join(HERE, "jetstream_pt_amd")
LIB = os.path.join(OUT_DIR, "libjpt_mi355.so")
BUILD = os.path.join(HERE, "build")

SOURCES = ["api.cpp", "pam.cpp", "kv_lines.hip", "prefill_insert.hip", "paged_kv.hip", "device_pages.hip", "attn_generic.hip", "attn_decode.hip",
           "attn_decode_i8.hip", "attn_decode_bf16.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
    # keep the compiler from forming packed-FP32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", INCLUDE, "-I", CSRC,
]


def _compile(src):
  obj = os.path.join(BUILD, os.path.splitext(src)[0] + ".o")
  cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
  r = subprocess.run(cmd, capture_output=True, text=True)
  # the host pass does not know the device-only target feature; drop its note
  err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
  if r.returncode != 0:
    raise RuntimeError(f"hipcc failed on {src}:\n{err}")
  if err.strip():
    print(err, file=sys.stderr)
  return obj


def build(verbose=True):
  os.makedirs(BUILD, exist_ok=True)
  with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
    objs = list(ex.map(_compile, SOURCES))
  tmp = LIB + ".tmp"
  cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
  r = subprocess.run(cmd, capture_output=True, text=True)
  if r.returncode != 0:
    raise RuntimeError(f"link failed:\n{r.stderr}")
  os.replace(tmp, LIB)
  if verbose:
    print(f"built {LIB}")
  return LIB


if __name__ == "__main__":
  build()
