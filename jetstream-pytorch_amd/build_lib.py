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
TIMELINE_LIB = os.path.join(OUT_DIR, "libjpt_mi355_timeline.so")
BUILD = os.path.join(HERE, "build")

# the units that hold the streaming attention kernel, one per cache type and way the new token comes
STREAMING = ["attn_decode_i8_raw.hip", "attn_decode_i8_raw_wide.hip", "attn_decode_i8_raw_rope.hip", "attn_decode_i8_raw_wide_rope.hip",
             "attn_decode_i8_none.hip", "attn_decode_i8_given.hip", "attn_decode_bf16_given.hip", "attn_decode_bf16_none.hip"]
SOURCES = STREAMING + ["api.cpp", "pam.cpp", "kv_lines.hip", "prefill_insert.hip", "paged_kv.hip", "device_pages.hip", "attn_generic.hip",
                       "attn_decode.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
    # keep the compiler from forming packed-FP32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", INCLUDE, "-I", CSRC,
]


def _compile(src, extra=(), tag=""):
  obj = os.path.join(BUILD, os.path.splitext(src)[0] + tag + ".o")
  cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
  r = subprocess.run(cmd, capture_output=True, text=True)
  # the host pass does not know the device-only target feature; drop its note
  err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
  if r.returncode != 0:
    raise RuntimeError(f"hipcc failed on {src}:\n{err}")
  if err.strip():
    print(err, file=sys.stderr)
  return obj


def _link(objs, lib):
  tmp = lib + ".tmp"
  cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
  r = subprocess.run(cmd, capture_output=True, text=True)
  if r.returncode != 0:
    raise RuntimeError(f"link failed:\n{r.stderr}")
  os.replace(tmp, lib)


def build(verbose=True, timeline=True):
  """The product library, and (timeline) its development twin libjpt_mi355_timeline.so, whose
  decode-attention kernel records when its waves start, stream and end (attn_timeline.py);
  nothing of the package loads the twin unless JPT_MI355_LIB names it."""
  os.makedirs(BUILD, exist_ok=True)
  # the twin's own units: what attn_timeline.py launches (int8 cache, raw token or none); the rest are the product's
  traced = ["attn_decode_i8_raw.hip", "attn_decode_i8_none.hip"]
  with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
    plain = [ex.submit(_compile, src) for src in SOURCES]
    twin = [ex.submit(_compile, src, ("-DJPT_ATTN_TIMELINE",), "_timeline") for src in traced] if timeline else []
    objs = [f.result() for f in plain]
    twin = [f.result() for f in twin]
  _link(objs, LIB)
  if verbose:
    print(f"built {LIB}")
  if timeline:
    swapped = [o for o, src in zip(objs, SOURCES) if src not in traced] + twin
    _link(swapped, TIMELINE_LIB)
    if verbose:
      print(f"built {TIMELINE_LIB}")
  return LIB


if __name__ == "__main__":
  build()
