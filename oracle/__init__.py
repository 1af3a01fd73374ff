"""CPU oracle for the decode-time KV-cache path.  TEST INFRASTRUCTURE ONLY.

This package restates, op for op, the algorithm of the reference
implementation (jetstream-pytorch 0.2.2) for the functions on the decode-time
KV-cache path, using torch-CPU and numpy only.  It exists to check the HIP
kernels; nothing in the shipped package imports it.  Only the test-suite, the
smoke check and the `cpu_baseline` leg of the benchmark may import it.

Every function cites the reference file:line it follows.  The restatement is
pinned by (see tests/test_oracle_*.py):

* the exact-integer scenarios held by the reference's own tests
  (tests/test_page_attention.py, tests/test_kv_cache_manager.py), committed as
  data under tests/golden/;
* closed forms: bit-level float64/integer recomputation of both int8
  quantisers, float64 masked-softmax attention, brute-force loops on tiny
  shapes for every copy/scatter/gather.

Parity unpinned (nothing in the reference pins it and the dependency is
absent): the numerics of JAX's external `paged_attention` TPU kernel that
`call_paged_attention` wraps (jax.experimental.pallas.ops.tpu.paged_attention,
installer pin jax 0.4.37) - in particular whether it applies 1/sqrt(head_dim).
`oracle.attention.paged_attention` therefore takes `sm_scale` explicitly.
"""

from . import attention, decode_state, insert, kv_cache, page_manager, quant, rope  # noqa: F401
from .env import Env  # noqa: F401
