"""MI355X-native decode-time KV-cache path with jetstream-pytorch's Python API.

Modules keep the reference's names: cache_manager, page_attention_manager,
attention_kernel, layers (attention orchestration only), environment (the
fields this path reads), quantize (KV quantisers), insert (the engine's
prefill -> decode insert), decode_state (the engine's per-step mask and
position bookkeeping).  Everything runs on HIP
kernels in libjpt_mi355.so; importing fails if the library is not built.
"""

from . import _ffi  # noqa: F401  (raises when the library is missing)
from . import (attention_kernel, cache_manager, decode_state, environment, insert, layers,  # noqa: F401
               page_attention_manager, quantize)

__all__ = ["attention_kernel", "cache_manager", "decode_state", "environment", "insert", "layers",
           "page_attention_manager", "quantize"]
