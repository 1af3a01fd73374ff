// bf16-KV instantiations of the streaming decode attention kernel: no new token.
#include "attn_decode_impl.h"

namespace jpt {
namespace decode {
void launch_decode_bf16_none(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream) {
  launch_decode<__bf16, kNewNone>(p, paged, blocks, stream);
}
}  // namespace decode
}  // namespace jpt
