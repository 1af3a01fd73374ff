// bf16-KV instantiations of the streaming decode attention kernel: new token given as the cache holds it.
#include "attn_decode_impl.h"

namespace jpt {
namespace decode {
void launch_decode_bf16_given(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream) {
  launch_decode<__bf16, kNewGiven>(p, paged, blocks, stream);
}
}  // namespace decode
}  // namespace jpt
