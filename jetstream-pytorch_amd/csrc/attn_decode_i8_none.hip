// int8-KV instantiations of the streaming decode attention kernel: no new token.
#include "attn_decode_impl.h"

namespace jpt {
namespace decode {
void launch_decode_i8_none(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream) {
  launch_decode<int8_t, kNewNone>(p, paged, blocks, stream);
}
}  // namespace decode
}  // namespace jpt
