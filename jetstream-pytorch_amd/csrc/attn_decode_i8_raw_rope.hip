// int8-KV instantiations of the streaming decode attention kernel: new token rotated and quantised in the launch.
#include "attn_decode_impl.h"

namespace jpt {
namespace decode {
void launch_decode_i8_raw_rope(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream) {
  launch_decode<int8_t, kNewRawRope>(p, paged, blocks, stream);
}
}  // namespace decode
}  // namespace jpt
