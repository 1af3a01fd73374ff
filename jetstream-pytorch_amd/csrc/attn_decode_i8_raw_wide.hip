// int8-KV instantiations of the streaming decode attention kernel: new token of more than 16 KV heads quantised in the launch.
#include "attn_decode_impl.h"

namespace jpt {
namespace decode {
void launch_decode_i8_raw_wide(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream) {
  launch_decode<int8_t, kNewRawWide>(p, paged, blocks, stream);
}
}  // namespace decode
}  // namespace jpt
