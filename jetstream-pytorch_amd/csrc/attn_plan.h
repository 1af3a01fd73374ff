// Plan records and kernel parameters shared by the planning kernel, the
// streaming attention kernel and the partial-merge kernel.
#pragma once

#include "common.h"

namespace jpt {

constexpr int kTile = 32;        // positions per tile
constexpr int kD = 128;          // head_dim
constexpr int kMaxRows = 16;     // rep * q_rows
constexpr int kPartFloats = kD + 4;  // a partial's row: o[128], max, sum, 2 unused (16-byte rows)

struct PlanEntry {
  int32_t slot;        // -1: unused record
  int32_t start;       // first position of the chunk
  int32_t count;       // positions in the chunk (0 for an empty slot)
  int32_t part;        // index of this chunk's partial record
  int32_t n_chunks;    // chunks of this slot
  int32_t slot_len;    // positions of the whole slot
  int32_t pad[2];
};
struct SlotChunks {
  int32_t n_chunks, first_part;
};

struct FastParams {
  jpt_attn_args a;
  const PlanEntry* entries;
  const SlotChunks* slots;
  float* partials;
  int32_t rows;         // rep * q_rows
  int32_t rep;
  int32_t total_items;  // max_entries * kv_heads
  int32_t* status;      // word 0 of the workspace's state block: sticky, set when a wave gave up
};

namespace decode {
// Defined in attn_decode_i8.hip / attn_decode_bf16.hip.
void launch_decode_i8(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
void launch_decode_bf16(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
}  // namespace decode

}  // namespace jpt
