// Plan records and kernel parameters shared by the planning kernel and the
// streaming attention kernel.
#pragma once

#include "common.h"

namespace jpt {

constexpr int kTile = 32;        // positions per tile
constexpr int kD = 128;          // head_dim
constexpr int kMaxRows = 16;     // rep * q_rows
constexpr int kPartFloats = kD + 4;  // a partial's row: o[128], max, sum, 2 unused (16-byte rows)

struct PlanEntry {
  int32_t slot;        // -1: unused record
  int32_t start;       // first position of the chunk; -1: a merge entry (see `part`)
  int32_t count;       // positions in the chunk (0 for an empty slot or a merge entry)
  int32_t part;        // index of this chunk's partial record; merge entry: of the slot's first one
  int32_t n_chunks;    // chunks of this slot
  int32_t slot_len;    // positions of the whole slot
  int32_t pad[2];
};

// words of the workspace's state block
constexpr int kStateStatus = 0;    // sticky JPT_ATTN_STATUS_* bits
constexpr int kStateEntries = 2;   // plan entries that are work items (chunks and whole slots)
constexpr int kStateMerges = 3;    // merge entries, which follow them
// where the plan's arrival counters lie (32-bit words from the workspace's start) and how many
// there are: what jpt_attn_status clears, with the hand-out counters, after a launch gave up
constexpr int kStateArrivalsAt = 4;
constexpr int kStateArrivalsCount = 5;
// merge entries handed out, one counter for the workers of workgroups equal mod 8
// (one XCD), each in a cache line of its own (see the streaming kernel)
constexpr int kStateHandOut = 16;
constexpr int kStateHandOutStride = 16;
constexpr int kHandOutCounters = 8;

struct FastParams {
  jpt_attn_args a;
  const PlanEntry* entries;
  float* partials;
  int32_t* arrivals;    // per (slot, KV head): chunks of a split slot whose partial is in memory; zero between launches
  int32_t rows;         // rep * q_rows
  int32_t rep;
  int32_t total_items;  // max_entries * kv_heads
  int32_t* status;      // the workspace's state block (kState* words)
};

// How the step's new token reaches the streaming kernel (a template argument of it).
constexpr int kNewNone = 0;     // no new token: the cache only
constexpr int kNewGiven = 1;    // rows as the cache holds them (bf16, or codes with their scales)
constexpr int kNewRaw = 2;      // int8 caches: unquantised rows of all heads in one tile, quantised in the launch
constexpr int kNewRawWide = 3;  // the same with more than 16 KV heads: two tiles, keys then values
constexpr int kNewRawRope = 4;      // kNewRaw, the key rotated (rotary embedding) before it is quantised
constexpr int kNewRawWideRope = 5;  // kNewRawWide, likewise

namespace decode {
// Defined in attn_decode_i8_new<N>.hip / attn_decode_bf16_new<N>.hip, one unit per way the new token comes.
void launch_decode_i8_none(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
void launch_decode_i8_given(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
void launch_decode_i8_raw(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
void launch_decode_i8_raw_wide(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
void launch_decode_i8_raw_rope(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
void launch_decode_i8_raw_wide_rope(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
void launch_decode_bf16_none(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
void launch_decode_bf16_given(const FastParams& p, bool paged, unsigned blocks, hipStream_t stream);
}  // namespace decode

}  // namespace jpt
