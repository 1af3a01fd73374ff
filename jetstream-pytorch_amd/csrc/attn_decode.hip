// Ragged / dense / paged GQA decode attention for gfx950, head_dim 128: host
// side and planning kernel.  The streaming attention
// kernel itself is in attn_decode_impl.h.
//
// Work decomposition (split-KV).  The planning kernel turns the per-slot
// lengths into a list of chunks (slot, first position, count), sized so the
// batch yields a few work items per persistent worker whatever the length
// distribution.  A slot that fits one chunk is finished by the worker that
// attends it.  A longer slot is cut into equal chunks.  Cut in two, its chunks
// go to the two groups of waves of one workgroup, which fold them through LDS:
// nothing of such a slot touches memory but its output.  Cut in three or more,
// its chunks come first in the list (every worker starts with one of them, if
// there are that many); each parks a float32 partial (o, max, sum) in memory
// and counts itself on the slot's arrival counter.  Merge entries, one per such
// slot and KV head, fold the partials into the slot's output; they are not
// dealt out: a worker's producer wave, once its last tile has landed, takes
// merge entries from a counter in memory for as long as there are any, while
// its consumers work off the tiles still in the ring - whoever is done first
// does the merging.  One launch: no second kernel, and no device-wide fence
// either; partials and counters are written through to memory and read past
// the caches.
//
// Bound: HBM bandwidth.  Algorithmic bytes per (slot, KV head) are
// len * 128 * (bytes(K) + bytes(V)) plus len * (bytes(k_scale) +
// bytes(v_scale)) / heads-sharing-a-scale.
#include <math.h>

#include <mutex>

#include "attn_common.h"
#include "attn_plan.h"

namespace jpt {
namespace {

constexpr int kChunkAlign = 128;

// ---- workspace layout --------------------------------------------------------
// [0, 64 KiB)   state block, zero before the first call; word 0 is the sticky
//               status word that jpt_attn_status reads and clears, words 2 and 3
//               the numbers of work entries and of merge entries in the plan,
//               words 16, 32, ... 128 the counters that hand out the merge
//               entries (cleared by every plan, advanced by the same amounts by
//               every launch)
// then          plan entries, arrival counters (batch x kv_heads), partials
struct Layout {
  int64_t entries, arrivals, partials, total;
  int32_t max_entries;
};

constexpr int kMaxPlanBatch = 4096;
constexpr int kMaxChunksPerSlot = 256;
constexpr int kMaxBins = 1024;         // entries of one round of the workers' walk: workers / kv_heads
constexpr int kDealtOneByOne = 512;  // entries dealt to the lightest bin one by one (about 0.12 us each)

// Workers of the streaming kernel: two groups of waves on every compute unit.
int32_t persistent_blocks() {
  static int32_t v = [] {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess)
      if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cus = 256;
    return (cus * 2 + 7) / 8 * 8;
  }();
  return v;
}

// Work items (chunk x KV head) the planner aims for: five for every four
// workers.  An item costs a few microseconds beyond its tiles (query rows,
// fold, output or partial), so chunks are made about as long as a worker's
// share of the positions, and the sort-and-deal of the plan evens out the rest.
int32_t target_items() { return persistent_blocks() * 5 / 4; }

Layout make_layout(int batch, int kv_heads, int rows) {
  Layout l;
  // one entry a slot, the extra chunks of split slots (at most the target's worth,
  // and every split slot has at least one), and a merge entry for each split slot
  const int extra = (target_items() + kv_heads - 1) / kv_heads + 1;
  // ... and the places a half-filled round of paired chunks leaves empty
  // Every bin (workers / kv_heads of them) may end one round short of the fullest: two rounds of
  // slack, and up to `batch` merge entries behind the places.
  l.max_entries = (2 * batch + 2 * extra + 3 * (persistent_blocks() / kv_heads + 8) + 7) / 8 * 8;
  auto up = [](int64_t x) { return (x + 255) / 256 * 256; };
  l.entries = JPT_ATTN_WS_STATE_BYTES;
  l.arrivals = up(l.entries + static_cast<int64_t>(l.max_entries) * sizeof(PlanEntry));
  l.partials = up(l.arrivals + static_cast<int64_t>(batch) * kv_heads * sizeof(int32_t));
  l.total = up(l.partials + static_cast<int64_t>(batch + extra) * kv_heads * rows * kPartFloats * 4);
  return l;
}

// ---- planning kernel -----------------------------------------------------------
// One workgroup.  chunk = max(128, total positions * kv_heads / target items,
// rounded up to 128); a slot longer than that is cut into ceil(len / chunk)
// equal chunks of whole tiles, any other slot is one entry (an empty slot still
// needs one item per head to write its output).  Entries are counting-sorted by
// tile count, longest first: the slots cut in two (their two chunks on a pair
// of places that one workgroup's groups walk in the same round, see below),
// then the chunks of the other cut slots, then whole slots; after the last
// place one merge entry for every slot cut in three or more; places nobody was
// put on are marked unused.  The arrival counters are cleared.
// Exclusive prefix sum of `x` over the 256 threads of the planning workgroup;
// *total gets the sum.
__device__ __forceinline__ int plan_exclusive_scan(int x, int* total) {
  __shared__ int s_wave[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = x;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int y = __shfl_up(incl, off);
    if (lane >= off) incl += y;
  }
  __syncthreads();  // s_wave may still be read from the previous call
  if (lane == 63) s_wave[wave] = incl;
  __syncthreads();
  int before = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    if (w < wave) before += s_wave[w];
    sum += s_wave[w];
  }
  *total = sum;
  return before + incl - x;
}

// Minimum of `x` over the wave, the same (scalar) value for every lane: within the
// 16-lane rows by data-parallel primitives, across the four rows by lane reads.
template <int CTRL>
__device__ __forceinline__ unsigned plan_dpp(unsigned v) {
  return static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ unsigned wave_min_u32(unsigned x) {
  x = min(x, plan_dpp<0xB1>(x));   // quad_perm [1, 0, 3, 2]
  x = min(x, plan_dpp<0x4E>(x));   // quad_perm [2, 3, 0, 1]
  x = min(x, plan_dpp<0x141>(x));  // row_half_mirror
  x = min(x, plan_dpp<0x140>(x));  // row_mirror
  const int v = static_cast<int>(x);
  const unsigned a = static_cast<unsigned>(__builtin_amdgcn_readlane(v, 0)), b = static_cast<unsigned>(__builtin_amdgcn_readlane(v, 16));
  const unsigned c = static_cast<unsigned>(__builtin_amdgcn_readlane(v, 32)), d = static_cast<unsigned>(__builtin_amdgcn_readlane(v, 48));
  return min(min(a, b), min(c, d));
}

// Longest-processing-time deal by one wave.  Entry `rank` (longest first, its
// tiles in rank_tiles) goes to the bin with the fewest tiles so far, into the
// bin's first free round; rank_place gets its place.  Everything lives in
// registers: lane l keeps bins l, l + 64, ... as (tiles << 10 | bin), and the
// tiles and places of the 64 ranks of the current block, one a lane; the loop
// body is a wave-wide minimum, two lane reads and a few selects, with no memory
// access and no branch (an entry costs about a quarter of a microsecond less
// than with LDS in the loop, and there are hundreds).
template <int PER_LANE>
__device__ __forceinline__ void deal_longest_first(int first, int n, int per_round, int max_rounds, int* bin_load,
                                                   int* bin_rounds, const int* rank_tiles, int* rank_place) {
  const int lane = threadIdx.x;
  unsigned mine[PER_LANE];
  int rounds[PER_LANE];
#pragma unroll
  for (int i = 0; i < PER_LANE; ++i) {
    const int x = lane + 64 * i;
    rounds[i] = x < per_round ? bin_rounds[x] : max_rounds;
    // a bin with no free round is out of the running (there is room for all: max_rounds * per_round)
    mine[i] = rounds[i] < max_rounds ? (static_cast<unsigned>(bin_load[x]) << 10) | static_cast<unsigned>(x) : ~0u;
  }
  for (int block = first; block < n; block += 64) {
    const int my_tiles = block + lane < n ? rank_tiles[block + lane] : 0;
    int my_place = 0;
    const int in_block = min(64, n - block);
    for (int j = 0; j < in_block; ++j) {
      const unsigned tiles = static_cast<unsigned>(__builtin_amdgcn_readlane(my_tiles, j));
      unsigned best = mine[0];
#pragma unroll
      for (int i = 1; i < PER_LANE; ++i) best = min(best, mine[i]);
      best = wave_min_u32(best);
      const int x = static_cast<int>(best & 1023u);
      int round = 0;
#pragma unroll
      for (int i = 0; i < PER_LANE; ++i) {
        const bool here = PER_LANE == 1 || (x >> 6) == i;  // wave-uniform
        if (here) round = __builtin_amdgcn_readlane(rounds[i], x & 63);
      }
      const int place = round * per_round + ((round & 1) ? per_round - 1 - x : x);
      const bool winner = (x & 63) == lane;
#pragma unroll
      for (int i = 0; i < PER_LANE; ++i) {
        const bool here = winner && (PER_LANE == 1 || (x >> 6) == i);
        rounds[i] += here ? 1 : 0;
        mine[i] = !here ? mine[i] : rounds[i] < max_rounds ? mine[i] + (tiles << 10) : ~0u;
      }
      my_place = lane == j ? place : my_place;
    }
    if (block + lane < n) rank_place[block + lane] = my_place;
  }
#pragma unroll
  for (int i = 0; i < PER_LANE; ++i) {
    const int x = lane + 64 * i;
    if (x < per_round) {
      bin_rounds[x] = rounds[i];
      bin_load[x] = static_cast<int>(mine[i] >> 10);  // a full bin reads as the heaviest, which suits what follows
    }
  }
}

// The same deal, many entries a step (at most 64 bins, one a lane).  The bins are
// sorted by (tiles, bin) across the wave; entry i + j goes to the j-th lightest bin
// for as long as that bin is lighter than every bin already given an entry of this
// step is afterwards - exactly the choices of the one-by-one deal, which picks bin
// j for entry i + j if and only if bin j's key is below the new keys of bins
// 0..j-1.  Entries come in levels (every bin gets one of the long entries before
// any gets a second), so a step usually places dozens: a sort of 21 exchanges and
// a running minimum instead of a minimum per entry.  When a step places fewer than
// eight (short entries on uneven bins), the rest is dealt one by one.  Returns the
// first rank that is still to be dealt.
__device__ __forceinline__ unsigned plan_sort_wave(unsigned key, int lane) {
#pragma unroll
  for (int k = 2; k <= 64; k <<= 1) {
#pragma unroll
    for (int j = k >> 1; j > 0; j >>= 1) {
      const unsigned other = static_cast<unsigned>(__shfl_xor(static_cast<int>(key), j));
      const bool up = (lane & k) == 0, lower = (lane & j) == 0;
      key = (lower == up) ? min(key, other) : max(key, other);
    }
  }
  return key;
}
__device__ __forceinline__ int deal_longest_first_in_steps(int n, int per_round, int max_rounds, int* bin_load,
                                                           int* bin_rounds, const int* rank_tiles, int* rank_place) {
  const int lane = threadIdx.x;
  int first = 0;
  while (first < n) {
    unsigned key = ~0u;  // a bin with no free round is out of the running
    if (lane < per_round && bin_rounds[lane] < max_rounds) key = (static_cast<unsigned>(bin_load[lane]) << 10) | static_cast<unsigned>(lane);
    key = plan_sort_wave(key, lane);
    const bool has_entry = first + lane < n && key != ~0u;
    const unsigned tiles = has_entry ? static_cast<unsigned>(rank_tiles[first + lane]) : 0u;
    const unsigned after = has_entry ? key + (tiles << 10) : ~0u;
    // the lightest of the bins before this lane once they have their entries (exclusive running minimum)
    unsigned before = after;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned y = static_cast<unsigned>(__shfl_up(static_cast<int>(before), off));
      if (lane >= off) before = min(before, y);
    }
    before = static_cast<unsigned>(__shfl_up(static_cast<int>(before), 1));
    if (lane == 0) before = ~0u;
    const bool ok = has_entry && key < before;
    const unsigned long long bad = ~__ballot(ok);  // lanes whose entry is not this step's
    const int placed = bad == 0 ? 64 : __ffsll(static_cast<long long>(bad)) - 1;
    if (lane < placed) {
      const int x = static_cast<int>(key & 1023u);
      const int round = bin_rounds[x];
      rank_place[first + lane] = round * per_round + ((round & 1) ? per_round - 1 - x : x);
      bin_rounds[x] = round + 1;
      bin_load[x] = static_cast<int>(key >> 10) + static_cast<int>(tiles);
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    first += placed;
    if (placed < 8) break;
  }
  return first;
}

__global__ void __launch_bounds__(256)
plan_kernel(const int32_t* lengths, int batch, int seq_cap, int kv_heads, int target, int workers,
            PlanEntry* entries, int32_t* arrivals, int max_entries, int32_t* status) {
  // An entry that does not fit the plan's array would be positions nobody attends: the capacity
  // (make_layout) is sized so that this cannot happen, and if it ever does the launch says so.
  auto overflow = [&]() { atomicOr(status, JPT_ATTN_STATUS_PLAN_OVERFLOW); };
  constexpr int kKeys = 3 * 257;  // tile count; + 257: chunks of slots cut in three or more; + 514: in two, paired
  __shared__ int s_len[kMaxPlanBatch];
  __shared__ int s_first[kMaxPlanBatch];
  __shared__ long long s_total;
  __shared__ int s_chunk, s_entries, s_merges, s_pairs, s_positions, s_sizes;
  __shared__ int s_hist[kKeys];
  __shared__ int s_base[kKeys];
  __shared__ int s_bin_load[kMaxBins];       // tiles dealt to a bin (the workers that take one entry's heads)
  __shared__ int s_bin_rounds[kMaxBins];     // rounds of the bin that are taken
  __shared__ int s_snake_load[kMaxBins];     // the entries a plain snake deal would add to a bin (pairs aside)
  __shared__ int s_snake_max, s_snake_sum;
  __shared__ int s_rank_tiles[kDealtOneByOne];
  __shared__ int s_rank_place[kDealtOneByOne];
  const int tid = threadIdx.x;
  if (tid == 0) {
    s_total = 0;
    s_merges = 0;
    s_positions = 0;
    s_pairs = 0;
    s_sizes = 0;
  }
  for (int i = tid; i < kKeys; i += blockDim.x) s_hist[i] = 0;
  for (int i = tid; i < batch * kv_heads; i += blockDim.x) arrivals[i] = 0;
  for (int i = tid; i < max_entries; i += blockDim.x) entries[i] = PlanEntry{-1, 0, 0, 0, 0, 0, {0, 0}};
  __syncthreads();
  long long mine = 0;
  bool full = false;  // a slot with no room left for the step's token
  for (int b = tid; b < batch; b += blockDim.x) {
    int n = lengths ? lengths[b] : seq_cap;
    full = full || (lengths && n >= seq_cap);
    n = n < 0 ? 0 : (n > seq_cap ? seq_cap : n);
    s_len[b] = n;
    mine += n;
  }
  if (full) atomicOr(status, JPT_ATTN_STATUS_SLOT_FULL);
  atomicAdd(reinterpret_cast<unsigned long long*>(&s_total), static_cast<unsigned long long>(mine));
  __syncthreads();
  if (tid == 0) {
    long long c = (s_total * kv_heads + target - 1) / target;
    const long long floor_c = (seq_cap + kMaxChunksPerSlot - 1) / kMaxChunksPerSlot;
    c = c < floor_c ? floor_c : c;  // at most kMaxChunksPerSlot chunks per slot
    c = (c + kChunkAlign - 1) / kChunkAlign * kChunkAlign;
    s_chunk = c < kChunkAlign ? kChunkAlign : static_cast<int>(c);
  }
  __syncthreads();
  const int chunk = s_chunk;
  auto chunks_of = [&](int b) { return s_len[b] == 0 ? 1 : (s_len[b] + chunk - 1) / chunk; };
  // positions of one chunk of slot b: the slot cut evenly, in whole tiles
  auto chunk_len = [&](int b) {
    const int nc = chunks_of(b);
    return nc == 1 ? s_len[b] : ((s_len[b] + nc - 1) / nc + kTile - 1) / kTile * kTile;
  };
  // Entries of one round of the streaming kernel's walk (see item_index there):
  // entry e of a round goes, head by head, to workers that differ by the
  // workgroups' count between e and e + per_round / 2 - the two groups of one
  // workgroup.  Where that holds, the two chunks of a slot cut in two are put
  // on such a pair of places: the groups then fold the slot through LDS and it
  // needs neither partials nor a merge entry.
  const int per_round = workers / kv_heads;
  const bool pairing = per_round <= kMaxBins && kv_heads * 16 <= workers && (workers / 16) % kv_heads == 0;
  auto paired = [&](int b) { return pairing && chunks_of(b) == 2; };
  // a slot's first partial record: running sum of the chunk counts, 256 slots a pass
  {
    int base = 0;
    for (int b0 = 0; b0 < batch; b0 += static_cast<int>(blockDim.x)) {
      const int b = b0 + tid;
      int total;
      const int before = plan_exclusive_scan(b < batch ? chunks_of(b) : 0, &total);
      if (b < batch) s_first[b] = base + before;
      base += total;
    }
    if (tid == 0) s_entries = base;
  }
  __syncthreads();
  // sort keys: paired slots (one key a slot, by its chunk's tiles), then the
  // chunks of the other cut slots, then whole slots, each longest first
  auto key_of = [&](int count, int kind) {
    const int tiles = (count + kTile - 1) / kTile;
    return (tiles > 256 ? 256 : tiles) + 257 * kind;
  };
  for (int b = tid; b < batch; b += blockDim.x) {
    const int nc = chunks_of(b), cl = chunk_len(b);
    if (paired(b)) {
      atomicAdd(&s_hist[key_of(cl, 2)], 1);
      atomicAdd(&s_pairs, 1);
    } else {
      for (int c = 0; c < nc; ++c) atomicAdd(&s_hist[key_of(min(cl, s_len[b] - c * cl), nc > 1 ? 1 : 0)], 1);
    }
  }
  __syncthreads();
  // how many different sizes the entries that are not a pair's have
  for (int key = tid; key < 2 * 257; key += blockDim.x)
    if (s_hist[key] > 0) atomicAdd(&s_sizes, 1);
  {
    // where each key's entries start, largest key first: thread t of pass i has key kKeys - 1 - (256 i + t)
    int base = 0;
    for (int k0 = 0; k0 < kKeys; k0 += static_cast<int>(blockDim.x)) {
      const int key = kKeys - 1 - (k0 + tid);
      int total;
      const int before = plan_exclusive_scan(key >= 0 ? s_hist[key] : 0, &total);
      if (key >= 0) s_base[key] = base + before;
      base += total;
    }
  }
  __syncthreads();
  const int n_pairs = s_pairs;  // ranks [0, n_pairs) are the paired slots (their keys come first)
  const int half = per_round / 2;
  // The deal.  A bin is the set of workers that take the heads of one entry of a
  // round; bin x has place x of even rounds and place per_round - 1 - x of odd
  // ones (the streaming kernel walks odd rounds backwards).  Pairs fill rounds
  // from the first, places x and x + half.  The other entries are dealt longest
  // first, each to the bin that holds the fewest tiles so far, into that bin's
  // first free round (longest-processing-time dealing, by one wave: see
  // deal_longest_first).  `regular`: the walk has whole entries per round, i.e.
  // bins exist; otherwise entries lie in sorted order.
  const bool regular = per_round >= 1 && per_round <= kMaxBins && workers % 8 == 0 && (workers / 8) % kv_heads == 0;
  const int n_others = s_entries - 2 * n_pairs;
  // (when all of them are equally long there is nothing to even out: they go round the bins)
  const int candidates = regular && s_sizes > 1 ? min(n_others, kDealtOneByOne) : 0;
  auto bin_of_place = [&](int round, int x) { return (round & 1) ? per_round - 1 - x : x; };
  const int max_rounds = regular ? max((max_entries - batch) / per_round, 1) : 0;  // up to `batch` merge entries follow the places
  int one_by_one = 0;  // entries dealt one by one (decided below)
  if (regular) {
    for (int x = tid; x < per_round; x += blockDim.x) {
      s_bin_load[x] = 0;
      s_bin_rounds[x] = 0;
      s_snake_load[x] = 0;
    }
    if (tid == 0) s_snake_max = s_snake_sum = 0;
    __syncthreads();
    // tiles of the entries by rank (a key is a tile count; ranks go down the keys), pairs' loads and rounds
    for (int rank = tid; rank < n_pairs + candidates; rank += blockDim.x) {
      int lo = 0, hi = kKeys - 1;  // the smallest key whose entries start at or before this rank
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (s_base[mid] <= rank) hi = mid; else lo = mid + 1;
      }
      const int tiles = lo % 257;
      if (rank < n_pairs) {  // a pair: both its bins get the chunk's tiles
        const int round = rank / half, x = rank % half;
        atomicAdd(&s_bin_load[bin_of_place(round, x)], tiles);
        atomicAdd(&s_bin_load[bin_of_place(round, x + half)], tiles);
        atomicMax(&s_bin_rounds[bin_of_place(round, x)], round + 1);
        atomicMax(&s_bin_rounds[bin_of_place(round, x + half)], round + 1);
      } else {
        // (and what the plain snake deal - entry i to bin i, 2E-1-i, 2E+i, ... - would give each bin)
        const int i = rank - n_pairs, lap = i / per_round;
        s_rank_tiles[i] = tiles;
        atomicAdd(&s_snake_load[(lap & 1) ? per_round - 1 - i % per_round : i % per_round], tiles);
      }
    }
    __syncthreads();
    // bins the pairs left behind start at the pairs' last full round, so that every round before a pair's is full
    if (pairing && n_pairs > 0)
      for (int x = tid; x < per_round; x += blockDim.x) s_bin_rounds[x] = max(s_bin_rounds[x], n_pairs / half);
    __syncthreads();
    // Is the one-by-one deal worth its time (0.12 us an entry)?  If the heaviest
    // bin of the plain snake deal over the sorted list is within 1/32 of the mean
    // (batches of similar lengths), the snake it is.
    if (candidates > 0) {
      // (one atomic a wave: a hundred of them on one LDS word took 4 us)
      int heaviest = 0, sum = 0;
      for (int x = tid; x < per_round; x += blockDim.x) {
        const int load = s_bin_load[x] + s_snake_load[x];
        heaviest = max(heaviest, load);
        sum += load;
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        heaviest = max(heaviest, __shfl_xor(heaviest, off));
        sum += __shfl_xor(sum, off);
      }
      if ((tid & 63) == 0) {
        atomicMax(&s_snake_max, heaviest);
        atomicAdd(&s_snake_sum, sum);
      }
      __syncthreads();
    }
    const bool uneven = candidates > 0 && static_cast<long long>(s_snake_max) * per_round * 32 > static_cast<long long>(s_snake_sum) * 33;
    one_by_one = uneven ? candidates : 0;
    // Entries beyond the first kDealtOneByOne (only large batches have them, and
    // they are the short ones) go round the bins in snake order, each into its
    // bin's next free round.
    const int laps_after = (n_others - one_by_one + per_round - 1) / per_round;
    if (tid < 64 && one_by_one > 0) {
      const int cap = max(max_rounds - laps_after, 1);
      if (per_round <= 64) {
        const int dealt = deal_longest_first_in_steps(one_by_one, per_round, cap, s_bin_load, s_bin_rounds, s_rank_tiles, s_rank_place);
        deal_longest_first<1>(dealt, one_by_one, per_round, cap, s_bin_load, s_bin_rounds, s_rank_tiles, s_rank_place);
      } else if (per_round <= 256) {
        deal_longest_first<4>(0, one_by_one, per_round, cap, s_bin_load, s_bin_rounds, s_rank_tiles, s_rank_place);
      } else {
        deal_longest_first<16>(0, one_by_one, per_round, cap, s_bin_load, s_bin_rounds, s_rank_tiles, s_rank_place);
      }
    }
    __syncthreads();
  }
  // place of the rank-th entry that is not a pair's
  auto place_of = [&](int rank) {
    if (!regular) return rank;  // no pairs either
    if (rank < one_by_one) return s_rank_place[rank];
    const int i = rank - one_by_one, lap = i / per_round, x = (lap & 1) ? per_round - 1 - i % per_round : i % per_round;
    const int round = s_bin_rounds[x] + lap;  // one entry a bin and lap
    return round * per_round + bin_of_place(round, x);
  };
  int last_place = 0;  // one past the last place this thread wrote
  for (int b = tid; b < batch; b += blockDim.x) {
    const int nc = chunks_of(b), cl = chunk_len(b), first = s_first[b];
    if (paired(b)) {
      const int q = atomicAdd(&s_base[key_of(cl, 2)], 1);
      const int at = (q / half) * per_round + q % half;
      // part = -1: folded with its partner through LDS, no partial record
      if (at + half < max_entries) {
        entries[at] = PlanEntry{b, 0, cl, -1, 2, s_len[b], {0, 0}};
        entries[at + half] = PlanEntry{b, cl, s_len[b] - cl, -1, 2, s_len[b], {0, 0}};
        last_place = max(last_place, at + half + 1);
      } else {
        overflow();
      }
      continue;
    }
    for (int c = 0; c < nc; ++c) {
      const int count = min(cl, s_len[b] - c * cl);
      const int at = place_of(atomicAdd(&s_base[key_of(count, nc > 1 ? 1 : 0)], 1) - n_pairs);
      if (at < max_entries) {
        entries[at] = PlanEntry{b, c * cl, count, first + c, nc, s_len[b], {0, 0}};
        last_place = max(last_place, at + 1);
      } else {
        overflow();
      }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) last_place = max(last_place, __shfl_xor(last_place, off));
  if ((tid & 63) == 0) atomicMax(&s_positions, last_place);
  __syncthreads();
  // merge entries, one for every slot cut in three or more (or in two where there is no pairing), after the last place
  const int n_places = min(s_positions, max_entries);
  for (int b = tid; b < batch; b += blockDim.x) {
    const int nc = chunks_of(b);
    if (nc > 1 && !paired(b)) {
      const int at = n_places + atomicAdd(&s_merges, 1);
      if (at < max_entries) entries[at] = PlanEntry{b, -1, 0, s_first[b], nc, s_len[b], {0, 0}};
      else overflow();
    }
  }
  // The order of a worker's items.  The deal gives every bin its entries longest first;
  // a worker ends sooner when its LONGEST whole slot comes last (its many tiles keep all
  // consumers busy to the end, the new token's tile and the change of item are long past
  // when the last tile lands) and the short ones before it, so the whole-slot entries of
  // a bin are rotated by one: b, ..., a, c for c >= b >= ... >= a.  (Measured on the same
  // tensors: the headline workload's launch 34.3 -> 33.6 us.)  Chunks of cut slots keep
  // their places: pairs must share a round, partials must be parked early.
  if (regular) {
    __threadfence_block();
    __syncthreads();
    const int rounds_used = (n_places + per_round - 1) / per_round;
    for (int x = tid; x < per_round; x += blockDim.x) {
      int first = -1, before = -1;
      PlanEntry longest{};
      for (int r = 0; r < rounds_used; ++r) {
        const int at = r * per_round + bin_of_place(r, x);
        if (at >= n_places) continue;
        const PlanEntry e = entries[at];
        if (e.slot < 0 || e.n_chunks != 1) continue;
        if (first < 0) {
          first = at;
          longest = e;
        } else {
          entries[before] = e;  // every later whole slot moves up one
        }
        before = at;
      }
      if (first >= 0 && before != first) entries[before] = longest;
    }
    // ... and where a workgroup's two bins hold a paired chunk each and, after it, equally many
    // whole slots and nothing else, the pair goes last as well - it is the longest item of both
    // walks - and the whole slots before it shortest first.  (Measured on the same tensors, the
    // plan rewritten from the host: the headline workload's launch 32.70 -> 32.29 us; the whole
    // slots longest first before the pair, or the pair in the middle, gain nothing.)  The pair
    // stays on one round in both walks with every earlier round of the two bins taken, which is
    // what the kernel's fold of the two groups' parts needs.  Only with one round of pairs, and
    // with as many bins as the staging area holds (the slots' lengths are no longer needed: their
    // LDS takes both bins' entries of eight rounds for 32 pairs of bins).
    constexpr int kMostWhole = 8;
    constexpr int kStagedBins = static_cast<int>(sizeof(s_len) / (2 * kMostWhole * sizeof(PlanEntry)));
    if (pairing && n_pairs > 0 && n_pairs <= half && half <= kStagedBins) {
      PlanEntry* const stage = reinterpret_cast<PlanEntry*>(s_len);
      __threadfence_block();
      __syncthreads();
      for (int x = tid; x < half; x += blockDim.x) {
        const int y = x + half;  // round 0: place = bin
        if (rounds_used - 1 > kMostWhole) continue;
        // both bins' entries of the first rounds, asked for all at once (one trip to memory, not one a round)
        const PlanEntry px = entries[x], py = entries[y];
        PlanEntry* const wx = stage + x * 2 * kMostWhole;
        PlanEntry* const wy = wx + kMostWhole;
#pragma unroll
        for (int r = 1; r <= kMostWhole; ++r) {
          const int ax = r * per_round + bin_of_place(r, x), ay = r * per_round + bin_of_place(r, y);
          wx[r - 1] = r < rounds_used && ax < n_places ? entries[ax] : PlanEntry{-1, 0, 0, 0, 0, 0, {0, 0}};
          wy[r - 1] = r < rounds_used && ay < n_places ? entries[ay] : PlanEntry{-1, 0, 0, 0, 0, 0, {0, 0}};
        }
        if (px.slot < 0 || px.n_chunks != 2 || px.part != -1 || py.slot != px.slot || py.n_chunks != 2 || py.part != -1) continue;
        int m = 0;  // whole slots after the pair, in both bins: rounds 1 .. m and nothing behind them
        bool fits = true;
#pragma unroll
        for (int r = 0; r < kMostWhole; ++r) {
          const bool hx = wx[r].slot >= 0, hy = wy[r].slot >= 0;
          if (!hx && !hy) continue;
          fits = fits && hx && hy && r == m && wx[r].n_chunks == 1 && wy[r].n_chunks == 1;
          ++m;
        }
        if (!fits || m == 0) continue;
        // after the rotation above the whole slots stand as w2, w3, ..., wm, w1 (w1 the longest)
        for (int r = 0; r < m; ++r) {
          const int from = r == m - 1 ? m - 1 : m - 2 - r;
          entries[r * per_round + bin_of_place(r, x)] = wx[from];
          entries[r * per_round + bin_of_place(r, y)] = wy[from];
        }
        entries[m * per_round + bin_of_place(m, x)] = px;
        entries[m * per_round + bin_of_place(m, y)] = py;
      }
    }
  }
  __syncthreads();
  if (tid < kHandOutCounters) status[kStateHandOut + tid * kStateHandOutStride] = 0;
  if (tid == 0) {
    status[kStateEntries] = n_places;
    status[kStateArrivalsAt] = static_cast<int32_t>(arrivals - status);
    status[kStateArrivalsCount] = batch * kv_heads;
    status[kStateMerges] = max(min(n_places + s_merges, max_entries) - n_places, 0);
  }
}

}  // namespace

bool attn_fast_supported(const jpt_attn_args& a, AttnMode mode) {
  if (a.force_generic) return false;
  if (a.dim != kD || a.q_dtype != JPT_BF16) return false;
  if (a.kv_dtype != JPT_I8 && a.kv_dtype != JPT_BF16) return false;
  const int rows = a.q_heads / a.kv_heads * a.q_rows;
  if (rows > kMaxRows) return false;
  if (a.batch > kMaxPlanBatch) return false;
  // tiles of 32 positions must stay inside a cache row / a page
  if (mode == kPaged ? a.page_size % kTile != 0 : a.seq % kTile != 0) return false;
  if (a.mask && (a.mask_stride_h != 0 || a.q_rows != 1 || a.mask_dtype != JPT_F32 ||
                 a.mask_stride_b % 4 != 0 || !aligned(a.mask, 16)))
    return false;
  if (a.k_scale && (!aligned(a.k_scale, 16) || !aligned(a.v_scale, 16))) return false;
  // the streaming kernel is built for the caches the path has: int8 codes with scales, bf16 without
  if ((a.kv_dtype == JPT_I8) != (a.k_scale != nullptr)) return false;
  if (!aligned(a.q, 16) || !aligned(a.k, 16) || !aligned(a.v, 16)) return false;
  if (a.new_k && (!aligned(a.new_k, 16) || !aligned(a.new_v, 16))) return false;
  // the new token's raw rows of all heads must fit a tile (its key and value areas together)
  if (a.new_k_raw && (a.kv_heads > 32 || !aligned(a.new_k_raw, 16) || !aligned(a.new_v_raw, 16))) return false;
  return true;
}

int64_t attn_fast_workspace_bytes(const jpt_attn_args& a) {
  const int rows = a.q_heads / a.kv_heads * a.q_rows;
  // shapes the streaming kernel never takes (prefill-shaped queries, huge
  // batches) run on the generic kernel, which uses neither plan nor partials
  if (rows > kMaxRows || a.batch > kMaxPlanBatch) return JPT_ATTN_WS_STATE_BYTES;
  return make_layout(a.batch, a.kv_heads, rows).total;
}

int32_t attn_plan_launch(const jpt_attn_args& a, bool paged, hipStream_t stream) {
  const int rows = a.q_heads / a.kv_heads * a.q_rows;
  if (rows > kMaxRows || a.batch > kMaxPlanBatch) return JPT_OK;  // generic kernel: nothing to plan
  const Layout l = make_layout(a.batch, a.kv_heads, rows);
  JPT_REQUIRE(a.workspace != nullptr && a.workspace_bytes >= l.total,
              "workspace of %lld bytes needed, %lld given", static_cast<long long>(l.total),
              static_cast<long long>(a.workspace_bytes));
  JPT_REQUIRE(aligned(a.workspace, 256), "workspace must be 256-byte aligned");
  char* ws = static_cast<char*>(a.workspace);
  const int cap = paged ? a.max_pages * a.page_size : a.seq;
  JPT_REQUIRE(cap > 0, "sequence capacity must be positive");
  hipLaunchKernelGGL(plan_kernel, dim3(1), dim3(256), 0, stream, a.lengths, a.batch, cap,
                     a.kv_heads, target_items(), persistent_blocks(), reinterpret_cast<PlanEntry*>(ws + l.entries),
                     reinterpret_cast<int32_t*>(ws + l.arrivals), l.max_entries,
                     reinterpret_cast<int32_t*>(ws));
  return launch_status("plan_kernel");
}

int32_t attn_fast_launch(const jpt_attn_args& a, AttnMode mode, hipStream_t stream) {
  const int rep = a.q_heads / a.kv_heads;
  const int rows = rep * a.q_rows;
  const Layout l = make_layout(a.batch, a.kv_heads, rows);
  JPT_REQUIRE(a.workspace != nullptr && a.workspace_bytes >= l.total,
              "workspace of %lld bytes needed, %lld given", static_cast<long long>(l.total),
              static_cast<long long>(a.workspace_bytes));
  JPT_REQUIRE(aligned(a.workspace, 256), "workspace must be 256-byte aligned");
  char* ws = static_cast<char*>(a.workspace);
  FastParams p{};
  p.a = a;
  p.entries = reinterpret_cast<const PlanEntry*>(ws + l.entries);
  p.arrivals = reinterpret_cast<int32_t*>(ws + l.arrivals);
  p.partials = reinterpret_cast<float*>(ws + l.partials);
  p.rows = rows;
  p.rep = rep;
  p.total_items = l.max_entries * a.kv_heads;
  p.status = reinterpret_cast<int32_t*>(ws);
  if (!a.reuse_plan) {
    int32_t st = attn_plan_launch(a, mode == kPaged, stream);
    if (st != JPT_OK) return st;
  }
  int32_t blocks = persistent_blocks();
  if (blocks > p.total_items) blocks = p.total_items;  // total_items is a multiple of 8
  const bool paged = mode == kPaged;
  if (a.kv_dtype == JPT_I8) {
    if (!a.new_k) decode::launch_decode_i8_none(p, paged, blocks, stream);
    else if (!a.new_k_raw) decode::launch_decode_i8_given(p, paged, blocks, stream);
    else if (a.kv_heads <= 16 && !a.new_k_rope) decode::launch_decode_i8_raw(p, paged, blocks, stream);
    else if (a.kv_heads <= 16) decode::launch_decode_i8_raw_rope(p, paged, blocks, stream);
    else if (!a.new_k_rope) decode::launch_decode_i8_raw_wide(p, paged, blocks, stream);
    else decode::launch_decode_i8_raw_wide_rope(p, paged, blocks, stream);
  } else {
    if (!a.new_k) decode::launch_decode_bf16_none(p, paged, blocks, stream);
    else decode::launch_decode_bf16_given(p, paged, blocks, stream);
  }
  return launch_status("attn_decode_kernel");
}

}  // namespace jpt

extern "C" {

int64_t jpt_attn_workspace_bytes(const jpt_attn_args* args) {
  if (args == nullptr || args->batch <= 0 || args->kv_heads <= 0 || args->q_heads <= 0 ||
      args->q_rows <= 0)
    return JPT_ATTN_WS_STATE_BYTES;
  return jpt::attn_fast_workspace_bytes(*args);
}

static int32_t attn_entry(const jpt_attn_args* args, jpt::AttnMode mode, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr, "args is NULL");
  int32_t st = check_attn_args(*args, mode);
  if (st != JPT_OK) return st;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (attn_fast_supported(*args, mode)) return attn_fast_launch(*args, mode, s);
  jpt_attn_args a = *args;
  if (a.new_k_raw) {  // no fused quantiser on this route: quantise first, then attend the codes
    jpt_quant_append_args q{};
    q.new_k = a.new_k_raw;
    q.new_v = a.new_v_raw;
    q.out_k = a.new_k;
    q.out_v = a.new_v;
    q.out_k_scale = a.new_k_scale;
    q.out_v_scale = a.new_v_scale;
    q.batch = a.batch;
    q.heads = a.kv_heads;
    q.dim = a.dim;
    q.seq = 1;
    q.in_dtype = JPT_BF16;
    q.scale_dtype = a.scale_dtype;
    q.scale_heads = a.scale_heads;
    q.rounding = a.new_rounding;
    q.rope = a.new_k_rope;
    st = jpt_kv_append_quant_i8(&q, stream);
    if (st != JPT_OK) return st;
    a.new_k_raw = a.new_v_raw = nullptr;
    a.new_k_rope = nullptr;
    if (attn_fast_supported(a, mode)) return attn_fast_launch(a, mode, s);
  }
  JPT_REQUIRE(!a.new_to_pages, "new_to_pages needs head_dim 128, a bf16 query and page_size a multiple of 32");
  return attn_generic_launch(a, mode, s);
}

int32_t jpt_attn_plan(const jpt_attn_args* args, int32_t paged, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr, "args is NULL");
  JPT_REQUIRE(args->batch > 0 && args->kv_heads > 0 && args->q_heads > 0 && args->q_rows > 0 &&
                  args->q_heads % args->kv_heads == 0, "batch, heads and q_rows must be positive");
  return attn_plan_launch(*args, paged != 0, static_cast<hipStream_t>(stream));
}

// ---- jpt_attn_ragged_static: the workspace is a device array of this library ----
// Device memory that exists from the moment the code object is loaded on a GPU
// (zero-filled then) until the process ends: callers that must not allocate
// need no workspace of their own.  Every GPU holds its own copy at its own
// address.
static __device__ __align__(256) unsigned char scratch[JPT_ATTN_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];  // the array's address on each device, once asked for
std::mutex g_scratch_mutex;

// Address of `scratch` on the current device (NULL and *st set on failure).  The
// array's name is only a handle on the host: the address comes from the runtime,
// once per device, with that device current.
void* static_scratch(int32_t* st) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    *st = jpt::fail(JPT_E_HIP, "hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      *st = jpt::fail(JPT_E_HIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *st = JPT_OK;
  return g_scratch_ptr[dev];
}
}  // namespace

int32_t jpt_attn_ragged_static(const jpt_attn_args* args, void* stream) {
  using namespace jpt;
  JPT_REQUIRE(args != nullptr, "args is NULL");
  JPT_REQUIRE(args->batch > 0 && args->kv_heads > 0 && args->q_heads > 0 && args->q_rows > 0 &&
                  args->q_heads % args->kv_heads == 0, "batch, heads and q_rows must be positive");
  const int64_t need = attn_fast_workspace_bytes(*args);
  JPT_REQUIRE(need <= JPT_ATTN_STATIC_SCRATCH_BYTES,
              "this shape needs a workspace of %lld bytes, the library's own holds %lld: use jpt_attn_ragged "
              "with a workspace of the caller's", static_cast<long long>(need),
              static_cast<long long>(JPT_ATTN_STATIC_SCRATCH_BYTES));
  int32_t st = JPT_OK;
  void* ptr = static_scratch(&st);
  if (ptr == nullptr) return st;
  jpt_attn_args a = *args;
  a.workspace = ptr;
  a.workspace_bytes = JPT_ATTN_STATIC_SCRATCH_BYTES;
  return attn_entry(&a, kRagged, stream);
}

int32_t jpt_attn_status(void* workspace, void* stream, int32_t* status) {
  using namespace jpt;
  JPT_REQUIRE(status != nullptr, "status must not be NULL");
  if (workspace == nullptr) {  // the library's own workspace on the current device
    int32_t st = JPT_OK;
    workspace = static_scratch(&st);
    if (workspace == nullptr) return st;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  // words 0 .. kStateArrivalsCount of the state block
  int32_t head[kStateArrivalsCount + 1] = {0};
  JPT_HIP(hipMemcpyAsync(head, workspace, sizeof(head), hipMemcpyDeviceToHost, s));
  JPT_HIP(hipStreamSynchronize(s));
  const int32_t word = head[kStateStatus];
  if (word != 0) {
    JPT_HIP(hipMemsetAsync(workspace, 0, sizeof(word), s));
    if (word & JPT_ATTN_STATUS_GAVE_UP) {
      // The launch that gave up may have left arrival counts behind, and chunks counted
      // without their merge; a launch reusing the plan would take them for this launch's.
      // Back to what a fresh plan holds.
      int32_t* ws = static_cast<int32_t*>(workspace);
      JPT_HIP(hipMemsetAsync(ws + kStateHandOut, 0, kHandOutCounters * kStateHandOutStride * sizeof(int32_t), s));
      if (head[kStateArrivalsAt] > 0 && head[kStateArrivalsCount] > 0)
        JPT_HIP(hipMemsetAsync(ws + head[kStateArrivalsAt], 0, static_cast<size_t>(head[kStateArrivalsCount]) * sizeof(int32_t), s));
    }
    JPT_HIP(hipStreamSynchronize(s));
  }
  *status = word;
  return JPT_OK;
}

int32_t jpt_attn_ragged(const jpt_attn_args* args, void* stream) { return attn_entry(args, jpt::kRagged, stream); }
int32_t jpt_attn_dense(const jpt_attn_args* args, void* stream) { return attn_entry(args, jpt::kDense, stream); }
int32_t jpt_attn_paged(const jpt_attn_args* args, void* stream) { return attn_entry(args, jpt::kPaged, stream); }

}  // extern "C"
