"""The decode-attention plan, read back from the workspace.  The streaming
kernel trusts the planner's records (it never checks one), so the properties
it relies on are checked here on the planner's own output: whatever the
lengths, the work entries cover every position of every slot exactly once;
the two chunks of a slot cut in two sit on places that one workgroup's two
groups walk in the same round, with an item of both on every earlier round; every
other cut slot has consecutive partial records and one merge entry that names them
all.  The deal itself is pinned too: a host model of the planner's rule - entries
that are not a pair's go, longest first, to the bin with the fewest tiles so far (or
round the bins in snake order when that is even enough already), every bin's whole
slots are then walked with the longest last, and a workgroup's pair goes behind
its two bins' whole slots where both hold equally many and nothing else - must put
the same number of tiles on every place as the plan read back from the device.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

TILE = 32
STATE_BYTES = 64 * 1024
ENTRY_INTS = 8  # slot, start, count, part, n_chunks, slot_len, unused, unused


def workers():
  cus = torch.cuda.get_device_properties(0).multi_processor_count
  return (cus * 2 + 7) // 8 * 8


def read_plan(plan):
  """(work places incl. unused ones, merge entries) as numpy int32 [n, 8]."""
  torch.cuda.synchronize()
  raw = plan.workspace.buf.cpu().numpy()
  state = raw[:STATE_BYTES].view(np.int32)
  n_places, n_merges = int(state[2]), int(state[3])
  entries = raw[STATE_BYTES:STATE_BYTES + (n_places + n_merges) * ENTRY_INTS * 4].view(np.int32).reshape(-1, ENTRY_INTS)
  return entries[:n_places], entries[n_places:]


DEALT_ONE_BY_ONE = 512  # entries the planner deals to the lightest bin; later ones go round the bins


def model_deal(places, batch, kv_heads):
  """Tiles the planner's rule puts on every place (-1: nobody), from the plan's own
  entries: pairs stay where they are; the other entries, in sort order (chunks of
  slots cut in three or more before whole slots, each longest first), are dealt
  as plan_kernel deals them."""
  w = workers()
  per_round, half = w // kv_heads, w // kv_heads // 2
  tiles_of = lambda count: min((count + TILE - 1) // TILE, 256)
  is_pair = lambda e: e[0] >= 0 and e[3] == -1 and e[4] == 2
  bin_of = lambda rnd, x: per_round - 1 - x if rnd & 1 else x
  load, rounds = [0] * per_round, [0] * per_round
  out = [-1] * len(places)
  # pairs: found where the plan has them, which is where the deal put them - round by round from
  # the first - unless the last pass moved them behind their bins' whole slots (one round of pairs
  # only: then they were dealt to round 0)
  members = [(at, e) for at, e in enumerate(places) if is_pair(e)]
  n_pairs = len(members) // 2
  pair_of_bin = {}
  for at, e in members:
    rnd, x = divmod(at, per_round)
    b = bin_of(rnd, x)
    if n_pairs <= half:
      rnd = 0
    partner = next(e2 for _, e2 in members if e2[0] == e[0] and e2[1] != e[1])
    first = e if e[1] == 0 else partner  # both bins are charged the first chunk's tiles
    load[b] += tiles_of(first[2])
    rounds[b] = max(rounds[b], rnd + 1)
    out[rnd * per_round + bin_of(rnd, b)] = tiles_of(e[2])
    pair_of_bin[b] = e[0]
  if n_pairs:
    rounds = [max(r, n_pairs // half) for r in rounds]
  others = sorted(((1 if e[4] > 1 else 0, tiles_of(e[2])) for e in places if e[0] >= 0 and not is_pair(e)), reverse=True)
  candidates = min(len(others), DEALT_ONE_BY_ONE) if len(set(others)) > 1 else 0
  snake = list(load)
  for i in range(candidates):
    lap, x = divmod(i, per_round)
    snake[per_round - 1 - x if lap & 1 else x] += others[i][1]
  one_by_one = candidates if candidates and max(snake) * per_round * 32 > sum(snake) * 33 else 0
  target = w * 5 // 4
  extra = (target + kv_heads - 1) // kv_heads + 1
  max_entries = (2 * batch + 2 * extra + 3 * (w // kv_heads + 8) + 7) // 8 * 8
  max_rounds = max((max_entries - batch) // per_round, 1)
  cap = max(max_rounds - (len(others) - one_by_one + per_round - 1) // per_round, 1)
  whole = [False] * len(places)  # places that hold a whole slot (not a chunk of a cut one)
  for kind, t in others[:one_by_one]:
    x = min((b for b in range(per_round) if rounds[b] < cap), key=lambda b: (load[b], b))
    at = rounds[x] * per_round + bin_of(rounds[x], x)
    out[at], whole[at] = t, kind == 0
    load[x] += t
    rounds[x] += 1
  for i, (kind, t) in enumerate(others[one_by_one:]):
    lap, x = divmod(i, per_round)
    x = per_round - 1 - x if lap & 1 else x
    rnd = rounds[x] + lap
    at = rnd * per_round + bin_of(rnd, x)
    out[at], whole[at] = t, kind == 0
  # the whole slots of a bin, dealt longest first, are walked with the longest last
  for x in range(per_round):
    mine = [rnd * per_round + bin_of(rnd, x) for rnd in range((len(places) + per_round - 1) // per_round)]
    mine = [at for at in mine if at < len(places) and whole[at]]
    tiles = [out[at] for at in mine]
    for at, t in zip(mine, tiles[1:] + tiles[:1]):
      out[at] = t
  # a workgroup's two bins that hold a paired chunk each and then equally many whole slots, nothing
  # else: the pair goes last in both, the whole slots before it shortest first
  n_rounds = (len(places) + per_round - 1) // per_round
  if 0 < n_pairs <= half <= 32 and n_rounds - 1 <= 8:  # (the planner stages eight rounds behind the pair's, for 32 pairs of bins)
    for x in range(half):
      y = x + half
      if x not in pair_of_bin or pair_of_bin.get(y) != pair_of_bin[x]:
        continue
      walk = lambda b: [r * per_round + bin_of(r, b) for r in range(n_rounds) if r * per_round + bin_of(r, b) < len(places)]
      wx, wy = walk(x), walk(y)
      held = lambda w: [r for r, at in enumerate(w) if out[at] >= 0]
      hx, hy = held(wx), held(wy)
      m = len(hx) - 1
      if hx != hy or hx != list(range(m + 1)) or not 1 <= m <= 8 or not all(whole[at] for w in (wx, wy) for at in w[1:m + 1]):
        continue
      for w in (wx, wy):
        pair_tiles, tiles = out[w[0]], [out[at] for at in w[1:m + 1]]
        new = [tiles[m - 1] if r == m - 1 else tiles[m - 2 - r] for r in range(m)] + [pair_tiles]
        for at, t in zip(w[:m + 1], new):
          out[at] = t
  return out


def check_plan(lengths, kv_heads, seq):
  from jetstream_pt_amd import attention_kernel as ak
  batch = len(lengths)
  dl = torch.tensor(lengths, dtype=torch.int32, device=DEV)
  plan = ak.DecodePlan(dl, batch, kv_heads * 4, kv_heads, seq=seq)
  places, merges = read_plan(plan)
  clipped = [min(max(n, 0), seq) for n in lengths]
  per_round = workers() // kv_heads
  pairing = kv_heads * 16 <= workers() and (workers() // 16) % kv_heads == 0
  covered = [np.zeros(n, dtype=np.int32) for n in clipped]
  chunks = [[] for _ in range(batch)]
  for at, (slot, start, count, part, n_chunks, slot_len, _, _) in enumerate(places):
    if slot < 0:
      continue  # a place nobody was put on
    assert 0 <= slot < batch and slot_len == clipped[slot]
    assert start >= 0 and start % TILE == 0 and start + count <= slot_len
    assert count > 0 or slot_len == 0
    covered[slot][start:start + count] += 1
    chunks[slot].append((start, count, part, n_chunks, at))
  merge_of = {}
  for slot, start, count, part, n_chunks, slot_len, _, _ in merges:
    assert start == -1 and slot not in merge_of
    merge_of[slot] = (part, n_chunks)
  used_parts = set()
  n_pairs = 0
  for slot in range(batch):
    assert np.all(covered[slot] == 1), slot
    cs = sorted(chunks[slot])
    assert len(cs) >= 1  # an empty slot still has an item that writes its output
    assert all(c[3] == len(cs) for c in cs)
    if len(cs) == 1:
      assert slot not in merge_of
      continue
    assert all(c[1] >= 1 for c in cs)
    if pairing and len(cs) == 2:
      # folded through LDS by the two groups of one workgroup: same round, half a round apart, no partials
      n_pairs += 1
      (s0, c0, p0, _, at0), (s1, c1, p1, _, at1) = cs
      assert p0 == -1 and p1 == -1 and slot not in merge_of
      bin_of = lambda at: at % per_round if (at // per_round) % 2 == 0 else per_round - 1 - at % per_round
      rnd, b0, b1 = at0 // per_round, bin_of(at0), bin_of(at1)
      assert at1 // per_round == rnd and abs(b1 - b0) == per_round // 2  # the two groups of one workgroup
      # the item has the same number in both groups' walks: both bins have an item on every round before
      for b in (b0, b1):
        for r in range(rnd):
          assert places[r * per_round + (b if r % 2 == 0 else per_round - 1 - b), 0] >= 0
      continue
    part0, n = merge_of[slot]
    assert n == len(cs)
    assert [c[2] for c in cs] == list(range(part0, part0 + n)), "partials numbered along the slot"
    assert not used_parts & set(range(part0, part0 + n))
    used_parts |= set(range(part0, part0 + n))
  assert len(merge_of) == sum(1 for s in range(batch) if len(chunks[s]) > 1) - n_pairs
  if 1 <= per_round <= 1024 and workers() % 8 == 0 and (workers() // 8) % kv_heads == 0:
    got = [min((int(e[2]) + TILE - 1) // TILE, 256) if e[0] >= 0 else -1 for e in places]
    assert got == model_deal([[int(v) for v in e] for e in places], batch, kv_heads), "the deal is not the model's"
  return n_pairs, len(merge_of)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_plan_covers_every_position_once_lognormal(seed):
  rng = np.random.default_rng(seed)
  lengths = [int(x) for x in np.clip(np.round(np.exp(np.log(400) + rng.standard_normal(128))), 16, 8192)]
  n_pairs, n_merges = check_plan(lengths, 8, 8192)
  assert n_pairs + n_merges > 0  # the distribution's tail is cut


@pytest.mark.parametrize("lengths,kv_heads,seq", [
    ([0], 1, 64),                       # one empty slot
    ([1], 1, 64),
    ([64], 8, 64),
    ([4096], 1, 4096),                  # one slot in many chunks
    ([4096, 3000, 1, 0, 17, 2049] * 4, 8, 4096),
    ([0] * 40, 4, 256),                 # nothing but empty slots
    ([33] * 700, 2, 64),                # many short slots, several rounds
    ([5000, -3, 70], 2, 2048),          # out-of-range lengths are clipped
    ([1024] * 8, 32, 1024),             # every slot cut in two: pairs only
    ([1024] * 8 + [100] * 3, 32, 1024), # pairs, and whole slots in the places they leave
    ([2048] * 40, 8, 2048),             # more pairs than one round holds
    ([1024] * 4096, 2, 1024),           # the largest batch the planner takes
    ([700] * 5, 3, 1024),               # a head count the workers do not divide by: no pairing
    ([0] * 100 + [3000, 17, 900], 8, 4096),          # many entries of no tiles: one bin takes them all
    (list(range(1, 2048, 7)), 8, 2048),               # evenly spread lengths
    ([16] * 300 + [4000] * 30 + [100] * 90, 8, 4096), # short entries on uneven bins: few a step, then one by one
    (list(range(5, 1500, 11)), 16, 2048),             # 32 bins
    (list(range(5, 900, 3)), 4, 1024),                # 128 bins: two a lane
])
def test_plan_covers_every_position_once_edge_cases(lengths, kv_heads, seq):
  check_plan(lengths, kv_heads, seq)
