// Dispatch plan of the varlen attention: which (request, query tile, head) unit each block of the grid takes.
//
// Host code only.  The hardware hands the blocks of a grid out in index order, block i to XCD i mod 8, each to
// the first workgroup slot that falls free there: list scheduling in the order of the block indices.  With two
// or three units per slot the order decides the makespan.  Longest unit first pairs well but then stacks the
// remaining short units on top of finished pairs; packing the units into one bin per slot first (first-fit
// decreasing under the smallest capacity that needs no more bins than slots) and issuing them in the order of
// their start times inside that packing brings the makespan close to the mean load.  A wrong cost model costs
// time, never correctness: every unit appears exactly once whatever the order.
//
// Units of one KV head stay on the XCDs that share that head's rows in L2, as in the kernel's own index map.
#include <algorithm>
#include <exception>
#include <numeric>
#include <queue>
#include <vector>

#include "attn_common.h"

namespace acache {
namespace {

struct Unit {
  int32_t b, tile, head;
  int32_t cost;
};

// Run time of a unit in hundredths of the time of one full 64-key tile: a fixed part (lookup, query load,
// epilogue) plus one term per key tile, cheaper when at most 64 / 32 query rows are live and two waves share
// a row block.
inline int32_t unit_cost(int rows, int kv_len) {
  const int kt = std::min(kv_len / 64 + (kv_len % 64 != 0), 1 << 20);  // beyond that only the order matters
  const int per_tile = rows > 64 ? 100 : (rows > 32 ? 85 : 60);
  return 290 + kt * per_tile;
}

// Order in which list scheduling on `slots` machines reproduces a tight packing of `costs`.
void plan_order(const std::vector<int32_t> &costs, int slots, std::vector<int32_t> &order) {
  const int n = (int)costs.size();
  order.resize(n);
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int a, int c) { return costs[a] > costs[c]; });
  if (n <= slots || n > 16 * slots) return;  // everything starts at once / long lists: longest first is tight

  // longest-first list scheduling: the packing to beat, and the upper end of the capacity search
  std::vector<int32_t> bin_of(n), best_bin(n);
  int64_t hi = 0, total = 0;
  {
    typedef std::pair<int64_t, int> Slot;
    std::priority_queue<Slot, std::vector<Slot>, std::greater<Slot>> free_at;
    for (int s = 0; s < slots; ++s) free_at.push(Slot(0, s));
    for (int i : order) {
      Slot s = free_at.top();
      free_at.pop();
      best_bin[i] = s.second;
      s.first += costs[i];
      hi = std::max(hi, s.first);
      total += costs[i];
      free_at.push(s);
    }
  }
  int64_t lo = std::max<int64_t>((total + slots - 1) / slots, costs[order[0]]);
  std::vector<int64_t> load(slots);
  for (int it = 0; it < 16 && lo < hi; ++it) {
    const int64_t cap = (lo + hi) / 2;
    int used = 0;
    bool fits = true;
    for (int i : order) {
      int s = 0;
      while (s < used && load[s] + costs[i] > cap) ++s;
      if (s == used) {
        if (used == slots) { fits = false; break; }
        load[used++] = 0;
      }
      load[s] += costs[i];
      bin_of[i] = s;
    }
    if (fits) { hi = cap; best_bin = bin_of; }
    else lo = cap + 1;
  }
  // Start time of every unit inside its bin, then issue by start time.  A bin runs its units shortest first:
  // measured on configs of two to three units per slot that order is about 1 % faster than longest first (the
  // long units then run last, when neighbours on the same CU have already finished).
  std::vector<int64_t> start(n), filled(slots, 0);
  for (auto it = order.rbegin(); it != order.rend(); ++it) {
    start[*it] = filled[best_bin[*it]];
    filled[best_bin[*it]] += costs[*it];
  }
  // units that start together (the first of every bin above all) go out longest first: the dispatch of a
  // round takes a few microseconds, and the long ones should have them (about 1 us on configs[3])
  std::stable_sort(order.begin(), order.end(), [&](int a, int c) {
    return start[a] != start[c] ? start[a] < start[c] : costs[a] > costs[c];
  });
}

}  // namespace
}  // namespace acache

using namespace acache;

static int64_t make_plan(const int32_t *cu_q_host, const int32_t *cu_k_host, int32_t B, int32_t H, int32_t H_kv,
                         int32_t slots_per_xcd, int32_t *plan_host, int64_t capacity_blocks) {
  if (B < 0 || H <= 0 || H_kv <= 0 || H % H_kv != 0 || H >= (1 << 11))
    return fail(ACACHE_E_SHAPE, "varlen_attn_plan: bad sizes (B=%d, H=%d, H_kv=%d)", B, H, H_kv);
  if (B > 0 && (!cu_q_host || !cu_k_host)) return fail(ACACHE_E_NULL, "varlen_attn_plan: NULL pointer");
  if (slots_per_xcd <= 0) slots_per_xcd = 64;  // 32 CUs per XCD, two workgroups each
  constexpr int BM = 128;
  const int group = H / H_kv;

  // the query tiles of the batch
  struct Tile { int32_t b, t, cost; };
  std::vector<Tile> tiles;
  for (int b = 0; b < B; ++b) {
    const int q_len = cu_q_host[b + 1] - cu_q_host[b], kv_len = cu_k_host[b + 1] - cu_k_host[b];
    if (q_len < 0 || kv_len < 0) return fail(ACACHE_E_SHAPE, "varlen_attn_plan: prefix sums must not decrease");
    const int n = (q_len + BM - 1) / BM;
    if (n >= (1 << 20)) return fail(ACACHE_E_SHAPE, "varlen_attn_plan: request %d is too long", b);
    for (int t = 0; t < n; ++t) tiles.push_back(Tile{b, t, unit_cost(std::min(BM, q_len - t * BM), kv_len)});
  }
  // Every unit's XCD.  KV head j owns the interval [8 j / H_kv, 8 (j + 1) / H_kv) of the XCD axis and its
  // query tiles (each with all heads of the group, which read the same K/V rows) are dealt to the XCDs that
  // the interval overlaps, in proportion to the overlap, longest tile first:
  //   H_kv a multiple of 8: the interval lies inside one XCD, which holds all tiles of the head;
  //   H_kv = 1, 2 or 4: 8 / H_kv XCDs share the head equally;
  //   otherwise (say 12 KV heads): a head's rows are read through at most two L2s and every XCD gets
  //     the same amount of work.
  std::vector<Unit> units[8];
  std::vector<int32_t> by_cost(tiles.size());
  std::iota(by_cost.begin(), by_cost.end(), 0);
  std::stable_sort(by_cost.begin(), by_cost.end(), [&](int a, int c) { return tiles[a].cost > tiles[c].cost; });
  for (int kvh = 0; kvh < H_kv; ++kvh) {
    // overlaps in units of 1 / H_kv of an XCD
    const int lo = 8 * kvh, hi = 8 * (kvh + 1);
    int64_t weight[8], work[8];
    for (int x = 0; x < 8; ++x) {
      weight[x] = std::max(0, std::min(hi, H_kv * (x + 1)) - std::max(lo, H_kv * x));
      work[x] = 0;
    }
    for (int i : by_cost) {
      int best = -1;
      for (int x = 0; x < 8; ++x) {
        if (weight[x] == 0) continue;
        // (work[x] + cost) / weight[x] < (work[best] + cost) / weight[best]
        if (best < 0 || (work[x] + tiles[i].cost) * weight[best] < (work[best] + tiles[i].cost) * weight[x]) best = x;
      }
      work[best] += tiles[i].cost;
      for (int hg = 0; hg < group; ++hg)
        units[best].push_back(Unit{tiles[i].b, tiles[i].t, kvh * group + hg, tiles[i].cost});
    }
  }
  size_t longest = 0;
  for (int x = 0; x < 8; ++x) longest = std::max(longest, units[x].size());
  const int64_t blocks = 8 * (int64_t)longest;
  if (!plan_host) return blocks;
  if (capacity_blocks < blocks)
    return fail(ACACHE_E_SHAPE, "varlen_attn_plan: the plan needs %lld blocks, the buffer holds %lld", (long long)blocks,
                (long long)capacity_blocks);
  for (int64_t i = 0; i < 2 * blocks; i += 2) { plan_host[i] = -1; plan_host[i + 1] = 0; }
  std::vector<int32_t> costs, order, first_costs, first_order;
  for (int x = 0; x < 8; ++x) {
    costs.resize(units[x].size());
    for (size_t i = 0; i < costs.size(); ++i) costs[i] = units[x][i].cost;
    if (x > 0 && costs == first_costs) order = first_order;  // the usual case: every XCD holds the same mix
    else plan_order(costs, slots_per_xcd, order);
    if (x == 0) { first_costs = costs; first_order = order; }
    for (size_t r = 0; r < order.size(); ++r) {
      const Unit &u = units[x][order[r]];
      plan_host[2 * (8 * r + x)] = u.b;
      plan_host[2 * (8 * r + x) + 1] = (int32_t)((uint32_t)u.tile | ((uint32_t)u.head << 20));
    }
  }
  return blocks;
}

extern "C" int64_t acache_varlen_attn_plan(const int32_t *cu_q_host, const int32_t *cu_k_host, int32_t B, int32_t H,
                                           int32_t H_kv, int32_t slots_per_xcd, int32_t *plan_host,
                                           int64_t capacity_blocks) {
  try {
    return make_plan(cu_q_host, cu_k_host, B, H, H_kv, slots_per_xcd, plan_host, capacity_blocks);
  } catch (const std::exception &e) {  // the planner's own vectors: nothing may unwind through the C boundary
    return fail(ACACHE_E_SHAPE, "varlen_attn_plan: %s", e.what());
  }
}
