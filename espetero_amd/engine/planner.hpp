// Attention tile planner: which (tree, row tile, cached-key range) units a pass
// runs and how split ranges merge. Host code, no device calls.
//
// Two rules share one implementation:
//   * reference rule  -- PlanOptions::reference(): the records are identical,
//     field for field, to what the reference's planner emits
//     (plan_tiles, src/model/impl/forest.h:1378-1433 without the sparse branch;
//      g4_plan_tiles, src/model/impl/gemma.h:77-116): 8-row tiles, every tree
//     gets the same split budget 256 / (groups * tiles), 32-key boundaries.
//   * balanced rule   -- PlanOptions::mi355x(): one chunk size for the whole
//     pass, derived from the pass's total key count, so every workgroup
//     streams about the same number of KV bytes whatever its sequence length
//     (the reference rule gives a 512-token and an 8192-token sequence the same
//     number of splits, which leaves most of 256 CUs idle while the longest
//     sequence finishes). Boundaries stay on page multiples.
// Only the algebra is contractual: the cached ranges of a tile group partition
// [k0, P), its batch ranges partition the batch keys from b0 on (one range - the
// last part's - unless the balanced rule cuts the batch keys too: `last` = e + 2
// ends a part's batch keys at row e of the tree, `last` = 1 leaves them open),
// parts merge in range order.
#pragma once

#include <algorithm>
#include <climits>
#include <cstdint>
#include <functional>
#include <queue>
#include <vector>

#include "../../include/espetero_attn.h"

namespace espetero::engine {

struct PlanOptions {
  int rows_per_tile = 8;    // query rows per tile
  int groups_target = 256;  // workgroups a few-tile pass is split up to
  int split = 512;          // reference rule: largest chunk a split tile is sized to; 0: never split
  int min_chunk = 32;       // fewest cached keys a split tile takes
  int granule = 32;         // split boundaries are multiples of this
  int max_splits = 64;      // parts per tile group
  int min_span = 64;        // shorter cached ranges are not split
  bool balanced = false;    // false: reference rule; true: equal keys per workgroup
  // Balanced rule on the tiled kernel (rows_per_tile > 32): groups_target is the number of workgroups
  // resident at once, and the chunk is the one whose workgroups, handed to those slots in the kernel's
  // dispatch order, finish earliest. item_steps: what a workgroup costs beside its key steps (set-up,
  // epilogue), in steps of `granule` keys.
  int item_steps = 0;
  int part_steps = 0;  // what a split part costs on top: its partial record written, read again and merged
  // Tiled kernel, balanced rule: a tile's batch keys are cut like its cached keys (a pass of fewer workgroups than
  // slots - one prompt's first chunk - is otherwise as long as its last tile, which scans every row of the chunk).
  // Off in mi355x(): measured on one 2048-row first chunk, 16 heads, the attention kernel gets shorter (head dim 256:
  // 80 -> 72 us, head dim 128: 42.5 -> 36.4 us) and the step with the merge of the partial records behind it does not
  // (79.5 -> 82.9 us, 42.0 -> 43.3 us).
  bool cut_batch = false;

  static PlanOptions reference() { return PlanOptions{}; }
  // rows: query rows per tile (decode 1..8 -> 8-row budget is irrelevant; prefill 64/128).
  static PlanOptions mi355x(int rows, int workgroups) {
    PlanOptions o;
    o.rows_per_tile = rows;
    o.groups_target = workgroups;
    o.split = 0;
    o.min_chunk = 64;
    o.granule = 32;
    o.max_splits = 256;
    o.min_span = 128;
    o.balanced = true;
    if (rows > 32) {  // tiled kernel: 64-key steps, and a split part must amortise its partial record
      o.granule = 64;
      o.min_chunk = 512;
      o.min_span = 1024;
      o.item_steps = 6;
      o.part_steps = 6;  // (8 before the merge of tiled passes got its own instantiation: config 3's four chunks 738.9 -> 736.2 us)
    }
    return o;
  }
};

struct AttnPlan {
  std::vector<esp_tree> trees;
  std::vector<esp_tile> tiles;
  std::vector<esp_combine> combine;
  int parts = 0;
  int rows_per_tile = 8;
};

// groups: workgroups per tile (KV heads, or KV heads x head splits).
// window > 0 needs pos (4 ints per row, pos[4 * row] = position).
inline void plan_tiles(AttnPlan& A, int groups, int window, const int32_t* pos, const PlanOptions& o) {
  A.tiles.clear();
  A.combine.clear();
  A.parts = 0;
  A.rows_per_tile = o.rows_per_tile;
  const int R = o.rows_per_tile;
  struct RowTile {
    int tree, r, k0, b0, span;
    int batch;  // batch keys the tile scans after its cached range (balanced rule: part of its work)
  };
  std::vector<RowTile> rts;
  long long total_span = 0;
  for (int ti = 0; ti < int(A.trees.size()); ++ti) {
    const esp_tree& t = A.trees[size_t(ti)];
    for (int r = 0; r < t.M; r += R) {
      int k0 = 0, b0 = 0;
      if (window > 0) {
        // The tile's earliest row bounds what any of its rows can still see:
        // cached key j sits at position j, root row j at P + j (gemma.h:88-94).
        int minpos = INT32_MAX;
        for (int i = r; i < std::min(t.M, r + R); ++i) minpos = std::min(minpos, pos[4 * (t.base + i)]);
        k0 = std::clamp(minpos - window + 1, 0, t.P);
        b0 = std::max(0, minpos - window + 1 - t.P);
      }
      // A causal tile scans the batch rows up to its own last row; one split part takes them all.
      const int batch = o.balanced ? std::max(0, std::min(t.M, r + R) - b0) : 0;
      rts.push_back({ti, r, k0, b0, t.P - k0, batch});
      total_span += t.P - k0 + batch;
    }
  }
  const int n_tiles = int(rts.size());
  int budget = std::max(1, o.groups_target / std::max(1, groups * n_tiles));
  int chunk_all = 0;  // balanced rule: keys per workgroup
  auto cuttable = [&](const RowTile& rt) { return rt.span + (o.cut_batch ? rt.batch : 0) >= o.min_span; };
  auto parts_of = [&](const RowTile& rt, long long chunk) {
    return cuttable(rt) ? std::min<long long>((rt.span + rt.batch + chunk - 1) / chunk, o.max_splits) : 1;
  };
  std::vector<int> ns_of;  // tiled kernel: parts of every row tile, once chosen
  if (o.balanced && o.item_steps > 0) {
    // Tiled kernel. A pass is tiles x groups workgroups of unequal length (a causal chunk's later tiles
    // see more keys) on groups_target slots; the hardware hands the next workgroup to the first free slot,
    // in the kernel's dispatch order (tile records last to first, the groups of a record together). The
    // time of the pass is when the last slot finishes, so the split is chosen by running that hand-out
    // for every candidate: a few long workgroups leave slots idle at the end, many short ones pay their
    // set-up, partial records and merge more often.
    const int slots = std::max(1, o.groups_target);
    long long max_work = 1;
    for (const RowTile& rt : rts) max_work = std::max<long long>(max_work, rt.span + rt.batch);
    const long long c_lo = std::max(1, o.min_chunk / o.granule), c_hi = (max_work + o.granule - 1) / o.granule;
    auto finish_time = [&](const std::vector<int>& ns_v) {
      std::priority_queue<long long, std::vector<long long>, std::greater<long long>> free_at;
      for (int i = 0; i < slots; ++i) free_at.push(0);
      long long end = 0;
      for (int i = n_tiles - 1; i >= 0; --i) {
        const RowTile& rt = rts[size_t(i)];
        const long long work = rt.span + rt.batch;
        const long long ns = ns_v[size_t(i)];
        const long long per = (work + ns - 1) / ns;
        for (long long p = ns - 1; p >= 0; --p) {  // a record's parts in reverse too
          const long long keys = std::min(per, work - p * per);
          const long long cost = o.item_steps + (ns > 1 ? o.part_steps : 0) + (std::max<long long>(keys, 0) + o.granule - 1) / o.granule;
          for (int g = 0; g < groups; ++g) {
            const long long t = free_at.top() + cost;
            free_at.pop();
            free_at.push(t);
            end = std::max(end, t);
          }
        }
      }
      return end;
    };
    std::vector<int> cand(size_t(n_tiles), 1);
    ns_of = cand;
    long long best = finish_time(cand);
    const long long items = 1LL * n_tiles * groups, rounds = items / slots;
    // Fewer workgroups than slots (with cut_batch: no more than slots): one chunk for every tile, the chunks that cut the longest tile into 2 .. 8
    // parts (fewer parts first: ties keep them). With a round or more of whole workgroups such a split was
    // measured slower than none (two workgroups share a compute unit and the older one is served first, so the
    // slots are less alike than this hand-out takes them to be).
    for (int parts = 2; parts <= 8 && (rounds == 0 || (o.cut_batch && items <= slots)); ++parts) {
      const long long c = std::max(c_lo, (c_hi + parts - 1) / parts) * o.granule;
      for (int i = 0; i < n_tiles; ++i) cand[size_t(i)] = int(parts_of(rts[size_t(i)], c));
      const long long t = finish_time(cand);
      if (t < best) best = t, ns_of = cand;
    }
    // A round or more, and some workgroups over (640 on 512 slots): those would run nearly alone at the end.
    // Only the tiles with the least work are split, just enough of them that the whole ones fill whole rounds,
    // and their parts fill the slots beside and behind those; the tile dispatched last gets the most parts, so
    // that the pass ends on short workgroups. (Measured on 2048-row causal chunks over 2048 .. 6144 cached keys:
    // 5 to 8 % faster than unsplit; splitting fewer tiles than that, so that some whole ones still spill into
    // another round, was 3 to 6 % slower.)
    if (rounds >= 1 && items % slots != 0) {
      std::vector<int> order(size_t(n_tiles), 0);  // tiles by work, least first (ties: dispatched last first)
      for (int i = 0; i < n_tiles; ++i) order[size_t(i)] = i;
      std::stable_sort(order.begin(), order.end(), [&](int x, int y) {
        return rts[size_t(x)].span + rts[size_t(x)].batch < rts[size_t(y)].span + rts[size_t(y)].batch;
      });
      const int n_tail = int((items - rounds * slots + groups - 1) / groups);
      for (int most = 3; most <= 6; ++most) {  // parts of the tile with the least work; the others one fewer each, down to 2
        std::fill(cand.begin(), cand.end(), 1);
        bool any = false;
        for (int j = 0; j < n_tail; ++j) {
          const RowTile& rt = rts[size_t(order[size_t(j)])];
          const long long cap = std::min<long long>((rt.span + rt.batch) / std::max(1, o.min_chunk), o.max_splits);
          const int want = std::max(2, most - j);
          const int ns = rt.span >= o.min_span ? int(std::min<long long>(want, cap)) : 1;
          cand[size_t(order[size_t(j)])] = std::max(1, ns);
          any = any || ns > 1;
        }
        if (!any) break;
        const long long t = finish_time(cand);
        if (t < best) best = t, ns_of = cand;
      }
    }
  } else if (o.balanced && budget > 1) {
    // The smallest chunk (a granule multiple) whose tile count fits the target: a pass
    // that overshoots the resident workgroup count by a few tiles pays a whole extra round.
    const long long cap = std::max(1, o.groups_target / std::max(1, groups));
    auto tiles_at = [&](long long chunk) {
      long long n = 0;
      for (const RowTile& rt : rts) n += parts_of(rt, chunk);
      return n;
    };
    long long lo = std::max(1, o.min_chunk / o.granule), hi = std::max<long long>(lo, (total_span + o.granule - 1) / o.granule + 1);
    while (lo < hi) {
      const long long mid = (lo + hi) / 2;
      if (tiles_at(mid * o.granule) <= cap) hi = mid;
      else lo = mid + 1;
    }
    chunk_all = int(lo * o.granule);
  }
  for (const RowTile& rt : rts) {
    const esp_tree& t = A.trees[size_t(rt.tree)];
    const int span = rt.span;
    int ns = 1;
    if (!ns_of.empty()) {
      ns = ns_of[size_t(&rt - rts.data())];
    } else if (budget > 1 && span >= o.min_span) {
      if (o.balanced) {
        ns = std::min((span + rt.batch + chunk_all - 1) / chunk_all, o.max_splits);
      } else if (o.split > 0) {
        const int chunk =
            std::max(std::max(32, o.min_chunk),
                     std::min(o.split, ((span + budget - 1) / budget + o.granule - 1) / o.granule * o.granule));
        ns = std::min({(span + chunk - 1) / chunk, budget, o.max_splits});
      }
    }
    // Balanced rule: the tile carries its tree's block-list offset (pad = table + 1), which
    // saves the kernels a dependent load; the reference rule leaves pad 0 as the reference does.
    const int pad = o.balanced ? t.table + 1 : 0;
    if (ns <= 1) {
      A.tiles.push_back({rt.tree, t.base + rt.r, rt.k0, t.P, -1, 1, rt.b0, pad});
      continue;
    }
    // Balanced rule: the batch keys count as work of the last part, so the cached range is
    // cut into parts of (cached + batch) / ns keys and the last part keeps what is left.
    const int per = (span + rt.batch + ns - 1) / ns;
    const int step = (per + o.granule - 1) / o.granule * o.granule;
    const int part0 = A.parts;
    int used = 0;
    if (o.balanced && o.cut_batch && span < (ns - 1) * step) {
      // Some cut falls among the batch keys: walk cached keys [k0, P) and then batch rows [b0, b0 + batch) in parts of
      // `step`, cached cuts on page multiples, batch cuts on multiples of the granule in the tree's rows. A part that
      // ends among the batch rows says where (`last` = its last row + 2); the last part's batch range stays open, so
      // rows that see beyond their own tile (ancestors, image spans) find those keys there.
      const int b_end = rt.b0 + rt.batch;  // one past the tile's last row
      int k = rt.k0, b = rt.b0;
      for (int p = 0; p < ns && (k < t.P || b < b_end); ++p) {
        const bool is_last = p + 1 == ns;
        int k1 = t.P, b1 = b_end;
        if (!is_last) {
          int room = step;
          if (k < t.P) {
            k1 = std::min(t.P, k + room);
            if (k1 < t.P) k1 = std::min(t.P, std::max(k + o.granule, k1 / o.granule * o.granule));
            room -= k1 - k;
          }
          if (k1 < t.P) {
            b1 = b;  // all of it cached keys
          } else {
            b1 = std::min(b_end, b + std::max(room, 0));
            if (b1 < b_end) b1 = std::min(b_end, std::max(b + (k1 > k ? 0 : o.granule), b1 / o.granule * o.granule));
            if (b1 < b) b1 = b;
          }
        }
        if (k1 == k && b1 == b) continue;
        const bool rest = b1 >= b_end;  // nothing left for a later part: this one is the group's last
        const int last = b1 > b ? (rest ? 1 : b1 + 1) : (rest && k1 >= t.P ? 1 : 0);
        A.tiles.push_back({rt.tree, t.base + rt.r, k, k1, A.parts++, last, b, pad});
        k = k1;
        b = b1;
        ++used;
        if (rest && k >= t.P) break;
      }
      if (used == 1) {  // nothing was cut after all
        A.tiles.back().part = -1;
        --A.parts;
        continue;
      }
    } else if (o.balanced) {
      // ns parts: all but the last are `step` cached keys on page multiples; the last keeps the
      // rest of the cached range (possibly nothing) and the batch keys.
      int k = rt.k0;
      for (int p = 0; p < ns; ++p) {
        const bool is_last = p + 1 == ns;
        int k1 = t.P;
        if (!is_last) {
          k1 = std::min(t.P, k + step);
          if (k1 < t.P) k1 = std::min(t.P, std::max(k + o.granule, k1 / o.granule * o.granule));
          if (k1 == k) continue;  // the cached range ran out: the batch keys alone fill the last part
        }
        A.tiles.push_back({rt.tree, t.base + rt.r, k, k1, A.parts++, is_last ? 1 : 0, rt.b0, pad});
        k = k1;
        ++used;
      }
    } else {
      for (int k = rt.k0; k < t.P; k += step, ++used) {
        const int k1 = std::min(t.P, k + step);
        A.tiles.push_back({rt.tree, t.base + rt.r, k, k1, A.parts++, k1 >= t.P ? 1 : 0, rt.b0, pad});
      }
    }
    A.combine.push_back({t.base + rt.r, std::min(R, t.M - rt.r), part0, used});
  }
  // Streaming kernel, balanced rule: every workgroup of the pass is resident at once and the hardware starts them
  // in record order over a few microseconds. The tiles that own their tree's batch keys go first - behind their
  // stream of cached keys they have a serial tail (the batch rows through the masked path) that the others'
  // streaming then covers - and the rest follow by cached range, longest first. (Measured on the batched decode of
  // 16 ragged sequences: 26.6 -> 25.8 us; with the owners of the batch keys last instead, 26.9 us.) The records'
  // partial-record indices stay as assigned, so the merge order does not change.
  if (o.balanced && o.item_steps == 0) {
    std::stable_sort(A.tiles.begin(), A.tiles.end(), [](const esp_tile& x, const esp_tile& y) {
      if (x.last != y.last) return x.last > y.last;
      return (x.k1 - x.k0) > (y.k1 - y.k0);
    });
  }
}

}  // namespace espetero::engine
