// KV block pool, sequence slots and the pass builder of the attention call
// surface. Host code, no device calls; single-threaded like the reference's
// model object (src/model/api.h:4-6).
//
// What it restates from the reference, for this path only:
//   pool + refcounts        src/model/impl/forest.h:60-62, model.h:722-737
//   target_blocks           src/model/impl/forest.h:1785-1811 (share / copy on write / in place)
//   target_new_blocks       src/model/impl/forest.h:1821-1829
//   tree validation         src/model/impl/forest.h:2136-2266 (the attention-relevant checks)
//   leaf hosting            src/model/impl/forest.h:2201-2220, commit chains :2223-2234
//   rows: desc / pos        src/model/impl/forest.h:2374-2443
//   block table, kv saves   src/model/impl/forest.h:2483-2520
//   sliding-layer rings     src/model/impl/forest.h:2657-2700 (trees, saves, window copies)
//   commit / rollback       src/model/impl/forest.h:2468-2482, 4743-4754
//   slot operations         src/model/model.mm:520-553
//   verify-commit           src/model/impl/forest.h:4755-4765, 4846-4861, 5058-5069 (length / position side)
// A pass never changes a slot before commit(): a failure (or abort()) gives
// the new blocks back and leaves every slot as it was.
#pragma once

#include <algorithm>
#include <array>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/espetero_engine.h"

namespace espetero::engine {

struct EngineError : std::runtime_error {
  using std::runtime_error::runtime_error;
};
[[noreturn]] inline void fail(const std::string& m) { throw EngineError(m); }

struct Slot {
  bool used = false;
  int len = 0;
  int next_pos = 0;
  std::vector<int> blocks;  // block ids covering positions [0, len) (and the kept chain rows behind them)
  // The commit record of the slot's last pass (forest.h:4755-4765): cm_k chain rows whose K / V already sit at
  // positions len .. len + cm_k - 1, the first at rotary position cm_pos0; valid until another pass begins.
  int cm_k = 0, cm_pos0 = 0;
  uint64_t cm_pass = 0;
};

struct KvPool {
  int bt = 16;
  int n_blocks = 0;
  std::vector<int> ref;
  std::vector<int> free_list;

  void init(int blocks, int block_tokens) {
    bt = block_tokens;
    n_blocks = blocks;
    ref.assign(size_t(blocks), 0);
    free_list.clear();
    for (int b = blocks - 1; b >= 0; --b) free_list.push_back(b);  // block 0 is handed out first
  }
  int n_free() const { return int(free_list.size()); }
  int alloc() {
    if (free_list.empty()) fail("KV cache full (raise the pool size or lower concurrency)");
    const int b = free_list.back();
    free_list.pop_back();
    ref[size_t(b)] = 1;
    return b;
  }
  void retain(int b) { ++ref[size_t(b)]; }
  void release(int b) {
    if (--ref[size_t(b)] == 0) free_list.push_back(b);
  }
};

struct TreePlan {
  esp_tree_spec spec{};
  int P = 0, Tr = 0, save_len = 0, NL = 0, M = 0, base = 0, cm_k = 0;
  int next_root = 0, next_save = 0, read_table = 0;
  std::vector<int> host, off;
  std::vector<int> dst_blocks, work_blocks;
};

// Per pass row the pool entries its K / V go to, (block, position, block2, position2), -1 none: what
// esp_attn_prep's folded append reads instead of a kv_save dispatch (kv_row_table,
// src/model/impl/forest.h:1737-1749). A row saved into more than two slots is refused, as there.
inline std::vector<int32_t> row_table(const esp_kvsave* saves, int n_saves, int rows) {
  std::vector<int32_t> t(size_t(std::max(rows, 1)) * 4, -1);
  for (int i = 0; i < n_saves; ++i) {
    const esp_kvsave& r = saves[i];
    if (r.src_row < 0 || r.src_row >= rows) throw EngineError("row_table: a save names a row outside the pass");
    int32_t* e = t.data() + size_t(r.src_row) * 4;
    const int j = e[0] < 0 ? 0 : 2;
    if (j == 2 && e[2] >= 0) throw EngineError("row_table: a row saved into more than two slots");
    e[j] = r.block;
    e[j + 1] = r.pos;
  }
  return t;
}

class KvEngine {
 public:
  KvEngine(int n_blocks, int bt, int n_slots, int max_ctx) : max_ctx_(max_ctx) {
    if (n_blocks <= 0 || bt <= 0 || bt % 16 || n_slots <= 0) fail("invalid pool geometry");
    pool_.init(n_blocks, bt);
    slots_.assign(size_t(n_slots), Slot{});
  }

  const KvPool& pool() const { return pool_; }
  const Slot& slot(int s) const { return slots_.at(size_t(s)); }

  int slot_alloc() {
    for (size_t i = 0; i < slots_.size(); ++i)
      if (!slots_[i].used) {
        slots_[i] = Slot{};
        slots_[i].used = true;
        return int(i);
      }
    return -1;
  }
  void slot_free(int s) {
    Slot& sl = checked(s);
    release_blocks(sl);
    sl = Slot{};
  }
  void slot_reset(int s) {
    Slot& sl = checked(s);
    release_blocks(sl);
    sl.len = sl.next_pos = 0;
    sl.cm_k = 0;
  }
  // dst becomes a copy of src sharing the blocks of its [0, len) by refcount; the chain rows stay the
  // source's (model.mm:542-553).
  void slot_fork(int src, int dst) {
    Slot& a = checked(src);
    Slot& b = checked(dst);
    if (src == dst) return;
    release_blocks(b);
    const size_t nb = std::min(size_t((a.len + pool_.bt - 1) / pool_.bt), a.blocks.size());
    b.blocks.assign(a.blocks.begin(), a.blocks.begin() + long(nb));
    for (int blk : b.blocks) pool_.retain(blk);
    b.len = a.len;
    b.next_pos = a.next_pos;
    b.cm_k = 0;
  }
  // Chain rows of `s` that chain_commit could still take: those its last pass kept, while no other pass has begun.
  int slot_chain(int s) const {
    const Slot& sl = slots_.at(size_t(s));
    return sl.used && sl.cm_pass == pass_seq_ ? sl.cm_k : 0;
  }
  // Verify-commit, the block-pool side (run_commit, forest.h:4846-4861, 5058-5069): the first n rows of the
  // chain the slot's last pass kept (esp_tree_spec::commit_chain) become part of the slot. Their K / V are
  // already at their positions; length and next position follow, and the rest of the chain is dropped.
  void chain_commit(int s, int n) {
    Slot& sl = checked(s);
    if (pass_.pending) fail("commit: a pass is pending");
    if (n < 0 || n > sl.cm_k || (n > 0 && sl.cm_pass != pass_seq_))
      fail("commit: slot " + std::to_string(s) + " holds no such chain rows of the last pass");
    if (n > 0) {
      sl.len += n;
      sl.next_pos = sl.cm_pos0 + n;
    }
    sl.cm_k = 0;
  }

  // Blocks Forest::target_blocks would allocate for one target (forest.h:1821-1829).
  int target_new_blocks(const Slot* parent, int P, int w0, int end, bool in_place) const {
    const int bt = pool_.bt;
    const int i = w0 / bt;
    int n = (end + bt - 1) / bt - i;
    if (n > 0 && in_place && parent && i < int(parent->blocks.size()) && i * bt < P &&
        pool_.ref[size_t(parent->blocks[size_t(i)])] == 1)
      --n;
    return std::max(n, 0);
  }

  // New block list of a target that continues `parent_blocks` (covering [0, P))
  // and writes positions [w0, end) (forest.h:1785-1811).
  std::vector<int> target_blocks(const std::vector<int>& parent_blocks, int P, int w0, int end,
                                 std::vector<std::pair<int, int>>& cow, bool in_place) {
    const int bt = pool_.bt;
    std::vector<int> out;
    const int keep = w0 / bt;  // blocks entirely below w0 are shared
    for (int i = 0; i < keep && i < int(parent_blocks.size()); ++i) {
      out.push_back(parent_blocks[size_t(i)]);
      pool_.retain(parent_blocks[size_t(i)]);
    }
    const int need = (end + bt - 1) / bt;
    for (int i = keep; i < need; ++i) {
      const bool has_parent = i < int(parent_blocks.size()) && i * bt < P;
      // An in-place append keeps a partial block it owns alone: the pass writes
      // positions >= w0 there while attention reads positions < P.
      if (has_parent && in_place && pool_.ref[size_t(parent_blocks[size_t(i)])] == 1) {
        out.push_back(parent_blocks[size_t(i)]);
        pool_.retain(parent_blocks[size_t(i)]);
        continue;
      }
      const int nb = pool_.alloc();
      if (has_parent) cow.push_back({parent_blocks[size_t(i)], nb});  // it also holds parent positions
      out.push_back(nb);
    }
    return out;
  }

  int pass_blocks(const esp_tree_spec* specs, int n) const {
    int need = 0;
    for (int t = 0; t < n; ++t) {
      const esp_tree_spec& b = specs[t];
      const Slot* parent = b.parent >= 0 && b.parent < int(slots_.size()) ? &slots_[size_t(b.parent)] : nullptr;
      const int P = parent ? parent->len : 0;
      const int save_len = b.save_len > 0 ? b.save_len : b.root_len;
      if (b.save >= 0) need += target_new_blocks(parent, P, P, P + save_len + b.commit_chain, b.save == b.parent);
      if (b.work >= 0) need += target_new_blocks(parent, P, P, P + b.root_len, false);
    }
    return need;
  }

  // ---- the pending pass
  struct Pass {
    bool pending = false;
    int M = 0;
    std::vector<TreePlan> trees;
    std::vector<esp_tree> recs;
    std::vector<int32_t> desc, pos, table;
    std::vector<esp_kvsave> saves;
    std::vector<std::array<int32_t, 2>> cow;
  };
  const Pass& pass() const { return pass_; }

  void pass_begin(const esp_tree_spec* specs, int n_trees) {
    if (pass_.pending) fail("a pass is already pending (commit or abort it)");
    if (n_trees <= 0 || !specs) fail("empty pass");
    Pass ps;
    ps.trees.resize(size_t(n_trees));
    const int n_user = int(slots_.size());
    std::vector<int> saved(size_t(n_user), -1);
    int M = 0;
    // ---- validation and sizes: nothing is modified until every tree passes
    for (int t = 0; t < n_trees; ++t) {
      const esp_tree_spec& b = specs[t];
      TreePlan& T = ps.trees[size_t(t)];
      T.spec = b;
      auto check_slot = [&](int s, const char* what) {
        if (s < -1 || s >= n_user || (s >= 0 && !slots_[size_t(s)].used))
          fail(std::string("invalid ") + what + " slot " + std::to_string(s));
      };
      check_slot(b.parent, "parent");
      check_slot(b.save, "save");
      check_slot(b.work, "work");
      if (b.root_len < 0 || b.n_leaves < 0) fail("invalid lengths");
      if (b.root_len == 0 && b.n_leaves == 0) fail("empty tree");
      T.Tr = b.root_len;
      T.save_len = b.save_len > 0 ? b.save_len : T.Tr;
      if (T.save_len > T.Tr) fail("save_len exceeds root_len");
      if (b.save >= 0 && T.Tr == 0) fail("nothing to save (use slot_fork)");
      if (b.work >= 0) {
        if (T.Tr == 0) fail("nothing to save in the work slot");
        if (b.work == b.save || b.work == b.parent) fail("work slot must differ from save and parent slots");
      }
      T.P = b.parent >= 0 ? slots_[size_t(b.parent)].len : 0;
      for (int s : {b.save, b.work}) {
        if (s < 0) continue;
        if (saved[size_t(s)] >= 0) fail("two trees save into one slot");
        saved[size_t(s)] = t;
      }
      T.NL = b.n_leaves;
      if (b.noncausal && (b.parent >= 0 || b.save >= 0 || b.work >= 0 || b.n_leaves > 0 || T.Tr == 0))
        fail("noncausal: a root alone (no parent, save or work slot, leaves)");
      int leaf_rows = 0, max_leaf = 0;
      if (T.NL > 0) {
        if (!b.leaf_offsets || !b.leaf_tokens) fail("leaf arrays missing");
        if (b.leaf_offsets[0] != 0) fail("offsets must start at 0");
        auto len_of = [&](int i) { return b.leaf_offsets[i + 1] - b.leaf_offsets[i]; };
        for (int i = 0; i < T.NL; ++i) {
          if (len_of(i) <= 0) fail("every leaf needs a token");
          max_leaf = std::max(max_leaf, len_of(i));
        }
        // A leaf whose tokens are a prefix of another leaf is read from that leaf's rows.
        T.host.assign(size_t(T.NL), -1);
        T.off.assign(size_t(T.NL), 0);
        for (int i = 0; i < T.NL; ++i) {
          int h = i;
          const int32_t* ti = b.leaf_tokens + b.leaf_offsets[i];
          for (int j = 0; j < T.NL; ++j) {
            if (j == i || len_of(j) < len_of(i)) continue;
            if (len_of(j) == len_of(i) && j > i) continue;
            if (len_of(j) < len_of(h) || (len_of(j) == len_of(h) && j >= h)) continue;
            if (std::equal(ti, ti + len_of(i), b.leaf_tokens + b.leaf_offsets[j])) h = j;
          }
          T.host[size_t(i)] = h;
        }
        for (int i = 0; i < T.NL; ++i)
          if (T.host[size_t(i)] == i) {
            T.off[size_t(i)] = leaf_rows;
            leaf_rows += len_of(i);
          }
        if (b.commit_chain > 0) {
          const int kc = b.commit_chain;
          if (kc > T.NL) fail("commit_chain exceeds the leaves");
          if (b.save < 0 || b.save != b.parent || b.work >= 0 || T.save_len != T.Tr)
            fail("commit_chain: in-place trees with a whole root only");
          for (int i = 0; i < kc; ++i)
            if (len_of(i) != i + 1 || T.host[size_t(i)] != kc - 1) fail("commit_chain: the leaves are not one chain");
          if (T.off[size_t(kc - 1)] != 0) fail("commit_chain: the chain must be the first leaf rows");
          T.cm_k = kc;
        }
      }
      if (b.commit_chain > 0 && T.NL == 0) fail("commit_chain without leaves");
      if (T.P + T.Tr + max_leaf > max_ctx_) fail("context exceeds max_ctx (" + std::to_string(max_ctx_) + ")");
      T.M = T.Tr + leaf_rows;
      T.base = M;
      M += T.M;
    }
    for (int t = 0; t < n_trees; ++t) {
      const int p = specs[t].parent;
      if (p >= 0 && saved[size_t(p)] >= 0 && saved[size_t(p)] != t) fail("a tree saves into another tree's parent");
    }
    {
      const int need = pass_blocks(specs, n_trees);
      if (need > pool_.n_free())
        fail("KV cache full: need " + std::to_string(need) + " blocks, " + std::to_string(pool_.n_free()) + " free");
    }

    // ---- rows: descriptors and positions
    ps.M = M;
    ps.desc.assign(size_t(4) * size_t(std::max(M, 1)), 0);
    ps.pos.assign(size_t(4) * size_t(std::max(M, 1)), 0);
    for (TreePlan& T : ps.trees) {
      const esp_tree_spec& b = T.spec;
      const int pnext = b.parent >= 0 ? slots_[size_t(b.parent)].next_pos : 0;
      int pmax = pnext - 1, pmax_save = pnext - 1;
      for (int j = 0; j < T.Tr; ++j) {
        const int r = T.base + j, pt = pnext + j;
        ps.pos[4 * r] = ps.pos[4 * r + 1] = ps.pos[4 * r + 2] = pt;
        pmax = std::max(pmax, pt);
        if (j < T.save_len) pmax_save = pmax;
        ps.desc[4 * r + 2] = b.noncausal ? T.Tr : 0;  // a noncausal root row sees the whole root
      }
      T.next_root = pmax + 1;
      T.next_save = pmax_save + 1;
      for (int i = 0; i < T.NL; ++i) {
        if (T.host[size_t(i)] != i) continue;
        const int start = T.Tr + T.off[size_t(i)];
        const int len = b.leaf_offsets[i + 1] - b.leaf_offsets[i];
        for (int j = 0; j < len; ++j) {
          const int r = T.base + start + j;
          ps.pos[4 * r] = ps.pos[4 * r + 1] = ps.pos[4 * r + 2] = T.next_root + j;
          ps.desc[4 * r] = start;   // own segment
          ps.desc[4 * r + 2] = T.Tr;  // the whole root
        }
      }
    }

    // ---- block tables, saves; from the first new block a failure gives them back
    struct Guard {
      KvEngine& e;
      Pass& ps;
      bool armed = true;
      ~Guard() {
        if (armed) e.release_pass(ps);
      }
    } guard{*this, ps};
    std::vector<std::pair<int, int>> cow;
    const int bt = pool_.bt;
    for (TreePlan& T : ps.trees) {
      const esp_tree_spec& b = T.spec;
      T.read_table = int(ps.table.size());
      static const std::vector<int> empty;
      const std::vector<int>& pb = b.parent >= 0 ? slots_[size_t(b.parent)].blocks : empty;
      for (int i = 0; i < (T.P + bt - 1) / bt; ++i) ps.table.push_back(pb[size_t(i)]);
      auto add_saves = [&](const std::vector<int>& blocks, int n) {
        for (int i = 0; i < n; ++i) {
          const int p = T.P + i;
          ps.saves.push_back({T.base + i, blocks[size_t(p / bt)], p % bt, 0});
        }
      };
      if (b.save >= 0) {
        T.dst_blocks = target_blocks(pb, T.P, T.P, T.P + T.save_len + T.cm_k, cow, b.save == b.parent);
        add_saves(T.dst_blocks, T.save_len);
        for (int j = 0; j < T.cm_k; ++j) {  // chain rows at the positions they take if committed
          const int p = T.P + T.Tr + j;
          ps.saves.push_back({T.base + T.Tr + j, T.dst_blocks[size_t(p / bt)], p % bt, 0});
        }
      }
      if (b.work >= 0) {
        T.work_blocks = target_blocks(pb, T.P, T.P, T.P + T.Tr, cow, false);
        add_saves(T.work_blocks, T.Tr);
      }
      ps.recs.push_back({T.base, T.P, T.read_table, T.M});
    }
    for (auto& [s, d] : cow) ps.cow.push_back({s, d});
    guard.armed = false;
    ps.pending = true;
    pass_ = std::move(ps);
    ++pass_seq_;  // the chain rows earlier passes kept are no longer committable
  }

  // The pending pass as the sliding layers see it (Gemma: the last `window` positions of slot s live in a second
  // pool, in the ring of `ring_blocks` consecutive blocks from s * ring_blocks on, position p in block
  // (p / bt) % ring_blocks; src/model/impl/forest.h:2657-2700):
  //   trees   read the parent's ring: table = the ring's first block;
  //   saves   of the rows that are still inside the window when the pass ends, into the ring of every target;
  //   copies  (ring block of the parent -> same ring block of the target) for a target that is another slot:
  //           the part of the parent's window the target still needs, each ring block once.
  // Copies run before the pass's attention and saves after it, like the other pool's.
  struct RingPlan {
    std::vector<esp_tree> trees;
    std::vector<esp_kvsave> saves;
    std::vector<std::array<int32_t, 2>> copies;
  };
  RingPlan ring_plan(int window, int ring_blocks) const {
    if (!pass_.pending) fail("no pending pass");
    const int bt = pool_.bt, rb = ring_blocks, W = window;
    if (W <= 0 || rb <= 0 || int64_t(rb) * bt < W) fail("ring_plan: the ring must hold the window");
    RingPlan out;
    for (const TreePlan& T : pass_.trees) {
      if (T.cm_k) fail("ring_plan: commit_chain is not supported on sliding layers");  // forest.h:2237
      const int parent = T.spec.parent;
      out.trees.push_back({T.base, T.P, parent >= 0 ? parent * rb : 0, T.M});
      auto target = [&](int slot, int S) {
        if (slot != parent && T.P > 0) {
          std::vector<char> seen(size_t(rb), 0);
          for (int b = std::max(0, T.P + S - W + 1) / bt; b * bt < T.P; ++b)
            if (!seen[size_t(b % rb)]++) out.copies.push_back({parent * rb + b % rb, slot * rb + b % rb});
        }
        for (int p = std::max(T.P, T.P + S - W + 1); p < T.P + S; ++p)
          out.saves.push_back({T.base + (p - T.P), slot * rb + (p / bt) % rb, p % bt, 0});
      };
      if (T.spec.save >= 0) target(T.spec.save, T.save_len);
      if (T.spec.work >= 0) target(T.spec.work, T.Tr);
    }
    return out;
  }

  void pass_commit() {
    if (!pass_.pending) fail("no pending pass");
    for (TreePlan& T : pass_.trees) {
      auto commit = [&](int s, std::vector<int>& blocks, int len, int next) {
        Slot& to = slots_[size_t(s)];
        release_blocks(to);
        to.blocks = std::move(blocks);
        to.len = len;
        to.next_pos = next;
      };
      if (T.spec.save >= 0) {
        commit(T.spec.save, T.dst_blocks, T.P + T.save_len, T.save_len == T.Tr ? T.next_root : T.next_save);
        Slot& to = slots_[size_t(T.spec.save)];
        to.cm_k = T.cm_k;
        to.cm_pos0 = T.next_root;
        to.cm_pass = pass_seq_;
      }
      if (T.spec.work >= 0) {
        commit(T.spec.work, T.work_blocks, T.P + T.Tr, T.next_root);
        slots_[size_t(T.spec.work)].cm_k = 0;
      }
    }
    pass_ = Pass{};
  }

  void pass_abort() {
    if (!pass_.pending) return;
    release_pass(pass_);
    pass_ = Pass{};
  }

 private:
  Slot& checked(int s) {
    if (s < 0 || s >= int(slots_.size()) || !slots_[size_t(s)].used) fail("invalid slot " + std::to_string(s));
    return slots_[size_t(s)];
  }
  void release_blocks(Slot& s) {
    for (int b : s.blocks) pool_.release(b);
    s.blocks.clear();
  }
  void release_pass(Pass& ps) {
    for (TreePlan& T : ps.trees) {
      for (int b : T.dst_blocks) pool_.release(b);
      for (int b : T.work_blocks) pool_.release(b);
      T.dst_blocks.clear();
      T.work_blocks.clear();
    }
  }

  KvPool pool_;
  std::vector<Slot> slots_;
  int max_ctx_;
  Pass pass_;
  uint64_t pass_seq_ = 0;
};

}  // namespace espetero::engine
