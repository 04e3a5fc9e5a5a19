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
  // A slot that the pending pass reads or replaces may not be freed, emptied or overwritten under it: the
  // commit would write the pass's block lists into a slot that is no longer the caller's.
  bool in_pending_pass(int s) const {
    if (!pass_.pending) return false;
    for (const TreePlan& T : pass_.trees)
      if (T.spec.parent == s || T.spec.save == s || T.spec.work == s) return true;
    return false;
  }
  void slot_free(int s) {
    Slot& sl = checked(s);
    if (in_pending_pass(s)) fail("slot " + std::to_string(s) + " belongs to the pending pass (commit or abort it first)");
    release_blocks(sl);
    sl = Slot{};
  }
  // A fresh slot holding `len` positions in `n_blocks` new blocks whose contents the caller brings in
  // afterwards (a loaded checkpoint file: slot_load, src/model/model.mm:694-752). Returns the slot, -1 for
  // counts that do not fit each other, -2 when the pool or the slot table has no room (the reference's codes).
  int slot_adopt(int len, int next_pos, int n_blocks) {
    if (len < 0 || n_blocks < 0 || next_pos < 0 || int64_t(len) > int64_t(n_blocks) * pool_.bt || len > max_ctx_) return -1;
    if (pool_.n_free() < n_blocks) return -2;
    const int s = slot_alloc();
    if (s < 0) return -2;
    Slot& sl = slots_[size_t(s)];
    sl.len = len;
    sl.next_pos = next_pos;
    for (int i = 0; i < n_blocks; ++i) sl.blocks.push_back(pool_.alloc());
    return s;
  }
  void slot_reset(int s) {
    Slot& sl = checked(s);
    if (in_pending_pass(s)) fail("slot " + std::to_string(s) + " belongs to the pending pass (commit or abort it first)");
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
    if (in_pending_pass(dst)) fail("slot " + std::to_string(dst) + " belongs to the pending pass (commit or abort it first)");
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

  // ---- the block list of a slot that continues a parent's cached keys [0, P) and takes positions
  // [w0, end) of this pass. Behaviour of the reference's Forest::target_blocks / target_new_blocks
  // (src/model/impl/forest.h:1785-1829), arrived at by classifying every block index of the new list once:
  //   Shared    lies wholly below w0: the parent's block, one more reference;
  //   InPlace   holds parent positions and positions of this pass, the parent is the target itself and
  //             nobody else references the block: kept, the pass appends into it;
  //   Copied    holds parent positions but may not be written (another slot reads it, or the target is
  //             another slot): a fresh block that first receives a copy of the parent's;
  //   Fresh     beyond the parent's keys: a fresh block.
  enum class BlockUse { Shared, InPlace, Copied, Fresh };
  BlockUse classify(const std::vector<int>& parent_blocks, int P, int w0, bool in_place, int index) const {
    const int bt = pool_.bt;
    if (index < w0 / bt) {
      if (index >= int(parent_blocks.size())) fail("a slot's block list is shorter than its length");
      return BlockUse::Shared;
    }
    const bool holds_parent_keys = index < int(parent_blocks.size()) && index * bt < P;
    if (!holds_parent_keys) return BlockUse::Fresh;
    return in_place && pool_.ref[size_t(parent_blocks[size_t(index)])] == 1 ? BlockUse::InPlace : BlockUse::Copied;
  }
  // How many blocks the list would take from the free list.
  int target_new_blocks(const Slot* parent, int P, int w0, int end, bool in_place) const {
    static const std::vector<int> none;
    const std::vector<int>& pb = parent ? parent->blocks : none;
    int taken = 0;
    for (int i = w0 / pool_.bt; i * pool_.bt < end; ++i) {
      const BlockUse u = classify(pb, P, w0, in_place, i);
      taken += u == BlockUse::Fresh || u == BlockUse::Copied;
    }
    return taken;
  }
  // The list itself; copies the pass has to run first are appended to `cow` as (source, destination).
  std::vector<int> target_blocks(const std::vector<int>& parent_blocks, int P, int w0, int end,
                                 std::vector<std::pair<int, int>>& cow, bool in_place) {
    std::vector<int> list;
    for (int i = 0; i * pool_.bt < std::max(end, w0 / pool_.bt * pool_.bt); ++i) {
      switch (classify(parent_blocks, P, w0, in_place, i)) {
        case BlockUse::Shared:
        case BlockUse::InPlace:
          pool_.retain(parent_blocks[size_t(i)]);
          list.push_back(parent_blocks[size_t(i)]);
          break;
        case BlockUse::Copied: {
          const int fresh = pool_.alloc();
          cow.emplace_back(parent_blocks[size_t(i)], fresh);
          list.push_back(fresh);
          break;
        }
        case BlockUse::Fresh:
          list.push_back(pool_.alloc());
          break;
      }
    }
    return list;
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

  // ---- what a pass can be refused for. Every check runs before anything is changed: a refused pass leaves the
  // pool and every slot as they were (the reference's contract, src/model/api.h:283-285).
  enum class Refusal {
    PassPending, EmptyPass, BadSlot, BadLength, EmptyTree, SaveBeyondRoot, NothingToSave, WorkSlotClash, SlotTakenTwice,
    ParentTaken, NoncausalShape, LeafArrays, LeafWithoutToken, ChainShape, ContextTooLong, PoolExhausted
  };
  struct PassRefused : EngineError {
    Refusal why;
    PassRefused(Refusal w, const std::string& m) : EngineError(m), why(w) {}
  };
  [[noreturn]] static void refuse(Refusal why, const std::string& message) { throw PassRefused(why, message); }

  // Which rows the leaves of a verify tree need. A leaf whose tokens open another leaf's token list is not
  // computed twice: its rows are the first rows of that longer leaf, its host (the reference hosts the same
  // way, src/model/impl/forest.h:2201-2220: the longest leaf that starts with it, the earliest of equals).
  // Leaves are visited longest first (earliest first among equals); a leaf is held up against the hosts
  // found so far, in that order, so the first match is the longest and earliest, and a leaf no host starts
  // with becomes a host itself. Rows are dealt to the hosts in leaf order.
  struct LeafLayout {
    std::vector<int> host, row0;  // per leaf: its host leaf; per host: first row among the tree's leaf rows
    int rows = 0, longest = 0;
  };
  static LeafLayout lay_out_leaves(const esp_tree_spec& spec) {
    const int n = spec.n_leaves;
    LeafLayout lay;
    if (n == 0) return lay;
    if (!spec.leaf_offsets || !spec.leaf_tokens) refuse(Refusal::LeafArrays, "leaf arrays missing");
    if (spec.leaf_offsets[0] != 0) refuse(Refusal::LeafArrays, "leaf offsets must start at 0");
    auto length = [&](int i) { return spec.leaf_offsets[i + 1] - spec.leaf_offsets[i]; };
    auto tokens = [&](int i) { return spec.leaf_tokens + spec.leaf_offsets[i]; };
    std::vector<int> order(size_t(n), 0);
    for (int i = 0; i < n; ++i) {
      if (length(i) <= 0) refuse(Refusal::LeafWithoutToken, "every leaf needs a token");
      lay.longest = std::max(lay.longest, length(i));
      order[size_t(i)] = i;
    }
    std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return length(x) > length(y); });
    lay.host.assign(size_t(n), -1);
    std::vector<int> hosts;
    for (int leaf : order) {
      int found = leaf;
      for (int h : hosts)
        if (std::equal(tokens(leaf), tokens(leaf) + length(leaf), tokens(h))) {
          found = h;
          break;
        }
      lay.host[size_t(leaf)] = found;
      if (found == leaf) hosts.push_back(leaf);
    }
    lay.row0.assign(size_t(n), 0);
    for (int i = 0; i < n; ++i)
      if (lay.host[size_t(i)] == i) {
        lay.row0[size_t(i)] = lay.rows;
        lay.rows += length(i);
      }
    return lay;
  }

  // One tree of a pass, checked and sized against the slots as they are.
  TreePlan size_tree(const esp_tree_spec& spec) const {
    auto slot_or_none = [&](int s, const char* role) {
      const bool none = s == -1, live = s >= 0 && s < int(slots_.size()) && slots_[size_t(s)].used;
      if (!none && !live) refuse(Refusal::BadSlot, std::string("invalid ") + role + " slot " + std::to_string(s));
    };
    slot_or_none(spec.parent, "parent");
    slot_or_none(spec.save, "save");
    slot_or_none(spec.work, "work");
    if (spec.root_len < 0 || spec.n_leaves < 0) refuse(Refusal::BadLength, "negative root or leaf count");
    if (spec.root_len + spec.n_leaves == 0) refuse(Refusal::EmptyTree, "empty tree: neither root rows nor leaves");
    TreePlan T;
    T.spec = spec;
    T.Tr = spec.root_len;
    T.NL = spec.n_leaves;
    T.save_len = spec.save_len > 0 ? spec.save_len : spec.root_len;
    T.P = spec.parent >= 0 ? slots_[size_t(spec.parent)].len : 0;
    if (T.save_len > T.Tr) refuse(Refusal::SaveBeyondRoot, "save_len exceeds root_len");
    if (T.Tr == 0 && (spec.save >= 0 || spec.work >= 0))
      refuse(Refusal::NothingToSave, "a tree without root rows has nothing to save (fork the slot instead)");
    if (spec.work >= 0 && (spec.work == spec.save || spec.work == spec.parent))
      refuse(Refusal::WorkSlotClash, "the work slot must differ from the save and parent slots");
    if (spec.noncausal && (spec.parent >= 0 || spec.save >= 0 || spec.work >= 0 || T.NL > 0 || T.Tr == 0))
      refuse(Refusal::NoncausalShape, "a noncausal tree is a root alone: no parent, save or work slot, no leaves");
    const LeafLayout lay = lay_out_leaves(spec);
    T.host = lay.host;
    T.off = lay.row0;
    if (spec.commit_chain > 0) {
      // The rows of leaves 0 .. k-1 are kept as a chain the caller may commit later: leaf i is the first
      // i + 1 tokens of leaf k-1, whose rows open the tree's leaf rows (forest.h:2223-2234).
      const int k = spec.commit_chain;
      if (k > T.NL) refuse(Refusal::ChainShape, "commit_chain names more leaves than the tree has");
      const bool in_place_whole_root = spec.save >= 0 && spec.save == spec.parent && spec.work < 0 && T.save_len == T.Tr;
      if (!in_place_whole_root) refuse(Refusal::ChainShape, "commit_chain needs a tree that appends its whole root to its own parent slot");
      for (int i = 0; i < k; ++i)
        if (spec.leaf_offsets[i + 1] - spec.leaf_offsets[i] != i + 1 || T.host[size_t(i)] != k - 1)
          refuse(Refusal::ChainShape, "commit_chain: leaf " + std::to_string(i) + " is not the first " + std::to_string(i + 1) +
                                          " tokens of leaf " + std::to_string(k - 1));
      if (T.off[size_t(k - 1)] != 0) refuse(Refusal::ChainShape, "commit_chain: the chain's rows must open the leaf rows");
      T.cm_k = k;
    }
    if (T.P + T.Tr + lay.longest > max_ctx_)
      refuse(Refusal::ContextTooLong, "context " + std::to_string(T.P + T.Tr + lay.longest) + " exceeds max_ctx " + std::to_string(max_ctx_));
    T.M = T.Tr + lay.rows;
    return T;
  }

  void pass_begin(const esp_tree_spec* specs, int n_trees) {
    if (pass_.pending) refuse(Refusal::PassPending, "a pass is already pending (commit or abort it)");
    if (n_trees <= 0 || !specs) refuse(Refusal::EmptyPass, "empty pass");
    Pass ps;
    ps.trees.reserve(size_t(n_trees));
    // Which tree writes each slot: a slot takes the result of at most one tree, and no tree may read a
    // slot that another tree of the pass replaces.
    std::vector<int> writer(slots_.size(), -1);
    int M = 0;
    for (int t = 0; t < n_trees; ++t) {
      TreePlan T = size_tree(specs[t]);
      for (int s : {specs[t].save, specs[t].work})
        if (s >= 0) {
          if (writer[size_t(s)] >= 0) refuse(Refusal::SlotTakenTwice, "two trees save into one slot (" + std::to_string(s) + ")");
          writer[size_t(s)] = t;
        }
      T.base = M;
      M += T.M;
      ps.trees.push_back(std::move(T));
    }
    for (int t = 0; t < n_trees; ++t) {
      const int p = specs[t].parent;
      if (p >= 0 && writer[size_t(p)] >= 0 && writer[size_t(p)] != t)
        refuse(Refusal::ParentTaken, "tree " + std::to_string(writer[size_t(p)]) + " saves into the parent slot of tree " + std::to_string(t));
    }
    if (const int need = pass_blocks(specs, n_trees); need > pool_.n_free())
      refuse(Refusal::PoolExhausted, "KV cache full: the pass needs " + std::to_string(need) + " blocks, " + std::to_string(pool_.n_free()) + " are free");

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
