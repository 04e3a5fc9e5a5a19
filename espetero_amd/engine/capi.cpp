// C view (include/espetero_engine.h) of the C++ planner and KV engine.
#include <cstdio>
#include <cstring>
#include <new>

#include "kv_engine.hpp"
#include "planner.hpp"
#include "slot_file.hpp"

using namespace espetero::engine;

struct esp_engine {
  KvEngine e;
  esp_engine(int nb, int bt, int ns, int mc) : e(nb, bt, ns, mc) {}
};

namespace {
int put_err(char* err, size_t errlen, int code, const char* msg) {
  if (err && errlen) snprintf(err, errlen, "%s", msg);
  return code;
}
PlanOptions to_cpp(const esp_plan_options& o) {
  PlanOptions p;
  p.rows_per_tile = o.rows_per_tile;
  p.groups_target = o.groups_target;
  p.split = o.split;
  p.min_chunk = o.min_chunk;
  p.granule = o.granule;
  p.max_splits = o.max_splits;
  p.min_span = o.min_span;
  p.balanced = o.balanced != 0;
  p.item_steps = o.item_steps;
  p.part_steps = o.part_steps;
  p.cut_batch = o.cut_batch != 0;
  return p;
}
void to_c(const PlanOptions& p, esp_plan_options* o) {
  o->rows_per_tile = p.rows_per_tile;
  o->groups_target = p.groups_target;
  o->split = p.split;
  o->min_chunk = p.min_chunk;
  o->granule = p.granule;
  o->max_splits = p.max_splits;
  o->min_span = p.min_span;
  o->balanced = p.balanced ? 1 : 0;
  o->item_steps = p.item_steps;
  o->part_steps = p.part_steps;
  o->cut_batch = p.cut_batch ? 1 : 0;
}
template <class F>
int guarded(F&& f) {
  try {
    f();
    return 0;
  } catch (...) {
    return -1;
  }
}
}  // namespace

extern "C" {

void esp_plan_options_reference(esp_plan_options* o) { to_c(PlanOptions::reference(), o); }
void esp_plan_options_mi355x(esp_plan_options* o, int32_t rows, int32_t workgroups) {
  to_c(PlanOptions::mi355x(rows, workgroups), o);
}

int esp_plan_tiles(const esp_tree* trees, int32_t n_trees, int32_t groups, int32_t window, const int32_t* pos,
                   const esp_plan_options* o, esp_tile* tiles, int32_t tiles_cap, int32_t* n_tiles, esp_combine* jobs,
                   int32_t jobs_cap, int32_t* n_jobs, int32_t* n_parts, char* err, size_t errlen) {
  if (!o || (n_trees > 0 && !trees) || !n_tiles || !n_jobs || !n_parts) return put_err(err, errlen, ESP_EINVAL, "NULL argument");
  if (n_trees < 0 || groups <= 0) return put_err(err, errlen, ESP_EINVAL, "n_trees / groups");
  if (o->rows_per_tile <= 0 || o->groups_target <= 0 || o->granule <= 0 || o->max_splits <= 0 || o->min_chunk <= 0)
    return put_err(err, errlen, ESP_EINVAL, "plan options must be positive");
  if (o->granule % 16) return put_err(err, errlen, ESP_EINVAL, "granule must be a multiple of 16");
  if (window > 0 && !pos) return put_err(err, errlen, ESP_EINVAL, "window needs pos");
  try {
    AttnPlan A;
    A.trees.assign(trees, trees + n_trees);
    plan_tiles(A, groups, window, pos, to_cpp(*o));
    *n_tiles = int32_t(A.tiles.size());
    *n_jobs = int32_t(A.combine.size());
    *n_parts = A.parts;
    if (int(A.tiles.size()) > tiles_cap || int(A.combine.size()) > jobs_cap || (!tiles && !A.tiles.empty()) ||
        (!jobs && !A.combine.empty()))
      return put_err(err, errlen, ESP_EWORKSPACE, "tiles / jobs capacity too small");
    if (!A.tiles.empty()) memcpy(tiles, A.tiles.data(), A.tiles.size() * sizeof(esp_tile));
    if (!A.combine.empty()) memcpy(jobs, A.combine.data(), A.combine.size() * sizeof(esp_combine));
    return ESP_OK;
  } catch (const std::exception& e) {
    return put_err(err, errlen, ESP_EINVAL, e.what());
  }
}

esp_engine* esp_engine_create(int32_t n_blocks, int32_t bt, int32_t n_slots, int32_t max_ctx) {
  try {
    return new esp_engine(n_blocks, bt, n_slots, max_ctx);
  } catch (...) {
    return nullptr;
  }
}
void esp_engine_destroy(esp_engine* e) { delete e; }
int esp_engine_slot_alloc(esp_engine* e) { return e->e.slot_alloc(); }
int esp_engine_slot_free(esp_engine* e, int32_t s) { return guarded([&] { e->e.slot_free(s); }); }
int esp_engine_slot_reset(esp_engine* e, int32_t s) { return guarded([&] { e->e.slot_reset(s); }); }
int esp_engine_slot_fork(esp_engine* e, int32_t a, int32_t b) { return guarded([&] { e->e.slot_fork(a, b); }); }
int esp_engine_slot_adopt(esp_engine* e, int32_t len, int32_t next_pos, int32_t n_blocks) {
  try {
    return e->e.slot_adopt(len, next_pos, n_blocks);
  } catch (...) {
    return -1;
  }
}
int esp_engine_slot_len(const esp_engine* e, int32_t s) {
  try {
    const Slot& sl = e->e.slot(s);
    return sl.used ? sl.len : -1;
  } catch (...) {
    return -1;
  }
}
int esp_engine_slot_blocks(const esp_engine* e, int32_t s, int32_t* out, int32_t cap) {
  try {
    const Slot& sl = e->e.slot(s);
    const int n = int(sl.blocks.size());
    for (int i = 0; i < n && i < cap; ++i) out[i] = sl.blocks[size_t(i)];
    return n;
  } catch (...) {
    return -1;
  }
}
int esp_engine_slot_next_pos(const esp_engine* e, int32_t s) {
  try {
    const Slot& sl = e->e.slot(s);
    return sl.used ? sl.next_pos : -1;
  } catch (...) {
    return -1;
  }
}
int esp_engine_slot_chain(const esp_engine* e, int32_t s) {
  try {
    return e->e.slot_chain(s);
  } catch (...) {
    return -1;
  }
}
int esp_engine_chain_commit(esp_engine* e, int32_t s, int32_t n, char* err, size_t errlen) {
  try {
    e->e.chain_commit(s, n);
    return ESP_OK;
  } catch (const std::exception& ex) {
    return put_err(err, errlen, ESP_EINVAL, ex.what());
  }
}
int esp_engine_free_blocks(const esp_engine* e) { return e->e.pool().n_free(); }
int esp_engine_block_ref(const esp_engine* e, int32_t b) {
  return (b < 0 || b >= e->e.pool().n_blocks) ? -1 : e->e.pool().ref[size_t(b)];
}
int esp_engine_pass_blocks(const esp_engine* e, const esp_tree_spec* specs, int32_t n) { return e->e.pass_blocks(specs, n); }

int esp_engine_pass_begin(esp_engine* e, const esp_tree_spec* specs, int32_t n, char* err, size_t errlen) {
  try {
    e->e.pass_begin(specs, n);
    return ESP_OK;
  } catch (const std::exception& ex) {
    return put_err(err, errlen, ESP_EINVAL, ex.what());
  }
}
int esp_engine_pass_rows(const esp_engine* e) { return e->e.pass().M; }
int esp_engine_pass_counts(const esp_engine* e, int32_t* n_table, int32_t* n_saves, int32_t* n_cow) {
  const auto& p = e->e.pass();
  if (n_table) *n_table = int32_t(p.table.size());
  if (n_saves) *n_saves = int32_t(p.saves.size());
  if (n_cow) *n_cow = int32_t(p.cow.size());
  return int(p.recs.size());
}
int esp_engine_pass_trees(const esp_engine* e, esp_tree* out) {
  const auto& p = e->e.pass();
  if (!p.recs.empty()) memcpy(out, p.recs.data(), p.recs.size() * sizeof(esp_tree));
  return int(p.recs.size());
}
int esp_engine_pass_desc(const esp_engine* e, int32_t* out) {
  const auto& p = e->e.pass();
  memcpy(out, p.desc.data(), size_t(4) * size_t(p.M) * 4);
  return p.M;
}
int esp_engine_pass_pos(const esp_engine* e, int32_t* out) {
  const auto& p = e->e.pass();
  memcpy(out, p.pos.data(), size_t(4) * size_t(p.M) * 4);
  return p.M;
}
int esp_engine_pass_table(const esp_engine* e, int32_t* out) {
  const auto& p = e->e.pass();
  if (!p.table.empty()) memcpy(out, p.table.data(), p.table.size() * 4);
  return int(p.table.size());
}
int esp_engine_pass_saves(const esp_engine* e, esp_kvsave* out) {
  const auto& p = e->e.pass();
  if (!p.saves.empty()) memcpy(out, p.saves.data(), p.saves.size() * sizeof(esp_kvsave));
  return int(p.saves.size());
}
int esp_engine_pass_cow(const esp_engine* e, int32_t* out) {
  const auto& p = e->e.pass();
  if (!p.cow.empty()) memcpy(out, p.cow.data(), p.cow.size() * 8);
  return int(p.cow.size());
}
int esp_engine_pass_rings(const esp_engine* e, int32_t window, int32_t ring_blocks, esp_tree* trees, esp_kvsave* saves,
                          int32_t saves_cap, int32_t* n_saves, int32_t* copies, int32_t copies_cap, int32_t* n_copies, char* err,
                          size_t errlen) {
  try {
    const auto r = e->e.ring_plan(window, ring_blocks);
    if (n_saves) *n_saves = int32_t(r.saves.size());
    if (n_copies) *n_copies = int32_t(r.copies.size());
    if (int(r.saves.size()) > saves_cap || int(r.copies.size()) > copies_cap || (!r.saves.empty() && !saves) ||
        (!r.copies.empty() && !copies) || !trees)
      return put_err(err, errlen, ESP_EWORKSPACE, "pass_rings: output arrays too small (counts written)");
    memcpy(trees, r.trees.data(), r.trees.size() * sizeof(esp_tree));
    if (!r.saves.empty()) memcpy(saves, r.saves.data(), r.saves.size() * sizeof(esp_kvsave));
    if (!r.copies.empty()) memcpy(copies, r.copies.data(), r.copies.size() * 8);
    return ESP_OK;
  } catch (const std::exception& ex) {
    return put_err(err, errlen, ESP_EINVAL, ex.what());
  }
}
int esp_kv_row_table(const esp_kvsave* saves, int32_t n_saves, int32_t rows, int32_t* out, char* err, size_t errlen) {
  try {
    const std::vector<int32_t> t = espetero::engine::row_table(saves, n_saves, rows);
    memcpy(out, t.data(), size_t(std::max(rows, 1)) * 16);
    return 0;
  } catch (const std::exception& ex) {
    if (err && errlen) snprintf(err, errlen, "%s", ex.what());
    return 1;
  }
}
int esp_slot_file_save(const char* path, int32_t len, int32_t next_pos, int32_t n_blocks, int32_t n_layers, uint64_t block_bytes,
                       const void* kv) {
  if (!path || len < 0 || n_blocks < 0 || n_layers < 0 || (!kv && n_blocks > 0 && n_layers > 0)) return -1;
  espetero::engine::SlotInfo s;
  s.len = len, s.next_pos = next_pos, s.n_blocks = n_blocks, s.n_layers = n_layers, s.block_bytes = block_bytes;
  return espetero::engine::slot_file_save(path, s, kv) ? 0 : -1;
}
int esp_slot_file_info(const char* path, int32_t bt, int32_t* len, int32_t* next_pos, int32_t* n_blocks, int32_t* n_layers,
                       uint64_t* block_bytes) {
  if (!path || bt <= 0) return -1;
  espetero::engine::SlotInfo s;
  if (espetero::engine::slot_file_info(path, bt, &s) != 0) return -1;
  *len = s.len, *next_pos = s.next_pos, *n_blocks = s.n_blocks, *n_layers = s.n_layers, *block_bytes = s.block_bytes;
  return 0;
}
int esp_slot_file_load(const char* path, int32_t bt, void* kv, uint64_t kv_bytes) {
  if (!path || bt <= 0) return -1;
  espetero::engine::SlotInfo s;
  if (espetero::engine::slot_file_info(path, bt, &s) != 0) return -1;
  if (kv_bytes < uint64_t(s.n_layers) * uint64_t(s.n_blocks) * s.block_bytes) return -1;
  return espetero::engine::slot_file_load(path, s, kv);
}
int esp_slot_file_save_rings(const char* path, int32_t len, int32_t next_pos, int32_t n_blocks, int32_t n_layers,
                             uint64_t block_bytes, const void* kv, int32_t r_layers, int32_t r_blocks, uint64_t rblock_bytes,
                             const void* rings) {
  if (!path || len < 0 || n_blocks < 0 || n_layers < 0 || (!kv && n_blocks > 0 && n_layers > 0)) return -1;
  if (r_layers < 0 || r_blocks < 0 || (!rings && r_layers > 0 && r_blocks > 0 && rblock_bytes > 0)) return -1;
  espetero::engine::SlotInfo s;
  s.len = len, s.next_pos = next_pos, s.n_blocks = n_blocks, s.n_layers = n_layers, s.block_bytes = block_bytes;
  s.r_layers = r_layers, s.r_blocks = r_blocks, s.rblock_bytes = rblock_bytes;
  return espetero::engine::slot_file_save(path, s, kv, rings) ? 0 : -1;
}
int esp_slot_file_info_rings(const char* path, int32_t bt, int32_t* len, int32_t* next_pos, int32_t* n_blocks, int32_t* n_layers,
                             uint64_t* block_bytes, int32_t* r_layers, int32_t* r_blocks, uint64_t* rblock_bytes) {
  if (!path || bt <= 0) return -1;
  espetero::engine::SlotInfo s;
  if (espetero::engine::slot_file_info(path, bt, &s, true) != 0) return -1;
  *len = s.len, *next_pos = s.next_pos, *n_blocks = s.n_blocks, *n_layers = s.n_layers, *block_bytes = s.block_bytes;
  *r_layers = s.r_layers, *r_blocks = s.r_blocks, *rblock_bytes = s.rblock_bytes;
  return 0;
}
int esp_slot_file_load_rings(const char* path, int32_t bt, void* kv, uint64_t kv_bytes, void* rings, uint64_t ring_bytes) {
  if (!path || bt <= 0) return -1;
  espetero::engine::SlotInfo s;
  if (espetero::engine::slot_file_info(path, bt, &s, true) != 0) return -1;
  if (kv_bytes < uint64_t(s.n_layers) * uint64_t(s.n_blocks) * s.block_bytes) return -1;
  if (ring_bytes < s.ring_bytes() || (s.ring_bytes() && !rings)) return -1;
  return espetero::engine::slot_file_load(path, s, kv, rings);
}
int esp_engine_pass_commit(esp_engine* e) { return guarded([&] { e->e.pass_commit(); }); }
int esp_engine_pass_abort(esp_engine* e) { return guarded([&] { e->e.pass_abort(); }); }

}  // extern "C"
