/* espetero_engine.h -- C view of the host-side attention call surface
 * (espetero_amd/engine/ *.hpp, C++20, no device calls): the tile planner, the
 * refcounted KV block pool with copy-on-write block lists, and the builder
 * that turns a pass's trees into the device records esp_attn_forward reads.
 *
 * It replaces, for this path only, what the reference keeps in
 *   plan_tiles / g4_plan_tiles     src/model/impl/forest.h:1378-1433, gemma.h:77-116
 *   kv_alloc / retain / release    src/model/impl/model.h:722-737
 *   Forest::target_blocks          src/model/impl/forest.h:1785-1811
 *   target_new_blocks              src/model/impl/forest.h:1821-1829
 *   leaf hosting, row descriptors  src/model/impl/forest.h:2201-2220, 2374-2443
 *   block tables, kv_save entries  src/model/impl/forest.h:2483-2520
 *   slot commit / PassGuard        src/model/impl/forest.h:2468-2482, 4743-4754
 *   sliding-layer ring planning    src/model/impl/forest.h:2657-2700
 *   slot_alloc/free/reset/fork/len src/model/model.mm:520-553
 *   verify-commit (lengths)        src/model/impl/forest.h:4755-4765, 4846-4861, 5058-5069
 * The C++ headers are the interface a C++ engine includes; these functions
 * exist so that other languages (and the tests) can drive the same code.
 * Errors: 0 / non-zero + message in err, as in espetero_attn.h. Host memory only.
 */
#ifndef ESPETERO_ENGINE_H
#define ESPETERO_ENGINE_H

#include "espetero_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct esp_plan_options {
  int32_t rows_per_tile; /* query rows per tile (reference: 8) */
  int32_t groups_target; /* workgroups a few-tile pass is split up to (reference: 256) */
  int32_t split;         /* reference rule: largest chunk a split is sized to (attn_split, 512) */
  int32_t min_chunk;     /* fewest cached keys of a split tile (attn_min_chunk, 32) */
  int32_t granule;       /* split boundaries are multiples of this (32) */
  int32_t max_splits;    /* parts per tile group (64) */
  int32_t min_span;      /* shorter cached ranges are not split (64) */
  int32_t balanced;      /* 0: the reference's per-tree budget rule; 1: equal keys per workgroup */
  int32_t item_steps;    /* balanced rule, tiled kernel (> 0): groups_target is the workgroups resident at once and the
                            split chunk is the one whose workgroups finish earliest when handed to those slots in
                            dispatch order; this is a workgroup's fixed cost in steps of `granule` keys */
  int32_t part_steps;    /* the same rule: what a split part costs on top (its partial record and the merge) */
  int32_t cut_batch;     /* the same rule: a tile's batch keys are cut like its cached keys where the hand-out says that finishes
                            earlier (a part whose batch range ends early carries esp_tile.last = its last row + 2); 0 in
                            esp_plan_options_mi355x: the merge dispatch costs what the shorter kernel wins */
} esp_plan_options;

/* The reference's constants. */
void esp_plan_options_reference(esp_plan_options* o);
/* Tuned for 256 CUs: rows query rows per tile, workgroups what esp_attn_plan_hint reports for the kernel. */
void esp_plan_options_mi355x(esp_plan_options* o, int32_t rows, int32_t workgroups);

/* Plan a pass. trees[n_trees] in; tiles / jobs out (capacities given; on
 * ESP_EWORKSPACE the needed counts are still written). groups: workgroups per
 * tile (KV heads). window > 0 needs pos (4 ints per row). */
int esp_plan_tiles(const esp_tree* trees, int32_t n_trees, int32_t groups, int32_t window, const int32_t* pos,
                   const esp_plan_options* o, esp_tile* tiles, int32_t tiles_cap, int32_t* n_tiles, esp_combine* jobs,
                   int32_t jobs_cap, int32_t* n_jobs, int32_t* n_parts, char* err, size_t errlen);

/* ---- KV engine: pool + slots + pass builder ---- */
typedef struct esp_engine esp_engine;

/* One tree of a pass: the attention-relevant part of the reference's TreeSpec
 * (src/model/api.h:105-176). Slots: -1 = none. */
typedef struct esp_tree_spec {
  int32_t parent;     /* slot whose cached keys the tree reads */
  int32_t save;       /* slot that receives parent + root[0, save_len) */
  int32_t work;       /* slot that receives parent + whole root */
  int32_t root_len;
  int32_t save_len;   /* 0: whole root */
  int32_t n_leaves;
  const int32_t* leaf_offsets; /* n_leaves + 1 */
  const int32_t* leaf_tokens;
  int32_t commit_chain; /* leaves [0, k) are one chain whose rows are also saved */
  int32_t noncausal;
} esp_tree_spec;

esp_engine* esp_engine_create(int32_t n_blocks, int32_t bt, int32_t n_slots, int32_t max_ctx);
void esp_engine_destroy(esp_engine* e);
int esp_engine_slot_alloc(esp_engine* e);                 /* slot or -1 */
int esp_engine_slot_free(esp_engine* e, int32_t slot);
int esp_engine_slot_reset(esp_engine* e, int32_t slot);
int esp_engine_slot_fork(esp_engine* e, int32_t src, int32_t dst);
/* The engine side of slot_load (src/model/model.mm:694-752): a fresh slot of `len` positions (next rotary position
 * next_pos) in n_blocks newly allocated blocks, for a caller that then brings the blocks' contents in
 * (esp_slot_file_load + esp_kv_import_blocks into esp_engine_slot_blocks). Returns the slot, -1 when the counts
 * do not fit each other (len > n_blocks * bt, or beyond max_ctx), -2 when the pool or the slot table has no room:
 * the reference's return codes. Free, reset and fork of a slot that the pending pass reads or writes are refused. */
int esp_engine_slot_adopt(esp_engine* e, int32_t len, int32_t next_pos, int32_t n_blocks);
int esp_engine_slot_len(const esp_engine* e, int32_t slot);
int esp_engine_slot_next_pos(const esp_engine* e, int32_t slot);        /* rotary position of the slot's next token */
/* Verify-commit, the block-pool side of the reference's run_commit (src/model/impl/forest.h:4846-4861,
 * 5058-5069): the first n rows of the chain the slot's last pass kept (esp_tree_spec.commit_chain) become
 * part of the slot - their K / V were saved at their positions by that pass - so its length grows by n and
 * its next position follows; the rest of the chain is dropped. Refused when n exceeds the kept rows or
 * another pass has begun since. slot_chain: the rows that could still be committed. */
int esp_engine_slot_chain(const esp_engine* e, int32_t slot);
int esp_engine_chain_commit(esp_engine* e, int32_t slot, int32_t n, char* err, size_t errlen);
int esp_engine_slot_blocks(const esp_engine* e, int32_t slot, int32_t* out, int32_t cap); /* count */
int esp_engine_free_blocks(const esp_engine* e);
int esp_engine_block_ref(const esp_engine* e, int32_t block);
/* Blocks a pass of these trees would take from the free list (pass_kv_tokens / bt). */
int esp_engine_pass_blocks(const esp_engine* e, const esp_tree_spec* specs, int32_t n);

/* Build a pass: validates every tree before touching anything, then plans
 * rows, descriptors, positions, the block table, kv_save entries and
 * copy-on-write pairs. The block table already names the copies: the caller
 * runs esp_kv_copy_blocks over the pairs before the pass's first attention
 * (the reference's order, forest.h:2726-2729), the saves after it. The pass
 * stays pending until committed or aborted. */
int esp_engine_pass_begin(esp_engine* e, const esp_tree_spec* specs, int32_t n, char* err, size_t errlen);
int esp_engine_pass_rows(const esp_engine* e);      /* M */
int esp_engine_pass_counts(const esp_engine* e, int32_t* n_table, int32_t* n_saves, int32_t* n_cow);
int esp_engine_pass_trees(const esp_engine* e, esp_tree* out);          /* n trees */
int esp_engine_pass_desc(const esp_engine* e, int32_t* out);            /* 4 * M */
int esp_engine_pass_pos(const esp_engine* e, int32_t* out);             /* 4 * M */
int esp_engine_pass_table(const esp_engine* e, int32_t* out);
int esp_engine_pass_saves(const esp_engine* e, esp_kvsave* out);
int esp_engine_pass_cow(const esp_engine* e, int32_t* out);             /* 2 * n_cow */
/* The pending pass on sliding layers (replaces the ring planning of src/model/impl/forest.h:2657-2700):
 * slot s keeps its last `window` positions in a second pool, in the ring_blocks consecutive blocks from
 * s * ring_blocks on, position p in block (p / bt) % ring_blocks. Writes the trees as those layers read
 * them (table = first block of the parent's ring; n trees of the pass), the save entries of the rows that
 * are still inside the window when the pass ends, and (source, destination) block copies that carry the
 * parent's window into the ring of a target that is another slot (copies before the attention, saves
 * after it). A pass whose ring saves have run is committed: an in-place chunk's saves reuse ring cells the
 * slot would still need if it did not advance. esp_engine_slot_fork has a ring side too, the caller's: copy
 * the source's whole ring, blocks src * ring_blocks + i -> dst * ring_blocks + i (copy_slot_state,
 * src/model/impl/forest.h:127-137), with esp_kv_copy_blocks on the ring pool.
 * ESP_EWORKSPACE when saves_cap / copies_cap are too small: the needed counts are still written. */
int esp_engine_pass_rings(const esp_engine* e, int32_t window, int32_t ring_blocks, esp_tree* trees, esp_kvsave* saves,
                          int32_t saves_cap, int32_t* n_saves, int32_t* copies, int32_t copies_cap, int32_t* n_copies,
                          char* err, size_t errlen);
/* Slot checkpoint files in the reference's format (src/model/model.mm:600-752), KV section: the
 * 120-byte CkptHeader (magic 0x554b5043, version 4), then n_layers x n_blocks blocks of block_bytes,
 * layer-major, logical block order, each in the reference's block layout (what
 * esp_kv_export_blocks produces per layer). The sections of other subsystems are written as absent;
 * a file with a ring section is refused here (the _rings variants below take it).
 * kv: host memory. save: 0 or -1. info / load: 0, or -1 for a missing, malformed, wrong-version or
 * wrong-size file or one with sections this build does not take (slot_load's -1, model.mm:700-714). */
int esp_slot_file_save(const char* path, int32_t len, int32_t next_pos, int32_t n_blocks, int32_t n_layers, uint64_t block_bytes,
                       const void* kv);
int esp_slot_file_info(const char* path, int32_t bt, int32_t* len, int32_t* next_pos, int32_t* n_blocks, int32_t* n_layers,
                       uint64_t* block_bytes);
int esp_slot_file_load(const char* path, int32_t bt, void* kv, uint64_t kv_bytes);
/* The same with the file's last section, Gemma's sliding rings (model.mm:664-669, 737-742): after the KV
 * blocks, r_layers x r_blocks ring blocks of rblock_bytes, layer-major, the slot's ring in ring order
 * (what esp_kv_export_blocks produces from the ring pool for blocks slot * r_blocks + 0 .. r_blocks - 1).
 * info / load take files with and without rings; a loader must still hold the counts against its own
 * model (r_layers, r_blocks, rblock_bytes: slot_load's checks, model.mm:703-705). */
int esp_slot_file_save_rings(const char* path, int32_t len, int32_t next_pos, int32_t n_blocks, int32_t n_layers,
                             uint64_t block_bytes, const void* kv, int32_t r_layers, int32_t r_blocks, uint64_t rblock_bytes,
                             const void* rings);
int esp_slot_file_info_rings(const char* path, int32_t bt, int32_t* len, int32_t* next_pos, int32_t* n_blocks, int32_t* n_layers,
                             uint64_t* block_bytes, int32_t* r_layers, int32_t* r_blocks, uint64_t* rblock_bytes);
int esp_slot_file_load_rings(const char* path, int32_t bt, void* kv, uint64_t kv_bytes, void* rings, uint64_t ring_bytes);
/* kv_row_table (src/model/impl/forest.h:1737-1749): the pass's save records as one int32[4] per row,
 * (block, position, block2, position2), -1 none - the row_table argument of esp_attn_prep.
 * out: 4 * max(rows, 1) ints. Fails on a row saved into more than two slots. Needs no engine. */
int esp_kv_row_table(const esp_kvsave* saves, int32_t n_saves, int32_t rows, int32_t* out, char* err, size_t errlen);
/* The slots take their new block lists (after the device work completed). */
int esp_engine_pass_commit(esp_engine* e);
/* Give the pass's new blocks back; slots are as before the pass. */
int esp_engine_pass_abort(esp_engine* e);

#ifdef __cplusplus
}
#endif
#endif
