/* espetero_attn.h -- C ABI of the MI355X (gfx950) paged-KV attention path.
 *
 * This is the boundary a host engine binds instead of the reference's
 * per-dispatch kernel ABI (pipeline name + buffers 0..11 + by-value params):
 *   reference kernels   kernels/40_attention.metal:155-905,
 *                       kernels/80_gemma.metal:157-601,
 *                       kernels/82_qwen3_omni.metal:97-106
 *   reference bindings  src/model/impl/forest.h:2855-2947,
 *                       src/model/impl/gemma.h:223-303,
 *                       src/model/impl/qwen3_omni.h:96-161
 *   host record structs src/model/impl/forest.h:1308-1345, gemma.h:29-35
 *
 * Conventions (the reference's dlopen'd C ABI uses the same ones,
 * tests/parity_test.mm:37-57): every function returns 0 on success or a
 * non-zero ESP_E* code and writes a NUL-terminated message into `err`
 * (may be NULL). No function throws, allocates or frees device memory, or
 * synchronises the device: work is enqueued on `stream` (a hipStream_t passed
 * as void*; NULL = the default stream) and the caller orders it. All pointer
 * arguments other than `p`, `err` are DEVICE pointers unless stated. Like the
 * reference's model object (src/model/api.h:4-6) the library is driven from
 * one thread at a time.
 *
 * KV pool layout ("native", ESP_LAYOUT_NATIVE). One region per attention
 * layer starting at element offset kv_base, n_blocks blocks per region, each
 * block 2 * bt * Hkv * head_dim elements (the reference's block size,
 * src/model/impl/model.h:396), arranged for 64-wide wavefronts as
 *   block b, KV head h : base = kv_base + (b * Hkv + h) * 2 * bt * head_dim
 *   K[token t][dim d]  : base + t * head_dim + d                (row major)
 *   V[token t][dim d]  : base + bt * head_dim + (t / 16) * 16 * head_dim + d * 16 + t % 16
 *                        (transposed, in sub-blocks of 16 tokens)
 * so one (block, head) is a single contiguous run, V is already the
 * k-contiguous operand of the P.V matrix product, and 16 keys of K or of V
 * are 32 * head_dim contiguous bytes whatever the block size. The reference's layout
 * (ESP_LAYOUT_REFERENCE, kernels/40_attention.metal:245-247) is
 *   K/V[which][t][h][d]: kv_base + (2 b + which) * bt * kv_ld + t * kv_ld + h * head_dim + d
 * and is accepted only by esp_kv_relayout (import / export of blocks).
 */
#ifndef ESPETERO_ATTN_H
#define ESPETERO_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ESP_ABI_VERSION 3

enum { ESP_OK = 0, ESP_EINVAL = 1, ESP_EUNSUPPORTED = 2, ESP_ELAUNCH = 3, ESP_EWORKSPACE = 4 };
enum { ESP_F16 = 0, ESP_BF16 = 1 };
enum { ESP_LAYOUT_REFERENCE = 0, ESP_LAYOUT_NATIVE = 1 };

/* One sequence-in-pass. Field for field AttnTree (kernels/40_attention.metal:134-139,
 * host AttnTreeRec src/model/impl/forest.h:1308-1310). */
typedef struct esp_tree {
  int32_t base;  /* absolute first row of the tree in Q/Kb/Vb/O/desc/pos */
  int32_t P;     /* cached keys [0, P) */
  int32_t table; /* first entry of its block list in `blocks`; ring layers: first ring block */
  int32_t M;     /* rows of the tree in this pass */
} esp_tree;

/* One unit of GPU work. Field for field G4Tile (kernels/80_gemma.metal:146-155,
 * host G4TileRec src/model/impl/gemma.h:29-31); AttnTile (40_:141-150) is the
 * same record with b0 = pad = 0. */
typedef struct esp_tile {
  int32_t tree;
  int32_t r0;   /* absolute first query row; the tile covers rows_per_tile rows (fewer at the tree's end) */
  int32_t k0;   /* cached-key range [k0, k1) */
  int32_t k1;
  int32_t part; /* -1: write O; else index of the partial record this tile writes */
  int32_t last; /* 0: cached keys only; 1 (the reference's value): also the tree's batch keys (this pass's own rows) from b0 on;
                   e + 2: also the batch keys b0 .. e and no further (no counterpart in the reference, whose planner never cuts
                   the batch keys: this library's balanced rule does when a pass has fewer workgroups than the chip has room
                   for; the parts of such a group partition the batch keys as they partition the cached ones) */
  int32_t b0;   /* first batch key (relative row) any row of the tile may see; of a part with a cut batch range, its first */
  int32_t pad;  /* 0 (the reference's value), or 1 + the tree's `table`: lets a kernel skip the tree lookup */
} esp_tile;

/* Merge job of one split tile group. Field for field AttnCombine (40_:804-809). */
typedef struct esp_combine {
  int32_t r0;     /* absolute first row */
  int32_t rows;   /* live rows */
  int32_t part0;  /* first partial record */
  int32_t nparts; /* records, merged in order part0, part0 + 1, ... */
} esp_combine;

/* KV append entry. Field for field KVSave (40_:868-873, forest.h:1317-1319). */
typedef struct esp_kvsave {
  int32_t src_row;
  int32_t block;
  int32_t pos; /* token index within the block */
  int32_t pad;
} esp_kvsave;

/* Per-layer constants: G4AttnParams (80_:134-144) + AttnParams' gate stride
 * (40_:124-132) + what the Metal templates fix at compile time (head_dim,
 * element type, score scale). */
typedef struct esp_attn_params {
  int32_t H;             /* query heads */
  int32_t Hkv;           /* KV heads; H % Hkv == 0, group G = H / Hkv */
  int32_t head_dim;      /* 128, 256 or 512 (512: the g4_attention512_s* / g4_attention_dec512_g* instantiations,
                            80_:355-358, :561-564; up to 32 packed rows on the streaming kernel like the other head dims, 64-row tiles
                            on the tiled one: esp_attn_plan_hint's max_rows) */
  int32_t dtype;         /* ESP_F16 | ESP_BF16: element type of Q, Kb, Vb, pool and O */
  int32_t q_ld;          /* Q / O row stride in elements (>= H * head_dim) */
  int32_t kv_ld;         /* Kb / Vb row stride in elements (>= Hkv * head_dim) */
  int32_t bt;            /* tokens per KV block, a multiple of 16 */
  int32_t window;        /* sliding window (0: none): key visible iff qpos - kpos < window */
  int32_t ring;          /* blocks per slot ring on sliding layers (0: block lists) */
  int32_t bidi;          /* image rows see their whole image (desc.w) */
  int32_t rows_per_tile; /* query rows per tile the planner used (the reference: 8) */
  float scale;           /* multiplies q.k (1 when q arrives pre-scaled) */
  uint64_t kv_base;      /* element offset of this layer's region in the pool */
  const float* gate;     /* optional sigmoid output gate (40_:334-342), NULL: none */
  int32_t gate_ld;       /* gate[row * gate_ld + h * gate_hs + gate_off + d] */
  int32_t gate_hs;
  int32_t gate_off;
  int32_t gate_headwise; /* 1: one gate value per (row, head), the address above without "+ d": the
                            head-wise gate of 85_spark.metal:96-128 taken into the output's one
                            rounding, its dots computed before the pass by esp_head_gate */
} esp_attn_params;

/* Library / device check and the per-device set-up: looks up this GPU's copy of the library's own
 * device arrays and raises the dynamic LDS limit of every kernel variant, so that the first launch of
 * any variant may happen inside a stream capture. Safe to call more than once; a call that was not
 * preceded by it does the same set-up on first use of a device. */
int esp_attn_init(int device, char* err, size_t errlen);
int esp_attn_abi_version(void);

/* What the planner needs to know about the kernel that serves these params
 * (rows_per_tile x G packed rows, head_dim, dtype):
 *   workgroups      how many workgroups of the kernel are resident at once: what the
 *                   streaming kernel's pass is split up to (a second round pays its
 *                   per-workgroup set-up again), and the slots the tiled kernel's
 *                   planner hands its workgroups to when it picks the split that
 *                   finishes earliest (the reference aims at a fixed 256
 *                   threadgroups, forest.h:1385);
 *   groups_per_tile workgroups one tile becomes: KV heads for the streaming
 *                   kernel (the G heads of a KV head share a workgroup), query
 *                   heads for the tiled kernel (the reference: KV heads x SPLIT,
 *                   forest.h:2920, gemma.h:231);
 *   max_rows        the largest rows_per_tile the tiled kernel takes at this
 *                   head_dim: what a prefill pass should plan with (the
 *                   reference: 8, or 16 on Spark prompt passes, gemma.h:137-142). */
int esp_attn_plan_hint(const esp_attn_params* p, int device, int32_t* workgroups, int32_t* groups_per_tile,
                       int32_t* max_rows, char* err, size_t errlen);

/* Bytes of `workspace` esp_attn_forward needs for a pass of n_rows batch rows
 * whose plan holds n_parts partial records (replaces the reference's `parts`
 * sizing, forest.h:2716, gemma.h:162-165). Host-only arithmetic. */
size_t esp_attn_workspace_bytes(const esp_attn_params* p, int32_t n_rows, int32_t n_parts);

/* Attention of one layer over a planned pass, then the split-K merge:
 * replaces the dispatch of flash_attention / attn_decode_gqa / g4_attention /
 * g4_attention_dec and attention_combine (forest.h:2895-2933, gemma.h:249-284).
 * Q [n_rows][q_ld], Kb/Vb [n_rows][kv_ld] (this pass's rows, not yet cached),
 * desc/pos: int32[4] per row (desc = seg_start, 0, anc_len, img_end; pos.x =
 * position); desc may be NULL (plain causal rows), pos may be NULL when
 * window == 0. O [n_rows][q_ld]. The kernel family is chosen from
 * rows_per_tile * G (streaming split-K kernel up to 32 packed rows, tiled
 * MFMA kernel above), as the reference chooses from its plan (forest.h:2863-2868).
 * n_jobs = 0 with n_parts > 0 skips the merge (see esp_attn_combine).
 * Kb and Vb both NULL: the pass's rows are already in the pool - appended before this call by esp_attn_prep with a
 * row_table (the reference's fold of kv_save into attn_prep, 40_:86-100) or by esp_kv_save - row j of a tree at
 * position P + j of the tree's own block list, and the kernels read them from there: no Kb / Vb round trip through
 * memory and no staging copy in front of the tiled kernel. What the caller promises with it is what
 * esp_attn_validate_for(ESP_PASS_ROWS_IN_POOL) checks; a pass that cannot promise it (verify trees whose rows are
 * not stored behind their parent's keys, P - base not a multiple of 16 on the tiled kernel) passes Kb / Vb. */
int esp_attn_forward(const esp_attn_params* p, const void* Q, const void* Kb, const void* Vb, const void* kv_pool,
                     const int32_t* blocks, const int32_t* desc, const int32_t* pos, void* O, const esp_tile* tiles,
                     int32_t n_tiles, const esp_tree* trees, int32_t n_trees, const esp_combine* jobs, int32_t n_jobs,
                     int32_t n_parts, int32_t n_rows, void* workspace, size_t workspace_bytes, void* stream, char* err,
                     size_t errlen);

/* esp_attn_forward without a workspace and without any allocation: no counterpart in the reference
 * (its encoder takes every buffer from the model's arena, forest.h:2716); it is for callers that
 * cannot allocate device memory - code under HIP graph capture, tight serving loops, harnesses that
 * forbid it. The partial records and the transposed batch V live in a device array of
 * ESP_STATIC_SCRATCH_BYTES that the library holds on every GPU it runs on until the process ends; a
 * pass that needs more (esp_attn_workspace_bytes) is refused with ESP_EWORKSPACE. Everything else as
 * esp_attn_forward, same kernels, same results. Every call on a GPU shares that GPU's array: calls that
 * overlap on one GPU (two streams, two threads) race; calls on one stream are ordered and safe. */
#define ESP_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
int esp_attn_forward_static(const esp_attn_params* p, const void* Q, const void* Kb, const void* Vb, const void* kv_pool,
                            const int32_t* blocks, const int32_t* desc, const int32_t* pos, void* O, const esp_tile* tiles,
                            int32_t n_tiles, const esp_tree* trees, int32_t n_trees, const esp_combine* jobs, int32_t n_jobs,
                            int32_t n_parts, int32_t n_rows, void* stream, char* err, size_t errlen);

/* Host-side check of a pass's records before they are uploaded; no counterpart in the reference, whose
 * planner and kernels live in one program (forest.h:2646-2716). The kernels trust every index they
 * read from device memory, and a bad one is an out-of-bounds access on the GPU. ALL pointers here are
 * HOST pointers to the same records esp_attn_forward will read: every tree's rows inside [0, n_rows),
 * its block list inside blocks[0, n_block_entries) with ids below pool_blocks (ring layers: its ring
 * inside the pool), every tile's tree, rows, cached range, partial record and table hint, every job's
 * rows and records, each record written by one tile and merged by one job. ESP_EINVAL + message names
 * the first offender. Touches no device. */
int esp_attn_validate(const esp_attn_params* p, const esp_tile* tiles, int32_t n_tiles, const esp_tree* trees, int32_t n_trees,
                      const esp_combine* jobs, int32_t n_jobs, int32_t n_parts, int32_t n_rows, const int32_t* blocks,
                      int32_t n_block_entries, int32_t pool_blocks, char* err, size_t errlen);

/* esp_attn_validate for a pass that will run in one of the forms whose promises only the records can answer (they
 * live in device memory when the pass runs). mode, a sum of
 *   ESP_PASS_FUSED         the pass goes to esp_attn_decode_fused: every tree at most rows_per_tile rows and every tile
 *                          starting at its tree's first row, i.e. one tile group per tree;
 *   ESP_PASS_ROWS_IN_POOL  the pass goes to esp_attn_forward without Kb / Vb: row j of every tree is read at position
 *                          P + j of the tree's own block list, which must reach that far; on the tiled kernel P - base
 *                          is a multiple of 16; on ring layers a tree's rows must not overwrite keys its first rows see.
 * Same arguments as esp_attn_validate otherwise. Host pointers; touches no device. */
enum { ESP_PASS_FUSED = 1, ESP_PASS_ROWS_IN_POOL = 2 };
int esp_attn_validate_for(const esp_attn_params* p, int32_t mode, const esp_tile* tiles, int32_t n_tiles, const esp_tree* trees,
                          int32_t n_trees, const esp_combine* jobs, int32_t n_jobs, int32_t n_parts, int32_t n_rows, const int32_t* blocks,
                          int32_t n_block_entries, int32_t pool_blocks, char* err, size_t errlen);

/* Measurement hook; no counterpart in the reference (its bench times command
 * buffers, src/model/impl/bench.h:697-722). The next esp_attn_forward (or
 * esp_attn_prep) hands the two HIP events (hipEvent_t, created with timing
 * enabled) to the launch of its main kernel - the streaming or the tiled
 * attention kernel, not the staging copy or the merge; the prep kernel - which
 * records the kernel's own begin and end
 * into them: hipEventElapsedTime(start, stop) is then that kernel's duration,
 * without marker packets between the kernels of the stream. The pair is used
 * once, by the next such call, whether or not that call launches anything (a call
 * that returns early drops it). One pending pair per calling thread: the
 * thread that arms it makes the call that takes it; other threads' calls neither see nor consume it. Both NULL clears a pending pair. */
int esp_attn_time_next(void* start_event, void* stop_event);

/* The split-K merge alone: attention_combine (40_:811-864, 80_:568-597) as its
 * own dispatch, for callers that passed n_jobs = 0 to esp_attn_forward (a
 * plan with n_parts > 0 then leaves its partial records in `workspace`). Same
 * params, O, workspace and counts as that call. */
int esp_attn_combine(const esp_attn_params* p, void* O, const esp_combine* jobs, int32_t n_jobs, int32_t n_parts,
                     int32_t n_rows, void* workspace, size_t workspace_bytes, void* stream, char* err, size_t errlen);

/* Append batch rows to the pool: replaces kv_save (40_:875-889; forest.h:2935-2947). */
int esp_kv_save(const esp_attn_params* p, const void* Kb, const void* Vb, void* kv_pool, const esp_kvsave* entries,
                int32_t n_entries, void* stream, char* err, size_t errlen);

/* Copy whole blocks src -> dst in every layer region (copy on write): replaces
 * kv_copy_blocks (40_:894-905; forest.h:1438-1449). pairs: int32[2] per pair;
 * region_elems: elements per layer region. */
int esp_kv_copy_blocks(const esp_attn_params* p, void* kv_pool, const int32_t* pairs, int32_t n_pairs, int32_t n_layers,
                       uint64_t region_elems, void* stream, char* err, size_t errlen);

/* Gather a block list's first n_tokens tokens into contiguous rows
 * K_out / V_out [n_tokens][Hkv * head_dim] (the order of the reference's slot
 * files, src/model/model.mm:600-752: logical token order, K then V). Bit copy. */
int esp_kv_gather(const esp_attn_params* p, const void* kv_pool, const int32_t* blocks, int32_t n_tokens, void* K_out,
                  void* V_out, void* stream, char* err, size_t errlen);

/* Convert n_blocks whole blocks of one layer region between the reference's
 * block layout and the native one. src_pool / dst_pool point at the first
 * block of the region (kv_base is not applied); they must not overlap.
 * src_layout / dst_layout: ESP_LAYOUT_*. Bit copy. */
int esp_kv_relayout(const esp_attn_params* p, const void* src_pool, int32_t src_layout, void* dst_pool, int32_t dst_layout,
                    int32_t n_blocks, void* stream, char* err, size_t errlen);

/* The KV payload of a slot checkpoint file (src/model/model.mm:649-655 writes, :727-729 reads): for one
 * layer (p->kv_base), the slot's blocks in logical order, each in the reference's block layout
 * [K plane | V plane][token][kv head][dim]. export: block blocks[i] of the native pool -> block i of
 * `out`; import: block i of `in` -> block blocks[i] of the native pool. kv_pool is the pool's base
 * (kv_base is applied). out / in: device memory, n_blocks * 2 * bt * Hkv * head_dim elements. Bit copies. */
int esp_kv_export_blocks(const esp_attn_params* p, const void* kv_pool, const int32_t* blocks, int32_t n_blocks, void* out,
                         void* stream, char* err, size_t errlen);
int esp_kv_import_blocks(const esp_attn_params* p, const void* in, const int32_t* blocks, int32_t n_blocks, void* kv_pool,
                         void* stream, char* err, size_t errlen);

/* ---- attn_prep: the step before the attention of a layer ----------------------
 * One entry point for the reference's three prep kernels:
 *   attn_prep        kernels/40_attention.metal:9-102   (AttnPrepParams; binding forest.h:2951-2977)
 *   g4_attn_prep<HD> kernels/80_gemma.metal:52-108      (G4PrepParams;   binding gemma.h:455-475)
 *   q3m_attn_prep<HD> kernels/82_qwen3_omni.metal:30-88 (Q3PrepParams;   binding qwen3_omni.h:286-302)
 * Per row of the fp32 fused projection X: every query and key head gets
 * x * rsqrt(mean(x^2) + eps) * weight, then the rotation of its first rope_dims
 * dims in the half-split pairing (d, d + rope_dims/2) by angle
 * position * inv_freq[d mod rope_dims/2], then the cast to the storage type;
 * queries are multiplied by q_scale after the rotation. Values are cast, or
 * normalised without weight first (v_norm). */
typedef struct esp_prep_params {
  int32_t H, Hkv, head_dim, dtype;
  int32_t x_ld;      /* floats between rows of X */
  int32_t q_off;     /* column of query head 0 */
  int32_t q_hs;      /* floats between query heads: head_dim, or 2 * head_dim with a gate beside each query (40_:47) */
  int32_t k_off;     /* column of key head 0 (key heads head_dim apart) */
  int32_t v_off;     /* column of value head 0 */
  int32_t q_ld;      /* Q output row stride, elements */
  int32_t kv_ld;     /* Kb / Vb output row stride, elements */
  int32_t rope_dims; /* 64 in 40_:58-71, head_dim in 80_:99-104 and 82_:75-82, 0: no rotation; a power of two >= 8
                        (>= 16 at head_dim 512, g4_attn_prep512, 80_:113) */
  int32_t v_norm;    /* 1: 80_:92-96; 0: 40_:81-83, 82_:58-62 */
  int32_t bt;        /* tokens per KV block, for the folded append */
  float eps;
  float q_scale;     /* 82_:84; 1 in the other two */
  uint64_t kv_base;  /* element offset of the layer's pool region, for the folded append */
} esp_prep_params;

/* X [n_rows][x_ld] fp32; qn_w / kn_w [head_dim] fp32; pos int32[4] per row (x, y, z
 * position components); inv_freq [rope_dims / 2]; rope_sel [rope_dims / 2]: which position
 * component each frequency rotates by (40_:62-63, 82_:77-79), NULL: all by pos.x (80_:99).
 * Q [n_rows][q_ld], Kb / Vb [n_rows][kv_ld]: storage type; with a row_table Kb and Vb may both be NULL (the rows
 * then live in the pool alone, for an attention call that reads them there).
 * row_table NULL, or int32[4] per row = (block, position, block2, position2), -1 none
 * (kv_row_table, forest.h:1737-1749): the row's K and V also go to those entries of
 * kv_pool in the native layout, which replaces the kv_save dispatch after the attention
 * (40_:86-100). The reference launches one SIMD group per (row, head); here one workgroup
 * takes a row and computes the row's cos / sin once. */
int esp_attn_prep(const esp_prep_params* p, const float* X, const float* qn_w, const float* kn_w, const int32_t* pos,
                  const float* inv_freq, const int32_t* rope_sel, void* Q, void* Kb, void* Vb, const int32_t* row_table,
                  void* kv_pool, int32_t n_rows, void* stream, char* err, size_t errlen);

/* attn_prep fused into the attention of a decode or short verify pass: replaces the attn_prep dispatch in front
 * of attn_decode_gqa / g4_attention_dec (the reference encodes the two one after the other, forest.h:4061-4078; its
 * own fold of kv_save into attn_prep is 40_attention.metal:86-100). Every workgroup of the streaming kernel
 * prepares what it needs itself from the fp32 projection X - the query heads of its tile, and on a tree's `last`
 * tile the rows' key and value of its KV head, which it also appends to the pool through row_table - with the
 * arithmetic of esp_attn_prep, bit for bit; Q, Kb and Vb are never written. Arguments as in esp_attn_prep
 * (pp, X .. rope_sel, row_table, kv_pool) and esp_attn_forward (the rest); pos serves both. Limits: head dim 128
 * or 256, rows_per_tile <= 4, packed rows within the streaming kernel's (rows_per_tile * G <= 32, <= 16 at head
 * dim 256), and every tree of the pass at most rows_per_tile rows, i.e. one tile group per tree. O is what
 * esp_attn_prep followed by esp_attn_forward gives, and so are the pool entries. */
int esp_attn_decode_fused(const esp_prep_params* pp, const esp_attn_params* p, const float* X, const float* qn_w, const float* kn_w,
                          const int32_t* pos, const float* inv_freq, const int32_t* rope_sel, const int32_t* row_table,
                          void* kv_pool, const int32_t* blocks, const int32_t* desc, void* O, const esp_tile* tiles,
                          int32_t n_tiles, const esp_tree* trees, int32_t n_trees, const esp_combine* jobs, int32_t n_jobs,
                          int32_t n_parts, int32_t n_rows, void* workspace, size_t workspace_bytes, void* stream, char* err,
                          size_t errlen);

/* ---- decode chains ---------------------------------------------------------------
 * The reference runs K greedy decode steps as one GPU chain (run_chain,
 * src/model/model.mm:779-850, docs/design.md:226-243): the host encodes the K
 * passes one after the other (run_forest per step, each with its own tree,
 * position and KV-entry records from the pass arena) and waits once at the end. Here the records stay where they are and the
 * device moves them on, so a chain is a sequence of enqueues with no host work
 * in between, and can be captured in a HIP graph:
 *   - a tile whose k1 is INT32_MAX ends at its tree's cached length P as the
 *     trees array holds it when the kernel runs (both attention kernels);
 *   - esp_chain_advance turns the records of a pass of single-row trees into
 *     those of the next step: P + 1, every position component + 1, and the
 *     row's row_table entry (esp_attn_prep) = the pool entry of position P + 1
 *     taken from the tree's block list (or its ring). The block lists must
 *     already hold the blocks the chain will reach (the reference reserves
 *     them before the pass too: target_new_blocks, forest.h:1821-1829, model.mm:575).
 * trees, pos (int32[4] per row), row_table (int32[4] per row, may be NULL),
 * blocks: device memory. Trees with M != 1 are not meant for it. */
int esp_chain_advance(esp_tree* trees, int32_t n_trees, int32_t* pos, int32_t* row_table, const int32_t* blocks, int32_t bt,
                      int32_t ring, void* stream, char* err, size_t errlen);

/* ---- the head-wise output gate: the step after the attention of a layer ----------
 * sp_head_gate (kernels/85_spark.metal:96-128, SpGateParams :99-104; binding
 * src/model/impl/gemma.h:481-492): O[row, h, :] *= sigmoid(x[row] . Wg[h]) with x the layer's
 * normed input and Wg = g_proj, one gate per (row, query head). The reference runs one
 * threadgroup per (head, row) after the attention and rounds O a second time. Two ways here:
 *   - O != NULL: as the reference, in place: O = storage(float(O) * gate), dots NULL or not;
 *   - dots != NULL: the pre-activation dots x . Wg[h] as fp32 [n_rows][H], to be handed to
 *     the attention as params.gate with gate_headwise = 1 (gate_ld = H, gate_hs = 1,
 *     gate_off = 0): the attention then multiplies before its one rounding and O makes no
 *     second trip through memory. This call can run before the attention (x is the layer's input).
 * At least one of O and dots. X [n_rows][x_ld], Wg [H][D], O [n_rows][q_ld]: storage type
 * (the reference: fp16). D % 8 == 0 (the reference: % 4), head_dim % 8 == 0 and <= 1024
 * as in the reference (:98), H <= 64. */
typedef struct esp_gate_params {
  int32_t H;        /* query heads */
  int32_t head_dim; /* SpGateParams.hd */
  int32_t D;        /* model width: length of the dots */
  int32_t dtype;    /* ESP_F16 | ESP_BF16 */
  int32_t q_ld;     /* O row stride, elements (SpGateParams.q_ld) */
  int32_t x_ld;     /* X row stride, elements (the reference: D) */
} esp_gate_params;

int esp_head_gate(const esp_gate_params* p, void* O, const void* X, const void* Wg, float* dots, int32_t n_rows,
                  void* stream, char* err, size_t errlen);

#ifdef __cplusplus
}
#endif
#endif /* ESPETERO_ATTN_H */
