// The C ABI (include/espetero_attn.h): argument checks, workspace carving and
// kernel selection. Nothing here allocates device memory or synchronises.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

#include "common.hpp"

namespace esp {
hipError_t launch_stream(int dt, int HD, int NC, const KArgs& a, const PrepArgs* pa, int n_tiles, hipStream_t st);
hipError_t launch_combine(int dt, int HD, const KArgs& a, const esp_combine* jobs, int n_jobs, int n_parts, hipStream_t st);
hipError_t launch_tiled(int dt, int HD, const KArgs& a, int n_tiles, hipStream_t st);
hipError_t launch_kv_save(const esp_attn_params* p, const void* Kb, const void* Vb, void* pool, const esp_kvsave* e, int n,
                          hipStream_t st);
hipError_t launch_kv_copy_blocks(const esp_attn_params* p, void* pool, const int32_t* pairs, int n_pairs, int n_layers,
                                 uint64_t region_elems, hipStream_t st);
hipError_t launch_kv_gather(const esp_attn_params* p, const void* pool, const int32_t* blocks, int n, void* K_out,
                            void* V_out, hipStream_t st);
hipError_t launch_kv_relayout(const esp_attn_params* p, const void* src, void* dst, int to_native, int n_blocks,
                              const int32_t* ids, hipStream_t st);
hipError_t launch_chain_advance(esp_tree* trees, int n_trees, int32_t* pos, int32_t* row_table, const int32_t* blocks, int bt,
                                int ring, hipStream_t st);
hipError_t launch_vt_stage(const esp_attn_params* p, const void* Vb, void* vt, int n_rows, hipStream_t st);
hipError_t launch_attn_prep(const PrepArgs& a, int n_rows, hipStream_t st);
hipError_t launch_head_gate(int dt, const GateArgs& a, hipStream_t st);
int stream_workgroups_per_cu(int HD, int NC);
int tiled_workgroups_per_cu(int HD);
int tiled_max_rows(int HD);
hipError_t stream_init_attributes();
hipError_t tiled_init_attributes();
hipError_t tiled512_init_attributes();
}  // namespace esp

// Library-owned device memory, one copy per GPU, held until the process ends: what
// esp_attn_forward_static uses in place of a caller's workspace (partial records of split tiles, the
// transposed batch V of the tiled kernels). In host code this name is a stand-in, not a device
// address: the address comes from hipGetSymbolAddress, once per device (device_state below), and only
// that is handed to kernels.
constexpr size_t kScratchBytes = ESP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

int fail(char* err, size_t errlen, int code, const char* fmt, ...) {
  if (err && errlen) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(err, errlen, fmt, ap);
    va_end(ap);
  }
  return code;
}

int hip_fail(char* err, size_t errlen, const char* what, hipError_t e) {
  return fail(err, errlen, ESP_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
}

// Checks shared by every entry point. Returns 0 or an error code.
int check_params(const esp_attn_params* p, char* err, size_t errlen) {
  if (!p) return fail(err, errlen, ESP_EINVAL, "params is NULL");
  if (p->H <= 0 || p->Hkv <= 0 || p->H % p->Hkv) return fail(err, errlen, ESP_EINVAL, "H=%d Hkv=%d: H must be a positive multiple of Hkv", p->H, p->Hkv);
  if (p->head_dim != 128 && p->head_dim != 256 && p->head_dim != 512)
    return fail(err, errlen, ESP_EUNSUPPORTED, "head_dim %d (128, 256 or 512)", p->head_dim);
  if (p->dtype != ESP_F16 && p->dtype != ESP_BF16) return fail(err, errlen, ESP_EINVAL, "dtype %d", p->dtype);
  if (p->bt <= 0 || p->bt % 16) return fail(err, errlen, ESP_EINVAL, "bt %d: tokens per block must be a positive multiple of 16", p->bt);
  if (p->q_ld < p->H * p->head_dim || p->q_ld % 8) return fail(err, errlen, ESP_EINVAL, "q_ld %d", p->q_ld);
  if (p->kv_ld < p->Hkv * p->head_dim || p->kv_ld % 8) return fail(err, errlen, ESP_EINVAL, "kv_ld %d", p->kv_ld);
  if (p->kv_base % 8) return fail(err, errlen, ESP_EINVAL, "kv_base must be a multiple of 8 elements");
  if (p->window < 0 || p->ring < 0) return fail(err, errlen, ESP_EINVAL, "window / ring negative");
  if (p->gate_headwise != 0 && p->gate_headwise != 1) return fail(err, errlen, ESP_EINVAL, "gate_headwise %d (0 or 1)", p->gate_headwise);
  return ESP_OK;
}

// Which kernel family serves rows_per_tile x G packed rows: 0 none, else the
// streaming kernel's column tiles (1, 2) or -1 for the tiled kernel.
int family(const esp_attn_params* p) {
  const int packed = p->rows_per_tile * (p->H / p->Hkv);
  const int nc = (packed + 15) / 16;
  // two column tiles: in one wavefront's registers at head dim 128, as two wavefront pairs of one workgroup at head dim 512
  if (nc == 1 || (nc == 2 && (p->head_dim == 128 || p->head_dim == 512))) return nc;
  return -1;
}

struct Carve {
  size_t parts_o, parts_ml, vt_stage, total;
};
Carve carve(const esp_attn_params* p, int n_rows, int n_parts) {
  const size_t cols = size_t(p->rows_per_tile) * size_t(p->H / p->Hkv);
  const size_t recs = size_t(n_parts > 0 ? n_parts : 0) * p->Hkv * cols;
  auto up = [](size_t x) { return (x + 255) & ~size_t(255); };
  Carve c;
  c.parts_o = 0;
  c.parts_ml = up(recs * p->head_dim * sizeof(float));
  c.vt_stage = c.parts_ml + up(recs * 2 * sizeof(float));
  const size_t groups = size_t(n_rows > 0 ? (n_rows + 15) / 16 : 0);
  c.total = c.vt_stage + (family(p) < 0 ? up(groups * 16 * p->Hkv * p->head_dim * sizeof(uint16_t)) : 0);
  if (c.total == 0) c.total = 256;
  return c;
}

esp::KArgs make_args(const esp_attn_params* p, const Carve& c, void* workspace, int n_rows) {
  char* ws = static_cast<char*>(workspace);
  esp::KArgs a{};
  a.parts_o = reinterpret_cast<float*>(ws + c.parts_o);
  a.parts_ml = reinterpret_cast<float*>(ws + c.parts_ml);
  a.vt_stage = reinterpret_cast<uint16_t*>(ws + c.vt_stage);
  a.gate = p->gate;
  a.gate_ld = p->gate_ld;
  a.gate_hs = p->gate_hs;
  a.gate_off = p->gate_off;
  a.gate_ds = p->gate_headwise ? 0 : 1;
  a.H = p->H;
  a.Hkv = p->Hkv;
  a.G = p->H / p->Hkv;
  a.q_ld = p->q_ld;
  a.kv_ld = p->kv_ld;
  a.bt = p->bt;
  a.window = p->window;
  a.ring = p->ring;
  a.bidi = p->bidi;
  a.R = p->rows_per_tile;
  a.cols = a.R * a.G;
  a.n_rows = n_rows;
  a.scale_log2 = p->scale * esp::kLog2e;
  a.kv_base = p->kv_base;
  return a;
}

// A pending event pair (esp_attn_time_next) belongs to the next call that could have used it, whatever becomes of
// that call: one that launches nothing or fails its checks must not leave it armed for some later launch.
struct DropPair {
  ~DropPair() { (void)esp::take_time_next(); }
};

constexpr int kMaxDevices = 64;
struct DeviceState {
  unsigned char* scratch = nullptr;  // this device's copy of `scratch`
  bool ready = false;
};
DeviceState g_dev[kMaxDevices];
std::mutex g_dev_mutex;

// State of the current device; the first call on a device looks its copy of `scratch` up and raises the
// kernels' dynamic LDS limits (both are process-wide facts of that device, neither is stream work).
int device_state(DeviceState** out, char* err, size_t errlen) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(err, errlen, "hipGetDevice", e);
  if (dev < 0 || dev >= kMaxDevices) return fail(err, errlen, ESP_EUNSUPPORTED, "device ordinal %d (at most %d devices)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_dev_mutex);
  DeviceState& d = g_dev[dev];
  if (!d.ready) {
    void* ps = nullptr;
    if ((e = hipGetSymbolAddress(&ps, HIP_SYMBOL(scratch))) != hipSuccess) return hip_fail(err, errlen, "hipGetSymbolAddress(scratch)", e);
    if ((e = esp::stream_init_attributes()) != hipSuccess) return hip_fail(err, errlen, "hipFuncSetAttribute (streaming kernels)", e);
    if ((e = esp::tiled_init_attributes()) != hipSuccess) return hip_fail(err, errlen, "hipFuncSetAttribute (tiled kernels)", e);
    if ((e = esp::tiled512_init_attributes()) != hipSuccess) return hip_fail(err, errlen, "hipFuncSetAttribute (tiled kernels, head dim 512)", e);
    d.scratch = static_cast<unsigned char*>(ps);
    d.ready = true;
  }
  *out = &d;
  return ESP_OK;
}

}  // namespace

namespace esp {
// One pending pair per calling thread: the thread that armed it is the one whose next launch takes it, so a
// second thread driving other streams neither sees nor consumes it.
static thread_local TimeNext g_time_next;
TimeNext take_time_next() {
  const TimeNext t = g_time_next;
  g_time_next = TimeNext{};
  return t;
}
}  // namespace esp

extern "C" {

int esp_attn_abi_version(void) { return ESP_ABI_VERSION; }

int esp_attn_init(int device, char* err, size_t errlen) {
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) return hip_fail(err, errlen, "hipGetDeviceProperties", e);
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(err, errlen, ESP_EUNSUPPORTED, "device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
  // Per-device set-up with that device current: the addresses of the library's own device arrays and
  // the kernels' LDS limits, so that no later call has anything but launches left to do.
  int prev = 0;
  if ((e = hipGetDevice(&prev)) != hipSuccess) return hip_fail(err, errlen, "hipGetDevice", e);
  if (prev != device && (e = hipSetDevice(device)) != hipSuccess) return hip_fail(err, errlen, "hipSetDevice", e);
  DeviceState* d = nullptr;
  const int rc = device_state(&d, err, errlen);
  if (prev != device) (void)hipSetDevice(prev);
  return rc;
}

int esp_attn_plan_hint(const esp_attn_params* p, int device, int32_t* workgroups, int32_t* groups_per_tile,
                       int32_t* max_rows, char* err, size_t errlen) {
  if (int rc = check_params(p, err, errlen)) return rc;
  if (!workgroups || !groups_per_tile || !max_rows || p->rows_per_tile <= 0)
    return fail(err, errlen, ESP_EINVAL, "NULL output or rows_per_tile <= 0");
  int cus = 0;
  hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
  if (e != hipSuccess) return hip_fail(err, errlen, "hipDeviceGetAttribute", e);
  const int fam = family(p);
  // What is resident at once. The streaming kernel's planner splits a pass up to that many workgroups (a
  // second round would pay its per-workgroup set-up again); the tiled kernel's planner hands the pass's
  // workgroups to that many slots and picks the split that finishes earliest.
  *workgroups = fam > 0 ? cus * esp::stream_workgroups_per_cu(p->head_dim, fam) : cus * esp::tiled_workgroups_per_cu(p->head_dim);
  *groups_per_tile = fam > 0 ? p->Hkv : p->H;
  *max_rows = esp::tiled_max_rows(p->head_dim);
  return ESP_OK;
}

size_t esp_attn_workspace_bytes(const esp_attn_params* p, int32_t n_rows, int32_t n_parts) {
  if (!p || p->Hkv <= 0 || p->H <= 0 || p->rows_per_tile <= 0) return 0;
  return carve(p, n_rows, n_parts).total;
}

// Attention of one layer over a planned pass. workspace NULL: the library's own scratch array
// (esp_attn_forward_static), whose size is the limit.
static int forward_impl(const esp_attn_params* p, const void* Q, const void* Kb, const void* Vb, const void* kv_pool,
                        const int32_t* blocks, const int32_t* desc, const int32_t* pos, void* O, const esp_tile* tiles,
                        int32_t n_tiles, const esp_tree* trees, int32_t n_trees, const esp_combine* jobs, int32_t n_jobs,
                        int32_t n_parts, int32_t n_rows, void* workspace, size_t workspace_bytes, bool own_scratch,
                        const esp::PrepArgs* prep, void* stream, char* err, size_t errlen) {
  DropPair drop_pair;
  if (int rc = check_params(p, err, errlen)) return rc;
  if (n_tiles < 0 || n_trees < 0 || n_jobs < 0 || n_parts < 0 || n_rows < 0) return fail(err, errlen, ESP_EINVAL, "negative count");
  if (n_tiles == 0) return ESP_OK;
  if ((!prep && !Q) || !O || !tiles || !trees) return fail(err, errlen, ESP_EINVAL, "Q, O, tiles, trees must not be NULL");
  if (!prep && ((Kb == nullptr) != (Vb == nullptr))) return fail(err, errlen, ESP_EINVAL, "Kb and Vb: both, or neither (the pass's rows are read from the pool)");
  const bool rows_in_pool = !prep && !Kb;
  if (n_trees == 0) return fail(err, errlen, ESP_EINVAL, "%d tiles without trees", n_tiles);
  if (!kv_pool) return fail(err, errlen, ESP_EINVAL, "kv_pool is NULL");
  if (!p->ring && !blocks) return fail(err, errlen, ESP_EINVAL, "blocks is NULL on a layer without rings");
  if (p->window > 0 && !pos) return fail(err, errlen, ESP_EINVAL, "pos is NULL on a sliding-window layer");
  if (p->rows_per_tile <= 0) return fail(err, errlen, ESP_EINVAL, "rows_per_tile %d", p->rows_per_tile);
  if (n_jobs > 0 && !jobs) return fail(err, errlen, ESP_EINVAL, "jobs is NULL");
  if (n_jobs > 0 && n_parts == 0) return fail(err, errlen, ESP_EINVAL, "n_jobs %d without partial records", n_jobs);
  if (!(p->scale > 0.0f)) return fail(err, errlen, ESP_EINVAL, "scale must be positive");
  const int fam = family(p);
  if (fam < 0 && p->rows_per_tile > esp::tiled_max_rows(p->head_dim))
    return fail(err, errlen, ESP_EUNSUPPORTED, "rows_per_tile %d: the tiled kernel takes at most %d rows per tile at head_dim %d",
                p->rows_per_tile, esp::tiled_max_rows(p->head_dim), p->head_dim);
  if (fam > 0 && n_tiles > 65535)
    return fail(err, errlen, ESP_EUNSUPPORTED, "%d tiles in one pass: the streaming kernel's grid takes at most 65535", n_tiles);
  DeviceState* dev = nullptr;
  if (int rc = device_state(&dev, err, errlen)) return rc;
  const Carve c = carve(p, n_rows, n_parts);
  if (own_scratch) {
    if (c.total > kScratchBytes)
      return fail(err, errlen, ESP_EWORKSPACE, "this pass needs %zu bytes of scratch; the library's own array holds %zu "
                  "(use esp_attn_forward with a workspace)", c.total, kScratchBytes);
    workspace = dev->scratch;
    workspace_bytes = kScratchBytes;
  }
  if (!workspace || workspace_bytes < c.total)
    return fail(err, errlen, ESP_EWORKSPACE, "workspace %zu bytes, %zu needed", workspace_bytes, c.total);
  if (reinterpret_cast<uintptr_t>(workspace) % 16) return fail(err, errlen, ESP_EINVAL, "workspace must be 16-byte aligned");

  hipStream_t st = static_cast<hipStream_t>(stream);
  esp::KArgs a = make_args(p, c, workspace, n_rows);
  a.Q = static_cast<const uint16_t*>(Q);
  a.Kb = static_cast<const uint16_t*>(Kb);
  a.Vb = static_cast<const uint16_t*>(Vb);
  a.pool = static_cast<const uint16_t*>(kv_pool);
  a.blocks = blocks;
  a.desc = reinterpret_cast<const int4*>(desc);
  a.pos = reinterpret_cast<const int4*>(pos);
  a.O = static_cast<uint16_t*>(O);
  a.tiles = tiles;
  a.trees = trees;

  hipError_t e;
  if (fam > 0) {
    e = esp::launch_stream(p->dtype, p->head_dim, fam, a, prep, n_tiles, st);
    if (e != hipSuccess) return hip_fail(err, errlen, "attn_stream launch", e);
  } else {
    if (n_rows > 0 && !rows_in_pool) {
      e = esp::launch_vt_stage(p, Vb, a.vt_stage, n_rows, st);
      if (e != hipSuccess) return hip_fail(err, errlen, "vt_stage launch", e);
    }
    e = esp::launch_tiled(p->dtype, p->head_dim, a, n_tiles, st);
    if (e != hipSuccess) return hip_fail(err, errlen, "attn_tiled launch", e);
  }
  if (n_jobs > 0) {
    e = esp::launch_combine(p->dtype, p->head_dim, a, jobs, n_jobs, n_parts, st);
    if (e != hipSuccess) return hip_fail(err, errlen, "attn_combine launch", e);
  }
  return ESP_OK;
}

int esp_attn_forward(const esp_attn_params* p, const void* Q, const void* Kb, const void* Vb, const void* kv_pool,
                     const int32_t* blocks, const int32_t* desc, const int32_t* pos, void* O, const esp_tile* tiles,
                     int32_t n_tiles, const esp_tree* trees, int32_t n_trees, const esp_combine* jobs, int32_t n_jobs,
                     int32_t n_parts, int32_t n_rows, void* workspace, size_t workspace_bytes, void* stream, char* err,
                     size_t errlen) {
  return forward_impl(p, Q, Kb, Vb, kv_pool, blocks, desc, pos, O, tiles, n_tiles, trees, n_trees, jobs, n_jobs, n_parts, n_rows,
                      workspace, workspace_bytes, false, nullptr, stream, err, errlen);
}

int esp_attn_forward_static(const esp_attn_params* p, const void* Q, const void* Kb, const void* Vb, const void* kv_pool,
                            const int32_t* blocks, const int32_t* desc, const int32_t* pos, void* O, const esp_tile* tiles,
                            int32_t n_tiles, const esp_tree* trees, int32_t n_trees, const esp_combine* jobs, int32_t n_jobs,
                            int32_t n_parts, int32_t n_rows, void* stream, char* err, size_t errlen) {
  return forward_impl(p, Q, Kb, Vb, kv_pool, blocks, desc, pos, O, tiles, n_tiles, trees, n_trees, jobs, n_jobs, n_parts, n_rows,
                      nullptr, 0, true, nullptr, stream, err, errlen);
}

int esp_attn_validate(const esp_attn_params* p, const esp_tile* tiles, int32_t n_tiles, const esp_tree* trees, int32_t n_trees,
                      const esp_combine* jobs, int32_t n_jobs, int32_t n_parts, int32_t n_rows, const int32_t* blocks,
                      int32_t n_block_entries, int32_t pool_blocks, char* err, size_t errlen) {
  if (int rc = check_params(p, err, errlen)) return rc;
  if (n_tiles < 0 || n_trees < 0 || n_jobs < 0 || n_parts < 0 || n_rows < 0 || n_block_entries < 0 || pool_blocks < 0)
    return fail(err, errlen, ESP_EINVAL, "negative count");
  if (p->rows_per_tile <= 0) return fail(err, errlen, ESP_EINVAL, "rows_per_tile %d", p->rows_per_tile);
  if ((n_tiles && !tiles) || (n_trees && !trees) || (n_jobs && !jobs)) return fail(err, errlen, ESP_EINVAL, "NULL record array");
  if (!p->ring && n_block_entries && !blocks) return fail(err, errlen, ESP_EINVAL, "blocks is NULL");
  const int64_t bt = p->bt;
  for (int i = 0; i < n_trees; ++i) {
    const esp_tree& t = trees[i];
    if (t.base < 0 || t.M < 0 || int64_t(t.base) + t.M > n_rows)
      return fail(err, errlen, ESP_EINVAL, "tree %d: rows [%d, %d + %d) outside the pass's %d rows", i, t.base, t.base, t.M, n_rows);
    if (t.P < 0 || t.table < 0) return fail(err, errlen, ESP_EINVAL, "tree %d: P %d, table %d", i, t.P, t.table);
    if (p->ring) {
      if (t.P > 0 && int64_t(t.table) + p->ring > pool_blocks)
        return fail(err, errlen, ESP_EINVAL, "tree %d: ring blocks [%d, %d + %d) outside the pool's %d blocks", i, t.table, t.table, p->ring, pool_blocks);
    } else {
      const int64_t nb = (t.P + bt - 1) / bt;
      if (t.table + nb > n_block_entries)
        return fail(err, errlen, ESP_EINVAL, "tree %d: block list [%d, %d + %lld) outside the %d entries of blocks", i, t.table, t.table,
                    (long long)nb, n_block_entries);
      for (int64_t b = 0; b < nb; ++b)
        if (blocks[t.table + b] < 0 || blocks[t.table + b] >= pool_blocks)
          return fail(err, errlen, ESP_EINVAL, "tree %d: block %d (entry %lld of its list) outside the pool's %d blocks", i, blocks[t.table + b],
                      (long long)b, pool_blocks);
    }
  }
  // every partial record is written by exactly one tile and read by exactly one job
  std::vector<int32_t> part_job(size_t(n_parts), -1);
  for (int j = 0; j < n_jobs; ++j) {
    const esp_combine& c = jobs[j];
    if (c.r0 < 0 || c.rows <= 0 || c.rows > p->rows_per_tile || int64_t(c.r0) + c.rows > n_rows)
      return fail(err, errlen, ESP_EINVAL, "job %d: rows [%d, %d + %d), %d rows per tile, %d rows in the pass", j, c.r0, c.r0, c.rows,
                  p->rows_per_tile, n_rows);
    if (c.part0 < 0 || c.nparts <= 0 || int64_t(c.part0) + c.nparts > n_parts)
      return fail(err, errlen, ESP_EINVAL, "job %d: parts [%d, %d + %d) outside the pass's %d records", j, c.part0, c.part0, c.nparts, n_parts);
    for (int q = c.part0; q < c.part0 + c.nparts; ++q) {
      if (part_job[size_t(q)] >= 0) return fail(err, errlen, ESP_EINVAL, "partial record %d is merged by jobs %d and %d", q, part_job[size_t(q)], j);
      part_job[size_t(q)] = j;
    }
  }
  std::vector<char> part_written(size_t(n_parts), 0);
  for (int i = 0; i < n_tiles; ++i) {
    const esp_tile& t = tiles[i];
    if (t.tree < 0 || t.tree >= n_trees) return fail(err, errlen, ESP_EINVAL, "tile %d: tree %d of %d", i, t.tree, n_trees);
    const esp_tree& tr = trees[t.tree];
    if (t.r0 < tr.base || t.r0 >= tr.base + tr.M)
      return fail(err, errlen, ESP_EINVAL, "tile %d: first row %d outside its tree's rows [%d, %d)", i, t.r0, tr.base, tr.base + tr.M);
    if ((t.r0 - tr.base) % p->rows_per_tile) return fail(err, errlen, ESP_EINVAL, "tile %d: first row %d is no multiple of %d rows into its tree", i, t.r0, p->rows_per_tile);
    const bool open = t.k1 == INT32_MAX;  // up to the tree's cached length when the kernel runs
    if (t.k0 < 0 || (!open && (t.k1 < t.k0 || t.k1 > tr.P)) || (open && t.k0 > tr.P))
      return fail(err, errlen, ESP_EINVAL, "tile %d: cached range [%d, %d) outside its tree's %d cached keys", i, t.k0, t.k1, tr.P);
    if (t.part < -1 || t.part >= n_parts) return fail(err, errlen, ESP_EINVAL, "tile %d: partial record %d of %d", i, t.part, n_parts);
    if (t.part >= 0) {
      if (part_written[size_t(t.part)]) return fail(err, errlen, ESP_EINVAL, "tile %d: partial record %d is written by another tile too", i, t.part);
      part_written[size_t(t.part)] = 1;
      if (n_jobs > 0) {
        const int j = part_job[size_t(t.part)];
        if (j < 0) return fail(err, errlen, ESP_EINVAL, "tile %d: no job merges its partial record %d", i, t.part);
        if (jobs[j].r0 != t.r0 || jobs[j].rows != (tr.base + tr.M - t.r0 < p->rows_per_tile ? tr.base + tr.M - t.r0 : p->rows_per_tile))
          return fail(err, errlen, ESP_EINVAL, "tile %d: job %d merges rows [%d, %d + %d), the tile holds rows from %d", i, j, jobs[j].r0,
                      jobs[j].r0, jobs[j].rows, t.r0);
      }
    }
    if (t.last < 0 || (t.last >= 2 && (t.last - 2 < t.b0 || t.last - 2 >= tr.M)))
      return fail(err, errlen, ESP_EINVAL, "tile %d: last %d (0: no batch keys, 1: from b0 on, e + 2: rows b0 = %d .. e of the tree's %d)", i, t.last,
                  t.b0, tr.M);
    if (t.b0 < 0 || t.b0 > tr.M) return fail(err, errlen, ESP_EINVAL, "tile %d: first batch key %d of %d rows", i, t.b0, tr.M);
    if (t.pad != 0 && t.pad - 1 != tr.table) return fail(err, errlen, ESP_EINVAL, "tile %d: pad %d is neither 0 nor 1 + its tree's table %d", i, t.pad, tr.table);
  }
  if (n_jobs > 0)
    for (int q = 0; q < n_parts; ++q)
      if (part_job[size_t(q)] >= 0 && !part_written[size_t(q)])
        return fail(err, errlen, ESP_EINVAL, "job %d merges partial record %d, which no tile writes", part_job[size_t(q)], q);
  return ESP_OK;
}

int esp_attn_validate_for(const esp_attn_params* p, int32_t mode, const esp_tile* tiles, int32_t n_tiles, const esp_tree* trees,
                          int32_t n_trees, const esp_combine* jobs, int32_t n_jobs, int32_t n_parts, int32_t n_rows, const int32_t* blocks,
                          int32_t n_block_entries, int32_t pool_blocks, char* err, size_t errlen) {
  if (int rc = esp_attn_validate(p, tiles, n_tiles, trees, n_trees, jobs, n_jobs, n_parts, n_rows, blocks, n_block_entries, pool_blocks,
                                 err, errlen))
    return rc;
  if (mode & ~(ESP_PASS_FUSED | ESP_PASS_ROWS_IN_POOL)) return fail(err, errlen, ESP_EINVAL, "mode %d", mode);
  if (mode & ESP_PASS_FUSED) {
    if (p->head_dim == 512 || p->rows_per_tile > 4 || family(p) <= 0)
      return fail(err, errlen, ESP_EUNSUPPORTED, "rows_per_tile %d at head_dim %d: the fused decode takes trees of 1 to 4 rows on the streaming kernel, head dim 128 or 256",
                  p->rows_per_tile, p->head_dim);
    // The fused kernel prepares the rows of its own tile only and reads a tree's batch keys from that tile's LDS
    // area: a tree is one tile group, whose first row is the tree's first row.
    for (int i = 0; i < n_trees; ++i)
      if (trees[i].M > p->rows_per_tile)
        return fail(err, errlen, ESP_EINVAL, "tree %d: %d rows; a fused pass takes trees of at most rows_per_tile = %d rows", i, trees[i].M,
                    p->rows_per_tile);
    for (int i = 0; i < n_tiles; ++i)
      if (tiles[i].r0 != trees[tiles[i].tree].base)
        return fail(err, errlen, ESP_EINVAL, "tile %d: first row %d is not its tree's first row %d (a fused pass has one tile group per tree)", i,
                    tiles[i].r0, trees[tiles[i].tree].base);
  }
  if (mode & ESP_PASS_ROWS_IN_POOL) {
    // Row j of a tree is read at position P + j of the tree's own block list (or ring).
    const int64_t bt = p->bt;
    for (int i = 0; i < n_trees; ++i) {
      const esp_tree& t = trees[i];
      if (t.M == 0) continue;
      if (family(p) < 0 && (t.P - t.base) % 16)
        return fail(err, errlen, ESP_EINVAL, "tree %d: P %d - base %d is no multiple of 16: the tiled kernel reads a pass's rows from the pool in "
                    "16-token sub-blocks (pass Kb / Vb for this pass)", i, t.P, t.base);
      if (p->ring) {
        if (int64_t(t.table) + p->ring > pool_blocks)
          return fail(err, errlen, ESP_EINVAL, "tree %d: ring blocks [%d, %d + %d) outside the pool's %d blocks", i, t.table, t.table, p->ring, pool_blocks);
        if (t.M > int64_t(p->ring) * bt - p->window + 1)
          return fail(err, errlen, ESP_EINVAL, "tree %d: %d rows appended to a ring of %d x %lld tokens overwrite keys that its first rows still see "
                      "(window %d): pass Kb / Vb for this pass", i, t.M, p->ring, (long long)bt, p->window);
      } else {
        const int64_t nb = (int64_t(t.P) + t.M + bt - 1) / bt;
        if (t.table + nb > n_block_entries)
          return fail(err, errlen, ESP_EINVAL, "tree %d: block list [%d, %d + %lld) with its own rows appended lies outside the %d entries of blocks", i,
                      t.table, t.table, (long long)nb, n_block_entries);
        for (int64_t b = (int64_t(t.P) + bt - 1) / bt; b < nb; ++b)
          if (blocks[t.table + b] < 0 || blocks[t.table + b] >= pool_blocks)
            return fail(err, errlen, ESP_EINVAL, "tree %d: block %d (entry %lld of its list) outside the pool's %d blocks", i, blocks[t.table + b],
                        (long long)b, pool_blocks);
      }
    }
  }
  return ESP_OK;
}

int esp_attn_time_next(void* start_event, void* stop_event) {
  if ((start_event == nullptr) != (stop_event == nullptr)) return ESP_EINVAL;
  esp::g_time_next.start = static_cast<hipEvent_t>(start_event);
  esp::g_time_next.stop = static_cast<hipEvent_t>(stop_event);
  return ESP_OK;
}

int esp_attn_combine(const esp_attn_params* p, void* O, const esp_combine* jobs, int32_t n_jobs, int32_t n_parts,
                     int32_t n_rows, void* workspace, size_t workspace_bytes, void* stream, char* err, size_t errlen) {
  if (int rc = check_params(p, err, errlen)) return rc;
  if (n_jobs < 0 || n_parts < 0 || n_rows < 0) return fail(err, errlen, ESP_EINVAL, "negative count");
  if (n_jobs == 0) return ESP_OK;
  if (!O || !jobs) return fail(err, errlen, ESP_EINVAL, "O and jobs must not be NULL");
  if (n_parts == 0) return fail(err, errlen, ESP_EINVAL, "n_jobs %d without partial records", n_jobs);
  if (p->rows_per_tile <= 0) return fail(err, errlen, ESP_EINVAL, "rows_per_tile %d", p->rows_per_tile);
  const Carve c = carve(p, n_rows, n_parts);
  if (!workspace || workspace_bytes < c.total)
    return fail(err, errlen, ESP_EWORKSPACE, "workspace %zu bytes, %zu needed", workspace_bytes, c.total);
  if (reinterpret_cast<uintptr_t>(workspace) % 16) return fail(err, errlen, ESP_EINVAL, "workspace must be 16-byte aligned");
  esp::KArgs a = make_args(p, c, workspace, n_rows);
  a.O = static_cast<uint16_t*>(O);
  hipError_t e = esp::launch_combine(p->dtype, p->head_dim, a, jobs, n_jobs, n_parts, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? ESP_OK : hip_fail(err, errlen, "attn_combine launch", e);
}

int esp_kv_save(const esp_attn_params* p, const void* Kb, const void* Vb, void* kv_pool, const esp_kvsave* entries,
                int32_t n_entries, void* stream, char* err, size_t errlen) {
  if (int rc = check_params(p, err, errlen)) return rc;
  if (n_entries < 0) return fail(err, errlen, ESP_EINVAL, "n_entries negative");
  if (n_entries == 0) return ESP_OK;
  if (!Kb || !Vb || !kv_pool || !entries) return fail(err, errlen, ESP_EINVAL, "NULL argument");
  hipError_t e = esp::launch_kv_save(p, Kb, Vb, kv_pool, entries, n_entries, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? ESP_OK : hip_fail(err, errlen, "kv_save launch", e);
}

int esp_kv_copy_blocks(const esp_attn_params* p, void* kv_pool, const int32_t* pairs, int32_t n_pairs, int32_t n_layers,
                       uint64_t region_elems, void* stream, char* err, size_t errlen) {
  if (int rc = check_params(p, err, errlen)) return rc;
  if (n_pairs < 0 || n_layers < 0) return fail(err, errlen, ESP_EINVAL, "negative count");
  if (n_pairs == 0 || n_layers == 0) return ESP_OK;
  if (!kv_pool || !pairs) return fail(err, errlen, ESP_EINVAL, "NULL argument");
  if (region_elems % 8) return fail(err, errlen, ESP_EINVAL, "region_elems must be a multiple of 8");
  hipError_t e = esp::launch_kv_copy_blocks(p, kv_pool, pairs, n_pairs, n_layers, region_elems, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? ESP_OK : hip_fail(err, errlen, "kv_copy_blocks launch", e);
}

int esp_kv_gather(const esp_attn_params* p, const void* kv_pool, const int32_t* blocks, int32_t n_tokens, void* K_out,
                  void* V_out, void* stream, char* err, size_t errlen) {
  if (int rc = check_params(p, err, errlen)) return rc;
  if (n_tokens < 0) return fail(err, errlen, ESP_EINVAL, "n_tokens negative");
  if (n_tokens == 0) return ESP_OK;
  if (!kv_pool || !blocks || !K_out || !V_out) return fail(err, errlen, ESP_EINVAL, "NULL argument");
  hipError_t e = esp::launch_kv_gather(p, kv_pool, blocks, n_tokens, K_out, V_out, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? ESP_OK : hip_fail(err, errlen, "kv_gather launch", e);
}

int esp_kv_relayout(const esp_attn_params* p, const void* src_pool, int32_t src_layout, void* dst_pool, int32_t dst_layout,
                    int32_t n_blocks, void* stream, char* err, size_t errlen) {
  if (int rc = check_params(p, err, errlen)) return rc;
  if (n_blocks < 0) return fail(err, errlen, ESP_EINVAL, "n_blocks negative");
  if (!((src_layout == ESP_LAYOUT_REFERENCE && dst_layout == ESP_LAYOUT_NATIVE) ||
        (src_layout == ESP_LAYOUT_NATIVE && dst_layout == ESP_LAYOUT_REFERENCE)))
    return fail(err, errlen, ESP_EINVAL, "layouts %d -> %d: one side reference, the other native", src_layout, dst_layout);
  if (n_blocks == 0) return ESP_OK;
  if (!src_pool || !dst_pool) return fail(err, errlen, ESP_EINVAL, "NULL argument");
  hipError_t e = esp::launch_kv_relayout(p, src_pool, dst_pool, dst_layout == ESP_LAYOUT_NATIVE, n_blocks, nullptr,
                                         static_cast<hipStream_t>(stream));
  return e == hipSuccess ? ESP_OK : hip_fail(err, errlen, "kv_relayout launch", e);
}

int esp_kv_export_blocks(const esp_attn_params* p, const void* kv_pool, const int32_t* blocks, int32_t n_blocks, void* out,
                         void* stream, char* err, size_t errlen) {
  if (int rc = check_params(p, err, errlen)) return rc;
  if (n_blocks < 0) return fail(err, errlen, ESP_EINVAL, "n_blocks negative");
  if (n_blocks == 0) return ESP_OK;
  if (!kv_pool || !blocks || !out) return fail(err, errlen, ESP_EINVAL, "NULL argument");
  hipError_t e = esp::launch_kv_relayout(p, static_cast<const uint16_t*>(kv_pool) + p->kv_base, out, 0, n_blocks, blocks,
                                         static_cast<hipStream_t>(stream));
  return e == hipSuccess ? ESP_OK : hip_fail(err, errlen, "kv_export_blocks launch", e);
}

int esp_kv_import_blocks(const esp_attn_params* p, const void* in, const int32_t* blocks, int32_t n_blocks, void* kv_pool,
                         void* stream, char* err, size_t errlen) {
  if (int rc = check_params(p, err, errlen)) return rc;
  if (n_blocks < 0) return fail(err, errlen, ESP_EINVAL, "n_blocks negative");
  if (n_blocks == 0) return ESP_OK;
  if (!kv_pool || !blocks || !in) return fail(err, errlen, ESP_EINVAL, "NULL argument");
  hipError_t e = esp::launch_kv_relayout(p, in, static_cast<uint16_t*>(kv_pool) + p->kv_base, 1, n_blocks, blocks,
                                         static_cast<hipStream_t>(stream));
  return e == hipSuccess ? ESP_OK : hip_fail(err, errlen, "kv_import_blocks launch", e);
}

int esp_chain_advance(esp_tree* trees, int32_t n_trees, int32_t* pos, int32_t* row_table, const int32_t* blocks, int32_t bt,
                      int32_t ring, void* stream, char* err, size_t errlen) {
  if (n_trees < 0) return fail(err, errlen, ESP_EINVAL, "negative count");
  if (n_trees == 0) return ESP_OK;
  if (!trees || !pos) return fail(err, errlen, ESP_EINVAL, "trees and pos must not be NULL");
  if (bt <= 0 || bt % 16) return fail(err, errlen, ESP_EINVAL, "bt %d: tokens per block must be a positive multiple of 16", bt);
  if (ring < 0) return fail(err, errlen, ESP_EINVAL, "ring negative");
  if (row_table && !ring && !blocks) return fail(err, errlen, ESP_EINVAL, "blocks is NULL on a layer without rings");
  const hipError_t e = esp::launch_chain_advance(trees, n_trees, pos, row_table, blocks, bt, ring, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(err, errlen, "chain_advance launch", e);
  return ESP_OK;
}

int esp_head_gate(const esp_gate_params* p, void* O, const void* X, const void* Wg, float* dots, int32_t n_rows,
                  void* stream, char* err, size_t errlen) {
  if (!p) return fail(err, errlen, ESP_EINVAL, "params is NULL");
  if (p->H <= 0 || p->H > 64) return fail(err, errlen, p->H <= 0 ? ESP_EINVAL : ESP_EUNSUPPORTED, "H=%d (1 .. 64)", p->H);
  if (p->head_dim <= 0 || p->head_dim % 8 || p->head_dim > 1024)
    return fail(err, errlen, ESP_EINVAL, "head_dim %d: a multiple of 8, at most 1024", p->head_dim);
  if (p->D <= 0 || p->D % 8) return fail(err, errlen, ESP_EINVAL, "D %d: a positive multiple of 8", p->D);
  if (p->dtype != ESP_F16 && p->dtype != ESP_BF16) return fail(err, errlen, ESP_EINVAL, "dtype %d", p->dtype);
  if (p->x_ld < p->D || p->x_ld % 8) return fail(err, errlen, ESP_EINVAL, "x_ld %d", p->x_ld);
  if (O && (p->q_ld < p->H * p->head_dim || p->q_ld % 8)) return fail(err, errlen, ESP_EINVAL, "q_ld %d", p->q_ld);
  if (n_rows < 0) return fail(err, errlen, ESP_EINVAL, "negative count");
  if (!O && !dots) return fail(err, errlen, ESP_EINVAL, "neither O nor dots");
  if (n_rows == 0) return ESP_OK;
  if (!X || !Wg) return fail(err, errlen, ESP_EINVAL, "X and Wg must not be NULL");
  int shift = -1;
  for (int s = 3; s <= 10; ++s)
    if (p->head_dim == 1 << s) shift = s;
  esp::GateArgs a{static_cast<uint16_t*>(O), static_cast<const uint16_t*>(X), static_cast<const uint16_t*>(Wg), dots,
                  n_rows, p->H, p->head_dim, shift, p->D, p->q_ld, p->x_ld};
  const hipError_t e = esp::launch_head_gate(p->dtype, a, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(err, errlen, "head_gate launch", e);
  return ESP_OK;
}

// Checks of esp_prep_params shared by esp_attn_prep and esp_attn_decode_fused.
static int check_prep(const esp_prep_params* p, bool with_table, const void* kv_pool, char* err, size_t errlen) {
  if (!p) return fail(err, errlen, ESP_EINVAL, "params is NULL");
  if (p->H <= 0 || p->Hkv <= 0) return fail(err, errlen, ESP_EINVAL, "H=%d Hkv=%d", p->H, p->Hkv);
  if (p->head_dim != 128 && p->head_dim != 256 && p->head_dim != 512)
    return fail(err, errlen, ESP_EUNSUPPORTED, "head_dim %d (128, 256 or 512)", p->head_dim);
  if (p->dtype != ESP_F16 && p->dtype != ESP_BF16) return fail(err, errlen, ESP_EINVAL, "dtype %d", p->dtype);
  const int HD = p->head_dim;
  if (p->x_ld % 4 || p->q_off % 4 || p->q_hs % 4 || p->k_off % 4 || p->v_off % 4 || p->q_off < 0 || p->k_off < 0 || p->v_off < 0)
    return fail(err, errlen, ESP_EINVAL, "x_ld, q_off, q_hs, k_off, v_off must be non-negative multiples of 4 floats");
  if (p->q_hs < HD) return fail(err, errlen, ESP_EINVAL, "q_hs %d < head_dim", p->q_hs);
  if (p->x_ld < p->q_off + (p->H - 1) * p->q_hs + HD || p->x_ld < p->k_off + p->Hkv * HD || p->x_ld < p->v_off + p->Hkv * HD)
    return fail(err, errlen, ESP_EINVAL, "x_ld %d does not hold the q / k / v columns", p->x_ld);
  if (p->q_ld < p->H * HD || p->q_ld % 4 || p->kv_ld < p->Hkv * HD || p->kv_ld % 4)
    return fail(err, errlen, ESP_EINVAL, "q_ld %d / kv_ld %d", p->q_ld, p->kv_ld);
  if (HD == 512 && (p->q_ld % 8 || p->kv_ld % 8)) return fail(err, errlen, ESP_EINVAL, "q_ld %d / kv_ld %d: multiples of 8 at head_dim 512", p->q_ld, p->kv_ld);
  const int rd = p->rope_dims, rd_min = HD == 512 ? 16 : 8;  // a lane holds 4 consecutive dims (8 at head_dim 512): half of rope_dims is a multiple of that
  if (rd < 0 || rd > HD || (rd != 0 && (rd < rd_min || (rd & (rd - 1)))))
    return fail(err, errlen, ESP_EINVAL, "rope_dims %d: 0 or a power of two in [%d, head_dim]", rd, rd_min);
  if (with_table) {
    if (!kv_pool) return fail(err, errlen, ESP_EINVAL, "row_table without kv_pool");
    if (p->bt <= 0 || p->bt % 16) return fail(err, errlen, ESP_EINVAL, "bt %d: tokens per block must be a positive multiple of 16", p->bt);
    if (p->kv_base % 8) return fail(err, errlen, ESP_EINVAL, "kv_base must be a multiple of 8 elements");
  }
  return ESP_OK;
}

int esp_attn_prep(const esp_prep_params* p, const float* X, const float* qn_w, const float* kn_w, const int32_t* pos,
                  const float* inv_freq, const int32_t* rope_sel, void* Q, void* Kb, void* Vb, const int32_t* row_table,
                  void* kv_pool, int32_t n_rows, void* stream, char* err, size_t errlen) {
  DropPair drop_pair;
  if (int rc = check_prep(p, row_table != nullptr, kv_pool, err, errlen)) return rc;
  if (n_rows < 0) return fail(err, errlen, ESP_EINVAL, "negative count");
  if (n_rows == 0) return ESP_OK;
  if (!X || !qn_w || !kn_w || !Q) return fail(err, errlen, ESP_EINVAL, "X, qn_w, kn_w, Q must not be NULL");
  if ((!Kb || !Vb) && (Kb || Vb || !row_table))
    return fail(err, errlen, ESP_EINVAL, "Kb and Vb may be left out together, and only with a row_table (the rows then live in the pool alone)");
  if (p->rope_dims > 0 && (!pos || !inv_freq)) return fail(err, errlen, ESP_EINVAL, "pos and inv_freq must not be NULL when dims rotate");
  esp::PrepArgs a{X, qn_w, kn_w, reinterpret_cast<const int4*>(pos), inv_freq, rope_sel, static_cast<uint16_t*>(Q),
                  static_cast<uint16_t*>(Kb), static_cast<uint16_t*>(Vb), reinterpret_cast<const int4*>(row_table),
                  static_cast<uint16_t*>(kv_pool), *p};
  const hipError_t e = esp::launch_attn_prep(a, n_rows, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(err, errlen, "attn_prep launch", e);
  return ESP_OK;
}

int esp_attn_decode_fused(const esp_prep_params* pp, const esp_attn_params* p, const float* X, const float* qn_w, const float* kn_w,
                          const int32_t* pos, const float* inv_freq, const int32_t* rope_sel, const int32_t* row_table,
                          void* kv_pool, const int32_t* blocks, const int32_t* desc, void* O, const esp_tile* tiles,
                          int32_t n_tiles, const esp_tree* trees, int32_t n_trees, const esp_combine* jobs, int32_t n_jobs,
                          int32_t n_parts, int32_t n_rows, void* workspace, size_t workspace_bytes, void* stream, char* err,
                          size_t errlen) {
  if (int rc = check_prep(pp, row_table != nullptr, kv_pool, err, errlen)) return rc;
  if (int rc = check_params(p, err, errlen)) return rc;
  if (pp->H != p->H || pp->Hkv != p->Hkv || pp->head_dim != p->head_dim || pp->dtype != p->dtype)
    return fail(err, errlen, ESP_EINVAL, "the prep and the attention parameters name different heads, head dims or element types");
  if (row_table && (pp->bt != p->bt || pp->kv_base != p->kv_base))
    return fail(err, errlen, ESP_EINVAL, "the prep and the attention parameters name different pool regions or block sizes");
  if (p->head_dim == 512) return fail(err, errlen, ESP_EUNSUPPORTED, "the fused decode serves head dims 128 and 256");
  if (p->rows_per_tile <= 0 || p->rows_per_tile > 4 || family(p) <= 0)
    return fail(err, errlen, ESP_EUNSUPPORTED, "rows_per_tile %d: the fused decode takes trees of 1 to 4 rows, one tile each, on the streaming kernel",
                p->rows_per_tile);
  if (n_tiles > 0 && (!X || !qn_w || !kn_w)) return fail(err, errlen, ESP_EINVAL, "X, qn_w, kn_w must not be NULL");
  if (pp->rope_dims > 0 && (!pos || !inv_freq)) return fail(err, errlen, ESP_EINVAL, "pos and inv_freq must not be NULL when dims rotate");
  if (!pos) return fail(err, errlen, ESP_EINVAL, "pos is NULL");
  const esp::PrepArgs a{X, qn_w, kn_w, reinterpret_cast<const int4*>(pos), inv_freq, rope_sel, nullptr, nullptr, nullptr,
                        reinterpret_cast<const int4*>(row_table), static_cast<uint16_t*>(kv_pool), *pp};
  return forward_impl(p, nullptr, nullptr, nullptr, kv_pool, blocks, desc, pos, O, tiles, n_tiles, trees, n_trees, jobs, n_jobs, n_parts,
                      n_rows, workspace, workspace_bytes, false, &a, stream, err, errlen);
}

}  // extern "C"
