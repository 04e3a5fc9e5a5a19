// Pool maintenance kernels over the native block layout: append rows, copy
// blocks (copy on write), gather a block list into contiguous rows, convert
// blocks between the reference's layout and the native one, and stage a
// pass's batch V rows transposed for the tiled attention kernel. All are bit
// copies of 16-bit storage elements.
#include "common.hpp"

namespace esp {

// kv_save (kernels/40_attention.metal:875-889): entry = (source row, block,
// position). One workgroup per (16 consecutive entries, KV head); a thread moves 8
// elements of a row. K rows are copied as they are. V lies transposed in 16-token
// sub-blocks: when the 16 entries fill one sub-block in order (every full group of
// a prefill chunk's append) their V rows meet in LDS and leave as the sub-block's
// contiguous [HD][16] bytes; any other arrangement (decode rows of different
// sequences, a ragged tail) stores elements.
constexpr int kSaveRows = 16;
__global__ __launch_bounds__(256) void kv_save_kernel(const uint16_t* Kb, const uint16_t* Vb, uint16_t* pool,
                                                      const esp_kvsave* entries, int n, int Hkv, int HD, int kv_ld, int bt,
                                                      uint64_t kv_base) {
  constexpr int R = kSaveRows;
  __shared__ __attribute__((aligned(16))) uint16_t vs[R][512 + 8];  // HD <= 512; the pad spreads the column reads over the banks
  const int tid = threadIdx.x, g0 = blockIdx.x * R, kvh = blockIdx.y;
  const int cnt = min(R, n - g0);
  const esp_kvsave e0 = entries[g0];
  bool mine = true;
  if (tid < R) {
    const esp_kvsave e = entries[g0 + min(tid, cnt - 1)];
    mine = tid < cnt && e.block == e0.block && e.pos == e0.pos + tid;
  }
  const bool run = __syncthreads_and(mine) && cnt == R && (e0.pos & 15) == 0;
  const int tpr = HD / 8;  // threads per row
  for (int r = tid / tpr; r < cnt; r += 256 / tpr) {
    const esp_kvsave e = entries[g0 + r];
    const int d = (tid % tpr) * 8;
    const size_t src = size_t(e.src_row) * kv_ld + size_t(kvh) * HD + d;
    uint16_t* hb = pool + kv_base + (size_t(e.block) * Hkv + kvh) * size_t(2 * bt * HD);
    *reinterpret_cast<u32x4*>(hb + size_t(e.pos) * HD + d) = *reinterpret_cast<const u32x4*>(Kb + src);
    const u32x4 v = *reinterpret_cast<const u32x4*>(Vb + src);
    if (run) {
      *reinterpret_cast<u32x4*>(&vs[r][d]) = v;
    } else {
      uint16_t* vt = hb + vt_elem(bt, HD, e.pos, d);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        vt[(2 * i) * kVtDim] = uint16_t(v[i] & 0xffffu);
        vt[(2 * i + 1) * kVtDim] = uint16_t(v[i] >> 16);
      }
    }
  }
  if (!run) return;
  __syncthreads();
  uint16_t* hb = pool + kv_base + (size_t(e0.block) * Hkv + kvh) * size_t(2 * bt * HD);
  for (int i = tid; i < 2 * HD; i += 256) {  // (dim, half of the 16 tokens): 16 contiguous bytes of the sub-block
    const int d = i >> 1, t8 = 8 * (i & 1);
    u32x4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = uint32_t(vs[t8 + 2 * e][d]) | (uint32_t(vs[t8 + 2 * e + 1][d]) << 16);
    *reinterpret_cast<u32x4*>(hb + vt_elem(bt, HD, e0.pos + t8, d)) = v;
  }
}

// kv_copy_blocks (40_:894-905): a block is one contiguous run of
// 2 * bt * Hkv * HD elements in the native layout as well.
__global__ __launch_bounds__(256) void kv_copy_blocks_kernel(uint16_t* pool, const int2* pairs, uint64_t blk2,
                                                             uint64_t region_elems) {
  const uint64_t x = (uint64_t(blockIdx.x) * 256 + threadIdx.x) * 8;
  if (x >= blk2) return;
  const int2 pr = pairs[blockIdx.y];
  uint16_t* base = pool + uint64_t(blockIdx.z) * region_elems;
  *reinterpret_cast<u32x4*>(base + uint64_t(pr.y) * blk2 + x) = *reinterpret_cast<const u32x4*>(base + uint64_t(pr.x) * blk2 + x);
}

// Tokens [0, n) of a block list -> K_out / V_out [n][Hkv * HD].
__global__ __launch_bounds__(256) void kv_gather_kernel(const uint16_t* pool, const int32_t* blocks, int n, uint16_t* K_out,
                                                        uint16_t* V_out, int Hkv, int HD, int bt, uint64_t kv_base) {
  const int per = Hkv * HD / 8;
  const long gid = long(blockIdx.x) * 256 + threadIdx.x;
  if (gid >= long(n) * per) return;
  const int j = int(gid / per);
  const int x = int(gid % per) * 8;
  const int kvh = x / HD, d = x % HD;
  const int b = blocks[j / bt], t = j % bt;
  const uint16_t* hb = pool + kv_base + (size_t(b) * Hkv + kvh) * size_t(2 * bt * HD);
  *reinterpret_cast<u32x4*>(K_out + size_t(j) * Hkv * HD + x) = *reinterpret_cast<const u32x4*>(hb + size_t(t) * HD + d);
  const uint16_t* vt = hb + vt_elem(bt, HD, t, d);
  u32x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = uint32_t(vt[(2 * i) * kVtDim]) | (uint32_t(vt[(2 * i + 1) * kVtDim]) << 16);
  *reinterpret_cast<u32x4*>(V_out + size_t(j) * Hkv * HD + x) = v;
}

// Whole blocks between layouts. Reference block: [K | V][t][h][d] (40_:245-247).
// One thread per (block, which, t, 8 elements of the row).
// ids (may be null): block b of the reference-layout side is block ids[b] of the native side - the
// blocks of one slot in logical order, as a slot checkpoint file holds them (src/model/model.mm:653-655).
__global__ __launch_bounds__(256) void kv_relayout_kernel(const uint16_t* src, uint16_t* dst, int to_native, int n_blocks,
                                                          int Hkv, int HD, int bt, const int32_t* ids) {
  const int w = Hkv * HD;
  const long per_block = long(2) * bt * (w / 8);
  const long gid = long(blockIdx.x) * 256 + threadIdx.x;
  if (gid >= long(n_blocks) * per_block) return;
  const int b = int(gid / per_block);
  long rem = gid % per_block;
  const int which = int(rem / (long(bt) * (w / 8)));
  rem -= long(which) * bt * (w / 8);
  const int t = int(rem / (w / 8));
  const int x = int(rem % (w / 8)) * 8;
  const int kvh = x / HD, d = x % HD;
  const size_t ref_off = size_t(b) * 2 * bt * w + (size_t(which) * bt + t) * w + x;
  const size_t hb = (size_t(ids ? ids[b] : b) * Hkv + kvh) * size_t(2 * bt * HD);
  if (which == 0) {
    const size_t nat = hb + size_t(t) * HD + d;
    if (to_native) *reinterpret_cast<u32x4*>(dst + nat) = *reinterpret_cast<const u32x4*>(src + ref_off);
    else *reinterpret_cast<u32x4*>(dst + ref_off) = *reinterpret_cast<const u32x4*>(src + nat);
  } else {
    const size_t nat = hb + vt_elem(bt, HD, t, d);
    if (to_native) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(src + ref_off);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dst[nat + (2 * i) * kVtDim] = uint16_t(v[i] & 0xffffu);
        dst[nat + (2 * i + 1) * kVtDim] = uint16_t(v[i] >> 16);
      }
    } else {
      u32x4 v;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = uint32_t(src[nat + (2 * i) * kVtDim]) | (uint32_t(src[nat + (2 * i + 1) * kVtDim]) << 16);
      *reinterpret_cast<u32x4*>(dst + ref_off) = v;
    }
  }
}

// Batch V rows [n_rows][kv_ld] -> vt_stage [Hkv][n_rows16 / 16][HD][16]
// (16-row groups, rows past n_rows zero). One workgroup per (16-row group, KV
// head): the 16 x HD tile is transposed through LDS.
__global__ __launch_bounds__(256) void vt_stage_kernel(const uint16_t* Vb, uint16_t* vt, int n_rows, int n_groups, int HD,
                                                       int kv_ld) {
  __shared__ uint16_t sh[16][512 + 2];  // HD <= 512
  const int g = blockIdx.x, kvh = blockIdx.y;
  for (int i = threadIdx.x; i < 16 * (HD / 8); i += 256) {
    const int r = i / (HD / 8), x = (i % (HD / 8)) * 8;
    const int row = 16 * g + r;
    u32x4 v = {0, 0, 0, 0};
    if (row < n_rows) v = *reinterpret_cast<const u32x4*>(Vb + size_t(row) * kv_ld + size_t(kvh) * HD + x);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      sh[r][x + 2 * e] = uint16_t(v[e] & 0xffffu);
      sh[r][x + 2 * e + 1] = uint16_t(v[e] >> 16);
    }
  }
  __syncthreads();
  uint16_t* out = vt + (size_t(kvh) * n_groups + g) * size_t(HD) * 16;
  for (int i = threadIdx.x; i < HD * 2; i += 256) {  // (dim, half of the 16 rows): 16 bytes each
    const int d = i >> 1, h8 = (i & 1) * 8;
    u32x4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = uint32_t(sh[h8 + 2 * e][d]) | (uint32_t(sh[h8 + 2 * e + 1][d]) << 16);
    *reinterpret_cast<u32x4*>(out + size_t(d) * 16 + h8) = v;
  }
}

// One decode step further for every single-row tree of a device-resident pass: the row's own
// key joins the cache (P + 1), its position components move on by one, and its pool entry becomes
// the next token's (block list, or the slot's ring). The reference's decode chain
// (src/model/model.mm:779-850) has the host encode every step's records; here the device moves
// them on, so a chain of steps is enqueued - or captured in a graph - with no host work between.
__global__ __launch_bounds__(256) void chain_advance_kernel(esp_tree* trees, int n_trees, int4* pos, int4* row_table,
                                                            const int32_t* blocks, int bt, int ring) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n_trees) return;
  esp_tree t = trees[i];
  t.P += 1;
  trees[i] = t;
  int4 ps = pos[t.base];
  ps.x += 1;
  ps.y += 1;
  ps.z += 1;
  pos[t.base] = ps;
  if (row_table) {
    const int bi = t.P / bt;
    const int b = ring ? t.table + bi % ring : blocks[t.table + bi];
    row_table[t.base] = make_int4(b, t.P % bt, -1, -1);
  }
}

hipError_t launch_chain_advance(esp_tree* trees, int n_trees, int32_t* pos, int32_t* row_table, const int32_t* blocks, int bt,
                                int ring, hipStream_t st) {
  hipLaunchKernelGGL(chain_advance_kernel, dim3((n_trees + 255) / 256), dim3(256), 0, st, trees, n_trees,
                     reinterpret_cast<int4*>(pos), reinterpret_cast<int4*>(row_table), blocks, bt, ring);
  return hipGetLastError();
}

hipError_t launch_kv_save(const esp_attn_params* p, const void* Kb, const void* Vb, void* pool, const esp_kvsave* e, int n,
                          hipStream_t st) {
  hipLaunchKernelGGL(kv_save_kernel, dim3(unsigned((n + kSaveRows - 1) / kSaveRows), unsigned(p->Hkv)), dim3(256), 0, st,
                     (const uint16_t*)Kb, (const uint16_t*)Vb, (uint16_t*)pool, e, n, p->Hkv, p->head_dim, p->kv_ld, p->bt,
                     p->kv_base);
  return hipGetLastError();
}

hipError_t launch_kv_copy_blocks(const esp_attn_params* p, void* pool, const int32_t* pairs, int n_pairs, int n_layers,
                                 uint64_t region_elems, hipStream_t st) {
  const uint64_t blk2 = uint64_t(2) * p->bt * p->Hkv * p->head_dim;
  hipLaunchKernelGGL(kv_copy_blocks_kernel, dim3((unsigned)((blk2 / 8 + 255) / 256), n_pairs, n_layers), dim3(256), 0, st,
                     (uint16_t*)pool, (const int2*)pairs, blk2, region_elems);
  return hipGetLastError();
}

hipError_t launch_kv_gather(const esp_attn_params* p, const void* pool, const int32_t* blocks, int n, void* K_out,
                            void* V_out, hipStream_t st) {
  const long total = long(n) * (p->Hkv * p->head_dim / 8);
  hipLaunchKernelGGL(kv_gather_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, (const uint16_t*)pool, blocks,
                     n, (uint16_t*)K_out, (uint16_t*)V_out, p->Hkv, p->head_dim, p->bt, p->kv_base);
  return hipGetLastError();
}

hipError_t launch_kv_relayout(const esp_attn_params* p, const void* src, void* dst, int to_native, int n_blocks,
                              const int32_t* ids, hipStream_t st) {
  const long total = long(n_blocks) * 2 * p->bt * (p->Hkv * p->head_dim / 8);
  hipLaunchKernelGGL(kv_relayout_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, (const uint16_t*)src,
                     (uint16_t*)dst, to_native, n_blocks, p->Hkv, p->head_dim, p->bt, ids);
  return hipGetLastError();
}

hipError_t launch_vt_stage(const esp_attn_params* p, const void* Vb, void* vt, int n_rows, hipStream_t st) {
  const int n_groups = (n_rows + 15) / 16;
  hipLaunchKernelGGL(vt_stage_kernel, dim3(n_groups, p->Hkv), dim3(256), 0, st, (const uint16_t*)Vb, (uint16_t*)vt, n_rows,
                     n_groups, p->head_dim, p->kv_ld);
  return hipGetLastError();
}

}  // namespace esp
