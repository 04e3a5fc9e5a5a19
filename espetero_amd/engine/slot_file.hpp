// Slot checkpoint files in the reference's format, KV section: header, then the
// slot's KV blocks layer-major, logical block order, each block in the
// reference's layout [K plane | V plane] (src/model/model.mm:600-752: CkptHeader
// :604-614, slot_save :629-676, slot_load :677-752). The sections the reference
// appends for other subsystems (linear-attention state, MTP rows, n-gram state,
// sparse-attention index blocks) are written as absent (zero counts and sizes):
// a file written here loads in the reference for a model without them, and a
// reference file with them is refused here. The last section, Gemma's sliding
// rings (model.mm:664-669, 737-742: per sliding layer the slot's r_blocks ring
// blocks in ring order, same block layout), is written and read when the
// caller brings rings; a file with rings is refused by a caller that takes none.
//
// Host-only: the block payload passes through host memory; esp_kv_export_blocks /
// esp_kv_import_blocks convert between it and the device pool's native layout.
#pragma once

#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

namespace espetero::engine {

struct SlotHeader {  // field for field CkptHeader (model.mm:604-614)
  uint32_t magic, version;
  int32_t len, next_pos, mtp_ok, n_lh, mh_pos[3];
  int32_t n_blocks, n_layers, n_linear;
  uint64_t block_bytes, conv_bytes, st_bytes, mtp_bytes, ple_bytes;
  int32_t i_layers, pad;
  uint64_t iblock_bytes;
  int32_t r_layers, r_blocks;
  uint64_t rblock_bytes;
};
static_assert(sizeof(SlotHeader) == 120, "header layout");
constexpr uint32_t kSlotMagic = 0x554b5043u;  // model.mm:615
constexpr uint32_t kSlotVersion = 4;          // model.mm:640

struct SlotInfo {
  int32_t len = 0, next_pos = 0, n_blocks = 0, n_layers = 0;
  uint64_t block_bytes = 0;  // 2 * bt * Hkv * head_dim * sizeof(element)
  int32_t r_layers = 0, r_blocks = 0;  // sliding layers, blocks per ring
  uint64_t rblock_bytes = 0;
  uint64_t ring_bytes() const { return uint64_t(r_layers) * uint64_t(r_blocks) * rblock_bytes; }
};

// kv: n_layers * n_blocks blocks of block_bytes, layer-major; rings: r_layers * r_blocks blocks of rblock_bytes,
// layer-major (nullptr with r_layers 0). Returns false when the file cannot be written.
inline bool slot_file_save(const std::string& path, const SlotInfo& s, const void* kv, const void* rings = nullptr) {
  SlotHeader h{};
  h.magic = kSlotMagic;
  h.version = kSlotVersion;
  h.len = s.len;
  h.next_pos = s.next_pos;
  h.n_blocks = s.n_blocks;
  h.n_layers = s.n_layers;
  h.block_bytes = s.block_bytes;
  h.r_layers = s.r_layers;
  h.r_blocks = s.r_layers ? s.r_blocks : 0;
  h.rblock_bytes = s.r_layers ? s.rblock_bytes : 0;
  FILE* f = std::fopen(path.c_str(), "wb");
  if (!f) return false;
  const size_t n = size_t(s.n_layers) * size_t(s.n_blocks) * s.block_bytes;
  const size_t nr = size_t(s.ring_bytes());
  bool ok = std::fwrite(&h, 1, sizeof h, f) == sizeof h;
  ok = ok && (n == 0 || std::fwrite(kv, 1, n, f) == n);
  ok = ok && (nr == 0 || (rings && std::fwrite(rings, 1, nr, f) == nr));
  return std::fclose(f) == 0 && ok;
}

// 0 and the header's slot fields, or -1 when the file is missing, malformed, of another version, holds
// sections this build does not take, or does not have exactly the size its header implies (the checks
// of model.mm:700-714; bt: tokens per block of the loading pool). take_rings: whether the caller has ring
// pools to load a ring section into.
inline int slot_file_info(const std::string& path, int bt, SlotInfo* out, bool take_rings = false) {
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) return -1;
  SlotHeader h;
  const bool got = std::fread(&h, 1, sizeof h, f) == sizeof h;
  long size = -1;
  if (got && std::fseek(f, 0, SEEK_END) == 0) size = std::ftell(f);
  std::fclose(f);
  if (!got || h.magic != kSlotMagic || h.version != kSlotVersion) return -1;
  if (h.n_linear || h.conv_bytes || h.st_bytes || h.mtp_bytes || h.ple_bytes || h.i_layers || h.iblock_bytes) return -1;
  if (!take_rings && (h.r_layers || h.r_blocks || h.rblock_bytes)) return -1;
  if (h.r_layers < 0 || h.r_blocks < 0 || (h.r_layers == 0 && (h.r_blocks || h.rblock_bytes))) return -1;
  if (h.n_blocks < 0 || h.n_layers < 0 || h.len < 0 || int64_t(h.len) > int64_t(h.n_blocks) * bt) return -1;
  const uint64_t need = sizeof h + uint64_t(h.n_blocks) * uint64_t(h.n_layers) * h.block_bytes +
                        uint64_t(h.r_layers) * uint64_t(h.r_blocks) * h.rblock_bytes;
  if (size < 0 || uint64_t(size) != need) return -1;
  out->len = h.len;
  out->next_pos = h.next_pos;
  out->n_blocks = h.n_blocks;
  out->n_layers = h.n_layers;
  out->block_bytes = h.block_bytes;
  out->r_layers = h.r_layers;
  out->r_blocks = h.r_blocks;
  out->rblock_bytes = h.rblock_bytes;
  return 0;
}

// The block payload of a file slot_file_info accepted. kv: room for n_layers * n_blocks * block_bytes;
// rings: room for s.ring_bytes() (nullptr when the file has none).
inline int slot_file_load(const std::string& path, const SlotInfo& s, void* kv, void* rings = nullptr) {
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) return -1;
  const size_t n = size_t(s.n_layers) * size_t(s.n_blocks) * s.block_bytes;
  const size_t nr = size_t(s.ring_bytes());
  bool ok = std::fseek(f, long(sizeof(SlotHeader)), SEEK_SET) == 0;
  ok = ok && (n == 0 || std::fread(kv, 1, n, f) == n);
  ok = ok && (nr == 0 || (rings && std::fread(rings, 1, nr, f) == nr));
  std::fclose(f);
  return ok ? 0 : -1;
}

}  // namespace espetero::engine
