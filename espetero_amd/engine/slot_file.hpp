// Slot checkpoint files in the reference's format, KV section: header, then the
// slot's KV blocks layer-major, logical block order, each block in the
// reference's layout [K plane | V plane] (src/model/model.mm:600-752: CkptHeader
// :604-614, slot_save :629-676, slot_load :677-752). The sections the reference
// appends for other subsystems (linear-attention state, MTP rows, n-gram state,
// sparse-attention index blocks, sliding rings) are written as absent (zero
// counts and sizes): a file written here loads in the reference for a model
// without them, and a reference file with them is refused here.
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
};

// kv: n_layers * n_blocks blocks of block_bytes, layer-major. Returns false when the file cannot be written.
inline bool slot_file_save(const std::string& path, const SlotInfo& s, const void* kv) {
  SlotHeader h{};
  h.magic = kSlotMagic;
  h.version = kSlotVersion;
  h.len = s.len;
  h.next_pos = s.next_pos;
  h.n_blocks = s.n_blocks;
  h.n_layers = s.n_layers;
  h.block_bytes = s.block_bytes;
  FILE* f = std::fopen(path.c_str(), "wb");
  if (!f) return false;
  const size_t n = size_t(s.n_layers) * size_t(s.n_blocks) * s.block_bytes;
  bool ok = std::fwrite(&h, 1, sizeof h, f) == sizeof h;
  ok = ok && (n == 0 || std::fwrite(kv, 1, n, f) == n);
  return std::fclose(f) == 0 && ok;
}

// 0 and the header's slot fields, or -1 when the file is missing, malformed, of another version, holds
// sections this build does not take, or does not have exactly the size its header implies (the checks
// of model.mm:700-714; bt: tokens per block of the loading pool).
inline int slot_file_info(const std::string& path, int bt, SlotInfo* out) {
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) return -1;
  SlotHeader h;
  const bool got = std::fread(&h, 1, sizeof h, f) == sizeof h;
  long size = -1;
  if (got && std::fseek(f, 0, SEEK_END) == 0) size = std::ftell(f);
  std::fclose(f);
  if (!got || h.magic != kSlotMagic || h.version != kSlotVersion) return -1;
  if (h.n_linear || h.conv_bytes || h.st_bytes || h.mtp_bytes || h.ple_bytes || h.i_layers || h.iblock_bytes || h.r_layers ||
      h.r_blocks || h.rblock_bytes)
    return -1;
  if (h.n_blocks < 0 || h.n_layers < 0 || h.len < 0 || int64_t(h.len) > int64_t(h.n_blocks) * bt) return -1;
  const uint64_t need = sizeof h + uint64_t(h.n_blocks) * uint64_t(h.n_layers) * h.block_bytes;
  if (size < 0 || uint64_t(size) != need) return -1;
  out->len = h.len;
  out->next_pos = h.next_pos;
  out->n_blocks = h.n_blocks;
  out->n_layers = h.n_layers;
  out->block_bytes = h.block_bytes;
  return 0;
}

// The block payload of a file slot_file_info accepted. kv: room for n_layers * n_blocks * block_bytes.
inline int slot_file_load(const std::string& path, const SlotInfo& s, void* kv) {
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) return -1;
  const size_t n = size_t(s.n_layers) * size_t(s.n_blocks) * s.block_bytes;
  bool ok = std::fseek(f, long(sizeof(SlotHeader)), SEEK_SET) == 0;
  ok = ok && (n == 0 || std::fread(kv, 1, n, f) == n);
  std::fclose(f);
  return ok ? 0 : -1;
}

}  // namespace espetero::engine
