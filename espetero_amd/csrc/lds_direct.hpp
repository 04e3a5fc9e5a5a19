// Direct global memory -> LDS loads (global_load_lds_dwordx4) and the wait-counter
// immediates the tiled attention kernels schedule them with.
#pragma once

#include "common.hpp"

namespace esp {

// 16 bytes per lane, global memory -> LDS, not through registers. `base` and
// `lds_addr` are wavefront-uniform; lane l reads base + lane_off and its bytes land
// at lds_addr + 16 l. Completion is tracked by the vector memory counter.
__device__ __forceinline__ void load_to_lds16(const void* base, uint32_t lane_off, uint32_t lds_addr) {
  // Uniform by construction; saying so lets the operands live in scalar registers. The builtin
  // returns a signed int: the halves go through uint32_t so the low one is not sign-extended.
  lds_addr = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_addr)));
  const uint64_t b64 = reinterpret_cast<uint64_t>(base);
  const uint32_t b_lo = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b64))));
  const uint32_t b_hi = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b64 >> 32))));
  base = reinterpret_cast<const void*>(uint64_t(b_lo) | (uint64_t(b_hi) << 32));
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(lane_off), "s"(base)
               : "memory");
}
// Four such loads whose global and LDS addresses both advance by 1024 bytes from one to the next:
// the instruction's immediate offset moves both, so one LDS base and one global base serve all four.
__device__ __forceinline__ void load_to_lds16_x4(const void* base, uint32_t o0, uint32_t o1, uint32_t o2, uint32_t o3,
                                                 uint32_t lds_addr) {
  lds_addr = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_addr)));
  const uint64_t b64 = reinterpret_cast<uint64_t>(base);
  const uint32_t b_lo = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b64))));
  const uint32_t b_hi = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b64 >> 32))));
  base = reinterpret_cast<const void*>(uint64_t(b_lo) | (uint64_t(b_hi) << 32));
  asm volatile(
      "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %5\n\t"
      "global_load_lds_dwordx4 %2, %5 offset:1024\n\t"
      "global_load_lds_dwordx4 %3, %5 offset:2048\n\t"
      "global_load_lds_dwordx4 %4, %5 offset:3072"
      :
      : "s"(lds_addr), "v"(o0), "v"(o1), "v"(o2), "v"(o3), "s"(base)
      : "memory");
}
__device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// s_waitcnt immediates (gfx9 layout): only the LDS / scalar-memory counter, at most 8 or 0 outstanding.
constexpr int kWaitLgkm8 = 0xC07F | (8 << 8), kWaitLgkm0 = 0xC07F;

constexpr int swap23(int x) { return (x & ~12) | ((x & 4) << 1) | ((x & 8) >> 1); }

}  // namespace esp
