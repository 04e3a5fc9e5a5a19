// Shared device helpers of the gfx950 attention kernels: vector types, MFMA
// wrappers for fp16 / bf16 operands, storage conversions, the native KV pool
// addressing and the kernel argument block.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <atomic>

#include "../../include/espetero_attn.h"

namespace esp {

using f32x4 = float __attribute__((ext_vector_type(4)));
using f32x16 = float __attribute__((ext_vector_type(16)));
using f16x8 = _Float16 __attribute__((ext_vector_type(8)));
using f16x4 = _Float16 __attribute__((ext_vector_type(4)));
using f16x2 = _Float16 __attribute__((ext_vector_type(2)));
using i16x4 = short __attribute__((ext_vector_type(4)));
using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));
using bf16x2 = __bf16 __attribute__((ext_vector_type(2)));
using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
using u32x2 = uint32_t __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;

// D(16x16) += A(16x32) * B(32x16). Lane l holds A[l % 16][8 (l / 16) .. + 7],
// B[8 (l / 16) .. + 7][l % 16] and D[4 (l / 16) .. + 3][l % 16].
template <int DT>
__device__ __forceinline__ f32x4 mfma16x32(u32x4 a, u32x4 b, f32x4 c) {
  if constexpr (DT == ESP_F16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
}

// D(16x16) += A(16x16) * B(16x16). Lane l holds A[l % 16][4 (l / 16) .. + 3],
// B[4 (l / 16) .. + 3][l % 16] and D[4 (l / 16) .. + 3][l % 16].
template <int DT>
__device__ __forceinline__ f32x4 mfma16x16(u32x2 a, u32x2 b, f32x4 c) {
  if constexpr (DT == ESP_F16) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(i16x4, a), __builtin_bit_cast(i16x4, b), c, 0, 0, 0);
  }
}

// D(32x32) += A(32x16) * B(16x32). Lane l holds A[l % 32][8 (l / 32) .. + 7],
// B[8 (l / 32) .. + 7][l % 32] and D[8 i + 4 (l / 32) + j][l % 32] at index 4 i + j.
template <int DT>
__device__ __forceinline__ f32x16 mfma32x16(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (DT == ESP_F16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
}

// Two fp32 -> one dword of two storage elements, round to nearest even.
template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (DT == ESP_F16) {
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  } else {
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
}

template <int DT>
__device__ __forceinline__ uint16_t pack1(float x) {
  if constexpr (DT == ESP_F16) {
    return __builtin_bit_cast(uint16_t, (_Float16)x);
  } else {
    return __builtin_bit_cast(uint16_t, (__bf16)x);
  }
}

// The two storage elements of a dword as fp32.
template <int DT>
__device__ __forceinline__ float unpack_lo(uint32_t w) {
  if constexpr (DT == ESP_F16) return float(__builtin_bit_cast(f16x2, w)[0]);
  else return __builtin_bit_cast(float, w << 16);
}
template <int DT>
__device__ __forceinline__ float unpack_hi(uint32_t w) {
  if constexpr (DT == ESP_F16) return float(__builtin_bit_cast(f16x2, w)[1]);
  else return __builtin_bit_cast(float, w & 0xffff0000u);
}

// acc + the two storage elements of a dword, in fp32: one v_dot2 against (1, 1).
template <int DT>
__device__ __forceinline__ float sum2(uint32_t w, float acc) {
  if constexpr (DT == ESP_F16) return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, w), __builtin_bit_cast(f16x2, 0x3c003c00u), acc, false);
  else return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), __builtin_bit_cast(bf16x2, 0x3f803f80u), acc, false);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Lets the matrix pipeline finish writing `acc` before anything after this point reads it. Matrix
// instructions are not interlocked against vector instructions that read their result: the compiler
// pads the distance with wait states, but only sees the instructions of one basic block. Where a branch
// follows the last matrix instruction and the first reader sits in the branch target, nothing was
// inserted, and the reader took the accumulator as it was before the last instruction landed
// (measured: the fourth register of a 16x16x32 result, read 3 instructions after the instruction's
// issue, lacked the last 32-dim slice of the dot products). Asking for the value in vector registers
// here, in the block of the matrix instruction, does it: a result the instruction left in vector
// registers waits out the 32 wait states below (the longest instruction, 16 passes, needs 19); one it
// left in accumulator registers is copied in front of this statement, in the same block, where the
// compiler does pad the distance.
template <typename T>
__device__ __forceinline__ void mfma_settle(T& acc) {
  asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc));
}

// Everything a kernel of this library reads: the call's device pointers and
// the per-layer constants, passed by value.
struct KArgs {
  const uint16_t* Q;
  const uint16_t* Kb;
  const uint16_t* Vb;
  const uint16_t* pool;
  const int32_t* blocks;
  const int4* desc;
  const int4* pos;
  uint16_t* O;
  const esp_tile* tiles;
  const esp_tree* trees;
  float* parts_o;   // [part][Hkv][cols][HD]   unnormalised O
  float* parts_ml;  // [part][Hkv][cols][2]    running max (log2 units), sum
  uint16_t* vt_stage;  // batch V transposed: [Hkv][n_rows16 / 16][HD][16]
  const float* gate;
  int32_t gate_ld, gate_hs, gate_off, gate_ds;  // gate_ds: 1 per-dim gates, 0 one gate per head
  int32_t H, Hkv, G, q_ld, kv_ld, bt, window, ring, bidi, R, cols, n_rows;
  float scale_log2;
  uint64_t kv_base;
};

// Native pool: element offset of (block b, KV head h); K rows follow at
// t * HD + d; V follows the K rows transposed in sub-blocks of 16 tokens,
// each [HD dims][16 tokens]: see vt_elem. A sub-block is 32 HD contiguous bytes
// at any block size, which is what both attention kernels load per 16 keys.
__device__ __forceinline__ size_t head_base(const KArgs& a, int HD, int b, int kvh) {
  return size_t(a.kv_base) + (size_t(b) * size_t(a.Hkv) + size_t(kvh)) * size_t(2 * a.bt * HD);
}

// Element offset of V[token t][dim d] from head_base; consecutive dims are kVtDim elements apart.
constexpr int kVtDim = 16;
__host__ __device__ __forceinline__ size_t vt_elem(int bt, int HD, int t, int d) {
  return size_t(bt) * HD + size_t(t >> 4) * size_t(16 * HD) + size_t(d) * kVtDim + size_t(t & 15);
}

// Block holding cached key j of a tree: its block list, or its slot's ring.
// The block list is read through the constant address space: no kernel writes it, and a kernel that
// stores to the pool (the fused prologue's append) would otherwise have to assume its stores reach the
// list and fetch every entry with a vector load whose wait drains the key and value loads in flight.
__device__ __forceinline__ int block_of(const KArgs& a, int table, int j) {
  using const_i32 = const int32_t __attribute__((address_space(4)));
  const int bi = j / a.bt;
  return a.ring ? table + bi % a.ring : ((const_i32*)a.blocks)[table + bi];
}

// Everything the prep kernel reads (esp_attn_prep).
struct PrepArgs {
  const float* X;
  const float* qn_w;
  const float* kn_w;
  const int4* pos;
  const float* inv_freq;
  const int32_t* rope_sel;
  uint16_t* Q;
  uint16_t* Kb;
  uint16_t* Vb;
  const int4* row_table;
  uint16_t* pool;
  esp_prep_params p;
};

// Everything the head gate kernel reads (esp_head_gate).
struct GateArgs {
  uint16_t* O;
  const uint16_t* X;
  const uint16_t* Wg;
  float* dots;
  int32_t n_rows, H, hd, hd_shift, D, q_ld, x_ld;  // hd_shift: log2(hd), -1 when hd is no power of two
};

// Events the next attention kernel launch records its own begin and end into (esp_attn_time_next);
// both null otherwise. One caller thread drives the library, so a plain pair is enough.
struct TimeNext {
  hipEvent_t start = nullptr, stop = nullptr;
};
TimeNext take_time_next();  // returns the pair and clears it

// Raises a kernel's dynamic LDS limit above the 48 KB default, once per device: the attribute
// belongs to the function on that device and stays for the life of the process.
template <auto Kern>
inline hipError_t allow_dynamic_lds(size_t bytes) {
  if (bytes <= 48 * 1024) return hipSuccess;
  static std::atomic<uint64_t> done{0};  // one bit per device ordinal
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = uint64_t(1) << (dev & 63);
  if (dev < 64 && (done.load(std::memory_order_acquire) & bit)) return hipSuccess;
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(Kern), hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes));
  if (e == hipSuccess && dev < 64) done.fetch_or(bit, std::memory_order_release);
  return e;
}

// Launches k; with a pending event pair the launch itself timestamps the kernel's begin and end.
template <typename K, typename... Args>
inline void launch_timed(K k, dim3 grid, dim3 block, size_t smem, hipStream_t st, Args... args) {
  const TimeNext t = take_time_next();
  if (t.start && t.stop)
    hipExtLaunchKernelGGL(k, grid, block, smem, st, t.start, t.stop, 0, args...);
  else
    hipLaunchKernelGGL(k, grid, block, smem, st, args...);
}

}  // namespace esp
