// Measured ceilings of one MI355X for the two bounds the attention kernels are held against, as kernels
// of their own (include/espetero_ceilings.h): what a plain streaming read reaches at a given size and
// page scatter, and what the matrix cores reach when the wavefront that feeds them also issues a given
// amount of vector arithmetic. The reference states its kernels against measured machine limits the
// same way (docs/kernel-guidelines.md:19-27: a measured stream peak and a measured MMA rate). A third kernel
// is the prefill kernel's step as a bare instruction stream, ingredient by ingredient.
// Measurement only: nothing in the attention path calls these.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "../../include/espetero_ceilings.h"

namespace {

using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
using f32x16 = float __attribute__((ext_vector_type(16)));
using f32x4 = float __attribute__((ext_vector_type(4)));
using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));

// Every wavefront reads whole pages, 16 bytes per lane per load, DEPTH pages in flight; page p of the
// launch is pages[p] (a scattered pool) or p itself (address order). The grid is what the streaming
// attention kernel uses: workgroups of 4 wavefronts, pages dealt round robin over all wavefronts.
template <int NT, int DEPTH>
__global__ __launch_bounds__(256, 2) void read_kernel(const char* __restrict__ base, const int32_t* __restrict__ pages, int n_pages,
                                                       int page_bytes, uint32_t* sink) {
  const int lane = threadIdx.x & 63;
  const int gw = blockIdx.x * 4 + (threadIdx.x >> 6), n_waves = gridDim.x * 4;
  const int per_page = page_bytes / 1024;  // 1 KB per load instruction and wavefront
  uint32_t acc = 0;
  for (int p0 = gw; p0 < n_pages; p0 += n_waves * DEPTH) {
    const char* pg[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int p = p0 + d * n_waves;
      const int q = p < n_pages ? p : p0;
      pg[d] = base + size_t(pages ? pages[q] : q) * size_t(page_bytes) + lane * 16;
    }
    for (int i = 0; i < per_page; i += 4) {
      u32x4 v[DEPTH][4];
#pragma unroll
      for (int d = 0; d < DEPTH; ++d)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const u32x4* src = reinterpret_cast<const u32x4*>(pg[d] + (i + j) * 1024);
          v[d][j] = NT ? __builtin_nontemporal_load(src) : *src;
        }
#pragma unroll
      for (int d = 0; d < DEPTH; ++d)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc ^= v[d][j].x ^ v[d][j].w;
    }
  }
  if (acc == 0x12345678u) sink[0] = acc;  // keeps the loads alive; never true for the bench's data
}

// One wavefront's instruction stream of a prefill step, nothing else: per matrix instruction
// (v_mfma_f32_32x32x16_bf16 over four accumulator chains, as Q K^T and P V alternate in the kernel) NV
// independent fp32 fused multiply-adds and NE v_exp_f32, interleaved by the scheduler one matrix
// instruction at a time. No memory, no LDS: what is left is the issue port the two kinds share.
template <int NV, int NE>
__global__ __launch_bounds__(256, 2) void issue_kernel(float* out, int iters, uint32_t seed, int random_data) {
  // Operands as an attention pass has them: eight different A and four different B fragments of random
  // 16-bit floats (sign and mantissa random, magnitude 0.25 .. 1), taken in turn. What the matrix cores
  // reach depends on it: with constant operands the same loop runs at the full 2.4 GHz, with random ones
  // the clock settles near 1.9 GHz under the power the multipliers then draw.
  auto rnd = [&](uint32_t x) {
    x = x * 2654435761u + seed;
    x ^= x >> 15;
    x *= 2246822519u;
    x ^= x >> 13;
    return random_data ? (x & 0x807f807fu) | 0x3e803e80u | ((x >> 3) & 0x01000100u) : 0x3f803f80u;
  };
  u32x4 a[8], b[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = u32x4{rnd(threadIdx.x + 64 * i), rnd(threadIdx.x + 64 * i + 1), rnd(threadIdx.x + 64 * i + 2), rnd(threadIdx.x + 64 * i + 3)};
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = u32x4{rnd(threadIdx.x + 999 * i + 7), rnd(threadIdx.x + 999 * i + 8), rnd(threadIdx.x + 999 * i + 9), rnd(threadIdx.x + 999 * i + 10)};
  f32x16 c[4] = {};
  float v[16], x[8];
#pragma unroll
  for (int i = 0; i < 16; ++i) v[i] = float(threadIdx.x + i) * 1e-3f;
#pragma unroll
  for (int i = 0; i < 8; ++i) x[i] = -float(threadIdx.x + i) * 1e-2f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      c[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[j & 7]), __builtin_bit_cast(bf16x8, b[(j >> 3) & 3]), c[j & 3], 0, 0, 0);
#pragma unroll
      for (int e = 0; e < NV; ++e) v[(j * NV + e) & 15] = __builtin_fmaf(v[(j * NV + e) & 15], 1.0001f, 0.5f);
#pragma unroll
      for (int e = 0; e < NE; ++e) x[(j * NE + e) & 7] = __builtin_amdgcn_exp2f(x[(j * NE + e) & 7]) - 1.5f;
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if (NV + 2 * NE > 0) __builtin_amdgcn_sched_group_barrier(0x002, NV + 2 * NE, 0);
    }
  }
  float r = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) r += c[0][i] + c[1][i] + c[2][i] + c[3][i] + v[i];
#pragma unroll
  for (int i = 0; i < 8; ++i) r += x[i];
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

// The prefill kernel's step as an instruction stream, built up one ingredient at a time (STAGE):
//   0  32 matrix instructions per step in chains of 8 on alternating accumulators, operands in registers
//   1  + the A operand of every matrix instruction read from LDS, 8 reads a group ahead of their use
//   2  + one workgroup barrier per step
//   3  + the softmax's share of vector work on the two middle groups (two v_exp_f32, two subtracts, two adds
//        per matrix instruction), laid by hand behind each matrix instruction
//   4  + each wavefront staging 8 KB per step from global memory straight into LDS (global_load_lds_dwordx4),
//        from a 4 MB window of `src` that stays in the caches
// ROWS: 1 = 32 query rows per wavefront (the kernels as built), 2 = 64 rows: every operand read feeds two
// matrix instructions, at one wavefront per SIMD. clk[2 w], clk[2 w + 1]: cycles and 100 MHz ticks workgroup w
// was alive, which give the clock the part ran at under this load.
__device__ __forceinline__ void stage_to_lds(const char* base, uint32_t lane_off, uint32_t lds_addr) {
  lds_addr = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_addr)));
  const uint64_t b64 = reinterpret_cast<uint64_t>(base);
  const uint32_t b_lo = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b64))));
  const uint32_t b_hi = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b64 >> 32))));
  base = reinterpret_cast<const char*>(uint64_t(b_lo) | (uint64_t(b_hi) << 32));
  asm volatile(
      "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2\n\t"
      "global_load_lds_dwordx4 %1, %2 offset:1024\n\t"
      "global_load_lds_dwordx4 %1, %2 offset:2048\n\t"
      "global_load_lds_dwordx4 %1, %2 offset:3072"
      :
      : "s"(lds_addr), "v"(lane_off), "s"(base)
      : "memory");
}

template <int STAGE, int ROWS>
__global__ __launch_bounds__(256, ROWS == 2 ? 1 : 2) void step_kernel(float* out, int iters, uint32_t seed, int random_data, const char* src,
                                                                       unsigned long long* clk) {
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  extern __shared__ __attribute__((aligned(16))) char lds[];  // 32 KB of operands, 32 KB of staging space
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  auto rnd = [&](uint32_t x) {
    x = x * 2654435761u + seed;
    x ^= x >> 15;
    x *= 2246822519u;
    x ^= x >> 13;
    return random_data ? (x & 0x807f807fu) | 0x3e803e80u | ((x >> 3) & 0x01000100u) : 0x3f803f80u;
  };
  const u32x4 a = {rnd(threadIdx.x), rnd(threadIdx.x + 999), rnd(threadIdx.x + 77), rnd(threadIdx.x + 5)};
  const u32x4 b = {rnd(threadIdx.x + 11), rnd(threadIdx.x + 13), rnd(threadIdx.x + 17), rnd(threadIdx.x + 19)};
  const u32x4 b2 = {rnd(threadIdx.x + 21), rnd(threadIdx.x + 23), rnd(threadIdx.x + 27), rnd(threadIdx.x + 29)};
  f32x16 c[4] = {}, c2[4] = {};
  float v[16], w[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    v[i] = -float(threadIdx.x + i) * 1e-3f;
    w[i] = v[i] * 0.5f;
  }
  for (int i = threadIdx.x; i < 16384; i += 256) reinterpret_cast<uint32_t*>(lds)[i] = rnd(i * 7 + blockIdx.x);
  __syncthreads();
  using lds_ptr = const __attribute__((address_space(3))) u32x4*;
  const uint32_t lds0 = uint32_t(uintptr_t(lds)), base = lds0 + lane * 16;
  auto mm = [](u32x4 x, u32x4 y, f32x16 z) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y), z, 0, 0, 0); };
  u32x4 ring[2][8];
  if constexpr (STAGE >= 1) {
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[0][j] = *reinterpret_cast<lds_ptr>(base + j * 1024);
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if constexpr (STAGE >= 1) {
#pragma unroll
        for (int j = 0; j < 8; ++j) ring[(g + 1) & 1][j] = *reinterpret_cast<lds_ptr>(base + ((g + 1) & 3) * 8192 + j * 1024);
        __builtin_amdgcn_s_waitcnt(0xC07F | (8 << 8));  // the 8 reads of a group ago have landed
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int ci = (g & 1) + 2 * (g >> 1);
        const u32x4 x = STAGE >= 1 ? ring[g & 1][j] : a;
        c[ci] = mm(x, b, c[ci]);
        if constexpr (ROWS == 2) c2[ci] = mm(x, b2, c2[ci]);
        if constexpr (STAGE >= 3) {
          if (g == 1 || g == 2) {
            v[2 * j] = __builtin_amdgcn_exp2f(v[2 * j] - c[3][0]);
            v[2 * j + 1] = __builtin_amdgcn_exp2f(v[2 * j + 1] - c[3][0]);
            v[(2 * j + 5) & 15] += v[(2 * j + 7) & 15];
            v[(2 * j + 9) & 15] += v[(2 * j + 11) & 15];
            asm volatile("" : "+v"(v[2 * j]), "+v"(v[2 * j + 1]));
            if constexpr (ROWS == 2) {
              w[2 * j] = __builtin_amdgcn_exp2f(w[2 * j] - c2[3][0]);
              w[2 * j + 1] = __builtin_amdgcn_exp2f(w[2 * j + 1] - c2[3][0]);
              w[(2 * j + 5) & 15] += w[(2 * j + 7) & 15];
              w[(2 * j + 9) & 15] += w[(2 * j + 11) & 15];
              asm volatile("" : "+v"(w[2 * j]), "+v"(w[2 * j + 1]));
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (STAGE >= 4) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (STAGE >= 2) __syncthreads();
    if constexpr (STAGE >= 4) {
      const size_t off = (size_t(blockIdx.x) * 977 * 16 + size_t(it) * 32768 + wave * 8192) & ((size_t(4) << 20) - 1 - 65535);
      stage_to_lds(src + off, lane * 16, lds0 + 32768 + wave * 8192);
      stage_to_lds(src + off + 4096, lane * 16, lds0 + 32768 + wave * 8192 + 4096);
    }
  }
  if constexpr (STAGE >= 4) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (threadIdx.x == 0 && clk) {
    clk[2 * blockIdx.x] = __builtin_readcyclecounter() - c0;
    clk[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
  float r = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) r += c[0][i] + c[1][i] + c[2][i] + c[3][i] + v[i] + c2[0][i] + c2[1][i] + c2[2][i] + c2[3][i] + w[i];
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

// The head-dim-256 prefill step as bare instruction streams: per step a compute unit multiplies 64 keys with 128 query
// rows of one 256-dim head (256 v_mfma_f32_32x32x16 or as many flops in 16x16x32), every A operand read from LDS,
// 32 scores per row-lane of softmax work, one barrier, 64 KB staged from `src` into LDS. Three shapes of the workgroup:
//   0  4 wavefronts x 32 rows, one per SIMD: the kernel as built (64 matrix instructions per wavefront and step)
//   1  8 wavefronts as 4 pairs: a wavefront takes half of the step's keys through Q K^T and the softmax, hands its
//      packed P to its partner through LDS and multiplies all 64 keys' P with its half of the dims
//   2  8 wavefronts x 16 rows on v_mfma_f32_16x16x32: every wavefront a whole head, reading all of K and V^T
// LOADS: 0 none, 1 all behind the barrier, 2 (shape 0) one behind each of the step's first 16 matrix instructions,
// 3 (shape 0) a second barrier in mid-step and each wavefront's loads beside groups of its own; 4, 5, 6 (shape 0): 0, 2, 1
// with the operand reads one by one behind the matrix instructions.
__device__ __forceinline__ void stage_one(const char* base, uint32_t lane_off, uint32_t lds_addr) {
  lds_addr = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_addr)));
  const uint64_t b64 = reinterpret_cast<uint64_t>(base);
  const uint32_t b_lo = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b64))));
  const uint32_t b_hi = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(b64 >> 32))));
  base = reinterpret_cast<const char*>(uint64_t(b_lo) | (uint64_t(b_hi) << 32));
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(lane_off), "s"(base) : "memory");
}
__device__ __forceinline__ uint32_t step256_rnd(uint32_t x) {
  x = x * 2654435761u + 12345u;
  x ^= x >> 15;
  x *= 2246822519u;
  x ^= x >> 13;
  return (x & 0x807f807fu) | 0x3e803e80u | ((x >> 3) & 0x01000100u);
}
__device__ __forceinline__ const char* step256_src(const char* src, int it, int wave, int per_wave) {
  return src + ((size_t(blockIdx.x) * 977 * 16 + size_t(it) * 65536) & ((size_t(8) << 20) - 1 - 131071)) + size_t(wave) * per_wave;
}

template <int LOADS, int W>
__device__ __forceinline__ void step256_body(float* out, int iters, const char* src, unsigned long long* clk) {
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  extern __shared__ __attribute__((aligned(16))) char lds[];  // 64 KB of operands, 64 KB of staging space
  const int lane = threadIdx.x & 63, wave = W >= 0 ? W : int(threadIdx.x >> 6);
  constexpr bool RI = LOADS >= 4;                                          // operand reads interleaved one by one
  constexpr int LD = LOADS == 4 ? 0 : LOADS == 5 ? 2 : LOADS == 6 ? 1 : LOADS;  // where the staging loads go
  const u32x4 b = {step256_rnd(threadIdx.x + 11), step256_rnd(threadIdx.x + 13), step256_rnd(threadIdx.x + 17), step256_rnd(threadIdx.x + 19)};
  f32x16 c[8] = {};
  float v[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) v[i] = -float(threadIdx.x + i) * 1e-3f;
  for (int i = threadIdx.x; i < 16384; i += 256) reinterpret_cast<uint32_t*>(lds)[i] = step256_rnd(i * 7 + blockIdx.x);
  __syncthreads();
  using lds_ptr = const __attribute__((address_space(3))) u32x4*;
  const uint32_t lds0 = uint32_t(uintptr_t(lds)), base = lds0 + lane * 16;
  auto mm = [](u32x4 x, u32x4 y, f32x16 z) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y), z, 0, 0, 0); };
  u32x4 ring[2][8];
#pragma unroll
  for (int j = 0; j < 8; ++j) ring[0][j] = *reinterpret_cast<lds_ptr>(base + j * 1024);
  for (int it = 0; it < iters; ++it) {
    const char* sp = step256_src(src, it, wave, 16384);
    const uint32_t dst = lds0 + 65536 + wave * 16384;
#pragma unroll
    for (int g = 0; g < 8; ++g) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if constexpr (!RI) ring[(g + 1) & 1][j] = *reinterpret_cast<lds_ptr>(base + ((g + 1) & 7) * 8192 + j * 1024);
      if constexpr (!RI) __builtin_amdgcn_s_waitcnt(0xC07F | (8 << 8));
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // reads one by one behind the matrix instructions: operand j of this group went out eight reads ago, and
        // seven younger ones are in flight when it is needed
        if constexpr (RI) __builtin_amdgcn_s_waitcnt(0xC07F | (7 << 8));
        c[g] = mm(ring[g & 1][j], b, c[g]);
        if constexpr (RI) ring[(g + 1) & 1][j] = *reinterpret_cast<lds_ptr>(base + ((g + 1) & 7) * 8192 + j * 1024);
        if (g >= 2 && g < 6) {  // the softmax's share: 32 scores per lane and step beside 32 of the matrix instructions
          v[(2 * j) & 15] = __builtin_amdgcn_exp2f(v[(2 * j) & 15] - c[7][0]);
          v[(2 * j + 5) & 15] += v[(2 * j + 7) & 15];
          asm volatile("" : "+v"(v[(2 * j) & 15]));
        }
        if constexpr (LD == 2) {
          if (g < 2) stage_one(sp + (8 * g + j) * 1024, lane * 16, dst + (8 * g + j) * 1024);
        }
        if constexpr (LOADS == 3) {  // wavefront w: half of its loads beside group w, the other half beside group 4 + w
          if ((g & 3) == W) stage_one(sp + (8 * (g >> 2) + j) * 1024, lane * 16, dst + (8 * (g >> 2) + j) * 1024);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (LOADS == 3) {
        if (g == 3) {  // the barrier in mid-step: the loads issued a step ago have landed, the later 16 stay in flight
          asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
          __syncthreads();
        }
      }
    }
    if constexpr (LOADS == 3) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else if constexpr (LD != 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if constexpr (LD == 1) {
#pragma unroll
      for (int q = 0; q < 16; ++q) stage_one(sp + q * 1024, lane * 16, dst + q * 1024);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (threadIdx.x == 0 && clk) {
    clk[2 * blockIdx.x] = __builtin_readcyclecounter() - c0;
    clk[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
  float r = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) r += c[0][i] + c[1][i] + c[2][i] + c[3][i] + c[4][i] + c[5][i] + c[6][i] + c[7][i] + v[i];
  out[blockIdx.x * 256 + threadIdx.x] = r;
}
template <int LOADS>
__global__ __launch_bounds__(256, 1) void step256_kernel(float* out, int iters, const char* src, unsigned long long* clk) {
  if constexpr (LOADS == 3) {  // a copy of the stream per wavefront, so that which groups carry its loads is fixed in the code
    switch (__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)) {
      case 0: step256_body<LOADS, 0>(out, iters, src, clk); break;
      case 1: step256_body<LOADS, 1>(out, iters, src, clk); break;
      case 2: step256_body<LOADS, 2>(out, iters, src, clk); break;
      default: step256_body<LOADS, 3>(out, iters, src, clk); break;
    }
  } else {
    step256_body<LOADS, -1>(out, iters, src, clk);
  }
}

template <int LOADS>
__global__ __launch_bounds__(512, 1) void step256_pairs_kernel(float* out, int iters, const char* src, unsigned long long* clk) {
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  extern __shared__ __attribute__((aligned(16))) char lds[];  // 64 KB of operands, 64 KB of staging space, 16 KB of exchange
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  u32x4 q[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) q[i] = u32x4{step256_rnd(threadIdx.x + 11 * i), step256_rnd(threadIdx.x + 13 * i), step256_rnd(threadIdx.x + 17), step256_rnd(threadIdx.x + 19)};
  f32x16 acc[4] = {};
  float l_run = 0.f;
  const float m_run = 3.0f;
  for (int i = threadIdx.x; i < 16384; i += 512) reinterpret_cast<uint32_t*>(lds)[i] = step256_rnd(i * 7 + blockIdx.x);
  __syncthreads();
  using lds_ptr = const __attribute__((address_space(3))) u32x4*;
  const uint32_t lds0 = uint32_t(uintptr_t(lds)), base = lds0 + lane * 16;
  u32x4* xch = reinterpret_cast<u32x4*>(lds + 131072);
  auto mm = [](u32x4 x, u32x4 y, f32x16 z) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y), z, 0, 0, 0); };
  auto pk = [](float a, float b) { return (__builtin_bit_cast(uint32_t, a) >> 16) | (__builtin_bit_cast(uint32_t, b) & 0xffff0000u); };
  u32x4 ring[2][8];
  u32x4 pb[4] = {};
  for (int it = 0; it < iters; ++it) {
    const char* sp = step256_src(src, it, wave, 8192);
    const uint32_t dst = lds0 + 65536 + wave * 8192;
    // Q K^T of this wavefront's 32 keys and their softmax
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[0][j] = *reinterpret_cast<lds_ptr>(base + (wave & 1) * 16384 + j * 1024);
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[1][j] = *reinterpret_cast<lds_ptr>(base + (wave & 1) * 16384 + 8192 + j * 1024);
    f32x16 s = {};
    __builtin_amdgcn_s_waitcnt(0xC07F | (8 << 8));
#pragma unroll
    for (int j = 0; j < 8; ++j) s = mm(ring[0][j], q[j], s);
    __builtin_amdgcn_s_waitcnt(0xC07F);
#pragma unroll
    for (int j = 0; j < 8; ++j) s = mm(ring[1][j], q[8 + j], s);
    __builtin_amdgcn_sched_barrier(0);
    float p[16], ps = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e], 0.088f, -m_run));
    pb[0] = u32x4{pk(p[0], p[1]), pk(p[2], p[3]), pk(p[4], p[5]), pk(p[6], p[7])};
    pb[1] = u32x4{pk(p[8], p[9]), pk(p[10], p[11]), pk(p[12], p[13]), pk(p[14], p[15])};
#pragma unroll
    for (int e = 0; e < 16; ++e) ps += p[e];
    l_run += ps;
    xch[(wave * 2 + 0) * 64 + lane] = pb[0];
    xch[(wave * 2 + 1) * 64 + lane] = pb[1];
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    if constexpr (LOADS != 0) {
#pragma unroll
      for (int qd = 0; qd < 8; ++qd) stage_one(sp + qd * 1024, lane * 16, dst + qd * 1024);
    }
    // P V: all 64 keys' P with this wavefront's 128 dims
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[0][j] = *reinterpret_cast<lds_ptr>(base + 32768 + j * 1024);
    pb[2] = xch[((wave ^ 1) * 2 + 0) * 64 + lane];
    pb[3] = xch[((wave ^ 1) * 2 + 1) * 64 + lane];
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[1][j] = *reinterpret_cast<lds_ptr>(base + 32768 + 8192 + j * 1024);
    __builtin_amdgcn_s_waitcnt(0xC07F | (8 << 8));
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j & 3] = mm(ring[0][j], pb[j >> 2], acc[j & 3]);
    __builtin_amdgcn_s_waitcnt(0xC07F);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j & 3] = mm(ring[1][j], pb[2 + (j >> 2)], acc[j & 3]);
    __builtin_amdgcn_sched_barrier(0);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (threadIdx.x == 0 && clk) {
    clk[2 * blockIdx.x] = __builtin_readcyclecounter() - c0;
    clk[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
  float r = l_run;
#pragma unroll
  for (int i = 0; i < 16; ++i) r += acc[0][i] + acc[1][i] + acc[2][i] + acc[3][i];
  out[blockIdx.x * 512 + threadIdx.x] = r;
}

template <int LOADS>
__global__ __launch_bounds__(512, 1) void step256_rows16_kernel(float* out, int iters, const char* src, unsigned long long* clk) {
  const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
  extern __shared__ __attribute__((aligned(16))) char lds[];  // 64 KB of operands, 64 KB of staging space
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  u32x4 q[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) q[i] = u32x4{step256_rnd(threadIdx.x + 11 * i), step256_rnd(threadIdx.x + 13 * i), step256_rnd(threadIdx.x + 17), step256_rnd(threadIdx.x + 19)};
  f32x4 acc[16] = {};
  float l_run = 0.f;
  const float m_run = 3.0f;
  for (int i = threadIdx.x; i < 16384; i += 512) reinterpret_cast<uint32_t*>(lds)[i] = step256_rnd(i * 7 + blockIdx.x);
  __syncthreads();
  using lds_ptr = const __attribute__((address_space(3))) u32x4*;
  const uint32_t lds0 = uint32_t(uintptr_t(lds)), base = lds0 + lane * 16;
  auto mm = [](u32x4 x, u32x4 y, f32x4 z) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y), z, 0, 0, 0); };
  auto pk = [](float a, float b) { return (__builtin_bit_cast(uint32_t, a) >> 16) | (__builtin_bit_cast(uint32_t, b) & 0xffff0000u); };
  u32x4 ring[2][8];
  u32x4 pb[2] = {};
  for (int it = 0; it < iters; ++it) {
    const char* sp = step256_src(src, it, wave, 8192);
    const uint32_t dst = lds0 + 65536 + wave * 8192;
    f32x4 s[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[0][j] = *reinterpret_cast<lds_ptr>(base + j * 1024);
#pragma unroll
    for (int t = 0; t < 4; ++t) {  // Q K^T: 4 tiles of 16 keys, 8 slices of 32 dims each
#pragma unroll
      for (int j = 0; j < 8; ++j) ring[(t + 1) & 1][j] = *reinterpret_cast<lds_ptr>(base + (t + 1) * 8192 + j * 1024);
      __builtin_amdgcn_s_waitcnt(0xC07F | (8 << 8));
      s[t] = f32x4{0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) s[t] = mm(ring[t & 1][j], q[j], s[t]);
      __builtin_amdgcn_sched_barrier(0);
    }
    float p[16], ps = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) p[4 * t + e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][e], 0.088f, -m_run));
    pb[0] = u32x4{pk(p[0], p[1]), pk(p[2], p[3]), pk(p[4], p[5]), pk(p[6], p[7])};
    pb[1] = u32x4{pk(p[8], p[9]), pk(p[10], p[11]), pk(p[12], p[13]), pk(p[14], p[15])};
#pragma unroll
    for (int e = 0; e < 16; ++e) ps += p[e];
    l_run += ps;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int g = 0; g < 4; ++g) {  // P V: 16 tiles of 16 dims x 2 halves of the step's keys
      if (g < 3) {
#pragma unroll
        for (int j = 0; j < 8; ++j) ring[(g + 1) & 1][j] = *reinterpret_cast<lds_ptr>(base + 32768 + (g + 1) * 8192 + j * 1024);
        __builtin_amdgcn_s_waitcnt(0xC07F | (8 << 8));
      } else {
        __builtin_amdgcn_s_waitcnt(0xC07F);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[4 * g + (j >> 1)] = mm(ring[g & 1][j], pb[j & 1], acc[4 * g + (j >> 1)]);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    if constexpr (LOADS != 0) {
#pragma unroll
      for (int qd = 0; qd < 8; ++qd) stage_one(sp + qd * 1024, lane * 16, dst + qd * 1024);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (threadIdx.x == 0 && clk) {
    clk[2 * blockIdx.x] = __builtin_readcyclecounter() - c0;
    clk[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
  float r = l_run;
#pragma unroll
  for (int i = 0; i < 16; ++i) r += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  out[blockIdx.x * 512 + threadIdx.x] = r;
}

template <typename K, typename... Args>
hipError_t launch_lds(K k, size_t lds_bytes, dim3 grid, dim3 block, hipStream_t st, hipEvent_t e0, hipEvent_t e1, Args... args) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
  if (e != hipSuccess) return e;
  if (e0 && e1) hipExtLaunchKernelGGL(k, grid, block, lds_bytes, st, e0, e1, 0, args...);
  else hipLaunchKernelGGL(k, grid, block, lds_bytes, st, args...);
  return hipGetLastError();
}

template <typename K, typename... Args>
hipError_t launch(K k, dim3 grid, dim3 block, hipStream_t st, hipEvent_t e0, hipEvent_t e1, Args... args) {
  if (e0 && e1) hipExtLaunchKernelGGL(k, grid, block, 0, st, e0, e1, 0, args...);
  else hipLaunchKernelGGL(k, grid, block, 0, st, args...);
  return hipGetLastError();
}

}  // namespace

extern "C" {

int esp_ceiling_hbm_read(const void* base, const int32_t* pages, int32_t n_pages, int32_t page_bytes, int32_t nontemporal,
                         int32_t workgroups, uint32_t* sink, void* stream, void* start_event, void* stop_event) {
  if (!base || !sink || n_pages <= 0 || page_bytes < 4096 || page_bytes % 4096 || workgroups <= 0) return 1;
  const auto st = static_cast<hipStream_t>(stream);
  const auto e0 = static_cast<hipEvent_t>(start_event), e1 = static_cast<hipEvent_t>(stop_event);
  const char* b = static_cast<const char*>(base);
  const hipError_t e = nontemporal ? launch(read_kernel<1, 2>, dim3(workgroups), dim3(256), st, e0, e1, b, pages, n_pages, page_bytes, sink)
                                   : launch(read_kernel<0, 2>, dim3(workgroups), dim3(256), st, e0, e1, b, pages, n_pages, page_bytes, sink);
  return e == hipSuccess ? 0 : 3;
}

int esp_ceiling_mfma_issue(int32_t valu_per_mfma, int32_t exp_per_mfma, int32_t random_data, int32_t workgroups, int32_t iters, float* out, void* stream,
                           void* start_event, void* stop_event) {
  if (!out || workgroups <= 0 || iters <= 0) return 1;
  const auto st = static_cast<hipStream_t>(stream);
  const auto e0 = static_cast<hipEvent_t>(start_event), e1 = static_cast<hipEvent_t>(stop_event);
  const dim3 g(workgroups), b(256);
  const int key = valu_per_mfma * 10 + exp_per_mfma;
  hipError_t e;
  switch (key) {
    case 0: e = launch(issue_kernel<0, 0>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 10: e = launch(issue_kernel<1, 0>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 20: e = launch(issue_kernel<2, 0>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 30: e = launch(issue_kernel<3, 0>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 40: e = launch(issue_kernel<4, 0>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 60: e = launch(issue_kernel<6, 0>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 1: e = launch(issue_kernel<0, 1>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 11: e = launch(issue_kernel<1, 1>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 21: e = launch(issue_kernel<2, 1>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 31: e = launch(issue_kernel<3, 1>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 41: e = launch(issue_kernel<4, 1>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    case 51: e = launch(issue_kernel<5, 1>, g, b, st, e0, e1, out, iters, 1u, random_data); break;
    default: return 2;
  }
  return e == hipSuccess ? 0 : 3;
}

int esp_ceiling_prefill_step(int32_t stage, int32_t rows, int32_t random_data, int32_t workgroups, int32_t iters, float* out, const void* src,
                             unsigned long long* clk, void* stream, void* start_event, void* stop_event) {
  if (!out || workgroups <= 0 || iters <= 0 || (stage >= 4 && !src)) return 1;
  const auto st = static_cast<hipStream_t>(stream);
  const auto e0 = static_cast<hipEvent_t>(start_event), e1 = static_cast<hipEvent_t>(stop_event);
  const dim3 g(workgroups), b(256);
  const char* s = static_cast<const char*>(src);
  hipError_t e;
  switch (stage * 10 + rows) {
    case 1: e = launch_lds(step_kernel<0, 1>, 65536, g, b, st, e0, e1, out, iters, 1u, random_data, s, clk); break;
    case 11: e = launch_lds(step_kernel<1, 1>, 65536, g, b, st, e0, e1, out, iters, 1u, random_data, s, clk); break;
    case 21: e = launch_lds(step_kernel<2, 1>, 65536, g, b, st, e0, e1, out, iters, 1u, random_data, s, clk); break;
    case 31: e = launch_lds(step_kernel<3, 1>, 65536, g, b, st, e0, e1, out, iters, 1u, random_data, s, clk); break;
    case 41: e = launch_lds(step_kernel<4, 1>, 65536, g, b, st, e0, e1, out, iters, 1u, random_data, s, clk); break;
    case 12: e = launch_lds(step_kernel<1, 2>, 65536, g, b, st, e0, e1, out, iters, 1u, random_data, s, clk); break;
    case 32: e = launch_lds(step_kernel<3, 2>, 65536, g, b, st, e0, e1, out, iters, 1u, random_data, s, clk); break;
    case 42: e = launch_lds(step_kernel<4, 2>, 65536, g, b, st, e0, e1, out, iters, 1u, random_data, s, clk); break;
    default: return 2;
  }
  return e == hipSuccess ? 0 : 3;
}

int esp_ceiling_prefill_step256(int32_t shape, int32_t loads, int32_t workgroups, int32_t iters, float* out, const void* src, unsigned long long* clk,
                                void* stream, void* start_event, void* stop_event) {
  if (!out || workgroups <= 0 || iters <= 0 || (loads != 0 && !src)) return 1;
  const auto st = static_cast<hipStream_t>(stream);
  const auto e0 = static_cast<hipEvent_t>(start_event), e1 = static_cast<hipEvent_t>(stop_event);
  const dim3 g(workgroups);
  const char* s = static_cast<const char*>(src);
  hipError_t e;
  switch (shape * 10 + loads) {
    case 0: e = launch_lds(step256_kernel<0>, 131072, g, dim3(256), st, e0, e1, out, iters, s, clk); break;
    case 1: e = launch_lds(step256_kernel<1>, 131072, g, dim3(256), st, e0, e1, out, iters, s, clk); break;
    case 2: e = launch_lds(step256_kernel<2>, 131072, g, dim3(256), st, e0, e1, out, iters, s, clk); break;
    case 3: e = launch_lds(step256_kernel<3>, 131072, g, dim3(256), st, e0, e1, out, iters, s, clk); break;
    case 4: e = launch_lds(step256_kernel<4>, 131072, g, dim3(256), st, e0, e1, out, iters, s, clk); break;
    case 5: e = launch_lds(step256_kernel<5>, 131072, g, dim3(256), st, e0, e1, out, iters, s, clk); break;
    case 6: e = launch_lds(step256_kernel<6>, 131072, g, dim3(256), st, e0, e1, out, iters, s, clk); break;
    case 10: e = launch_lds(step256_pairs_kernel<0>, 147456, g, dim3(512), st, e0, e1, out, iters, s, clk); break;
    case 11: e = launch_lds(step256_pairs_kernel<1>, 147456, g, dim3(512), st, e0, e1, out, iters, s, clk); break;
    case 20: e = launch_lds(step256_rows16_kernel<0>, 131072, g, dim3(512), st, e0, e1, out, iters, s, clk); break;
    case 21: e = launch_lds(step256_rows16_kernel<1>, 131072, g, dim3(512), st, e0, e1, out, iters, s, clk); break;
    default: return 2;
  }
  return e == hipSuccess ? 0 : 3;
}

}  // extern "C"
