// head_gate: the head-wise output gate that follows the attention of a layer,
// O[row, h, :] *= sigmoid(x[row] . Wg[h]) (sp_head_gate, kernels/85_spark.metal:96-128;
// dispatched at src/model/impl/gemma.h:481-492). The reference runs one threadgroup
// of scalar dots per (head, row); its own note says a GEMM dispatch cost more than
// the dots at 16 rows (src/model/impl/gemma_load.h:292-294).
//
// Mapping to gfx950: HBM bound (X once, O there and back; Wg stays in L2). One
// workgroup takes 16 rows. The dots of 16 rows x 16 heads x 32 model dims are one
// v_mfma_f32_16x16x32 whose operands are 16-byte loads straight from X and Wg; the
// four wavefronts take a quarter of the model dims each and their sums meet in LDS. Then
// the workgroup streams its 16 rows of O through registers, 16 bytes per lane and
// 16 loads in flight per lane (the first 16 issued before the dots, so that their
// latency lies under the dots'), or writes the dots out for the attention kernels'
// own epilogue to use.
#include "common.hpp"

namespace esp {

constexpr int kGateRows = 16;

template <int DT>
__device__ __forceinline__ float2 unpack2(uint32_t u) {
  if constexpr (DT == ESP_F16) {
    const f16x2 v = __builtin_bit_cast(f16x2, u);
    return make_float2(float(v[0]), float(v[1]));
  } else {
    return make_float2(__builtin_bit_cast(float, u << 16), __builtin_bit_cast(float, u & 0xffff0000u));
  }
}

template <int DT, int NB>  // NB: blocks of 16 heads
__global__ __launch_bounds__(256) void head_gate_kernel(const GateArgs a) {
  constexpr int R = kGateRows, U = NB == 1 ? 8 : (NB == 2 ? 4 : 2), B = 16;
  __shared__ float sums[4][R][16 * NB + 1];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int c16 = lane & 15, q4 = lane >> 4;
  const int row0 = blockIdx.x * R;
  const int rows = min(R, a.n_rows - row0);

  // The workgroup's part of O is rows x vpr 16-byte vectors; a thread takes every 256th of them in
  // row-major order, B at a time: with rows that follow one another in memory a batch is one
  // contiguous 64 KB. (r, v) walk that order without a division.
  const int vpr = a.H * a.hd / 8;
  int r_ld = 0, v_ld = tid;
  auto normalise = [&](int& r, int& v) {
    while (v >= vpr) {
      v -= vpr;
      ++r;
    }
  };
  normalise(r_ld, v_ld);
  u32x4 o[B];
  auto load_batch = [&]() {
#pragma unroll
    for (int j = 0; j < B; ++j) {
      o[j] = (a.O && r_ld < rows) ? *reinterpret_cast<const u32x4*>(a.O + size_t(row0 + r_ld) * a.q_ld + 8 * v_ld) : u32x4{0, 0, 0, 0};
      v_ld += 256;
      normalise(r_ld, v_ld);
    }
  };
  load_batch();  // in flight while the dots are formed

  // ---- dots: rows past the end repeat the last row, heads past H repeat the last head; neither is read back
  const uint16_t* xp = a.X + size_t(row0 + min(c16, rows - 1)) * a.x_ld + 8 * q4;
  const uint16_t* wp[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) wp[nb] = a.Wg + size_t(min(16 * nb + c16, a.H - 1)) * a.D + 8 * q4;
  f32x4 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0, 0, 0, 0};
  // A wavefront's chunks follow one another; each workgroup starts its walk somewhere else, so that
  // the workgroups of an XCD do not all ask its L2 for the same lines of Wg at the same moment.
  const int n_chunks = (a.D + 31) / 32, per_wave = (n_chunks + 3) / 4;
  const int rot = int((blockIdx.x * 7u) % unsigned(per_wave));
  for (int i = 0; i < per_wave; i += U) {
    u32x4 xa[U], wb[NB][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int ci = i + u + rot;
      if (ci >= per_wave) ci -= per_wave;
      const int k = 32 * (wave * per_wave + ci);
      const bool ok = i + u < per_wave && k + 8 * q4 < a.D;  // D is a multiple of 8: a lane's 8 dims exist or do not
      xa[u] = ok ? *reinterpret_cast<const u32x4*>(xp + k) : u32x4{0, 0, 0, 0};
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) wb[nb][u] = ok ? *reinterpret_cast<const u32x4*>(wp[nb] + k) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nb] = mfma16x32<DT>(xa[u], wb[nb][u], acc[nb]);
  }
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int i = 0; i < 4; ++i) sums[wave][4 * q4 + i][16 * nb + c16] = acc[nb][i];
  __syncthreads();
  for (int i = tid; i < R * 16 * NB; i += 256) {
    const int r = i / (16 * NB), h = i % (16 * NB);
    const float dot = (sums[0][r][h] + sums[1][r][h]) + (sums[2][r][h] + sums[3][r][h]);
    if (a.dots && r < rows && h < a.H) a.dots[size_t(row0 + r) * a.H + h] = dot;
    sums[0][r][h] = 1.0f / (1.0f + __expf(-dot));
  }
  if (!a.O) return;
  __syncthreads();

  // ---- O = storage(float(O) * gate), 8 elements per lane and load
  int r_st = 0, v_st = tid;
  normalise(r_st, v_st);
  while (r_st < rows) {
#pragma unroll
    for (int j = 0; j < B; ++j) {
      if (r_st < rows) {
        const int h = a.hd_shift >= 0 ? (8 * v_st) >> a.hd_shift : (8 * v_st) / a.hd;
        const float g = sums[0][r_st][h];
        u32x4 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float2 f = unpack2<DT>(o[j][e]);
          out[e] = pack2<DT>(f.x * g, f.y * g);
        }
        *reinterpret_cast<u32x4*>(a.O + size_t(row0 + r_st) * a.q_ld + 8 * v_st) = out;
      }
      v_st += 256;
      normalise(r_st, v_st);
    }
    if (r_ld < rows) load_batch();
  }
}

hipError_t launch_head_gate(int dt, const GateArgs& a, hipStream_t st) {
  const dim3 grid((a.n_rows + kGateRows - 1) / kGateRows), block(256);
  const int nb = (a.H + 15) / 16;
#define ESP_GATE_CASE(DT, NB) \
  if (dt == DT && nb == NB) { launch_timed(head_gate_kernel<DT, NB>, grid, block, 0, st, a); return hipGetLastError(); }
  ESP_GATE_CASE(ESP_F16, 1) ESP_GATE_CASE(ESP_F16, 2) ESP_GATE_CASE(ESP_F16, 3) ESP_GATE_CASE(ESP_F16, 4)
  ESP_GATE_CASE(ESP_BF16, 1) ESP_GATE_CASE(ESP_BF16, 2) ESP_GATE_CASE(ESP_BF16, 3) ESP_GATE_CASE(ESP_BF16, 4)
#undef ESP_GATE_CASE
  return hipErrorInvalidValue;
}

}  // namespace esp
