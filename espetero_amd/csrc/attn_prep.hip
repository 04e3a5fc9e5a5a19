// attn_prep: what runs between the fused in-projection and the attention of a
// layer. Per (row, head) of the fp32 projection: RMSNorm over the head with a
// learned weight (queries and keys), rotary embedding of the leading
// `rope_dims` dims in the half-split pairing (d, d + rope_dims / 2), cast to the
// storage type; values are cast (or normalised without weight); the rows' K / V
// also go straight into their pool entries, so no kv_save dispatch follows.
//
// One kernel for the reference's three: attn_prep (kernels/40_attention.metal:9-102:
// head_dim 256, 64 rotating dims, the gate beside each query head, the folded
// append), g4_attn_prep<HD> (kernels/80_gemma.metal:52-108: all dims rotate,
// values normalised) and q3m_attn_prep<HD> (kernels/82_qwen3_omni.metal:30-88:
// per-frequency position component, query scale).
//
// Mapping to gfx950: HBM bound (fp32 in, 16-bit out). One workgroup = 8 consecutive
// rows x 1024 columns (8 heads of 128 dims, 4 of 256); a lane owns 4 consecutive dims (one 16-byte load, one 8-byte store), so a
// head is 32 or 64 lanes and the norm's sum and the rotation's partner are lane
// exchanges inside a wavefront. A thread works on the same (head, dims) of all 8
// rows at once: 8 independent loads in flight. The rows' cos / sin tables
// (rope_dims / 2 entries each) are computed once per workgroup into LDS and shared
// by its heads: the reference computes them once per (row, head).
// The folded append writes K rows as they are. V lies transposed in the pool
// (16-token sub-blocks, tokens contiguous per dim): when the 8 rows go to 8 consecutive, 8-aligned
// positions of one block - every full group of a prefill chunk - their V is
// staged in LDS and leaves as one 16-byte store per (head, dim); any other
// arrangement (decode rows of different sequences, a row saved into two slots)
// takes element stores.
#include <type_traits>

#include "common.hpp"
#include "prep_math.hpp"

namespace esp {


constexpr int kPrepRows = 8;

template <int DT, int HD>
__global__ __launch_bounds__(256) void attn_prep_kernel(const PrepArgs a, int n_rows) {
  constexpr int R = kPrepRows;
  constexpr int EPL = prep_epl(HD);  // consecutive dims per lane: a head never spans more than one wavefront
  constexpr int LPH = HD / EPL;      // lanes per head
  constexpr int HPP = 256 / LPH;         // heads of the workgroup
  __shared__ float2 cs[R][HD / 2];       // (cos, sin) per row and frequency
  __shared__ int run_ok;
  __shared__ __attribute__((aligned(16))) uint16_t vstage[R][HPP * HD];  // the workgroup's V heads, for the transposed append
  const esp_prep_params& p = a.p;
  const int row0 = blockIdx.x * R;
  const int rows = min(R, n_rows - row0);
  const int tid = threadIdx.x;
  const int half = p.rope_dims / 2;
  for (int i = tid; i < rows * half; i += 256) {
    const int r = i / half, f = i % half;
    cs[r][f] = prep_cos_sin(a.pos[row0 + r], a.rope_sel, a.inv_freq, f);
  }
  // Do the 8 rows go to positions ps0 .. ps0 + 7 (ps0 a multiple of 8) of one block, nowhere else?
  int4 ent[R];
#pragma unroll
  for (int r = 0; r < R; ++r) ent[r] = (a.row_table && r < rows) ? a.row_table[row0 + r] : make_int4(-1, -1, -1, -1);
  bool run = rows == R && ent[0].x >= 0 && (ent[0].y & (R - 1)) == 0;
#pragma unroll
  for (int r = 0; r < R; ++r) run = run && ent[r].x == ent[0].x && ent[r].y == ent[0].y + r && ent[r].z < 0;
  if (tid == 0) run_ok = run;
  __syncthreads();
  run = run_ok != 0;  // the same value everywhere; through LDS so that the compiler treats it as uniform

  const int li = tid % LPH, d0 = EPL * li;
  const int n_slots = p.H + 2 * p.Hkv;
  const int slot0 = blockIdx.y * HPP;  // the workgroup's first head: queries, then keys, then values
  for (int slot = slot0 + tid / LPH; slot < n_slots; slot += n_slots) {  // at most one head per thread
    const int kind = slot < p.H ? 0 : (slot < p.H + p.Hkv ? 1 : 2);  // q, k, v
    const int h = kind == 0 ? slot : (kind == 1 ? slot - p.H : slot - p.H - p.Hkv);
    const size_t col = size_t(kind == 0 ? p.q_off + h * p.q_hs : (kind == 1 ? p.k_off : p.v_off) + h * HD) + d0;
    f32x4 xv[R][EPL / 4];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int v = 0; v < EPL / 4; ++v)
        xv[r][v] = r < rows ? __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(a.X + size_t(row0 + r) * p.x_ld + col) + v)
                            : f32x4{0, 0, 0, 0};  // read once: no reason to keep it in a cache
    float w[EPL];
#pragma unroll
    for (int i = 0; i < EPL; ++i) w[i] = kind != 2 ? (kind == 0 ? a.qn_w : a.kn_w)[d0 + i] : 1.0f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (r >= rows) break;
      const size_t row = size_t(row0 + r);
      float x[EPL];
#pragma unroll
      for (int i = 0; i < EPL; ++i) x[i] = xv[r][i / 4][i % 4];
      prep_lane<HD>(x, kind, w, cs[r], p, d0);
      using out_t = std::conditional_t<EPL == 8, u32x4, u32x2>;  // EPL storage elements
      out_t out;
#pragma unroll
      for (int i = 0; i < EPL / 2; ++i) out[i] = pack2<DT>(x[2 * i], x[2 * i + 1]);
      if (kind == 0) {
        *reinterpret_cast<out_t*>(a.Q + row * size_t(p.q_ld) + size_t(h) * HD + d0) = out;
        continue;
      }
      // Kb / Vb may be left out when the rows go to the pool anyway (a pass whose attention reads them from there)
      if (uint16_t* kv = kind == 1 ? a.Kb : a.Vb) *reinterpret_cast<out_t*>(kv + row * size_t(p.kv_ld) + size_t(h) * HD + d0) = out;
      // The folded append: the same bits into the row's pool entries (a row saved into two slots has two).
      if (kind == 2 && run) {
        *reinterpret_cast<out_t*>(&vstage[r][(slot - slot0) * HD + d0]) = out;
        continue;
      }
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int b = e ? ent[r].z : ent[r].x, ps = e ? ent[r].w : ent[r].y;
        if (b < 0) continue;
        uint16_t* hb = a.pool + p.kv_base + (size_t(b) * p.Hkv + h) * size_t(2 * p.bt * HD);
        if (kind == 1) {
          *reinterpret_cast<out_t*>(hb + size_t(ps) * HD + d0) = out;
        } else {
          uint16_t* vt = hb + vt_elem(p.bt, HD, ps, d0);
#pragma unroll
          for (int i = 0; i < EPL / 2; ++i) {
            vt[(2 * i) * kVtDim] = uint16_t(out[i] & 0xffffu);
            vt[(2 * i + 1) * kVtDim] = uint16_t(out[i] >> 16);
          }
        }
      }
    }
  }
  if (!run) return;
  __syncthreads();
  // 8 tokens of one (head, dim): 16 contiguous bytes inside one 16-token sub-block of the transposed V plane.
  for (int i = tid; i < HPP * HD; i += 256) {
    const int slot = slot0 + i / HD, d = i % HD;
    if (slot < p.H + p.Hkv || slot >= n_slots) continue;  // not a value head
    const int h = slot - p.H - p.Hkv;
    uint16_t* hb = a.pool + p.kv_base + (size_t(ent[0].x) * p.Hkv + h) * size_t(2 * p.bt * HD);
    uint16_t* dst = hb + vt_elem(p.bt, HD, ent[0].y, d);
#pragma unroll
    for (int g = 0; g < R / 8; ++g) {
      u32x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = uint32_t(vstage[8 * g + 2 * e][i]) | (uint32_t(vstage[8 * g + 2 * e + 1][i]) << 16);
      *reinterpret_cast<u32x4*>(dst + 8 * g) = v;
    }
  }
}

hipError_t launch_attn_prep(const PrepArgs& a, int n_rows, hipStream_t st) {
  const int dt = a.p.dtype, HD = a.p.head_dim;
  const int hpp = 256 / (HD / (HD > 256 ? 8 : 4)), n_slots = a.p.H + 2 * a.p.Hkv;
  const dim3 grid((n_rows + kPrepRows - 1) / kPrepRows, (n_slots + hpp - 1) / hpp), block(256);
  if (dt == ESP_F16 && HD == 128) launch_timed(attn_prep_kernel<ESP_F16, 128>, grid, block, 0, st, a, n_rows);
  else if (dt == ESP_F16 && HD == 256) launch_timed(attn_prep_kernel<ESP_F16, 256>, grid, block, 0, st, a, n_rows);
  else if (dt == ESP_BF16 && HD == 128) launch_timed(attn_prep_kernel<ESP_BF16, 128>, grid, block, 0, st, a, n_rows);
  else if (dt == ESP_BF16 && HD == 256) launch_timed(attn_prep_kernel<ESP_BF16, 256>, grid, block, 0, st, a, n_rows);
  else if (dt == ESP_F16 && HD == 512) launch_timed(attn_prep_kernel<ESP_F16, 512>, grid, block, 0, st, a, n_rows);
  else if (dt == ESP_BF16 && HD == 512) launch_timed(attn_prep_kernel<ESP_BF16, 512>, grid, block, 0, st, a, n_rows);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace esp
