// Split-K streaming attention for passes with few query rows per tree: decode
// (one row) and speculative verify (a handful of rows). Bandwidth bound: the
// job of this kernel is to keep KV pages in flight.
//
// Semantics: the reference's single-row decode kernels and its 8-row tiles on
// small trees (kernels/40_attention.metal:597-781, kernels/80_gemma.metal:157-342,
// :371-550): cached keys [k0, k1) through the block table (or ring), the batch
// keys of the tree on the `last` tile with the tree mask and the window, online
// softmax in fp32 with P rounded to the storage type before P.V, a partial
// record (O unnormalised, m, l) or the normalised (optionally gated) output.
//
// Mapping to gfx950. One workgroup = one tile x one KV head, 4 wavefronts. The
// G query heads of the KV head times the tile's rows are packed into the 16 (or
// 32) columns of the MFMA tiles ("packed rows": col = row_in_tile * G + head),
// so K and V are read from HBM once for all of them. Per 32 keys a wavefront
//   S^T[32 keys][cols]  = K[32][HD] . Q^T          v_mfma_f32_16x16x32 (A = K straight from HBM, 16-byte loads)
//   P^T = exp2(S^T - m) rounded to fp16 / bf16    (D layout of S^T == B layout of P^T: no shuffles)
//   O^T[HD][cols]      += V^T[HD][32] . P^T        v_mfma_f32_16x16x32 (A = V^T straight from HBM: the pool keeps V transposed)
// with no LDS on the way. The 4 wavefronts take 32-key units round robin and
// merge their (m, l, O) through LDS in wave order at the end. Each wavefront
// alternates between two register sets: the loads of the next unit are in flight
// while the current unit is in the matrix cores.
//
// Head dim 512 (the full-attention layers of kernels/80_gemma.metal:355-358, :561-564)
// does not fit one wavefront's registers (accumulators, Q fragments and two operand
// sets are 448). There the wavefronts work in pairs: both take the same 16-key unit,
// each loads and multiplies 256 of the 512 dims, the two partial S^T meet in LDS (one
// workgroup barrier per unit; the reference sums its per-simdgroup score partials through
// threadgroup memory the same way, 80_gemma.metal:272-282), both run the same softmax and
// each accumulates its 256 output dims. A workgroup is one such pair (128 threads, two
// workgroups per compute unit), so the barrier ties no more than the two wavefronts
// that need each other - or, for 17 to 32 packed rows, two pairs with one column tile each
// that walk the same units together, so that K and V come from memory once for both.
#include <type_traits>

#include "common.hpp"
#include "prep_math.hpp"

namespace esp {

// Merge of the partial records of one split tile group for 4 dims of one (row, query head), in part
// order (attention_combine, kernels/40_attention.metal:811-864; kernels/80_gemma.metal:568-597), then
// the normalised (optionally gated) output.
// LP lanes share one output (consecutive lanes of a wavefront, `lp` = this lane's place among them): lane lp
// merges records lp, lp + LP, .. in that order, and the LP running triples (max, sum, O) are then merged pairwise
// across the lanes. One lane (LP = 1) is the plain merge in part order.
// MAXN: the most records in flight at a time. 32 serves decode passes (a group of up to 16 parts in one round of loads);
// 8 costs a quarter of the registers, and with them four times the wavefronts per SIMD, which is what the merges of
// prefill tiles want: few parts per group, many outputs, a kernel that lives on bytes in flight.
template <int DT, int HD, int LP = 1, int MAXN = 32>
__device__ __forceinline__ void merge_records(const KArgs& a, const esp_combine& job, int r, int h, int d, int lp = 0) {
  const int kvh = h / a.G, hg = h - kvh * a.G;
  const int col = r * a.G + hg;
  const size_t stride = size_t(a.Hkv) * a.cols;  // records from one part to the next
  const size_t rec0 = (size_t(job.part0) * a.Hkv + kvh) * a.cols + col;
  // One pass, up to 32 records in flight at a time, merged in part order with a running maximum
  // (a loop that waits for each record's loads in turn is latency bound: the reference
  // measured 39 us against 11 us for the same change, 40_attention.metal:801-803).
  float M = -INFINITY, L = 0.0f;
  f32x4 o = {0, 0, 0, 0};
  // N records at a time, all their loads issued before the first use. Slots past the last record
  // repeat record s (a cache hit) with weight 0: loads under a branch would wait for one another.
  auto merge = [&]<int N>(int s, std::integral_constant<int, N>) __attribute__((always_inline)) {
    float mN[N], lN[N];
    f32x4 oN[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const bool in = s + i * LP < job.nparts;
      const size_t rec = rec0 + size_t(in ? s + i * LP : min(s, job.nparts - 1)) * stride;
      mN[i] = in ? a.parts_ml[rec * 2] : -INFINITY;
      lN[i] = a.parts_ml[rec * 2 + 1];
      oN[i] = *reinterpret_cast<const f32x4*>(a.parts_o + rec * HD + d);
    }
    float Mn = M;
#pragma unroll
    for (int i = 0; i < N; ++i) Mn = fmaxf(Mn, mN[i]);
    const float c = (M == -INFINITY) ? 0.0f : fast_exp2(M - Mn);
    L *= c;
    o *= c;
    M = Mn;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const float w = (mN[i] == -INFINITY) ? 0.0f : fast_exp2(mN[i] - M);
      L += w * lN[i];
      o += oN[i] * w;
    }
  };
  // As many records in flight as the group has, in four sizes: every round of loads is a memory latency, and a
  // finely split sequence (a single long one has dozens of parts) would otherwise pay one per 8 records.
  if constexpr (LP > 1) {
    for (int s = lp; s < job.nparts; s += 4 * LP) merge(s, std::integral_constant<int, 4>{});
    // pairwise across the LP lanes; a + b == b + a, so both lanes of a pair go on with the same triple
#pragma unroll
    for (int off = 1; off < LP; off <<= 1) {
      const float M2 = __shfl_xor(M, off), L2 = __shfl_xor(L, off);
      f32x4 o2;
#pragma unroll
      for (int e = 0; e < 4; ++e) o2[e] = __shfl_xor(o[e], off);
      const float Mn = fmaxf(M, M2);
      const float c1 = (M == -INFINITY) ? 0.0f : fast_exp2(M - Mn), c2 = (M2 == -INFINITY) ? 0.0f : fast_exp2(M2 - Mn);
      L = L * c1 + L2 * c2;
      o = o * c1 + o2 * c2;
      M = Mn;
    }
    if (lp != 0) return;
  } else if (job.nparts <= 2) {  // the split of a prefill tile: two records, nothing to repeat
    merge(0, std::integral_constant<int, 2>{});
  } else if constexpr (MAXN <= 8) {
    if (job.nparts <= 4) merge(0, std::integral_constant<int, 4>{});
    else for (int s = 0; s < job.nparts; s += 8) merge(s, std::integral_constant<int, 8>{});
  } else if (job.nparts <= 8) {
    merge(0, std::integral_constant<int, 8>{});
  } else if (job.nparts <= 16) {
    merge(0, std::integral_constant<int, 16>{});
  } else {
    for (int s = 0; s < job.nparts; s += 32) merge(s, std::integral_constant<int, 32>{});
  }
  const int row = job.r0 + r;
  const float inv = L > 0.0f ? 1.0f / L : 0.0f;
  o *= inv;
  if (a.gate) {
    const float* g = a.gate + size_t(row) * a.gate_ld + size_t(h) * a.gate_hs + a.gate_off + d * a.gate_ds;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = o[e] / (1.0f + __expf(-g[e * a.gate_ds]));
  }
  u32x2 out = {pack2<DT>(o[0], o[1]), pack2<DT>(o[2], o[3])};
  *reinterpret_cast<u32x2*>(a.O + size_t(row) * a.q_ld + size_t(h) * HD + d) = out;
}

template <int HD, int SBU>
struct Unit {  // operands of one unit of SBU 16-key sub-blocks
  u32x4 k[SBU][HD / 32];  // [sub-block][32-dim group]: key = lane % 16, dims 32 kk + 8 (lane / 16) ..
  u32x2 v[SBU][HD / 16];  // [sub-block][16-dim group]: dim = 16 mt + lane % 16, keys 4 (lane / 16) ..
};

// SBU: 16-key sub-blocks per unit (2: P.V on 16x16x32 tiles; 1: on 16x16x16 tiles, for
// head dims whose operands would not fit two register sets otherwise).
// BT: tokens per block when known at compile time (0: read from the arguments).
// FUSED: the pass's rows come as the fp32 fused projection and the workgroup applies attn_prep to what it
// needs of them itself (its tile's query heads; on the `last` tile the rows' key and value head of this KV
// head, which it also appends to the pool): no prep dispatch in front, no Q / Kb / Vb round trip through
// memory. For passes whose trees have at most rows_per_tile <= 4 rows (decode, short verify trees).
template <int DT, int HD, int NC, int SBU, int BT, int OCC, int FUSED>
__global__ __launch_bounds__(HD >= 512 ? 128 * NC : 256, OCC) void attn_stream_kernel(const KArgs a, const PrepArgs pa) {
  constexpr bool PAIR = HD >= 512;      // two wavefronts per unit, HW dims each
  constexpr int HW = PAIR ? HD / 2 : HD;
  constexpr int NS = PAIR ? 1 : 4;       // unit streams of the workgroup
  constexpr int NW = PAIR ? 2 * NC : 4;  // wavefronts of the workgroup
  // Column tiles a wavefront holds. Paired wavefronts have registers for one; a second column tile (32 packed rows:
  // a 4-row verify tree at 8 query heads per KV head) is a second pair of the same workgroup that walks the same
  // units in step with the first - one barrier per unit ties all four wavefronts - so that its requests for the
  // unit's K and V meet the first pair's in L2 and the pool is read from memory once.
  constexpr int NCW = PAIR ? 1 : NC;
  static_assert(!PAIR || SBU == 1, "paired wavefronts: 16-key units");
  static_assert(!PAIR || !FUSED, "the fused prologue is built for one wavefront per head");
  constexpr int kFusedRows = 4;  // most rows of a tile on the fused path
  constexpr int KK = HW / 32, MT = HW / 16, LDO = HD + 4, UK = 16 * SBU, USH = SBU == 2 ? 5 : 4;
  extern __shared__ float smem[];  // [NS][NC * 16 cols][LDO] O, then [NS][NC * 16][2] m, l, then (PAIR) [2][NW][64] partial S^T

  const int bt = BT ? BT : a.bt;
  const int kvh = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int strm = PAIR ? 0 : wave;          // which of the NS unit streams
  const int dw = PAIR ? (wave & 1) * HW : 0; // first dim of this wavefront's share of the head
  const int cbase = PAIR ? 16 * (wave >> 1) : 0;  // first packed row (column) of this wavefront's column tiles
  const int c16 = lane & 15, q4 = lane >> 4;
  esp_tile tile = a.tiles[blockIdx.y];
  const esp_tree tree = a.trees[tile.tree];
  if (tile.k1 == INT32_MAX) tile.k1 = tree.P;  // open-ended range: up to the tree's cached length as it is now
  // The planner may carry the tree's block-list offset in the tile (pad = table + 1): one
  // dependent load less before the first KV page can be requested.
  const int table = tile.pad > 0 ? tile.pad - 1 : tree.table;
  const int end = tree.base + tree.M;
  const int rows_live = min(a.R, end - tile.r0);
  const int rr0 = tile.r0 - tree.base;

  // ---- fused prologue: attn_prep of this workgroup's heads into LDS (the area the final merge uses later),
  // with the arithmetic and the lane arrangement of the prep kernel (prep_math.hpp), so the bits are its bits.
  uint16_t* q_lds = reinterpret_cast<uint16_t*>(smem);   // [NC * 16 packed rows][HD]
  uint16_t* k_lds = q_lds + NC * 16 * HD;                  // [kFusedRows][HD] this KV head's key rows
  uint16_t* v_lds = k_lds + kFusedRows * HD;               // [kFusedRows][HD] and value rows
  if constexpr (FUSED) {
    constexpr int EPL = prep_epl(HD), LPH = HD / EPL, HPP = 256 / LPH;
    float2* cs = reinterpret_cast<float2*>(v_lds + kFusedRows * HD);  // [kFusedRows][HD / 2]
    const esp_prep_params& pp = pa.p;
    const int half = pp.rope_dims / 2;
    for (int i = threadIdx.x; i < rows_live * half; i += 256) {
      const int r = i / half, f = i - r * half;
      cs[r * (HD / 2) + f] = prep_cos_sin(pa.pos[tile.r0 + r], pa.rope_sel, pa.inv_freq, f);
    }
    __syncthreads();
    const int n_q = rows_live * a.G, n_items = n_q + (tile.last ? 2 * rows_live : 0);
    const int li = threadIdx.x % LPH, d0 = EPL * li;
    for (int it = threadIdx.x / LPH; it < n_items; it += HPP) {
      const int kind = it < n_q ? 0 : 1 + (it - n_q) / rows_live;
      const int m = it < n_q ? it / a.G : (it - n_q) % rows_live;
      const int h = it < n_q ? kvh * a.G + (it - m * a.G) : kvh;
      const size_t row = size_t(tile.r0 + m);
      const size_t col = size_t(kind == 0 ? pp.q_off + h * pp.q_hs : (kind == 1 ? pp.k_off : pp.v_off) + h * HD) + d0;
      float x[EPL], w[EPL];
#pragma unroll
      for (int v = 0; v < EPL / 4; ++v) {
        const f32x4 xv = *(reinterpret_cast<const f32x4*>(pa.X + row * pp.x_ld + col) + v);
#pragma unroll
        for (int i = 0; i < 4; ++i) x[4 * v + i] = xv[i];
      }
#pragma unroll
      for (int i = 0; i < EPL; ++i) w[i] = kind != 2 ? (kind == 0 ? pa.qn_w : pa.kn_w)[d0 + i] : 1.0f;
      prep_lane<HD>(x, kind, w, cs + m * (HD / 2), pp, d0);
      using out_t = std::conditional_t<EPL == 8, u32x4, u32x2>;
      out_t out;
#pragma unroll
      for (int i = 0; i < EPL / 2; ++i) out[i] = pack2<DT>(x[2 * i], x[2 * i + 1]);
      uint16_t* dst = kind == 0 ? q_lds + it * HD : (kind == 1 ? k_lds : v_lds) + m * HD;
      *reinterpret_cast<out_t*>(dst + d0) = out;
      if (kind == 0 || !pa.row_table) continue;
      // the folded append: the row's key and value of this KV head into its pool entries
      const int4 ent = pa.row_table[row];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int b = e ? ent.z : ent.x, ps = e ? ent.w : ent.y;
        if (b < 0) continue;
        uint16_t* hb = pa.pool + pp.kv_base + (size_t(b) * pp.Hkv + h) * size_t(2 * pp.bt * HD);
        if (kind == 1) {
          *reinterpret_cast<out_t*>(hb + size_t(ps) * HD + d0) = out;
        } else {
          uint16_t* vt = hb + vt_elem(pp.bt, HD, ps, d0);
#pragma unroll
          for (int i = 0; i < EPL / 2; ++i) {
            vt[(2 * i) * kVtDim] = uint16_t(out[i] & 0xffffu);
            vt[(2 * i + 1) * kVtDim] = uint16_t(out[i] >> 16);
          }
        }
      }
    }
    __syncthreads();
  }

  // ---- this lane's packed rows: Q fragments, position, descriptor
  u32x4 qf[NCW][KK];
  int rr[NCW], qpos[NCW];
  int4 dsc[NCW];
  bool ok[NCW];
#pragma unroll
  for (int c = 0; c < NCW; ++c) {
    const int col = cbase + 16 * c + c16;
    const int m = col / a.G, hg = col - m * a.G;
    ok[c] = col < a.cols && m < rows_live;
    rr[c] = rr0 + m;
    const int row = ok[c] ? tile.r0 + m : tile.r0;
    qpos[c] = (a.window > 0) ? a.pos[row].x : 0;
    dsc[c] = a.desc ? a.desc[row] : make_int4(0, 0, 0, 0);
    const uint16_t* qp = FUSED ? q_lds + (ok[c] ? col : 0) * HD + dw + 8 * q4
                               : a.Q + size_t(row) * a.q_ld + size_t(kvh * a.G + (ok[c] ? hg : 0)) * HD + dw + 8 * q4;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
      qf[c][kk] = ok[c] ? *reinterpret_cast<const u32x4*>(qp + 32 * kk) : u32x4{0, 0, 0, 0};
  }

  // ---- the cached range in units of UK keys. Interior units lie wholly inside
  // [k0, k1) and, on a windowed layer, wholly inside the window of every packed row:
  // they need no masks and go through the pipelined loop. The partial units at the
  // ends of the range, the units the window's lower edge cuts, and the tree's batch
  // rows take the general path.
  const int cp0 = tile.k0 >> USH;
  const bool has_cached = tile.k1 > tile.k0;
  const int ulast = has_cached ? (tile.k1 - 1) >> USH : cp0 - 1;
  const int n_cached = ulast - cp0 + 1;
  int ui0, ui1;  // interior units [ui0, ui1); general ones [cp0, ui0) and [ui1, ulast]
  if (!has_cached) {
    ui0 = ui1 = cp0;
  } else {
    int lo_key = tile.k0;  // first key every row sees
    if (a.window > 0) {
      int qm = INT32_MIN;
      if constexpr (PAIR && NC > 1) {
        // The pairs of the workgroup hold different rows but pass the same barriers: the range every row sees
        // is taken over all rows of the tile, by every wavefront alike.
        for (int m = lane; m < rows_live; m += 64) qm = max(qm, a.pos[tile.r0 + m].x);
#pragma unroll
        for (int o = 32; o >= 16; o >>= 1) qm = max(qm, __shfl_xor(qm, o));
      } else {
#pragma unroll
        for (int c = 0; c < NCW; ++c)
          if (ok[c]) qm = max(qm, qpos[c]);
      }
#pragma unroll
      for (int o = 8; o >= 1; o >>= 1) qm = max(qm, __shfl_xor(qm, o));
      qm = __builtin_amdgcn_readfirstlane(qm);  // the 16 columns repeat in every quarter of the wavefront
      lo_key = max(lo_key, qm - a.window + 1);
    }
    ui0 = min((lo_key + UK - 1) >> USH, ulast + 1);
    ui1 = max(ui0, tile.k1 >> USH);  // units wholly below k1
  }
  const int n_lo = ui0 - cp0, n_edge = n_cached - (ui1 - ui0);
  int k_last = -1, bp0 = 0, n_batch = 0;  // batch range: set once the cached range has been streamed
  f32x4 acc[NCW][MT];
  float m_run[NCW], l_run[NCW];  // running max in log2 units of the scaled score; this lane's share of the sum
#pragma unroll
  for (int c = 0; c < NCW; ++c) {
    m_run[c] = -INFINITY;
    l_run[c] = 0.0f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[c][mt] = f32x4{0, 0, 0, 0};
  }

  // K rows and V^T rows of cached unit u (absolute unit index) straight from the pool.
  // A sub-block past the range's last page re-reads that page.
  const int last_js = (max(tile.k1, tile.k0 + 1) - 1) & ~15;
  const int lane_k = (c16 * HD + dw + 8 * q4), lane_v = (dw + c16) * kVtDim + 4 * q4;
  auto load_cached = [&](int u, Unit<HW, SBU>& U) {
    const int j0 = u << USH;
#pragma unroll
    for (int sb = 0; sb < SBU; ++sb) {
      const int js = min(j0 + 16 * sb, last_js);  // first key of the sub-block
      const int b = block_of(a, table, js);
      const int t0 = js % bt;
      const uint16_t* hb = a.pool + head_base(a, HD, b, kvh);
      const uint16_t* kp = hb + t0 * HD + lane_k;
      const uint16_t* vp = hb + vt_elem(bt, HD, t0, 0) + lane_v;  // t0 is a multiple of 16: the sub-block's start
      constexpr int ks = 32, vs = 16 * kVtDim;
      // Every cached byte is read once per pass: non-temporal loads keep the stream from displacing
      // what the caches could still serve (measured: 184 -> 164 us on 1 GB of keys at head dim 256).
      // (Two pairs that walk the same units want the opposite: the first pair's lines must still be in L2 when the
      // second pair asks for them, so those loads are ordinary ones.)
      constexpr bool kOnce = !(PAIR && NC > 1);
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
        U.k[sb][kk] = kOnce ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kp + ks * kk)) : *reinterpret_cast<const u32x4*>(kp + ks * kk);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        U.v[sb][mt] = kOnce ? __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(vp + vs * mt)) : *reinterpret_cast<const u32x2*>(vp + vs * mt);
    }
  };

  // Batch units: rows of the pass (row major Kb / Vb); V gathered element by element. Without Kb / Vb the rows
  // are read from the pool: they were appended before the attention (esp_attn_prep with a row table, or
  // esp_kv_save), row j of a tree at position P + j of the tree's own block list.
  const bool in_pool = !FUSED && a.Kb == nullptr;
  auto load_batch = [&](int u, Unit<HW, SBU>& U) {
    const int j0 = u << USH;
#pragma unroll
    for (int sb = 0; sb < SBU; ++sb) {
      const int js = j0 + 16 * sb;
      const int jk = js + c16;
      const bool k_ok = jk <= k_last;
      // fused: a tree's rows are its one tile's rows, prepared into LDS by the prologue
      const uint16_t* kp;
      if (FUSED) {
        kp = k_lds + (k_ok ? jk : 0) * HD + dw + 8 * q4;
      } else if (in_pool) {
        const int q = tree.P + (k_ok ? jk : 0);
        kp = a.pool + head_base(a, HD, block_of(a, table, q), kvh) + (q % bt) * HD + dw + 8 * q4;
      } else {
        kp = a.Kb + size_t(tree.base + (k_ok ? jk : 0)) * a.kv_ld + size_t(kvh) * HD + dw + 8 * q4;
      }
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
        U.k[sb][kk] = k_ok ? *reinterpret_cast<const u32x4*>(kp + 32 * kk) : u32x4{0, 0, 0, 0};
      const int jv = js + 4 * q4;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) U.v[sb][mt] = u32x2{0, 0};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (jv + i > k_last) continue;
        const uint16_t* vp;
        int vs = 16;  // elements from dim d to dim d + 16
        if (FUSED) {
          vp = v_lds + (jv + i) * HD + dw + c16;
        } else if (in_pool) {
          const int q = tree.P + jv + i;
          vp = a.pool + head_base(a, HD, block_of(a, table, q), kvh) + vt_elem(bt, HD, q % bt, dw + c16);
          vs = 16 * kVtDim;
        } else {
          vp = a.Vb + size_t(tree.base + jv + i) * a.kv_ld + size_t(kvh) * HD + dw + c16;
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const uint32_t e = uint32_t(vp[vs * mt]) << (16 * (i & 1));
          if (i < 2) U.v[sb][mt].x |= e;
          else U.v[sb][mt].y |= e;
        }
      }
    }
  };

  // S^T = K . Q^T of one unit. Paired wavefronts: each has the sum over its HW dims; the halves are
  // exchanged through LDS slot (unit count & 1) and added in the same order on both sides, so the
  // two wavefronts of a pair go on with identical S^T. One workgroup barrier per unit: every
  // wavefront of the workgroup passes through here (or through the bare barriers after the loops)
  // the same number of times. A slot is rewritten two units later, behind the barrier of the unit
  // in between, which the partner reaches only after it has read the slot.
  int n_done = 0;  // units this wavefront has computed
  f32x4* xch = reinterpret_cast<f32x4*>(smem + NS * NC * 16 * (LDO + 2));
  auto scores = [&](const Unit<HW, SBU>& U, f32x4 (&s)[NCW][SBU]) {
#pragma unroll
    for (int c = 0; c < NCW; ++c)
#pragma unroll
      for (int sb = 0; sb < SBU; ++sb) {
        s[c][sb] = f32x4{0, 0, 0, 0};
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) s[c][sb] = mfma16x32<DT>(U.k[sb][kk], qf[c][kk], s[c][sb]);
      }
    if constexpr (PAIR) {
      f32x4* slot = xch + (n_done & 1) * (NW * 64);
      slot[wave * 64 + lane] = s[0][0];
      __syncthreads();
      const f32x4 other = slot[(wave ^ 1) * 64 + lane];
      s[0][0] = (wave & 1) ? other + s[0][0] : s[0][0] + other;
      ++n_done;
    }
  };
  // Online softmax over a unit's scores x (log2 units, -inf where masked), then O^T += V^T . P^T.
  auto softmax_pv = [&](const Unit<HW, SBU>& U, f32x4 (&x)[NCW][SBU], const float (&mx_in)[NCW]) {
    bool any_change = false;
    u32x2 pb[NCW][SBU];
    float corr[NCW];
#pragma unroll
    for (int c = 0; c < NCW; ++c) {
      float mx = mx_in[c];
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run[c], mx);
      const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
      corr[c] = fast_exp2(m_run[c] - m_safe);  // -inf -> 0: nothing accumulated yet
      any_change = any_change || (m_new > m_run[c]);
      m_run[c] = m_new;
      float ps = 0.0f;
#pragma unroll
      for (int sb = 0; sb < SBU; ++sb) {
        float p[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          p[e] = fast_exp2(x[c][sb][e] - m_safe);
          ps += p[e];
        }
        pb[c][sb] = u32x2{pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3])};
      }
      l_run[c] = l_run[c] * corr[c] + ps;
    }
    if (__any(any_change)) {
#pragma unroll
      for (int c = 0; c < NCW; ++c)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[c][mt] *= corr[c];
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      if constexpr (SBU == 2) {
        const u32x4 va = {U.v[0][mt].x, U.v[0][mt].y, U.v[1][mt].x, U.v[1][mt].y};
#pragma unroll
        for (int c = 0; c < NCW; ++c)
          acc[c][mt] = mfma16x32<DT>(va, u32x4{pb[c][0].x, pb[c][0].y, pb[c][1].x, pb[c][1].y}, acc[c][mt]);
      } else {
#pragma unroll
        for (int c = 0; c < NCW; ++c) acc[c][mt] = mfma16x16<DT>(U.v[0][mt], pb[c][0], acc[c][mt]);
      }
    }
  };

  // Interior unit: every key visible to every row.
  auto compute_interior = [&](const Unit<HW, SBU>& U) {
    f32x4 s[NCW][SBU];
    scores(U, s);
    float mx[NCW];
#pragma unroll
    for (int c = 0; c < NCW; ++c) {
      mx[c] = -INFINITY;
#pragma unroll
      for (int sb = 0; sb < SBU; ++sb)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s[c][sb][e] *= a.scale_log2;
          mx[c] = fmaxf(mx[c], s[c][sb][e]);
        }
    }
    softmax_pv(U, s, mx);
  };

  // General unit: per-key visibility. BATCH: the keys are the tree's batch rows j0 .. (tree
  // mask and window), else cached keys j0 .. (range ends and window).
  auto compute_general = [&]<bool BATCH>(int j0, Unit<HW, SBU>& U) {
    if constexpr (!BATCH) {
      // Cached keys outside [k0, k1) may be memory never written: their V must not reach the products.
#pragma unroll
      for (int sb = 0; sb < SBU; ++sb) {
        const int jv = j0 + 16 * sb + 4 * q4;
        const uint32_t m0 = (jv >= tile.k0 && jv < tile.k1) ? 0xffffu : 0u;
        const uint32_t m1 = (jv + 1 >= tile.k0 && jv + 1 < tile.k1) ? 0xffff0000u : 0u;
        const uint32_t m2 = (jv + 2 >= tile.k0 && jv + 2 < tile.k1) ? 0xffffu : 0u;
        const uint32_t m3 = (jv + 3 >= tile.k0 && jv + 3 < tile.k1) ? 0xffff0000u : 0u;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          U.v[sb][mt].x &= (m0 | m1);
          U.v[sb][mt].y &= (m2 | m3);
        }
      }
    }
    f32x4 s[NCW][SBU];
    scores(U, s);
    // The first readers of s sit behind the branches of the visibility rules below.
#pragma unroll
    for (int c = 0; c < NCW; ++c)
#pragma unroll
      for (int sb = 0; sb < SBU; ++sb) mfma_settle(s[c][sb]);
    int kpos[SBU][4];
    if (BATCH && a.window > 0) {
#pragma unroll
      for (int sb = 0; sb < SBU; ++sb)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int j = j0 + 16 * sb + 4 * q4 + e;
          kpos[sb][e] = a.pos[tree.base + min(j, tree.M - 1)].x;
        }
    }
    float mx[NCW];
#pragma unroll
    for (int c = 0; c < NCW; ++c) {
      mx[c] = -INFINITY;
#pragma unroll
      for (int sb = 0; sb < SBU; ++sb)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int j = j0 + 16 * sb + 4 * q4 + e;
          bool vis;
          if constexpr (!BATCH) {
            vis = j >= tile.k0 && j < tile.k1;
            if (a.window > 0) vis = vis && (qpos[c] - j < a.window);
          } else {
            vis = j <= k_last && ((j < dsc[c].z) || (j >= dsc[c].x && (j <= rr[c] || (a.bidi && j < dsc[c].w))));
            if (a.window > 0) vis = vis && (qpos[c] - kpos[sb][e] < a.window);
          }
          const float x = vis ? s[c][sb][e] * a.scale_log2 : -INFINITY;
          s[c][sb][e] = x;
          mx[c] = fmaxf(mx[c], x);
        }
    }
    softmax_pv(U, s, mx);
  };

  {
    Unit<HW, SBU> U[2];
    // ---- interior units through two register sets: while one unit is in the matrix cores,
    // the loads of the next are in flight. Stream w takes interior units w, w + NS, ...:
    // n_mine of them.
    const int n_int = ui1 - ui0;
    const int n_mine = n_int > strm ? (n_int - strm + NS - 1) / NS : 0;
    if (n_mine > 0) {
      // Two register sets, the next unit requested before the current one is consumed, and no request
      // without a unit behind it: at the top of the loop set 0 holds (or awaits) unit i. (A deeper
      // ring that refilled every set it consumed - with dummy loads once the units ran out, to keep
      // the count of loads in flight fixed - was 2 to 10 % slower on every shape, short ranges most.)
      const int u0 = ui0 + strm;
      load_cached(u0, U[0]);
      int i = 0;
      for (; i + 2 < n_mine; i += 2) {
        load_cached(u0 + NS * (i + 1), U[1]);
        compute_interior(U[0]);
        load_cached(u0 + NS * (i + 2), U[0]);
        compute_interior(U[1]);
      }
      if (i + 2 == n_mine) {
        load_cached(u0 + NS * (i + 1), U[1]);
        compute_interior(U[0]);
        compute_interior(U[1]);
      } else {
        compute_interior(U[0]);
      }
    }
    // ---- then the units that need masks: partial or windowed cached units, batch rows.
    // They continue the round robin after the interior units.
    if (tile.last) {
      // Last batch key any row of the tile sees: its last row, a root it sees whole
      // (anc_len), the end of its image (bidi).
      int kl = -1;
      if constexpr (PAIR && NC > 1) {  // over all rows of the tile: every pair scans the same batch units
        for (int m = lane; m < rows_live; m += 64) {
          const int4 dm = a.desc ? a.desc[tile.r0 + m] : make_int4(0, 0, 0, 0);
          kl = max(kl, max(rr0 + m, max(dm.z - 1, a.bidi ? dm.w - 1 : -1)));
        }
      } else {
#pragma unroll
        for (int c = 0; c < NCW; ++c)
          if (ok[c]) kl = max(kl, max(rr[c], max(dsc[c].z - 1, a.bidi ? dsc[c].w - 1 : -1)));
      }
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) kl = max(kl, __shfl_xor(kl, o));
      // fused: the batch keys are the tile's own rows in LDS, never more than the tile holds
      k_last = __builtin_amdgcn_readfirstlane(min(kl, (FUSED ? min(tree.M, rows_live) : tree.M) - 1));
      if (tile.last >= 2) k_last = min(k_last, tile.last - 2);  // a part whose batch range ends at row last - 2 of the tree
      bp0 = tile.b0 >> USH;
      n_batch = max(0, ((k_last + UK) >> USH) - bp0);
    }
    const int n_slow = n_edge + n_batch;
    for (int i = (strm + NS - n_int % NS) % NS; i < n_slow; i += NS) {
      if (i < n_edge) {
        const int u = i < n_lo ? cp0 + i : ui1 + (i - n_lo);
        load_cached(u, U[0]);
        compute_general.template operator()<false>(u << USH, U[0]);
      } else {
        const int u = bp0 + (i - n_edge);
        load_batch(u, U[0]);
        compute_general.template operator()<true>(u << USH, U[0]);
      }
    }
    if constexpr (PAIR && NS > 1) {  // another pair may have one unit more: its barrier needs this wavefront too
      const int most = (n_int + n_slow + NS - 1) / NS;
      for (int i = n_done; i < most; ++i) __syncthreads();
    }
  }

  // ---- merge the NS streams in order (paired wavefronts hold the same m and l and one half of the dims each).
  // Every wavefront leaves its (m, l) and its accumulators as they are; behind one barrier each thread reads, for
  // the 4 dims of a packed row it finishes, the NS references, sums and vectors in one round of LDS reads and
  // weighs them itself. (Accumulators scaled by the writer, which first had to read every stream's reference
  // behind a barrier of its own, cost a second barrier and two more dependent LDS round trips at the end of
  // every workgroup's life.)
  float* o_sh = smem;                          // [NS][NC * 16][LDO]
  float* ml_sh = smem + NS * NC * 16 * LDO;    // [NS][NC * 16][2]
  if constexpr (FUSED) __syncthreads();        // the prepared rows lie where the accumulators go: every wavefront is done with them
#pragma unroll
  for (int c = 0; c < NCW; ++c) {
    const int col = cbase + 16 * c + c16;
    float l = l_run[c];
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    l_run[c] = l;
    if (q4 == 0) {
      ml_sh[(strm * NC * 16 + col) * 2] = m_run[c];
      ml_sh[(strm * NC * 16 + col) * 2 + 1] = l;
    }
    float* dst = o_sh + size_t(strm * NC * 16 + col) * LDO + dw + 4 * q4;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *reinterpret_cast<f32x4*>(dst + 16 * mt) = acc[c][mt];
  }
  __syncthreads();
  // Each thread finishes 4 dims of one packed row at a time.
  const int cols_live = min(a.cols, rows_live * a.G);  // packed rows m G + head, m < rows_live
  for (int i = threadIdx.x; i < NC * 16 * (HD / 4); i += NW * 64) {
    const int col = i / (HD / 4), d = (i % (HD / 4)) * 4;
    if (col >= cols_live) continue;  // (no division by G where a partial record is all that is written)
    float mw[NS], lw[NS];
    f32x4 ow[NS];
#pragma unroll
    for (int w = 0; w < NS; ++w) {
      mw[w] = ml_sh[(w * NC * 16 + col) * 2];
      lw[w] = ml_sh[(w * NC * 16 + col) * 2 + 1];
      ow[w] = *reinterpret_cast<const f32x4*>(o_sh + size_t(w * NC * 16 + col) * LDO + d);
    }
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NS; ++w) M = fmaxf(M, mw[w]);
    float L = 0.0f, fw[NS];
#pragma unroll
    for (int w = 0; w < NS; ++w) {
      fw[w] = (mw[w] == -INFINITY) ? 0.0f : fast_exp2(mw[w] - M);
      L += fw[w] * lw[w];
    }
    f32x4 o = {0, 0, 0, 0};
    {
#pragma clang fp contract(off)  // product, then sum: the bits of a writer that scaled and a reader that added
#pragma unroll
      for (int w = 0; w < NS; ++w) {
        const f32x4 t = ow[w] * fw[w];
        o += t;
      }
    }
    if (tile.part >= 0) {
      const size_t rec = (size_t(tile.part) * a.Hkv + kvh) * a.cols + col;
      *reinterpret_cast<f32x4*>(a.parts_o + rec * HD + d) = o;
      if (d == 0) {
        a.parts_ml[rec * 2] = M;
        a.parts_ml[rec * 2 + 1] = L;
      }
    } else {
      const int m = col / a.G, hg = col - m * a.G;
      const int row = tile.r0 + m, h = kvh * a.G + hg;
      const float inv = L > 0.0f ? 1.0f / L : 0.0f;
      o *= inv;
      if (a.gate) {
        const float* g = a.gate + size_t(row) * a.gate_ld + size_t(h) * a.gate_hs + a.gate_off + d * a.gate_ds;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = o[e] / (1.0f + __expf(-g[e * a.gate_ds]));
      }
      u32x2 out = {pack2<DT>(o[0], o[1]), pack2<DT>(o[2], o[3])};
      *reinterpret_cast<u32x2*>(a.O + size_t(row) * a.q_ld + size_t(h) * HD + d) = out;
    }
  }
}

// The merge as its own dispatch: LP threads per (job, row, head, 4 dims). One thread each is what a pass of many
// tile groups wants; a pass of few groups with many parts each (one long sequence decoded alone: 1024 outputs of 65
// records) would leave all but a handful of compute units idle, so there 8 lanes share an output.
template <int DT, int HD, int LP, int MAXN = 32>
__global__ __launch_bounds__(256) void attn_combine_kernel(const KArgs a, const esp_combine* jobs, int n_jobs) {
  const int per_job = a.R * a.H * (HD / 4);
  const long tid_g = long(blockIdx.x) * 256 + threadIdx.x;
  const long gid = tid_g / LP;
  const int lp = int(tid_g % LP);
  if (gid >= long(n_jobs) * per_job) return;
  const int ji = int(gid / per_job);
  int rem = int(gid % per_job);
  const int r = rem / (a.H * (HD / 4));
  rem -= r * a.H * (HD / 4);
  const int h = rem / (HD / 4), d = (rem % (HD / 4)) * 4;
  const esp_combine job = jobs[ji];
  if (r >= job.rows) return;
  merge_records<DT, HD, LP, MAXN>(a, job, r, h, d, lp);
}

size_t stream_smem_bytes(int HD, int NC) {
  if (HD >= 512) return size_t(NC * 16) * (HD + 4 + 2) * sizeof(float) + 2 * (2 * NC) * 64 * 16;  // one stream + the partial S^T slots of every wavefront
  return size_t(4 * NC * 16) * (HD + 4 + 2) * sizeof(float);
}

// Resident workgroups per CU of each variant: the single-column-tile head_dim-128 kernel
// fits two; the wider ones need more than 256 VGPRs and run one.
constexpr int stream_occ(int HD, int NC) { return (HD == 128 && NC == 1) ? 2 : 1; }  // wavefronts per SIMD
// Head dim 512: workgroups of one wavefront pair per column tile, one wavefront per SIMD: two pairs fill a compute unit.
int stream_workgroups_per_cu(int HD, int NC) { return HD >= 512 ? 2 / NC : stream_occ(HD, NC); }

template <int DT, int HD, int NC, int FUSED>
static hipError_t launch_stream_t(const KArgs& a, const PrepArgs& pa, int n_tiles, hipStream_t st) {
  constexpr int SBU = HD == 128 ? 2 : 1;  // 256 and 512 (256 dims per wavefront): 16-key units
  constexpr int OCC = stream_occ(HD, NC);
  const size_t smem = stream_smem_bytes(HD, NC);
  constexpr auto k16 = attn_stream_kernel<DT, HD, NC, SBU, 16, OCC, FUSED>;
  constexpr auto kbt = attn_stream_kernel<DT, HD, NC, SBU, 0, OCC, FUSED>;
  const auto k = a.bt == 16 ? k16 : kbt;
  const hipError_t e = a.bt == 16 ? allow_dynamic_lds<k16>(smem) : allow_dynamic_lds<kbt>(smem);
  if (e != hipSuccess) return e;
  launch_timed(k, dim3(a.Hkv, n_tiles), dim3(HD >= 512 ? 128 * NC : 256), smem, st, a, pa);
  return hipGetLastError();
}

template <int DT, int HD, int NC>
static hipError_t stream_attributes_t() {
  constexpr int SBU = HD == 128 ? 2 : 1;
  constexpr int OCC = stream_occ(HD, NC);
  const size_t smem = stream_smem_bytes(HD, NC);
  hipError_t e = allow_dynamic_lds<attn_stream_kernel<DT, HD, NC, SBU, 16, OCC, 0>>(smem);
  if (e == hipSuccess) e = allow_dynamic_lds<attn_stream_kernel<DT, HD, NC, SBU, 0, OCC, 0>>(smem);
  if constexpr (HD < 512) {
    if (e == hipSuccess) e = allow_dynamic_lds<attn_stream_kernel<DT, HD, NC, SBU, 16, OCC, 1>>(smem);
    if (e == hipSuccess) e = allow_dynamic_lds<attn_stream_kernel<DT, HD, NC, SBU, 0, OCC, 1>>(smem);
  }
  return e;
}

// The dynamic LDS limit of every variant on the current device, ahead of the first launch (which may
// happen while a stream is being captured, where a function attribute cannot be set).
hipError_t stream_init_attributes() {
  hipError_t e = stream_attributes_t<ESP_F16, 128, 1>();
  if (e == hipSuccess) e = stream_attributes_t<ESP_F16, 128, 2>();
  if (e == hipSuccess) e = stream_attributes_t<ESP_F16, 256, 1>();
  if (e == hipSuccess) e = stream_attributes_t<ESP_F16, 512, 1>();
  if (e == hipSuccess) e = stream_attributes_t<ESP_F16, 512, 2>();
  if (e == hipSuccess) e = stream_attributes_t<ESP_BF16, 128, 1>();
  if (e == hipSuccess) e = stream_attributes_t<ESP_BF16, 128, 2>();
  if (e == hipSuccess) e = stream_attributes_t<ESP_BF16, 256, 1>();
  if (e == hipSuccess) e = stream_attributes_t<ESP_BF16, 512, 1>();
  if (e == hipSuccess) e = stream_attributes_t<ESP_BF16, 512, 2>();
  return e;
}

// dt, HD, NC are validated by the caller: (HD, NC) in {(128, 1), (128, 2), (256, 1), (512, 1), (512, 2)}; with a prep
// argument block (the fused prologue) head dim 512 is not served.
hipError_t launch_stream(int dt, int HD, int NC, const KArgs& a, const PrepArgs* pa, int n_tiles, hipStream_t st) {
  static const PrepArgs none{};
#define ESP_STREAM_CASE(D, H_, N_)                                                                   \
  if (dt == D && HD == H_ && NC == N_)                                                               \
    return pa ? launch_stream_t<D, H_, N_, 1>(a, *pa, n_tiles, st) : launch_stream_t<D, H_, N_, 0>(a, none, n_tiles, st);
  ESP_STREAM_CASE(ESP_F16, 128, 1)
  ESP_STREAM_CASE(ESP_F16, 128, 2)
  ESP_STREAM_CASE(ESP_F16, 256, 1)
  ESP_STREAM_CASE(ESP_BF16, 128, 1)
  ESP_STREAM_CASE(ESP_BF16, 128, 2)
  ESP_STREAM_CASE(ESP_BF16, 256, 1)
#undef ESP_STREAM_CASE
  if (HD == 512 && !pa) {
    if (dt == ESP_F16 && NC == 1) return launch_stream_t<ESP_F16, 512, 1, 0>(a, none, n_tiles, st);
    if (dt == ESP_BF16 && NC == 1) return launch_stream_t<ESP_BF16, 512, 1, 0>(a, none, n_tiles, st);
    if (dt == ESP_F16 && NC == 2) return launch_stream_t<ESP_F16, 512, 2, 0>(a, none, n_tiles, st);
    if (dt == ESP_BF16 && NC == 2) return launch_stream_t<ESP_BF16, 512, 2, 0>(a, none, n_tiles, st);
  }
  return hipErrorInvalidValue;
}

template <int DT, int HD>
static void launch_combine_t(const KArgs& a, const esp_combine* jobs, int n_jobs, int n_parts, hipStream_t st) {
  const long n = long(n_jobs) * a.R * a.H * (HD / 4);
  // more than 8 records per group on average and few outputs: share each output among 8 lanes
  if (n_parts > 8 * n_jobs && n * 8 <= (1L << 22)) {
    hipLaunchKernelGGL((attn_combine_kernel<DT, HD, 8>), dim3((unsigned)((n * 8 + 255) / 256)), dim3(256), 0, st, a, jobs, n_jobs);
  } else if (a.R > 32) {  // tiles of the tiled kernels: many outputs, few parts each
    hipLaunchKernelGGL((attn_combine_kernel<DT, HD, 1, 8>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a, jobs, n_jobs);
  } else {
    hipLaunchKernelGGL((attn_combine_kernel<DT, HD, 1>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a, jobs, n_jobs);
  }
}

hipError_t launch_combine(int dt, int HD, const KArgs& a, const esp_combine* jobs, int n_jobs, int n_parts, hipStream_t st) {
  if (dt == ESP_F16 && HD == 128) launch_combine_t<ESP_F16, 128>(a, jobs, n_jobs, n_parts, st);
  else if (dt == ESP_F16 && HD == 256) launch_combine_t<ESP_F16, 256>(a, jobs, n_jobs, n_parts, st);
  else if (dt == ESP_BF16 && HD == 128) launch_combine_t<ESP_BF16, 128>(a, jobs, n_jobs, n_parts, st);
  else if (dt == ESP_BF16 && HD == 256) launch_combine_t<ESP_BF16, 256>(a, jobs, n_jobs, n_parts, st);
  else if (dt == ESP_F16 && HD == 512) launch_combine_t<ESP_F16, 512>(a, jobs, n_jobs, n_parts, st);
  else if (dt == ESP_BF16 && HD == 512) launch_combine_t<ESP_BF16, 512>(a, jobs, n_jobs, n_parts, st);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace esp
