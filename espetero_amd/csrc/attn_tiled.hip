// Tiled MFMA attention for passes with many query rows per tree: prefill,
// chunked prefill against the paged cache, large verify batches. Compute
// bound: Q K^T and P V run on v_mfma_f32_32x32x16 with K and V^T staged in LDS.
//
// Semantics: the reference's 8-row tile kernels (kernels/40_attention.metal:155-343,
// kernels/80_gemma.metal:157-342) with the tile enlarged to up to 128 rows:
// cached keys [k0, k1) through the block table or ring, then the tree's batch
// keys (`last` tiles) under the tree mask (80_:284) and the window (80_:285),
// online softmax in fp32, P rounded to the storage type before P.V, output
// O / l (0 when no key is visible) with the optional sigmoid gate, or a
// partial record for attention_combine.
//
// Mapping to gfx950. One workgroup = one tile of up to 128 query rows x one
// query head, 4 wavefronts of 32 rows. Keys advance in steps of 64 (four
// 16-key sub-blocks: one page each at page size 16); wavefront w stages
// sub-block w of the step: K rows as they lie in the pool, V already
// transposed in the pool (batch rows: K from the pass's row-major Kb, V from the
// transposed staging copy made before the launch). Each wavefront computes
//   S^T[64 keys][32 rows] = K . Q^T     A = K from LDS, B = Q^T in registers
//   P^T = exp2(S^T - m)                 registers; the D layout of S^T is the B layout of P^T
//   O^T[HD][32 rows]     += V^T . P^T   A = V^T from LDS
// so the softmax runs along registers of one lane plus one cross-lane step, and
// nothing is transposed on the way. The 8 P values a lane packs for one P.V
// step are keys {8 a + 4 hb + j}: the staging writes V^T with key bits 2 and 3
// swapped (kappa), which makes them one 16-byte LDS read.
// Two LDS stages: while a step is in the matrix cores the next step's tile is
// written to the other stage and the loads of the step after are in flight.
#include "common.hpp"

namespace esp {

__device__ __forceinline__ int kappa(int r) {  // swap bits 2 and 3: key <-> LDS column within a 16-key group
  return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1);
}

struct SubBlock {  // one 16-key sub-block of a step: where its K rows and V^T rows lie
  const uint16_t* k;
  const uint16_t* v;
  int k_ld, v_ld;  // elements between K rows / between V^T rows
  int j0;          // first key: cached index, or relative batch row
  int kind;        // 0 cached, 1 batch, 2 none
};

template <int DT, int HD>
__global__ __launch_bounds__(256, (HD == 128 ? 2 : 1)) void attn_tiled_kernel(const KArgs a, int n_tiles) {
  constexpr int KS = HD / 16, NT = HD / 32, LDK = HD + 8, LDV = 64 + 8;
  constexpr int CH = HD / 8;      // 16-byte chunks per K row
  constexpr int KP = CH / 4;      // K fill passes of a wavefront (64 / CH keys each)
  constexpr int VP = HD / 32;     // V^T fill passes (32 dims each)
  constexpr int STAGE = 64 * LDK + HD * LDV;  // elements of one LDS stage: K [64 keys][LDK], V^T [HD dims][LDV]
  extern __shared__ uint16_t lds[];
  __shared__ int red[4][6];

  // Workgroup -> (KV head, head in group, tile): consecutive ids differ in KV
  // head first, so the heads sharing a KV head land on the same XCD's L2, and
  // the tiles run last to first (the longest key ranges of a causal pass start first).
  const int kvh = blockIdx.x % a.Hkv;
  const int rest = blockIdx.x / a.Hkv;
  const int hg = rest % a.G;
  const int tile_i = n_tiles - 1 - rest / a.G;
  const int h = kvh * a.G + hg;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l32 = lane & 31, hb = lane >> 5;
  const esp_tile tile = a.tiles[tile_i];
  const esp_tree tree = a.trees[tile.tree];
  const int end = tree.base + tree.M;
  const int rows_live = min(a.R, end - tile.r0);
  const int rr0 = tile.r0 - tree.base;

  const int m = 32 * wave + l32;
  const bool row_ok = m < rows_live;
  const int row = row_ok ? tile.r0 + m : tile.r0;
  const int rr = rr0 + m;
  const int4 d = a.desc ? a.desc[row] : make_int4(0, 0, 0, 0);
  const int qpos = a.window > 0 ? a.pos[row].x : 0;

  u32x4 qf[KS];
  {
    const uint16_t* qp = a.Q + size_t(row) * a.q_ld + size_t(h) * HD + 8 * hb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = row_ok ? *reinterpret_cast<const u32x4*>(qp + 16 * ks) : u32x4{0, 0, 0, 0};
  }

  // ---- tile-wide facts about the rows (for the batch range and the no-mask fast paths)
  int k_last = -1, seg_max = 0, qpos_max = 0;
  {
    int kl = row_ok ? max(rr, max(d.z - 1, a.bidi ? d.w - 1 : -1)) : -1;
    int sm = row_ok ? d.x : 0, am = row_ok ? d.z : 0, qm = row_ok ? qpos : INT32_MIN;
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      kl = max(kl, __shfl_xor(kl, o));
      sm = max(sm, __shfl_xor(sm, o));
      am = max(am, __shfl_xor(am, o));
      qm = max(qm, __shfl_xor(qm, o));
    }
    if (lane == 0) {
      red[wave][0] = kl;
      red[wave][1] = sm;
      red[wave][2] = am;
      red[wave][3] = qm;
    }
    __syncthreads();
    int anc_max = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      k_last = max(k_last, red[w][0]);
      seg_max = max(seg_max, red[w][1]);
      anc_max = max(anc_max, red[w][2]);
      qpos_max = max(qpos_max, red[w][3]);
    }
    k_last = min(k_last, tree.M - 1);
    if (anc_max > 0 || a.bidi) seg_max = INT32_MAX;  // rows that see beyond the causal rule: always mask
  }

  // ---- the key range as 16-key sub-blocks: cached [k0, k1), then batch rows [b0, k_last]
  const int c0 = tile.k0 >> 4;
  const int n_c = tile.k1 > tile.k0 ? ((tile.k1 + 15) >> 4) - c0 : 0;
  const int a0 = (tree.base + tile.b0) >> 4;  // batch sub-blocks are groups of 16 absolute rows
  const int n_b = (tile.last && k_last >= tile.b0) ? ((tree.base + k_last) >> 4) - a0 + 1 : 0;
  const int n_sb = n_c + n_b;
  const int n_steps = (n_sb + 3) >> 2;
  const int n_groups = (a.n_rows + 15) >> 4;

  auto sub_block = [&](int s) {
    SubBlock sb;
    if (s < n_c) {
      const int js = (c0 + s) << 4;
      const int b = block_of(a, tree.table, js);
      const uint16_t* hbp = a.pool + head_base(a, HD, b, kvh);
      const int t0 = js % a.bt;
      sb.k = hbp + size_t(t0) * HD;
      sb.v = hbp + size_t(a.bt) * HD + t0;
      sb.k_ld = HD;
      sb.v_ld = a.bt;
      sb.j0 = js;
      sb.kind = 0;
    } else if (s < n_sb) {
      const int g = a0 + (s - n_c);
      sb.k = a.Kb + size_t(16 * g) * a.kv_ld + size_t(kvh) * HD;
      sb.v = a.vt_stage + (size_t(kvh) * n_groups + g) * size_t(HD) * 16;
      sb.k_ld = a.kv_ld;
      sb.v_ld = 16;
      sb.j0 = 16 * g - tree.base;
      sb.kind = 1;
    } else {
      sb.k = sb.v = nullptr;
      sb.k_ld = sb.v_ld = 0;
      sb.j0 = 0;
      sb.kind = 2;
    }
    return sb;
  };

  // Registers of one wavefront's share of a step's fill.
  u32x4 fk[KP], fv[VP];
  auto fill_load = [&](int step) {
    const SubBlock sb = sub_block(4 * step + wave);
    if (sb.kind == 2) {
#pragma unroll
      for (int p = 0; p < KP; ++p) fk[p] = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int p = 0; p < VP; ++p) fv[p] = u32x4{0, 0, 0, 0};
      return;
    }
    const int kpp = 64 / CH;  // keys per pass
#pragma unroll
    for (int p = 0; p < KP; ++p) {
      const int key = kpp * p + lane / CH;
      // Batch rows past the pass's last row do not exist.
      const bool in = sb.kind == 0 || (sb.j0 + tree.base + key) < a.n_rows;
      fk[p] = in ? *reinterpret_cast<const u32x4*>(sb.k + size_t(key) * sb.k_ld + 8 * (lane % CH)) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int p = 0; p < VP; ++p)
      fv[p] = *reinterpret_cast<const u32x4*>(sb.v + size_t(32 * p + (lane >> 1)) * sb.v_ld + 8 * (lane & 1));
    // Cached keys outside [k0, k1) may be memory never written: their V must not reach the products.
    if (sb.kind == 0 && (sb.j0 < tile.k0 || sb.j0 + 16 > tile.k1)) {
      const int jv = sb.j0 + 8 * (lane & 1);
      uint32_t msk[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool lo = jv + 2 * e >= tile.k0 && jv + 2 * e < tile.k1;
        const bool hi = jv + 2 * e + 1 >= tile.k0 && jv + 2 * e + 1 < tile.k1;
        msk[e] = (lo ? 0xffffu : 0u) | (hi ? 0xffff0000u : 0u);
      }
#pragma unroll
      for (int p = 0; p < VP; ++p) {
        fv[p].x &= msk[0];
        fv[p].y &= msk[1];
        fv[p].z &= msk[2];
        fv[p].w &= msk[3];
      }
    }
  };
  auto fill_store = [&](int stage) {
    uint16_t* Ks = lds + stage * STAGE;
    uint16_t* Vs = Ks + 64 * LDK;
    const int kpp = 64 / CH;
#pragma unroll
    for (int p = 0; p < KP; ++p)
      *reinterpret_cast<u32x4*>(Ks + (16 * wave + kpp * p + lane / CH) * LDK + 8 * (lane % CH)) = fk[p];
    // This lane holds keys 8 a .. 8 a + 7 of one dim (a = lane & 1): keys 8 a + 4 b + j go to column 8 b + 4 a + j.
#pragma unroll
    for (int p = 0; p < VP; ++p) {
      uint16_t* vrow = Vs + (32 * p + (lane >> 1)) * LDV + 16 * wave + 4 * (lane & 1);
      *reinterpret_cast<u32x2*>(vrow) = u32x2{fv[p].x, fv[p].y};
      *reinterpret_cast<u32x2*>(vrow + 8) = u32x2{fv[p].z, fv[p].w};
    }
  };

  f32x16 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[nt][i] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  // Batch steps past this wavefront's last row hold nothing it can see (plain causal rows).
  const int wave_last = rr0 + min(32 * wave + 31, rows_live - 1);

  if (n_steps > 0) {
    fill_load(0);
    fill_store(0);
    if (n_steps > 1) fill_load(1);
  }
  __syncthreads();
  for (int step = 0; step < n_steps; ++step) {
    const int cur = step & 1;
    if (step + 1 < n_steps) fill_store(cur ^ 1);   // the tile loaded during the previous step
    if (step + 2 < n_steps) fill_load(step + 2);
    const uint16_t* Ks = lds + cur * STAGE;
    const uint16_t* Vs = Ks + 64 * LDK;

    // Sub-block kinds of this step; a step whose keys are all batch rows after this
    // wavefront's rows is skipped (its rows see none of them).
    bool skip = false;
    {
      const int s0 = 4 * step;
      if (s0 >= n_c && seg_max != INT32_MAX) {
        const int jfirst = ((a0 + s0 - n_c) << 4) - tree.base;
        skip = jfirst > wave_last;
      }
    }
    if (!skip) {
      // ---- S^T = K . Q^T
      f32x16 s[2];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kt][i] = 0.0f;
        const uint16_t* kp = Ks + (32 * kt + l32) * LDK + 8 * hb;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          s[kt] = mfma32x16<DT>(*reinterpret_cast<const u32x4*>(kp + 16 * ks), qf[ks], s[kt]);
      }

      // ---- mask, online softmax. s[kt][4 i + j] is key 32 kt + 8 i + 4 hb + j of the step.
      // One uniform test per step: are all 64 keys visible to every row of this wavefront?
      bool step_full;
      {
        const int s0 = 4 * step;
        if (s0 + 4 <= n_c) {
          const int j0 = (c0 + s0) << 4;
          step_full = j0 >= tile.k0 && j0 + 64 <= tile.k1 && (a.window == 0 || qpos_max - j0 < a.window);
        } else if (s0 >= n_c && s0 + 4 <= n_sb) {
          const int j0 = ((a0 + s0 - n_c) << 4) - tree.base;
          step_full = a.window == 0 && j0 >= seg_max && j0 + 63 <= rr0 + 32 * wave && j0 >= 0;
        } else {
          step_full = false;
        }
      }
      if (!step_full) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const int sidx = 4 * step + 2 * kt + t;  // sub-block of the range
            // Visible keys of the sub-block for this lane's row: j in [lo, hi], plus j < anc.
            int j0, lo, hi, anc = 0;
            if (sidx < n_c) {
              j0 = (c0 + sidx) << 4;
              lo = tile.k0;
              hi = tile.k1 - 1;
              if (a.window > 0) lo = max(lo, qpos - a.window + 1);
            } else if (sidx < n_sb) {
              j0 = ((a0 + sidx - n_c) << 4) - tree.base;
              lo = max(d.x, 0);
              hi = min(k_last, (a.bidi && d.w > 0) ? max(rr, d.w - 1) : rr);
              anc = min(d.z, k_last + 1);
            } else {
              j0 = 0;
              lo = 1;
              hi = 0;
            }
            const bool batch_window = sidx >= n_c && sidx < n_sb && a.window > 0;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const int idx = 8 * t + e;  // = 4 i + j with i = 2 t + e / 4, j = e % 4
              const int j = j0 + 8 * (e >> 2) + 4 * hb + (e & 3);
              bool vis = (j >= lo && j <= hi) || (j >= 0 && j < anc);
              if (batch_window && vis) vis = qpos - a.pos[tree.base + j].x < a.window;
              s[kt][idx] = vis ? s[kt][idx] : -INFINITY;
            }
          }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kt][i]);
      mx *= a.scale_log2;  // scale > 0: the max commutes with it
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run, mx);
      const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
      const float corr = fast_exp2(m_run - m_safe);
      const bool changed = m_new > m_run;
      m_run = m_new;
      float ps = 0.0f;
      u32x4 pb[2][2];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          float p[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            p[e] = fast_exp2(__builtin_fmaf(s[kt][8 * t + e], a.scale_log2, -m_safe));
            ps += p[e];
          }
          pb[kt][t] = u32x4{pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7])};
        }
      l_run = l_run * corr + ps;
      if (__any(changed)) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[nt] *= corr;
      }

      // ---- O^T += V^T . P^T. pb[kt][t] holds keys 32 kt + 16 t + {8 a + 4 hb + j}: LDS columns 32 kt + 16 t + 8 hb ..
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const uint16_t* vp = Vs + (32 * nt + l32) * LDV + 8 * hb;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int t = 0; t < 2; ++t)
            acc[nt] = mfma32x16<DT>(*reinterpret_cast<const u32x4*>(vp + 32 * kt + 16 * t), pb[kt][t], acc[nt]);
      }
    }
    __syncthreads();
  }

  // ---- output: lane (row l32, half hb) holds dims 32 nt + 8 i + 4 hb + j at acc[nt][4 i + j]
  l_run += __shfl_xor(l_run, 32);
  if (!row_ok) return;
  if (tile.part >= 0) {
    const size_t rec = (size_t(tile.part) * a.Hkv + kvh) * a.cols + size_t(m) * a.G + hg;
    float* po = a.parts_o + rec * HD;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<f32x4*>(po + 32 * nt + 8 * i + 4 * hb) =
            f32x4{acc[nt][4 * i], acc[nt][4 * i + 1], acc[nt][4 * i + 2], acc[nt][4 * i + 3]};
    if (hb == 0) {
      a.parts_ml[rec * 2] = m_run;
      a.parts_ml[rec * 2 + 1] = l_run;
    }
    return;
  }
  const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
  uint16_t* op = a.O + size_t(row) * a.q_ld + size_t(h) * HD;
  const float* gp = a.gate ? a.gate + size_t(row) * a.gate_ld + size_t(h) * a.gate_hs + a.gate_off : nullptr;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int dd = 32 * nt + 8 * i + 4 * hb;
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        o[j] = acc[nt][4 * i + j] * inv;
        if (gp) o[j] = o[j] / (1.0f + __expf(-gp[dd + j]));
      }
      *reinterpret_cast<u32x2*>(op + dd) = u32x2{pack2<DT>(o[0], o[1]), pack2<DT>(o[2], o[3])};
    }
}

int tiled_workgroups_per_cu(int HD) { return HD == 128 ? 2 : 1; }

size_t tiled_smem_bytes(int HD) { return size_t(2) * size_t(64 * (HD + 8) + HD * (64 + 8)) * sizeof(uint16_t); }

template <int DT, int HD>
static hipError_t launch_tiled_t(const KArgs& a, int n_tiles, hipStream_t st) {
  const size_t smem = tiled_smem_bytes(HD);
  auto k = attn_tiled_kernel<DT, HD>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, int(smem));
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(k, dim3(unsigned(n_tiles) * a.H), dim3(256), smem, st, a, n_tiles);
  return hipGetLastError();
}

hipError_t launch_tiled(int dt, int HD, const KArgs& a, int n_tiles, hipStream_t st) {
  if (dt == ESP_F16 && HD == 128) return launch_tiled_t<ESP_F16, 128>(a, n_tiles, st);
  if (dt == ESP_F16 && HD == 256) return launch_tiled_t<ESP_F16, 256>(a, n_tiles, st);
  if (dt == ESP_BF16 && HD == 128) return launch_tiled_t<ESP_BF16, 128>(a, n_tiles, st);
  if (dt == ESP_BF16 && HD == 256) return launch_tiled_t<ESP_BF16, 256>(a, n_tiles, st);
  return hipErrorInvalidValue;
}

}  // namespace esp
