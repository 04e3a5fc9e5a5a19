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
// Mapping to gfx950. One workgroup = one tile of query rows x one query head,
// 4 wavefronts; a wavefront owns CT column tiles of 32 rows. CT = 1 (128-row
// tiles) is what is built: at CT = 2 the accumulators of two column tiles no
// longer fit the 256 architectural registers next to the operands and the
// compiler's copies through the accumulation registers cost more than the
// halved LDS reads gain. Keys advance in steps
// of 64 (four 16-key sub-blocks: one page each at page size 16); wavefront w
// stages sub-block w of a step: K rows as they lie in the pool, V already
// transposed in the pool (batch rows: K from the pass's row-major Kb, V from the
// transposed staging copy made before the launch). Per step a wavefront computes
//   S^T[64 keys][rows] = K . Q^T     A = K from LDS, B = Q^T in registers
//   P^T = exp2(S^T - m)              registers; the D layout of S^T is the B layout of P^T
//   O^T[HD][rows]     += V^T . P^T   A = V^T from LDS
// The 8 P values a lane packs for one P.V instruction are keys {8 a + 4 hb + j};
// the staging writes V^T with key bits 2 and 3 swapped, which makes them one
// 16-byte LDS read.
// Two LDS stages: while step i is in the matrix cores, step i + 1 (loaded during
// the previous step) is written to the other stage and the loads of step i + 2
// are in flight. One barrier per step. A step's math runs in two halves of 32
// keys so the second half's Q K^T sits next to the first half's softmax.
#include "common.hpp"

namespace esp {

struct SubBlock {  // one 16-key sub-block of a step: where its K rows and V^T rows lie
  const uint16_t* k;
  const uint16_t* v;
  int k_ld, v_ld;  // elements between K rows / between V^T rows
  int j0;          // first key: cached index, or relative batch row
  int kind;        // 0 cached, 1 batch, 2 none
};

// KST: LDS stages of K and V^T (2: step i + 1 is written while step i is in the matrix cores).
template <int DT, int HD, int CT, int KST, int OCC>
__global__ __launch_bounds__(256, OCC) void attn_tiled_kernel(const KArgs a, int n_tiles) {
  constexpr int KS = HD / 16, NT = HD / 32, LDK = HD + 8, LDV = 64 + 8;
  constexpr int CH = HD / 8;      // 16-byte chunks per K row
  constexpr int KP = CH / 4;      // K fill passes of a wavefront (64 / CH keys each)
  constexpr int VP = HD / 32;     // V^T fill passes (32 dims each)
  constexpr int KBUF = 64 * LDK, VBUF = HD * LDV;  // elements of one K / V^T stage
  extern __shared__ uint16_t lds[];  // K[KST][KBUF], V[2][VBUF]
  __shared__ int red[4][4];

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
  const int table = tile.pad > 0 ? tile.pad - 1 : tree.table;
  const int end = tree.base + tree.M;
  const int rows_live = min(a.R, end - tile.r0);
  const int rr0 = tile.r0 - tree.base;

  // ---- this lane's rows: one per column tile
  bool row_ok[CT];
  int row[CT], rr[CT], qpos[CT];
  int4 d[CT];
  u32x4 qf[CT][KS];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int m = 32 * (CT * wave + c) + l32;
    row_ok[c] = m < rows_live;
    row[c] = row_ok[c] ? tile.r0 + m : tile.r0;
    rr[c] = rr0 + m;
    d[c] = a.desc ? a.desc[row[c]] : make_int4(0, 0, 0, 0);
    qpos[c] = a.window > 0 ? a.pos[row[c]].x : 0;
    const uint16_t* qp = a.Q + size_t(row[c]) * a.q_ld + size_t(h) * HD + 8 * hb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qf[c][ks] = row_ok[c] ? *reinterpret_cast<const u32x4*>(qp + 16 * ks) : u32x4{0, 0, 0, 0};
  }

  // ---- tile-wide facts about the rows (for the batch range and the no-mask fast path)
  int k_last = -1, seg_max = 0, qpos_max = 0;
  {
    int kl = -1, sm = 0, am = 0, qm = INT32_MIN;
#pragma unroll
    for (int c = 0; c < CT; ++c)
      if (row_ok[c]) {
        kl = max(kl, max(rr[c], max(d[c].z - 1, a.bidi ? d[c].w - 1 : -1)));
        sm = max(sm, d[c].x);
        am = max(am, d[c].z);
        qm = max(qm, qpos[c]);
      }
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

  // Block ids of this wavefront's cached sub-blocks, 64 steps at a time: lane l holds the
  // block of sub-block 4 (ids_step0 + l) + wave, so the per-step lookup is a lane read
  // instead of a dependent memory access in front of every staging load.
  int ids = 0, ids_step0 = -(1 << 30);
  auto block_id = [&](int step, int s) {
    if (step < ids_step0 || step >= ids_step0 + 64) {
      ids_step0 = step;
      const int sl = 4 * (step + lane) + wave;
      ids = sl < n_c ? block_of(a, table, (c0 + sl) << 4) : 0;
    }
    (void)s;
    return __builtin_amdgcn_readlane(ids, step - ids_step0);
  };

  auto sub_block = [&](int s) {
    SubBlock sb;
    if (s < n_c) {
      const int js = (c0 + s) << 4;
      const int b = block_id(s >> 2, s);
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

  // Registers of one wavefront's share of a step's staging: K rows and V^T rows travel separately.
  u32x4 fk[KP], fv[VP];
  auto load_k = [&](int step) {
    if (step >= n_steps) return;
    const SubBlock sb = sub_block(4 * step + wave);
    constexpr int kpp = 64 / CH;  // keys per pass
#pragma unroll
    for (int p = 0; p < KP; ++p) {
      const int key = kpp * p + lane / CH;
      // Batch rows past the pass's last row do not exist; a sub-block past the range is zero.
      const bool in = sb.kind == 0 || (sb.kind == 1 && (sb.j0 + tree.base + key) < a.n_rows);
      fk[p] = in ? *reinterpret_cast<const u32x4*>(sb.k + size_t(key) * sb.k_ld + 8 * (lane % CH)) : u32x4{0, 0, 0, 0};
    }
  };
  auto load_v = [&](int step) {
    if (step >= n_steps) return;
    const SubBlock sb = sub_block(4 * step + wave);
#pragma unroll
    for (int p = 0; p < VP; ++p)
      fv[p] = sb.kind != 2 ? *reinterpret_cast<const u32x4*>(sb.v + size_t(32 * p + (lane >> 1)) * sb.v_ld + 8 * (lane & 1))
                           : u32x4{0, 0, 0, 0};
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
  auto store_k = [&](int step) {
    if (step >= n_steps) return;
    uint16_t* Ks = lds + (step % KST) * KBUF;
    constexpr int kpp = 64 / CH;
#pragma unroll
    for (int p = 0; p < KP; ++p)
      *reinterpret_cast<u32x4*>(Ks + (16 * wave + kpp * p + lane / CH) * LDK + 8 * (lane % CH)) = fk[p];
  };
  auto store_v = [&](int step) {
    if (step >= n_steps) return;
    uint16_t* Vs = lds + KST * KBUF + (step & 1) * VBUF;
    // This lane holds keys 8 a .. 8 a + 7 of one dim (a = lane & 1): keys 8 a + 4 b + j go to column 8 b + 4 a + j.
#pragma unroll
    for (int p = 0; p < VP; ++p) {
      uint16_t* vrow = Vs + (32 * p + (lane >> 1)) * LDV + 16 * wave + 4 * (lane & 1);
      *reinterpret_cast<u32x2*>(vrow) = u32x2{fv[p].x, fv[p].y};
      *reinterpret_cast<u32x2*>(vrow + 8) = u32x2{fv[p].z, fv[p].w};
    }
  };

  f32x16 acc[CT][NT];
  float m_run[CT], l_run[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    m_run[c] = -INFINITY;
    l_run[c] = 0.0f;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[c][nt][i] = 0.0f;
  }

  // Batch steps past this wavefront's last row hold nothing it can see (plain causal rows).
  const int wave_last = rr0 + min(32 * CT * wave + 32 * CT - 1, rows_live - 1);
  auto skipped = [&](int step) {
    const int s0 = 4 * step;
    if (s0 < n_c || seg_max == INT32_MAX) return false;
    return ((a0 + s0 - n_c) << 4) - tree.base > wave_last;
  };

  // S^T of half step (step, kt): s[c][4 i + j] is key 32 kt + 8 i + 4 hb + j of the step for the
  // lane's row of column tile c.
  auto qk = [&](int step, int kt, f32x16 (&s)[CT]) {
    const uint16_t* kp = lds + (step % KST) * KBUF + (32 * kt + l32) * LDK + 8 * hb;
#pragma unroll
    for (int c = 0; c < CT; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[c][i] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const u32x4 kf = *reinterpret_cast<const u32x4*>(kp + 16 * ks);
#pragma unroll
      for (int c = 0; c < CT; ++c) s[c] = mfma32x16<DT>(kf, qf[c][ks], s[c]);
    }
  };

  // Masks (cold path), online softmax, O^T += V^T . P^T of half step (step, kt).
  auto softmax_pv = [&](int step, int kt, f32x16 (&s)[CT]) {
    bool half_full;  // all 32 keys visible to every row of this wavefront?
    {
      const int s0 = 4 * step + 2 * kt;
      if (s0 + 2 <= n_c) {
        const int j0 = (c0 + s0) << 4;
        half_full = j0 >= tile.k0 && j0 + 32 <= tile.k1 && (a.window == 0 || qpos_max - j0 < a.window);
      } else if (s0 >= n_c && s0 + 2 <= n_sb) {
        const int j0 = ((a0 + s0 - n_c) << 4) - tree.base;
        half_full = a.window == 0 && j0 >= seg_max && j0 + 31 <= rr0 + 32 * CT * wave && j0 >= 0;
      } else {
        half_full = false;
      }
    }
    if (!half_full) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int sidx = 4 * step + 2 * kt + t;  // sub-block of the range
        const bool cached = sidx < n_c, batch = !cached && sidx < n_sb;
        const int j0 = cached ? (c0 + sidx) << 4 : ((a0 + sidx - n_c) << 4) - tree.base;
#pragma unroll
        for (int c = 0; c < CT; ++c) {
          // Visible keys of the sub-block for this lane's row: j in [lo, hi], or 0 <= j < anc.
          int lo, hi, anc = 0;
          if (cached) {
            lo = tile.k0;
            hi = tile.k1 - 1;
            if (a.window > 0) lo = max(lo, qpos[c] - a.window + 1);
          } else if (batch) {
            lo = max(d[c].x, 0);
            hi = min(k_last, (a.bidi && d[c].w > 0) ? max(rr[c], d[c].w - 1) : rr[c]);
            anc = min(d[c].z, k_last + 1);
          } else {
            lo = 1;
            hi = 0;
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int idx = 8 * t + e;  // = 4 i + j with i = 2 t + e / 4, j = e % 4
            const int j = j0 + 8 * (e >> 2) + 4 * hb + (e & 3);
            bool vis = (j >= lo && j <= hi) || (j >= 0 && j < anc);
            if (batch && a.window > 0 && vis) vis = qpos[c] - a.pos[tree.base + j].x < a.window;
            s[c][idx] = vis ? s[c][idx] : -INFINITY;
          }
        }
      }
    }
    u32x4 pb[CT][2];
    // Lazy rescale: the running reference m_run only moves when a row's maximum exceeds it by
    // more than 8 (log2 units), so P stays below 2^8 and the accumulators are rescaled a handful
    // of times per row instead of once per step.
    float mx[CT];
    bool grow = false;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      float x = -INFINITY;
#pragma unroll
      for (int i = 0; i < 16; ++i) x = fmaxf(x, s[c][i]);
      x *= a.scale_log2;  // scale > 0: the max commutes with it
      mx[c] = fmaxf(x, __shfl_xor(x, 32));
      grow = grow || (mx[c] > m_run[c] + 8.0f);
    }
    if (__any(grow)) {
      asm volatile("s_nop 0");  // a real branch: this block must not be speculated into the loop body
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const float m_new = fmaxf(m_run[c], mx[c]);
        const float corr = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_run[c] - m_new);
        m_run[c] = m_new;
        l_run[c] *= corr;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[c][nt] *= corr;
      }
    }
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      const float m_safe = (m_run[c] == -INFINITY) ? 0.0f : m_run[c];
      float ps = 0.0f;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float p[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          p[e] = fast_exp2(__builtin_fmaf(s[c][8 * t + e], a.scale_log2, -m_safe));
          ps += p[e];
        }
        pb[c][t] = u32x4{pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7])};
      }
      l_run[c] += ps;
    }
    // pb[c][t] holds keys 32 kt + 16 t + {8 a + 4 hb + j}: LDS columns 32 kt + 16 t + 8 hb ..
    const uint16_t* Vs = lds + KST * KBUF + (step & 1) * VBUF;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const uint16_t* vp = Vs + (32 * nt + l32) * LDV + 32 * kt + 8 * hb;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const u32x4 vf = *reinterpret_cast<const u32x4*>(vp + 16 * t);
#pragma unroll
        for (int c = 0; c < CT; ++c) acc[c][nt] = mfma32x16<DT>(vf, pb[c][t], acc[c][nt]);
      }
    }
  };

  // ---- prologue: step 0 staged, step 1 in registers
  f32x16 sa[CT], sb[CT];
  load_k(0);
  load_v(0);
  store_k(0);
  store_v(0);
  load_k(1);
  load_v(1);
  __syncthreads();

  // Iteration i: stage step i + 1 (loaded during the previous iteration) into the other
  // LDS stage, request step i + 2, then the math of step i in two halves of 32 keys so the
  // second half's Q K^T sits next to the first half's softmax.
  // Steps this wavefront computes: batch steps past its last row hold nothing it can see.
  int my_steps = n_steps;
  while (my_steps > 0 && skipped(my_steps - 1)) --my_steps;
  int i = 0;
  for (; i < my_steps; ++i) {
    store_k(i + 1);
    store_v(i + 1);
    load_k(i + 2);
    load_v(i + 2);
    qk(i, 0, sa);
    qk(i, 1, sb);
    softmax_pv(i, 0, sa);
    softmax_pv(i, 1, sb);
    __syncthreads();
  }
  for (; i < n_steps; ++i) {  // keep staging for the wavefronts whose rows reach further
    store_k(i + 1);
    store_v(i + 1);
    load_k(i + 2);
    load_v(i + 2);
    __syncthreads();
  }

  // ---- output: lane (row l32 of column tile c, half hb) holds dims 32 nt + 8 i + 4 hb + j at acc[c][nt][4 i + j]
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const float l = l_run[c] + __shfl_xor(l_run[c], 32);
    if (!row_ok[c]) continue;
    const int m = 32 * (CT * wave + c) + l32;
    if (tile.part >= 0) {
      const size_t rec = (size_t(tile.part) * a.Hkv + kvh) * a.cols + size_t(m) * a.G + hg;
      float* po = a.parts_o + rec * HD;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          *reinterpret_cast<f32x4*>(po + 32 * nt + 8 * i + 4 * hb) =
              f32x4{acc[c][nt][4 * i], acc[c][nt][4 * i + 1], acc[c][nt][4 * i + 2], acc[c][nt][4 * i + 3]};
      if (hb == 0) {
        a.parts_ml[rec * 2] = m_run[c];
        a.parts_ml[rec * 2 + 1] = l;
      }
      continue;
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    uint16_t* op = a.O + size_t(row[c]) * a.q_ld + size_t(h) * HD;
    const float* gp = a.gate ? a.gate + size_t(row[c]) * a.gate_ld + size_t(h) * a.gate_hs + a.gate_off : nullptr;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int dd = 32 * nt + 8 * i + 4 * hb;
        float o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          o[j] = acc[c][nt][4 * i + j] * inv;
          if (gp) o[j] = o[j] / (1.0f + __expf(-gp[dd + j]));
        }
        *reinterpret_cast<u32x2*>(op + dd) = u32x2{pack2<DT>(o[0], o[1]), pack2<DT>(o[2], o[3])};
      }
  }
}

// Column tiles per wavefront and the largest tile each variant takes.
constexpr int tiled_ct(int) { return 1; }
constexpr int tiled_occ(int HD) { return HD == 128 ? 2 : 1; }
int tiled_max_rows(int HD) { return 128 * tiled_ct(HD); }
int tiled_workgroups_per_cu(int HD) { return tiled_occ(HD); }

constexpr int tiled_kst(int) { return 2; }
size_t tiled_smem_bytes(int HD) { return (size_t(tiled_kst(HD)) * 64 * (HD + 8) + size_t(2) * HD * (64 + 8)) * sizeof(uint16_t); }

template <int DT, int HD>
static hipError_t launch_tiled_t(const KArgs& a, int n_tiles, hipStream_t st) {
  const size_t smem = tiled_smem_bytes(HD);
  auto k = attn_tiled_kernel<DT, HD, tiled_ct(HD), tiled_kst(HD), tiled_occ(HD)>;
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
