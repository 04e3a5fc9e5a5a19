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
// query head, 4 wavefronts of 32 rows each. Keys advance in steps of 64 (four
// 16-key sub-blocks: one page each at page size 16). Wavefront w stages
// sub-block w of a step with global_load_lds_dwordx4: 16 bytes per lane travel
// from global memory straight into LDS (lane l's bytes land at base + 16 l),
// no staging registers and no LDS store instructions. Per step a wavefront computes
//   S^T[64 keys][32 rows] = K . Q^T    A = K from LDS, B = Q^T in registers
//   P^T = exp2(S^T - m)                registers; the D layout of S^T is the B layout of P^T
//   O^T[HD][32 rows]     += V^T . P^T  A = V^T from LDS
//
// LDS layout of one stage.
//   K: 64 rows of HD elements, unpadded; the 16-byte chunk c of row r lies at
//      chunk position c ^ (pi(r) & 15), where pi swaps bits 2 and 3 of a row
//      index. The lane with S^T row l reads key row pi(l): its chunk position is
//      c ^ (l & 15), distinct over any 8 or 16 consecutive lanes -> no bank
//      conflicts. With the rows permuted by pi the 8 P values a lane packs for one
//      P.V instruction are 8 consecutive keys, which is how V^T lies in memory.
//   V^T: per sub-block, per group of 32 dims: [half of the 16 keys][32 dims][8 keys],
//      i.e. exactly the order in which the 64 lanes of a P.V operand read it.
// Two stages: step i + 1 lands in the other stage while step i is in the matrix
// cores; one barrier per step. A step's math runs in two halves of 32 keys.
//
// Keys a row must not see get S = -inf before the softmax; V of keys outside the
// tile's range (cached memory possibly never written) is zeroed in LDS by the
// wavefront that staged it, so 0 * garbage never reaches the accumulators.
#include <utility>

#include "common.hpp"
#include "lds_direct.hpp"

namespace esp {

template <int DT, int HD, int OCC>
__global__ __launch_bounds__(256, OCC) void attn_tiled_kernel(const KArgs a, int n_tiles) {
  constexpr int KS = HD / 16, NT = HD / 32;
  // Head dim 128 runs the softmax without a per-step maximum, in slices laid between the matrix instructions by
  // hand (measured 3 % faster there); at head dim 256, with one wavefront per SIMD and every register taken,
  // the same code spilled and ran 3 to 8 % slower than the form with a lazily moved maximum, which it keeps.
  constexpr bool LEAN = HD == 128;
  constexpr int ROWB = HD * 2;     // bytes of one K row
  constexpr int CH = HD / 8;       // 16-byte chunks per K row
  constexpr int RPI = 64 / CH;     // K rows one load instruction covers
  constexpr int KP = 16 / RPI;     // K load instructions per sub-block
  constexpr int VP = HD / 32;      // V^T load instructions per sub-block
  constexpr int KBUF = 64 * ROWB;  // bytes of one K stage
  constexpr int SUBV = HD * 32;    // bytes of one V^T sub-block
  constexpr int VBUF = 4 * SUBV;   // bytes of one V^T stage
  constexpr int VOFF = 2 * KBUF;   // layout: K stage 0, K stage 1, V^T stage 0, V^T stage 1
  extern __shared__ __attribute__((aligned(16))) char lds[];  // the only LDS object: operand offsets fold into the reads
  int(*red)[4] = reinterpret_cast<int(*)[4]>(lds + 4 * KBUF);  // 4 x 4 ints behind the stages
  const uint32_t lds_base = uint32_t(uintptr_t(lds));  // LDS byte address of lds[0]

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
  esp_tile tile = a.tiles[tile_i];

  // ---- this lane's row. Its loads need the tile's record only (a row past the tree's last one reads the pass's
  // last row instead and is zeroed once the tree's record says so): they are in flight while that record arrives.
  const int m_row = 32 * wave + l32;
  const int row = min(tile.r0 + m_row, a.n_rows - 1);
  int4 d = a.desc ? a.desc[row] : make_int4(0, 0, 0, 0);
  int qpos = a.window > 0 ? a.pos[row].x : 0;
  // Q fragments as stored. The scale (times log2 e) is applied to the fp32 score in the same fused
  // multiply-add that subtracts the row's reference: multiplying Q itself and rounding it back to the
  // storage type would cost every score a relative 2^-9 (bf16) before the exponential, which at logits
  // of a few units is more than the 2e-3 the path promises (the reference pre-scales Q only by an
  // exact power of two, kernels/40_attention.metal:195-200).
  u32x4 qf[KS];
  {
    const uint16_t* qp = a.Q + size_t(row) * a.q_ld + size_t(h) * HD + 8 * hb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const u32x4*>(qp + 16 * ks);
  }

  const esp_tree tree = a.trees[tile.tree];
  if (tile.k1 == INT32_MAX) tile.k1 = tree.P;  // open-ended range: up to the tree's cached length as it is now
  const int table = tile.pad > 0 ? tile.pad - 1 : tree.table;
  const int end = tree.base + tree.M;
  const int rows_live = min(a.R, end - tile.r0);
  const int rr0 = tile.r0 - tree.base;
  const int rr = rr0 + m_row;

  // ---- the key range as 16-key sub-blocks: cached [k0, k1), then batch rows [b0, k_last]
  const int c0 = tile.k0 >> 4;
  const int n_c = tile.k1 > tile.k0 ? ((tile.k1 + 15) >> 4) - c0 : 0;
  const int a0 = (tree.base + tile.b0) >> 4;  // batch sub-blocks are groups of 16 absolute rows
  // Batch rows in the pool (no Kb / Vb): the pass's rows were appended before the attention (esp_attn_prep with a
  // row table, or esp_kv_save), row j of a tree at position P + j of the tree's own block list, and P - base is a
  // multiple of 16 (the caller's promise; esp_attn_validate checks it). A batch sub-block - 16 absolute rows - is
  // then one 16-token sub-block of the pool and is staged like a cached one; the masks stay in row numbers.
  const bool in_pool = a.Kb == nullptr;
  const int pool_shift = tree.P - tree.base;  // pool position of absolute row r: r + pool_shift
  // Sub-blocks the tree's block list can name for this tile: the cached ones and, with the rows in the pool, the
  // batch ones up to the tree's last row - at least those the tile will use (its batch range ends at a row that the
  // rows' own facts give, which are still on their way here).
  const int n_sb_list = n_c + ((in_pool && tile.last && tree.M > tile.b0) ? ((end - 1) >> 4) - a0 + 1 : 0);

  // Pool addresses of this wavefront's sub-blocks, 64 steps at a time: lane l holds the byte address of the K rows of
  // sub-block 4 (adr_step0 + l) + wave - the block list entry, the head's place in the block and the sub-block's place
  // in the head worked out by 64 lanes at once - so that in front of a step's staging loads stand two lane reads
  // instead of a dependent memory access and the scalar arithmetic behind it. V^T of a 16-token sub-block lies
  // bt rows' worth of bytes behind its K rows whatever the sub-block.
  uint32_t kadr_lo = 0, kadr_hi = 0;
  int adr_step0 = -(1 << 30);
  auto pool_k = [&](int step) __attribute__((always_inline)) {
    if (step < adr_step0 || step >= adr_step0 + 64) {
      adr_step0 = step;
      const int sl = 4 * (step + lane) + wave;
      const int js = sl < n_c ? (c0 + sl) << 4 : sl < n_sb_list ? ((a0 + sl - n_c) << 4) + pool_shift : -1;
      uint64_t adr = 0;
      if (js >= 0) {
        const int b = block_of(a, table, js);
        const int t0 = a.bt == 16 ? 0 : js % a.bt;
        adr = reinterpret_cast<uint64_t>(a.pool + head_base(a, HD, b, kvh)) + uint64_t(t0) * ROWB;
      }
      kadr_lo = uint32_t(adr);
      kadr_hi = uint32_t(adr >> 32);
    }
    const int idx = step - adr_step0;
    const uint32_t lo = uint32_t(__builtin_amdgcn_readlane(int(kadr_lo), idx)), hi = uint32_t(__builtin_amdgcn_readlane(int(kadr_hi), idx));
    return reinterpret_cast<const char*>(uint64_t(lo) | (uint64_t(hi) << 32));
  };

  // ---- staging: per-lane constants of the load instructions
  // K instruction q covers rows q RPI .. of the sub-block; this lane brings chunk
  // position `lane % CH` of row q RPI + lane / CH, i.e. global chunk position ^ pi(row).
  const int r0 = lane / CH;
  const uint32_t kcol0 = uint32_t(((lane % CH) ^ r0) << 4);
  // cached keys: rows HD elements apart, i.e. instruction q's rows start 1024 q bytes further; that part
  // travels in the instruction's immediate offset. Instruction q's lane offset is
  // r0 ROWB + (kcol0 ^ kswz(q)); the staging code derives it where it is used.
  auto kswz = [](int q) constexpr { return uint32_t(swap23(q * RPI) << 4); };
  // V^T instruction q covers dims 32 q ..: this lane brings keys 8 (lane / 32) .. + 7 of dim 32 q + lane % 32.
  // (32 V^T rows of 16 tokens are 1024 bytes, in the pool's sub-blocks and in the staged batch rows alike)
  const uint32_t voff = uint32_t(l32 * 32 + hb * 16);

  // This wavefront's sub-block of `step`, one the pool holds, into `stage`.
  // The per-instruction lane offsets are derived here, in every call, from two registers. Computed
  // once in front of the loops (which the compiler does with anything loop-invariant, hence the
  // empty asm) they would occupy a register each for the whole kernel and end up in scratch
  // memory, whose reloads wait on the same counter as the staging loads and serialise them.
  auto stage_pool = [&](int step, int stage) __attribute__((always_inline)) {
    const uint32_t kdst = lds_base + stage * KBUF + wave * (16 * ROWB);
    const uint32_t vdst = lds_base + VOFF + stage * VBUF + wave * SUBV;
    uint32_t kc = kcol0, kr = uint32_t(r0);
    asm volatile("" : "+v"(kc), "+v"(kr));
    const char* kb = pool_k(step);
    const char* vb = kb + size_t(a.bt) * ROWB;  // the 16-token sub-block: 32 HD contiguous bytes
    const uint32_t kro = kr * ROWB;
#pragma unroll
    for (int q = 0; q < KP; q += 4)
      load_to_lds16_x4(kb + q * 1024, kro + (kc ^ kswz(q)), kro + (kc ^ kswz(q + 1)), kro + (kc ^ kswz(q + 2)),
                       kro + (kc ^ kswz(q + 3)), kdst + q * 1024);
#pragma unroll
    for (int q = 0; q < VP; q += 4) load_to_lds16_x4(vb + q * 1024, voff, voff, voff, voff, vdst + q * 1024);
  };
  // Where the tile's first step is four sub-blocks of the pool whatever the rows' facts say - cached ones, or batch
  // ones up to the tile's first row, which that row sees - its staging needs nothing of the rows: it leaves now,
  // and the rows' facts below are worked out while it lands.
  int n_b_sure = 0;
  if (in_pool && tile.last) {
    const int k_sure = min(min(rr0, tree.M - 1), tile.last >= 2 ? tile.last - 2 : INT32_MAX);
    if (k_sure >= tile.b0) n_b_sure = ((tree.base + k_sure) >> 4) - a0 + 1;
  }
  const bool early = n_c + n_b_sure >= 4;
  if (early) stage_pool(0, 0);

  const bool row_ok = m_row < rows_live;
  if (!row_ok) {
    d = make_int4(0, 0, 0, 0);
    qpos = 0;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = u32x4{0, 0, 0, 0};
  }

  // ---- tile-wide facts about the rows (for the batch range and the no-mask fast path)
  int k_last = -1, seg_max = 0, qpos_max = 0;
  bool anc_any = false;  // does any row of the tile see ancestors (keys below its segment)?
  {
    int kl = -1, sm = 0, am = 0, qm = INT32_MIN;
    if (row_ok) {
      kl = max(rr, max(d.z - 1, a.bidi ? d.w - 1 : -1));
      sm = d.x;
      am = d.z;
      qm = qpos;
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
    // The same in every lane; saying so keeps everything derived from them in scalar registers.
    // a part whose batch range is cut ends at row last - 2 of the tree (last = 1: open, up to what its rows see)
    k_last = __builtin_amdgcn_readfirstlane(min(min(k_last, tree.M - 1), tile.last >= 2 ? tile.last - 2 : INT32_MAX));
    seg_max = __builtin_amdgcn_readfirstlane(seg_max);
    anc_max = __builtin_amdgcn_readfirstlane(anc_max);
    qpos_max = __builtin_amdgcn_readfirstlane(qpos_max);
    if (anc_max > 0 || a.bidi) seg_max = INT32_MAX;  // rows that see beyond the causal rule: always mask
    anc_any = anc_max > 0;
  }

  const int n_b = (tile.last && k_last >= tile.b0) ? ((tree.base + k_last) >> 4) - a0 + 1 : 0;
  const int n_sb = n_c + n_b;
  const int n_steps = (n_sb + 3) >> 2;
  const int n_groups = (a.n_rows + 15) >> 4;

  // Windowed layers: do this tile's batch keys need a window test at all? Not when the oldest position among
  // them is inside the window of the row with the largest position. Where they do and their positions rise by
  // one per row (position of row j = j + pos_shift: a plain chunk of prompt), the window is one more lower
  // bound in row numbers, j >= qpos - w_off, and a step whose rows lie at or above bw_lo is inside every row's
  // window; only other position patterns (trees) take the per-key position test.
  bool batch_window = false;
  int w_off = 1 << 30, bw_lo = INT32_MIN;
  if (a.window > 0 && n_b > 0) {
    int kp = INT32_MAX, dmin = INT32_MAX, dmax = INT32_MIN;
    for (int j = tile.b0 + int(threadIdx.x); j <= k_last; j += 256) {
      const int p = a.pos[tree.base + j].x;
      kp = min(kp, p);
      dmin = min(dmin, p - j);
      dmax = max(dmax, p - j);
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      kp = min(kp, __shfl_xor(kp, o));
      dmin = min(dmin, __shfl_xor(dmin, o));
      dmax = max(dmax, __shfl_xor(dmax, o));
    }
    __syncthreads();  // every wavefront has read the facts above
    if (lane == 0) {
      red[wave][0] = kp;
      red[wave][1] = dmin;
      red[wave][2] = dmax;
    }
    __syncthreads();
    kp = __builtin_amdgcn_readfirstlane(min(min(red[0][0], red[1][0]), min(red[2][0], red[3][0])));
    dmin = __builtin_amdgcn_readfirstlane(min(min(red[0][1], red[1][1]), min(red[2][1], red[3][1])));
    dmax = __builtin_amdgcn_readfirstlane(max(max(red[0][2], red[1][2]), max(red[2][2], red[3][2])));
    if (qpos_max - kp >= a.window) {
      if (dmin == dmax) {
        w_off = a.window - 1 + dmin;
        bw_lo = qpos_max - w_off;
      } else {
        batch_window = true;
      }
    }
  }

  // interior: the caller knows that all four sub-blocks of the step are cached keys, or batch rows that exist.
  auto fill = [&](int step, int stage, auto interior) __attribute__((always_inline)) {
    const int s = 4 * step + wave;
    const bool batch_sb = s >= n_c && (decltype(interior)::value || s < n_sb);
    if (s < n_c || (in_pool && batch_sb)) {
      stage_pool(step, stage);
    } else if (batch_sb) {
      const uint32_t kdst = lds_base + stage * KBUF + wave * (16 * ROWB);
      const uint32_t vdst = lds_base + VOFF + stage * VBUF + wave * SUBV;
      uint32_t kc = kcol0, kr = uint32_t(r0);
      asm volatile("" : "+v"(kc), "+v"(kr));
      const int g = a0 + (s - n_c);
      const int lim = decltype(interior)::value ? 15 : a.n_rows - 1 - 16 * g;  // batch rows past the pass's last row do not exist
      const char* kb = reinterpret_cast<const char*>(a.Kb + size_t(16 * g) * a.kv_ld + size_t(kvh) * HD);
      const char* vb = reinterpret_cast<const char*>(a.vt_stage + (size_t(kvh) * n_groups + g) * size_t(HD) * 16);
      const uint32_t kld = uint32_t(a.kv_ld) * 2;
      if (lim >= 15) {  // all 16 rows exist: instruction q's rows start q RPI rows further, which goes into its base
        const uint32_t kro = kr * kld;
#pragma unroll
        for (int q = 0; q < KP; ++q) load_to_lds16(kb + size_t(q * RPI) * kld, kro + (kc ^ kswz(q)), kdst + q * 1024);
      } else {  // the pass's last group: rows past the end repeat the last one (their scores are masked)
#pragma unroll
        for (int q = 0; q < KP; ++q)
          load_to_lds16(kb, uint32_t(min(q * RPI + int(kr), lim)) * kld + (kc ^ kswz(q)), kdst + q * 1024);
      }
#pragma unroll
      for (int q = 0; q < VP; q += 4) load_to_lds16_x4(vb + q * 1024, voff, voff, voff, voff, vdst + q * 1024);
    } else {  // past the range: K stays whatever it was (S is masked), V^T must be finite
#pragma unroll
      for (int q = 0; q < VP; ++q)
        *reinterpret_cast<u32x4*>(lds + VOFF + stage * VBUF + wave * SUBV + q * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
    }
  };
  // After this wavefront's loads of `step` have landed: cached keys outside [k0, k1) may be
  // memory never written; their V must not reach the products.
  auto fix = [&](int step, int stage) __attribute__((always_inline)) {
    const int s = 4 * step + wave;
    // keys [v0, v1) of the sub-block's own numbering are memory that has been written: the tile's cached range, or,
    // for batch rows read from the pool, everything up to the tree's last row (what lies below its first row is the
    // end of its cached keys)
    int j0, v0, v1;
    if (s < n_c) {
      j0 = (c0 + s) << 4;
      v0 = tile.k0;
      v1 = tile.k1;
    } else if (in_pool && s < n_sb) {
      j0 = ((a0 + s - n_c) << 4) - tree.base;
      v0 = INT32_MIN;
      v1 = tree.M;
    } else {
      return;
    }
    if (j0 >= v0 && j0 + 16 <= v1) return;
    const int jv = j0 + 8 * hb;
    u32x4 msk;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool lo = jv + 2 * e >= v0 && jv + 2 * e < v1;
      const bool hi = jv + 2 * e + 1 >= v0 && jv + 2 * e + 1 < v1;
      msk[e] = (lo ? 0xffffu : 0u) | (hi ? 0xffff0000u : 0u);
    }
#pragma unroll
    for (int q = 0; q < VP; ++q) {
      u32x4* p = reinterpret_cast<u32x4*>(lds + VOFF + stage * VBUF + wave * SUBV + q * 1024 + lane * 16);
      *p = *p & msk;
    }
  };

  // ---- operand reads: per-lane byte offsets inside a K stage, one per 16-dim slice
  uint32_t kaddr[KS];
  {
    const int prow = (l32 & 0x13) | ((l32 & 4) << 1) | ((l32 & 8) >> 1);  // pi(l32)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kaddr[ks] = lds_base + uint32_t(prow * ROWB + (((2 * ks + hb) ^ (l32 & 15)) << 4));
  }

  const uint32_t vaddr = lds_base + uint32_t(VOFF + lane * 16);  // the V^T stages start at VOFF: immediates stay below 64 KB
  // Operand reads take LDS byte addresses (base register + immediate): stage, half step and operand
  // number are compile-time parts of the immediate, so no address arithmetic is issued in the loop.
  using lds_u32x4 = const __attribute__((address_space(3))) u32x4;
  auto lds_ptr = [](uint32_t addr) __attribute__((always_inline)) { return reinterpret_cast<lds_u32x4*>(addr); };

  f32x16 acc[NT];
  // The row's running reference m_run (log2 units of the scaled score; -inf: no key seen yet).
  // l_run: this lane's share (16 of every 32 keys) of the row's sum. p_limit: what a half step's share
  // of the sum may reach before the reference has to move (-1: it has to be set first).
  float m_run = -INFINITY, l_run = 0.0f, p_limit = -1.0f;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[nt][i] = 0.0f;

  // Batch steps past this wavefront's last row hold nothing it can see (plain causal rows).
  const int wave_last = rr0 + min(32 * wave + 31, rows_live - 1);
  auto skipped = [&](int step) {
    const int s0 = 4 * step;
    if (s0 < n_c || seg_max == INT32_MAX) return false;
    return ((a0 + s0 - n_c) << 4) - tree.base > wave_last;
  };

  // A step's matrix work is 4 KS operand reads from LDS, each feeding one matrix instruction:
  // Q K^T of keys 0..31 (KS reads of K), Q K^T of keys 32..63, P V of keys 0..31 (KS reads of
  // V^T), P V of keys 32..63. They run in groups of GP operands through two register buffers:
  // while the matrix cores consume one group, the reads of the next are in flight, and the
  // softmax of a half step sits beside the matrix work of the following group.
  constexpr int GP = 8;           // operands per group
  constexpr int GK = KS / GP;     // groups per half step of Q K^T (and of P V)
  constexpr int NG = 4 * GK;      // groups per step
  f32x16 s[2];                    // S^T of the two half steps: s[kt][4 i + j] is S^T row 8 i + 4 hb + j, which is key
                                  // 32 kt + pi(8 i + 4 hb + j) = 32 kt + 16 (i / 2) + 8 hb + 4 (i % 2) + j of the step
  u32x4 pb[2][2];                 // P^T of the two half steps as matrix operands
  u32x4 ring[2][GP];

  auto read_group = [&]<int S, int G>(u32x4 (&buf)[GP]) __attribute__((always_inline)) {
    if constexpr (G < 2 * GK) {
      constexpr int kt = G / GK, ks0 = (G % GK) * GP;
#pragma unroll
      for (int j = 0; j < GP; ++j) buf[j] = *lds_ptr(kaddr[ks0 + j] + uint32_t(S * KBUF + kt * 32 * ROWB));
    } else {
      // Operand o = 2 nt + t of half step kt: keys 8 hb .. 8 hb + 7 of sub-block 2 kt + t, dims 32 nt .. : the
      // lane's 16 bytes of that sub-block's dim group.
      constexpr int kt = (G - 2 * GK) / GK, o0 = ((G - 2 * GK) % GK) * GP;
#pragma unroll
      for (int j = 0; j < GP; ++j)
        buf[j] = *lds_ptr(vaddr + uint32_t(S * VBUF + 2 * kt * SUBV + ((o0 + j) & 1) * SUBV + ((o0 + j) >> 1) * 1024));
    }
  };
  // Operands [J0, J1) of group G.
  auto mma_group = [&]<int G, int J0, int J1>(const u32x4 (&buf)[GP]) __attribute__((always_inline)) {
    if constexpr (G < 2 * GK) {
      constexpr int kt = G / GK, ks0 = (G % GK) * GP;
      if constexpr (ks0 == 0 && J0 == 0) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kt][i] = 0.0f;
      }
#pragma unroll
      for (int j = J0; j < J1; ++j) s[kt] = mfma32x16<DT>(buf[j], qf[ks0 + j], s[kt]);
    } else {
      constexpr int kt = (G - 2 * GK) / GK, o0 = ((G - 2 * GK) % GK) * GP;
#pragma unroll
      for (int j = J0; j < J1; ++j) acc[(o0 + j) >> 1] = mfma32x16<DT>(buf[j], pb[kt][(o0 + j) & 1], acc[(o0 + j) >> 1]);
    }
  };

  // Online softmax of half step (step, kt) in three parts.
  //   softmax_pre     the masks (nothing on the mask-free path); branchy.
  //   softmax_exp     straight-line: P = exp2(S * scale - m_run), one fused multiply-add and one exponential
  //                   per score, packed to the storage type, and the lane's share of the row sum, taken from
  //                   the packed P two at a time (v_dot2 against (1, 1), fp32 accumulation): the sum is that
  //                   of the rounded P the products use, so O = sum(P~ v) / sum(P~) and a row that one key
  //                   dominates returns that key's V whatever P~ was rounded to. The reference sums the
  //                   unrounded P (kernels/40_attention.metal:292-297) against an exact running maximum,
  //                   where the dominant P is exactly 1 and carries no rounding; under a reference that
  //                   moves lazily the dominant P is any number up to 2^8, and summing the unrounded P would
  //                   leave its rounding (2^-9 relative on bf16) in the output. No maximum is
  //                   taken: all P >= 0, so a share <= 2^8 bounds every one of them, P fits its 16 bits and
  //                   the accumulators need no rescaling. This is the code the scheduler lays between the
  //                   matrix instructions of the next group: one v_exp and one and a half other vector
  //                   instructions per score.
  //   softmax_settle  almost never taken: some lane's share says the reference is too low (or not set: a
  //                   row without one has p_limit = -1). Then the whole wavefront takes the half step's
  //                   maximum, moves the reference, rescales what it has accumulated and redoes the half
  //                   step's P. The two lanes of a row agree on the reference because both take the
  //                   maximum over the pair.
  float corr_late = 1.0f;
  bool late = false;
  auto softmax_pre = [&](int step, auto kt_c, auto interior) __attribute__((always_inline)) {
    constexpr int kt = decltype(kt_c)::value;
    f32x16& sv = s[kt];
    bool half_full = true;  // all 32 keys visible to every row of this wavefront?
    if constexpr (!decltype(interior)::value) {
      const int s0 = 4 * step + 2 * kt;
      if (s0 + 2 <= n_c) {
        const int j0 = (c0 + s0) << 4;
        half_full = j0 >= tile.k0 && j0 + 32 <= tile.k1 && (a.window == 0 || qpos_max - j0 < a.window);
      } else if (s0 >= n_c && s0 + 2 <= n_sb) {
        const int j0 = ((a0 + s0 - n_c) << 4) - tree.base;
        // (j0 + 31 <= k_last matters where the part's batch range ends early: without a cut every row of the tile lies below k_last)
        half_full = !batch_window && j0 >= seg_max && j0 + 31 <= min(rr0 + 32 * wave, k_last) && j0 >= tile.b0 && j0 >= bw_lo;
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
        // Visible keys of the sub-block for this lane's row: j in [lo, hi], or 0 <= j < anc.
        int lo, hi, anc = 0;
        if (cached) {
          lo = tile.k0;
          hi = tile.k1 - 1;
          if (a.window > 0) lo = max(lo, qpos - a.window + 1);
        } else if (batch) {
          // b0 is the first batch key any row of the tile sees (the window's lower edge; 0 without one). The
          // first sub-block starts at a multiple of 16 rows at or below it: what lies below b0 is invisible.
          lo = max(max(d.x, tile.b0), qpos - w_off);
          hi = min(k_last, (a.bidi && d.w > 0) ? max(rr, d.w - 1) : rr);
          anc = min(d.z, k_last + 1);
        } else {
          lo = 1;
          hi = 0;
        }
        // In units of this lane's 8 keys (j = jb + e): e in [ea, ea + ew], one unsigned compare per key;
        // an empty interval becomes ea = 8, ew = 0, which no e in 0 .. 7 satisfies.
        const int jb = j0 + 8 * hb;
        int ea = lo - jb, ew = hi - lo;
        if (ew < 0) {
          ea = 8;
          ew = 0;
        }
        if (batch && (anc_any || batch_window)) {  // ancestors, per-key positions: the rare shapes
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int j = jb + e;
            bool vis = unsigned(e - ea) <= unsigned(ew) || (j >= tile.b0 && j < anc);
            if (batch_window && vis) vis = qpos - a.pos[tree.base + j].x < a.window;
            sv[8 * t + e] = vis ? sv[8 * t + e] : -INFINITY;
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) sv[8 * t + e] = unsigned(e - ea) <= unsigned(ew) ? sv[8 * t + e] : -INFINITY;
        }
      }
    }
    // The lane's maximum over the half step (head dim 256's lazy rescale; see softmax_move).
    float x = -INFINITY;
    if constexpr (!LEAN) {
#pragma unroll
      for (int i = 0; i < 16; ++i) x = fmaxf(x, sv[i]);
      x *= a.scale_log2;  // scale > 0: the max commutes with it
    }
    return x;
  };
  // Lazy rescale: the running reference m_run only moves when some lane's maximum exceeds
  // it by more than 8 (log2 units), so P stays below 2^8 and the accumulators are rescaled
  // a handful of times per row instead of once per step. The two lanes of a row agree on
  // m_run because both take the maximum over the pair whenever either wants to move.
  auto softmax_move = [&](auto kt_c, float x, bool move) __attribute__((always_inline)) {
    constexpr int kt = decltype(kt_c)::value;
    if (move) {
      asm volatile("s_nop 0");  // a real branch: this block must not be speculated into the loop body
      const float m_new = fmaxf(m_run, fmaxf(x, __shfl_xor(x, 32)));
      const float corr = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_run - m_new);
      m_run = m_new;
      l_run *= corr;
      if constexpr (kt == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[nt] *= corr;
      } else {
        // P V of the first half step is still to be accumulated and its P is relative to the old
        // reference: the accumulators take this factor once those products are in.
        corr_late = corr;
        late = true;
      }
    }
  };
  // Head dim 256: the straight-line part with the scale and the reference in one fused multiply-add per score.
  // T0 .. T1: which of the half step's two sub-blocks of 16 keys (8 scores of this lane each) to do now: with
  // two groups of matrix instructions per half step the second sub-block waits for the second group.
  auto softmax_exp_fma = [&]<int T0, int T1>(auto kt_c) __attribute__((always_inline)) {
    constexpr int kt = decltype(kt_c)::value;
    const float m_safe = (m_run == -INFINITY) ? 0.0f : m_run;
    float ps = 0.0f;
#pragma unroll
    for (int t = T0; t < T1; ++t) {
      float p[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) p[e] = fast_exp2(__builtin_fmaf(s[kt][8 * t + e], a.scale_log2, -m_safe));
      pb[kt][t] = u32x4{pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7])};
#pragma unroll
      for (int e = 0; e < 4; ++e) ps = sum2<DT>(pb[kt][t][e], ps);  // the sum of the P the products use (see slice_pack)
      // Pin the results here: without a use in this block the arithmetic above is sunk to the
      // block of its first real use, away from the matrix instructions it should overlap with.
      asm volatile("" : "+v"(pb[kt][t]));
    }
    l_run += ps;
    asm volatile("" : "+v"(l_run));
  };
  // The straight-line part in eight slices, one pair of scores each: slice q subtracts the reference and
  // takes the exponentials of pair q, and packs and sums pair q - 1, whose exponentials have had a slice's
  // time to come back. The caller lays the slices between the matrix instructions itself (the
  // scheduler's grouping hints lumped them behind the first few); finish() packs and sums the last pair.
  float pv[16], ps0 = 0.0f, ps1 = 0.0f, m_sub = 0.0f;
  auto slice_pack = [&]<int KT, int Q>() __attribute__((always_inline)) {
    uint32_t w = pack2<DT>(pv[2 * Q], pv[2 * Q + 1]);
    asm volatile("" : "+v"(w));  // packed here, not sunk to the block of its first use
    pb[KT][Q / 4][Q % 4] = w;
    if constexpr (Q & 1) ps1 = sum2<DT>(w, ps1);
    else ps0 = sum2<DT>(w, ps0);
  };
  auto slice = [&]<int KT, int Q>() __attribute__((always_inline)) {
    if constexpr (Q == 0) {
      ps0 = ps1 = 0.0f;
      m_sub = (m_run == -INFINITY) ? 0.0f : m_run;
    }
    pv[2 * Q] = fast_exp2(__builtin_fmaf(s[KT][2 * Q], a.scale_log2, -m_sub));
    pv[2 * Q + 1] = fast_exp2(__builtin_fmaf(s[KT][2 * Q + 1], a.scale_log2, -m_sub));
    if constexpr (Q > 0) slice_pack.template operator()<KT, Q - 1>();
  };
  auto softmax_finish = [&]<int KT>() __attribute__((always_inline)) -> float {
    slice_pack.template operator()<KT, 7>();
    return ps0 + ps1;
  };
  // The whole straight-line part at once (the rare pass that redoes a half step).
  auto softmax_exp = [&](auto kt_c) __attribute__((always_inline)) -> float {
    constexpr int kt = decltype(kt_c)::value;
    [&]<int... Q>(std::integer_sequence<int, Q...>) __attribute__((always_inline)) {
      (slice.template operator()<kt, Q>(), ...);
    }(std::make_integer_sequence<int, 8>{});
    return softmax_finish.template operator()<kt>();
  };
  auto softmax_settle = [&](auto kt_c, float ps, bool out_of_range) __attribute__((always_inline)) {
    constexpr int kt = decltype(kt_c)::value;
    if (out_of_range) {
      asm volatile("s_nop 0");  // a real branch: this block must not be speculated into the loop body
      f32x16& sv = s[kt];
      mfma_settle(sv);  // the tile's last matrix instruction was issued in another block
      float x = -INFINITY;
#pragma unroll
      for (int i = 0; i < 16; ++i) x = fmaxf(x, sv[i]);
      x *= a.scale_log2;  // scale > 0: the max commutes with it
      const float m_new = fmaxf(m_run, fmaxf(x, __shfl_xor(x, 32)));
      const float corr = (m_run == -INFINITY) ? 1.0f : fast_exp2(m_run - m_new);
      m_run = m_new;
      p_limit = (m_new == -INFINITY) ? -1.0f : 256.0f;
      l_run *= corr;
      if constexpr (kt == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[nt] *= corr;
      } else {
        // P V of the first half step is still to be accumulated and its P is relative to the old
        // reference: the accumulators take this factor once those products are in.
        corr_late = late ? corr_late * corr : corr;
        late = true;
      }
      ps = softmax_exp(kt_c);
    }
    l_run += ps;
  };

  // Phase G of a step: reads of group G + 1, matrix work of group G, and the softmax whose
  // Q K^T finished with the previous group.
  auto phase = [&]<int S, int G>(int step, auto interior) __attribute__((always_inline)) {
    if constexpr (G + 1 < NG) read_group.template operator()<S, G + 1>(ring[(G + 1) & 1]);
    // One wait for the whole group (its GP reads went out a group ago; the GP just issued stay in
    // flight) instead of one in front of every matrix instruction: at one wavefront per SIMD every
    // issued instruction, a wait included, is time the matrix pipe idles.
    __builtin_amdgcn_s_waitcnt(G + 1 < NG ? kWaitLgkm8 : kWaitLgkm0);
    if constexpr (G == GK || G == 2 * GK) {
      if constexpr (LEAN) {
        // On the mask-free path there is no branchy part and the whole group carries the arithmetic.
        constexpr int HEAD = decltype(interior)::value ? 0 : 3;  // (2, 4, 5: equal or slower - measured)
        mma_group.template operator()<G, 0, HEAD>(ring[G & 1]);
        __builtin_amdgcn_sched_barrier(0);
        softmax_pre(step, std::integral_constant<int, G == GK ? 0 : 1>{}, interior);
        __builtin_amdgcn_sched_barrier(0);
        // One matrix instruction, then its share of the eight slices, fenced so that the order stands.
        // The group's last matrix instructions wait until the half step's sum has been compared with its limit:
        // they do not depend on P, and the branch on that comparison - a vector compare that the scalar unit has
        // to wait for - then stands behind matrix instructions in flight instead of behind an idle pipe.
        constexpr int TAILM = 2;  // (1: the same, 3: no gain - measured)
        constexpr int NM = GP - HEAD - TAILM, KT = G == GK ? 0 : 1;
        [&]<int... M>(std::integer_sequence<int, M...>) __attribute__((always_inline)) {
          ([&]<int MI>() __attribute__((always_inline)) {
            mma_group.template operator()<G, HEAD + MI, HEAD + MI + 1>(ring[G & 1]);
            [&]<int... Q>(std::integer_sequence<int, Q...>) __attribute__((always_inline)) {
              (slice.template operator()<KT, (8 * MI) / NM + Q>(), ...);
            }(std::make_integer_sequence<int, (8 * (MI + 1)) / NM - (8 * MI) / NM>{});
            __builtin_amdgcn_sched_barrier(0);
          }.template operator()<M>(), ...);
        }(std::make_integer_sequence<int, NM>{});
        const float ps = softmax_finish.template operator()<KT>();
        const bool out_of_range = __any(!(ps <= p_limit));
        __builtin_amdgcn_sched_barrier(0);
        mma_group.template operator()<G, GP - TAILM, GP>(ring[G & 1]);
        __builtin_amdgcn_sched_barrier(0);
        softmax_settle(std::integral_constant<int, G == GK ? 0 : 1>{}, ps, out_of_range);
      } else {
        // The first matrix instructions of the group go out before the branchy part of the softmax,
        // whose wait for the previous group's results they cover; the rest carry the arithmetic,
        // one matrix instruction then its share.
        // (On steps with masks to work out five go first: 3 -> 5 is 1.3 % on sliding layers, 1 costs as much; 6 as 5.)
        constexpr int HEAD = decltype(interior)::value ? 3 : 5, TAILH = 1;  // (TAILH 0: 1 % slower on full layers, 2: as 1 - measured)
        constexpr std::integral_constant<int, G == GK ? 0 : 1> kt_c{};
        mma_group.template operator()<G, 0, HEAD>(ring[G & 1]);
        __builtin_amdgcn_sched_barrier(0);
        const float x = softmax_pre(step, kt_c, interior);
        const bool move = __any(x > m_run + 8.0f);
        __builtin_amdgcn_sched_barrier(0);
        // (matrix instructions between the comparison and the branch on it, as at head dim 128)
        mma_group.template operator()<G, HEAD, HEAD + TAILH>(ring[G & 1]);
        __builtin_amdgcn_sched_barrier(0);
        softmax_move(kt_c, x, move);
        __builtin_amdgcn_sched_barrier(0);
        mma_group.template operator()<G, HEAD + TAILH, GP>(ring[G & 1]);
        constexpr bool TWO = GK >= 2;  // the half step's Q K^T (or P V) is two groups: the second carries the other half
        softmax_exp_fma.template operator()<0, TWO ? 1 : 2>(kt_c);
#pragma unroll
        for (int j = HEAD + TAILH; j < GP; ++j) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, (TWO ? 35 : 65) / (GP - HEAD - TAILH), 0);
        }
      }
    } else if constexpr (!LEAN && GK >= 2 && (G == GK + 1 || G == 2 * GK + 1)) {
      // the second sub-block's share of the softmax beside the half step's second group of matrix instructions
      __builtin_amdgcn_sched_barrier(0);
      mma_group.template operator()<G, 0, GP>(ring[G & 1]);
      softmax_exp_fma.template operator()<1, 2>(std::integral_constant<int, G == GK + 1 ? 0 : 1>{});
#pragma unroll
      for (int j = 0; j < GP; ++j) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      }
    } else {
      __builtin_amdgcn_sched_barrier(0);
      mma_group.template operator()<G, 0, GP>(ring[G & 1]);
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (G == 3 * GK - 1) {  // P V of the first half step is in: the deferred rescale
      if (late) {
        asm volatile("s_nop 0");
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[nt] *= corr_late;
        late = false;
      }
    }
  };
  auto phases = [&]<int S, int... G>(int step, auto interior, std::integer_sequence<int, G...>) __attribute__((always_inline)) {
    (phase.template operator()<S, G>(step, interior), ...);
  };

  // Steps this wavefront computes: batch steps past its last row hold nothing it can see.
  int my_steps = n_steps;
  while (my_steps > 0 && skipped(my_steps - 1)) --my_steps;

  // At the top of iteration i the barrier that publishes step i has been passed, step i + 1 is
  // on its way into the other stage and the first operand group of step i is being read.
  // The iteration: all groups but the last (reads one group ahead), then - every operand of the
  // step now in registers - wait for the own loads of step i + 1, barrier, request step i + 2
  // into the stage just left, start reading step i + 1, and only then the last group's matrix
  // work: it covers the barrier, the address arithmetic of the loads and the first read latency.
  // interior: every key of steps i .. i + 2 is a cached key inside [k0, k1) that every row of
  // the tile sees: no masks, no edges, one kind of load.
  auto iter = [&]<int S>(int i, auto interior) __attribute__((always_inline)) {
    phases.template operator()<S>(i, interior, std::make_integer_sequence<int, NG - 1>{});
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // loads of step i + 1 landed, reads of stage S done
    if constexpr (!decltype(interior)::value) {
      if (i + 1 < n_steps) fix(i + 1, S ^ 1);
    }
    __syncthreads();
    if (decltype(interior)::value || i + 2 < n_steps) fill(i + 2, S, interior);
    read_group.template operator()<S ^ 1, 0>(ring[0]);
    __builtin_amdgcn_s_waitcnt(kWaitLgkm8);
    __builtin_amdgcn_sched_barrier(0);
    mma_group.template operator()<NG - 1, 0, GP>(ring[(NG - 1) & 1]);
    __builtin_amdgcn_sched_barrier(0);
  };
  // Mask-free steps: every key is one that every row of the tile sees and nothing needs fixing up. Two runs
  // of them: cached steps [int_lo, c_hi) - inside [k0, k1) and inside every row's window - and batch steps
  // [b_lo, b_hi), whose rows all lie below the tile's first row (and at or above b0, inside every segment,
  // with no ancestors and no per-key window test pending). Where the cached range ends on a step boundary
  // the two runs are one. An interior iteration i needs steps i .. i + 2 in one run.
  int int_lo, c_hi, b_lo = 0, b_hi = 0;
  {
    const int first = c0 << 4;  // key of sub-block 0
    int lo_key = tile.k0;
    if (a.window > 0) lo_key = max(lo_key, qpos_max - a.window + 1);
    int_lo = lo_key <= first ? 0 : (lo_key - first + 63) >> 6;
    c_hi = ((tile.k1 >> 4) - c0) >> 2;  // steps wholly inside the cached range
    if (n_b > 0 && !batch_window && !anc_any && seg_max != INT32_MAX) {
      const int lo_b = max(max(max(tile.b0, seg_max), bw_lo), 0);
      const int g_lo = (tree.base + lo_b + 15) >> 4;           // first group of 16 rows wholly at or above lo_b
      const int g_hi = min(((tree.base + rr0) >> 4), ((tree.base + k_last + 1) >> 4)) - 1;  // last group wholly below the tile's first row (and inside the part's batch range)
      const int s_lo = n_c + g_lo - a0, s_hi = n_c + g_hi - a0;  // as sub-blocks of the range
      b_lo = (s_lo + 3) >> 2;
      b_hi = max(b_lo, (s_hi + 1) >> 2);
      if (b_lo == c_hi && (n_c & 3) == 0 && (tile.k1 & 15) == 0 && c_hi > int_lo) {  // one run
        c_hi = b_hi;
        b_lo = b_hi = 0;
      }
    }
  }
  constexpr std::false_type general{};
  constexpr std::true_type inner{};

  if (n_steps > 0) {
    if (!early) fill(0, 0, general);
    wait_loads();
    fix(0, 0);
  }
  __syncthreads();
  if (n_steps > 1) fill(1, 1, general);
  read_group.template operator()<0, 0>(ring[0]);
  __builtin_amdgcn_sched_barrier(0);
  // Pairs of steps (one per stage): general ones up to the first mask-free run, that run, general ones,
  // the second run, general ones again. The general stretches share one loop's code, and so do the runs.
  const int even_steps = my_steps & ~1;
  const int a_hi = min(c_hi - 2, my_steps), bb_hi = min(b_hi - 2, my_steps);  // interior iterations end two steps short of a run
  const int in0 = min((int_lo + 1) & ~1, even_steps);
  const int in1 = a_hi > in0 ? in0 + ((a_hi - in0) & ~1) : in0;
  const int in2 = max(in1, min((b_lo + 1) & ~1, even_steps));
  const int in3 = bb_hi > in2 ? in2 + ((bb_hi - in2) & ~1) : in2;
  int i = 0;
#pragma nounroll
  for (int seg = 0; seg < 3; ++seg) {
    const int bound = seg == 0 ? in0 : (seg == 1 ? in2 : my_steps);
#pragma nounroll
    for (; i + 2 <= bound; i += 2) {
      iter.template operator()<0>(i, general);
      iter.template operator()<1>(i + 1, general);
    }
    if (seg < 2) {
      const int end = seg == 0 ? in1 : in3;
#pragma nounroll
      for (; i + 2 <= end; i += 2) {
        iter.template operator()<0>(i, inner);
        iter.template operator()<1>(i + 1, inner);
      }
    }
  }
  if (i < my_steps) {
    iter.template operator()<0>(i, general);
    ++i;
  }
  for (; i < n_steps; ++i) {  // keep staging for the wavefronts whose rows reach further
    wait_loads();
    if (i + 1 < n_steps) fix(i + 1, (i + 1) & 1);
    __syncthreads();
    if (i + 2 < n_steps) fill(i + 2, i & 1, general);
  }

  // ---- output: lane (row l32, half hb) holds dims 32 nt + 8 i + 4 hb + j at acc[nt][4 i + j]
  const float l = l_run + __shfl_xor(l_run, 32);
  if (!row_ok) return;
  if (tile.part >= 0) {
    const size_t rec = (size_t(tile.part) * a.Hkv + kvh) * a.cols + size_t(m_row) * a.G + hg;
    float* po = a.parts_o + rec * HD;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        *reinterpret_cast<f32x4*>(po + 32 * nt + 8 * i4 + 4 * hb) =
            f32x4{acc[nt][4 * i4], acc[nt][4 * i4 + 1], acc[nt][4 * i4 + 2], acc[nt][4 * i4 + 3]};
    if (hb == 0) {
      a.parts_ml[rec * 2] = m_run;
      a.parts_ml[rec * 2 + 1] = l;
    }
    return;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  uint16_t* op = a.O + size_t(row) * a.q_ld + size_t(h) * HD;
  const float* gp = a.gate ? a.gate + size_t(row) * a.gate_ld + size_t(h) * a.gate_hs + a.gate_off : nullptr;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int dd = 32 * nt + 8 * i4 + 4 * hb;
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        o[j] = acc[nt][4 * i4 + j] * inv;
        if (gp) o[j] = o[j] / (1.0f + __expf(-gp[(dd + j) * a.gate_ds]));
      }
      *reinterpret_cast<u32x2*>(op + dd) = u32x2{pack2<DT>(o[0], o[1]), pack2<DT>(o[2], o[3])};
    }
}

// Workgroups per compute unit and the largest tile each variant takes.
constexpr int tiled_occ(int HD) { return HD == 128 ? 2 : 1; }
int tiled_max_rows(int HD) { return HD == 512 ? 64 : 128; }  // 512: attn_tiled512_kernel's 2 row groups x 2 dim halves
int tiled_workgroups_per_cu(int HD) { return tiled_occ(HD); }
size_t tiled_smem_bytes(int HD) { return size_t(4) * 64 * HD * 2 + 64; }  // two stages of K (64 rows) and V^T (64 keys), 16 ints

template <int DT, int HD>
static hipError_t launch_tiled_t(const KArgs& a, int n_tiles, hipStream_t st) {
  const size_t smem = tiled_smem_bytes(HD);
  constexpr auto k = attn_tiled_kernel<DT, HD, tiled_occ(HD)>;
  const hipError_t e = allow_dynamic_lds<k>(smem);
  if (e != hipSuccess) return e;
  launch_timed(k, dim3(unsigned(n_tiles) * a.H), dim3(256), smem, st, a, n_tiles);
  return hipGetLastError();
}

hipError_t launch_tiled512(int dt, const KArgs& a, int n_tiles, hipStream_t st);

// The dynamic LDS limit of every variant on the current device, ahead of the first launch.
hipError_t tiled_init_attributes() {
  hipError_t e = allow_dynamic_lds<attn_tiled_kernel<ESP_F16, 128, tiled_occ(128)>>(tiled_smem_bytes(128));
  if (e == hipSuccess) e = allow_dynamic_lds<attn_tiled_kernel<ESP_F16, 256, tiled_occ(256)>>(tiled_smem_bytes(256));
  if (e == hipSuccess) e = allow_dynamic_lds<attn_tiled_kernel<ESP_BF16, 128, tiled_occ(128)>>(tiled_smem_bytes(128));
  if (e == hipSuccess) e = allow_dynamic_lds<attn_tiled_kernel<ESP_BF16, 256, tiled_occ(256)>>(tiled_smem_bytes(256));
  return e;
}

hipError_t launch_tiled(int dt, int HD, const KArgs& a, int n_tiles, hipStream_t st) {
  if (HD == 512 && (dt == ESP_F16 || dt == ESP_BF16)) return launch_tiled512(dt, a, n_tiles, st);
  if (dt == ESP_F16 && HD == 128) return launch_tiled_t<ESP_F16, 128>(a, n_tiles, st);
  if (dt == ESP_F16 && HD == 256) return launch_tiled_t<ESP_F16, 256>(a, n_tiles, st);
  if (dt == ESP_BF16 && HD == 128) return launch_tiled_t<ESP_BF16, 128>(a, n_tiles, st);
  if (dt == ESP_BF16 && HD == 256) return launch_tiled_t<ESP_BF16, 256>(a, n_tiles, st);
  return hipErrorInvalidValue;
}

}  // namespace esp
