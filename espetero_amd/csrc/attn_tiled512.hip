// Tiled MFMA attention at head dim 512: prefill and chunked prefill of the
// full-attention layers whose heads are 512 wide (the reference's
// g4_attention512_s{1,2,4,8}, kernels/80_gemma.metal:157-342, :355-358).
//
// Semantics as in the tiled kernel of the narrower heads: cached keys [k0, k1)
// through the block table or ring, then the tree's batch keys (`last` tiles) under
// the tree mask (80_:284) and the window (80_:285), online softmax in fp32, P
// rounded to the storage type before P.V, output O / l (0 when no key is visible)
// with the optional sigmoid gate, or a partial record for the merge.
//
// Mapping to gfx950. A 512-dim head does not fit one wavefront (32 rows x 512 dims
// of fp32 accumulators alone are 256 registers), so a workgroup is one tile of up to
// 64 query rows x one query head, and its 4 wavefronts are 2 row groups x 2 dim
// halves: wavefront (rg, dh) owns rows 32 rg .. and dims 256 dh .. of them. Keys
// advance in steps of 32 (two 16-key sub-blocks). Per step a wavefront computes
//   S^T[32 keys][32 rows] over its 256 dims    v_mfma_f32_32x32x16, A = K from LDS, B = Q^T in registers
//   the two halves of a row group meet in LDS and are added in one order on both sides
//   (the reference sums its per-simdgroup score partials the same way, 80_:272-282)
//   P^T = exp2(S^T - m)                         identical in both wavefronts of the pair
//   O^T[256 dims][32 rows] += V^T . P^T         A = V^T (its 256 dims) from LDS
// The next step travels global memory -> the other LDS stage with global_load_lds_dwordx4
// (no staging registers) while the current step is in the matrix cores.
//
// LDS layout: K of stage 0, K of stage 1, V^T of stage 0, V^T of stage 1 (an operand read is a per-lane base
// register plus an immediate, which takes 16 bits: with a stage's K and V^T side by side the second stage would lie
// beyond it and every read of it would cost an addition). K of a stage: 32 rows of 1024 bytes, unpadded; the 16-byte chunk c of row r
// lies at chunk position c ^ (pi(r) & 15), pi = swap of row bits 2 and 3. The lane with S^T
// row l reads key row pi(l) at position c ^ (l & 15): 16 consecutive lanes hit 16 different
// positions, and with the rows permuted by pi the 8 P values a lane packs for one P.V
// instruction are 8 consecutive keys, which is how V^T lies in memory. V^T per sub-block:
// [dim][2 halves of 8 keys], the two 16-byte halves of dim d swapped when bit 3 of d is set
// (lanes d and d + 8 of an operand read would otherwise share banks).
#include <utility>

#include "common.hpp"
#include "lds_direct.hpp"

namespace esp {

namespace {
constexpr int kHD = 512, kHW = 256;                  // dims of a head; dims one wavefront multiplies and accumulates
constexpr int kKStage = 32 * kHD * 2;                // K of one stage: 32 rows
constexpr int kVSub = kHD * 32;                      // V^T of one sub-block
constexpr int kVStage = 2 * kVSub;                   // V^T of one stage: two sub-blocks
constexpr int kVBase = 2 * kKStage;                  // layout: K stage 0, K stage 1, V^T stage 0, V^T stage 1 - every operand read is
                                                     // a per-lane base plus an immediate below 64 KB, whichever the stage
constexpr int kStage = kKStage + kVStage;
constexpr int kXch = 4 * 4 * 64 * 16;                // partial S^T: [wavefront][4][lane] 16-byte pieces
constexpr int kLds = 2 * kStage + kXch + 64;         // two stages, the exchange, 16 ints
}  // namespace

template <int DT>
__global__ __launch_bounds__(256, 1) void attn_tiled512_kernel(const KArgs a, int n_tiles) {
  constexpr int KS = kHW / 16, NT = kHW / 32;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  f32x4* xch = reinterpret_cast<f32x4*>(lds + 2 * kStage);
  int(*red)[4] = reinterpret_cast<int(*)[4]>(lds + 2 * kStage + kXch);

  // Workgroup -> (KV head, head in group, tile): consecutive ids differ in KV head first, the heads
  // sharing a KV head land on the same XCD's L2; tiles run last to first (longest key ranges first).
  const int kvh = blockIdx.x % a.Hkv;
  const int rest = blockIdx.x / a.Hkv;
  const int hg = rest % a.G;
  const int tile_i = n_tiles - 1 - rest / a.G;
  const int h = kvh * a.G + hg;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rg = wave >> 1, dw = (wave & 1) * kHW;
  const int l32 = lane & 31, hb = lane >> 5;
  esp_tile tile = a.tiles[tile_i];
  const esp_tree tree = a.trees[tile.tree];
  if (tile.k1 == INT32_MAX) tile.k1 = tree.P;  // open-ended range: up to the tree's cached length as it is now
  const int table = tile.pad > 0 ? tile.pad - 1 : tree.table;
  const int end = tree.base + tree.M;
  const int rows_live = min(a.R, end - tile.r0);
  const int rr0 = tile.r0 - tree.base;

  // ---- this lane's row and its Q fragments (this wavefront's dims)
  const int m_row = 32 * rg + l32;
  const bool row_ok = m_row < rows_live;
  const int row = row_ok ? tile.r0 + m_row : tile.r0;
  const int rr = rr0 + m_row;
  const int4 d = a.desc ? a.desc[row] : make_int4(0, 0, 0, 0);
  const int qpos = a.window > 0 ? a.pos[row].x : 0;
  u32x4 qf[KS];
  {
    const uint16_t* qp = a.Q + size_t(row) * a.q_ld + size_t(h) * kHD + dw + 8 * hb;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = row_ok ? *reinterpret_cast<const u32x4*>(qp + 16 * ks) : u32x4{0, 0, 0, 0};
  }

  // ---- the last batch key any row of the tile sees
  int k_last = -1;
  {
    int kl = row_ok ? max(rr, max(d.z - 1, a.bidi ? d.w - 1 : -1)) : -1;
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) kl = max(kl, __shfl_xor(kl, o));
    if (lane == 0) red[wave][0] = kl;
    __syncthreads();
    k_last = max(max(red[0][0], red[1][0]), max(red[2][0], red[3][0]));
    k_last = __builtin_amdgcn_readfirstlane(min(min(k_last, tree.M - 1), tile.last >= 2 ? tile.last - 2 : INT32_MAX));  // last >= 2: the part's batch range ends at row last - 2
  }

  // ---- the key range as 16-key sub-blocks: cached [k0, k1), then batch rows [b0, k_last]
  const int c0 = tile.k0 >> 4;
  const int n_c = tile.k1 > tile.k0 ? ((tile.k1 + 15) >> 4) - c0 : 0;
  const int a0 = (tree.base + tile.b0) >> 4;  // batch sub-blocks are groups of 16 absolute rows
  const int n_b = (tile.last && k_last >= tile.b0) ? ((tree.base + k_last) >> 4) - a0 + 1 : 0;
  const int n_sb = n_c + n_b;
  const int n_steps = (n_sb + 1) >> 1;
  const int n_groups = (a.n_rows + 15) >> 4;
  // Batch rows in the pool (no Kb / Vb): row j of a tree lies at position P + j of the tree's block list, P - base a
  // multiple of 16: a batch sub-block of 16 absolute rows is one 16-token sub-block of the pool, staged like a cached one.
  const bool in_pool = a.Kb == nullptr;
  const int pool_shift = tree.P - tree.base;

  // ---- staging, 16 bytes per lane straight into LDS. K: this wavefront brings rows 4 wave .. + 3 of each
  // sub-block; the lane that fills chunk position `lane` of row r brings chunk lane ^ (pi(r) & 15), and
  // pi(4 wave + q) = pi(4 wave) + q. V^T: this wavefront brings pieces 256 wave .. + 255 of each sub-block's
  // 1024 (piece c: keys 8 (c % 2) .. + 7 of dim c / 2); position p holds piece p ^ ((p >> 4) & 1).
  const uint32_t lds_base = uint32_t(uintptr_t(lds));
  // Pool addresses of the sub-blocks, 64 at a time: lane l holds the byte address of the K rows of sub-block adr0 + l
  // (block list entry, the head's place in the block, the sub-block's place in the head, worked out by 64 lanes at
  // once), so that in front of a sub-block's staging loads stand two lane reads instead of a dependent memory access
  // and the scalar arithmetic behind it. V^T of a sub-block lies bt rows' worth of bytes behind its K rows.
  uint32_t kadr_lo = 0, kadr_hi = 0;
  int adr0 = -(1 << 30);
  auto pool_k = [&](int sidx) __attribute__((always_inline)) {
    if (sidx < adr0 || sidx >= adr0 + 64) {
      adr0 = sidx;
      const int sl = sidx + lane;
      const int js = sl < n_c ? (c0 + sl) << 4 : (in_pool && sl < n_sb) ? ((a0 + sl - n_c) << 4) + pool_shift : -1;
      uint64_t adr = 0;
      if (js >= 0) {
        const int b = block_of(a, table, js);
        adr = reinterpret_cast<uint64_t>(a.pool + head_base(a, kHD, b, kvh)) + uint64_t(js % a.bt) * 1024;
      }
      kadr_lo = uint32_t(adr);
      kadr_hi = uint32_t(adr >> 32);
    }
    const int idx = sidx - adr0;
    const uint32_t lo = uint32_t(__builtin_amdgcn_readlane(int(kadr_lo), idx)), hi = uint32_t(__builtin_amdgcn_readlane(int(kadr_hi), idx));
    return reinterpret_cast<const char*>(uint64_t(lo) | (uint64_t(hi) << 32));
  };
  const uint32_t kx = uint32_t(swap23(4 * wave));
  const uint32_t voff = uint32_t((lane ^ ((lane >> 4) & 1)) << 4);
  // plain: the caller knows that both sub-blocks of the step are cached keys.
  auto fill = [&](int step, int stage, auto plain) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int sidx = 2 * step + t;
      const uint32_t kdst = lds_base + stage * kKStage + (16 * t + 4 * wave) * 1024;
      const uint32_t vdst = lds_base + kVBase + stage * kVStage + t * kVSub + wave * 4096;
      const uint32_t kl = uint32_t(lane);
      if (decltype(plain)::value || sidx < n_c || (in_pool && sidx < n_sb)) {
        const char* kb = pool_k(sidx) + wave * 4096;
        const char* vb = kb + size_t(a.bt) * 1024;  // the 16-token sub-block: 16 KB contiguous
        load_to_lds16_x4(kb, (kl ^ kx) << 4, (kl ^ (kx + 1)) << 4, (kl ^ (kx + 2)) << 4, (kl ^ (kx + 3)) << 4, kdst);
        load_to_lds16_x4(vb, voff, voff, voff, voff, vdst);
      } else if (sidx < n_sb) {
        const int g = a0 + (sidx - n_c);
        const int lim = a.n_rows - 1 - 16 * g;  // batch rows past the pass's last row do not exist: repeat the last (masked)
        const char* kb = reinterpret_cast<const char*>(a.Kb + size_t(16 * g) * a.kv_ld + size_t(kvh) * kHD);
        const char* vb = reinterpret_cast<const char*>(a.vt_stage + (size_t(kvh) * n_groups + g) * size_t(kHD) * 16) + wave * 4096;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          load_to_lds16(kb + size_t(min(4 * wave + q, lim)) * size_t(a.kv_ld) * 2, (kl ^ (kx + q)) << 4, kdst + q * 1024);
        load_to_lds16_x4(vb, voff, voff, voff, voff, vdst);
      } else {  // past the range: K stays whatever it was (S is masked), V^T must be finite
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<u32x4*>(lds + kVBase + stage * kVStage + t * kVSub + wave * 4096 + q * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
      }
    }
  };
  // After this wavefront's loads of `step` have landed: cached keys outside [k0, k1) may be memory
  // never written; their V must not reach the products.
  auto fix = [&](int step, int stage) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int sidx = 2 * step + t;
      // keys [v0, v1) of the sub-block's own numbering are memory that has been written: the tile's cached range,
      // or, for batch rows read from the pool, everything up to the tree's last row
      int j0, v0, v1;
      if (sidx < n_c) {
        j0 = (c0 + sidx) << 4;
        v0 = tile.k0;
        v1 = tile.k1;
      } else if (in_pool && sidx < n_sb) {
        j0 = ((a0 + sidx - n_c) << 4) - tree.base;
        v0 = INT32_MIN;
        v1 = tree.M;
      } else {
        continue;
      }
      if (j0 >= v0 && j0 + 16 <= v1) continue;
      const int jv = j0 + 8 * ((lane & 1) ^ ((lane >> 4) & 1));  // the half of the piece at this lane's position
      u32x4 msk;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool lo = jv + 2 * e >= v0 && jv + 2 * e < v1;
        const bool hi = jv + 2 * e + 1 >= v0 && jv + 2 * e + 1 < v1;
        msk[e] = (lo ? 0xffffu : 0u) | (hi ? 0xffff0000u : 0u);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        u32x4* p = reinterpret_cast<u32x4*>(lds + kVBase + stage * kVStage + t * kVSub + wave * 4096 + q * 1024 + lane * 16);
        *p = *p & msk;
      }
    }
  };

  // ---- operand reads: LDS byte addresses (base register + immediate)
  using lds_u32x4 = const __attribute__((address_space(3))) u32x4;
  auto lds_ptr = [](uint32_t addr) __attribute__((always_inline)) { return reinterpret_cast<lds_u32x4*>(addr); };
  // K slice ks = 8 g + j of this wavefront's dims is chunk dw / 8 + 16 g + 2 j + hb of key row pi(l32).
  uint32_t kaddr[8];
  {
    const int prow = (l32 & 0x13) | ((l32 & 4) << 1) | ((l32 & 8) >> 1);  // pi(l32)
#pragma unroll
    for (int j = 0; j < 8; ++j) kaddr[j] = lds_base + uint32_t(prow * 1024 + dw * 2 + (((2 * j + hb) ^ (l32 & 15)) << 4));
  }
  // V^T operand nt of sub-block t: keys 8 hb .. + 7 of dim dw + 32 nt + l32.
  const uint32_t vaddr = lds_base + uint32_t(kVBase + (dw + l32) * 32 + ((hb ^ ((l32 >> 3) & 1)) << 4));

  f32x16 acc[NT];
  float m_run = -INFINITY, l_run = 0.0f;  // l_run: this lane's share (16 of every 32 keys) of the row's sum
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[nt][i] = 0.0f;

  // A step's matrix work is 32 operand reads from LDS, each feeding one matrix instruction, in 4 groups of 8
  // through two register buffers: K slices 0..7, K slices 8..15, V^T of sub-block 0, V^T of sub-block 1.
  // The reads of a group are in flight while the matrix cores consume the group before it; the V^T reads
  // do not depend on the softmax and cover the exchange of the partial scores.
  //
  // At the top of iteration i stage i % 2 holds step i, step i + 1 is on its way into the other stage and
  // the first group of K slices of step i is being read. The iteration: both score groups, the exchange,
  // the softmax - its second sub-block's share laid between the first sub-block's P V instructions - then,
  // every operand of the step now in registers, the wait for the own loads of step i + 1, the barrier that
  // publishes them, the request for step i + 2 into the stage just left, the first reads of step i + 1, and
  // only then the second sub-block's P V instructions: they cover the barrier, the address arithmetic of the
  // loads and the first read latency. (A wavefront issues in order: a matrix instruction hides only what
  // stands right behind it.)
  u32x4 ring[2][8];
  auto read_k0 = [&]<int S>(std::integral_constant<int, S>) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[0][j] = *lds_ptr(kaddr[j] + uint32_t(S * kKStage));
  };
  // plain: steps `step` .. `step + 2` are cached keys wholly inside [k0, k1) of a layer without a window: every key is
  // visible to every row, nothing staged needs fixing up, one kind of load.
  auto iter = [&]<int S>(int step, std::integral_constant<int, S>, auto plain) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[1][j] = *lds_ptr(kaddr[j] + uint32_t(S * kKStage + 256));
    __builtin_amdgcn_sched_barrier(0);
    // s[4 i + j] is S^T row 8 i + 4 hb + j, which is key 16 (i / 2) + 8 hb + 4 (i % 2) + j of the step:
    // s[8 t + e] is key 8 hb + e of sub-block t.
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) s = mfma32x16<DT>(ring[0][j], qf[j], s);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[0][j] = *lds_ptr(vaddr + uint32_t(S * kVStage + j * 1024));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; ++j) s = mfma32x16<DT>(ring[1][j], qf[8 + j], s);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; ++j) ring[1][j] = *lds_ptr(vaddr + uint32_t(S * kVStage + kVSub + j * 1024));
    // The other half of the dims: through LDS, added in the same order in both wavefronts of the pair.
#pragma unroll
    for (int v = 0; v < 4; ++v) xch[(wave * 4 + v) * 64 + lane] = f32x4{s[4 * v], s[4 * v + 1], s[4 * v + 2], s[4 * v + 3]};
    __syncthreads();
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const f32x4 o = xch[((wave ^ 1) * 4 + v) * 64 + lane];
#pragma unroll
      for (int j = 0; j < 4; ++j) s[4 * v + j] = (wave & 1) ? o[j] + s[4 * v + j] : s[4 * v + j] + o[j];
    }
    // ---- visibility
#pragma unroll
    for (int t = 0; t < (decltype(plain)::value ? 0 : 2); ++t) {
      const int sidx = 2 * step + t;
      const bool cached = sidx < n_c, batch = !cached && sidx < n_sb;
      const int j0 = cached ? (c0 + sidx) << 4 : ((a0 + sidx - n_c) << 4) - tree.base;
      if (cached && a.window == 0 && j0 >= tile.k0 && j0 + 16 <= tile.k1) continue;  // every key visible to every row
      // Visible keys of the sub-block for this lane's row: j in [lo, hi], or 0 <= j < anc.
      int lo, hi, anc = 0;
      if (cached) {
        lo = tile.k0;
        hi = tile.k1 - 1;
        if (a.window > 0) lo = max(lo, qpos - a.window + 1);
      } else if (batch) {
        lo = max(d.x, tile.b0);  // below b0 (the window's lower edge over the tile's rows) nothing is visible
        hi = min(k_last, (a.bidi && d.w > 0) ? max(rr, d.w - 1) : rr);
        anc = min(d.z, k_last + 1);
      } else {
        lo = 1;
        hi = 0;
      }
      const int jb = j0 + 8 * hb;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = jb + e;
        bool vis = (j >= lo && j <= hi) || (j >= tile.b0 && j < anc);
        if (batch && a.window > 0 && vis) vis = qpos - a.pos[tree.base + j].x < a.window;
        s[8 * t + e] = vis ? s[8 * t + e] : -INFINITY;
      }
    }
    // ---- online softmax; the two lanes of a row (hb = 0, 1) agree on the maximum. The running reference
    // m_run only moves when some row's maximum exceeds it by more than 8 (log2 units): P stays below
    // 2^8 and the 128 accumulator registers are rescaled a handful of times per row.
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[i]);
    mx *= a.scale_log2;  // scale > 0: the max commutes with it
    if (__any(mx > m_run + 8.0f)) {
      const float m_new = fmaxf(m_run, fmaxf(mx, __shfl_xor(mx, 32)));
      const float corr = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_run - m_new);  // m_run = -inf -> 0: nothing accumulated yet
      l_run *= corr;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) acc[nt] *= corr;
      m_run = m_new;
    }
    const float m_safe = (m_run == -INFINITY) ? 0.0f : m_run;
    u32x4 pb[2];
    float ps = 0.0f;
    // The row sum is that of the rounded P the products use: under a lazily moved reference the dominant P is
    // not exactly 1, and O = sum(P~ v) / sum(P~) keeps its rounding out of a row that one key dominates.
    auto exp_pack = [&]<int T>(std::integral_constant<int, T>) __attribute__((always_inline)) {
      float p[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) p[e] = fast_exp2(__builtin_fmaf(s[8 * T + e], a.scale_log2, -m_safe));
      pb[T] = u32x4{pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7])};
#pragma unroll
      for (int e = 0; e < 4; ++e) ps = sum2<DT>(pb[T][e], ps);
    };
    exp_pack(std::integral_constant<int, 0>{});
    __builtin_amdgcn_sched_barrier(0);
    // ---- O^T += V^T . P^T over this wavefront's dims: the first sub-block's products, the second sub-block's
    // exponentials between them
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = mfma32x16<DT>(ring[0][nt], pb[0], acc[nt]);
    exp_pack(std::integral_constant<int, 1>{});
    asm volatile("" : "+v"(pb[1]), "+v"(ps));  // worked out here, not where pb[1] is first used
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    l_run += ps;
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // own loads of step + 1 landed, own reads of stage S done
    if constexpr (decltype(plain)::value) {
      __syncthreads();
      fill(step + 2, S, plain);
      read_k0(std::integral_constant<int, S ^ 1>{});
    } else {
      if (step + 1 < n_steps) fix(step + 1, S ^ 1);
      __syncthreads();
      if (step + 2 < n_steps) fill(step + 2, S, plain);
      if (step + 1 < n_steps) read_k0(std::integral_constant<int, S ^ 1>{});
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = mfma32x16<DT>(ring[1][nt], pb[1], acc[nt]);
    __builtin_amdgcn_sched_barrier(0);
  };
  constexpr std::false_type general{};
  constexpr std::true_type plain{};
  if (n_steps > 0) {
    fill(0, 0, general);
    wait_loads();
    fix(0, 0);
  }
  __syncthreads();
  if (n_steps > 1) fill(1, 1, general);
  if (n_steps > 0) read_k0(std::integral_constant<int, 0>{});
  {
    // Plain iterations: pairs of steps i, i + 1 whose steps up to i + 3 are sub-blocks wholly inside the cached range.
    int p0 = 0, p1 = 0;  // iterations [p0, p1), both even
    if (a.window == 0 && n_c > 0) {
      const int sb_lo = (tile.k0 & 15) ? 1 : 0, sb_hi = n_c - ((tile.k1 & 15) ? 1 : 0);  // sub-blocks [sb_lo, sb_hi) are whole
      p0 = (((sb_lo + 1) >> 1) + 1) & ~1;
      const int last = (sb_hi >> 1) - 3;  // last iteration i with 2 (i + 2) + 1 < sb_hi
      p1 = last >= p0 ? p0 + ((last + 1 - p0) & ~1) : p0;
    }
    int i = 0;
#pragma nounroll
    for (; i + 2 <= min(p0, n_steps); i += 2) {
      iter(i, std::integral_constant<int, 0>{}, general);
      iter(i + 1, std::integral_constant<int, 1>{}, general);
    }
    if (i == p0) {
#pragma nounroll
      for (; i + 2 <= p1; i += 2) {
        iter(i, std::integral_constant<int, 0>{}, plain);
        iter(i + 1, std::integral_constant<int, 1>{}, plain);
      }
    }
#pragma nounroll
    for (; i + 2 <= n_steps; i += 2) {
      iter(i, std::integral_constant<int, 0>{}, general);
      iter(i + 1, std::integral_constant<int, 1>{}, general);
    }
    if (i < n_steps) iter(i, std::integral_constant<int, 0>{}, general);
  }

  // ---- output: lane (row l32, half hb) holds dims dw + 32 nt + 8 i + 4 hb + j at acc[nt][4 i + j]
  const float l = l_run + __shfl_xor(l_run, 32);
  if (!row_ok) return;
  if (tile.part >= 0) {
    const size_t rec = (size_t(tile.part) * a.Hkv + kvh) * a.cols + size_t(m_row) * a.G + hg;
    float* po = a.parts_o + rec * kHD + dw;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4)
        *reinterpret_cast<f32x4*>(po + 32 * nt + 8 * i4 + 4 * hb) =
            f32x4{acc[nt][4 * i4], acc[nt][4 * i4 + 1], acc[nt][4 * i4 + 2], acc[nt][4 * i4 + 3]};
    if (hb == 0 && dw == 0) {
      a.parts_ml[rec * 2] = m_run;
      a.parts_ml[rec * 2 + 1] = l;
    }
    return;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  uint16_t* op = a.O + size_t(row) * a.q_ld + size_t(h) * kHD + dw;
  const float* gp = a.gate ? a.gate + size_t(row) * a.gate_ld + size_t(h) * a.gate_hs + a.gate_off + dw * a.gate_ds : nullptr;
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

// The dynamic LDS limit of both variants on the current device, ahead of the first launch.
hipError_t tiled512_init_attributes() {
  const hipError_t e = allow_dynamic_lds<attn_tiled512_kernel<ESP_F16>>(kLds);
  return e != hipSuccess ? e : allow_dynamic_lds<attn_tiled512_kernel<ESP_BF16>>(kLds);
}

hipError_t launch_tiled512(int dt, const KArgs& a, int n_tiles, hipStream_t st) {
  constexpr auto kf = attn_tiled512_kernel<ESP_F16>;
  constexpr auto kb = attn_tiled512_kernel<ESP_BF16>;
  const hipError_t e = dt == ESP_F16 ? allow_dynamic_lds<kf>(kLds) : allow_dynamic_lds<kb>(kLds);
  if (e != hipSuccess) return e;
  launch_timed(dt == ESP_F16 ? kf : kb, dim3(unsigned(n_tiles) * a.H), dim3(256), size_t(kLds), st, a, n_tiles);
  return hipGetLastError();
}

}  // namespace esp
