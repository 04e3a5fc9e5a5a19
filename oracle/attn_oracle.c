/* attn_oracle.c -- CPU restatement of the reference's paged-KV attention.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the product (espetero_amd/, include/)
 * links, loads or calls this file; it is the checker the parity tests and the
 * bench's cpu_baseline leg compare the HIP path against.
 *
 * Scalar C, fp32 accumulation, fp16 / bf16 storage emulated by bit-exact
 * round-to-nearest-even conversions. The KV pool is in the REFERENCE's block
 * layout  kv_base + (2 b + which) * bt * kv_ld + t * kv_ld + h * HD + d
 * (kernels/40_attention.metal:245-247), not the product's native layout.
 *
 * What follows which reference lines:
 *   esp_oracle_attn_direct   the semantics of one call stated row by row:
 *                            visible cached keys 80_gemma.metal:283-285 (40_:281),
 *                            page address 40_:245-247 / ring 80_:250, batch-key
 *                            tree mask 80_:284 (40_:104-113, :282), window 80_:285,
 *                            softmax with fp32 l and P rounded to the storage
 *                            type before P.V 40_:286-317, O/l and l == 0 -> 0
 *                            40_:334, sigmoid gate 40_:335-341.
 *   esp_oracle_attn_tiles    the same through the kernels' structure: tiles of
 *                            rows_per_tile rows, 16-key blocks, online softmax
 *                            (80_:226-322), block skipping of the batch range
 *                            (80_:218-239), partial records (80_:324-336) and
 *                            the split merge attention_combine (40_:811-864,
 *                            80_:568-597).
 *   esp_oracle_kv_save       40_:875-889.   esp_oracle_kv_copy_blocks  40_:894-905.
 *   esp_oracle_kv_gather     the page walk alone (40_:245-247).
 *   esp_oracle_attn_prep     the prep kernels, one (row, head) at a time: attn_prep
 *                            40_:41-101, g4_attn_prep 80_:76-107, q3m_attn_prep
 *                            82_:52-87 (norm, weight, half-split rotation, query
 *                            scale, value cast / weightless norm, folded append
 *                            into the reference-layout pool 40_:86-100).
 *
 *   esp_oracle_head_gate     sp_head_gate 85_spark.metal:108-128: the fp32 dot of the
 *                            row's input with the head's gate row, the sigmoid, and
 *                            O rounded a second time after the product.
 *
 * esp_oracle_head_gate is pinned in tests/test_gate.py by closed forms (x == 0 halves
 * O exactly, a one-hot gate row gives sigmoid of one input element, a saturated
 * dot leaves O or clears it) and by a float64 restatement; its summation order
 * (left to right) is not the reference's (strided partial sums, 85_:121-122), so
 * gates agree to fp32 rounding and outputs to one unit in the last place.
 *
 * esp_oracle_attn_prep is pinned by a float64 restatement of the closed forms
 * (RMSNorm, rotation matrix) in tests/test_prep.py, by norm preservation of the
 * rotation, by position 0 == no rotation, and by the folded append == kv_save of
 * the outputs. Its cos / sin are libm's on the fp32 angle the kernels form; the
 * reference's precise::cos / sin and rsqrt are not bit-reproducible here, so
 * outputs agree to one unit in the last place of the storage type, not bit for bit.
 *
 * Pinned by tests/test_oracle.py: float64 brute force on gathered K/V, torch
 * CPU scaled_dot_product_attention, closed forms (V == 1, single key, equal
 * keys, q == 0, fully masked row), split invariance, window >= context ==
 * causal, page-permutation invariance. The reference holds no golden vectors
 * for this path; the exp() it uses is Metal fast-math and the MMA summation
 * order is not reproducible on a CPU, so last-ulp equality with the Metal
 * kernels is not claimed: the contract is max-abs 2e-3.
 */
#include "../include/espetero_attn.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---- storage conversions (round to nearest even) ---- */
float esp_oracle_h2f(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = -1;
      do {
        ++e;
        man <<= 1;
      } while (!(man & 0x400u));
      bits = sign | (uint32_t)(127 - 15 - e) << 23 | (man & 0x3ffu) << 13;
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | man << 13;
  } else {
    bits = sign | (exp + 112u) << 23 | man << 13;
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t esp_oracle_f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* rounds to inf */
  if (x < 0x33000001u) return sign;                        /* below half the smallest subnormal */
  if (x < 0x38800000u) {                                   /* subnormal half */
    const int shift = 126 - (int)(x >> 23);               /* 14..24 */
    const uint32_t man = (x & 0x7fffffu) | 0x800000u;
    uint32_t r = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (r & 1u))) ++r;
    return (uint16_t)(sign | r);
  }
  uint32_t r = (x - 0x38000000u) >> 13;
  const uint32_t rem = x & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) ++r;
  return (uint16_t)(sign | r);
}

float esp_oracle_bf2f(uint16_t b) {
  const uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t esp_oracle_f2bf(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

static inline float ld(const esp_attn_params* p, const uint16_t* a, size_t i) {
  return p->dtype == ESP_BF16 ? esp_oracle_bf2f(a[i]) : esp_oracle_h2f(a[i]);
}
static inline uint16_t st(const esp_attn_params* p, float f) {
  return p->dtype == ESP_BF16 ? esp_oracle_f2bf(f) : esp_oracle_f2h(f);
}
static inline float rnd(const esp_attn_params* p, float f) { return ld(p, (uint16_t[]){st(p, f)}, 0); }

/* Address (element index) of cached key j of a tree, head kvh, K (which 0) or V (1):
 * 40_:245-247, ring form 80_:250. */
static inline size_t cached_addr(const esp_attn_params* p, const int32_t* blocks, const esp_tree* t, int j, int which,
                                 int kvh) {
  const size_t blk = (size_t)p->bt * (size_t)p->kv_ld;
  const size_t b = p->ring ? (size_t)(t->table + (j / p->bt) % p->ring) : (size_t)blocks[t->table + j / p->bt];
  return (size_t)p->kv_base + (b * 2 + (size_t)which) * blk + (size_t)(j % p->bt) * (size_t)p->kv_ld +
         (size_t)kvh * (size_t)p->head_dim;
}

/* Is batch key j (relative row) visible to relative row rr with descriptor d = desc[row]? 80_:284-285. */
static inline int batch_visible(const esp_attn_params* p, const int32_t* d, const int32_t* pos, const esp_tree* t, int rr,
                                int j) {
  const int seg = d ? d[0] : 0, anc = d ? d[2] : 0, img = d ? d[3] : 0;
  int vis = (j < anc) || (j >= seg && (j <= rr || (p->bidi && j < img)));
  if (p->window > 0 && vis) vis = pos[4 * (t->base + rr)] - pos[4 * (t->base + j)] < p->window;
  return vis;
}
static inline int cached_visible(const esp_attn_params* p, const int32_t* pos, int row, int j) {
  return p->window > 0 ? pos[4 * row] - j < p->window : 1;
}

static inline float gate_of(const esp_attn_params* p, int row, int h, int d) {
  if (!p->gate) return 1.0f;
  const float g = p->gate[(size_t)row * p->gate_ld + (size_t)h * p->gate_hs + p->gate_off + (p->gate_headwise ? 0 : d)];
  return 1.0f / (1.0f + expf(-g));
}

/* ---- the call, row by row ---- */
int esp_oracle_attn_direct(const esp_attn_params* p, const uint16_t* Q, const uint16_t* Kb, const uint16_t* Vb,
                           const uint16_t* pool, const int32_t* blocks, const int32_t* desc, const int32_t* pos,
                           uint16_t* O, const esp_tree* trees, int n_trees, int n_threads) {
  const int HD = p->head_dim, G = p->H / p->Hkv;
  if (n_threads < 1) n_threads = 1;
  long n_units = 0;
  for (int t = 0; t < n_trees; ++t) n_units += (long)trees[t].M * p->Hkv;
  /* unit = (tree, row, kv head); prefix sums to find the tree of a unit */
  long* first = (long*)malloc(sizeof(long) * (size_t)(n_trees + 1));
  first[0] = 0;
  for (int t = 0; t < n_trees; ++t) first[t + 1] = first[t] + (long)trees[t].M * p->Hkv;
#pragma omp parallel num_threads(n_threads)
  {
    int cap = 0;
    const uint16_t **kp = NULL, **vp = NULL;
    float* s = NULL;
    float* acc = (float*)malloc(sizeof(float) * (size_t)HD);
    int ti = 0;
#pragma omp for schedule(dynamic, 1)
    for (long u = 0; u < n_units; ++u) {
      while (ti > 0 && u < first[ti]) --ti;
      while (u >= first[ti + 1]) ++ti;
      const esp_tree* t = &trees[ti];
      const int rr = (int)((u - first[ti]) / p->Hkv), kvh = (int)((u - first[ti]) % p->Hkv);
      const int row = t->base + rr;
      const int32_t* d = desc ? desc + 4 * row : NULL;
      if (t->P + t->M > cap) {
        cap = t->P + t->M;
        kp = (const uint16_t**)realloc((void*)kp, sizeof(void*) * (size_t)cap);
        vp = (const uint16_t**)realloc((void*)vp, sizeof(void*) * (size_t)cap);
        s = (float*)realloc(s, sizeof(float) * (size_t)cap);
      }
      int n = 0;
      for (int j = 0; j < t->P; ++j)
        if (cached_visible(p, pos, row, j)) {
          kp[n] = pool + cached_addr(p, blocks, t, j, 0, kvh);
          vp[n] = pool + cached_addr(p, blocks, t, j, 1, kvh);
          ++n;
        }
      for (int j = 0; j < t->M; ++j)
        if (batch_visible(p, d, pos, t, rr, j)) {
          kp[n] = Kb + (size_t)(t->base + j) * p->kv_ld + (size_t)kvh * HD;
          vp[n] = Vb + (size_t)(t->base + j) * p->kv_ld + (size_t)kvh * HD;
          ++n;
        }
      for (int hg = 0; hg < G; ++hg) {
        const int h = kvh * G + hg;
        const uint16_t* q = Q + (size_t)row * p->q_ld + (size_t)h * HD;
        float m = -INFINITY;
        for (int i = 0; i < n; ++i) {
          float a = 0.0f;
          for (int x = 0; x < HD; ++x) a += ld(p, q, x) * ld(p, kp[i], x);
          s[i] = a * p->scale;
          if (s[i] > m) m = s[i];
        }
        float l = 0.0f;
        for (int x = 0; x < HD; ++x) acc[x] = 0.0f;
        for (int i = 0; i < n; ++i) {
          const float pv = expf(s[i] - m);
          l += pv;
          const float pr = rnd(p, pv);
          for (int x = 0; x < HD; ++x) acc[x] += pr * ld(p, vp[i], x);
        }
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        uint16_t* o = O + (size_t)row * p->q_ld + (size_t)h * HD;
        for (int x = 0; x < HD; ++x) o[x] = st(p, acc[x] * inv * gate_of(p, row, h, x));
      }
    }
    free((void*)kp);
    free((void*)vp);
    free(s);
    free(acc);
  }
  free(first);
  return 0;
}

/* ---- the call through tiles, partial records and the merge ----
 * parts: float [n_parts][Hkv][rows_per_tile][G][HD + 2] (80_:324-336 with 8 -> rows_per_tile). */
#define OBK 16
int esp_oracle_attn_tiles(const esp_attn_params* p, const uint16_t* Q, const uint16_t* Kb, const uint16_t* Vb,
                          const uint16_t* pool, const int32_t* blocks, const int32_t* desc, const int32_t* pos,
                          uint16_t* O, const esp_tile* tiles, int n_tiles, const esp_tree* trees, int n_trees,
                          const esp_combine* jobs, int n_jobs, float* parts) {
  (void)n_trees;
  const int HD = p->head_dim, G = p->H / p->Hkv, R = p->rows_per_tile, RS = HD + 2;
  float* acc = (float*)malloc(sizeof(float) * (size_t)HD);
  for (int ti = 0; ti < n_tiles; ++ti) {
    const esp_tile* tile = &tiles[ti];
    const esp_tree* t = &trees[tile->tree];
    const int end = t->base + t->M;
    const int r_last = (tile->r0 + R - 1 < end - 1 ? tile->r0 + R - 1 : end - 1) - t->base;
    int anc_max = 0, seg_min = 1 << 30, k_last = r_last;
    for (int r = tile->r0; r <= t->base + r_last; ++r) {
      const int32_t* dr = desc ? desc + 4 * r : NULL;
      const int z = dr ? dr[2] : 0, x = dr ? dr[0] : 0, w = dr ? dr[3] : 0;
      if (z > anc_max) anc_max = z;
      if (x < seg_min) seg_min = x;
      if (p->bidi && w - 1 > k_last) k_last = w - 1;
    }
    if (anc_max - 1 > k_last) k_last = anc_max - 1; /* noncausal roots, 40_:220 */
    /* a part whose batch range is cut (this library's balanced planner; the reference never does): rows b0 .. last - 2 */
    if (tile->last >= 2 && tile->last - 2 < k_last) k_last = tile->last - 2;
    const int n_slot_blocks = (tile->k1 - tile->k0 + OBK - 1) / OBK;
    const int bb0 = tile->last ? tile->b0 / OBK : 0;
    int n_batch_blocks = tile->last ? (k_last + OBK) / OBK - bb0 : 0;
    if (n_batch_blocks < 0) n_batch_blocks = 0;
    for (int kvh = 0; kvh < p->Hkv; ++kvh)
      for (int row = tile->r0; row < tile->r0 + R && row < end; ++row) {
        const int rr = row - t->base;
        const int32_t* d = desc ? desc + 4 * row : NULL;
        for (int hg = 0; hg < G; ++hg) {
          const int h = kvh * G + hg;
          const uint16_t* q = Q + (size_t)row * p->q_ld + (size_t)h * HD;
          float m_run = -INFINITY, l_run = 0.0f;
          for (int x = 0; x < HD; ++x) acc[x] = 0.0f;
          for (int blk = 0; blk < n_slot_blocks + n_batch_blocks; ++blk) {
            const int in_slot = blk < n_slot_blocks;
            const int j0 = in_slot ? tile->k0 + blk * OBK : (bb0 + blk - n_slot_blocks) * OBK;
            const int j_end = in_slot ? tile->k1 : k_last + 1;
            if (!in_slot) {
              const int anc_vis = j0 < anc_max;
              const int own_vis = (j0 + OBK - 1 >= seg_min) && (j0 <= k_last);
              if (!anc_vis && !own_vis) continue;
            }
            float sv[OBK];
            const uint16_t* vrow[OBK];
            float mx = -INFINITY;
            for (int kc = 0; kc < OBK; ++kc) {
              const int j = j0 + kc;
              int vis = j < j_end && (in_slot || j >= tile->b0); /* below b0 no row of the tile sees anything */
              if (vis) vis = in_slot ? cached_visible(p, pos, row, j) : batch_visible(p, d, pos, t, rr, j);
              sv[kc] = -INFINITY;
              vrow[kc] = NULL;
              if (!vis) continue;
              const uint16_t* k = in_slot ? pool + cached_addr(p, blocks, t, j, 0, kvh)
                                          : Kb + (size_t)(t->base + j) * p->kv_ld + (size_t)kvh * HD;
              vrow[kc] = in_slot ? pool + cached_addr(p, blocks, t, j, 1, kvh)
                                 : Vb + (size_t)(t->base + j) * p->kv_ld + (size_t)kvh * HD;
              float a = 0.0f;
              for (int x = 0; x < HD; ++x) a += ld(p, q, x) * ld(p, k, x);
              sv[kc] = a * p->scale;
              if (sv[kc] > mx) mx = sv[kc];
            }
            const float m_new = m_run > mx ? m_run : mx;
            const float corr = (m_new == -INFINITY) ? 1.0f : expf(m_run - m_new);
            float ps = 0.0f;
            for (int x = 0; x < HD; ++x) acc[x] *= corr;
            for (int kc = 0; kc < OBK; ++kc) {
              const float pv = (m_new == -INFINITY || !vrow[kc]) ? 0.0f : expf(sv[kc] - m_new);
              ps += pv;
              if (!vrow[kc]) continue;
              const float pr = rnd(p, pv);
              for (int x = 0; x < HD; ++x) acc[x] += pr * ld(p, vrow[kc], x);
            }
            l_run = l_run * corr + ps;
            m_run = m_new;
          }
          if (tile->part >= 0) {
            float* rec = parts + ((((size_t)tile->part * p->Hkv + kvh) * R + (size_t)(row - tile->r0)) * G + hg) * RS;
            memcpy(rec, acc, sizeof(float) * (size_t)HD);
            rec[HD] = m_run;
            rec[HD + 1] = l_run;
          } else {
            const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
            uint16_t* o = O + (size_t)row * p->q_ld + (size_t)h * HD;
            for (int x = 0; x < HD; ++x) o[x] = st(p, acc[x] * inv * gate_of(p, row, h, x));
          }
        }
      }
  }
  for (int ji = 0; ji < n_jobs; ++ji) {
    const esp_combine* job = &jobs[ji];
    for (int r = 0; r < job->rows; ++r)
      for (int h = 0; h < p->H; ++h) {
        const int kvh = h / G, hg = h % G;
        float M = -INFINITY, L = 0.0f;
        for (int s = 0; s < job->nparts; ++s) {
          const float* rec = parts + ((((size_t)(job->part0 + s) * p->Hkv + kvh) * R + r) * G + hg) * RS;
          if (rec[HD] > M) M = rec[HD];
        }
        for (int x = 0; x < HD; ++x) acc[x] = 0.0f;
        for (int s = 0; s < job->nparts; ++s) {
          const float* rec = parts + ((((size_t)(job->part0 + s) * p->Hkv + kvh) * R + r) * G + hg) * RS;
          const float w = (rec[HD] == -INFINITY) ? 0.0f : expf(rec[HD] - M);
          L += w * rec[HD + 1];
          for (int x = 0; x < HD; ++x) acc[x] += w * rec[x];
        }
        const float inv = L > 0.0f ? 1.0f / L : 0.0f;
        const int row = job->r0 + r;
        uint16_t* o = O + (size_t)row * p->q_ld + (size_t)h * HD;
        for (int x = 0; x < HD; ++x) o[x] = st(p, acc[x] * inv * gate_of(p, row, h, x));
      }
  }
  free(acc);
  return 0;
}

/* ---- pool writes and the page walk (reference layout) ---- */
void esp_oracle_kv_save(const esp_attn_params* p, const uint16_t* Kb, const uint16_t* Vb, uint16_t* pool,
                        const esp_kvsave* e, int n) {
  const size_t blk = (size_t)p->bt * (size_t)p->kv_ld;
  const size_t w = (size_t)p->Hkv * p->head_dim;
  for (int i = 0; i < n; ++i) {
    uint16_t* dst = pool + p->kv_base + (size_t)e[i].block * 2 * blk + (size_t)e[i].pos * p->kv_ld;
    memcpy(dst, Kb + (size_t)e[i].src_row * p->kv_ld, 2 * w);
    memcpy(dst + blk, Vb + (size_t)e[i].src_row * p->kv_ld, 2 * w);
  }
}

void esp_oracle_kv_copy_blocks(const esp_attn_params* p, uint16_t* pool, const int32_t* pairs, int n_pairs, int n_layers,
                               uint64_t region_elems) {
  const size_t blk2 = 2 * (size_t)p->bt * (size_t)p->kv_ld;
  for (int l = 0; l < n_layers; ++l)
    for (int i = 0; i < n_pairs; ++i)
      memcpy(pool + (size_t)l * region_elems + (size_t)pairs[2 * i + 1] * blk2,
             pool + (size_t)l * region_elems + (size_t)pairs[2 * i] * blk2, 2 * blk2);
}

void esp_oracle_kv_gather(const esp_attn_params* p, const uint16_t* pool, const int32_t* blocks, int n_tokens,
                          uint16_t* K_out, uint16_t* V_out) {
  const esp_tree t = {0, n_tokens, 0, 0};
  const size_t w = (size_t)p->Hkv * p->head_dim;
  esp_attn_params q = *p;
  q.ring = 0;
  for (int j = 0; j < n_tokens; ++j) {
    memcpy(K_out + (size_t)j * w, pool + cached_addr(&q, blocks, &t, j, 0, 0), 2 * w);
    memcpy(V_out + (size_t)j * w, pool + cached_addr(&q, blocks, &t, j, 1, 0), 2 * w);
  }
}

/* ---- attn_prep ---- */
static inline uint16_t st_dt(int dtype, float f) { return dtype == ESP_F16 ? esp_oracle_f2h(f) : esp_oracle_f2bf(f); }

void esp_oracle_attn_prep(const esp_prep_params* p, const float* X, const float* qn_w, const float* kn_w, const int32_t* pos,
                          const float* inv_freq, const int32_t* rope_sel, uint16_t* Q, uint16_t* Kb, uint16_t* Vb,
                          const int32_t* row_table, uint16_t* pool_ref, int n_rows) {
  const int HD = p->head_dim, half = p->rope_dims / 2;
  float* x = (float*)malloc(sizeof(float) * (size_t)HD);
  float* y = (float*)malloc(sizeof(float) * (size_t)HD);
  for (int row = 0; row < n_rows; ++row) {
    const float* xr = X + (size_t)row * p->x_ld;
    for (int slot = 0; slot < p->H + 2 * p->Hkv; ++slot) {
      const int kind = slot < p->H ? 0 : (slot < p->H + p->Hkv ? 1 : 2);
      const int h = kind == 0 ? slot : (kind == 1 ? slot - p->H : slot - p->H - p->Hkv);
      const float* src = xr + (kind == 0 ? p->q_off + h * p->q_hs : (kind == 1 ? p->k_off : p->v_off) + h * HD);
      float ss = 0.0f;
      for (int d = 0; d < HD; ++d) {
        x[d] = src[d];
        ss += x[d] * x[d];
      }
      const float inv = 1.0f / sqrtf(ss / (float)HD + p->eps);
      if (kind == 2) {
        for (int d = 0; d < HD; ++d) y[d] = p->v_norm ? x[d] * inv : x[d];
      } else {
        const float* nw = kind == 0 ? qn_w : kn_w;
        for (int d = 0; d < HD; ++d) x[d] = x[d] * inv * nw[d];
        for (int d = 0; d < HD; ++d) y[d] = x[d];
        for (int f = 0; f < half; ++f) {
          const int sel = rope_sel ? rope_sel[f] : 0;
          const float position = (float)pos[4 * row + (sel == 0 ? 0 : (sel == 1 ? 1 : 2))];
          const float ang = position * inv_freq[f];
          const float c = cosf(ang), sn = sinf(ang);
          y[f] = x[f] * c - x[f + half] * sn;
          y[f + half] = x[f + half] * c + x[f] * sn;
        }
        if (kind == 0)
          for (int d = 0; d < HD; ++d) y[d] *= p->q_scale;
      }
      uint16_t* out = kind == 0 ? Q + (size_t)row * p->q_ld + (size_t)h * HD
                                : (kind == 1 ? Kb : Vb) + (size_t)row * p->kv_ld + (size_t)h * HD;
      for (int d = 0; d < HD; ++d) out[d] = st_dt(p->dtype, y[d]);
      if (kind != 0 && row_table) {
        const size_t blk = (size_t)p->bt * p->kv_ld;
        for (int w = 0; w < 2; ++w) {
          const int b = row_table[4 * row + 2 * w], ps = row_table[4 * row + 2 * w + 1];
          if (b < 0) continue;
          uint16_t* dst = pool_ref + p->kv_base + (size_t)b * 2 * blk + (kind == 2 ? blk : 0) + (size_t)ps * p->kv_ld + (size_t)h * HD;
          memcpy(dst, out, sizeof(uint16_t) * (size_t)HD);
        }
      }
    }
  }
  free(x);
  free(y);
}

/* ---- sp_head_gate ---- */
void esp_oracle_head_gate(const esp_gate_params* p, uint16_t* O, const uint16_t* X, const uint16_t* Wg, float* dots, int n_rows) {
  for (int row = 0; row < n_rows; ++row)
    for (int h = 0; h < p->H; ++h) {
      const uint16_t* x = X + (size_t)row * p->x_ld;
      const uint16_t* w = Wg + (size_t)h * p->D;
      float acc = 0.0f;
      for (int i = 0; i < p->D; ++i)
        acc += (p->dtype == ESP_F16 ? esp_oracle_h2f(x[i]) : esp_oracle_bf2f(x[i])) *
               (p->dtype == ESP_F16 ? esp_oracle_h2f(w[i]) : esp_oracle_bf2f(w[i]));
      if (dots) dots[(size_t)row * p->H + h] = acc;
      if (!O) continue;
      const float g = 1.0f / (1.0f + expf(-acc));
      uint16_t* o = O + (size_t)row * p->q_ld + (size_t)h * p->head_dim;
      for (int d = 0; d < p->head_dim; ++d)
        o[d] = st_dt(p->dtype, (p->dtype == ESP_F16 ? esp_oracle_h2f(o[d]) : esp_oracle_bf2f(o[d])) * g);
    }
}
