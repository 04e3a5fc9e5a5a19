// The arithmetic of attn_prep for one lane's share of one (row, head), shared by the prep kernel and by
// the streaming attention kernel's fused prologue so that both give the same bits: RMSNorm over the head
// (queries and keys with the learned weight, values without), rotary embedding of the leading rope_dims
// dims in the half-split pairing, the query scale (kernels/40_attention.metal:23-102,
// kernels/80_gemma.metal:63-108, kernels/82_qwen3_omni.metal:39-88).
// A head is HD / prep_epl(HD) consecutive lanes of one wavefront, aligned to that count; lane i of the
// head holds dims prep_epl * i ..; every lane of the head must call (the sums and the rotation's partner
// are lane exchanges).
#pragma once

#include "common.hpp"

namespace esp {

constexpr int prep_epl(int HD) { return HD > 256 ? 8 : 4; }

// x: the lane's dims of the fp32 projection, rewritten in place. kind: 0 query, 1 key, 2 value.
// w: the norm weight of those dims (unused for values). cs: (cos, sin) per frequency of this row.
template <int HD>
__device__ __forceinline__ void prep_lane(float (&x)[prep_epl(HD)], int kind, const float (&w)[prep_epl(HD)], const float2* cs,
                                          const esp_prep_params& p, int d0) {
  // Two kernels inline this function and must agree to the bit, so nothing here is left to the compiler's
  // choice of which multiply to fuse with which add: the fused operations are spelled out, the rest stays apart.
#pragma clang fp contract(off)
  constexpr int EPL = prep_epl(HD), LPH = HD / EPL;
  const int half = p.rope_dims / 2;
  if (kind != 2 || p.v_norm) {
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < EPL; ++i) ss = __builtin_fmaf(x[i], x[i], ss);
#pragma unroll
    for (int o = LPH / 2; o >= 1; o >>= 1) ss += __shfl_xor(ss, o);
    const float inv = rsqrtf(ss / float(HD) + p.eps);
#pragma unroll
    for (int i = 0; i < EPL; ++i) x[i] = kind == 2 ? x[i] * inv : x[i] * inv * w[i];
  }
  if (kind != 2 && half > 0) {
    // The partner of dim d < half is d + half: half / EPL lanes away. Every lane of the head takes
    // part in the exchange; only the rotating dims use it.
    const bool lower = d0 < half;
#pragma unroll
    for (int i = 0; i < EPL; ++i) {
      const float partner = __shfl_xor(x[i], half / EPL);
      if (d0 < p.rope_dims) {
        const float2 t = cs[(lower ? d0 : d0 - half) + i];
        const float turned = partner * t.y;
        x[i] = __builtin_fmaf(x[i], t.x, lower ? -turned : turned);
      }
    }
  }
  if (kind == 0) {
#pragma unroll
    for (int i = 0; i < EPL; ++i) x[i] *= p.q_scale;
  }
}

// (cos, sin) of one row's rotation angles: frequency f turns by position component rope_sel[f] (x when
// there is no selector) times inv_freq[f].
__device__ __forceinline__ float2 prep_cos_sin(const int4 pr, const int32_t* rope_sel, const float* inv_freq, int f) {
  const int sel = rope_sel ? rope_sel[f] : 0;
  const float position = float(sel == 0 ? pr.x : (sel == 1 ? pr.y : pr.z));
  float sn, c;
  sincosf(position * inv_freq[f], &sn, &c);
  return make_float2(c, sn);
}

}  // namespace esp
