// The SwiGLU gate and its backward on two packed bf16 pairs, shared by the stand-alone kernels (neighbours.hip) and the
// epilogues of the GEMMs around them (nf4_gemm_dense.hip) so that both produce the same bits:
//   a = bf16(g * sigmoid(g)) (F.silu in bf16), out = bf16(a * u)     torchtune/modules/feed_forward.py:50-53
//   backward, what autograd derives for those two bf16 ops from the gradient o of out:
//     grad u = bf16(o * a),  grad g = bf16(bf16(o * u) * silu'(g)),  silu'(g) = s * (1 + g * (1 - s)), s = sigmoid(g)
#pragma once
#include <stdint.h>

#include "nf4_math.h"

namespace ttamd {

#if defined(__HIPCC__)
__device__ __forceinline__ float sigmoid_f(float g) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
}

// g2, u2: two bf16 values each (low half first) -> the two products, packed the same way
__device__ __forceinline__ uint32_t swiglu_gate_pair(uint32_t g2, uint32_t u2) {
  typedef __bf16 pair_t __attribute__((ext_vector_type(2)));
  const float g0 = bits_f32(g2 << 16), g1 = bits_f32(g2 & 0xffff0000u);
  const float a0 = round_to_bf16(g0 * sigmoid_f(g0)), a1 = round_to_bf16(g1 * sigmoid_f(g1));
  pair_t v;
  v.x = (__bf16)(a0 * bits_f32(u2 << 16));
  v.y = (__bf16)(a1 * bits_f32(u2 & 0xffff0000u));
  return __builtin_bit_cast(uint32_t, v);
}

// o2, g2, u2: two bf16 values each of grad out, gate and up -> the two packed pairs grad gate, grad up
__device__ __forceinline__ void swiglu_bwd_pair(uint32_t o2, uint32_t g2, uint32_t u2, uint32_t& gg2, uint32_t& gu2) {
  typedef __bf16 pair_t __attribute__((ext_vector_type(2)));
  float rg[2], ru[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const float gval = e ? bits_f32(g2 & 0xffff0000u) : bits_f32(g2 << 16);
    const float uval = e ? bits_f32(u2 & 0xffff0000u) : bits_f32(u2 << 16);
    const float oval = e ? bits_f32(o2 & 0xffff0000u) : bits_f32(o2 << 16);
    const float s = sigmoid_f(gval);
    const float a = round_to_bf16(gval * s);
    ru[e] = oval * a;
    const float ga = round_to_bf16(oval * uval);
    rg[e] = ga * (s * (1.0f + gval * (1.0f - s)));
  }
  pair_t vg, vu;
  vg.x = (__bf16)rg[0]; vg.y = (__bf16)rg[1];
  vu.x = (__bf16)ru[0]; vu.y = (__bf16)ru[1];
  gg2 = __builtin_bit_cast(uint32_t, vg);
  gu2 = __builtin_bit_cast(uint32_t, vu);
}
#endif

}  // namespace ttamd
