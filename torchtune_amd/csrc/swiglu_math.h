// The SwiGLU gate on two packed bf16 pairs, shared by the stand-alone kernel (neighbours.hip) and the epilogue of the
// gate / up GEMM (nf4_gemm_dense.hip) so that both produce the same bits:
//   a = bf16(g * sigmoid(g)) (F.silu in bf16), out = bf16(a * u)     torchtune/modules/feed_forward.py:50-53
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
#endif

}  // namespace ttamd
