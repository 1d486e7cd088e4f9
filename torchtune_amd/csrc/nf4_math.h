// Scalar arithmetic shared by the NF4 kernels.  Everything here compiles for the host as well as for
// gfx950, so the rounding rules can be tested exhaustively on a CPU.
//
// The eager reference performs every step of to_nf4 / get_original_weight in the weight's own dtype
// (torchao NF4Tensor, called from torchtune/modules/peft/lora.py:86 and
// torchtune/modules/low_precision/nf4_linear.py:49).  For bfloat16 that means: compute in fp32, round to
// nearest-even bf16 after every single operation.  `Arith<BF16>::rnd` is that rounding step.
#pragma once
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define TT_HD __host__ __device__ __forceinline__
#else
#define TT_HD inline
#endif

namespace ttamd {

// The 16 NormalFloat4 code points (QLoRA paper, table in appendix E); each is exactly representable in fp32.
#define TT_NF4_TABLE                                                                                              \
  {-1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f, -0.28444138169288635f,              \
   -0.18477343022823334f, -0.09105003625154495f, 0.0f, 0.07958029955625534f, 0.16093020141124725f,               \
   0.24611230194568634f, 0.33791524171829224f, 0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f,  \
   1.0f}

TT_HD uint32_t f32_bits(float f) {
  uint32_t u;
#if defined(__HIP_DEVICE_COMPILE__)
  u = __builtin_bit_cast(uint32_t, f);
#else
  memcpy(&u, &f, 4);
#endif
  return u;
}
TT_HD float bits_f32(uint32_t u) {
  float f;
#if defined(__HIP_DEVICE_COMPILE__)
  f = __builtin_bit_cast(float, u);
#else
  memcpy(&f, &u, 4);
#endif
  return f;
}

// fp32 -> bf16 bit pattern, round to nearest even, NaN stays a (quiet) NaN.
TT_HD uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
TT_HD float bf16_bits_to_f32(uint16_t b) { return bits_f32(((uint32_t)b) << 16); }

// fp32 value rounded to bf16 precision, returned as fp32.
TT_HD float round_to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (float)(__bf16)f;  // v_cvt_pk_bf16_f32: round to nearest even
#else
  return bf16_bits_to_f32(f32_to_bf16_bits(f));
#endif
}

template <bool BF16>
struct Arith {
  static TT_HD float rnd(float f) { return BF16 ? round_to_bf16(f) : f; }
};

// Index of the NF4 code nearest to `scaled` under the reference's rule: distances |scaled - nf4[j]| are
// computed and rounded in the tensor dtype, and the FIRST minimum wins (torch.argmin over dim=-1).
// `scaled` must already be rounded to the dtype.  NaN (0/0 from an all-zero block) yields index 0, the
// position torch.argmin reports for an all-NaN row.
template <bool BF16>
TT_HD int nf4_nearest_code(float scaled) {
  const float tab[16] = TT_NF4_TABLE;
  int best = 0;
  float bestd = __builtin_fabsf(Arith<BF16>::rnd(scaled - Arith<BF16>::rnd(tab[0])));
#pragma unroll
  for (int j = 1; j < 16; ++j) {
    float d = __builtin_fabsf(Arith<BF16>::rnd(scaled - Arith<BF16>::rnd(tab[j])));
    if (d < bestd) {  // strict: ties keep the lower index; NaN never wins
      bestd = d;
      best = j;
    }
  }
  return best;
}

// Dequantised value of one block scaler: (int8 / factor) rounded to dtype, plus mean, rounded again.
template <bool BF16>
TT_HD float nf4_block_scaler(int q, float factor, float mean) {
  float s = Arith<BF16>::rnd((float)q / factor);
  return Arith<BF16>::rnd(s + mean);
}

}  // namespace ttamd
