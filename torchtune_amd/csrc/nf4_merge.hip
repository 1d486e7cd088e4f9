// Dequantise an NF4 weight and fold the LoRA update into it in one pass:
//
//     out[n][k] = bf16( D(W)[n][k] + bf16( scale * bf16( sum_r B[n][r] * A[r][k] ) ) )
//
// which is the rounding sequence of the eager checkpoint path: the state-dict hook first turns the NF4 weight into
// a bf16 tensor (torchtune/modules/common_utils.py:55-59), then get_merged_lora_ckpt adds
// `(alpha / rank) * lora_b @ lora_a` in bf16 (torchtune/modules/peft/_utils.py:264-266).  The rank-r sum is
// accumulated in fp32 in ascending r with fused multiply-adds.
//
// HBM-bound: 0.5625 B/element read (codes + fp32 block scalers), 2 B/element written.  A workgroup owns a strip of
// 2048 columns and 16 rows: each lane keeps A[0..R)[its 8 columns] in registers for all rows of the strip, so the
// adapter matrices are read from L2 once per workgroup, not once per output.
#include "common.h"
#include "nf4_math.h"

namespace ttamd {
namespace {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __constant__ float kNF4Merge[16] = TT_NF4_TABLE;

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  bf16x2_t v;
  v.x = (__bf16)lo;
  v.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}

constexpr int kRowsPerWg = 16;

template <int R8>  // rank / 8
__global__ __launch_bounds__(256) void nf4_dequant_merge_kernel(const uint32_t* __restrict__ qdata,
                                                                const float* __restrict__ block_scalers,
                                                                const uint16_t* __restrict__ A,
                                                                const uint16_t* __restrict__ B, float scale, int N, int K,
                                                                uint16_t* __restrict__ out) {
  constexpr int R = 8 * R8;
  __shared__ float2 lut[256];
  __shared__ float bsh[kRowsPerWg][R];
  const int t = threadIdx.x;
  lut[t] = make_float2(round_to_bf16(kNF4Merge[t >> 4]), round_to_bf16(kNF4Merge[t & 15]));
  const int n0 = blockIdx.y * kRowsPerWg;
  for (int i = t; i < kRowsPerWg * R; i += 256) {
    const int n = n0 + i / R;
    bsh[i / R][i % R] = n < N ? bf16_bits_to_f32(B[(int64_t)n * R + i % R]) : 0.f;
  }
  const int k = blockIdx.x * 2048 + t * 8;
  const bool live = k < K;  // K % 8 == 0
  // adapter columns of this lane, as packed bf16 pairs: a[r][d] = (A[r][k + 2d], A[r][k + 2d + 1])
  u32x4_t a[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    a[r] = u32x4_t{0, 0, 0, 0};
    if (live) a[r] = *reinterpret_cast<const u32x4_t*>(A + (int64_t)r * K + k);
  }
  __syncthreads();
  if (!live) return;
  for (int i = 0; i < kRowsPerWg; ++i) {
    const int n = n0 + i;
    if (n >= N) break;
    const int64_t e = (int64_t)n * K + k;
    const uint32_t code = __builtin_nontemporal_load(qdata + (e >> 3));
    const float sc = block_scalers[e >> 6];
    float m[8];
#pragma unroll
    for (int d = 0; d < 8; ++d) m[d] = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float b = bsh[i][r];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        m[2 * d] = __builtin_fmaf(b, bits_f32(a[r][d] << 16), m[2 * d]);
        m[2 * d + 1] = __builtin_fmaf(b, bits_f32(a[r][d] & 0xffff0000u), m[2 * d + 1]);
      }
    }
    u32x4_t o;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const float2 pr = lut[(code >> (8 * d)) & 0xffu];
      const float w0 = round_to_bf16(pr.x * sc), w1 = round_to_bf16(pr.y * sc);
      const float u0 = round_to_bf16(scale * round_to_bf16(m[2 * d])), u1 = round_to_bf16(scale * round_to_bf16(m[2 * d + 1]));
      o[d] = pack2(w0 + u0, w1 + u1);
    }
    __builtin_nontemporal_store(o, reinterpret_cast<u32x4_t*>(out + e));
  }
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" int ttamd_nf4_dequantize_merge_bf16(const uint8_t* quantized_data, const void* block_scalers, const void* lora_a,
                                               const void* lora_b, int rank, float scale, void* out, int64_t N, int64_t K,
                                               void* stream) {
  TT_REQUIRE(quantized_data && block_scalers && lora_a && lora_b && out, "nf4_dequantize_merge: null pointer argument");
  TT_REQUIRE(aligned16(quantized_data) && aligned16(lora_a) && aligned16(out) &&
                 (reinterpret_cast<uintptr_t>(block_scalers) & 3u) == 0,
             "nf4_dequantize_merge: quantized_data, lora_a and out must be 16-byte aligned");
  TT_REQUIRE(N > 0 && K > 0 && N < (1 << 30) && K < (1 << 30) && K % 64 == 0,
             "nf4_dequantize_merge: bad shape N=%lld K=%lld (K must be a multiple of the NF4 block size 64)", (long long)N,
             (long long)K);
  TT_REQUIRE(rank > 0 && rank <= 64 && rank % 8 == 0, "nf4_dequantize_merge: rank (%d) must be a multiple of 8 in [8, 64]", rank);
  const dim3 grid((unsigned)((K + 2047) / 2048), (unsigned)((N + kRowsPerWg - 1) / kRowsPerWg)), block(256);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const uint32_t* q = reinterpret_cast<const uint32_t*>(quantized_data);
  const float* bs = reinterpret_cast<const float*>(block_scalers);
  const uint16_t* a = reinterpret_cast<const uint16_t*>(lora_a);
  const uint16_t* b = reinterpret_cast<const uint16_t*>(lora_b);
  uint16_t* o = reinterpret_cast<uint16_t*>(out);
  switch (rank / 8) {
    case 1: nf4_dequant_merge_kernel<1><<<grid, block, 0, s>>>(q, bs, a, b, scale, (int)N, (int)K, o); break;
    case 2: nf4_dequant_merge_kernel<2><<<grid, block, 0, s>>>(q, bs, a, b, scale, (int)N, (int)K, o); break;
    case 3: nf4_dequant_merge_kernel<3><<<grid, block, 0, s>>>(q, bs, a, b, scale, (int)N, (int)K, o); break;
    case 4: nf4_dequant_merge_kernel<4><<<grid, block, 0, s>>>(q, bs, a, b, scale, (int)N, (int)K, o); break;
    case 5: nf4_dequant_merge_kernel<5><<<grid, block, 0, s>>>(q, bs, a, b, scale, (int)N, (int)K, o); break;
    case 6: nf4_dequant_merge_kernel<6><<<grid, block, 0, s>>>(q, bs, a, b, scale, (int)N, (int)K, o); break;
    case 7: nf4_dequant_merge_kernel<7><<<grid, block, 0, s>>>(q, bs, a, b, scale, (int)N, (int)K, o); break;
    default: nf4_dequant_merge_kernel<8><<<grid, block, 0, s>>>(q, bs, a, b, scale, (int)N, (int)K, o); break;
  }
  return check_launch("nf4_dequantize_merge");
}
