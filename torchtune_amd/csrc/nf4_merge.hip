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
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __constant__ float kNF4Merge[16] = TT_NF4_TABLE;

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  bf16x2_t v;
  v.x = (__bf16)lo;
  v.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}

constexpr int kRowsPerWg = 16;

// NORM = false: store the merged weight.  NORM = true: store nothing but the sum of squares of every merged row over
// this workgroup's column strip, norm_part[strip][n] (DoRA's weight norm; finished by dora_norm_finish_kernel).
template <int R8, bool NORM>  // R8 = rank / 8
__global__ __launch_bounds__(256) void nf4_dequant_merge_kernel(const uint32_t* __restrict__ qdata,
                                                                const float* __restrict__ block_scalers,
                                                                const uint16_t* __restrict__ A,
                                                                const uint16_t* __restrict__ B, float scale, int N, int K,
                                                                uint16_t* __restrict__ out, float* __restrict__ norm_part) {
  constexpr int R = 8 * R8;
  __shared__ float2 lut[256];
  __shared__ float bsh[kRowsPerWg][R];
  __shared__ float ssq[4][kRowsPerWg];
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
  if (!NORM && !live) return;
  for (int i = 0; i < kRowsPerWg; ++i) {
    const int n = n0 + i;
    if (n >= N) break;  // uniform over the workgroup
    const int64_t e = (int64_t)n * K + (live ? k : 0);
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
        uint32_t ar = a[r][d];
        // ranks above 32: keep the pair packed inside the row loop; unpacked ahead of it (which the compiler does when it
        // can) the adapter columns take twice the registers and the kernel spills
        if constexpr (R8 > 4 && !NORM) asm volatile("" : "+v"(ar));
        m[2 * d] = __builtin_fmaf(b, bits_f32(ar << 16), m[2 * d]);
        m[2 * d + 1] = __builtin_fmaf(b, bits_f32(ar & 0xffff0000u), m[2 * d + 1]);
      }
    }
    u32x4_t o;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const float2 pr = lut[(code >> (8 * d)) & 0xffu];
      const float w0 = round_to_bf16(pr.x * sc), w1 = round_to_bf16(pr.y * sc);
      const float u0 = round_to_bf16(scale * round_to_bf16(m[2 * d])), u1 = round_to_bf16(scale * round_to_bf16(m[2 * d + 1]));
      if constexpr (NORM) {
        o[d] = 0;
        const float v0 = round_to_bf16(w0 + u0), v1 = round_to_bf16(w1 + u1);
        m[2 * d] = v0 * v0;
        m[2 * d + 1] = v1 * v1;
      } else {
        o[d] = pack2(w0 + u0, w1 + u1);
      }
    }
    if constexpr (NORM) {
      float ss = 0.f;
      if (live) {
#pragma unroll
        for (int d = 0; d < 8; ++d) ss += m[d];
      }
#pragma unroll
      for (int off = 1; off < kWave; off <<= 1) ss += __shfl_xor(ss, off, kWave);
      if ((t & 63) == 0) ssq[t >> 6][i] = ss;
    } else {
      __builtin_nontemporal_store(o, reinterpret_cast<u32x4_t*>(out + e));
    }
  }
  if constexpr (NORM) {
    __syncthreads();
    if (t < kRowsPerWg && n0 + t < N)
      norm_part[(int64_t)blockIdx.x * N + n0 + t] = ((ssq[0][t] + ssq[1][t]) + ssq[2][t]) + ssq[3][t];
  }
}

// norm[n] = bf16(sqrt(sum over strips of norm_part[strip][n])), and optionally mag_norm_scale[n] = bf16(magnitude[n] / norm[n])
__global__ __launch_bounds__(256) void dora_norm_finish_kernel(const float* __restrict__ norm_part, int strips, int N,
                                                               const uint16_t* __restrict__ magnitude,
                                                               uint16_t* __restrict__ norm, uint16_t* __restrict__ mns) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  float s = 0.f;
  for (int p = 0; p < strips; ++p) s += norm_part[(int64_t)p * N + n];
  const float nv = round_to_bf16(__builtin_sqrtf(s));
  norm[n] = f32_to_bf16_bits(nv);
  if (mns) mns[n] = f32_to_bf16_bits(bf16_bits_to_f32(magnitude[n]) / nv);
}

// DoRA backward prologue, one pass over gy and the layer's saved output:
//   gy0 = bf16(gy * mns)              (the gradient reaching the LoRA-fused linear)
//   gmag_part[w][n] = sum over the rows of wave w of gy * out   (d out / d magnitude = out / magnitude)
// A workgroup owns 512 columns (8 per lane) and a slice of rows; its 4 waves take rows in turn.
__global__ __launch_bounds__(256) void dora_bwd_prologue_kernel(const uint16_t* __restrict__ gy, const uint16_t* __restrict__ out,
                                                                const uint16_t* __restrict__ mns, uint16_t* __restrict__ gy0,
                                                                float* __restrict__ gmag_part, int M, int N,
                                                                int rows_per_split) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.x * 512 + lane * 8;
  const bool live = col < N;  // N % 8 == 0
  const int m_begin = blockIdx.y * rows_per_split;
  int m_end = m_begin + rows_per_split;
  m_end = m_end < M ? m_end : M;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if (live) {
    const u32x4_t sv = *reinterpret_cast<const u32x4_t*>(mns + col);
    for (int m = m_begin + wave; m < m_end; m += 4) {
      const int64_t e0 = (int64_t)m * N + col;
      const u32x4_t g = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(gy + e0));
      const u32x4_t o = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(out + e0));
      u32x4_t r;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const float g0 = bits_f32(g[d] << 16), g1 = bits_f32(g[d] & 0xffff0000u);
        acc[2 * d] += g0 * bits_f32(o[d] << 16);
        acc[2 * d + 1] += g1 * bits_f32(o[d] & 0xffff0000u);
        r[d] = pack2(g0 * bits_f32(sv[d] << 16), g1 * bits_f32(sv[d] & 0xffff0000u));
      }
      __builtin_nontemporal_store(r, reinterpret_cast<u32x4_t*>(gy0 + e0));
    }
    float* p = gmag_part + ((int64_t)(blockIdx.y * 4 + wave)) * N + col;
    *reinterpret_cast<f32x4_t*>(p) = f32x4_t{acc[0], acc[1], acc[2], acc[3]};
    *reinterpret_cast<f32x4_t*>(p + 4) = f32x4_t{acc[4], acc[5], acc[6], acc[7]};
  }
}

// gmag[n] = bf16(sum_w gmag_part[w][n] / magnitude[n]), fixed order
__global__ __launch_bounds__(256) void dora_gmag_finish_kernel(const float* __restrict__ part, int n_parts, int N,
                                                               const uint16_t* __restrict__ magnitude,
                                                               uint16_t* __restrict__ gmag) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  float s = 0.f;
#pragma unroll 8
  for (int p = 0; p < n_parts; ++p) s += part[(int64_t)p * N + n];
  gmag[n] = f32_to_bf16_bits(s / bf16_bits_to_f32(magnitude[n]));
}

constexpr int kDoraBwdSplits = 64;  // row slices of the backward prologue: 256 partial rows

template <bool NORM>
void launch_merge(int rank, dim3 grid, hipStream_t s, const uint32_t* q, const float* bs, const uint16_t* a, const uint16_t* b,
                  float scale, int N, int K, uint16_t* o, float* part) {
  const dim3 block(256);
  switch (rank / 8) {
    case 1: nf4_dequant_merge_kernel<1, NORM><<<grid, block, 0, s>>>(q, bs, a, b, scale, N, K, o, part); break;
    case 2: nf4_dequant_merge_kernel<2, NORM><<<grid, block, 0, s>>>(q, bs, a, b, scale, N, K, o, part); break;
    case 3: nf4_dequant_merge_kernel<3, NORM><<<grid, block, 0, s>>>(q, bs, a, b, scale, N, K, o, part); break;
    case 4: nf4_dequant_merge_kernel<4, NORM><<<grid, block, 0, s>>>(q, bs, a, b, scale, N, K, o, part); break;
    case 5: nf4_dequant_merge_kernel<5, NORM><<<grid, block, 0, s>>>(q, bs, a, b, scale, N, K, o, part); break;
    case 6: nf4_dequant_merge_kernel<6, NORM><<<grid, block, 0, s>>>(q, bs, a, b, scale, N, K, o, part); break;
    case 7: nf4_dequant_merge_kernel<7, NORM><<<grid, block, 0, s>>>(q, bs, a, b, scale, N, K, o, part); break;
    default: nf4_dequant_merge_kernel<8, NORM><<<grid, block, 0, s>>>(q, bs, a, b, scale, N, K, o, part); break;
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
  launch_merge<false>(rank, grid, s, q, bs, a, b, scale, (int)N, (int)K, o, nullptr);
  return check_launch("nf4_dequantize_merge");
}

extern "C" size_t ttamd_dora_weight_norm_workspace_bytes(int64_t N, int64_t K) {
  if (N <= 0 || K <= 0) return 0;
  return (size_t)((K + 2047) / 2048) * (size_t)N * sizeof(float);
}

extern "C" int ttamd_nf4_dora_weight_norm_bf16(const uint8_t* quantized_data, const void* block_scalers, const void* lora_a,
                                               const void* lora_b, int rank, float scale, const void* magnitude,
                                               void* weight_norm, void* mag_norm_scale, int64_t N, int64_t K, void* workspace,
                                               size_t workspace_bytes, void* stream) {
  TT_REQUIRE(quantized_data && block_scalers && lora_a && lora_b && weight_norm && workspace,
             "nf4_dora_weight_norm: null pointer argument");
  TT_REQUIRE((magnitude == nullptr) == (mag_norm_scale == nullptr),
             "nf4_dora_weight_norm: magnitude and mag_norm_scale must both be given or both be null");
  TT_REQUIRE(aligned16(quantized_data) && aligned16(lora_a) && aligned16(workspace) &&
                 (reinterpret_cast<uintptr_t>(block_scalers) & 3u) == 0,
             "nf4_dora_weight_norm: quantized_data, lora_a and workspace must be 16-byte aligned");
  TT_REQUIRE(N > 0 && K > 0 && N < (1 << 30) && K < (1 << 30) && K % 64 == 0,
             "nf4_dora_weight_norm: bad shape N=%lld K=%lld (K must be a multiple of the NF4 block size 64)", (long long)N,
             (long long)K);
  TT_REQUIRE(rank > 0 && rank <= 64 && rank % 8 == 0, "nf4_dora_weight_norm: rank (%d) must be a multiple of 8 in [8, 64]", rank);
  if (workspace_bytes < ttamd_dora_weight_norm_workspace_bytes(N, K))
    return fail(TTAMD_EWORKSPACE, "nf4_dora_weight_norm: workspace has %zu bytes, needs %zu", workspace_bytes,
                ttamd_dora_weight_norm_workspace_bytes(N, K));
  const int strips = (int)((K + 2047) / 2048);
  const dim3 grid((unsigned)strips, (unsigned)((N + kRowsPerWg - 1) / kRowsPerWg));
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  float* part = reinterpret_cast<float*>(workspace);
  launch_merge<true>(rank, grid, s, reinterpret_cast<const uint32_t*>(quantized_data), reinterpret_cast<const float*>(block_scalers),
                     reinterpret_cast<const uint16_t*>(lora_a), reinterpret_cast<const uint16_t*>(lora_b), scale, (int)N, (int)K,
                     nullptr, part);
  dora_norm_finish_kernel<<<dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s>>>(
      part, strips, (int)N, reinterpret_cast<const uint16_t*>(magnitude), reinterpret_cast<uint16_t*>(weight_norm),
      reinterpret_cast<uint16_t*>(mag_norm_scale));
  return check_launch("nf4_dora_weight_norm");
}

extern "C" size_t ttamd_dora_bwd_workspace_bytes(int64_t N) {
  return N > 0 ? (size_t)kDoraBwdSplits * 4 * (size_t)N * sizeof(float) : 0;
}

extern "C" int ttamd_dora_bwd_prologue_bf16(const void* gy, const void* out, const void* mag_norm_scale, const void* magnitude,
                                            void* gy0, void* gmagnitude, int64_t M, int64_t N, void* workspace,
                                            size_t workspace_bytes, void* stream) {
  TT_REQUIRE(gy && out && mag_norm_scale && magnitude && gy0 && gmagnitude && workspace, "dora_bwd_prologue: null pointer argument");
  TT_REQUIRE(aligned16(gy) && aligned16(out) && aligned16(mag_norm_scale) && aligned16(gy0) && aligned16(workspace),
             "dora_bwd_prologue: pointers must be 16-byte aligned");
  TT_REQUIRE(M > 0 && N > 0 && N % 8 == 0 && M < (1 << 30) && N < (1 << 30), "dora_bwd_prologue: bad shape M=%lld N=%lld (N must be a multiple of 8)",
             (long long)M, (long long)N);
  if (workspace_bytes < ttamd_dora_bwd_workspace_bytes(N))
    return fail(TTAMD_EWORKSPACE, "dora_bwd_prologue: workspace has %zu bytes, needs %zu", workspace_bytes,
                ttamd_dora_bwd_workspace_bytes(N));
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  int64_t rows_per_split = (M + kDoraBwdSplits - 1) / kDoraBwdSplits;
  rows_per_split = (rows_per_split + 3) / 4 * 4;
  const int splits = (int)((M + rows_per_split - 1) / rows_per_split);
  float* part = reinterpret_cast<float*>(workspace);
  dora_bwd_prologue_kernel<<<dim3((unsigned)((N + 511) / 512), (unsigned)splits), dim3(256), 0, s>>>(
      reinterpret_cast<const uint16_t*>(gy), reinterpret_cast<const uint16_t*>(out), reinterpret_cast<const uint16_t*>(mag_norm_scale),
      reinterpret_cast<uint16_t*>(gy0), part, (int)M, (int)N, (int)rows_per_split);
  dora_gmag_finish_kernel<<<dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s>>>(
      part, splits * 4, (int)N, reinterpret_cast<const uint16_t*>(magnitude), reinterpret_cast<uint16_t*>(gmagnitude));
  return check_launch("dora_bwd_prologue");
}
