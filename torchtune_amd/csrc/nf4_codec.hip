// NF4 double-quantisation codec for gfx950: to_nf4 (quantise) and get_original_weight (dequantise).
//
// Both directions are HBM-bound streaming kernels.  Algorithmic traffic per weight element for a bf16
// tensor with block 64 / scaler block 256:  0.5 B codes + 1/64 B int8 scaler + 2/16384 B factor on the
// packed side, 2 B on the dense side = 2.515747 B.
//
// Layout (all row-major, flattened):
//   quantized_data   u8  [numel/2]        byte b = code(2b) << 4 | code(2b+1)
//   quantized_scalers i8 [numel/bs]       one per block of `bs` consecutive elements
//   quantization_factor T [numel/bs/SB]   one per `SB` consecutive blocks
//   scaler_mean      T   [1]
#include "common.h"
#include "nf4_math.h"

namespace ttamd {
namespace {

__device__ __constant__ float kNF4Dev[16] = TT_NF4_TABLE;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2_t v;
  v.x = (__bf16)lo;
  v.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}

// max that propagates NaN the way torch.max does
__device__ __forceinline__ float nanmax(float a, float b) { return (a != a) ? a : ((b != b) ? b : (a > b ? a : b)); }

template <bool BF16>
__device__ __forceinline__ void load8(const void* base, int64_t chunk, float v[8]) {
  if constexpr (BF16) {
    uint4 r = reinterpret_cast<const uint4*>(base)[chunk];
    uint32_t d[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = bits_f32(d[i] << 16);
      v[2 * i + 1] = bits_f32(d[i] & 0xffff0000u);
    }
  } else {
    const float4* p = reinterpret_cast<const float4*>(base) + 2 * chunk;
    float4 a = p[0], b = p[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
}

template <bool BF16>
__device__ __forceinline__ float load1(const void* base, int64_t i) {
  if constexpr (BF16)
    return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(base)[i]);
  else
    return reinterpret_cast<const float*>(base)[i];
}

template <bool BF16>
__device__ __forceinline__ void store1(void* base, int64_t i, float v) {
  if constexpr (BF16)
    reinterpret_cast<uint16_t*>(base)[i] = f32_to_bf16_bits(v);
  else
    reinterpret_cast<float*>(base)[i] = v;
}

// ---------------------------------------------------------------------------------------------------
// quantise, pass 1: per-block absmax and the 4-bit codes.  One lane owns 8 consecutive elements (one
// 128-bit load for bf16); a block of `bs` elements is spread over bs/8 neighbouring lanes of one wave.
// ---------------------------------------------------------------------------------------------------
template <bool BF16>
__global__ __launch_bounds__(256) void nf4_quantize_blocks_kernel(const void* __restrict__ w, int64_t n_chunks,
                                                                  int lanes_per_block, int log2_lpb,
                                                                  uint32_t* __restrict__ qdata, float* __restrict__ absmax) {
  const int64_t chunk = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const bool live = chunk < n_chunks;
  float v[8];
  if (live) {
    load8<BF16>(w, chunk, v);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 0.f;
  }
  float m = __builtin_fabsf(v[0]);
#pragma unroll
  for (int i = 1; i < 8; ++i) m = nanmax(m, __builtin_fabsf(v[i]));
  for (int off = 1; off < lanes_per_block; off <<= 1) m = nanmax(m, __shfl_xor(m, off, kWave));
  if (!live) return;
  if ((threadIdx.x & (lanes_per_block - 1)) == 0) absmax[chunk >> log2_lpb] = m;
  uint32_t packed = 0;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    int hi = nf4_nearest_code<BF16>(Arith<BF16>::rnd(v[2 * b] / m));
    int lo = nf4_nearest_code<BF16>(Arith<BF16>::rnd(v[2 * b + 1] / m));
    packed |= (uint32_t)((hi << 4) | lo) << (8 * b);
  }
  qdata[chunk] = packed;
}

// ---------------------------------------------------------------------------------------------------
// quantise, pass 1 for bfloat16, the fast form of the kernel above (identical results).
//
// (a) The scaled value bf16(x / absmax) is one of 65536 bit patterns, so "nearest code under the reference's rule"
//     is a table lookup.  Every pattern with |value| < 2^-5 maps to code 7 (the zero code: its neighbours' midpoints
//     are -0.0455 and +0.0398) and |value| <= 1 always, so the table only spans magnitudes 0x3D00 (2^-5) .. 0x3F80
//     (1.0) for each sign: 2 x 641 bytes.  The host fills it once with nf4_nearest_code<true>, checks the two
//     claims above over all patterns, and passes it by value; NaN (0/0 of an all-zero block) yields code 0.
// (b) x / absmax for 64 elements shares the divisor: y = 1 / absmax is divided once (correctly rounded) and each
//     quotient is q0 = x * y, r = fma(-q0, absmax, x), q = fma(r, y, q0).  For bf16 operands with absmax >= 2^-119
//     and |x| <= absmax this rounds to the same bf16 as the correctly rounded quotient for EVERY operand pair
//     (checked exhaustively on a CPU, 5.3e8 pairs); smaller or non-finite divisors take the plain division.
// ---------------------------------------------------------------------------------------------------
constexpr int kCodeTabBase = 0x3D00;
constexpr int kCodeTabLast = 0x3F80;
constexpr int kCodeTabN = kCodeTabLast - kCodeTabBase + 1;  // 641
constexpr int kCodeTabStride = 644;                          // per sign, padded to a multiple of 4
struct Nf4CodeTable {
  uint32_t words[2 * kCodeTabStride / 4];
};
constexpr int kQuantChunksPerThread = 4;

__global__ __launch_bounds__(256) void nf4_quantize_blocks_bf16_kernel(const void* __restrict__ w, int64_t n_chunks,
                                                                       int lanes_per_block, int log2_lpb,
                                                                       uint32_t* __restrict__ qdata, float* __restrict__ absmax,
                                                                       const Nf4CodeTable table) {
  __shared__ uint32_t tab_words[2 * kCodeTabStride / 4];
  for (int i = threadIdx.x; i < 2 * kCodeTabStride / 4; i += 256) tab_words[i] = table.words[i];
  __syncthreads();
  const uint8_t* tab = reinterpret_cast<const uint8_t*>(tab_words);
#pragma unroll
  for (int u = 0; u < kQuantChunksPerThread; ++u) {
    const int64_t chunk = ((int64_t)blockIdx.x * kQuantChunksPerThread + u) * 256 + threadIdx.x;
    const bool live = chunk < n_chunks;  // uniform per block of lanes: n_chunks is a multiple of lanes_per_block
    float v[8];
    if (live) {
      load8<true>(w, chunk, v);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = 0.f;
    }
    float m = __builtin_fabsf(v[0]);
#pragma unroll
    for (int i = 1; i < 8; ++i) m = nanmax(m, __builtin_fabsf(v[i]));
    for (int off = 1; off < lanes_per_block; off <<= 1) m = nanmax(m, __shfl_xor(m, off, kWave));
    if (!live) continue;
    if ((threadIdx.x & (lanes_per_block - 1)) == 0) absmax[chunk >> log2_lpb] = m;
    const bool fast = m >= 0x1p-119f && m < __builtin_inff();  // false for NaN too
    const float y = 1.0f / m;
    uint32_t packed = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      float qf[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float x = v[2 * b + e];
        if (fast) {
          const float q0 = x * y;
          const float r = __builtin_fmaf(-q0, m, x);
          qf[e] = __builtin_fmaf(r, y, q0);
        } else {
          qf[e] = x / m;
        }
      }
      const uint32_t pr = pack_bf16x2(qf[0], qf[1]);  // low half: element 2b (high nibble), high half: element 2b+1
      uint32_t code[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const uint32_t bits = e ? (pr >> 16) : (pr & 0xffffu);
        const uint32_t mag = bits & 0x7fffu;
        uint32_t idx = mag > (uint32_t)kCodeTabBase ? mag - kCodeTabBase : 0u;
        idx = idx < (uint32_t)(kCodeTabN - 1) ? idx : (uint32_t)(kCodeTabN - 1);
        idx += (bits >> 15) * kCodeTabStride;
        const uint32_t c = tab[idx];
        code[e] = mag > 0x7f80u ? 0u : c;
      }
      packed |= ((code[0] << 4) | code[1]) << (8 * b);
    }
    qdata[chunk] = packed;
  }
}

// Host side of (a): the table, filled and verified once per process.
struct Nf4CodeTableHost {
  Nf4CodeTable table;
  bool ok;
  Nf4CodeTableHost() : ok(true) {
    uint8_t* bytes = reinterpret_cast<uint8_t*>(table.words);
    memset(table.words, 0, sizeof(table.words));
    for (int sign = 0; sign < 2; ++sign) {
      for (int mag = 0; mag <= kCodeTabLast; ++mag) {
        const uint16_t bits = (uint16_t)((sign << 15) | mag);
        const int c = nf4_nearest_code<true>(bf16_bits_to_f32(bits));
        if (mag < kCodeTabBase) {
          if (c != 7) ok = false;  // claim: everything below 2^-5 is the zero code
        } else {
          bytes[sign * kCodeTabStride + (mag - kCodeTabBase)] = (uint8_t)c;
        }
      }
    }
    if (nf4_nearest_code<true>(bf16_bits_to_f32(0x7fc0)) != 0) ok = false;  // NaN -> code 0
  }
};
const Nf4CodeTableHost& code_table() {
  static const Nf4CodeTableHost t;
  return t;
}

// ---------------------------------------------------------------------------------------------------
// quantise, pass 2: mean of the block absmaxes.  Summed in fp64 in a fixed order (256 partial sums, each
// a fixed strided walk followed by a fixed LDS tree) so the result does not depend on scheduling; for
// realistic dynamic ranges the fp64 sum is exact.  mean = dtype(float(sum / n)).
// ---------------------------------------------------------------------------------------------------
constexpr int kMeanPartials = 256;

__device__ __forceinline__ double block_sum_256(double s, double* sh) {
  sh[threadIdx.x] = s;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if ((int)threadIdx.x < off) sh[threadIdx.x] += sh[threadIdx.x + off];
    __syncthreads();
  }
  return sh[0];
}

__global__ __launch_bounds__(256) void nf4_absmax_partial_sum_kernel(const float* __restrict__ absmax, int64_t n_blocks,
                                                                     double* __restrict__ partial) {
  __shared__ double sh[256];
  double s = 0.0;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_blocks; i += (int64_t)kMeanPartials * 256)
    s += (double)absmax[i];
  s = block_sum_256(s, sh);
  if (threadIdx.x == 0) partial[blockIdx.x] = s;
}

template <bool BF16>
__global__ __launch_bounds__(256) void nf4_absmax_mean_kernel(const double* __restrict__ partial, int64_t n_blocks,
                                                              void* __restrict__ scaler_mean, float* __restrict__ mean_f32) {
  __shared__ double sh[256];
  double s = block_sum_256(partial[threadIdx.x], sh);
  if (threadIdx.x == 0) {
    float mean = Arith<BF16>::rnd((float)(s / (double)n_blocks));
    store1<BF16>(scaler_mean, 0, mean);
    *mean_f32 = mean;
  }
}

// ---------------------------------------------------------------------------------------------------
// quantise, pass 3: double quantisation of the block scalers.  One wave per scaler block of SB blocks.
// ---------------------------------------------------------------------------------------------------
template <bool BF16>
__global__ __launch_bounds__(256) void nf4_quantize_scalers_kernel(const float* __restrict__ absmax,
                                                                   const float* __restrict__ mean_f32, int64_t n_sb, int SB,
                                                                   int8_t* __restrict__ qscalers, void* __restrict__ qfactor) {
  const int64_t sb = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (sb >= n_sb) return;  // whole wave leaves together
  const int lane = threadIdx.x & 63;
  const float mean = *mean_f32;
  const float* a = absmax + sb * SB;
  float m = 0.f;
  for (int i = lane; i < SB; i += kWave) m = nanmax(m, __builtin_fabsf(Arith<BF16>::rnd(a[i] - mean)));
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) m = nanmax(m, __shfl_xor(m, off, kWave));
  const float factor = Arith<BF16>::rnd(256.0f / Arith<BF16>::rnd(2.0f * m));
  if (lane == 0) store1<BF16>(qfactor, sb, factor);
  for (int i = lane; i < SB; i += kWave) {
    float s1 = Arith<BF16>::rnd(a[i] - mean);
    float q = __builtin_rintf(Arith<BF16>::rnd(s1 * factor));  // torch.round: half to even
    q = (q != q) ? 0.f : (q < -128.f ? -128.f : (q > 127.f ? 127.f : q));
    qscalers[sb * SB + i] = (int8_t)(int)q;
  }
}

// ---------------------------------------------------------------------------------------------------
// dequantise.  A workgroup expands 256 * DW * 8 elements (DW = dwords of codes per lane).  It first evaluates the
// block scalers of its span once (one thread per block, into LDS: the division is done once per block, not once per
// lane), then every lane turns one dword of codes (8 elements) into one 128-bit bf16 store (two for fp32), so each load and
// store instruction of a wave covers one contiguous span.  Code pairs are looked up a byte at a time in a
// 256-entry LDS table of (nf4[hi], nf4[lo]) in fp32; for bf16 the product is rounded once, by the packing
// conversion (round to nearest even, the same rounding the eager reference applies to the product).
//
// DW is chosen by the launch: 8 (16384 elements per workgroup) while codes and output together fit the 256 MB
// last-level cache, where fewer, longer workgroups win (measured 5.9 against 5.6 TB/s on 14336 x 4096), and 4 beyond
// it, where twice the number of workgroups keeps more HBM requests in flight (6.1 against 5.4 TB/s on 28672 x 8192
// with the cache defeated by rotating over four weights).
// ---------------------------------------------------------------------------------------------------
constexpr int64_t kDequantCacheResidentBytes = int64_t(192) << 20;

template <bool BF16, int DW>
__global__ __launch_bounds__(256) void nf4_dequantize_kernel(const uint32_t* __restrict__ qdata,
                                                             const int8_t* __restrict__ qscalers,
                                                             const void* __restrict__ qfactor,
                                                             const void* __restrict__ scaler_mean, int64_t n_dwords,
                                                             int log2_dwords_per_block, int SB, int log2_SB,
                                                             int64_t n_blocks, void* __restrict__ out) {
  __shared__ float2 lut[256];
  __shared__ float scal[256 * DW];  // smallest block size is 8 elements = one dword
  const int t = threadIdx.x;
  const int64_t base = (int64_t)blockIdx.x * (256 * DW) + t;
  uint32_t code[DW];
#pragma unroll
  for (int u = 0; u < DW; ++u) {
    const int64_t idx = base + u * 256;
    code[u] = idx < n_dwords ? __builtin_nontemporal_load(qdata + idx) : 0u;
  }
  lut[t] = make_float2(Arith<BF16>::rnd(kNF4Dev[t >> 4]), Arith<BF16>::rnd(kNF4Dev[t & 15]));
  {
    const float mean = load1<BF16>(scaler_mean, 0);
    const int blocks_per_wg = (256 * DW) >> log2_dwords_per_block;
    const int64_t blk0 = (int64_t)blockIdx.x * blocks_per_wg;
    for (int i = t; i < blocks_per_wg; i += 256) {
      const int64_t blk = blk0 + i;
      if (blk >= n_blocks) break;
      const int64_t sb = log2_SB >= 0 ? (blk >> log2_SB) : (blk / SB);
      scal[i] = nf4_block_scaler<BF16>((int)qscalers[blk], load1<BF16>(qfactor, sb), mean);
    }
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < DW; ++u) {
    const int64_t idx = base + u * 256;
    if (idx >= n_dwords) continue;
    const float sc = scal[(u * 256 + t) >> log2_dwords_per_block];
    float v[8];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const float2 pr = lut[(code[u] >> (8 * b)) & 0xffu];
      v[2 * b] = pr.x * sc;
      v[2 * b + 1] = pr.y * sc;
    }
    if constexpr (BF16) {
      u32x4_t o;
      o.x = pack_bf16x2(v[0], v[1]);
      o.y = pack_bf16x2(v[2], v[3]);
      o.z = pack_bf16x2(v[4], v[5]);
      o.w = pack_bf16x2(v[6], v[7]);
      __builtin_nontemporal_store(o, reinterpret_cast<u32x4_t*>(out) + idx);
    } else {
      f32x4_t* o = reinterpret_cast<f32x4_t*>(out) + 2 * idx;
      f32x4_t a = {v[0], v[1], v[2], v[3]}, b = {v[4], v[5], v[6], v[7]};
      __builtin_nontemporal_store(a, o);
      __builtin_nontemporal_store(b, o + 1);
    }
  }
}

int log2_exact(int64_t v) {
  int l = 0;
  while ((int64_t(1) << l) < v) ++l;
  return l;
}

struct QuantWorkspace {
  float* absmax;    // [n_blocks]
  double* partial;  // [kMeanPartials]
  float* mean;      // [1]
};

size_t quant_ws_bytes(int64_t n_blocks) {
  size_t absmax_bytes = ((size_t)n_blocks * sizeof(float) + 255) & ~size_t(255);
  return absmax_bytes + kMeanPartials * sizeof(double) + 256;
}

int check_nf4_shape(int64_t numel, int block_size, int scaler_block_size) {
  TT_REQUIRE(numel > 0, "nf4: numel must be positive (got %lld)", (long long)numel);
  TT_REQUIRE(block_size >= 8 && block_size <= 512 && is_pow2(block_size),
             "nf4: block_size must be a power of two in [8, 512] (got %d)", block_size);
  TT_REQUIRE(scaler_block_size >= 1, "nf4: scaler_block_size must be positive (got %d)", scaler_block_size);
  TT_REQUIRE(numel % block_size == 0, "nf4: numel (%lld) must be divisible by block_size (%d)", (long long)numel,
             block_size);
  TT_REQUIRE((numel / block_size) % scaler_block_size == 0,
             "nf4: number of blocks (%lld) must be divisible by scaler_block_size (%d)",
             (long long)(numel / block_size), scaler_block_size);
  return TTAMD_OK;
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" size_t ttamd_nf4_quantize_workspace_bytes(int64_t numel, int block_size) {
  if (numel <= 0 || block_size <= 0) return 0;
  return quant_ws_bytes(numel / block_size);
}

extern "C" int ttamd_nf4_quantize(const void* w, int dtype, int64_t numel, int block_size, int scaler_block_size,
                                  uint8_t* quantized_data, int8_t* quantized_scalers, void* quantization_factor,
                                  void* scaler_mean, void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_nf4_shape(numel, block_size, scaler_block_size)) return rc;
  TT_REQUIRE(dtype == TTAMD_BF16 || dtype == TTAMD_F32, "nf4_quantize: unknown dtype code %d", dtype);
  TT_REQUIRE(w && quantized_data && quantized_scalers && quantization_factor && scaler_mean && workspace,
             "nf4_quantize: null pointer argument");
  TT_REQUIRE(aligned16(w) && (reinterpret_cast<uintptr_t>(quantized_data) & 3u) == 0 && aligned16(workspace),
             "nf4_quantize: w/workspace must be 16-byte aligned and quantized_data 4-byte aligned");
  const int64_t n_blocks = numel / block_size;
  const int64_t n_sb = n_blocks / scaler_block_size;
  if (workspace_bytes < quant_ws_bytes(n_blocks))
    return fail(TTAMD_EWORKSPACE, "nf4_quantize: workspace has %zu bytes, needs %zu", workspace_bytes,
                quant_ws_bytes(n_blocks));
  QuantWorkspace ws;
  ws.absmax = reinterpret_cast<float*>(workspace);
  size_t absmax_bytes = ((size_t)n_blocks * sizeof(float) + 255) & ~size_t(255);
  ws.partial = reinterpret_cast<double*>(reinterpret_cast<char*>(workspace) + absmax_bytes);
  ws.mean = reinterpret_cast<float*>(ws.partial + kMeanPartials);

  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int64_t n_chunks = numel / 8;
  const int lpb = block_size / 8;
  const int64_t grid1 = (n_chunks + 255) / 256;
  TT_REQUIRE(grid1 < (int64_t(1) << 31), "nf4_quantize: tensor too large for one launch");
  const int64_t grid3 = (n_sb + 3) / 4;
  if (dtype == TTAMD_BF16) {
    const Nf4CodeTableHost& ct = code_table();
    if (ct.ok) {
      const int64_t per_wg = 256 * kQuantChunksPerThread;
      nf4_quantize_blocks_bf16_kernel<<<dim3((unsigned)((n_chunks + per_wg - 1) / per_wg)), dim3(256), 0, s>>>(
          w, n_chunks, lpb, log2_exact(lpb), reinterpret_cast<uint32_t*>(quantized_data), ws.absmax, ct.table);
    } else {  // the table's premises failed their check: search the 16 codes directly
      nf4_quantize_blocks_kernel<true><<<dim3((unsigned)grid1), dim3(256), 0, s>>>(
          w, n_chunks, lpb, log2_exact(lpb), reinterpret_cast<uint32_t*>(quantized_data), ws.absmax);
    }
    nf4_absmax_partial_sum_kernel<<<dim3(kMeanPartials), dim3(256), 0, s>>>(ws.absmax, n_blocks, ws.partial);
    nf4_absmax_mean_kernel<true><<<dim3(1), dim3(256), 0, s>>>(ws.partial, n_blocks, scaler_mean, ws.mean);
    nf4_quantize_scalers_kernel<true><<<dim3((unsigned)grid3), dim3(256), 0, s>>>(
        ws.absmax, ws.mean, n_sb, scaler_block_size, quantized_scalers, quantization_factor);
  } else {
    nf4_quantize_blocks_kernel<false><<<dim3((unsigned)grid1), dim3(256), 0, s>>>(
        w, n_chunks, lpb, log2_exact(lpb), reinterpret_cast<uint32_t*>(quantized_data), ws.absmax);
    nf4_absmax_partial_sum_kernel<<<dim3(kMeanPartials), dim3(256), 0, s>>>(ws.absmax, n_blocks, ws.partial);
    nf4_absmax_mean_kernel<false><<<dim3(1), dim3(256), 0, s>>>(ws.partial, n_blocks, scaler_mean, ws.mean);
    nf4_quantize_scalers_kernel<false><<<dim3((unsigned)grid3), dim3(256), 0, s>>>(
        ws.absmax, ws.mean, n_sb, scaler_block_size, quantized_scalers, quantization_factor);
  }
  return check_launch("nf4_quantize");
}

extern "C" int ttamd_nf4_dequantize(const uint8_t* quantized_data, const int8_t* quantized_scalers,
                                    const void* quantization_factor, const void* scaler_mean, int dtype, int64_t numel,
                                    int block_size, int scaler_block_size, void* out, void* stream) {
  if (int rc = check_nf4_shape(numel, block_size, scaler_block_size)) return rc;
  TT_REQUIRE(dtype == TTAMD_BF16 || dtype == TTAMD_F32, "nf4_dequantize: unknown dtype code %d", dtype);
  TT_REQUIRE(quantized_data && quantized_scalers && quantization_factor && scaler_mean && out,
             "nf4_dequantize: null pointer argument");
  TT_REQUIRE((reinterpret_cast<uintptr_t>(quantized_data) & 3u) == 0 && aligned16(out),
             "nf4_dequantize: quantized_data must be 4-byte aligned and out 16-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int64_t n_dwords = numel / 8;
  const int l2dpb = log2_exact(block_size / 8);
  const int l2sb = is_pow2(scaler_block_size) ? log2_exact(scaler_block_size) : -1;
  const int64_t bytes_moved = numel / 2 + numel * (dtype == TTAMD_BF16 ? 2 : 4);
  const int dw = bytes_moved <= kDequantCacheResidentBytes ? 8 : 4;
  const int64_t per_wg = 256 * dw;
  const int64_t grid = (n_dwords + per_wg - 1) / per_wg;
  TT_REQUIRE(grid < (int64_t(1) << 31), "nf4_dequantize: tensor too large for one launch");
  auto launch = [&](auto kernel) {
    kernel<<<dim3((unsigned)grid), dim3(256), 0, s>>>(reinterpret_cast<const uint32_t*>(quantized_data), quantized_scalers,
                                                      quantization_factor, scaler_mean, n_dwords, l2dpb, scaler_block_size,
                                                      l2sb, numel / block_size, out);
  };
  if (dtype == TTAMD_BF16) {
    if (dw == 8) launch(nf4_dequantize_kernel<true, 8>); else launch(nf4_dequantize_kernel<true, 4>);
  } else {
    if (dw == 8) launch(nf4_dequantize_kernel<false, 8>); else launch(nf4_dequantize_kernel<false, 4>);
  }
  return check_launch("nf4_dequantize");
}
