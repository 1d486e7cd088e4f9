// QAT fake-quantisation kernels for gfx950 (8da4w scheme): per-token asymmetric int8 for activations,
// per-group symmetric int4 for weights, and the real int4 conversion.  All three are HBM-bound streaming
// kernels: one read and one write of the tensor (4 B/element in bf16) plus the small qparam arrays.
//
// Reductions are wavefront reductions: a token row (or a weight group) lives in the registers of one
// wave (or of g/8 neighbouring lanes) and min/max travel over cross-lane shuffles, so the data is read
// from HBM exactly once.
#include "common.h"
#include "nf4_math.h"

namespace ttamd {
namespace {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr float kF32Eps = 1.1920928955078125e-07f;  // torch.finfo(torch.float32).eps

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2_t v;
  v.x = (__bf16)lo;
  v.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}

// Eight consecutive elements held in registers in their storage format.
template <bool BF16>
struct Chunk8;

template <>
struct Chunk8<true> {
  u32x4_t raw;
  __device__ __forceinline__ void load(const void* base, int64_t chunk) {
    raw = reinterpret_cast<const u32x4_t*>(base)[chunk];
  }
  __device__ __forceinline__ void zero() { raw = u32x4_t{0, 0, 0, 0}; }
  __device__ __forceinline__ float get(int i) const {
    uint32_t d = raw[i >> 1];
    return bits_f32((i & 1) ? (d & 0xffff0000u) : (d << 16));
  }
  static __device__ __forceinline__ void store(void* base, int64_t chunk, const float v[8]) {
    u32x4_t o;
    o.x = pack_bf16x2(v[0], v[1]);
    o.y = pack_bf16x2(v[2], v[3]);
    o.z = pack_bf16x2(v[4], v[5]);
    o.w = pack_bf16x2(v[6], v[7]);
    __builtin_nontemporal_store(o, reinterpret_cast<u32x4_t*>(base) + chunk);
  }
};

template <>
struct Chunk8<false> {
  f32x4_t a, b;
  __device__ __forceinline__ void load(const void* base, int64_t chunk) {
    const f32x4_t* p = reinterpret_cast<const f32x4_t*>(base) + 2 * chunk;
    a = p[0];
    b = p[1];
  }
  __device__ __forceinline__ void zero() {
    a = f32x4_t{0, 0, 0, 0};
    b = a;
  }
  __device__ __forceinline__ float get(int i) const { return i < 4 ? a[i] : b[i - 4]; }
  static __device__ __forceinline__ void store(void* base, int64_t chunk, const float v[8]) {
    f32x4_t* p = reinterpret_cast<f32x4_t*>(base) + 2 * chunk;
    f32x4_t lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
    __builtin_nontemporal_store(lo, p);
    __builtin_nontemporal_store(hi, p + 1);
  }
};

struct TokenQParams {
  float scale, inv_scale, zp;
};

// asymmetric int8 qparams from the row extrema (already widened to include 0)
// (the zero point is chosen with the fp32 scale; a bf16 qparam precision rounds the scale afterwards, and the rounded
// scale is what quantises and dequantises)
__device__ __forceinline__ TokenQParams token_qparams(float mn, float mx, bool qp_bf16, float eps) {
  TokenQParams p;
  float scale = (mx - mn) / 255.0f;
  scale = scale > eps ? scale : eps;
  const float dmin = mn / scale, dmax = mx / scale;
  float zp = ((-128.0f + dmin) + (127.0f + dmax) > 0.0f) ? (-128.0f - dmin) : (127.0f - dmax);
  zp = zp < -128.0f ? -128.0f : (zp > 127.0f ? 127.0f : zp);
  p.zp = __builtin_rintf(zp);
  if (qp_bf16) scale = round_to_bf16(scale);
  p.scale = scale;
  p.inv_scale = 1.0f / scale;
  return p;
}

template <bool BF16>
__device__ __forceinline__ float token_fq(float x, const TokenQParams& p) {
  float q = __builtin_rintf(x * p.inv_scale) + p.zp;
  q = q < -128.0f ? -128.0f : (q > 127.0f ? 127.0f : q);
  return Arith<BF16>::rnd((q - p.zp) * p.scale);
}

__device__ __forceinline__ void wave_minmax(float& mn, float& mx) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    mn = fminf(mn, __shfl_xor(mn, off, kWave));
    mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
  }
}

// One wave per token row, the whole row resident in registers: NV chunks of 8 elements per lane.
template <bool BF16, int NV>
__global__ __launch_bounds__(256) void fq_per_token_regs_kernel(const void* __restrict__ x, int64_t rows, int64_t K,
                                                                void* __restrict__ out, float* __restrict__ scale_out,
                                                                int32_t* __restrict__ zp_out, bool qp_bf16, float eps) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const int chunks_per_row = (int)(K >> 3);
  const int64_t row_chunk0 = row * chunks_per_row;
  Chunk8<BF16> c[NV];
  float mn = 0.f, mx = 0.f;  // the qparams use min(amin, 0) and max(amax, 0): zero is the neutral start
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int ch = i * kWave + lane;
    if (ch < chunks_per_row)
      c[i].load(x, row_chunk0 + ch);
    else
      c[i].zero();
  }
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = c[i].get(e);
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
  wave_minmax(mn, mx);
  const TokenQParams p = token_qparams(mn, mx, qp_bf16, eps);
  if (lane == 0) {
    if (scale_out) scale_out[row] = p.scale;
    if (zp_out) zp_out[row] = (int32_t)p.zp;
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int ch = i * kWave + lane;
    if (ch < chunks_per_row) {
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = token_fq<BF16>(c[i].get(e), p);
      Chunk8<BF16>::store(out, row_chunk0 + ch, v);
    }
  }
}

// One workgroup (four waves) per token row, NV chunks of 8 elements per lane: rows of more than 4096 elements.  A wave
// that held such a row alone would need most of the register file (one wave per SIMD: nothing else runs while it
// computes between its loads and its stores); a quarter of the row per wave leaves room for eight.  The extrema of
// the four waves meet in LDS (min and max do not depend on the order).
template <bool BF16, int NV>
__global__ __launch_bounds__(256) void fq_per_token_wg_kernel(const void* __restrict__ x, int64_t rows, int64_t K,
                                                              void* __restrict__ out, float* __restrict__ scale_out,
                                                              int32_t* __restrict__ zp_out, bool qp_bf16, float eps) {
  __shared__ float ext[2][4];
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x;
  const int chunks_per_row = (int)(K >> 3);
  const int64_t row_chunk0 = row * chunks_per_row;
  Chunk8<BF16> c[NV];
  float mn = 0.f, mx = 0.f;  // the qparams use min(amin, 0) and max(amax, 0): zero is the neutral start
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int ch = i * 256 + tid;
    if (ch < chunks_per_row)
      c[i].load(x, row_chunk0 + ch);
    else
      c[i].zero();
  }
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = c[i].get(e);
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
  wave_minmax(mn, mx);
  if ((tid & 63) == 0) {
    ext[0][tid >> 6] = mn;
    ext[1][tid >> 6] = mx;
  }
  __syncthreads();
  mn = fminf(fminf(ext[0][0], ext[0][1]), fminf(ext[0][2], ext[0][3]));
  mx = fmaxf(fmaxf(ext[1][0], ext[1][1]), fmaxf(ext[1][2], ext[1][3]));
  const TokenQParams p = token_qparams(mn, mx, qp_bf16, eps);
  if (tid == 0) {
    if (scale_out) scale_out[row] = p.scale;
    if (zp_out) zp_out[row] = (int32_t)p.zp;
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int ch = i * 256 + tid;
    if (ch < chunks_per_row) {
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = token_fq<BF16>(c[i].get(e), p);
      Chunk8<BF16>::store(out, row_chunk0 + ch, v);
    }
  }
}

// Rows too long for the register file: two passes over the row (the second one normally hits in L2).
template <bool BF16>
__global__ __launch_bounds__(256) void fq_per_token_stream_kernel(const void* __restrict__ x, int64_t rows, int64_t K,
                                                                  void* __restrict__ out, float* __restrict__ scale_out,
                                                                  int32_t* __restrict__ zp_out, bool qp_bf16, float eps) {
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const int64_t chunks_per_row = K >> 3;
  const int64_t row_chunk0 = row * chunks_per_row;
  float mn = 0.f, mx = 0.f;
  for (int64_t ch = lane; ch < chunks_per_row; ch += kWave) {
    Chunk8<BF16> c;
    c.load(x, row_chunk0 + ch);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = c.get(e);
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
  }
  wave_minmax(mn, mx);
  const TokenQParams p = token_qparams(mn, mx, qp_bf16, eps);
  if (lane == 0) {
    if (scale_out) scale_out[row] = p.scale;
    if (zp_out) zp_out[row] = (int32_t)p.zp;
  }
  for (int64_t ch = lane; ch < chunks_per_row; ch += kWave) {
    Chunk8<BF16> c;
    c.load(x, row_chunk0 + ch);
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = token_fq<BF16>(c.get(e), p);
    Chunk8<BF16>::store(out, row_chunk0 + ch, v);
  }
}

// Per-group symmetric int4.  A group of g elements is held by g/8 neighbouring lanes.
// EMIT_INT = false: write the fake-quantised tensor (training).  true: write int8-held int4 values (convert).
constexpr int kGroupChunksPerThread = 4;

template <bool BF16, bool EMIT_INT>
__global__ __launch_bounds__(256) void fq_per_group_kernel(const void* __restrict__ w, int64_t n_chunks, int lanes_per_group,
                                                           int log2_lpg, void* __restrict__ out_fq,
                                                           int8_t* __restrict__ out_q, float* __restrict__ scale_out,
                                                           float* __restrict__ zero_out, bool qp_bf16, float eps) {
  const int64_t base = (int64_t)blockIdx.x * (256 * kGroupChunksPerThread) + threadIdx.x;
  Chunk8<BF16> c[kGroupChunksPerThread];
#pragma unroll
  for (int u = 0; u < kGroupChunksPerThread; ++u) {
    const int64_t ch = base + u * 256;
    if (ch < n_chunks)
      c[u].load(w, ch);
    else
      c[u].zero();
  }
#pragma unroll
  for (int u = 0; u < kGroupChunksPerThread; ++u) {
    const int64_t ch = base + u * 256;
    float mn = 0.f, mx = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = c[u].get(e);
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
    for (int off = 1; off < lanes_per_group; off <<= 1) {
      mn = fminf(mn, __shfl_xor(mn, off, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
    }
    if (ch >= n_chunks) continue;
    const float amax = fmaxf(-mn, mx);
    float scale = amax / 7.5f;
    scale = scale > eps ? scale : eps;
    if (qp_bf16) scale = round_to_bf16(scale);  // the rounded scale quantises and dequantises
    const float inv = 1.0f / scale;
    if ((threadIdx.x & (lanes_per_group - 1)) == 0) {
      if (scale_out) scale_out[ch >> log2_lpg] = scale;
      if (zero_out) zero_out[ch >> log2_lpg] = 0.0f;
    }
    float q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float t = __builtin_rintf(c[u].get(e) * inv);
      t = t < -8.0f ? -8.0f : (t > 7.0f ? 7.0f : t);
      q[e] = (float)(int)t;  // through the integer grid: rint(-0.3) = -0.0 must dequantise to +0.0
    }
    if constexpr (EMIT_INT) {
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo |= ((uint32_t)(int)q[e] & 0xffu) << (8 * e);
        hi |= ((uint32_t)(int)q[e + 4] & 0xffu) << (8 * e);
      }
      reinterpret_cast<uint2*>(out_q)[ch] = make_uint2(lo, hi);
    } else {
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = Arith<BF16>::rnd(q[e] * scale);
      Chunk8<BF16>::store(out_fq, ch, v);
    }
  }
}

int log2_exact(int64_t v) {
  int l = 0;
  while ((int64_t(1) << l) < v) ++l;
  return l;
}

template <bool BF16>
int launch_per_token(const void* x, int64_t rows, int64_t K, void* out, float* scale, int32_t* zp, bool qp_bf16, float eps,
                     hipStream_t s) {
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  const int64_t nv = (K / 8 + kWave - 1) / kWave;     // chunks per lane with a wave per row
  const int64_t nvw = (K / 8 + 255) / 256;            // with a workgroup per row
#define TT_LAUNCH_TOKEN(NV)                                                                          \
  if (nv <= NV) {                                                                                    \
    fq_per_token_regs_kernel<BF16, NV><<<grid, block, 0, s>>>(x, rows, K, out, scale, zp, qp_bf16, eps);  \
    return check_launch("fq_per_token_int8_asym");                                                   \
  }
  TT_LAUNCH_TOKEN(1)
  TT_LAUNCH_TOKEN(2)
  TT_LAUNCH_TOKEN(4)
  TT_LAUNCH_TOKEN(8)
#undef TT_LAUNCH_TOKEN
  // more than 4096 elements a row (up to 32768): a workgroup per row
#define TT_LAUNCH_TOKEN_WG(NV)                                                                                         \
  if (nvw <= NV && rows < (int64_t(1) << 31)) {                                                                        \
    fq_per_token_wg_kernel<BF16, NV><<<dim3((unsigned)rows), block, 0, s>>>(x, rows, K, out, scale, zp, qp_bf16, eps); \
    return check_launch("fq_per_token_int8_asym");                                                                     \
  }
  TT_LAUNCH_TOKEN_WG(4)
  TT_LAUNCH_TOKEN_WG(8)
  TT_LAUNCH_TOKEN_WG(16)
#undef TT_LAUNCH_TOKEN_WG
  fq_per_token_stream_kernel<BF16><<<grid, block, 0, s>>>(x, rows, K, out, scale, zp, qp_bf16, eps);
  return check_launch("fq_per_token_int8_asym");
}

// Dense weight of a converted 8da4w linear: out = dtype((q - zero) * scale), q int8-held int4 values, one fp32 scale
// and zero per group of the last dimension.  One lane = 8 elements (8 bytes in, 16 or 32 bytes out).
template <bool BF16>
__global__ __launch_bounds__(256) void dequant_per_group_kernel(const int8_t* __restrict__ q, const float* __restrict__ scale,
                                                                const float* __restrict__ zero, int64_t n_chunks, int log2_lpg,
                                                                void* __restrict__ out) {
  const int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (ch >= n_chunks) return;
  const uint2 raw = reinterpret_cast<const uint2*>(q)[ch];
  const float sc = scale[ch >> log2_lpg];
  const float z = zero ? zero[ch >> log2_lpg] : 0.0f;
  float v[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[e] = Arith<BF16>::rnd(((float)(int8_t)(raw.x >> (8 * e)) - z) * sc);
    v[e + 4] = Arith<BF16>::rnd(((float)(int8_t)(raw.y >> (8 * e)) - z) * sc);
  }
  Chunk8<BF16>::store(out, ch, v);
}

// Per-group asymmetric uint4 with a floating-point zero point (the weight-only "4w" scheme).  Same lane layout
// as the symmetric kernel.  Every operation is rounded to the tensor dtype, the qparams additionally to their
// own precision, so the result equals the op-by-op eager sequence:
//   scale = clamp((max - min) / 15, 1e-6);  zero = min + scale * 8
//   q     = clamp(round((w - (zero - scale * 8)) / scale), 0, 15);  fq = (q - 8) * scale + zero
// EMIT_INT = true writes the codes packed two per byte (even element in the high nibble) instead of fq.
template <bool BF16, bool QP_BF16, bool EMIT_INT>
__global__ __launch_bounds__(256) void fq_per_group_asym_kernel(const void* __restrict__ w, int64_t n_chunks,
                                                                int lanes_per_group, int log2_lpg,
                                                                void* __restrict__ out_fq, uint32_t* __restrict__ out_q,
                                                                float* __restrict__ scale_out, float* __restrict__ zero_out,
                                                                float min_scale, bool clamp_range_first) {
  using A = Arith<BF16>;
  using Q = Arith<QP_BF16>;
  const int64_t base = (int64_t)blockIdx.x * (256 * kGroupChunksPerThread) + threadIdx.x;
  Chunk8<BF16> c[kGroupChunksPerThread];
#pragma unroll
  for (int u = 0; u < kGroupChunksPerThread; ++u) {
    const int64_t ch = base + u * 256;
    if (ch < n_chunks)
      c[u].load(w, ch);
    else
      c[u].zero();
  }
#pragma unroll
  for (int u = 0; u < kGroupChunksPerThread; ++u) {
    const int64_t ch = base + u * 256;
    float mn = c[u].get(0), mx = mn;
#pragma unroll
    for (int e = 1; e < 8; ++e) {
      const float v = c[u].get(e);
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
    for (int off = 1; off < lanes_per_group; off <<= 1) {
      mn = fminf(mn, __shfl_xor(mn, off, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
    }
    if (ch >= n_chunks) continue;
    // default: divide, then clamp the scale; the other order clamps the range (max - min) first
    float scale = clamp_range_first ? A::rnd(A::rnd(fmaxf(A::rnd(mx - mn), min_scale)) / 15.0f)
                                    : A::rnd(fmaxf(A::rnd(A::rnd(mx - mn) / 15.0f), min_scale));
    float zero = A::rnd(mn + A::rnd(scale * 8.0f));
    scale = Q::rnd(scale);
    zero = Q::rnd(zero);
    if ((threadIdx.x & (lanes_per_group - 1)) == 0) {
      if (scale_out) scale_out[ch >> log2_lpg] = scale;
      if (zero_out) zero_out[ch >> log2_lpg] = zero;
    }
    const float lowest = A::rnd(zero - A::rnd(scale * 8.0f));
    // bf16 tensors: the eight divisions share one reciprocal, each quotient is corrected by two fused multiply-adds.
    // For bf16 operands with the divisor >= 2^-20 (the scale is at least 1e-6) and a quotient up to 17 the bf16-rounded
    // result equals that of the correctly rounded division (enumerated over all operand pairs by the test suite);
    // larger quotients clamp to 15 either way.  fp32 tensors keep the exact division.
    const bool fast = BF16 && scale < __builtin_inff() && scale >= 9.5367431640625e-07f;  // 2^-20: the proven range
    const float y = 1.0f / scale;
    float q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float d = A::rnd(c[u].get(e) - lowest);
      float t;
      if (fast) {
        const float q0 = d * y;
        const float r = __builtin_fmaf(-q0, scale, d);
        t = __builtin_fmaf(r, y, q0);
      } else {
        t = d / scale;
      }
      t = __builtin_rintf(A::rnd(t));
      q[e] = t < 0.0f ? 0.0f : (t > 15.0f ? 15.0f : t);
    }
    if constexpr (EMIT_INT) {
      uint32_t packed = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        packed |= (((uint32_t)(int)q[2 * e] << 4) | (uint32_t)(int)q[2 * e + 1]) << (8 * e);
      out_q[ch] = packed;
    } else {
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = A::rnd(A::rnd((q[e] - 8.0f) * scale) + zero);
      Chunk8<BF16>::store(out_fq, ch, v);
    }
  }
}

template <bool BF16>
__global__ __launch_bounds__(256) void dequant_per_group_uint4_kernel(const uint32_t* __restrict__ q,
                                                                      const float* __restrict__ scale,
                                                                      const float* __restrict__ zero, int64_t n_chunks,
                                                                      int log2_lpg, void* __restrict__ out) {
  using A = Arith<BF16>;
  const int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (ch >= n_chunks) return;
  const uint32_t raw = q[ch];
  const float sc = scale[ch >> log2_lpg];
  const float z = zero[ch >> log2_lpg];
  float v[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t b = (raw >> (8 * e)) & 0xffu;
    v[2 * e] = A::rnd(A::rnd(((float)(b >> 4) - 8.0f) * sc) + z);
    v[2 * e + 1] = A::rnd(A::rnd(((float)(b & 15u) - 8.0f) * sc) + z);
  }
  Chunk8<BF16>::store(out, ch, v);
}

template <bool EMIT_INT>
int launch_group_asym(const void* w, int dtype, int qparam_dtype, int64_t rows, int64_t K, int group_size, void* out_fq,
                      uint32_t* out_q, float* scale, float* zero, const ttamd_fq_conventions& conv, hipStream_t s,
                      const char* what) {
  const int64_t n_chunks = rows * K / 8;
  const int64_t per_wg = 256 * kGroupChunksPerThread;
  const int64_t grid = (n_chunks + per_wg - 1) / per_wg;
  TT_REQUIRE(grid < (int64_t(1) << 31), "%s: tensor too large for one launch", what);
  const int lpg = group_size / 8, l2 = log2_exact(lpg);
  const dim3 g((unsigned)grid), b(256);
  const bool bf = dtype == TTAMD_BF16, qbf = qparam_dtype == TTAMD_BF16;
  if (bf && qbf)
    fq_per_group_asym_kernel<true, true, EMIT_INT><<<g, b, 0, s>>>(w, n_chunks, lpg, l2, out_fq, out_q, scale, zero, conv.min_scale_uint4,
                                                                     conv.uint4_clamp_range_first != 0);
  else if (bf)
    fq_per_group_asym_kernel<true, false, EMIT_INT><<<g, b, 0, s>>>(w, n_chunks, lpg, l2, out_fq, out_q, scale, zero, conv.min_scale_uint4,
                                                                     conv.uint4_clamp_range_first != 0);
  else if (qbf)
    fq_per_group_asym_kernel<false, true, EMIT_INT><<<g, b, 0, s>>>(w, n_chunks, lpg, l2, out_fq, out_q, scale, zero, conv.min_scale_uint4,
                                                                     conv.uint4_clamp_range_first != 0);
  else
    fq_per_group_asym_kernel<false, false, EMIT_INT><<<g, b, 0, s>>>(w, n_chunks, lpg, l2, out_fq, out_q, scale, zero, conv.min_scale_uint4,
                                                                     conv.uint4_clamp_range_first != 0);
  return check_launch(what);
}

int check_group_args(const void* w, int dtype, int64_t rows, int64_t K, int group_size) {
  TT_REQUIRE(dtype == TTAMD_BF16 || dtype == TTAMD_F32, "fake_quant: unknown dtype code %d", dtype);
  TT_REQUIRE(w != nullptr && aligned16(w), "fake_quant: input must be a non-null 16-byte aligned pointer");
  TT_REQUIRE(rows > 0 && K > 0, "fake_quant: rows and K must be positive");
  TT_REQUIRE(group_size >= 8 && group_size <= 512 && is_pow2(group_size),
             "fake_quant: group_size must be a power of two in [8, 512] (got %d)", group_size);
  TT_REQUIRE(K % group_size == 0, "fake_quant: K (%lld) must be divisible by group_size (%d)", (long long)K,
             group_size);
  return TTAMD_OK;
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

namespace {
// The caller's conventions, or the defaults (what the plain entry points use); validated.
int resolve_conventions(const ttamd_fq_conventions* in, ttamd_fq_conventions* out, const char* who) {
  out->eps_per_token = kF32Eps;
  out->eps_per_group_sym = kF32Eps;
  out->min_scale_uint4 = 1e-6f;
  out->uint4_clamp_range_first = 0;
  if (in != nullptr) {
    *out = *in;
    TT_REQUIRE(out->eps_per_token > 0.0f && out->eps_per_group_sym > 0.0f && out->min_scale_uint4 > 0.0f,
               "%s: the lower bounds of the scales must be positive", who);
    TT_REQUIRE(out->uint4_clamp_range_first == 0 || out->uint4_clamp_range_first == 1,
               "%s: uint4_clamp_range_first must be 0 or 1", who);
  }
  return TTAMD_OK;
}
}  // namespace

extern "C" int ttamd_fq_per_token_int8_asym(const void* x, int dtype, int64_t rows, int64_t K, int qparam_dtype, void* out,
                                            float* scale, int32_t* zero_point, void* stream) {
  return ttamd_fq_per_token_int8_asym_conv(x, dtype, rows, K, qparam_dtype, out, scale, zero_point, nullptr, stream);
}

extern "C" int ttamd_fq_per_token_int8_asym_conv(const void* x, int dtype, int64_t rows, int64_t K, int qparam_dtype, void* out,
                                                 float* scale, int32_t* zero_point, const ttamd_fq_conventions* conventions,
                                                 void* stream) {
  ttamd_fq_conventions conv;
  if (int rc = resolve_conventions(conventions, &conv, "fq_per_token")) return rc;
  TT_REQUIRE(qparam_dtype == TTAMD_BF16 || qparam_dtype == TTAMD_F32, "fq_per_token: unknown qparam dtype code %d", qparam_dtype);
  const bool qbf = qparam_dtype == TTAMD_BF16;
  TT_REQUIRE(dtype == TTAMD_BF16 || dtype == TTAMD_F32, "fq_per_token: unknown dtype code %d", dtype);
  TT_REQUIRE(x && out && aligned16(x) && aligned16(out), "fq_per_token: x/out must be non-null, 16-byte aligned");
  TT_REQUIRE(rows > 0 && K > 0 && K % 8 == 0, "fq_per_token: K (%lld) must be a positive multiple of 8",
             (long long)K);
  TT_REQUIRE((rows + 3) / 4 < (int64_t(1) << 31), "fq_per_token: too many rows for one launch");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  return dtype == TTAMD_BF16 ? launch_per_token<true>(x, rows, K, out, scale, zero_point, qbf, conv.eps_per_token, s)
                             : launch_per_token<false>(x, rows, K, out, scale, zero_point, qbf, conv.eps_per_token, s);
}

extern "C" int ttamd_fq_per_group_int4_sym(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype,
                                           void* out, float* scale, void* stream) {
  return ttamd_fq_per_group_int4_sym_conv(w, dtype, rows, K, group_size, qparam_dtype, out, scale, nullptr, stream);
}

extern "C" int ttamd_fq_per_group_int4_sym_conv(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype,
                                                void* out, float* scale, const ttamd_fq_conventions* conventions, void* stream) {
  ttamd_fq_conventions conv;
  if (int rc = resolve_conventions(conventions, &conv, "fq_per_group")) return rc;
  if (int rc = check_group_args(w, dtype, rows, K, group_size)) return rc;
  TT_REQUIRE(qparam_dtype == TTAMD_BF16 || qparam_dtype == TTAMD_F32, "fq_per_group: unknown qparam dtype code %d", qparam_dtype);
  const bool qbf = qparam_dtype == TTAMD_BF16;
  TT_REQUIRE(out && aligned16(out), "fq_per_group: out must be non-null, 16-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int64_t n_chunks = rows * K / 8;
  const int64_t per_wg = 256 * kGroupChunksPerThread;
  const int64_t grid = (n_chunks + per_wg - 1) / per_wg;
  TT_REQUIRE(grid < (int64_t(1) << 31), "fq_per_group: tensor too large for one launch");
  const int lpg = group_size / 8;
  if (dtype == TTAMD_BF16)
    fq_per_group_kernel<true, false><<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, n_chunks, lpg, log2_exact(lpg), out,
                                                                                 nullptr, scale, nullptr, qbf, conv.eps_per_group_sym);
  else
    fq_per_group_kernel<false, false><<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, n_chunks, lpg, log2_exact(lpg), out,
                                                                                  nullptr, scale, nullptr, qbf, conv.eps_per_group_sym);
  return check_launch("fq_per_group_int4_sym");
}

extern "C" int ttamd_quantize_per_group_int4(const void* w, int dtype, int64_t rows, int64_t K, int group_size,
                                             int qparam_dtype, int8_t* q, float* scale, float* zero_point, void* stream) {
  return ttamd_quantize_per_group_int4_conv(w, dtype, rows, K, group_size, qparam_dtype, q, scale, zero_point, nullptr, stream);
}

extern "C" int ttamd_quantize_per_group_int4_conv(const void* w, int dtype, int64_t rows, int64_t K, int group_size,
                                                  int qparam_dtype, int8_t* q, float* scale, float* zero_point,
                                                  const ttamd_fq_conventions* conventions, void* stream) {
  ttamd_fq_conventions conv;
  if (int rc = resolve_conventions(conventions, &conv, "quantize_per_group_int4")) return rc;
  if (int rc = check_group_args(w, dtype, rows, K, group_size)) return rc;
  TT_REQUIRE(qparam_dtype == TTAMD_BF16 || qparam_dtype == TTAMD_F32, "quantize_per_group_int4: unknown qparam dtype code %d",
             qparam_dtype);
  const bool qbf = qparam_dtype == TTAMD_BF16;
  TT_REQUIRE(q && scale && (reinterpret_cast<uintptr_t>(q) & 7u) == 0,
             "quantize_per_group_int4: q (8-byte aligned) and scale must be non-null");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int64_t n_chunks = rows * K / 8;
  const int64_t per_wg = 256 * kGroupChunksPerThread;
  const int64_t grid = (n_chunks + per_wg - 1) / per_wg;
  TT_REQUIRE(grid < (int64_t(1) << 31), "quantize_per_group_int4: tensor too large for one launch");
  const int lpg = group_size / 8;
  if (dtype == TTAMD_BF16)
    fq_per_group_kernel<true, true><<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, n_chunks, lpg, log2_exact(lpg), nullptr,
                                                                                q, scale, zero_point, qbf, conv.eps_per_group_sym);
  else
    fq_per_group_kernel<false, true><<<dim3((unsigned)grid), dim3(256), 0, s>>>(w, n_chunks, lpg, log2_exact(lpg), nullptr,
                                                                                 q, scale, zero_point, qbf, conv.eps_per_group_sym);
  return check_launch("quantize_per_group_int4");
}

extern "C" int ttamd_dequantize_per_group_int4(const int8_t* q, const float* scale, const float* zero_point, int dtype,
                                               int64_t rows, int64_t K, int group_size, void* out, void* stream) {
  TT_REQUIRE(dtype == TTAMD_BF16 || dtype == TTAMD_F32, "dequantize_per_group_int4: unknown dtype code %d", dtype);
  TT_REQUIRE(q && scale && out && (reinterpret_cast<uintptr_t>(q) & 7u) == 0 && aligned16(out),
             "dequantize_per_group_int4: q (8-byte aligned), scale and out (16-byte aligned) must be non-null");
  TT_REQUIRE(rows > 0 && K > 0, "dequantize_per_group_int4: rows and K must be positive");
  TT_REQUIRE(group_size >= 8 && group_size <= 512 && is_pow2(group_size) && K % group_size == 0,
             "dequantize_per_group_int4: group_size (%d) must be a power of two in [8, 512] dividing K (%lld)", group_size,
             (long long)K);
  const int64_t n_chunks = rows * K / 8;
  const int64_t grid = (n_chunks + 255) / 256;
  TT_REQUIRE(grid < (int64_t(1) << 31), "dequantize_per_group_int4: tensor too large for one launch");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int l2 = log2_exact(group_size / 8);
  if (dtype == TTAMD_BF16)
    dequant_per_group_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, s>>>(q, scale, zero_point, n_chunks, l2, out);
  else
    dequant_per_group_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, s>>>(q, scale, zero_point, n_chunks, l2, out);
  return check_launch("dequantize_per_group_int4");
}

extern "C" int ttamd_fq_per_group_uint4_asym(const void* w, int dtype, int64_t rows, int64_t K, int group_size,
                                             int qparam_dtype, void* out, float* scale, float* zero_point, void* stream) {
  return ttamd_fq_per_group_uint4_asym_conv(w, dtype, rows, K, group_size, qparam_dtype, out, scale, zero_point, nullptr, stream);
}

extern "C" int ttamd_fq_per_group_uint4_asym_conv(const void* w, int dtype, int64_t rows, int64_t K, int group_size,
                                                  int qparam_dtype, void* out, float* scale, float* zero_point,
                                                  const ttamd_fq_conventions* conventions, void* stream) {
  ttamd_fq_conventions conv;
  if (int rc = resolve_conventions(conventions, &conv, "fq_per_group_uint4_asym")) return rc;
  if (int rc = check_group_args(w, dtype, rows, K, group_size)) return rc;
  TT_REQUIRE(qparam_dtype == TTAMD_BF16 || qparam_dtype == TTAMD_F32, "fq_per_group_uint4_asym: unknown qparam dtype code %d",
             qparam_dtype);
  TT_REQUIRE(out && aligned16(out), "fq_per_group_uint4_asym: out must be non-null, 16-byte aligned");
  return launch_group_asym<false>(w, dtype, qparam_dtype, rows, K, group_size, out, nullptr, scale, zero_point, conv,
                                  reinterpret_cast<hipStream_t>(stream), "fq_per_group_uint4_asym");
}

extern "C" int ttamd_quantize_per_group_uint4(const void* w, int dtype, int64_t rows, int64_t K, int group_size,
                                              int qparam_dtype, uint8_t* q, float* scale, float* zero_point, void* stream) {
  return ttamd_quantize_per_group_uint4_conv(w, dtype, rows, K, group_size, qparam_dtype, q, scale, zero_point, nullptr, stream);
}

extern "C" int ttamd_quantize_per_group_uint4_conv(const void* w, int dtype, int64_t rows, int64_t K, int group_size,
                                                   int qparam_dtype, uint8_t* q, float* scale, float* zero_point,
                                                   const ttamd_fq_conventions* conventions, void* stream) {
  ttamd_fq_conventions conv;
  if (int rc = resolve_conventions(conventions, &conv, "quantize_per_group_uint4")) return rc;
  if (int rc = check_group_args(w, dtype, rows, K, group_size)) return rc;
  TT_REQUIRE(qparam_dtype == TTAMD_BF16 || qparam_dtype == TTAMD_F32, "quantize_per_group_uint4: unknown qparam dtype code %d",
             qparam_dtype);
  TT_REQUIRE(q && scale && zero_point && (reinterpret_cast<uintptr_t>(q) & 3u) == 0,
             "quantize_per_group_uint4: q (4-byte aligned), scale and zero_point must be non-null");
  return launch_group_asym<true>(w, dtype, qparam_dtype, rows, K, group_size, nullptr, reinterpret_cast<uint32_t*>(q), scale,
                                 zero_point, conv, reinterpret_cast<hipStream_t>(stream), "quantize_per_group_uint4");
}

extern "C" int ttamd_dequantize_per_group_uint4(const uint8_t* q, const float* scale, const float* zero_point, int dtype,
                                                int64_t rows, int64_t K, int group_size, void* out, void* stream) {
  TT_REQUIRE(dtype == TTAMD_BF16 || dtype == TTAMD_F32, "dequantize_per_group_uint4: unknown dtype code %d", dtype);
  TT_REQUIRE(q && scale && zero_point && out && (reinterpret_cast<uintptr_t>(q) & 3u) == 0 && aligned16(out),
             "dequantize_per_group_uint4: q (4-byte aligned), scale, zero_point and out (16-byte aligned) must be non-null");
  TT_REQUIRE(rows > 0 && K > 0, "dequantize_per_group_uint4: rows and K must be positive");
  TT_REQUIRE(group_size >= 8 && group_size <= 512 && is_pow2(group_size) && K % group_size == 0,
             "dequantize_per_group_uint4: group_size (%d) must be a power of two in [8, 512] dividing K (%lld)", group_size,
             (long long)K);
  const int64_t n_chunks = rows * K / 8;
  const int64_t grid = (n_chunks + 255) / 256;
  TT_REQUIRE(grid < (int64_t(1) << 31), "dequantize_per_group_uint4: tensor too large for one launch");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int l2 = log2_exact(group_size / 8);
  const uint32_t* q32 = reinterpret_cast<const uint32_t*>(q);
  if (dtype == TTAMD_BF16)
    dequant_per_group_uint4_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, s>>>(q32, scale, zero_point, n_chunks, l2, out);
  else
    dequant_per_group_uint4_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, s>>>(q32, scale, zero_point, n_chunks, l2, out);
  return check_launch("dequantize_per_group_uint4");
}
