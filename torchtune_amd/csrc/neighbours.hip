// The memory-bound neighbours of the quantized linears inside a decoder layer, one pass over HBM each:
//
//   RMSNorm in fp32        torchtune/modules/rms_norm.py:28-41
//   rotary embedding       torchtune/models/llama3_1/_position_embeddings.py:128-190 (interleaved pairs, fp32 math)
//   SwiGLU gate            torchtune/modules/feed_forward.py:50-53   silu(w1 x) * w3 x
//
// and their backward passes.  In the eager reference each is a chain of 5-10 elementwise / reduction kernels that
// each read and write the whole activation; here a forward or backward is one kernel that touches every tensor once.
// Rounding points follow the eager sequence (a bf16 rounding wherever eager materialises a bf16 tensor); sums and
// transcendental functions are fp32 but not bit-identical to eager's (different summation order, hardware exp / rsqrt),
// so these kernels are checked to a tolerance, not bit for bit.
#include "common.h"
#include "nf4_math.h"
#include "swiglu_math.h"

namespace ttamd {
namespace {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  bf16x2_t v;
  v.x = (__bf16)lo;
  v.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float lo_f(uint32_t d) { return bits_f32(d << 16); }
__device__ __forceinline__ float hi_f(uint32_t d) { return bits_f32(d & 0xffff0000u); }
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// ---------------------------------------------------------------------------------------------------
// RMSNorm.  One workgroup per row, the row held in registers (NV 16-byte chunks per lane).
//   forward : xn = bf16(x * rsqrt(mean(x^2) + eps));  y = bf16(xn * scale);  rstd saved for backward
//   backward: g = bf16(gy * scale) (eager's bf16 product), c = mean(g * x) * rstd^2,
//             gx = bf16(rstd * (g - x * c));  gscale partial[w][d] = sum over workgroup w's rows of gy * xn
// ---------------------------------------------------------------------------------------------------
// Forward: a workgroup per row (four waves, NV chunks of 8 columns per lane, chunk = thread + 256 i); the sums of squares
// of the four waves meet in LDS in wave order.
// ADD: the row normalised is h = bf16(x + res) (the residual stream's addition, torchtune/modules/transformer.py:129-141),
// which the launch also writes to h_out; same bits as the addition and the norm one after the other.
template <int NV, bool ADD>
__global__ __launch_bounds__(256) void rms_norm_fwd_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ res,
                                                           const uint16_t* __restrict__ scale, float eps,
                                                           uint16_t* __restrict__ h_out, uint16_t* __restrict__ y,
                                                           float* __restrict__ rstd_out, int D) {
  __shared__ float part[4];
  const int t = threadIdx.x;
  const int64_t row = blockIdx.x;
  const int chunks = D >> 3;
  const u32x4_t* xr = reinterpret_cast<const u32x4_t*>(x + row * D);
  const u32x4_t* sr = reinterpret_cast<const u32x4_t*>(scale);
  u32x4_t v[NV], sv[NV];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = t + 256 * i;
    v[i] = u32x4_t{0, 0, 0, 0};
    sv[i] = u32x4_t{0, 0, 0, 0};
    if (c < chunks) {
      v[i] = __builtin_nontemporal_load(xr + c);
      sv[i] = sr[c];
      if constexpr (ADD) {
        const u32x4_t rv = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(res + row * D) + c);
#pragma unroll
        for (int d = 0; d < 4; ++d) v[i][d] = pack2(lo_f(v[i][d]) + lo_f(rv[d]), hi_f(v[i][d]) + hi_f(rv[d]));
        *(reinterpret_cast<u32x4_t*>(h_out + row * D) + c) = v[i];  // read again soon: by the next addition and the backward
      }
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const float a = lo_f(v[i][d]), b = hi_f(v[i][d]);
      ss += a * a;
      ss += b * b;
    }
  }
  ss = wave_sum(ss);
  if ((t & 63) == 0) part[t >> 6] = ss;
  __syncthreads();
  ss = ((part[0] + part[1]) + part[2]) + part[3];
  const float rstd = __builtin_amdgcn_rsqf(ss / (float)D + eps);
  if (t == 0 && rstd_out) rstd_out[row] = rstd;
  u32x4_t* yr = reinterpret_cast<u32x4_t*>(y + row * D);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = t + 256 * i;
    if (c >= chunks) continue;
    u32x4_t o;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const float n0 = round_to_bf16(lo_f(v[i][d]) * rstd), n1 = round_to_bf16(hi_f(v[i][d]) * rstd);
      o[d] = pack2(n0 * lo_f(sv[i][d]), n1 * hi_f(sv[i][d]));
    }
    __builtin_nontemporal_store(o, yr + c);
  }
}

// Backward: a workgroup per row (four waves, NV chunks of 8 columns per lane, chunk = thread + 256 i).  Without a scale
// gradient the grid has one workgroup per row.  With it (GSCALE) a fixed number of workgroups walk the rows with a
// stride of the grid, and a lane keeps the partial scale gradient of its own columns over all the rows its workgroup
// sees (8 NV floats); held by one wave per row, those sums took 64 registers beside the row itself and left two waves
// per SIMD with nothing in flight while they computed (3.4 TB/s at 4096 columns).  The row's dot product meets in LDS in
// wave order - the same order in both forms, so the input gradient does not depend on whether the scale is trained; the
// slot alternates with the row, so one barrier per row is enough.  Workgroup w writes row w of the partial sums (zeros
// if it saw no row).
// g_add (or null): a gradient that reaches x on another way (the residual stream); the launch then writes
// bf16(bf16(gx) + g_add), what autograd's accumulation of the two would give.
template <int NV, bool GSCALE>
__global__ __launch_bounds__(256) void rms_norm_bwd_kernel(const uint16_t* __restrict__ gy, const uint16_t* __restrict__ x,
                                                           const uint16_t* __restrict__ scale, const float* __restrict__ rstd_in,
                                                           const uint16_t* __restrict__ g_add, uint16_t* __restrict__ gx,
                                                           float* __restrict__ gscale_part, int64_t rows, int D) {
  __shared__ float dots[2][4];
  const int t = threadIdx.x, wave = t >> 6;
  const int chunks = D >> 3;
  const u32x4_t* sr = reinterpret_cast<const u32x4_t*>(scale);
  float gs[GSCALE ? NV : 1][8];
  u32x4_t sv[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if constexpr (GSCALE) {
#pragma unroll
      for (int e = 0; e < 8; ++e) gs[i][e] = 0.f;
    }
    const int c = t + 256 * i;
    sv[i] = c < chunks ? sr[c] : u32x4_t{0, 0, 0, 0};
  }
  // the next row of the workgroup is asked for before this one is worked on
  u32x4_t xv[NV], gov[NV], xn[NV], gon[NV];
  auto fetch = [&](int64_t row, u32x4_t (&xd)[NV], u32x4_t (&gd)[NV]) {
    const u32x4_t* xr = reinterpret_cast<const u32x4_t*>(x + row * D);
    const u32x4_t* gr = reinterpret_cast<const u32x4_t*>(gy + row * D);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = t + 256 * i;
      xd[i] = u32x4_t{0, 0, 0, 0};
      gd[i] = u32x4_t{0, 0, 0, 0};
      if (c < chunks) {
        xd[i] = __builtin_nontemporal_load(xr + c);
        gd[i] = __builtin_nontemporal_load(gr + c);
      }
    }
  };
  int par = 0;
  if ((int64_t)blockIdx.x < rows) fetch(blockIdx.x, xv, gov);
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x, par ^= 1) {
    const float rstd = rstd_in[row];
    if (GSCALE && row + gridDim.x < rows) fetch(row + gridDim.x, xn, gon);
    u32x4_t gv[NV];
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      // chunks beyond the row are zeros: they add nothing to the dot product and are never stored
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        if constexpr (GSCALE) {
          gs[i][2 * d] += lo_f(gov[i][d]) * round_to_bf16(lo_f(xv[i][d]) * rstd);
          gs[i][2 * d + 1] += hi_f(gov[i][d]) * round_to_bf16(hi_f(xv[i][d]) * rstd);
        }
        gv[i][d] = pack2(lo_f(gov[i][d]) * lo_f(sv[i][d]), hi_f(gov[i][d]) * hi_f(sv[i][d]));  // g = bf16(gy * scale)
        dot += lo_f(gv[i][d]) * lo_f(xv[i][d]);
        dot += hi_f(gv[i][d]) * hi_f(xv[i][d]);
      }
    }
    dot = wave_sum(dot);
    if ((t & 63) == 0) dots[par][wave] = dot;
    __syncthreads();
    dot = ((dots[par][0] + dots[par][1]) + dots[par][2]) + dots[par][3];
    const float c2 = dot / (float)D * rstd * rstd;
    u32x4_t* outr = reinterpret_cast<u32x4_t*>(gx + row * D);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = t + 256 * i;
      if (c >= chunks) continue;
      u32x4_t o;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        o[d] = pack2(rstd * (lo_f(gv[i][d]) - lo_f(xv[i][d]) * c2), rstd * (hi_f(gv[i][d]) - hi_f(xv[i][d]) * c2));
      if (g_add) {  // uniform
        const u32x4_t ga = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(g_add + row * D) + c);
#pragma unroll
        for (int d = 0; d < 4; ++d) o[d] = pack2(lo_f(o[d]) + lo_f(ga[d]), hi_f(o[d]) + hi_f(ga[d]));
      }
      __builtin_nontemporal_store(o, outr + c);
    }
    if constexpr (GSCALE) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        xv[i] = xn[i];
        gov[i] = gon[i];
      }
    }
  }
  if constexpr (!GSCALE) return;
#pragma unroll
  for (int i = 0; i < (GSCALE ? NV : 0); ++i) {
    const int c = t + 256 * i;
    if (c >= chunks) continue;
    float* p = gscale_part + (int64_t)blockIdx.x * D + 8 * c;
    *reinterpret_cast<f32x4_t*>(p) = f32x4_t{gs[i][0], gs[i][1], gs[i][2], gs[i][3]};
    *reinterpret_cast<f32x4_t*>(p + 4) = f32x4_t{gs[i][4], gs[i][5], gs[i][6], gs[i][7]};
  }
}

// gscale[d] = bf16(sum_w part[w][d]) in a fixed order: a workgroup owns 64 columns, its 16 slices of 64 threads each
// sum a contiguous range of partial rows, then the 16 slice sums are added in slice order.
__global__ __launch_bounds__(1024) void rms_norm_gscale_kernel(const float* __restrict__ part, int n_waves, int D,
                                                               uint16_t* __restrict__ gscale) {
  __shared__ float red[16][64];
  const int col = threadIdx.x & 63, slice = threadIdx.x >> 6;
  const int d = blockIdx.x * 64 + col;
  const int per = (n_waves + 15) / 16;
  const int w0 = slice * per;
  int w1 = w0 + per;
  w1 = w1 < n_waves ? w1 : n_waves;
  float s = 0.f;
  if (d < D) {
#pragma unroll 8
    for (int w = w0; w < w1; ++w) s += part[(int64_t)w * D + d];
  }
  red[slice][col] = s;
  __syncthreads();
  if (slice == 0 && d < D) {
    float t = red[0][col];
#pragma unroll
    for (int i = 1; i < 16; ++i) t += red[i][col];
    gscale[d] = f32_to_bf16_bits(t);
  }
}

constexpr int kRmsBwdWgs = 512;  // the workspace of the backward with a scale gradient holds 4 x this many partial rows
// workgroups of that backward: four per CU, all resident at once with equal shares of the rows (2048 left a second,
// mostly empty round: 46 us against 42 at 8192 x 4096; asking for a workgroup's next row ahead of time: 37 us)
constexpr int kRmsBwdGrid = 1024;
static_assert(kRmsBwdGrid <= kRmsBwdWgs * 4, "one partial row per workgroup");

// ---------------------------------------------------------------------------------------------------
// Rotary embedding on [b, s, n_h, h_d] with a [s, h_d/2, 2] fp32 (cos, sin) table; `inverse` rotates by -theta,
// which is the backward pass (the map is orthogonal).  One lane = 8 elements = 4 pairs.
// ---------------------------------------------------------------------------------------------------
// four pairs of one head at position pos, starting at element d of the head
__device__ __forceinline__ u32x4_t rope_rotate(u32x4_t v, const float* __restrict__ cache, int pos, int d, int h_d, int inverse) {
  const f32x4_t* cp = reinterpret_cast<const f32x4_t*>(cache + ((int64_t)pos * (h_d >> 1) + (d >> 1)) * 2);
  const f32x4_t c01 = cp[0], c23 = cp[1];
  const float cs[4] = {c01.x, c01.z, c23.x, c23.z};
  float sn[4] = {c01.y, c01.w, c23.y, c23.w};
  u32x4_t o;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const float a = lo_f(v[p]), b = hi_f(v[p]);
    const float s = inverse ? -sn[p] : sn[p];
    o[p] = pack2(a * cs[p] - b * s, b * cs[p] + a * s);
  }
  return o;
}

__global__ __launch_bounds__(256) void rope_kernel(const uint16_t* __restrict__ x, const float* __restrict__ cache,
                                                   uint16_t* __restrict__ y, int64_t n_chunks, int S, int row_elems, int h_d,
                                                   int inverse) {
  const int64_t chunk = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (chunk >= n_chunks) return;
  const int64_t e = chunk * 8;
  const int pos = (int)((e / row_elems) % S);
  const int d = (int)(e % h_d);  // even; h_d % 8 == 0 keeps the 4 pairs inside one head
  const u32x4_t v = *(reinterpret_cast<const u32x4_t*>(x) + chunk);
  __builtin_nontemporal_store(rope_rotate(v, cache, pos, d, h_d, inverse), reinterpret_cast<u32x4_t*>(y) + chunk);
}

// ---------------------------------------------------------------------------------------------------
// SwiGLU gate.  forward: a = bf16(silu(g)); out = bf16(a * u).
// backward: gu = bf16(go * a); ga = bf16(go * u); gg = bf16(ga * silu'(g)), silu'(g) = s (1 + g (1 - s)), s = sigmoid(g).
// ---------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const uint16_t* __restrict__ g, const uint16_t* __restrict__ u,
                                                         uint16_t* __restrict__ out, int64_t n_chunks) {
  const int64_t chunk = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (chunk >= n_chunks) return;
  const u32x4_t gv = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(g) + chunk);
  const u32x4_t uv = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(u) + chunk);
  u32x4_t o;
#pragma unroll
  for (int d = 0; d < 4; ++d) o[d] = swiglu_gate_pair(gv[d], uv[d]);
  __builtin_nontemporal_store(o, reinterpret_cast<u32x4_t*>(out) + chunk);
}

constexpr int kSwigluBwdChunks = 1;  // 16-byte chunks per lane (two measured 9 % slower)

// go and gg may be the same buffer (a lane reads its chunk of go before it writes that chunk of gg; no other lane touches it)
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const uint16_t* go, const uint16_t* __restrict__ g,
                                                         const uint16_t* __restrict__ u, uint16_t* gg,
                                                         uint16_t* __restrict__ gu, int64_t n_chunks) {
  const int64_t base = (int64_t)blockIdx.x * (256 * kSwigluBwdChunks) + threadIdx.x;
  u32x4_t ov[kSwigluBwdChunks], gv[kSwigluBwdChunks], uv[kSwigluBwdChunks];
#pragma unroll
  for (int c = 0; c < kSwigluBwdChunks; ++c) {
    const int64_t chunk = base + 256 * c;
    ov[c] = gv[c] = uv[c] = u32x4_t{0, 0, 0, 0};
    if (chunk < n_chunks) {
      ov[c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(go) + chunk);
      gv[c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(g) + chunk);
      uv[c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(u) + chunk);
    }
  }
#pragma unroll
  for (int c = 0; c < kSwigluBwdChunks; ++c) {
    const int64_t chunk = base + 256 * c;
    if (chunk >= n_chunks) continue;
    u32x4_t og, ou;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t dg, du;
      swiglu_bwd_pair(ov[c][d], gv[c][d], uv[c][d], dg, du);
      og[d] = dg;
      ou[d] = du;
    }
    __builtin_nontemporal_store(og, reinterpret_cast<u32x4_t*>(gg) + chunk);
    __builtin_nontemporal_store(ou, reinterpret_cast<u32x4_t*>(gu) + chunk);
  }
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

namespace {
int rms_norm_fwd(const char* who, const void* x, const void* res, const void* scale, float eps, void* h, void* y, float* rstd,
                 int64_t rows, int64_t D, void* stream) {
  TT_REQUIRE(x && scale && y && (res == nullptr) == (h == nullptr), "%s: null pointer argument", who);
  TT_REQUIRE(aligned16(x) && aligned16(scale) && aligned16(y) && aligned16(res) && aligned16(h), "%s: pointers must be 16-byte aligned", who);
  TT_REQUIRE(rows > 0 && D > 0 && D % 8 == 0 && D <= 8192 && rows < (int64_t(1) << 31),
             "%s: bad shape rows=%lld D=%lld (D must be a multiple of 8, at most 8192)", who, (long long)rows, (long long)D);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)rows), block(256);
  const uint16_t* X = reinterpret_cast<const uint16_t*>(x);
  const uint16_t* R = reinterpret_cast<const uint16_t*>(res);
  const uint16_t* S = reinterpret_cast<const uint16_t*>(scale);
  uint16_t* H = reinterpret_cast<uint16_t*>(h);
  uint16_t* Y = reinterpret_cast<uint16_t*>(y);
#define TT_RMS_FWD(NVV)                                                                       \
  if (res)                                                                                    \
    rms_norm_fwd_kernel<NVV, true><<<grid, block, 0, s>>>(X, R, S, eps, H, Y, rstd, (int)D);  \
  else                                                                                        \
    rms_norm_fwd_kernel<NVV, false><<<grid, block, 0, s>>>(X, nullptr, S, eps, nullptr, Y, rstd, (int)D);
  const int64_t nv = (D / 8 + 255) / 256;  // D <= 8192: at most 4
  if (nv <= 1) {
    TT_RMS_FWD(1)
  } else if (nv <= 2) {
    TT_RMS_FWD(2)
  } else {
    TT_RMS_FWD(4)
  }
#undef TT_RMS_FWD
  return check_launch(who);
}
}  // namespace

extern "C" int ttamd_rms_norm_fwd_bf16(const void* x, const void* scale, float eps, void* y, float* rstd, int64_t rows,
                                       int64_t D, void* stream) {
  return rms_norm_fwd("rms_norm_fwd", x, nullptr, scale, eps, nullptr, y, rstd, rows, D, stream);
}

extern "C" int ttamd_add_rms_norm_fwd_bf16(const void* x, const void* residual, const void* scale, float eps, void* h, void* y,
                                           float* rstd, int64_t rows, int64_t D, void* stream) {
  TT_REQUIRE(residual && h, "add_rms_norm_fwd: null pointer argument");
  return rms_norm_fwd("add_rms_norm_fwd", x, residual, scale, eps, h, y, rstd, rows, D, stream);
}

extern "C" size_t ttamd_rms_norm_bwd_workspace_bytes(int64_t D) {
  return D > 0 ? (size_t)kRmsBwdWgs * 4 * (size_t)D * sizeof(float) : 0;
}

extern "C" int ttamd_rms_norm_bwd_bf16(const void* gy, const void* x, const void* scale, const float* rstd, void* gx,
                                       void* gscale, int64_t rows, int64_t D, void* workspace, size_t workspace_bytes,
                                       void* stream) {
  return ttamd_rms_norm_bwd_add_bf16(gy, x, scale, rstd, nullptr, gx, gscale, rows, D, workspace, workspace_bytes, stream);
}

extern "C" int ttamd_rms_norm_bwd_add_bf16(const void* gy, const void* x, const void* scale, const float* rstd, const void* g_add,
                                           void* gx, void* gscale, int64_t rows, int64_t D, void* workspace,
                                           size_t workspace_bytes, void* stream) {
  TT_REQUIRE(gy && x && scale && rstd && gx, "rms_norm_bwd: null pointer argument");
  TT_REQUIRE(aligned16(gy) && aligned16(x) && aligned16(scale) && aligned16(gx) && aligned16(g_add),
             "rms_norm_bwd: pointers must be 16-byte aligned");
  TT_REQUIRE(rows > 0 && D > 0 && D % 8 == 0 && D <= 8192 && rows < (int64_t(1) << 31),
             "rms_norm_bwd: bad shape rows=%lld D=%lld (D must be a multiple of 8, at most 8192)", (long long)rows, (long long)D);
  if (gscale) {
    TT_REQUIRE(workspace && aligned16(workspace), "rms_norm_bwd: the scale gradient needs a 16-byte aligned workspace");
    if (workspace_bytes < ttamd_rms_norm_bwd_workspace_bytes(D))
      return fail(TTAMD_EWORKSPACE, "rms_norm_bwd: workspace has %zu bytes, needs %zu", workspace_bytes,
                  ttamd_rms_norm_bwd_workspace_bytes(D));
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const dim3 block(256);
  const uint16_t* G = reinterpret_cast<const uint16_t*>(gy);
  const uint16_t* X = reinterpret_cast<const uint16_t*>(x);
  const uint16_t* S = reinterpret_cast<const uint16_t*>(scale);
  uint16_t* GX = reinterpret_cast<uint16_t*>(gx);
  const uint16_t* GA = reinterpret_cast<const uint16_t*>(g_add);
  // with a scale gradient: a fixed number of workgroups that walk the rows, each of which writes one row of partial
  // sums; without: a workgroup per row
  float* part = reinterpret_cast<float*>(workspace);
  const dim3 grid(gscale ? (unsigned)kRmsBwdGrid : (unsigned)rows);
  const int64_t nv = (D / 8 + 255) / 256;  // D <= 8192: at most 4
#define TT_RMS_BWD(NVV)                                                                                          \
  if (gscale)                                                                                                    \
    rms_norm_bwd_kernel<NVV, true><<<grid, block, 0, s>>>(G, X, S, rstd, GA, GX, part, rows, (int)D);            \
  else                                                                                                           \
    rms_norm_bwd_kernel<NVV, false><<<grid, block, 0, s>>>(G, X, S, rstd, GA, GX, nullptr, rows, (int)D);
  if (nv <= 1) {
    TT_RMS_BWD(1)
  } else if (nv <= 2) {
    TT_RMS_BWD(2)
  } else {
    TT_RMS_BWD(4)
  }
#undef TT_RMS_BWD
  if (gscale)
    rms_norm_gscale_kernel<<<dim3((unsigned)((D + 63) / 64)), dim3(1024), 0, s>>>(part, kRmsBwdGrid, (int)D,
                                                                                 reinterpret_cast<uint16_t*>(gscale));
  return check_launch("rms_norm_bwd");
}

extern "C" int ttamd_rope_bf16(const void* x, const float* cache, void* y, int64_t B, int64_t S, int64_t n_heads,
                               int64_t head_dim, int inverse, void* stream) {
  TT_REQUIRE(x && cache && y, "rope: null pointer argument");
  TT_REQUIRE(aligned16(x) && aligned16(cache) && aligned16(y), "rope: pointers must be 16-byte aligned");
  TT_REQUIRE(B > 0 && S > 0 && n_heads > 0 && head_dim > 0 && head_dim % 8 == 0 && S < (1 << 30) && n_heads * head_dim < (1 << 30),
             "rope: bad shape b=%lld s=%lld n_h=%lld h_d=%lld (h_d must be a multiple of 8)", (long long)B, (long long)S,
             (long long)n_heads, (long long)head_dim);
  const int64_t n_chunks = B * S * n_heads * head_dim / 8;
  TT_REQUIRE((n_chunks + 255) / 256 < (int64_t(1) << 31), "rope: tensor too large for one launch");
  rope_kernel<<<dim3((unsigned)((n_chunks + 255) / 256)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const uint16_t*>(x), cache, reinterpret_cast<uint16_t*>(y), n_chunks, (int)S, (int)(n_heads * head_dim),
      (int)head_dim, inverse);
  return check_launch("rope");
}

namespace ttamd {
namespace {

// Grouped-query expansion: y[t][kv * rep + r][:] = x[t][kv][:] for r < rep (t = token).  One thread per 16-byte chunk of
// the OUTPUT, so the writes (rep times the reads) are whole lines; the repeated reads hit in cache.
__global__ __launch_bounds__(256) void repeat_kv_kernel(const u32x4_t* __restrict__ x, u32x4_t* __restrict__ y, int64_t n_out,
                                                        int chunks_per_head, int n_kv, int rep) {
  const int64_t oc = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (oc >= n_out) return;
  const int64_t out_head = oc / chunks_per_head;  // token * (n_kv * rep) + kv * rep + r
  const int c = (int)(oc - out_head * chunks_per_head);
  const int64_t tok = out_head / (n_kv * rep);
  const int kv = (int)(out_head - tok * (n_kv * rep)) / rep;
  y[oc] = x[(tok * n_kv + kv) * chunks_per_head + c];
}

// bf16(sum_r gy[in_head * rep + r][c]), fp32 sums in the order r = 0 .. rep - 1
__device__ __forceinline__ u32x4_t sum_head_copies(const u32x4_t* __restrict__ gy, int64_t in_head, int c, int chunks_per_head,
                                                   int rep) {
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int r = 0; r < rep; ++r) {
    const u32x4_t v = gy[(in_head * rep + r) * chunks_per_head + c];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      acc[2 * d] += bits_f32(v[d] << 16);
      acc[2 * d + 1] += bits_f32(v[d] & 0xffff0000u);
    }
  }
  u32x4_t o;
#pragma unroll
  for (int d = 0; d < 4; ++d) o[d] = (uint32_t)f32_to_bf16_bits(acc[2 * d]) | ((uint32_t)f32_to_bf16_bits(acc[2 * d + 1]) << 16);
  return o;
}

// Its backward: gx[t][kv][:] = bf16(sum_r gy[t][kv * rep + r][:]).
__global__ __launch_bounds__(256) void repeat_kv_bwd_kernel(const u32x4_t* __restrict__ gy, u32x4_t* __restrict__ gx, int64_t n_in,
                                                            int chunks_per_head, int rep) {
  const int64_t ic = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (ic >= n_in) return;
  const int64_t in_head = ic / chunks_per_head;
  const int c = (int)(ic - in_head * chunks_per_head);
  gx[ic] = sum_head_copies(gy, in_head, c, chunks_per_head, rep);
}

// Everything between the q / k / v projections and the attention in one launch
// (torchtune/modules/attention.py:255-290: rotary embedding of q and k, expansion of the k / v heads):
// q_out = rope(q), k_out = repeat(rope(k)), v_out = repeat(v).  One thread per 16-byte chunk of the three outputs
// (nq chunks each); the same bits as rope_kernel followed by repeat_kv_kernel.
__global__ __launch_bounds__(256) void qkv_rope_repeat_kernel(const u32x4_t* __restrict__ q, const u32x4_t* __restrict__ k,
                                                              const u32x4_t* __restrict__ v, const float* __restrict__ cache,
                                                              u32x4_t* __restrict__ qo, u32x4_t* __restrict__ ko,
                                                              u32x4_t* __restrict__ vo, int64_t nq, int S, int n_heads, int n_kv,
                                                              int chunks_per_head) {
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= 3 * nq) return;
  const int seg = (int)(g / nq);
  const int64_t oc = g - seg * nq;
  const int64_t out_head = oc / chunks_per_head;  // token * n_heads + head
  const int c = (int)(oc - out_head * chunks_per_head);
  const int64_t tok = out_head / n_heads;
  const int pos = (int)(tok % S);
  const int h_d = chunks_per_head * 8;
  if (seg == 0) {
    __builtin_nontemporal_store(rope_rotate(__builtin_nontemporal_load(q + oc), cache, pos, c * 8, h_d, 0), qo + oc);
    return;
  }
  const int rep = n_heads / n_kv;
  const int kv = (int)(out_head - tok * n_heads) / rep;
  const int64_t src = (tok * n_kv + kv) * chunks_per_head + c;
  if (seg == 1)
    __builtin_nontemporal_store(rope_rotate(k[src], cache, pos, c * 8, h_d, 0), ko + oc);
  else
    __builtin_nontemporal_store(v[src], vo + oc);
}

// Its backward: gq = rope^-1(gq_out), gk = rope^-1(bf16(sum of the copies' gradients)), gv = bf16(sum of the copies'
// gradients); the same bits as repeat_kv_bwd_kernel followed by rope_kernel with inverse = 1.  The k / v threads (rep
// reads each) come first.
__global__ __launch_bounds__(256) void qkv_rope_repeat_bwd_kernel(const u32x4_t* __restrict__ gqo, const u32x4_t* __restrict__ gko,
                                                                  const u32x4_t* __restrict__ gvo, const float* __restrict__ cache,
                                                                  u32x4_t* __restrict__ gq, u32x4_t* __restrict__ gk,
                                                                  u32x4_t* __restrict__ gv, int64_t nq, int64_t nkv, int S,
                                                                  int n_heads, int n_kv, int chunks_per_head) {
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= 2 * nkv + nq) return;
  const int h_d = chunks_per_head * 8;
  if (g >= 2 * nkv) {
    const int64_t oc = g - 2 * nkv;
    const int64_t head = oc / chunks_per_head;
    const int c = (int)(oc - head * chunks_per_head);
    const int pos = (int)((head / n_heads) % S);
    __builtin_nontemporal_store(rope_rotate(__builtin_nontemporal_load(gqo + oc), cache, pos, c * 8, h_d, 1), gq + oc);
    return;
  }
  const bool is_k = g < nkv;
  const int64_t ic = is_k ? g : g - nkv;
  const int64_t in_head = ic / chunks_per_head;  // token * n_kv + kv
  const int c = (int)(ic - in_head * chunks_per_head);
  const u32x4_t sum = sum_head_copies(is_k ? gko : gvo, in_head, c, chunks_per_head, n_heads / n_kv);
  if (is_k)
    __builtin_nontemporal_store(rope_rotate(sum, cache, (int)((in_head / n_kv) % S), c * 8, h_d, 1), gk + ic);
  else
    __builtin_nontemporal_store(sum, gv + ic);
}

int check_repeat_kv(const char* who, const void* a, const void* b, int64_t tokens, int64_t n_kv, int64_t rep, int64_t head_dim) {
  TT_REQUIRE(a && b, "%s: null pointer argument", who);
  TT_REQUIRE(aligned16(a) && aligned16(b), "%s: pointers must be 16-byte aligned", who);
  TT_REQUIRE(tokens > 0 && n_kv > 0 && rep > 0 && head_dim > 0 && head_dim % 8 == 0 && n_kv * rep < (1 << 20) &&
                 head_dim < (1 << 20),
             "%s: bad shape tokens=%lld n_kv=%lld rep=%lld h_d=%lld (h_d must be a multiple of 8)", who, (long long)tokens,
             (long long)n_kv, (long long)rep, (long long)head_dim);
  TT_REQUIRE((tokens * n_kv * rep * (head_dim / 8) + 255) / 256 < (int64_t(1) << 31), "%s: tensor too large for one launch", who);
  return TTAMD_OK;
}

}  // namespace
}  // namespace ttamd

extern "C" int ttamd_repeat_kv_bf16(const void* x, void* y, int64_t tokens, int64_t n_kv, int64_t rep, int64_t head_dim,
                                    void* stream) {
  if (int rc = check_repeat_kv("repeat_kv", x, y, tokens, n_kv, rep, head_dim)) return rc;
  const int64_t n_out = tokens * n_kv * rep * (head_dim / 8);
  repeat_kv_kernel<<<dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const u32x4_t*>(x), reinterpret_cast<u32x4_t*>(y), n_out, (int)(head_dim / 8), (int)n_kv, (int)rep);
  return check_launch("repeat_kv");
}

extern "C" int ttamd_repeat_kv_bwd_bf16(const void* gy, void* gx, int64_t tokens, int64_t n_kv, int64_t rep, int64_t head_dim,
                                        void* stream) {
  if (int rc = check_repeat_kv("repeat_kv_bwd", gy, gx, tokens, n_kv, rep, head_dim)) return rc;
  const int64_t n_in = tokens * n_kv * (head_dim / 8);
  repeat_kv_bwd_kernel<<<dim3((unsigned)((n_in + 255) / 256)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const u32x4_t*>(gy), reinterpret_cast<u32x4_t*>(gx), n_in, (int)(head_dim / 8), (int)rep);
  return check_launch("repeat_kv_bwd");
}

namespace {
int check_qkv_rope_repeat(const char* who, const void* const* ptrs, const float* cache, int64_t B, int64_t S, int64_t n_heads,
                          int64_t n_kv, int64_t head_dim) {
  for (int i = 0; i < 6; ++i) {
    TT_REQUIRE(ptrs[i], "%s: null pointer argument", who);
    TT_REQUIRE(aligned16(ptrs[i]), "%s: pointers must be 16-byte aligned", who);
  }
  TT_REQUIRE(cache && aligned16(cache), "%s: the cache must be a 16-byte aligned pointer", who);
  TT_REQUIRE(B > 0 && S > 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0 && head_dim > 0 && head_dim % 8 == 0 &&
                 S < (1 << 30) && n_heads < (1 << 20) && head_dim < (1 << 20),
             "%s: bad shape b=%lld s=%lld n_h=%lld n_kv=%lld h_d=%lld (n_h a multiple of n_kv, h_d a multiple of 8)", who,
             (long long)B, (long long)S, (long long)n_heads, (long long)n_kv, (long long)head_dim);
  TT_REQUIRE((3 * B * S * n_heads * (head_dim / 8) + 255) / 256 < (int64_t(1) << 31), "%s: tensors too large for one launch", who);
  return TTAMD_OK;
}
}  // namespace

extern "C" int ttamd_qkv_rope_repeat_bf16(const void* q, const void* k, const void* v, const float* cache, void* q_out,
                                          void* k_out, void* v_out, int64_t B, int64_t S, int64_t n_heads, int64_t n_kv,
                                          int64_t head_dim, void* stream) {
  const void* ptrs[6] = {q, k, v, q_out, k_out, v_out};
  if (int rc = check_qkv_rope_repeat("qkv_rope_repeat", ptrs, cache, B, S, n_heads, n_kv, head_dim)) return rc;
  const int64_t nq = B * S * n_heads * (head_dim / 8);
  qkv_rope_repeat_kernel<<<dim3((unsigned)((3 * nq + 255) / 256)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const u32x4_t*>(q), reinterpret_cast<const u32x4_t*>(k), reinterpret_cast<const u32x4_t*>(v), cache,
      reinterpret_cast<u32x4_t*>(q_out), reinterpret_cast<u32x4_t*>(k_out), reinterpret_cast<u32x4_t*>(v_out), nq, (int)S,
      (int)n_heads, (int)n_kv, (int)(head_dim / 8));
  return check_launch("qkv_rope_repeat");
}

extern "C" int ttamd_qkv_rope_repeat_bwd_bf16(const void* gq_out, const void* gk_out, const void* gv_out, const float* cache,
                                              void* gq, void* gk, void* gv, int64_t B, int64_t S, int64_t n_heads, int64_t n_kv,
                                              int64_t head_dim, void* stream) {
  const void* ptrs[6] = {gq_out, gk_out, gv_out, gq, gk, gv};
  if (int rc = check_qkv_rope_repeat("qkv_rope_repeat_bwd", ptrs, cache, B, S, n_heads, n_kv, head_dim)) return rc;
  const int64_t nq = B * S * n_heads * (head_dim / 8), nkv = B * S * n_kv * (head_dim / 8);
  qkv_rope_repeat_bwd_kernel<<<dim3((unsigned)((2 * nkv + nq + 255) / 256)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const u32x4_t*>(gq_out), reinterpret_cast<const u32x4_t*>(gk_out),
      reinterpret_cast<const u32x4_t*>(gv_out), cache, reinterpret_cast<u32x4_t*>(gq), reinterpret_cast<u32x4_t*>(gk),
      reinterpret_cast<u32x4_t*>(gv), nq, nkv, (int)S, (int)n_heads, (int)n_kv, (int)(head_dim / 8));
  return check_launch("qkv_rope_repeat_bwd");
}

extern "C" int ttamd_swiglu_fwd_bf16(const void* gate, const void* up, void* out, int64_t numel, void* stream) {
  TT_REQUIRE(gate && up && out, "swiglu_fwd: null pointer argument");
  TT_REQUIRE(aligned16(gate) && aligned16(up) && aligned16(out), "swiglu_fwd: pointers must be 16-byte aligned");
  TT_REQUIRE(numel > 0 && numel % 8 == 0 && (numel / 8 + 255) / 256 < (int64_t(1) << 31), "swiglu_fwd: numel (%lld) must be a positive multiple of 8",
             (long long)numel);
  const int64_t n_chunks = numel / 8;
  swiglu_fwd_kernel<<<dim3((unsigned)((n_chunks + 255) / 256)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const uint16_t*>(gate), reinterpret_cast<const uint16_t*>(up), reinterpret_cast<uint16_t*>(out), n_chunks);
  return check_launch("swiglu_fwd");
}

extern "C" int ttamd_swiglu_bwd_bf16(const void* gout, const void* gate, const void* up, void* ggate, void* gup, int64_t numel,
                                     void* stream) {
  TT_REQUIRE(gout && gate && up && ggate && gup, "swiglu_bwd: null pointer argument");
  TT_REQUIRE(aligned16(gout) && aligned16(gate) && aligned16(up) && aligned16(ggate) && aligned16(gup),
             "swiglu_bwd: pointers must be 16-byte aligned");
  TT_REQUIRE(numel > 0 && numel % 8 == 0 && (numel / 8 + 255) / 256 < (int64_t(1) << 31), "swiglu_bwd: numel (%lld) must be a positive multiple of 8",
             (long long)numel);
  const int64_t n_chunks = numel / 8;
  const int64_t per_wg = 256 * kSwigluBwdChunks;
  swiglu_bwd_kernel<<<dim3((unsigned)((n_chunks + per_wg - 1) / per_wg)), dim3(256), 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const uint16_t*>(gout), reinterpret_cast<const uint16_t*>(gate), reinterpret_cast<const uint16_t*>(up),
      reinterpret_cast<uint16_t*>(ggate), reinterpret_cast<uint16_t*>(gup), n_chunks);
  return check_launch("swiglu_bwd");
}

// ---------------------------------------------------------------------------------------------------
// Cross entropy over bf16 logits, forward and backward in one pass (the per-chunk body of the reference's
// LinearCrossEntropyLoss, torchtune/modules/loss/cross_entropy_loss.py:86-112: F.cross_entropy(logits.float(),
// target, reduction="sum", ignore_index)).  A workgroup of 1024 threads holds one row of logits in registers
// (16 chunks of 8 per thread: up to 131072 classes), reduces max and sum of exponentials through LDS, and writes
//   loss[row]  = logsumexp(row) - row[target]                      (0 for an ignored row)
//   grad[row]  = bf16(grad_scale * (softmax(row) - onehot(target)))  (0 for an ignored row)
// so the logits are read once and never widened to fp32 in memory.
// ---------------------------------------------------------------------------------------------------
namespace ttamd {
namespace {

constexpr int kCeThreads = 1024;
constexpr int kCeChunks = 16;

__global__ __launch_bounds__(kCeThreads) void cross_entropy_kernel(const uint16_t* __restrict__ logits,
                                                                    const int64_t* __restrict__ target, int64_t ignore_index,
                                                                    float grad_scale, float* __restrict__ loss,
                                                                    uint16_t* __restrict__ grad, int V) {
  __shared__ float red[kCeThreads / 64];
  __shared__ float bcast;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int64_t row = blockIdx.x;
  const int chunks = V >> 3;
  const u32x4_t* xr = reinterpret_cast<const u32x4_t*>(logits + row * V);
  u32x4_t* gr = reinterpret_cast<u32x4_t*>(grad + row * V);
  const int64_t tgt = target[row];
  if (tgt == ignore_index) {  // uniform over the workgroup
    for (int i = 0; i < kCeChunks; ++i) {
      const int c = t + kCeThreads * i;
      if (c < chunks) __builtin_nontemporal_store(u32x4_t{0, 0, 0, 0}, gr + c);
    }
    if (t == 0) loss[row] = 0.f;
    return;
  }
  u32x4_t v[kCeChunks];
  float mx = -__builtin_inff();
#pragma unroll
  for (int i = 0; i < kCeChunks; ++i) {
    const int c = t + kCeThreads * i;
    v[i] = u32x4_t{0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u};  // -inf pairs: neutral for max and exp
    if (c < chunks) v[i] = __builtin_nontemporal_load(xr + c);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      mx = __builtin_fmaxf(mx, lo_f(v[i][d]));
      mx = __builtin_fmaxf(mx, hi_f(v[i][d]));
    }
  }
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) mx = __builtin_fmaxf(mx, __shfl_xor(mx, off, kWave));
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  if (t == 0) {
    float m = red[0];
    for (int w = 1; w < kCeThreads / 64; ++w) m = __builtin_fmaxf(m, red[w]);
    bcast = m;
  }
  __syncthreads();
  mx = bcast;
  // Each pass unpacks the row from its packed registers again: the barriers stop the compiler from keeping the 128
  // unpacked (or exponentiated) values of one pass alive for the next, which would not fit the 128 registers a
  // 1024-thread workgroup leaves each lane and would spill to scratch memory (three times the kernel's HBM traffic).
#pragma unroll
  for (int i = 0; i < kCeChunks; ++i) asm volatile("" : "+v"(v[i]));
  float se = 0.f;
#pragma unroll
  for (int i = 0; i < kCeChunks; ++i)
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      se += __builtin_amdgcn_exp2f((lo_f(v[i][d]) - mx) * 1.4426950408889634f);
      se += __builtin_amdgcn_exp2f((hi_f(v[i][d]) - mx) * 1.4426950408889634f);
    }
  se = wave_sum(se);
  __syncthreads();  // everyone has read bcast
  if (lane == 0) red[wave] = se;
  __syncthreads();
  if (t == 0) {
    float s = red[0];
    for (int w = 1; w < kCeThreads / 64; ++w) s += red[w];
    bcast = s;
  }
  __syncthreads();
  se = bcast;
  const float inv = grad_scale / se;
#pragma unroll
  for (int i = 0; i < kCeChunks; ++i) asm volatile("" : "+v"(v[i]));
  if (t == 0) {
    const bool valid = tgt >= 0 && tgt < V;  // an out-of-range class gives NaN, never an out-of-bounds read
    const float xt = bf16_bits_to_f32(logits[row * V + (valid ? tgt : 0)]);
    loss[row] = valid ? (mx - xt) + __builtin_logf(se) : __builtin_nanf("");
  }
#pragma unroll
  for (int i = 0; i < kCeChunks; ++i) {
    const int c = t + kCeThreads * i;
    if (c >= chunks) continue;
    float p[8];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      p[2 * d] = __builtin_amdgcn_exp2f((lo_f(v[i][d]) - mx) * 1.4426950408889634f) * inv;
      p[2 * d + 1] = __builtin_amdgcn_exp2f((hi_f(v[i][d]) - mx) * 1.4426950408889634f) * inv;
    }
    const int64_t e0 = (int64_t)c * 8;
    if (tgt >= e0 && tgt < e0 + 8) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (e0 + e == tgt) p[e] -= grad_scale;
    }
    u32x4_t o;
#pragma unroll
    for (int d = 0; d < 4; ++d) o[d] = pack2(p[2 * d], p[2 * d + 1]);
    __builtin_nontemporal_store(o, gr + c);
  }
}

}  // namespace
}  // namespace ttamd

extern "C" int ttamd_cross_entropy_fwd_bwd_bf16(const void* logits, const int64_t* target, int64_t ignore_index, float grad_scale,
                                                float* loss, void* grad_logits, int64_t rows, int64_t V, void* stream) {
  TT_REQUIRE(logits && target && loss && grad_logits, "cross_entropy: null pointer argument");
  TT_REQUIRE(aligned16(logits) && aligned16(grad_logits), "cross_entropy: logits and grad_logits must be 16-byte aligned");
  TT_REQUIRE(rows > 0 && rows < (int64_t(1) << 31) && V > 0 && V % 8 == 0, "cross_entropy: bad shape rows=%lld V=%lld (V must be a multiple of 8)",
             (long long)rows, (long long)V);
  if (V > (int64_t)kCeThreads * kCeChunks * 8)
    return fail(TTAMD_EUNSUPPORTED, "cross_entropy: V (%lld) exceeds the %d classes one workgroup holds in registers", (long long)V,
                kCeThreads * kCeChunks * 8);
  cross_entropy_kernel<<<dim3((unsigned)rows), dim3(kCeThreads), 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const uint16_t*>(logits), target, ignore_index, grad_scale, loss, reinterpret_cast<uint16_t*>(grad_logits),
      (int)V);
  return check_launch("cross_entropy");
}
