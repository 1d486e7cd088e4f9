// The rank-r ("skinny") products of the LoRA adapter on gfx950.  All four are HBM-bound: each streams one
// [M, K] or [M, N] activation once and produces an output with only `rank` rows or columns.
//
//   h  = x  . A^T        [M,R]   contraction over K  (forward)
//   gh = s . gy . B      [M,R]   contraction over N  (backward)
//   gA = gh^T . x        [R,K]   contraction over M  (backward)
//   gB = s . gy^T . h    [N,R]   contraction over M  (backward)
//
// The first two contract along the contiguous dimension of the activation: MFMA with the activation rows
// as the A operand, fragments loaded straight from global memory (a lane's 8 contraction elements are 16
// contiguous bytes).  The last two contract over rows; a lane owns 4 consecutive columns and accumulates
// 4 x 16 outputs with scalar-broadcast adapter values.  Both split the contraction over many workgroups to
// put enough loads in flight and combine the fp32 partial sums in a second, fixed-order pass, so results
// are deterministic.
#include "common.h"
#include "nf4_math.h"

namespace ttamd {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------------------------------------------
// skinny_nt: part[split][m][r] = sum_{k in split} X[m][k] * Bm[r][k]        (X [M,Kc], Bm [R,Kc], R <= 64)
// One wave = 32 rows of X x one split of Kc; RT = number of 32-column tiles of R.
// ---------------------------------------------------------------------------------------------------
template <int RT>
__global__ __launch_bounds__(256) void skinny_nt_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ Bm,
                                                        float* __restrict__ part, int M, int Kc, int R, int m_tiles,
                                                        int splits, int chunks_per_split) {
  const int wave_global = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wave_global >= m_tiles * splits) return;
  const int mt = wave_global % m_tiles, split = wave_global / m_tiles;
  const int lane = threadIdx.x & 63, l31 = lane & 31, lhi = lane >> 5;
  int row = mt * 32 + l31;
  row = row < M ? row : M - 1;
  const uint16_t* xrow = X + (int64_t)row * Kc + 8 * lhi;
  const uint16_t* brow[RT];
  bool bvalid[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int r = t * 32 + l31;
    bvalid[t] = r < R;
    brow[t] = Bm + (int64_t)(bvalid[t] ? r : 0) * Kc + 8 * lhi;
  }
  f32x16_t acc[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

  const int total_chunks = Kc >> 6;
  const int c0 = split * chunks_per_split;
  int c1 = c0 + chunks_per_split;
  c1 = c1 < total_chunks ? c1 : total_chunks;
  for (int c = c0; c < c1; ++c) {
    const int k0 = c * 64;
    bf16x8_t a[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) a[s] = *reinterpret_cast<const bf16x8_t*>(xrow + k0 + 16 * s);
#pragma unroll
    for (int t = 0; t < RT; ++t) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        u32x4_t raw = {0, 0, 0, 0};
        if (bvalid[t]) raw = *reinterpret_cast<const u32x4_t*>(brow[t] + k0 + 16 * s);
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s], __builtin_bit_cast(bf16x8_t, raw), acc[t], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int col = t * 32 + l31;
    if (col >= R) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int r = mt * 32 + 8 * (v >> 2) + 4 * lhi + (v & 3);
      if (r < M) part[((int64_t)split * M + r) * R + col] = acc[t][v];
    }
  }
}

// out[i] = bf16(scale * sum_s part[s][i]) for i < n (out and part share the [M,R] layout)
__global__ __launch_bounds__(256) void sum_partials_kernel(const float* __restrict__ part, int64_t n, int splits, float scale,
                                                           uint16_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
  for (int p = 0; p < splits; ++p) s += part[(int64_t)p * n + i];
  out[i] = f32_to_bf16_bits(s * scale);
}

// out[r][n] = in[n][r]
__global__ __launch_bounds__(256) void transpose_small_kernel(const uint16_t* __restrict__ in, int64_t rows, int cols,
                                                              uint16_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * cols) return;
  const int64_t r = i / cols;
  const int c = (int)(i % cols);
  out[(int64_t)c * rows + r] = in[i];
}

// ---------------------------------------------------------------------------------------------------
// skinny_tn: part[split][r][k] = sum_{m in split} G[m][r0 + r] * X[m][k]      (G [M,R], X [M,Kc])
// Workgroup = 4 waves on the same 256 columns, each wave a quarter of the split's rows; lane owns 4 columns.
// ---------------------------------------------------------------------------------------------------
template <int RC>
__global__ __launch_bounds__(256) void skinny_tn_kernel(const uint16_t* __restrict__ G, const uint16_t* __restrict__ X,
                                                        float* __restrict__ part, int M, int Kc, int R, int r0,
                                                        int rows_per_split) {
  __shared__ float red[3][RC * 4][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int col = blockIdx.x * 256 + lane * 4;
  const bool col_ok = col < Kc;  // Kc % 8 == 0, so a lane's 4 columns are in or out together
  const int split = blockIdx.y;
  const int m_begin = split * rows_per_split;
  int m_end = m_begin + rows_per_split;
  m_end = m_end < M ? m_end : M;
  float acc[RC][4];
#pragma unroll
  for (int r = 0; r < RC; ++r)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[r][e] = 0.f;

  const uint16_t* xcol = X + (col_ok ? col : 0);
  for (int m = m_begin + wave; m < m_end; m += 4) {
    u32x2_t xv = {0, 0};
    if (col_ok) xv = *reinterpret_cast<const u32x2_t*>(xcol + (int64_t)m * Kc);
    const float x0 = bits_f32(xv.x << 16), x1 = bits_f32(xv.x & 0xffff0000u);
    const float x2 = bits_f32(xv.y << 16), x3 = bits_f32(xv.y & 0xffff0000u);
    const uint32_t* grow = reinterpret_cast<const uint32_t*>(G + (int64_t)m * R + r0);  // wave-uniform address
#pragma unroll
    for (int rp = 0; rp < RC / 2; ++rp) {
      const uint32_t gp = grow[rp];
      const float g0 = bits_f32(gp << 16), g1 = bits_f32(gp & 0xffff0000u);
      acc[2 * rp][0] += g0 * x0; acc[2 * rp][1] += g0 * x1; acc[2 * rp][2] += g0 * x2; acc[2 * rp][3] += g0 * x3;
      acc[2 * rp + 1][0] += g1 * x0; acc[2 * rp + 1][1] += g1 * x1; acc[2 * rp + 1][2] += g1 * x2; acc[2 * rp + 1][3] += g1 * x3;
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int r = 0; r < RC; ++r)
#pragma unroll
      for (int e = 0; e < 4; ++e) red[wave - 1][r * 4 + e][lane] = acc[r][e];
  }
  __syncthreads();
  if (wave == 0 && col_ok) {
#pragma unroll
    for (int r = 0; r < RC; ++r) {
      f32x4_t o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = ((acc[r][e] + red[0][r * 4 + e][lane]) + red[1][r * 4 + e][lane]) + red[2][r * 4 + e][lane];
      *reinterpret_cast<f32x4_t*>(part + ((int64_t)split * R + r0 + r) * Kc + col) = o;
    }
  }
}

// out[r*stride_r + k*stride_k] = bf16(scale * sum_s part[s][r][k])
__global__ __launch_bounds__(256) void sum_partials_tn_kernel(const float* __restrict__ part, int R, int Kc, int splits,
                                                              float scale, int64_t stride_r, int64_t stride_k,
                                                              uint16_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t n = (int64_t)R * Kc;
  if (i >= n) return;
  float s = 0.f;
  for (int p = 0; p < splits; ++p) s += part[(int64_t)p * n + i];
  const int64_t r = i / Kc, k = i % Kc;
  out[r * stride_r + k * stride_k] = f32_to_bf16_bits(s * scale);
}

constexpr int kTargetWaves = 4096;

struct NtPlan {
  int m_tiles, splits, chunks_per_split;
};
NtPlan plan_nt(int64_t M, int64_t Kc) {
  NtPlan p;
  p.m_tiles = (int)((M + 31) / 32);
  const int total_chunks = (int)(Kc / 64);
  int s = kTargetWaves / p.m_tiles;
  s = s < 1 ? 1 : s;
  s = s > total_chunks ? total_chunks : s;
  p.chunks_per_split = (total_chunks + s - 1) / s;
  p.splits = (total_chunks + p.chunks_per_split - 1) / p.chunks_per_split;
  return p;
}
size_t nt_ws_bytes(int64_t M, int64_t Kc, int R) { return (size_t)plan_nt(M, Kc).splits * M * R * sizeof(float); }

struct TnPlan {
  int col_groups, splits, rows_per_split;
};
TnPlan plan_tn(int64_t M, int64_t Kc) {
  TnPlan p;
  p.col_groups = (int)((Kc + 255) / 256);
  int s = kTargetWaves / 4 / p.col_groups;
  s = s < 1 ? 1 : s;
  const int max_s = (int)((M + 15) / 16);  // at least 4 rows per wave
  s = s > max_s ? max_s : s;
  p.rows_per_split = (int)((M + s - 1) / s);
  p.splits = (int)((M + p.rows_per_split - 1) / p.rows_per_split);
  return p;
}
size_t tn_ws_bytes(int64_t M, int64_t Kc, int R) { return (size_t)plan_tn(M, Kc).splits * R * Kc * sizeof(float); }

size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

int run_nt(const uint16_t* X, const uint16_t* Bm, int64_t M, int64_t Kc, int R, float scale, uint16_t* out, float* ws,
           hipStream_t s) {
  const NtPlan p = plan_nt(M, Kc);
  const int waves = p.m_tiles * p.splits;
  const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  if (R <= 32)
    skinny_nt_kernel<1><<<grid, block, 0, s>>>(X, Bm, ws, (int)M, (int)Kc, R, p.m_tiles, p.splits, p.chunks_per_split);
  else
    skinny_nt_kernel<2><<<grid, block, 0, s>>>(X, Bm, ws, (int)M, (int)Kc, R, p.m_tiles, p.splits, p.chunks_per_split);
  const int64_t n = M * R;
  sum_partials_kernel<<<dim3((unsigned)((n + 255) / 256)), block, 0, s>>>(ws, n, p.splits, scale, out);
  return check_launch("skinny_nt");
}

int run_tn(const uint16_t* G, const uint16_t* X, int64_t M, int64_t Kc, int R, float scale, int64_t stride_r,
           int64_t stride_k, uint16_t* out, float* ws, hipStream_t s) {
  const TnPlan p = plan_tn(M, Kc);
  const dim3 grid((unsigned)p.col_groups, (unsigned)p.splits), block(256);
  int r0 = 0;
  for (; r0 + 16 <= R; r0 += 16)
    skinny_tn_kernel<16><<<grid, block, 0, s>>>(G, X, ws, (int)M, (int)Kc, R, r0, p.rows_per_split);
  if (r0 < R) skinny_tn_kernel<8><<<grid, block, 0, s>>>(G, X, ws, (int)M, (int)Kc, R, r0, p.rows_per_split);
  const int64_t n = (int64_t)R * Kc;
  sum_partials_tn_kernel<<<dim3((unsigned)((n + 255) / 256)), block, 0, s>>>(ws, R, (int)Kc, p.splits, scale, stride_r,
                                                                             stride_k, out);
  return check_launch("skinny_tn");
}

int check_skinny(const char* who, int64_t M, int64_t N, int64_t K, int rank) {
  TT_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1 << 30) && N < (1 << 30) && K < (1 << 30), "%s: bad shape M=%lld N=%lld K=%lld",
             who, (long long)M, (long long)N, (long long)K);
  TT_REQUIRE(K % 64 == 0 && N % 64 == 0, "%s: K (%lld) and N (%lld) must be multiples of 64", who, (long long)K, (long long)N);
  TT_REQUIRE(rank > 0 && rank <= 64 && rank % 8 == 0, "%s: rank (%d) must be a multiple of 8 in [8, 64]", who, rank);
  return TTAMD_OK;
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" size_t ttamd_lora_fwd_workspace_bytes(int64_t M, int64_t K, int rank) {
  if (M <= 0 || K <= 0 || rank <= 0 || K % 64) return 0;
  return align256(nt_ws_bytes(M, K, rank));
}

extern "C" int ttamd_lora_hidden_bf16(const void* x, const void* lora_a, void* h, int64_t M, int64_t K, int rank,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_skinny("lora_hidden", M, 64, K, rank)) return rc;
  TT_REQUIRE(x && lora_a && h && workspace, "lora_hidden: null pointer argument");
  TT_REQUIRE(aligned16(x) && aligned16(lora_a) && aligned16(workspace), "lora_hidden: pointers must be 16-byte aligned");
  if (workspace_bytes < ttamd_lora_fwd_workspace_bytes(M, K, rank))
    return fail(TTAMD_EWORKSPACE, "lora_hidden: workspace has %zu bytes, needs %zu", workspace_bytes,
                ttamd_lora_fwd_workspace_bytes(M, K, rank));
  return run_nt(reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint16_t*>(lora_a), M, K, rank, 1.0f,
                reinterpret_cast<uint16_t*>(h), reinterpret_cast<float*>(workspace), reinterpret_cast<hipStream_t>(stream));
}

extern "C" size_t ttamd_lora_bwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int rank) {
  if (M <= 0 || N <= 0 || K <= 0 || rank <= 0 || K % 64 || N % 64) return 0;
  size_t a = nt_ws_bytes(M, N, rank), b = tn_ws_bytes(M, K, rank), c = tn_ws_bytes(M, N, rank);
  size_t big = a > b ? a : b;
  big = big > c ? big : c;
  return align256((size_t)N * rank * sizeof(uint16_t)) + align256(big);
}

extern "C" int ttamd_lora_bwd_bf16(const void* gy, const void* x, const void* h, const void* lora_b, float scale, void* gh,
                                   void* ga, void* gb, int64_t M, int64_t N, int64_t K, int rank, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  if (int rc = check_skinny("lora_bwd", M, N, K, rank)) return rc;
  TT_REQUIRE(gy && x && h && lora_b && gh && ga && gb && workspace, "lora_bwd: null pointer argument");
  TT_REQUIRE(aligned16(gy) && aligned16(x) && aligned16(h) && aligned16(lora_b) && aligned16(workspace),
             "lora_bwd: pointers must be 16-byte aligned");
  if (workspace_bytes < ttamd_lora_bwd_workspace_bytes(M, N, K, rank))
    return fail(TTAMD_EWORKSPACE, "lora_bwd: workspace has %zu bytes, needs %zu", workspace_bytes,
                ttamd_lora_bwd_workspace_bytes(M, N, K, rank));
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  uint16_t* bt = reinterpret_cast<uint16_t*>(workspace);  // lora_b^T [R, N]
  float* part = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + align256((size_t)N * rank * sizeof(uint16_t)));
  const uint16_t* GY = reinterpret_cast<const uint16_t*>(gy);
  const int64_t nb = N * rank;
  transpose_small_kernel<<<dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, s>>>(reinterpret_cast<const uint16_t*>(lora_b), N,
                                                                                  rank, bt);
  // gh = scale * gy . B
  if (int rc = run_nt(GY, bt, M, N, rank, scale, reinterpret_cast<uint16_t*>(gh), part, s)) return rc;
  // gA[r][k] = sum_m gh[m][r] x[m][k]
  if (int rc = run_tn(reinterpret_cast<const uint16_t*>(gh), reinterpret_cast<const uint16_t*>(x), M, K, rank, 1.0f, K, 1,
                      reinterpret_cast<uint16_t*>(ga), part, s))
    return rc;
  // gB[n][r] = scale * sum_m h[m][r] gy[m][n]
  return run_tn(reinterpret_cast<const uint16_t*>(h), GY, M, N, rank, scale, 1, rank, reinterpret_cast<uint16_t*>(gb), part, s);
}
