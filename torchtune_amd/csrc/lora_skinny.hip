// The rank-r ("skinny") products of the LoRA adapter on gfx950.  All four are HBM-bound: each streams one
// [M, K] or [M, N] activation once and produces an output with only `rank` rows or columns.
//
//   h  = x  . A^T        [M,R]   contraction over K  (forward)
//   gh = s . gy . B      [M,R]   contraction over N  (backward)
//   gA = gh^T . x        [R,K]   contraction over M  (backward)
//   gB = s . gy^T . h    [N,R]   contraction over M  (backward)
//
// The first two contract along the contiguous dimension of the activation: bf16 MFMA with the activation rows
// as the A operand, fragments loaded straight from global memory (a lane's 8 contraction elements are 16
// contiguous bytes).  The last two contract over rows: fp32 MFMA (one contraction index per lane, so both
// operands are read row-major as they lie in memory).  Both split the contraction over many workgroups to
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
// Workgroup = 4 waves on the same 32 rows of X; the split's 64-wide contraction chunks are dealt to the waves in
// turn and the four partial sums are combined through LDS in a fixed order.  MFMA v_mfma_f32_16x16x32_bf16 with the
// rows of X as the row operand: lane (g = l / 16, i = l % 16) loads the 32 contiguous bytes X[m + i][k0 + 16 g ..
// + 16) - the four lane groups cover one whole 128-byte line per row - and uses its first 8 elements for one MFMA and
// the last 8 for the next (the contraction index may be permuted freely as long as both operands agree).
// RT = number of 16-wide tiles of R.
// ---------------------------------------------------------------------------------------------------
template <int RT>
__global__ __launch_bounds__(256) void skinny_nt_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ Bm,
                                                        float* __restrict__ part, int M, int Kc, int R,
                                                        int chunks_per_split, uint16_t* __restrict__ direct_out,
                                                        float scale) {
  // direct_out != null (only with a single split): write bf16(scale * sum) straight to the [M, R] output
  __shared__ float red[3][2 * RT * 4][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, i = lane & 15;
  const int m0 = blockIdx.x * 32;
  const int split = blockIdx.y;
  const uint16_t* xrow[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    int row = m0 + 16 * t + i;
    row = row < M ? row : M - 1;
    xrow[t] = X + (int64_t)row * Kc + 16 * g;
  }
  const uint16_t* brow[RT];
  bool bvalid[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int r = t * 16 + i;
    bvalid[t] = r < R;
    brow[t] = Bm + (int64_t)(bvalid[t] ? r : 0) * Kc + 16 * g;
  }
  f32x4_t acc[2][RT];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int u = 0; u < RT; ++u) acc[t][u] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int total_chunks = Kc >> 6;
  const int c0 = split * chunks_per_split;
  int c1 = c0 + chunks_per_split;
  c1 = c1 < total_chunks ? c1 : total_chunks;
  // Workgroups that run side by side differ in their row tile only; were they all to start at the same column, every
  // one of them would be on the same few memory channels (rows are a power-of-two number of bytes apart).  Each row
  // tile therefore walks its chunks in a rotated order.  The order is a fixed function of the tile: deterministic.
  const int nc = c1 - c0;
  const int rot = nc > 0 ? (int)((blockIdx.x * 4u) % (unsigned)nc) : 0;
#pragma unroll 2
  for (int j = wave; j < nc; j += 4) {
    int c = j + rot;
    c = c0 + (c >= nc ? c - nc : c);
    const int k0 = c * 64;
    u32x4_t xa[2][2], wb[RT][2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
        xa[t][hh] = *reinterpret_cast<const u32x4_t*>(xrow[t] + k0 + 8 * hh);
#pragma unroll
    for (int u = 0; u < RT; ++u)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        wb[u][hh] = u32x4_t{0, 0, 0, 0};
        if (bvalid[u]) wb[u][hh] = *reinterpret_cast<const u32x4_t*>(brow[u] + k0 + 8 * hh);
      }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int u = 0; u < RT; ++u)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh)
          acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, xa[t][hh]),
                                                             __builtin_bit_cast(bf16x8_t, wb[u][hh]), acc[t][u], 0, 0, 0);
  }
  // acc[t][u][v] = C[m0 + 16 t + 4 g + v][16 u + i]
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int u = 0; u < RT; ++u)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave - 1][(t * RT + u) * 4 + v][lane] = acc[t][u][v];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int u = 0; u < RT; ++u) {
        const int col = 16 * u + i;
        if (col >= R) continue;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int r = m0 + 16 * t + 4 * g + v;
          const int e = (t * RT + u) * 4 + v;
          if (r >= M) continue;
          const float sum = ((acc[t][u][v] + red[0][e][lane]) + red[1][e][lane]) + red[2][e][lane];
          if (direct_out)
            direct_out[(int64_t)r * R + col] = f32_to_bf16_bits(sum * scale);
          else
            part[((int64_t)split * M + r) * R + col] = sum;
        }
      }
  }
}

// out[i] = bf16(scale * sum_s part[s][i]) for i < n (out and part share the [M,R] layout)
__global__ __launch_bounds__(256) void sum_partials_kernel(const float* __restrict__ part, int64_t n, int splits, float scale,
                                                           uint16_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
#pragma unroll 8
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
// skinny_tn: part[split][r0 + r][c] = sum_{m in split} G[m][r0 + r] * X[m][c]   (G [M,R], X [M,Kc], r < 16)
// The contraction runs over rows, so both operands are read in their natural row-major layout by the fp32 MFMA
// v_mfma_f32_16x16x4_f32, whose operands hold ONE contraction index per lane: lane (g = l / 16, q = l % 16) supplies
// G[m + g][r0 + q] as the row operand and X[m + g][c] as the column operand, four rows m..m+3 per instruction.
// A lane loads 8 consecutive columns (16 bytes) of its row and feeds them to 8 MFMAs, so MFMA e of the wave covers the
// columns {c0 + 8 q + e}; its 16x16 result D[r][.] is lane q's column c0 + 8 q + e, i.e. a lane ends up with 8
// consecutive columns for each of its 4 result rows r = 4 g + v.
// Workgroup = 4 waves on the same 128 columns, taking the split's 4-row steps in turn; partial sums are combined
// through LDS in a fixed order, then across splits by sum_partials_tn_kernel.
// ---------------------------------------------------------------------------------------------------
constexpr int kTnCols = 128;   // columns per workgroup
constexpr int kTnUnroll = 4;   // 4-row steps in flight per wave

__global__ __launch_bounds__(256) void skinny_tn_kernel(const uint16_t* __restrict__ G, const uint16_t* __restrict__ X,
                                                        float* __restrict__ part, int M, int Kc, int R, int r0,
                                                        int rows_per_split) {
  __shared__ float red[3][32][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, q = lane & 15;
  const int col = blockIdx.x * kTnCols + q * 8;
  const bool col_ok = col < Kc;  // Kc % 8 == 0: a lane's 8 columns are in or out together
  const bool r_ok = r0 + q < R;
  const int split = blockIdx.y;
  const int m_begin = split * rows_per_split;
  int m_end = m_begin + rows_per_split;
  m_end = m_end < M ? m_end : M;

  f32x4_t acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const uint16_t* xp = X + (col_ok ? col : 0);
  const uint16_t* gp = G + (r_ok ? r0 + q : 0);
  for (int m = m_begin + 4 * wave; m < m_end; m += 16 * kTnUnroll) {
    u32x4_t xv[kTnUnroll];
    uint32_t gv[kTnUnroll];
#pragma unroll
    for (int u = 0; u < kTnUnroll; ++u) {
      const int row = m + 16 * u + g;
      const bool ok = row < m_end;
      xv[u] = u32x4_t{0, 0, 0, 0};
      gv[u] = 0;
      if (ok && col_ok) xv[u] = *reinterpret_cast<const u32x4_t*>(xp + (int64_t)row * Kc);
      if (ok && r_ok) gv[u] = gp[(int64_t)row * R];
    }
#pragma unroll
    for (int u = 0; u < kTnUnroll; ++u) {
      const float a = bits_f32(gv[u] << 16);
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        acc[2 * d] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bits_f32(xv[u][d] << 16), acc[2 * d], 0, 0, 0);
        acc[2 * d + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bits_f32(xv[u][d] & 0xffff0000u), acc[2 * d + 1], 0, 0, 0);
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[wave - 1][v * 8 + e][lane] = acc[e][v];
  }
  __syncthreads();
  if (wave == 0 && col_ok) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int r = r0 + 4 * g + v;
      if (r >= R) continue;
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        o[e] = ((acc[e][v] + red[0][v * 8 + e][lane]) + red[1][v * 8 + e][lane]) + red[2][v * 8 + e][lane];
      float* dst = part + ((int64_t)split * R + r) * Kc + col;
      *reinterpret_cast<f32x4_t*>(dst) = f32x4_t{o[0], o[1], o[2], o[3]};
      *reinterpret_cast<f32x4_t*>(dst + 4) = f32x4_t{o[4], o[5], o[6], o[7]};
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
#pragma unroll 8
  for (int p = 0; p < splits; ++p) s += part[(int64_t)p * n + i];
  const int64_t r = i / Kc, k = i % Kc;
  out[r * stride_r + k * stride_k] = f32_to_bf16_bits(s * scale);
}

constexpr int kTargetWaves = 4096;    // row contractions (skinny_tn)
constexpr int kTargetWavesNt = 1024;  // column contractions (skinny_nt): few, long waves; one split needs no second pass

struct NtPlan {
  int m_tiles, splits, chunks_per_split;
};
NtPlan plan_nt(int64_t M, int64_t Kc) {
  NtPlan p;
  p.m_tiles = (int)((M + 31) / 32);
  const int total_chunks = (int)(Kc / 64);
  int s = kTargetWavesNt / 4 / p.m_tiles;  // workgroups of 4 waves
  s = s < 1 ? 1 : s;
  const int max_s = (total_chunks + 7) / 8;  // at least two chunks per wave
  s = s > max_s ? max_s : s;
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
  p.col_groups = (int)((Kc + kTnCols - 1) / kTnCols);
  int s = kTargetWaves / 4 / p.col_groups;  // workgroups of 4 waves
  s = s < 1 ? 1 : s;
  const int max_s = (int)((M + 63) / 64);  // at least 64 rows per split: four 4-row steps per wave
  s = s > max_s ? max_s : s;
  p.rows_per_split = (int)(((M + s - 1) / s + 15) / 16 * 16);  // whole rounds of the four waves
  p.splits = (int)((M + p.rows_per_split - 1) / p.rows_per_split);
  return p;
}
size_t tn_ws_bytes(int64_t M, int64_t Kc, int R) { return (size_t)plan_tn(M, Kc).splits * R * Kc * sizeof(float); }

size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

int run_nt(const uint16_t* X, const uint16_t* Bm, int64_t M, int64_t Kc, int R, float scale, uint16_t* out, float* ws,
           hipStream_t s) {
  const NtPlan p = plan_nt(M, Kc);
  const dim3 grid((unsigned)p.m_tiles, (unsigned)p.splits), block(256);
  uint16_t* direct = p.splits == 1 ? out : nullptr;
  if (R <= 16)
    skinny_nt_kernel<1><<<grid, block, 0, s>>>(X, Bm, ws, (int)M, (int)Kc, R, p.chunks_per_split, direct, scale);
  else if (R <= 32)
    skinny_nt_kernel<2><<<grid, block, 0, s>>>(X, Bm, ws, (int)M, (int)Kc, R, p.chunks_per_split, direct, scale);
  else
    skinny_nt_kernel<4><<<grid, block, 0, s>>>(X, Bm, ws, (int)M, (int)Kc, R, p.chunks_per_split, direct, scale);
  if (!direct) {
    const int64_t n = M * R;
    sum_partials_kernel<<<dim3((unsigned)((n + 255) / 256)), block, 0, s>>>(ws, n, p.splits, scale, out);
  }
  return check_launch("skinny_nt");
}

int run_tn(const uint16_t* G, const uint16_t* X, int64_t M, int64_t Kc, int R, float scale, int64_t stride_r,
           int64_t stride_k, uint16_t* out, float* ws, hipStream_t s) {
  const TnPlan p = plan_tn(M, Kc);
  const dim3 grid((unsigned)p.col_groups, (unsigned)p.splits), block(256);
  for (int r0 = 0; r0 < R; r0 += 16)
    skinny_tn_kernel<<<grid, block, 0, s>>>(G, X, ws, (int)M, (int)Kc, R, r0, p.rows_per_split);
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
