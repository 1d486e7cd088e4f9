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
// contiguous bytes).  The last two contract over rows: bf16 MFMA as well, with both operands transposed on the way
// through LDS (ds_read_b64_tr_b16).  Both split the contraction over many workgroups to
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
// BT: Bm is given as it lies in memory for the other contraction, [Kc, R] row-major (lora_b [N, R] for gh = gy . B).
// The operand then needs 8 consecutive rows of one column in a lane; each wave copies the 64 x R piece of its chunk
// (contiguous in memory) into a private LDS region and reads it back transposed with ds_read_b64_tr_b16 (lane j of a
// 16-lane group points at row j / 4, columns 4 (j % 4) .. + 3 of a 4 x 16 piece; lane i receives column i of its 4 rows).
// ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ u32x2_t lds_read_tr16(uint32_t addr, int imm) {
  u32x2_t v;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(imm) : "memory");
  return v;
}

template <int RT, bool BT>
__global__ __launch_bounds__(256) void skinny_nt_kernel(const uint16_t* __restrict__ X, const uint16_t* __restrict__ Bm,
                                                        float* __restrict__ part, int M, int Kc, int R,
                                                        int chunks_per_split, uint16_t* __restrict__ direct_out,
                                                        float scale) {
  // direct_out != null (only with a single split): write bf16(scale * sum) straight to the [M, R] output
  __shared__ float red[3][2 * RT * 4][64];
  constexpr int kPitchB = 32 * RT;  // bytes per LDS row of the transposed-operand piece: 16 RT columns
  __shared__ __attribute__((aligned(16))) char bstage[BT ? 4 * 64 * kPitchB : 16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, i = lane & 15;
  const int m0 = blockIdx.x * 32;
  const int split = blockIdx.y;
  char* myb = bstage + (BT ? wave * 64 * kPitchB : 0);
  const uint32_t brd = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)myb) + (16 * g + (i >> 2)) * kPitchB + 8 * (i & 3);
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
  auto chunk_start = [&](int j) {
    int c = j + rot;
    c = c0 + (c >= nc ? c - nc : c);
    return c * 64;
  };
  auto multiply = [&](const u32x4_t (&xa)[2][2], const u32x4_t (&wb)[RT][2]) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int u = 0; u < RT; ++u)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh)
          acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, xa[t][hh]),
                                                             __builtin_bit_cast(bf16x8_t, wb[u][hh]), acc[t][u], 0, 0, 0);
  };
  if constexpr (BT) {
#if defined(__HIP_DEVICE_COMPILE__)
    // rows k0 .. k0 + 63 of Bm are 64 R contiguous elements: 8 R pieces of 16 bytes, R / 8 pieces to a row.  The piece
    // of a chunk is requested one chunk ahead, so that waiting for it never waits for the younger loads of X.
    const int ppr = R >> 3;
    u32x4_t piece[2 * RT];
    auto load_piece = [&](int k0) {
#pragma unroll
      for (int q = 0; q < 2 * RT; ++q) {
        const int pc = lane + 64 * q;
        if (pc < 8 * R) piece[q] = *reinterpret_cast<const u32x4_t*>(Bm + (int64_t)k0 * R + 8 * pc);
      }
    };
    u32x4_t xa[2][2], xn[2][2];
    auto load_x = [&](u32x4_t (&dst)[2][2], int k0) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) dst[t][hh] = *reinterpret_cast<const u32x4_t*>(xrow[t] + k0 + 8 * hh);
    };
    if (wave < nc) {
      load_piece(chunk_start(wave));
      load_x(xa, chunk_start(wave));
    }
    for (int j = wave; j < nc; j += 4) {
#pragma unroll
      for (int q = 0; q < 2 * RT; ++q) {
        const int pc = lane + 64 * q;
        if (pc < 8 * R) *reinterpret_cast<u32x4_t*>(myb + (pc / ppr) * kPitchB + 16 * (pc % ppr)) = piece[q];
      }
      if (j + 4 < nc) {  // the next chunk's loads are in flight while this one is multiplied
        load_piece(chunk_start(j + 4));
        load_x(xn, chunk_start(j + 4));
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the piece has landed (LDS operations of a wave complete in order)
      u32x4_t wb[RT][2];
      u32x2_t lo[RT][2], hi[RT][2];
#pragma unroll
      for (int u = 0; u < RT; ++u)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          lo[u][hh] = lds_read_tr16(brd, 32 * u + (8 * hh) * kPitchB);
          hi[u][hh] = lds_read_tr16(brd, 32 * u + (8 * hh + 4) * kPitchB);
        }
#pragma unroll
      for (int u = 0; u < RT; ++u)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          // waits that name the registers they release: no use can be scheduled ahead of them
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[u][hh]), "+v"(hi[u][hh]));
          wb[u][hh] = u32x4_t{lo[u][hh].x, lo[u][hh].y, hi[u][hh].x, hi[u][hh].y};
        }
      multiply(xa, wb);
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) xa[t][hh] = xn[t][hh];
    }
#endif
  } else {
#pragma unroll 2
    for (int j = wave; j < nc; j += 4) {
      const int k0 = chunk_start(j);
      u32x4_t xa[2][2], wb[RT][2];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) xa[t][hh] = *reinterpret_cast<const u32x4_t*>(xrow[t] + k0 + 8 * hh);
#pragma unroll
      for (int u = 0; u < RT; ++u)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          wb[u][hh] = u32x4_t{0, 0, 0, 0};
          if (bvalid[u]) wb[u][hh] = *reinterpret_cast<const u32x4_t*>(brow[u] + k0 + 8 * hh);
        }
      multiply(xa, wb);
    }
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

// ---------------------------------------------------------------------------------------------------
// skinny_tn: part[split][r0 + r][c] = sum_{m in split} G[m][r0 + r] * X[m][c]   (G [M,R], X [M,Kc], r < 16)
// The contraction runs over rows.  The fp32 MFMA v_mfma_f32_16x16x4_f32 takes one contraction index per lane and
// could read both operands as they lie in memory, but it consumes only 64 elements of X per 32-cycle instruction,
// which caps a kernel built on it near the HBM rate (measured: 3.7 - 4.8 TB/s).  v_mfma_f32_16x16x32_bf16
// takes 512, but wants 8 consecutive contraction indices (rows m) of one column in a lane, while memory has 8
// consecutive columns of one row.  The transposition is done by the LDS: a wave copies its 32 rows x 128 columns of X
// (and the matching 32 x 16 piece of G) row-major into a private LDS region and reads them back with
// ds_read_b64_tr_b16.  In a 16-lane group that instruction returns to lane i, as element t, the 16-bit element
// (i % 4) of the 8 bytes that lane 4 t + i / 4 points at; with lane j pointing at row j / 4, columns 4 (j % 4) .. + 3
// of a 4 x 16 piece, lane i receives column i of rows 0 .. 3: exactly an MFMA operand.
// Workgroup = 4 waves on the same 128 columns; wave w takes the 32-row steps w, w + 4, ... of the split.  The partial
// sums are combined through LDS in a fixed order, then across splits by sum_partials_tn_pair_kernel.
// ---------------------------------------------------------------------------------------------------
constexpr int kTnCols = 128;    // columns per workgroup
constexpr int kTrPitchX = 288;  // bytes per LDS row of the X piece: 256 + 32, so that 4 consecutive rows fall on disjoint banks
constexpr int kTrWaveLds = 32 * kTrPitchX + 32 * 32;  // X piece + G piece (32 rows x 16 bf16)

// One launch serves the two row contractions of a LoRA backward (gA over x, gB over gy): they share M, R and the row
// splits, and differ in the operands and the width.  Workgroups [0, col_groups0) belong to problem 0, the rest to 1.
struct TnProblem {
  const uint16_t* G;  // [M, R]
  const uint16_t* X;  // [M, Kc]
  float* part;        // [splits, R, Kc]
  int Kc;
};
struct TnPair {
  TnProblem p[2];
  int col_groups0;
  int M, R, r0, rows_per_split;
};

__global__ __launch_bounds__(256) void skinny_tn_kernel(const TnPair a) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int which = (int)blockIdx.x >= a.col_groups0 ? 1 : 0;  // uniform over the workgroup
  const uint16_t* __restrict__ G = a.p[which].G;
  const uint16_t* __restrict__ X = a.p[which].X;
  float* __restrict__ part = a.p[which].part;
  const int Kc = a.p[which].Kc, M = a.M, R = a.R, r0 = a.r0, rows_per_split = a.rows_per_split;
  const int col_group = (int)blockIdx.x - (which ? a.col_groups0 : 0);
  __shared__ __attribute__((aligned(16))) char stage[4 * kTrWaveLds];
  static_assert(sizeof(stage) >= 3 * 32 * 64 * sizeof(float), "the reduction reuses the staging memory");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, i = lane & 15;
  const int c0 = col_group * kTnCols;
  const int split = blockIdx.y;
  const int m_begin = split * rows_per_split;
  int m_end = m_begin + rows_per_split;
  m_end = m_end < M ? m_end : M;

  char* my = stage + wave * kTrWaveLds;
  // copy-in roles: X piece, instruction u (0..7): row 4 u + lane / 16, 16-byte chunk lane % 16 (a row is 16 chunks)
  const int xcol = c0 + 8 * i;
  const bool xcol_ok = xcol < Kc;  // Kc % 8 == 0
  const uint16_t* xsrc = X + (xcol_ok ? xcol : 0);
  char* xdst = my + g * kTrPitchX + 16 * i;
  // G piece: row lane / 2, half lane % 2 (8 of the 16 adapter columns r0 .. r0 + 15)
  const int gcol = r0 + 8 * (lane & 1);
  const bool gcol_ok = gcol < R;  // R % 8 == 0
  const uint16_t* gsrc = G + (gcol_ok ? gcol : 0);
  char* gdst = my + 32 * kTrPitchX + (lane >> 1) * 32 + 16 * (lane & 1);
  // read-back roles: lane j = lane % 16 of group g points at row 8 g + j / 4 (+ 4 for the second half of the operand),
  // columns 4 (j % 4) .. + 3 of a 16-column group
  const uint32_t my_lds = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)my);
  const uint32_t xrd = my_lds + (8 * g + (i >> 2)) * kTrPitchX + 8 * (i & 3);
  const uint32_t grd = my_lds + 32 * kTrPitchX + (8 * g + (i >> 2)) * 32 + 8 * (i & 3);

  f32x4_t acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  u32x4_t xv[8], gv;
  auto fetch = [&](int m) {  // rows m .. m + 31 into registers
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int row = m + 4 * u + g;
      xv[u] = u32x4_t{0, 0, 0, 0};
      if (row < m_end && xcol_ok) xv[u] = *reinterpret_cast<const u32x4_t*>(xsrc + (int64_t)row * Kc);
    }
    const int grow = m + (lane >> 1);
    gv = u32x4_t{0, 0, 0, 0};
    if (grow < m_end && gcol_ok) gv = *reinterpret_cast<const u32x4_t*>(gsrc + (int64_t)grow * R);
  };
  int m = m_begin + 32 * wave;
  if (m < m_end) fetch(m);
  for (; m < m_end; m += 128) {
    // the previous step's reads of this region are complete: they were waited for before its MFMAs
#pragma unroll
    for (int u = 0; u < 8; ++u) *reinterpret_cast<u32x4_t*>(xdst + 4 * u * kTrPitchX) = xv[u];
    *reinterpret_cast<u32x4_t*>(gdst) = gv;
    if (m + 128 < m_end) fetch(m + 128);  // in flight while this step is multiplied
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the copy-in has landed (LDS operations of a wave complete in order)
    u32x2_t ga = lds_read_tr16(grd, 0), gb = lds_read_tr16(grd, 4 * 32);
    u32x2_t xa[8], xb[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      xa[e] = lds_read_tr16(xrd, 32 * e);
      xb[e] = lds_read_tr16(xrd, 32 * e + 4 * kTrPitchX);
    }
    // The 18 reads return in order.  Each wait names the registers it releases, so that no use can be scheduled
    // ahead of it: column group e may go once at most 14 - 2 e younger reads are outstanding.
    asm volatile("s_waitcnt lgkmcnt(14)" : "+v"(ga), "+v"(gb), "+v"(xa[0]), "+v"(xb[0]));
    const u32x4_t gop = {ga.x, ga.y, gb.x, gb.y};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (e > 0) asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(xa[e]), "+v"(xb[e]) : "n"(14 - 2 * e));
      const u32x4_t xop = {xa[e].x, xa[e].y, xb[e].x, xb[e].y};
      acc[e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, gop), __builtin_bit_cast(bf16x8_t, xop),
                                                      acc[e], 0, 0, 0);
    }
  }
  __syncthreads();  // the staging regions are free: the partial sums meet in them
  float (*red)[32][64] = reinterpret_cast<float (*)[32][64]>(stage);
  // acc[e][v] = sum over this wave's rows of G[.][r0 + 4 g + v] * X[.][c0 + 16 e + i]
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[wave - 1][v * 8 + e][lane] = acc[e][v];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int r = r0 + 4 * g + v;
      if (r >= R) continue;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int col = c0 + 16 * e + i;
        if (col >= Kc) continue;
        part[((int64_t)split * R + r) * Kc + col] =
            ((acc[e][v] + red[0][v * 8 + e][lane]) + red[1][v * 8 + e][lane]) + red[2][v * 8 + e][lane];
      }
    }
  }
#endif
}

// out[r*stride_r + k*stride_k] = bf16(scale * sum_s part[s][r][k])
struct TnSum {
  const float* part;
  uint16_t* out;
  int Kc;
  float scale;
  int64_t stride_r, stride_k;
};
struct TnSumPair {
  TnSum p[2];
  int64_t n0;  // elements of problem 0: R * Kc
  int R, splits;
};
// The reductions of the two row contractions in one launch: thread i < n0 finishes problem 0, the rest problem 1.
__global__ __launch_bounds__(256) void sum_partials_tn_pair_kernel(const TnSumPair a) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int which = i >= a.n0 ? 1 : 0;
  if (which) i -= a.n0;
  const TnSum& P = a.p[which];
  const int64_t n = (int64_t)a.R * P.Kc;
  if (i >= n) return;
  float s = 0.f;
#pragma unroll 8
  for (int q = 0; q < a.splits; ++q) s += P.part[(int64_t)q * n + i];
  const int64_t r = i / P.Kc, k = i % P.Kc;
  P.out[r * P.stride_r + k * P.stride_k] = f32_to_bf16_bits(s * P.scale);
}

constexpr int kTargetWaves = 2048;    // row contractions (skinny_tn)
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
  int col_groups0, col_groups1, splits, rows_per_split;
};
// Both products of a backward in one grid: widths K (gA) and N (gB), the same row splits.
TnPlan plan_tn_pair(int64_t M, int64_t K, int64_t N) {
  TnPlan p;
  p.col_groups0 = (int)((K + kTnCols - 1) / kTnCols);
  p.col_groups1 = (int)((N + kTnCols - 1) / kTnCols);
  int s = kTargetWaves / 4 / (p.col_groups0 + p.col_groups1);  // workgroups of 4 waves
  s = s < 1 ? 1 : s;
  const int max_s = (int)((M + 127) / 128);  // at least 128 rows per split: one 32-row step per wave
  s = s > max_s ? max_s : s;
  p.rows_per_split = (int)(((M + s - 1) / s + 127) / 128 * 128);  // whole rounds of the four waves
  p.splits = (int)((M + p.rows_per_split - 1) / p.rows_per_split);
  return p;
}
size_t tn_pair_ws_bytes(int64_t M, int64_t K, int64_t N, int R) {
  return (size_t)plan_tn_pair(M, K, N).splits * R * (size_t)(K + N) * sizeof(float);
}

size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

// b_is_kr: Bm is [Kc, R] row-major (transposed inside the kernel) instead of [R, Kc]
template <bool BT>
void launch_nt(const dim3& grid, const uint16_t* X, const uint16_t* Bm, float* ws, int M, int Kc, int R, int chunks_per_split,
               uint16_t* direct, float scale, hipStream_t s) {
  const dim3 block(256);
  if (R <= 16)
    skinny_nt_kernel<1, BT><<<grid, block, 0, s>>>(X, Bm, ws, M, Kc, R, chunks_per_split, direct, scale);
  else if (R <= 32)
    skinny_nt_kernel<2, BT><<<grid, block, 0, s>>>(X, Bm, ws, M, Kc, R, chunks_per_split, direct, scale);
  else
    skinny_nt_kernel<4, BT><<<grid, block, 0, s>>>(X, Bm, ws, M, Kc, R, chunks_per_split, direct, scale);
}

int run_nt(const uint16_t* X, const uint16_t* Bm, bool b_is_kr, int64_t M, int64_t Kc, int R, float scale, uint16_t* out,
           float* ws, hipStream_t s) {
  const NtPlan p = plan_nt(M, Kc);
  const dim3 grid((unsigned)p.m_tiles, (unsigned)p.splits), block(256);
  uint16_t* direct = p.splits == 1 ? out : nullptr;
  if (b_is_kr)
    launch_nt<true>(grid, X, Bm, ws, (int)M, (int)Kc, R, p.chunks_per_split, direct, scale, s);
  else
    launch_nt<false>(grid, X, Bm, ws, (int)M, (int)Kc, R, p.chunks_per_split, direct, scale, s);
  if (!direct) {
    const int64_t n = M * R;
    sum_partials_kernel<<<dim3((unsigned)((n + 255) / 256)), block, 0, s>>>(ws, n, p.splits, scale, out);
  }
  return check_launch("skinny_nt");
}

// gA[r][k] = sum_m gh[m][r] x[m][k]  and  gB[n][r] = scale * sum_m h[m][r] gy[m][n]
int run_tn_pair(const uint16_t* gh, const uint16_t* x, const uint16_t* h, const uint16_t* gy, int64_t M, int64_t K, int64_t N,
                int R, float scale, uint16_t* ga, uint16_t* gb, float* ws, hipStream_t s) {
  const TnPlan p = plan_tn_pair(M, K, N);
  TnPair a;
  a.p[0] = TnProblem{gh, x, ws, (int)K};
  a.p[1] = TnProblem{h, gy, ws + (size_t)p.splits * R * K, (int)N};
  a.col_groups0 = p.col_groups0;
  a.M = (int)M;
  a.R = R;
  a.rows_per_split = p.rows_per_split;
  const dim3 grid((unsigned)(p.col_groups0 + p.col_groups1), (unsigned)p.splits), block(256);
  for (int r0 = 0; r0 < R; r0 += 16) {
    a.r0 = r0;
    skinny_tn_kernel<<<grid, block, 0, s>>>(a);
  }
  TnSumPair f;
  f.p[0] = TnSum{a.p[0].part, ga, (int)K, 1.0f, K, 1};
  f.p[1] = TnSum{a.p[1].part, gb, (int)N, scale, 1, R};
  f.n0 = (int64_t)R * K;
  f.R = R;
  f.splits = p.splits;
  const int64_t n = (int64_t)R * (K + N);
  sum_partials_tn_pair_kernel<<<dim3((unsigned)((n + 255) / 256)), block, 0, s>>>(f);
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
  return run_nt(reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint16_t*>(lora_a), false, M, K, rank, 1.0f,
                reinterpret_cast<uint16_t*>(h), reinterpret_cast<float*>(workspace), reinterpret_cast<hipStream_t>(stream));
}

// ---- the same product for callers that cannot allocate ---------------------------------------------------------------
// Partial sums of a launch that is cut along K live in this file-scope device array instead of a caller's workspace.
// Every GPU the library runs on holds its own copy until the process ends.  The plan never needs more: with fewer than
// 256 row tiles it uses at most 256 / row_tiles slices of 32 * row_tiles rows, i.e. at most 8192 partial rows of at most
// 64 fp32 values, and with 256 row tiles or more it writes the result directly.
constexpr size_t kStaticScratchBytes = size_t(2) << 20;
static __device__ __align__(256) unsigned char g_hidden_scratch[kStaticScratchBytes];

namespace {
// Device address of g_hidden_scratch on the current device.  In host code the array's name is only a handle for the
// runtime, not a device address: the address is asked for once per device (with that device current) and kept.
int static_scratch(float** out) {
  static void* ptr[64] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(TTAMD_ELAUNCH, "lora_hidden_static: hipGetDevice: %s", hipGetErrorString(e));
  void* p = (dev >= 0 && dev < 64) ? ptr[dev] : nullptr;
  if (p == nullptr) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_hidden_scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(TTAMD_ELAUNCH, "lora_hidden_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    if (dev >= 0 && dev < 64) ptr[dev] = p;  // a race between threads stores the same value twice
  }
  *out = reinterpret_cast<float*>(p);
  return TTAMD_OK;
}
}  // namespace

extern "C" size_t ttamd_lora_hidden_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int ttamd_lora_hidden_static_bf16(const void* x, const void* lora_a, void* h, int64_t M, int64_t K, int rank,
                                             void* stream) {
  if (int rc = check_skinny("lora_hidden_static", M, 64, K, rank)) return rc;
  TT_REQUIRE(x && lora_a && h, "lora_hidden_static: null pointer argument");
  TT_REQUIRE(aligned16(x) && aligned16(lora_a), "lora_hidden_static: pointers must be 16-byte aligned");
  const size_t need = plan_nt(M, K).splits > 1 ? nt_ws_bytes(M, K, rank) : 0;  // one slice writes the result directly
  if (need > kStaticScratchBytes)
    return fail(TTAMD_EWORKSPACE, "lora_hidden_static: M=%lld K=%lld rank=%d needs %zu bytes of partial sums, the built-in "
                "scratch holds %zu; use ttamd_lora_hidden_bf16 with a workspace", (long long)M, (long long)K, rank, need,
                kStaticScratchBytes);
  float* scratch = nullptr;
  if (int rc = static_scratch(&scratch)) return rc;
  // every partial sum the reduction reads is written by this call's first kernel: nothing has to start at zero
  return run_nt(reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint16_t*>(lora_a), false, M, K, rank, 1.0f,
                reinterpret_cast<uint16_t*>(h), scratch, reinterpret_cast<hipStream_t>(stream));
}

extern "C" size_t ttamd_lora_bwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int rank) {
  if (M <= 0 || N <= 0 || K <= 0 || rank <= 0 || K % 64 || N % 64) return 0;
  const size_t a = nt_ws_bytes(M, N, rank), b = tn_pair_ws_bytes(M, K, N, rank);
  return align256(a > b ? a : b);
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
  float* part = reinterpret_cast<float*>(workspace);
  const uint16_t* GY = reinterpret_cast<const uint16_t*>(gy);
  // gh = scale * gy . B, lora_b [N, R] as it lies (the kernel transposes its pieces)
  if (int rc = run_nt(GY, reinterpret_cast<const uint16_t*>(lora_b), true, M, N, rank, scale, reinterpret_cast<uint16_t*>(gh),
                      part, s))
    return rc;
  return run_tn_pair(reinterpret_cast<const uint16_t*>(gh), reinterpret_cast<const uint16_t*>(x),
                     reinterpret_cast<const uint16_t*>(h), GY, M, K, N, rank, scale, reinterpret_cast<uint16_t*>(ga),
                     reinterpret_cast<uint16_t*>(gb), part, s);
}
