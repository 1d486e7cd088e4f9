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
// are deterministic.  For wide layers of rank <= 16 the two products that read gy (gh and gB) come from one pass over
// it (skinny_tn_gh_kernel).
#include <atomic>
#include "common.h"
#include "group.h"
#include "nf4_math.h"
#include "swiglu_math.h"

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

constexpr int kMaxGroup = kGroupMax;

// One column contraction.  The R rows of the second operand may be stacked from several matrices (the adapters of a
// group's members): rows [r_off[b], r_off[b + 1]) are the rows of bm[b].  A launch takes a batch of problems over the
// same M (blockIdx.z), each with its own operands, width, slicing and output columns.
struct NtProblem {
  const uint16_t* X;              // [M, Kc]
  const uint16_t* bm[kMaxGroup];  // BT: bm[0] is [Kc, R]; otherwise bm[b] is [r_off[b + 1] - r_off[b], Kc]
  int r_off[kMaxGroup + 1];
  int nb;                         // matrices in bm
  float* part;                    // [splits, M, R] fp32, used when splits > 1
  uint16_t* out;                  // bf16 rows `ldo` elements apart; the problem's R columns start here
  int Kc, R, ldo, splits, chunks_per_split;
  float scale;
};
struct NtBatch {
  NtProblem p[kMaxGroup];
  int M;
};

template <int RT, bool BT>
__global__ __launch_bounds__(256) void skinny_nt_kernel(const NtBatch a) {
  const NtProblem& P = a.p[blockIdx.z];
  const int split = blockIdx.y;
  if (split >= P.splits) return;  // the batch's grid is as deep as its most sliced problem
  const uint16_t* __restrict__ X = P.X;
  const uint16_t* __restrict__ Bm = P.bm[0];
  float* __restrict__ part = P.part;
  const int M = a.M, Kc = P.Kc, R = P.R, chunks_per_split = P.chunks_per_split;
  // a single slice writes bf16(scale * sum) straight to the output
  uint16_t* __restrict__ direct_out = P.splits == 1 ? P.out : nullptr;
  const int ldo = P.ldo;
  const float scale = P.scale;
  __shared__ float red[3][2 * RT * 4][64];
  constexpr int kPitchB = 32 * RT;  // bytes per LDS row of the transposed-operand piece: 16 RT columns
  __shared__ __attribute__((aligned(16))) char bstage[BT ? 4 * 64 * kPitchB : 16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, i = lane & 15;
  const int m0 = blockIdx.x * 32;
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
    brow[t] = Bm + 16 * g;
    if (!BT && bvalid[t]) {
#pragma unroll
      for (int b = 0; b < kMaxGroup; ++b)
        if (b < P.nb && r >= P.r_off[b] && r < P.r_off[b + 1]) brow[t] = P.bm[b] + (int64_t)(r - P.r_off[b]) * Kc + 16 * g;
    }
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
            direct_out[(int64_t)r * ldo + col] = f32_to_bf16_bits(sum * scale);
          else
            part[((int64_t)split * M + r) * R + col] = sum;
        }
      }
  }
}

// The second pass of the sliced problems of a batch (blockIdx.y = problem): out[m][c] = bf16(scale * sum_s part[s][m][c])
__global__ __launch_bounds__(256) void sum_partials_kernel(const NtBatch a) {
  const NtProblem& P = a.p[blockIdx.y];
  if (P.splits == 1) return;  // written directly by the first pass
  const int64_t n = (int64_t)a.M * P.R;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
#pragma unroll 8
  for (int p = 0; p < P.splits; ++p) s += P.part[(int64_t)p * n + i];
  P.out[(i / P.R) * P.ldo + i % P.R] = f32_to_bf16_bits(s * P.scale);
}

// ---------------------------------------------------------------------------------------------------
// skinny_tn: part[split][r][c] = sum_{m in split} G[m][r] * X[m][c]   (G [M,R], X [M,Kc], R <= 64)
// The contraction runs over rows.  The fp32 MFMA v_mfma_f32_16x16x4_f32 takes one contraction index per lane and
// could read both operands as they lie in memory, but it consumes only 64 elements of X per 32-cycle instruction,
// which caps a kernel built on it near the HBM rate (measured: 3.7 - 4.8 TB/s).  v_mfma_f32_16x16x32_bf16
// takes 512, but wants 8 consecutive contraction indices (rows m) of one column in a lane, while memory has 8
// consecutive columns of one row.  The transposition is done by the LDS: a wave copies its 32 rows x 128 columns of X
// (and the matching 32 x R piece of G, in groups of 16 columns) row-major into a private LDS region and reads them
// back with ds_read_b64_tr_b16.  In a 16-lane group that instruction returns to lane i, as element t, the 16-bit
// element (i % 4) of the 8 bytes that lane 4 t + i / 4 points at; with lane j pointing at row j / 4, columns
// 4 (j % 4) .. + 3 of a 4 x 16 piece, lane i receives column i of rows 0 .. 3: exactly an MFMA operand.
// All R columns of G (up to four groups of 16) are multiplied in the one pass over X.
// Workgroup = 4 waves on the same 128 columns; wave w takes the 32-row steps w, w + 4, ... of the split.  The partial
// sums are combined through LDS in a fixed order, then across splits by sum_partials_tn_kernel.
// ---------------------------------------------------------------------------------------------------
constexpr int kTnCols = 128;    // columns per workgroup
constexpr int kTnMaxRG = 4;     // groups of 16 columns of G
constexpr int kTrPitchX = 288;  // bytes per LDS row of the X piece: 256 + 32, so that 4 consecutive rows fall on disjoint banks
constexpr int tn_wave_lds(int rgm) { return 32 * kTrPitchX + rgm * 32 * 32; }  // X piece + G pieces (32 rows x 16 bf16 each)

// One launch serves every row contraction of a backward that shares M and the row splits: gA over x (for a group of
// layers with a common input: the members' gh side by side as one G) and one gB over gy per layer.  They differ in
// the operands and the width; a workgroup finds its problem from its x index.
struct TnProblem {
  const uint16_t* G;  // rows `ldg` elements apart; the problem's R columns start here
  const uint16_t* X;  // [M, Kc]
  float* part;        // [splits, R, Kc]
  int Kc, R, ldg;
};
constexpr int kTnMaxProblems = 1 + kMaxGroup;
struct TnBatch {
  TnProblem p[kTnMaxProblems];
  int cg_end[kTnMaxProblems];  // workgroups [cg_end[i - 1], cg_end[i]) along x work on problem i
  int n, M, rows_per_split;
};

// RGM: most column groups of G any problem of the batch has (registers and LDS are sized for it)
template <int RGM>
__global__ __launch_bounds__(256) void skinny_tn_kernel(const TnBatch a) {
  constexpr int kTrWaveLds = tn_wave_lds(RGM);
#if defined(__HIP_DEVICE_COMPILE__)
  int which = 0;  // uniform over the workgroup
#pragma unroll
  for (int q = 0; q < kTnMaxProblems - 1; ++q)
    if (q < a.n - 1 && (int)blockIdx.x >= a.cg_end[q]) which = q + 1;
  const TnProblem& P = a.p[which];
  const uint16_t* __restrict__ G = P.G;
  const uint16_t* __restrict__ X = P.X;
  float* __restrict__ part = P.part;
  const int Kc = P.Kc, M = a.M, R = P.R, ldg = P.ldg, rows_per_split = a.rows_per_split;
  const int rg = (R + 15) >> 4;  // groups of 16 columns of G in use
  const int col_group = (int)blockIdx.x - (which ? a.cg_end[which - 1] : 0);
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
  // G piece of column group q: row lane / 2, half lane % 2 (8 of the group's 16 columns)
  const int gcol = 8 * (lane & 1);  // + 16 q;  R % 8 == 0: a lane's 8 columns are all in or all out
  char* gdst = my + 32 * kTrPitchX + (lane >> 1) * 32 + 16 * (lane & 1);  // + 1024 q
  // read-back roles: lane j = lane % 16 of group g points at row 8 g + j / 4 (+ 4 for the second half of the operand),
  // columns 4 (j % 4) .. + 3 of a 16-column group
  const uint32_t my_lds = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)my);
  const uint32_t xrd = my_lds + (8 * g + (i >> 2)) * kTrPitchX + 8 * (i & 3);
  const uint32_t grd = my_lds + 32 * kTrPitchX + (8 * g + (i >> 2)) * 32 + 8 * (i & 3);

  f32x4_t acc[RGM][8];
#pragma unroll
  for (int q = 0; q < RGM; ++q)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[q][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  u32x4_t xv[8], gv[RGM];
  auto fetch = [&](int m) {  // rows m .. m + 31 into registers
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int row = m + 4 * u + g;
      xv[u] = u32x4_t{0, 0, 0, 0};
      if (row < m_end && xcol_ok) xv[u] = *reinterpret_cast<const u32x4_t*>(xsrc + (int64_t)row * Kc);
    }
    const int grow = m + (lane >> 1);
#pragma unroll
    for (int q = 0; q < RGM; ++q) {
      gv[q] = u32x4_t{0, 0, 0, 0};
      if (grow < m_end && gcol + 16 * q < R) gv[q] = *reinterpret_cast<const u32x4_t*>(G + (int64_t)grow * ldg + gcol + 16 * q);
    }
  };
  int m = m_begin + 32 * wave;
  if (m < m_end) fetch(m);
  for (; m < m_end; m += 128) {
    // the previous step's reads of this region are complete: they were waited for before its MFMAs
#pragma unroll
    for (int u = 0; u < 8; ++u) *reinterpret_cast<u32x4_t*>(xdst + 4 * u * kTrPitchX) = xv[u];
#pragma unroll
    for (int q = 0; q < RGM; ++q) *reinterpret_cast<u32x4_t*>(gdst + 1024 * q) = gv[q];  // zeros beyond R
    if (m + 128 < m_end) fetch(m + 128);  // in flight while this step is multiplied
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the copy-in has landed (LDS operations of a wave complete in order)
    u32x2_t ga[RGM], gb[RGM];
#pragma unroll
    for (int q = 0; q < RGM; ++q) {
      ga[q] = lds_read_tr16(grd, 1024 * q);
      gb[q] = lds_read_tr16(grd, 1024 * q + 4 * 32);
    }
    // a wait that names the registers it releases, so that no use can be scheduled ahead of it
#pragma unroll
    for (int q = 0; q < RGM; ++q) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ga[q]), "+v"(gb[q]));
    u32x2_t xa[8], xb[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      xa[e] = lds_read_tr16(xrd, 32 * e);
      xb[e] = lds_read_tr16(xrd, 32 * e + 4 * kTrPitchX);
    }
    // The 16 reads return in order: column group e may go once at most 14 - 2 e younger reads are outstanding.
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(xa[e]), "+v"(xb[e]) : "n"(14 - 2 * e));
      const u32x4_t xop = {xa[e].x, xa[e].y, xb[e].x, xb[e].y};
#pragma unroll
      for (int q = 0; q < RGM; ++q) {
        if (q < rg) {
          const u32x4_t gop = {ga[q].x, ga[q].y, gb[q].x, gb[q].y};
          acc[q][e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, gop),
                                                             __builtin_bit_cast(bf16x8_t, xop), acc[q][e], 0, 0, 0);
        }
      }
    }
  }
  float (*red)[32][64] = reinterpret_cast<float (*)[32][64]>(stage);
  // acc[q][e][v] = sum over this wave's rows of G[.][16 q + 4 g + v] * X[.][c0 + 16 e + i]; one column group of G at a
  // time meets in the staging memory
  for (int q = 0; q < rg; ++q) {
    __syncthreads();  // the staging regions (or the previous group's sums) are free
    if (wave > 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float val = acc[0][e][v];
#pragma unroll
          for (int qq = 1; qq < RGM; ++qq) val = q == qq ? acc[qq][e][v] : val;
          red[wave - 1][v * 8 + e][lane] = val;
        }
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int r = 16 * q + 4 * g + v;
        if (r >= R) continue;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int col = c0 + 16 * e + i;
          if (col >= Kc) continue;
          float mine = acc[0][e][v];
#pragma unroll
          for (int qq = 1; qq < RGM; ++qq) mine = q == qq ? acc[qq][e][v] : mine;
          part[((int64_t)split * R + r) * Kc + col] =
              ((mine + red[0][v * 8 + e][lane]) + red[1][v * 8 + e][lane]) + red[2][v * 8 + e][lane];
        }
      }
    }
  }
#endif
}

// ---------------------------------------------------------------------------------------------------
// skinny_tn_gh: both products of a backward that read gy, from one pass over it (rank <= 16):
//   part  [split][r][c] = sum_{m in split} H[m][r] * GY[m][c]                   gB, as skinny_tn
//   part_h[cg][m][r]    = sum_{c in column group cg} GY[m][c] * Bm[c][r]        gh, before scale and rounding
// A workgroup owns 256 columns (two pieces of 128) and a range of rows; wave w takes the 32-row steps w, w + 4, ... as
// in skinny_tn.  A piece that has been copied into the wave's LDS region for the transposed read-back is read back a
// second time as it lies (16 bytes = 8 consecutive columns of one row: the row operand of an MFMA whose contraction runs
// over columns) and multiplied with the matching 128 x R piece of Bm, which the wave holds in registers for the whole
// launch (transposed once through LDS like the operand of skinny_nt<., true>).  The 32 x R sums of a step over the
// workgroup's 256 columns go to part_h; a second pass (sum_partials_kernel) adds the column groups in a fixed order.
// Against a pass of its own over gy for gh this costs Kc / 256 partial rows of R fp32 per row of gy, written and read
// once: an eighth of gy's bytes at R = 16.
// ---------------------------------------------------------------------------------------------------
constexpr int kTnGhCols = 256;
struct TnGhProblem {
  const uint16_t* G;   // h: rows `ldg` elements apart; the problem's R columns start here
  const uint16_t* X;   // gy [M, Kc]
  const uint16_t* Bm;  // lora_b [Kc, R]
  float* part;         // [splits, R, Kc]
  float* part_h;       // [column groups, M, R]
  int Kc, R, ldg;
};
struct TnGhBatch {
  TnGhProblem p[kMaxGroup];
  int cg_end[kMaxGroup];  // workgroups [cg_end[i - 1], cg_end[i]) along x work on problem i
  int n, M, rows_per_split;
};

__global__ __launch_bounds__(256) void skinny_tn_gh_kernel(const TnGhBatch a) {
  constexpr int kTrWaveLds = tn_wave_lds(1);
#if defined(__HIP_DEVICE_COMPILE__)
  int which = 0;  // uniform over the workgroup
#pragma unroll
  for (int q = 0; q < kMaxGroup - 1; ++q)
    if (q < a.n - 1 && (int)blockIdx.x >= a.cg_end[q]) which = q + 1;
  const TnGhProblem& P = a.p[which];
  const uint16_t* __restrict__ G = P.G;
  const uint16_t* __restrict__ X = P.X;
  const uint16_t* __restrict__ Bm = P.Bm;
  float* __restrict__ part = P.part;
  float* __restrict__ part_h = P.part_h;
  const int Kc = P.Kc, M = a.M, R = P.R, ldg = P.ldg, rows_per_split = a.rows_per_split;
  const int col_group = (int)blockIdx.x - (which ? a.cg_end[which - 1] : 0);
  __shared__ __attribute__((aligned(16))) char stage[4 * kTrWaveLds];
  static_assert(sizeof(stage) >= 3 * 32 * 64 * sizeof(float), "the reduction reuses the staging memory");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, i = lane & 15;
  const int c0 = col_group * kTnGhCols;
  const int split = blockIdx.y;
  const int m_begin = split * rows_per_split;
  int m_end = m_begin + rows_per_split;
  m_end = m_end < M ? m_end : M;

  char* my = stage + wave * kTrWaveLds;
  // copy-in and transposed read-back roles as in skinny_tn; piece p holds columns c0 + 128 p .. + 127
  bool xcol_ok[2];
  const uint16_t* xsrc[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int xcol = c0 + 128 * p + 8 * i;
    xcol_ok[p] = xcol < Kc;  // Kc % 8 == 0
    xsrc[p] = X + (xcol_ok[p] ? xcol : 0);
  }
  char* xdst = my + g * kTrPitchX + 16 * i;
  const int gcol = 8 * (lane & 1);  // R % 8 == 0: a lane's 8 columns are all in or all out
  char* gdst = my + 32 * kTrPitchX + (lane >> 1) * 32 + 16 * (lane & 1);
  const uint32_t my_lds = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)my);
  const uint32_t xrd = my_lds + (8 * g + (i >> 2)) * kTrPitchX + 8 * (i & 3);
  const uint32_t grd = my_lds + 32 * kTrPitchX + (8 * g + (i >> 2)) * 32 + 8 * (i & 3);
  // the piece as it lies, for gh: row 16 t + i, the 8 columns 64 H + 16 g + 8 hh .. + 7 (16 bytes)
  const char* prd = my + i * kTrPitchX + 32 * g;

  // ---- the operand Bm[c0 + 128 p + 64 H + 16 g + 8 hh + (0 .. 7)][i] of every (p, H, hh): rows of Bm are R contiguous
  //      elements, so a piece is 16 R chunks of 16 bytes; staged at 32 bytes a row (columns R .. 15 stay unwritten: they
  //      only reach output columns that are never stored), rows beyond Kc as zeros
  u32x4_t bfrag[2][2][2];
  {
    const int ppr = R >> 3;  // chunks per row
    const uint32_t brd = my_lds + (16 * g + (i >> 2)) * 32 + 8 * (i & 3);
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int pc = lane + 64 * q;
        if (pc < 16 * R) {
          const int n = c0 + 128 * p + pc / ppr;
          u32x4_t v = u32x4_t{0, 0, 0, 0};
          if (n < Kc) v = *reinterpret_cast<const u32x4_t*>(Bm + (int64_t)n * R + 8 * (pc % ppr));
          *reinterpret_cast<u32x4_t*>(my + (pc / ppr) * 32 + 16 * (pc % ppr)) = v;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // LDS operations of a wave complete in order
      u32x2_t lo[2][2], hi[2][2];
#pragma unroll
      for (int H = 0; H < 2; ++H)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          lo[H][hh] = lds_read_tr16(brd, (64 * H + 8 * hh) * 32);
          hi[H][hh] = lds_read_tr16(brd, (64 * H + 8 * hh + 4) * 32);
        }
#pragma unroll
      for (int H = 0; H < 2; ++H)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[H][hh]), "+v"(hi[H][hh]));
          bfrag[p][H][hh] = u32x4_t{lo[H][hh].x, lo[H][hh].y, hi[H][hh].x, hi[H][hh].y};
        }
    }
  }

  f32x4_t acc[2][8];
#pragma unroll
  for (int p = 0; p < 2; ++p)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[p][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  u32x4_t xv[2][8], gv;
  auto fetch = [&](int m) {  // rows m .. m + 31 into registers
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int row = m + 4 * u + g;
        xv[p][u] = u32x4_t{0, 0, 0, 0};
        if (row < m_end && xcol_ok[p]) xv[p][u] = *reinterpret_cast<const u32x4_t*>(xsrc[p] + (int64_t)row * Kc);
      }
    const int grow = m + (lane >> 1);
    gv = u32x4_t{0, 0, 0, 0};
    if (grow < m_end && gcol < R) gv = *reinterpret_cast<const u32x4_t*>(G + (int64_t)grow * ldg + gcol);
  };
  int m = m_begin + 32 * wave;
  if (m < m_end) fetch(m);
  for (; m < m_end; m += 128) {
    f32x4_t acc_h[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};
    u32x4_t gop;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      // every read of this region has been waited for before the MFMA that used it
#pragma unroll
      for (int u = 0; u < 8; ++u) *reinterpret_cast<u32x4_t*>(xdst + 4 * u * kTrPitchX) = xv[p][u];
      if (p == 0) *reinterpret_cast<u32x4_t*>(gdst) = gv;  // zeros beyond R
      if (p == 1 && m + 128 < m_end) fetch(m + 128);      // in flight while this step is multiplied
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the copy-in has landed
      if (p == 0) {
        u32x2_t ga = lds_read_tr16(grd, 0), gb = lds_read_tr16(grd, 4 * 32);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ga), "+v"(gb));
        gop = u32x4_t{ga.x, ga.y, gb.x, gb.y};
      }
      u32x2_t xa[8], xb[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        xa[e] = lds_read_tr16(xrd, 32 * e);
        xb[e] = lds_read_tr16(xrd, 32 * e + 4 * kTrPitchX);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(xa[e]), "+v"(xb[e]) : "n"(14 - 2 * e));
        const u32x4_t xop = {xa[e].x, xa[e].y, xb[e].x, xb[e].y};
        acc[p][e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, gop), __builtin_bit_cast(bf16x8_t, xop),
                                                           acc[p][e], 0, 0, 0);
      }
      u32x4_t pr[2][2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int H = 0; H < 2; ++H)
#pragma unroll
          for (int hh = 0; hh < 2; ++hh)
            pr[t][H][hh] = *reinterpret_cast<const u32x4_t*>(prd + 16 * t * kTrPitchX + 128 * H + 16 * hh);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // before the region is written again
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int H = 0; H < 2; ++H)
#pragma unroll
          for (int hh = 0; hh < 2; ++hh)
            acc_h[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, pr[t][H][hh]),
                                                              __builtin_bit_cast(bf16x8_t, bfrag[p][H][hh]), acc_h[t], 0, 0, 0);
    }
    // acc_h[t][v] = sum over the workgroup's columns of GY[m + 16 t + 4 g + v][.] * Bm[.][i]
    if (i < R) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int row = m + 16 * t + 4 * g + v;
          if (row < m_end) part_h[((int64_t)col_group * M + row) * R + i] = acc_h[t][v];
        }
    }
  }
  float (*red)[32][64] = reinterpret_cast<float (*)[32][64]>(stage);
  // acc[p][e][v] = sum over this wave's rows of H[.][4 g + v] * GY[.][c0 + 128 p + 16 e + i]; one piece at a time meets in
  // the staging memory
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    __syncthreads();  // the staging regions (or the previous piece's sums) are free
    if (wave > 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave - 1][v * 8 + e][lane] = acc[p][e][v];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int r = 4 * g + v;
        if (r >= R) continue;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int col = c0 + 128 * p + 16 * e + i;
          if (col >= Kc) continue;
          part[((int64_t)split * R + r) * Kc + col] =
              ((acc[p][e][v] + red[0][v * 8 + e][lane]) + red[1][v * 8 + e][lane]) + red[2][v * 8 + e][lane];
        }
      }
    }
  }
#endif
}

// ---------------------------------------------------------------------------------------------------
// swiglu_bwd_tn_gh: the backward of act = silu(gate) * up (torchtune/modules/feed_forward.py:50-53) and, from the same
// pass, both products of the gate / up pair's adapters that read the gradients it produces.  The stand-alone sequence is
// ttamd_swiglu_bwd_bf16 (reads gact, gate, up; writes ggate, gup) followed by skinny_tn_gh on (ggate, gup), which reads
// the two gradients back; here a wave computes a 32 x 128 piece of ggate and of gup from the matching pieces of gact,
// gate and up (swiglu_math.h: the bits of the stand-alone kernel), stores both, and feeds them from its registers to
// the LDS copy-in of skinny_tn_gh's two products, member 0 (gate) and then member 1 (up).  Sums, their order and the
// partial-sum layouts are those of skinny_tn_gh_kernel on a batch of the two members, so every result is the same bits.
// The inputs of the next piece are requested while the current one is multiplied.
// ---------------------------------------------------------------------------------------------------
struct SwigluGhArgs {
  const uint16_t* gact;  // [M, Kc]
  const uint16_t* gate;  // [M, Kc]
  const uint16_t* up;    // [M, Kc]
  uint16_t* gx[2];       // out: ggate, gup [M, Kc]
  const uint16_t* G[2];  // h of the member: rows ldg elements apart
  const uint16_t* Bm[2]; // lora_b [Kc, R]
  float* part[2];        // [splits, R, Kc]
  float* part_h[2];      // [column groups, M, R]
  int R[2];
  int Kc, ldg, M, rows_per_split;
};

__global__ __launch_bounds__(256) void swiglu_bwd_tn_gh_kernel(const SwigluGhArgs a) {
  constexpr int kTrWaveLds = tn_wave_lds(1);
#if defined(__HIP_DEVICE_COMPILE__)
  const int Kc = a.Kc, M = a.M, ldg = a.ldg, rows_per_split = a.rows_per_split;
  const int col_group = (int)blockIdx.x;
  __shared__ __attribute__((aligned(16))) char stage[4 * kTrWaveLds];
  static_assert(sizeof(stage) >= 3 * 32 * 64 * sizeof(float), "the reduction reuses the staging memory");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g = lane >> 4, i = lane & 15;
  const int c0 = col_group * kTnGhCols;
  const int split = blockIdx.y;
  const int m_begin = split * rows_per_split;
  int m_end = m_begin + rows_per_split;
  m_end = m_end < M ? m_end : M;

  char* my = stage + wave * kTrWaveLds;
  bool xcol_ok[2];
  int64_t xcol[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int c = c0 + 128 * p + 8 * i;
    xcol_ok[p] = c < Kc;  // Kc % 8 == 0
    xcol[p] = xcol_ok[p] ? c : 0;
  }
  char* xdst = my + g * kTrPitchX + 16 * i;
  const int gcol = 8 * (lane & 1);
  char* gdst = my + 32 * kTrPitchX + (lane >> 1) * 32 + 16 * (lane & 1);
  const uint32_t my_lds = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)my);
  const uint32_t xrd = my_lds + (8 * g + (i >> 2)) * kTrPitchX + 8 * (i & 3);
  const uint32_t grd = my_lds + 32 * kTrPitchX + (8 * g + (i >> 2)) * 32 + 8 * (i & 3);
  const char* prd = my + i * kTrPitchX + 32 * g;

  // Bm operands of both members, staged and read back as in skinny_tn_gh_kernel
  u32x4_t bfrag[2][2][2][2];
#pragma unroll
  for (int mem = 0; mem < 2; ++mem) {
    const uint16_t* __restrict__ Bm = a.Bm[mem];
    const int R = a.R[mem];
    const int ppr = R >> 3;
    const uint32_t brd = my_lds + (16 * g + (i >> 2)) * 32 + 8 * (i & 3);
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int pc = lane + 64 * q;
        if (pc < 16 * R) {
          const int n = c0 + 128 * p + pc / ppr;
          u32x4_t v = u32x4_t{0, 0, 0, 0};
          if (n < Kc) v = *reinterpret_cast<const u32x4_t*>(Bm + (int64_t)n * R + 8 * (pc % ppr));
          *reinterpret_cast<u32x4_t*>(my + (pc / ppr) * 32 + 16 * (pc % ppr)) = v;
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // LDS operations of a wave complete in order
      u32x2_t lo[2][2], hi[2][2];
#pragma unroll
      for (int H = 0; H < 2; ++H)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          lo[H][hh] = lds_read_tr16(brd, (64 * H + 8 * hh) * 32);
          hi[H][hh] = lds_read_tr16(brd, (64 * H + 8 * hh + 4) * 32);
        }
#pragma unroll
      for (int H = 0; H < 2; ++H)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[H][hh]), "+v"(hi[H][hh]));
          bfrag[mem][p][H][hh] = u32x4_t{lo[H][hh].x, lo[H][hh].y, hi[H][hh].x, hi[H][hh].y};
        }
    }
  }

  f32x4_t acc[2][2][8];
#pragma unroll
  for (int mem = 0; mem < 2; ++mem)
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[mem][p][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // the inputs of one piece: rows m + 4 u + g, the 8 columns at xcol[p]
  u32x4_t in_o[8], in_g[8], in_u[8], gv[2];
  auto fetch_u = [&](int m, int p, int u) {
    const int row = m + 4 * u + g;
    in_o[u] = in_g[u] = in_u[u] = u32x4_t{0, 0, 0, 0};
    if (row < m_end && xcol_ok[p]) {
      const int64_t at = (int64_t)row * Kc + xcol[p];
      in_o[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(a.gact + at));
      in_g[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(a.gate + at));
      in_u[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(a.up + at));
    }
  };
  auto fetch = [&](int m, int p) {
#pragma unroll
    for (int u = 0; u < 8; ++u) fetch_u(m, p, u);
  };
  auto fetch_h = [&](int m) {
    const int grow = m + (lane >> 1);
#pragma unroll
    for (int mem = 0; mem < 2; ++mem) {
      gv[mem] = u32x4_t{0, 0, 0, 0};
      if (grow < m_end && gcol < a.R[mem]) gv[mem] = *reinterpret_cast<const u32x4_t*>(a.G[mem] + (int64_t)grow * ldg + gcol);
    }
  };
  int m = m_begin + 32 * wave;
  if (m < m_end) {
    fetch(m, 0);
    fetch_h(m);
  }
  for (; m < m_end; m += 128) {
    f32x4_t acc_h[2][2];
#pragma unroll
    for (int mem = 0; mem < 2; ++mem) acc_h[mem][0] = acc_h[mem][1] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    u32x4_t gop[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      // the piece of both gradients, stored and kept in registers for the two copy-ins below; as soon as a row group's
      // inputs are used up, the same registers are asked for the next piece's, so that those requests are in flight
      // through the arithmetic of the remaining row groups and the products below
      u32x4_t xg[2][8];
      const bool more = p == 0 || m + 128 < m_end;  // uniform over the wave
      const int next_m = p == 0 ? m : m + 128, next_p = p ^ 1;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          uint32_t dg, du;
          swiglu_bwd_pair(in_o[u][d], in_g[u][d], in_u[u][d], dg, du);
          xg[0][u][d] = dg;
          xg[1][u][d] = du;
        }
        if (more) fetch_u(next_m, next_p, u);
        const int row = m + 4 * u + g;
        if (row < m_end && xcol_ok[p]) {
          const int64_t at = (int64_t)row * Kc + xcol[p];
          __builtin_nontemporal_store(xg[0][u], reinterpret_cast<u32x4_t*>(a.gx[0] + at));
          __builtin_nontemporal_store(xg[1][u], reinterpret_cast<u32x4_t*>(a.gx[1] + at));
        }
      }
      u32x4_t gvn[2] = {gv[0], gv[1]};
      if (p == 1 && more) fetch_h(m + 128);
#pragma unroll
      for (int mem = 0; mem < 2; ++mem) {
        // every read of this region has been waited for before the MFMA that used it
#pragma unroll
        for (int u = 0; u < 8; ++u) *reinterpret_cast<u32x4_t*>(xdst + 4 * u * kTrPitchX) = xg[mem][u];
        if (p == 0) *reinterpret_cast<u32x4_t*>(gdst) = gvn[mem];  // zeros beyond R
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // the copy-in has landed
        if (p == 0) {
          u32x2_t ga = lds_read_tr16(grd, 0), gb = lds_read_tr16(grd, 4 * 32);
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ga), "+v"(gb));
          gop[mem] = u32x4_t{ga.x, ga.y, gb.x, gb.y};
        }
        u32x2_t xa[8], xb[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          xa[e] = lds_read_tr16(xrd, 32 * e);
          xb[e] = lds_read_tr16(xrd, 32 * e + 4 * kTrPitchX);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(xa[e]), "+v"(xb[e]) : "n"(14 - 2 * e));
          const u32x4_t xop = {xa[e].x, xa[e].y, xb[e].x, xb[e].y};
          acc[mem][p][e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, gop[mem]), __builtin_bit_cast(bf16x8_t, xop),
                                                                  acc[mem][p][e], 0, 0, 0);
        }
        u32x4_t pr[2][2][2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int H = 0; H < 2; ++H)
#pragma unroll
            for (int hh = 0; hh < 2; ++hh)
              pr[t][H][hh] = *reinterpret_cast<const u32x4_t*>(prd + 16 * t * kTrPitchX + 128 * H + 16 * hh);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // before the region is written again
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int H = 0; H < 2; ++H)
#pragma unroll
            for (int hh = 0; hh < 2; ++hh)
              acc_h[mem][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, pr[t][H][hh]),
                                                                     __builtin_bit_cast(bf16x8_t, bfrag[mem][p][H][hh]), acc_h[mem][t], 0, 0, 0);
      }
    }
#pragma unroll
    for (int mem = 0; mem < 2; ++mem) {
      const int R = a.R[mem];
      if (i < R) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int row = m + 16 * t + 4 * g + v;
            if (row < m_end) a.part_h[mem][((int64_t)col_group * M + row) * R + i] = acc_h[mem][t][v];
          }
      }
    }
  }
  float (*red)[32][64] = reinterpret_cast<float (*)[32][64]>(stage);
#pragma unroll
  for (int mem = 0; mem < 2; ++mem) {
    const int R = a.R[mem];
    float* __restrict__ part = a.part[mem];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      __syncthreads();  // the staging regions (or the previous piece's sums) are free
      if (wave > 0) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
#pragma unroll
          for (int v = 0; v < 4; ++v) red[wave - 1][v * 8 + e][lane] = acc[mem][p][e][v];
      }
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int r = 4 * g + v;
          if (r >= R) continue;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int col = c0 + 128 * p + 16 * e + i;
            if (col >= Kc) continue;
            part[((int64_t)split * R + r) * Kc + col] =
                ((acc[mem][p][e][v] + red[0][v * 8 + e][lane]) + red[1][v * 8 + e][lane]) + red[2][v * 8 + e][lane];
          }
        }
      }
    }
  }
#endif
}

// out[r * stride_r + k * stride_k] = bf16(scale * sum_s part[s * split_stride + r * Kc + k]) for r < R, k < Kc
struct TnSum {
  const float* part;
  uint16_t* out;
  int Kc, R;
  float scale;
  int64_t split_stride, stride_r, stride_k;
  int splits;
};
constexpr int kTnMaxSums = 2 * kMaxGroup;
struct TnSumBatch {
  TnSum p[kTnMaxSums];
  int64_t end[kTnMaxSums];  // threads [end[i - 1], end[i]) finish problem i
  int n;
};
// The reductions of every row contraction of a backward in one launch.
__global__ __launch_bounds__(256) void sum_partials_tn_kernel(const TnSumBatch a) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  int which = 0;
#pragma unroll
  for (int q = 0; q < kTnMaxSums - 1; ++q)
    if (q < a.n - 1 && i >= a.end[q]) which = q + 1;
  if (i >= a.end[a.n - 1]) return;
  if (which) i -= a.end[which - 1];
  const TnSum& P = a.p[which];
  float s = 0.f;
#pragma unroll 8
  for (int q = 0; q < P.splits; ++q) s += P.part[(int64_t)q * P.split_stride + i];
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
size_t align256(size_t v) { return (v + 255) & ~size_t(255); }
// fp32 partial sums of one column contraction; 0 when a single slice writes the result directly
size_t nt_part_bytes(int64_t M, int64_t Kc, int R) {
  const int sp = plan_nt(M, Kc).splits;
  return sp > 1 ? align256((size_t)sp * M * R * sizeof(float)) : 0;
}

// Fills in the slicing of the batch's problems (operands, Kc, R, ldo, out, scale are the caller's), hands each sliced
// problem its piece of `ws` and launches: first pass, then the fixed-order sums of the sliced problems.
// bt: the second operand is [Kc, R] row-major (transposed inside the kernel) instead of [R, Kc].
int run_nt_batch(NtBatch& b, int n, bool bt, float* ws, hipStream_t s) {
  int max_splits = 1, max_r = 0;
  int64_t max_mr = 0;
  const int m_tiles = plan_nt(b.M, 64).m_tiles;
  char* w = reinterpret_cast<char*>(ws);
  for (int i = 0; i < n; ++i) {
    NtProblem& P = b.p[i];
    const NtPlan pl = plan_nt(b.M, P.Kc);
    P.splits = pl.splits;
    P.chunks_per_split = pl.chunks_per_split;
    P.part = reinterpret_cast<float*>(w);
    w += nt_part_bytes(b.M, P.Kc, P.R);
    max_splits = pl.splits > max_splits ? pl.splits : max_splits;
    max_r = P.R > max_r ? P.R : max_r;
    if (pl.splits > 1 && (int64_t)b.M * P.R > max_mr) max_mr = (int64_t)b.M * P.R;
  }
  const dim3 grid((unsigned)m_tiles, (unsigned)max_splits, (unsigned)n), block(256);
  if (bt) {
    if (max_r <= 16) skinny_nt_kernel<1, true><<<grid, block, 0, s>>>(b);
    else if (max_r <= 32) skinny_nt_kernel<2, true><<<grid, block, 0, s>>>(b);
    else skinny_nt_kernel<4, true><<<grid, block, 0, s>>>(b);
  } else {
    if (max_r <= 16) skinny_nt_kernel<1, false><<<grid, block, 0, s>>>(b);
    else if (max_r <= 32) skinny_nt_kernel<2, false><<<grid, block, 0, s>>>(b);
    else skinny_nt_kernel<4, false><<<grid, block, 0, s>>>(b);
  }
  if (max_mr > 0) sum_partials_kernel<<<dim3((unsigned)((max_mr + 255) / 256), (unsigned)n), block, 0, s>>>(b);
  return check_launch("skinny_nt");
}

struct TnPlan {
  int splits, rows_per_split;
};
// Every row contraction of a backward in one grid: `col_groups` workgroups along x, the same row splits for all.
TnPlan plan_tn(int64_t M, int64_t col_groups) {
  TnPlan p;
  int s = (int)(kTargetWaves / 4 / col_groups);  // workgroups of 4 waves
  s = s < 1 ? 1 : s;
  const int max_s = (int)((M + 127) / 128);  // at least 128 rows per split: one 32-row step per wave
  s = s > max_s ? max_s : s;
  p.rows_per_split = (int)(((M + s - 1) / s + 127) / 128 * 128);  // whole rounds of the four waves
  p.splits = (int)((M + p.rows_per_split - 1) / p.rows_per_split);
  return p;
}
int64_t tn_col_groups(int64_t Kc) { return (Kc + kTnCols - 1) / kTnCols; }

// The caller fills G, X, Kc, R, ldg of the n problems of `b` and the outputs of the ns sums of `f` (part, split_stride,
// splits and end are set here: sum i reads rows [sum_row0[i], + f.p[i].R) of problem sum_problem[i]).  The ns_ready sums
// that follow them in `f` are complete already (partial sums of an earlier launch) and ride along in the one reduction.
int run_tn_batch(TnBatch& b, int n, TnSumBatch& f, int ns, const int* sum_problem, const int* sum_row0, float* ws, hipStream_t s,
                 int ns_ready = 0) {
  int64_t groups = 0;
  for (int i = 0; i < n; ++i) {
    groups += tn_col_groups(b.p[i].Kc);
    b.cg_end[i] = (int)groups;
  }
  const TnPlan pl = plan_tn(b.M, groups);
  b.n = n;
  b.rows_per_split = pl.rows_per_split;
  float* w = ws;
  for (int i = 0; i < n; ++i) {
    b.p[i].part = w;
    w += (size_t)pl.splits * b.p[i].R * b.p[i].Kc;
  }
  int rgm = 1;
  for (int i = 0; i < n; ++i) rgm = (b.p[i].R + 15) / 16 > rgm ? (b.p[i].R + 15) / 16 : rgm;
  const dim3 grid((unsigned)groups, (unsigned)pl.splits), block(256);
  if (rgm == 1) skinny_tn_kernel<1><<<grid, block, 0, s>>>(b);
  else if (rgm == 2) skinny_tn_kernel<2><<<grid, block, 0, s>>>(b);
  else if (rgm == 3) skinny_tn_kernel<3><<<grid, block, 0, s>>>(b);
  else skinny_tn_kernel<4><<<grid, block, 0, s>>>(b);
  int64_t end = 0;
  for (int i = 0; i < ns; ++i) {
    const TnProblem& P = b.p[sum_problem[i]];
    f.p[i].part = P.part + (int64_t)sum_row0[i] * P.Kc;
    f.p[i].Kc = P.Kc;
    f.p[i].split_stride = (int64_t)P.R * P.Kc;
    f.p[i].splits = pl.splits;
    end += (int64_t)f.p[i].R * P.Kc;
    f.end[i] = end;
  }
  for (int i = ns; i < ns + ns_ready; ++i) {
    end += (int64_t)f.p[i].R * f.p[i].Kc;
    f.end[i] = end;
  }
  f.n = ns + ns_ready;
  sum_partials_tn_kernel<<<dim3((unsigned)((end + 255) / 256)), dim3(256), 0, s>>>(f);
  return check_launch("skinny_tn");
}
// fp32 partial sums of a batch of row contractions: sum over problems of splits * R * Kc
size_t tn_part_bytes(int64_t M, int n, const int64_t* Kc, const int* R) {
  int64_t groups = 0, elems = 0;
  for (int i = 0; i < n; ++i) {
    groups += tn_col_groups(Kc[i]);
    elems += (int64_t)R[i] * Kc[i];
  }
  return (size_t)plan_tn(M, groups).splits * elems * sizeof(float);
}

// ---- gh and gB from one pass over gy (skinny_tn_gh_kernel) ------------------------------------------------------------
// Taken when every member is wide and of rank <= 16: the pass over gy that gh alone would need then costs more than the
// partial sums the fused kernel writes and the launch of their reduction (measured on [8192, 14336] pairs: 88 us for the
// pass against ~30 us for the partial sums, the second reduction and the extra launch; at 4096 columns both are ~15 us).
constexpr int64_t kTnGhMinCols = 8192, kTnGhMinRows = 1024;  // fewer rows: the launches themselves are what a backward costs
bool tn_gh_applies(const GroupSkinny& g) {
  for (int i = 0; i < g.n; ++i)
    if (g.N[i] < kTnGhMinCols || g.rank[i] > 16) return false;
  return g.n >= 1 && g.n <= kMaxGroup && g.M >= kTnGhMinRows;
}
int64_t tn_gh_col_groups(int64_t Kc) { return (Kc + kTnGhCols - 1) / kTnGhCols; }
TnPlan plan_tn_gh(const GroupSkinny& g) {
  int64_t groups = 0;
  for (int i = 0; i < g.n; ++i) groups += tn_gh_col_groups(g.N[i]);
  return plan_tn(g.M, groups);
}
// The pair kernel (swiglu_bwd_tn_gh_kernel) serves both members from one workgroup per column group.
bool tn_gh_pair(const GroupSkinny& g) { return g.n == 2 && g.N[0] == g.N[1]; }
TnPlan plan_tn_gh_pair(const GroupSkinny& g) {
  // The pair kernel holds a compute unit by itself (one workgroup of four waves at its register count), and what a
  // workgroup does once - staging lora_b, the reduction of its sums - is a tenth of a 1024-row range's time: one round of
  // long ranges beats two of short ones (8192 x 14336: 288 us with 4 splits = 224 workgroups against 302 with 8 and 388
  // with 5, which start a second round; 4096 x 28672: 284 with 2, 303 with 4; 8192 x 8192: 170 with 8, 186 with 16).
  // Hence: as many row splits as still fit one round of the chip.
  const int64_t col_groups = tn_gh_col_groups(g.N[0]);
  constexpr int64_t kCUs = 256;  // MI355X
  int s = (int)(kCUs / col_groups);
  s = s < 1 ? 1 : s;
  const int max_s = (int)((g.M + 127) / 128);
  s = s > max_s ? max_s : s;
  TnPlan p;
  p.rows_per_split = (int)(((g.M + s - 1) / s + 127) / 128 * 128);
  p.splits = (int)((g.M + p.rows_per_split - 1) / p.rows_per_split);
  return p;
}
// fp32 partial sums of the fused pass: per member the column groups' [M, R] and the row splits' [R, N] (room for the
// plan with more splits where both kernels can serve the group)
size_t tn_gh_part_bytes(const GroupSkinny& g) {
  TnPlan pl = plan_tn_gh(g);
  if (tn_gh_pair(g) && plan_tn_gh_pair(g).splits > pl.splits) pl = plan_tn_gh_pair(g);
  size_t total = 0;
  for (int i = 0; i < g.n; ++i)
    total += align256(((size_t)tn_gh_col_groups(g.N[i]) * g.M + (size_t)pl.splits * g.N[i]) * g.rank[i] * sizeof(float));
  return total;
}

// h = x . A^T for one layer
int run_hidden(const uint16_t* x, const uint16_t* lora_a, int64_t M, int64_t K, int R, uint16_t* h, float* ws, hipStream_t s) {
  NtBatch b = {};
  b.M = (int)M;
  NtProblem& P = b.p[0];
  P.X = x;
  P.bm[0] = lora_a;
  P.r_off[0] = 0;
  P.r_off[1] = R;
  P.nb = 1;
  P.out = h;
  P.Kc = (int)K; P.R = R; P.ldo = R;
  P.scale = 1.0f;
  return run_nt_batch(b, 1, false, ws, s);
}

int check_skinny(const char* who, int64_t M, int64_t N, int64_t K, int rank) {
  TT_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1 << 30) && N < (1 << 30) && K < (1 << 30), "%s: bad shape M=%lld N=%lld K=%lld",
             who, (long long)M, (long long)N, (long long)K);
  TT_REQUIRE(K % 64 == 0 && N % 64 == 0, "%s: K (%lld) and N (%lld) must be multiples of 64", who, (long long)K, (long long)N);
  TT_REQUIRE(rank > 0 && rank <= 64 && rank % 8 == 0, "%s: rank (%d) must be a multiple of 8 in [8, 64]", who, rank);
  return TTAMD_OK;
}

}  // namespace

size_t group_hidden_ws_bytes(int64_t M, int64_t K, int r_total) { return nt_part_bytes(M, K, r_total); }

int run_group_hidden(const uint16_t* x, const GroupSkinny& g, uint16_t* h_cat, float* ws, hipStream_t s) {
  NtBatch b = {};
  b.M = (int)g.M;
  NtProblem& P = b.p[0];
  P.X = x;
  for (int i = 0; i < g.n; ++i) {
    P.bm[i] = g.lora_a[i];
    P.r_off[i] = g.r_off[i];
  }
  P.r_off[g.n] = g.r_off[g.n];
  P.nb = g.n;
  P.out = h_cat;
  P.Kc = (int)g.K; P.R = g.r_off[g.n]; P.ldo = g.r_off[g.n];
  P.scale = 1.0f;
  return run_nt_batch(b, 1, false, ws, s);
}

size_t group_lora_bwd_ws_bytes(const GroupSkinny& g) {
  if (tn_gh_applies(g)) {
    const int64_t width = g.K;
    const int r_total = g.r_off[g.n];
    return align256(tn_gh_part_bytes(g) + tn_part_bytes(g.M, 1, &width, &r_total));
  }
  size_t nt = 0;
  int64_t widths[kTnMaxProblems];
  int ranks[kTnMaxProblems];
  widths[0] = g.K;
  ranks[0] = g.r_off[g.n];
  for (int i = 0; i < g.n; ++i) {
    nt += nt_part_bytes(g.M, g.N[i], g.rank[i]);
    widths[1 + i] = g.N[i];
    ranks[1 + i] = g.rank[i];
  }
  const size_t tn = tn_part_bytes(g.M, 1 + g.n, widths, ranks);
  return align256(nt > tn ? nt : tn);
}

int run_group_lora_bwd(const uint16_t* x, const uint16_t* h_cat, const GroupSkinny& g, uint16_t* gh_cat, float* ws, hipStream_t s,
                       const SwigluBwdInputs* sw) {
  const int rt = g.r_off[g.n];
  // the pair's gradients from the pass that reads them (swiglu_bwd_tn_gh_kernel) where that pass exists
  const bool sw_fused = sw && tn_gh_pair(g) && tn_gh_applies(g);
  if (sw) {
    TT_REQUIRE(g.n == 2 && g.N[0] == g.N[1] && sw->gact && sw->gate && sw->up && aligned16(sw->gact) && aligned16(sw->gate) &&
                   aligned16(sw->up) && aligned16(g.gy[0]) && aligned16(g.gy[1]),
               "lora_group_swiglu_bwd: takes the gate and the up projection (equal widths) and 16-byte aligned gact, gate, up, ggate, gup");
    if (!sw_fused)
      if (int rc = ttamd_swiglu_bwd_bf16(sw->gact, sw->gate, sw->up, const_cast<uint16_t*>(g.gy[0]), const_cast<uint16_t*>(g.gy[1]),
                                         g.M * g.N[0], s))
        return rc;
  }
  if (tn_gh_applies(g)) {
    // one pass over every gy for gB and gh, the column groups of gh summed, then gA over x; the reductions of gA and gB
    // share the last launch
    const TnPlan pl = sw_fused ? plan_tn_gh_pair(g) : plan_tn_gh(g);
    TnGhBatch b = {};
    NtBatch sums = {};
    TnSumBatch f = {};
    b.M = sums.M = (int)g.M;
    b.n = g.n;
    b.rows_per_split = pl.rows_per_split;
    char* w = reinterpret_cast<char*>(ws);
    int64_t groups = 0;
    for (int i = 0; i < g.n; ++i) {
      const int64_t cg = tn_gh_col_groups(g.N[i]);
      TnGhProblem& P = b.p[i];
      P.G = h_cat + g.r_off[i];
      P.X = g.gy[i];
      P.Bm = g.lora_b[i];
      P.part_h = reinterpret_cast<float*>(w);
      P.part = P.part_h + (size_t)cg * g.M * g.rank[i];
      w += align256(((size_t)cg * g.M + (size_t)pl.splits * g.N[i]) * g.rank[i] * sizeof(float));
      P.Kc = (int)g.N[i]; P.R = g.rank[i]; P.ldg = rt;
      groups += cg;
      b.cg_end[i] = (int)groups;
      NtProblem& S = sums.p[i];  // gh_cat[:, member i] = bf16(scale . sum over column groups)
      S.part = P.part_h;
      S.out = gh_cat + g.r_off[i];
      S.R = g.rank[i]; S.ldo = rt; S.splits = (int)cg;
      S.scale = g.scale[i];
      f.p[g.n + i] = TnSum{P.part, g.gb[i], (int)g.N[i], g.rank[i], g.scale[i], (int64_t)g.rank[i] * g.N[i], 1, g.rank[i], pl.splits};
    }
    if (sw_fused) {
      SwigluGhArgs f2 = {};
      f2.gact = sw->gact; f2.gate = sw->gate; f2.up = sw->up;
      for (int i = 0; i < 2; ++i) {
        f2.gx[i] = const_cast<uint16_t*>(g.gy[i]);
        f2.G[i] = b.p[i].G; f2.Bm[i] = b.p[i].Bm; f2.part[i] = b.p[i].part; f2.part_h[i] = b.p[i].part_h; f2.R[i] = b.p[i].R;
      }
      f2.Kc = (int)g.N[0]; f2.ldg = rt; f2.M = (int)g.M; f2.rows_per_split = pl.rows_per_split;
      swiglu_bwd_tn_gh_kernel<<<dim3((unsigned)tn_gh_col_groups(g.N[0]), (unsigned)pl.splits), dim3(256), 0, s>>>(f2);
    } else {
      skinny_tn_gh_kernel<<<dim3((unsigned)groups, (unsigned)pl.splits), dim3(256), 0, s>>>(b);
    }
    sum_partials_kernel<<<dim3((unsigned)((g.M * 16 + 255) / 256), (unsigned)g.n), dim3(256), 0, s>>>(sums);
    if (int rc = check_launch("skinny_tn_gh")) return rc;
    TnBatch t = {};
    t.M = (int)g.M;
    t.p[0] = TnProblem{gh_cat, x, nullptr, (int)g.K, rt, rt};
    int sum_problem[kTnMaxSums], sum_row0[kTnMaxSums];
    for (int i = 0; i < g.n; ++i) {
      f.p[i] = TnSum{nullptr, g.ga[i], 0, g.rank[i], 1.0f, 0, g.K, 1};
      sum_problem[i] = 0;
      sum_row0[i] = g.r_off[i];
    }
    return run_tn_batch(t, 1, f, g.n, sum_problem, sum_row0, reinterpret_cast<float*>(w), s, g.n);
  }
  {
    NtBatch b = {};
    b.M = (int)g.M;
    for (int i = 0; i < g.n; ++i) {
      NtProblem& P = b.p[i];
      P.X = g.gy[i];
      P.bm[0] = g.lora_b[i];
      P.r_off[1] = g.rank[i];
      P.nb = 1;
      P.out = gh_cat + g.r_off[i];
      P.Kc = (int)g.N[i]; P.R = g.rank[i]; P.ldo = rt;
      P.scale = g.scale[i];
    }
    if (int rc = run_nt_batch(b, g.n, true, ws, s)) return rc;
  }
  TnBatch t = {};
  t.M = (int)g.M;
  t.p[0] = TnProblem{gh_cat, x, nullptr, (int)g.K, rt, rt};
  TnSumBatch f = {};
  int sum_problem[kTnMaxSums], sum_row0[kTnMaxSums];
  for (int i = 0; i < g.n; ++i) {
    t.p[1 + i] = TnProblem{h_cat + g.r_off[i], g.gy[i], nullptr, (int)g.N[i], g.rank[i], rt};
    f.p[i] = TnSum{nullptr, g.ga[i], 0, g.rank[i], 1.0f, 0, g.K, 1};
    sum_problem[i] = 0;
    sum_row0[i] = g.r_off[i];
    f.p[g.n + i] = TnSum{nullptr, g.gb[i], 0, g.rank[i], g.scale[i], 0, 1, g.rank[i]};
    sum_problem[g.n + i] = 1 + i;
    sum_row0[g.n + i] = 0;
  }
  return run_tn_batch(t, 1 + g.n, f, 2 * g.n, sum_problem, sum_row0, ws, s);
}

}  // namespace ttamd

using namespace ttamd;

extern "C" size_t ttamd_lora_fwd_workspace_bytes(int64_t M, int64_t K, int rank) {
  if (M <= 0 || K <= 0 || rank <= 0 || K % 64) return 0;
  return nt_part_bytes(M, K, rank);
}

extern "C" int ttamd_lora_hidden_bf16(const void* x, const void* lora_a, void* h, int64_t M, int64_t K, int rank,
                                      void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_skinny("lora_hidden", M, 64, K, rank)) return rc;
  TT_REQUIRE(x && lora_a && h, "lora_hidden: null pointer argument");
  const size_t need = ttamd_lora_fwd_workspace_bytes(M, K, rank);
  TT_REQUIRE(need == 0 || workspace, "lora_hidden: null workspace");
  TT_REQUIRE(aligned16(x) && aligned16(lora_a) && aligned16(workspace), "lora_hidden: pointers must be 16-byte aligned");
  if (workspace_bytes < need)
    return fail(TTAMD_EWORKSPACE, "lora_hidden: workspace has %zu bytes, needs %zu", workspace_bytes, need);
  return run_hidden(reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint16_t*>(lora_a), M, K, rank,
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
// runtime, not a device address: the address is asked for once per device (with that device current) and kept.  The
// slots are atomics because threads of different streams may make a device's first call together (both then store the
// same value).
int static_scratch(float** out) {
  static std::atomic<void*> ptr[64] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(TTAMD_ELAUNCH, "lora_hidden_static: hipGetDevice: %s", hipGetErrorString(e));
  void* p = (dev >= 0 && dev < 64) ? ptr[dev].load(std::memory_order_relaxed) : nullptr;
  if (p == nullptr) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_hidden_scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(TTAMD_ELAUNCH, "lora_hidden_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    if (dev >= 0 && dev < 64) ptr[dev].store(p, std::memory_order_relaxed);
  }
  *out = reinterpret_cast<float*>(p);
  return TTAMD_OK;
}
}  // namespace

// Resolves the scratch array's address on the current device.  The query may load the code object, which must not
// happen while a stream is being captured: callers that capture make this call (or one eager call of the entry point
// below) once per device beforehand.
extern "C" int ttamd_lora_hidden_static_init(void) {
  float* scratch = nullptr;
  return static_scratch(&scratch);
}

extern "C" size_t ttamd_lora_hidden_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int ttamd_lora_hidden_static_bf16(const void* x, const void* lora_a, void* h, int64_t M, int64_t K, int rank,
                                             void* stream) {
  if (int rc = check_skinny("lora_hidden_static", M, 64, K, rank)) return rc;
  TT_REQUIRE(x && lora_a && h, "lora_hidden_static: null pointer argument");
  TT_REQUIRE(aligned16(x) && aligned16(lora_a), "lora_hidden_static: pointers must be 16-byte aligned");
  const size_t need = nt_part_bytes(M, K, rank);  // 0: one slice writes the result directly
  if (need > kStaticScratchBytes)
    return fail(TTAMD_EWORKSPACE, "lora_hidden_static: M=%lld K=%lld rank=%d needs %zu bytes of partial sums, the built-in "
                "scratch holds %zu; use ttamd_lora_hidden_bf16 with a workspace", (long long)M, (long long)K, rank, need,
                kStaticScratchBytes);
  float* scratch = nullptr;
  if (int rc = static_scratch(&scratch)) return rc;
  // every partial sum the reduction reads is written by this call's first kernel: nothing has to start at zero
  return run_hidden(reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint16_t*>(lora_a), M, K, rank,
                    reinterpret_cast<uint16_t*>(h), scratch, reinterpret_cast<hipStream_t>(stream));
}

namespace {
// One layer as a group of one: the same launches, the same bits.
GroupSkinny single_layer(int64_t M, int64_t N, int64_t K, int rank, float scale, const void* gy, const void* lora_b, void* ga, void* gb) {
  GroupSkinny g = {};
  g.n = 1;
  g.M = M; g.K = K;
  g.N[0] = N;
  g.rank[0] = rank;
  g.r_off[1] = rank;
  g.scale[0] = scale;
  g.lora_b[0] = reinterpret_cast<const uint16_t*>(lora_b);
  g.gy[0] = reinterpret_cast<const uint16_t*>(gy);
  g.ga[0] = reinterpret_cast<uint16_t*>(ga);
  g.gb[0] = reinterpret_cast<uint16_t*>(gb);
  return g;
}
}  // namespace

extern "C" size_t ttamd_lora_bwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int rank) {
  if (M <= 0 || N <= 0 || K <= 0 || rank <= 0 || K % 64 || N % 64) return 0;
  return group_lora_bwd_ws_bytes(single_layer(M, N, K, rank, 1.0f, nullptr, nullptr, nullptr, nullptr));
}

extern "C" int ttamd_lora_bwd_bf16(const void* gy, const void* x, const void* h, const void* lora_b, float scale, void* gh,
                                   void* ga, void* gb, int64_t M, int64_t N, int64_t K, int rank, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  if (int rc = check_skinny("lora_bwd", M, N, K, rank)) return rc;
  TT_REQUIRE(gy && x && h && lora_b && gh && ga && gb && workspace, "lora_bwd: null pointer argument");
  TT_REQUIRE(aligned16(gy) && aligned16(x) && aligned16(h) && aligned16(lora_b) && aligned16(workspace) && aligned16(gh),
             "lora_bwd: pointers must be 16-byte aligned");
  if (workspace_bytes < ttamd_lora_bwd_workspace_bytes(M, N, K, rank))
    return fail(TTAMD_EWORKSPACE, "lora_bwd: workspace has %zu bytes, needs %zu", workspace_bytes,
                ttamd_lora_bwd_workspace_bytes(M, N, K, rank));
  // gh = scale . gy . B (lora_b [N, R] as it lies: the kernels transpose its pieces), gA[r][k] = sum_m gh[m][r] x[m][k],
  // gB[n][r] = scale . sum_m h[m][r] gy[m][n]
  return run_group_lora_bwd(reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint16_t*>(h),
                            single_layer(M, N, K, rank, scale, gy, lora_b, ga, gb), reinterpret_cast<uint16_t*>(gh),
                            reinterpret_cast<float*>(workspace), reinterpret_cast<hipStream_t>(stream));
}
