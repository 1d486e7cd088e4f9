// Many-token path of linear_nf4 / LoRALinear.forward (torchtune/modules/peft/lora.py:128-147; torchao's linear_nf4 =
// F.linear(x, W.to(dtype))) and of its grad-input: the reference's own order of work.  The NF4 weight is expanded ONCE
// per call into caller-provided scratch memory, then a plain bf16 GEMM runs on the matrix cores with the adapter, bias
// and column scale in its epilogue.  The fused kernel (nf4_gemm_rs.hip) repeats the expansion once per 256-row tile of
// the activations; from a few thousand tokens up that repetition costs more than one pass of the dequantise kernel.
//
//     C[M, Nout] = X[M, Kc] . Wd[Nout, Kc]^T  (+ bias, * cscale)  + sum_a (lscale_a . lX_a)[M, R_a] . lW_a[Nout, R_a]^T
//
// Layers with a common input run as one launch either way round.  Grad-input: the contraction is the concatenation of
// up to kGroupMax segments (X_s = gy_s, Wd_s = W_s^T), each with its own activation tensor, and every member's adapter
// adds to all output columns.  Forward: the output columns are the concatenation of the members' columns (widths
// multiples of the 256-wide tile), each member with its own output tensor, bias and adapter.
//
// The scratch copy `Wd` is written in the order the matrix cores consume it (v_mfma_f32_16x16x32_bf16): for every block
// of 16 output columns T and every 32-wide k-step t one 1 KiB piece in which lane l of a wave finds, at byte 16 l, the
// eight bf16 values Wd[16 T + l % 16][32 t + 8 (l / 16) .. + 7]:
//
//     tiled[T][t][lane][8]        T < Nout / 16, t < Kc / 32, lane < 64
//
// GEMM kernel: workgroup = 8 waves (two per SIMD), tile 256 x 256, k-step 32.  Both operands reach LDS by direct-to-LDS
// loads (activations as whole 128-byte lines into a ring of three 64-wide entries, weights into a ring of four stages).
// Wave (wm, wn) owns rows [128 wm, +128) x columns [64 wn, +64): 8 x 4 MFMA tiles, 128 accumulators per lane.  The two
// waves of a SIMD run half a step apart: while one issues the 32 MFMAs of a step, the other requests loads and reads its
// operands of the next step, and they swap at a workgroup barrier.  Measured on MI355X, the matrix pipe of a SIMD is
// handed back and forth without the vector-memory instructions of a wave ever delaying its own MFMAs, which is what
// limited the one-wave-per-SIMD form of this loop.  The 16 x 16 x 32 MFMA is used because this part is power-limited
// under matrix load and that shape sustains 13 % more FLOP/s than 32 x 32 x 16 at the same power (2.04 against
// 1.80 PFLOP/s for MFMA-only loops on random operands).
#include <type_traits>

#include "common.h"
#include "group.h"
#include "nf4_math.h"
#include "swiglu_math.h"

namespace ttamd {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2_t v;
  v.x = (__bf16)lo;
  v.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}

#define TT_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

__constant__ float kNF4Dense[16] = TT_NF4_TABLE;

// ---------------------------------------------------------------------------------------------------------------------
// Expansion into the tiled scratch copy.  A thread takes 32 consecutive contraction indices of one output column
// (16 bytes of codes) and writes the four 16-byte operands that lanes (col % 16) + 16 g, g = 0..3, of that piece read.
// Values are the bits ttamd_nf4_dequantize produces: nf4[code] * block scaler in fp32, rounded once to bf16.
//   MODE 0: codes [Nout, Kc / 2], block scalers [Nout, Kc / 64]            (forward, natural layout)
//   MODE 2: codes [Nout, Kc / 2], block scalers transposed [Kc / 64, Nout] (forward, when the backward copy exists)
//   MODE 1: codes of W^T [Nout, Kc / 2] with per-element scalers [Nout / 64, Kc] (grad-input: Nout = K, Kc = N)
//   (mode 3 of the launcher: grad-input from the weight's own codes, nf4_expand_tiled_transposed_kernel below)
// A workgroup of 256 threads covers 16 columns (one T) x 16 k-steps per iteration of its loop over the contraction.
// ---------------------------------------------------------------------------------------------------------------------
// One launch expands the weights of up to kGroupMax layers (the members of a group: stacked output columns in the forward,
// the concatenated contraction in the grad-input); workgroups [blk_end[i - 1], blk_end[i]) along x work on member i.
struct ExpandMember {
  const uint8_t* codes;
  const float* scal;
  char* tiled;   // the copy this member writes into (its own stretch of the forward copy, or the shared grad-input copy)
  int nout, kc;  // output columns and contraction length of the member's operand
  int t_off;     // its first 32-wide step in the copy's contraction
};
struct ExpandGroup {
  ExpandMember m[kGroupMax];
  int blk_end[kGroupMax];
  int n;
};
__device__ __forceinline__ int expand_member(const ExpandGroup& eg, int& blk) {
  int which = 0;  // uniform over the workgroup
#pragma unroll
  for (int q = 0; q < kGroupMax - 1; ++q)
    if (q < eg.n - 1 && blk >= eg.blk_end[q]) which = q + 1;
  if (which) blk -= eg.blk_end[which - 1];
  return which;
}

template <int MODE>
__global__ __launch_bounds__(256) void nf4_expand_tiled_kernel(const ExpandGroup eg, int nk_total, int paired) {
  __shared__ float2 lut[256];
  const int tid = threadIdx.x;
  lut[tid] = make_float2(round_to_bf16(kNF4Dense[tid >> 4]), round_to_bf16(kNF4Dense[tid & 15]));
  __syncthreads();
  int T = blockIdx.x;
  const ExpandMember& me = eg.m[expand_member(eg, T)];
  const uint8_t* __restrict__ codes = me.codes;
  const float* __restrict__ scal = me.scal;
  char* __restrict__ tiled = me.tiled;
  const int Nout = me.nout, Kc = me.kc, t_off = me.t_off;
  // paired: two weights of equal shape share one tiled copy, 128 columns (8 blocks) of the one followed by the same
  // 128 columns of the other (whose `tiled` starts 8 blocks further), so that a 256-wide tile of the GEMM holds both
  const int To = paired ? ((T >> 3) << 4) + (T & 7) : T;
  const int r = tid & 15;        // column inside the block
  const int col = 16 * T + r;
  const int nk = Kc >> 5;
  const int chunks = (nk + 15) >> 4;
  const int per = (chunks + gridDim.y - 1) / gridDim.y;
  const int c0 = blockIdx.y * per, c1 = c0 + per < chunks ? c0 + per : chunks;
  for (int c = c0; c < c1; ++c) {
    const int t = 16 * c + (tid >> 4);
    if (t >= nk) break;
    const u32x4_t cd = *reinterpret_cast<const u32x4_t*>(codes + (int64_t)col * (Kc >> 1) + 16 * t);
    float sc[32];
    if (MODE == 1) {
      const float* sp = scal + (int64_t)(col >> 6) * Kc + 32 * t;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const f32x4_t v = *reinterpret_cast<const f32x4_t*>(sp + 4 * q);
        sc[4 * q] = v.x; sc[4 * q + 1] = v.y; sc[4 * q + 2] = v.z; sc[4 * q + 3] = v.w;
      }
    } else {
      const float s1 = MODE == 0 ? scal[(int64_t)col * (Kc >> 6) + (t >> 1)] : scal[(int64_t)(t >> 1) * Nout + col];
#pragma unroll
      for (int q = 0; q < 32; ++q) sc[q] = s1;
    }
    char* piece = tiled + ((int64_t)To * nk_total + t_off + t) * 1024;
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const uint32_t w = cd[g4];
      u32x4_t o;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const float2 pr = lut[(w >> (8 * b)) & 0xffu];
        o[b] = pack_bf16x2(pr.x * sc[8 * g4 + 2 * b], pr.y * sc[8 * g4 + 2 * b + 1]);
      }
      *reinterpret_cast<u32x4_t*>(piece + (16 * g4 + r) * 16) = o;
    }
  }
}

// The same for the grad-input when the weight has no transposed copy: codes [N, K / 2] and block scalers [N, K / 64] as
// they lie, output = tiles of W^T (rows: k, contraction: n).  A workgroup expands 32 rows n (one 32-wide step of the
// contraction) x 256 columns k, turns the block through LDS (row pitch 80 bytes: both the 2-byte writes down a column
// and the 16-byte reads along a row spread over the banks) and writes sixteen 1 KiB pieces.
__global__ __launch_bounds__(256) void nf4_expand_tiled_transposed_kernel(const ExpandGroup eg, int K, int nk_total) {
  constexpr int kPitch = 80;
  __shared__ float2 lut[256];
  __shared__ __attribute__((aligned(16))) char sm[256 * kPitch];
  const int tid = threadIdx.x;
  lut[tid] = make_float2(round_to_bf16(kNF4Dense[tid >> 4]), round_to_bf16(kNF4Dense[tid & 15]));
  __syncthreads();
  int step = blockIdx.x;  // 32-row step of the member's contraction
  const ExpandMember& me = eg.m[expand_member(eg, step)];
  const uint8_t* __restrict__ codes = me.codes;
  const float* __restrict__ scal = me.scal;
  char* __restrict__ tiled = me.tiled;
  const int t_off = me.t_off;
  const int r = tid & 31, c = tid >> 5;
  const int n = 32 * step + r;
  const int kk0 = 256 * blockIdx.y + 32 * c;
  if (kk0 < K) {
    const u32x4_t cd = *reinterpret_cast<const u32x4_t*>(codes + (int64_t)n * (K >> 1) + (kk0 >> 1));
    const float sc = scal[(int64_t)n * (K >> 6) + (kk0 >> 6)];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t w = cd[d];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const float2 pr = lut[(w >> (8 * b)) & 0xffu];
        const uint32_t two = pack_bf16x2(pr.x * sc, pr.y * sc);
        const int j = 32 * c + 8 * d + 2 * b;
        *reinterpret_cast<uint16_t*>(sm + j * kPitch + 2 * r) = (uint16_t)two;
        *reinterpret_cast<uint16_t*>(sm + (j + 1) * kPitch + 2 * r) = (uint16_t)(two >> 16);
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = tid + 256 * i;
    const int Tl = idx >> 6, l = idx & 63;
    const int T = 16 * blockIdx.y + Tl;
    if (16 * T >= K) break;
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(sm + (16 * Tl + (l & 15)) * kPitch + 16 * (l >> 4));
    *reinterpret_cast<u32x4_t*>(tiled + ((int64_t)T * nk_total + t_off + step) * 1024 + l * 16) = v;
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// Per-group symmetric int4 fake quantisation of a bf16 weight [N, K] (FakeQuantizer.forward of the weight in
// FakeQuantizedLinear, torchao; same arithmetic, bit for bit, as fq_per_group_kernel in fake_quant.hip) written straight
// into the tiled layout the GEMM reads, for the forward (tiles of fq(W)) and / or the grad-input (tiles of fq(W)^T), so that
// the row-major fq(W) never exists.  A workgroup takes 32 rows x 256 columns; a thread 32 consecutive columns of one row
// (t = tid % 8, row = tid / 8), so the lanes of a group of up to 256 elements are neighbours.  Both outputs are staged in
// LDS in tile order and leave as 1 KiB pieces.
// ---------------------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fq_int4_sym_tiled_kernel(const uint16_t* __restrict__ w, int N, int K, int threads_per_group,
                                                                char* __restrict__ tiled_fwd, char* __restrict__ tiled_bwd,
                                                                float* __restrict__ scale_out, int groups_per_row, bool qp_bf16, float eps,
                                                                int bwd_nk_total, int bwd_t_off, int fwd_paired) {
  constexpr int kPieceF = 1040;  // forward staging: piece pitch, 16 bytes of padding spread the 16-byte writes over the banks
  constexpr int kPitchB = 80;    // backward staging: bytes per column k (32 rows x 2 bytes + padding)
  __shared__ __attribute__((aligned(16))) char smf[16 * kPieceF];
  __shared__ __attribute__((aligned(16))) char smb[256 * kPitchB];
  const int tid = threadIdx.x;
  const int t8 = tid & 7, r = tid >> 3;
  const int n = 32 * blockIdx.x + r;
  const int t = 8 * blockIdx.y + t8;  // 32-wide step along K
  const int nk = K >> 5;
  const bool live = t < nk;
  float v[32];
  if (live) {
    const u32x4_t* src = reinterpret_cast<const u32x4_t*>(w + (int64_t)n * K + 32 * t);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const u32x4_t raw = src[q];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        v[8 * q + 2 * d] = bits_f32(raw[d] << 16);
        v[8 * q + 2 * d + 1] = bits_f32(raw[d] & 0xffff0000u);
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < 32; ++e) v[e] = 0.f;
  }
  // a thread holds 32 elements; a group is 32, 64, 128 or 256 elements = 1, 2, 4 or 8 neighbouring threads of a row
  uint32_t o[16];
  {
    float mn = 0.f, mx = 0.f;
#pragma unroll
    for (int e = 0; e < 32; ++e) {
      mn = fminf(mn, v[e]);
      mx = fmaxf(mx, v[e]);
    }
    for (int off = 1; off < threads_per_group; off <<= 1) {
      mn = fminf(mn, __shfl_xor(mn, off, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, off, kWave));
    }
    const float amax = fmaxf(-mn, mx);
    float scale = amax / 7.5f;
    scale = scale > eps ? scale : eps;
    if (qp_bf16) scale = round_to_bf16(scale);  // the rounded scale quantises and dequantises
    const float inv = 1.0f / scale;
    if (live && scale_out && (t8 & (threads_per_group - 1)) == 0) scale_out[(int64_t)n * groups_per_row + t / threads_per_group] = scale;
#pragma unroll
    for (int e = 0; e < 32; e += 2) {
      float q2[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        float tq = __builtin_rintf(v[e + h] * inv);
        tq = tq < -8.0f ? -8.0f : (tq > 7.0f ? 7.0f : tq);
        q2[h] = (float)(int)tq;  // through the integer grid: rint(-0.3) = -0.0 must dequantise to +0.0
      }
      o[e >> 1] = pack_bf16x2(q2[0] * scale, q2[1] * scale);
    }
  }
  // ---- stage: forward piece t8 of row block r / 16, lane (r % 16) + 16 g4; backward column 32 t8 + j, row r
  if (tiled_fwd) {
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4)
      *reinterpret_cast<u32x4_t*>(smf + ((r >> 4) * 8 + t8) * kPieceF + (16 * g4 + (r & 15)) * 16) =
          u32x4_t{o[4 * g4], o[4 * g4 + 1], o[4 * g4 + 2], o[4 * g4 + 3]};
  }
  if (tiled_bwd) {
#pragma unroll
    for (int j = 0; j < 32; ++j)
      *reinterpret_cast<uint16_t*>(smb + (32 * t8 + j) * kPitchB + 2 * r) = (uint16_t)(o[j >> 1] >> (16 * (j & 1)));
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = tid + 256 * i;
    const int p = idx >> 6, l = idx & 63;  // 16 pieces of 64 lanes each
    if (tiled_fwd) {
      const int tp = 8 * blockIdx.y + (p & 7);
      if (tp < nk) {
        const u32x4_t val = *reinterpret_cast<const u32x4_t*>(smf + p * kPieceF + l * 16);
        const int T = 2 * blockIdx.x + (p >> 3);
        // paired: the forward tiles of two weights of equal shape alternate 8 blocks (128 columns) by 8 (see nf4_expand_tiled_kernel)
        const int To = fwd_paired ? ((T >> 3) << 4) + (T & 7) : T;
        *reinterpret_cast<u32x4_t*>(tiled_fwd + ((int64_t)To * nk + tp) * 1024 + l * 16) = val;
      }
    }
    if (tiled_bwd) {
      const int Tk = 16 * blockIdx.y + p;  // block of 16 columns k
      if (16 * Tk < K) {
        const u32x4_t val = *reinterpret_cast<const u32x4_t*>(smb + (16 * p + (l & 15)) * kPitchB + 16 * (l >> 4));
        // this weight's 32-row step blockIdx.x sits at step bwd_t_off + blockIdx.x of a contraction of bwd_nk_total steps
        *reinterpret_cast<u32x4_t*>(tiled_bwd + ((int64_t)Tk * bwd_nk_total + bwd_t_off + blockIdx.x) * 1024 + l * 16) = val;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------------
struct DenseSeg {
  const uint16_t* X;  // [M, Kc] bf16 activations of one segment of the contraction
  int Kc;
};
struct DenseAdapter {   // adds (lscale . lX) . lW^T to the output columns [n_begin, n_end)
  const uint16_t* lX;   // [M, R] bf16, rows ldlx apart
  const uint16_t* lW;   // [n_end - n_begin, R] (lw_row_major) or [R, n_end - n_begin] bf16
  int R, n_begin, n_end;
  float lscale;
};
struct DenseOut {          // output columns [n_begin, n_begin + width) go to their own tensor
  uint16_t* C;             // [M, width] bf16
  const uint16_t* bias;    // [width] bf16 or null
  const uint16_t* cscale;  // [width] bf16 or null: C = (acc + bias) * cscale per column
  int n_begin, width;
};
struct DenseArgs {
  DenseSeg seg[kGroupMax];
  DenseAdapter ad[kGroupMax];
  DenseOut out[kGroupMax];
  int nseg, nad, nout;
  const char* Wt;   // tiled weight: all output columns, all segments side by side along the contraction
  int M, Nout, Kc;  // Nout, Kc: totals
  int lw_row_major, ldlx;
  int tiles_m, tiles_n;
  // grad-input from the FORWARD tiles: Wt holds tiled[n / 16][k / 32][lane][8] of the weight W [Kc, Nout] (rows n = this
  // launch's contraction, columns k = its output columns) and the kernel transposes on its way out of LDS.  w_paired:
  // those tiles are the gated pair's (128 columns of the one member, then 128 of the other): the contraction then visits
  // the two segments alternately, 128 wide.
  int w_tr, w_paired;
  uint16_t* act;    // gated launches only: [M, out[0].width] bf16 = silu(out 0) * out 1
  int stream_members;  // gated launches only: out 0 and out 1 go out as streaming (non-temporal) stores
  // SwiGLU-backward launches only (one output): the result is the gradient of silu(gate) * up; out[0].C receives the
  // gradient of gate and sw_gup that of up, both [M, out[0].width] like gate and up themselves
  const uint16_t* sw_gate;
  const uint16_t* sw_up;
  uint16_t* sw_gup;
};

constexpr int kEpiPlain = 0, kEpiGated = 1, kEpiSwigluBwd = 2;
constexpr int kSegWalk = 0, kSegOne = 1, kSegPaired = 2, kSegHalves = 3;

// what the direct-to-LDS requests of the adapter's operands read for ranks beyond R
static __device__ __attribute__((aligned(16))) const uint32_t kZero16[4] = {0u, 0u, 0u, 0u};

constexpr int kAEntry = 32768;  // activation ring: 3 entries of 256 rows x 64 k
constexpr int kWBase = 3 * kAEntry;
constexpr int kWStage = 16384;  // weight ring: 4 stages of 256 columns x 32 k
constexpr int kLdsDense = kWBase + 4 * kWStage;

// GATED (forward of a gate / up pair, torchtune/modules/feed_forward.py:50-53): the two members' columns alternate in
// the tiled weight 128 by 128 (the paired layout of the expansion), so a tile holds columns [128 tile_n, + 128) of both:
// the waves with wn < 2 own the gate's, the others the up projection's.  Each wave writes its member's output as usual;
// the bf16 bands then meet in LDS and the workgroup also writes act = bf16(bf16(silu(gate)) * up), the arithmetic of
// ttamd_swiglu_fwd_bf16 on the rounded outputs, bit for bit.
// kEpiSwigluBwd (grad-input of the layer that follows the gated product, feed_forward.py:53): the result o = bf16(...)
// is the gradient of silu(gate) * up and is not stored; each 16-byte piece of it meets the same piece of gate and up
// on its way out and the launch writes the gradients of gate and up instead, the arithmetic of ttamd_swiglu_bwd_bf16 on
// the rounded result, bit for bit.
// W_TR (grad-input launches only): the weight operand comes from the tiles the forward launch of the same layer read.
// A stage then holds, for the 32 rows n of a step, the eight 1 KiB pieces that cover the tile's 256 columns k (row
// blocks 2 s and 2 s + 1, pieces 8 tile_n .. + 7 of each: 8 KiB contiguous per block), and a lane gathers its operand -
// 8 consecutive n of one column k - with two ds_read_b64_tr_b16, each of which hands lane i of a 16-lane group element
// i % 4 of the 8 bytes lane 4 t + i / 4 points at (t = 0..3).  Inside a piece the 16-byte chunk of (row n % 16 = p,
// k-group kg) sits in slot (p ^ 4 (kg & 1)) + 16 kg (applied on the global-address side of the direct-to-LDS loads), so
// that the 32 lanes served together touch 64 different banks.  Same products, same order of summation as the launch on
// tiles of W^T: the results are equal bit for bit.
// SEGS: how the contraction's activation segments are found - kSegOne: there is one (every forward launch; checked on the
// host); kSegPaired (W_TR only): two of equal width, visited 128 columns at a time, chosen by mask arithmetic on two base
// addresses held in scalar registers; kSegHalves: two of equal width one after the other (the gate / up pair's output
// gradients), the second base taken from the entry on where the first ends; kSegWalk: up to kGroupMax, walked as the
// requests move forward.  With all but the walk the main loop is one block with one backward branch; the walk costs two more taken branches per trip,
// which the single-segment launches on forward tiles paid with 5 % of their time while they shared its code.  (A
// branch-free table for the general case - every segment's first entry, base and pitch in scalar registers, selected
// per request - was 2 - 3 % slower than the walk: 30 more scalar instructions per trip in a loop that is bound by
// what a wave can issue.)
template <bool LW_ROW_MAJOR, int EPI, bool W_TR = false, int SEGS = LW_ROW_MAJOR ? kSegOne : kSegWalk>
__device__ __forceinline__ void gemm_dense_tile(const DenseArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr bool GATED = EPI == kEpiGated;
  constexpr int MT = 8, NT = 4;  // 16 x 16 MFMA tiles per wave
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wv >> 2, wn = wv & 3;
  const int l15 = lane & 15, g4 = lane >> 4;

  int tile_m, tile_n;
  {
    // workgroup ids are dealt round-robin to the 8 XCDs (one L2 each): every XCD gets a band of m-tiles and walks it
    // column by column, so the workgroups resident on an XCD share each weight tile through its L2
    const int id = blockIdx.x;
    const int bands4 = g.tiles_m >> 2;  // bands of four m-tiles
    if ((g.tiles_m == 4 || g.tiles_m == 8 || g.tiles_m == 16) && g.tiles_n % (8 / bands4) == 0) {
      // Fewer than 32 m-tiles: a band of tiles_m / 8 rows per XCD would put 2 x 16 (or 1 x 32) tiles on an XCD at a time,
      // 2 activation panels + 16 weight panels through its L2 per round.  8 / bands4 XCDs share a band of four rows
      // instead and take turns at the columns in runs of up to eight: 4 x 8 tiles at a time, 4 + 8 panels (4096 tokens
      // of the 70B shape: GEMM time of the step -1.5 %; with runs of one column -0.6 %: neighbouring columns of the
      // forward tiles that a grad-input launch reads lie next to each other in memory).
      const int xcd = id & 7, slot = id >> 3, share = 8 / bands4, cb = slot >> 2;
      int run = 8;
      while (g.tiles_n % (run * share) != 0) run >>= 1;  // tiles_n % share == 0: ends at 1 at the latest
      tile_m = 4 * (xcd % bands4) + (slot & 3);
      tile_n = (cb / run) * (run * share) + (xcd / bands4) * run + cb % run;
    } else if ((g.tiles_m & 7) == 0) {
      const int xcd = id & 7, slot = id >> 3, band = g.tiles_m >> 3;
      tile_m = xcd * band + slot % band;
      tile_n = slot / band;
    } else {
      tile_m = id / g.tiles_n;
      tile_n = id % g.tiles_n;
    }
  }
  const int m0 = tile_m * 256, n0 = tile_n * 256;
  const int nk = g.Kc >> 5;        // k-steps of 32
  const int nk2 = g.Kc >> 6;       // activation entries (pairs of k-steps)

  // ---- loads.  Activations: every two k-steps, four instructions per wave (rows [32 wv, +32) of the tile, 8 rows of 128
  //      bytes each: whole cache lines); chunk c of row r is stored in slot c ^ ((r >> 1) & 7).  Weights: every k-step the
  //      1 KiB pieces of column blocks 2 wv and 2 wv + 1.
  int a_row[4], a_chunk[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int trow = wv * 32 + 8 * i + (lane >> 3);
    a_chunk[i] = ((lane & 7) ^ ((trow >> 1) & 7)) * 16;
    const int row = m0 + trow;
    a_row[i] = row < g.M ? row : g.M - 1;
  }
  // segment q: entries [seg_first[q], seg_first[q + 1]) of the contraction, rows seg_pitch[q] bytes apart (absent ones
  // begin beyond every entry)
  // The four requests of an entry (and the two of a weight step) name their LDS destinations through the instruction's
  // offset field, which moves the global address along with the LDS address: one M0 write per entry / step instead of
  // one per request.  Request i therefore carries offset 1024 i and a lane offset that is 1024 i short, all of them
  // lifted by kAShift so that none is negative, against a base lowered by as much.
  constexpr int kAShift = 3072;
  uint32_t a_off[4];
  int seg = 0, seg_begin = 0, seg_end = g.seg[0].Kc >> 6;  // kSegWalk: entries [seg_begin, seg_end) belong to segment seg
  const char* a_base = reinterpret_cast<const char*>(g.seg[0].X) - kAShift;
  auto set_segment = [&]() {
    const uint32_t pitch = (uint32_t)g.seg[seg].Kc * 2u;
#pragma unroll
    for (int i = 0; i < 4; ++i) a_off[i] = (uint32_t)a_row[i] * pitch + (uint32_t)a_chunk[i] + (uint32_t)(kAShift - 1024 * i);
  };
  set_segment();
  // kSegPaired: the two bases as integers (a select among pointers read from the argument struct becomes an indexed load
  // inside the loop, and the wait for it drains the ring's requests)
  const int64_t pair_base0 = (int64_t)(uintptr_t)g.seg[0].X - kAShift, pair_base1 = (int64_t)(uintptr_t)g.seg[SEGS == kSegPaired || SEGS == kSegHalves ? 1 : 0].X - kAShift;
  // kSegHalves: what the second segment's entries add to an address counted from the first segment's base
  const int half_entries = g.seg[0].Kc >> 6;
  const int64_t half_jump = pair_base1 - pair_base0 - ((int64_t)half_entries << 7);
  const int nblocks = g.Nout >> 4;
  const char* wsrc0;
  const char* wsrc1;
  int64_t wstep;  // bytes from one k-step's pieces to the next
  uint32_t lane16;
  if constexpr (W_TR) {
    const int npieces = g.Nout >> 5;  // 32-wide pieces along the weight's columns k
    int p0 = 8 * tile_n + 2 * (wv & 3), p1 = p0 + 1;
    p0 = p0 < npieces ? p0 : npieces - 1;
    p1 = p1 < npieces ? p1 : npieces - 1;
    const int64_t blk = (int64_t)(wv >> 2) * npieces;  // row block 2 s + (wv >> 2) of step s
    wsrc0 = g.Wt + (blk + p0) * 1024;
    wsrc1 = g.Wt + (blk + p1) * 1024;
    wstep = (int64_t)npieces * 2048;
    lane16 = (uint32_t)(((lane & 15) ^ (((lane >> 4) & 1) << 2)) | (lane & 48)) * 16u;
  } else {
    int T0 = (n0 >> 4) + 2 * wv, T1 = T0 + 1;
    T0 = T0 < nblocks ? T0 : nblocks - 1;
    T1 = T1 < nblocks ? T1 : nblocks - 1;
    wsrc0 = g.Wt + (int64_t)T0 * ((int64_t)nk * 1024);
    wsrc1 = g.Wt + (int64_t)T1 * ((int64_t)nk * 1024);
    wstep = 1024;
    lane16 = (uint32_t)lane * 16u;
  }

  // the two requests of a weight step: one base (the first piece's, lowered by 1024) and the second piece's distance in
  // the lane offset
  const char* const wbase = wsrc0 - 1024;
  const uint32_t w_voff0 = lane16 + 1024u, w_voff1 = lane16 + (uint32_t)(wsrc1 - wsrc0);
  const uint32_t lds0 = (uint32_t)(uintptr_t)TT_LDS_PTR(smem);
  // inside: the caller knows that the step / entry exists (no clamp: the address is then a constant distance from the
  // loop's counter, which the compiler carries as a running pointer)
  auto issue_w = [&](int t, int stage, bool inside = false) {
    const int tk = inside || t < nk ? t : nk - 1;
    const uint32_t sw = lds0 + kWBase + stage * kWStage + wv * 2048;
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, %2\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:1024"
                 ::"v"(w_voff0), "v"(w_voff1), "s"(wbase + (int64_t)tk * wstep), "s"(sw) : "memory", "m0");
  };
  auto issue_a = [&](int T2, int entry, bool inside = false) {
    const int tk = inside || T2 < nk2 ? T2 : nk2 - 1;
    const char* xb;
    if constexpr (SEGS == kSegOne) {
      xb = a_base + ((int64_t)tk << 7);  // + 64 elements * 2 bytes per entry
    } else if constexpr (SEGS == kSegPaired) {
      // two segments of equal width, visited 128 columns (two entries) at a time: entry tk is entry
      // 2 (tk / 4) + tk % 2 of segment (tk / 2) % 2; the row pitch is the same for both
      const int64_t second = -(int64_t)((tk >> 1) & 1);
      xb = reinterpret_cast<const char*>((uintptr_t)((pair_base0 ^ ((pair_base0 ^ pair_base1) & second)) +
                                                     ((int64_t)(((tk >> 2) << 1) + (tk & 1)) << 7)));
    } else if constexpr (SEGS == kSegHalves) {
      xb = reinterpret_cast<const char*>((uintptr_t)(pair_base0 + ((int64_t)tk << 7) + (half_jump & -(int64_t)(tk >= half_entries))));
    } else {
      // entries are requested in increasing order (past the end: the last one again), so the segment only moves forward
      while (tk >= seg_end) {
        ++seg;
        seg_begin = seg_end;
        seg_end += g.seg[seg].Kc >> 6;
        a_base = reinterpret_cast<const char*>(g.seg[seg].X) - kAShift;
        set_segment();
      }
      xb = a_base + ((int64_t)(tk - seg_begin) << 7);
    }
    const uint32_t sa = lds0 + entry * kAEntry + wv * 4096;
    asm volatile("s_mov_b32 m0, %5\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, %4\n\t"
                 "global_load_lds_dwordx4 %1, %4 offset:1024\n\t"
                 "global_load_lds_dwordx4 %2, %4 offset:2048\n\t"
                 "global_load_lds_dwordx4 %3, %4 offset:3072"
                 ::"v"(a_off[0]), "v"(a_off[1]), "v"(a_off[2]), "v"(a_off[3]), "s"(xb), "s"(sa) : "memory", "m0");
  };

  // ---- forward launches: the adapter's operands travel through the same rings as further k-steps of the contraction.
  //      The loop's last trips request past the end of the weight (the waits count a fixed number of requests in flight,
  //      so the requests keep coming); in a forward launch with an adapter those requests fetch the adapter instead:
  //      16 bytes (8 ranks of one row of lX / one row of lW) per lane, zeros beyond R, so that by the end of the loop the
  //      operands sit in LDS in the loop's own layout and the adapter costs one more k-step per 32 ranks instead of a trip
  //      to memory.  Ranks of at most 32 (ad_compact) need activation entry nk2 and weight step nk only: the entry's first
  //      half holds the 32 ranks of lX (GATED: of the gate's lX, and the second half those of the up projection's), the
  //      step the ranks of lW for the tile's 256 columns; nothing is requested in the loop's last trip then, and nothing
  //      is in flight when the loop ends.  Otherwise entry nk2 holds 64 ranks (GATED: the gate's, and entry nk2 + 1 the up
  //      projection's) and steps nk, nk + 1 ranks [0, 32) and [32, 64).
  bool ad_rings = false;  // uniform over the workgroup
  bool ad_compact = false;
  // the tile's adapter ([0]; GATED: the two members'), read once and held in scalar registers: R = 0 where there is none
  int ad_R[2] = {0, 0}, ad_ncols[2] = {0, 0};
  const uint16_t* ad_lX[2] = {nullptr, nullptr};
  const uint16_t* ad_lW[2] = {nullptr, nullptr};
  float ad_lscale[2] = {1.0f, 1.0f};
  int ad_col0 = 0;  // first column of the tile among the adapter's columns
  const char* const zero_src = reinterpret_cast<const char*>(kZero16);
  auto ad_src_a = [&](int q, int i) -> const char* {  // what request i of entry nk2 + q reads
    const int c = a_chunk[i] >> 4;                    // 16-byte chunk of the entry's row: 8 ranks
    int a, r0;                                        // member and first rank this chunk holds
    if (GATED) {
      a = ad_compact ? c >> 2 : q;
      r0 = ad_compact ? 8 * (c & 3) : 8 * c;
    } else {
      a = 0;
      r0 = q == 0 ? 8 * c : 64;
    }
    const uint16_t* lX = a ? ad_lX[1] : ad_lX[0];
    return r0 < (a ? ad_R[1] : ad_R[0]) ? reinterpret_cast<const char*>(lX + (int64_t)a_row[i] * g.ldlx + r0) : zero_src;
  };
  auto ad_src_w = [&](int step, int b) -> const char* {  // what request b of step nk + step reads
    const int a = GATED ? wm : 0;                        // GATED: column blocks 2 wv, 2 wv + 1 are the gate's for wv < 4
    const int R = a ? ad_R[1] : ad_R[0], ncols = a ? ad_ncols[1] : ad_ncols[0];
    const uint16_t* lW = a ? ad_lW[1] : ad_lW[0];
    const int r0 = 32 * step + 8 * g4;
    int col = ad_col0 + 16 * (GATED ? (2 * wv + b) & 7 : 2 * wv + b) + l15;
    col = col < ncols ? col : ncols - 1;
    return r0 < R ? reinterpret_cast<const char*>(lW + (int64_t)col * R + r0) : zero_src;
  };
  // per-lane sources of entry nk2 and step nk, worked out while the prologue's requests are on their way
  const char* ad_a0[4] = {zero_src, zero_src, zero_src, zero_src};
  const char* ad_w0[2] = {zero_src, zero_src};
  auto ad_setup = [&]() {
    if constexpr (LW_ROW_MAJOR) {
      auto take = [&](int slot, int aidx) {
        ad_R[slot] = g.ad[aidx].R;
        ad_ncols[slot] = g.ad[aidx].n_end - g.ad[aidx].n_begin;
        ad_lX[slot] = g.ad[aidx].lX;
        ad_lW[slot] = g.ad[aidx].lW;
        ad_lscale[slot] = g.ad[aidx].lscale;
      };
      if constexpr (GATED) {
        if (g.nad > 0 && g.ad[0].R > 0) take(0, 0);
        if (g.nad > 1 && g.ad[1].R > 0) take(1, 1);
        ad_col0 = 128 * tile_n;
      } else {
        int ad_idx = -1;
        for (int aidx = 0; aidx < g.nad; ++aidx)
          if (g.ad[aidx].R > 0 && n0 >= g.ad[aidx].n_begin && n0 < g.ad[aidx].n_end) ad_idx = aidx;
        ad_idx = __builtin_amdgcn_readfirstlane(ad_idx);  // the same in every lane: the fields come through scalar loads
        if (ad_idx >= 0) {
          take(0, ad_idx);
          ad_col0 = n0 - g.ad[ad_idx].n_begin;
        }
      }
      ad_rings = ad_R[0] > 0 || ad_R[1] > 0;
      ad_compact = ad_R[0] <= 32 && ad_R[1] <= 32;
      if (ad_rings) {
#pragma unroll
        for (int i = 0; i < 4; ++i) ad_a0[i] = ad_src_a(0, i);
#pragma unroll
        for (int b = 0; b < 2; ++b) ad_w0[b] = ad_src_w(0, b);
      }
    }
  };
  auto dma16v = [&](const char* src, uint32_t lds, int imm) {
    asm volatile("s_add_u32 m0, %1, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 ::"v"(src), "s"(lds), "n"(imm) : "memory", "m0", "scc");
  };
  auto issue_a_ad = [&](int q, int entry) {  // q = 0: entry nk2, 1: entry nk2 + 1
    const uint32_t sa = lds0 + entry * kAEntry + wv * 4096;
    dma16v(q == 0 ? ad_a0[0] : ad_src_a(1, 0), sa, 0);
    dma16v(q == 0 ? ad_a0[1] : ad_src_a(1, 1), sa, 1024);
    dma16v(q == 0 ? ad_a0[2] : ad_src_a(1, 2), sa, 2048);
    dma16v(q == 0 ? ad_a0[3] : ad_src_a(1, 3), sa, 3072);
  };
  auto issue_w_ad = [&](int step, int stage) {  // step = 0: ranks [0, 32), 1: ranks [32, 64)
    const uint32_t sw = lds0 + kWBase + stage * kWStage + wv * 2048;
    dma16v(step == 0 ? ad_w0[0] : ad_src_w(1, 0), sw, 0);
    dma16v(step == 0 ? ad_w0[1] : ad_src_w(1, 1), sw, 1024);
  };

  // operand read offsets: activation tile 0 of this wave, half hf of the entry: row 128 wm + l15, chunk 4 hf + g4
  int xo[2];
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) xo[hf] = (128 * wm + l15) * 128 + (((4 * hf + g4) ^ ((l15 >> 1) & 7)) << 4);
  const int wo = kWBase + (4 * wn) * 1024 + lane * 16;  // weight block 4 wn + j at + j * 1024

  f32x4_t acc[NT][MT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[j][i][v] = 0.f;

  // W_TR: lane (l15, g4) of a transposing read points at row n = 8 g4 + l15 / 4 (+ 4 for the second half) of the step,
  // columns 4 (l15 % 4) .. + 3 of the wave's block j: piece 2 wn + j / 2 of row block g4 / 2, k-group 2 (j % 2) + (l15 % 4) / 2
  int wtr[2] = {0, 0};
  if constexpr (W_TR) {
    const int c = l15 & 3, kg1 = c >> 1;
    const int np = 8 * (g4 & 1) + (l15 >> 2);
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
      wtr[h2] = kWBase + (g4 >> 1) * 8192 + 2 * wn * 1024 + 256 * kg1 + (((np + 4 * h2) ^ (4 * kg1)) << 4) + 8 * (c & 1);
  }
  bf16x8_t xf[MT], wf[NT];
  auto read_step = [&](int entry, int hf, int wstage) {
    const char* sw = smem + wstage * kWStage;
    const char* sa = smem + entry * kAEntry + xo[hf];
    if constexpr (W_TR) {
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        typedef short s16x4_t __attribute__((ext_vector_type(4)));
        typedef short s16x8_t __attribute__((ext_vector_type(8)));
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(sw + wtr[0] + j * 512));
        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(sw + wtr[1] + j * 512));
        const s16x8_t both = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        wf[j] = __builtin_bit_cast(bf16x8_t, both);
      }
    } else {
#pragma unroll
      for (int j = 0; j < NT; ++j) wf[j] = *reinterpret_cast<const bf16x8_t*>(sw + wo + j * 1024);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) xf[i] = *reinterpret_cast<const bf16x8_t*>(sa + i * 2048);
  };
  auto compute = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < MT; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j], xf[i], acc[j][i], 0, 0, 0);
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- pipeline.  Every wave alternates memory part M(t) / barrier / compute part C(t) / barrier; the waves with
  //      wm = 1 pass one extra barrier first, so that between two barriers one wave of each SIMD computes while the other
  //      is in its memory part.  Numbering the barriers from the one that ends the prologue, the waves with wm = 0 read
  //      step t between barriers 2t and 2t+1, the others between 2t+1 and 2t+2.  Hence:
  //        * what M(t) requests may overwrite the stage of step t-1 (last read before barrier 2t): W(t+3) into a ring of
  //          four stages, and for even t activation entry t/2 + 2 into a ring of three;
  //        * at the end of M(t) a wave's own loads of step t+1 must have landed (the other waves read them after the
  //          next barrier).  Loads of a wave complete in order.  Its program order: prologue A(0) x4, W(0) x2, W(1) x2,
  //          A(1) x4, W(2) x2; M(t): W(t+3) x2, then for even t A(t/2 + 2) x4.  W(t+1) came from M(t-2) and the
  //          activation entry of step t+1 is older; newer than W(t+1) are 4 + 2 + 6 = 12 loads (t even), 0 + 6 + 2 = 8 (t odd).
  //      The operand reads of M(t) are awaited by the compiler's own counts before the first MFMA that needs them, after
  //      the barrier: the other wave's MFMAs are still draining then.  The waves with wm = 1 are the exception: what they
  //      read in one interval is overwritten by requests the waves with wm = 0 issue right after the next barrier, so
  //      they let their reads complete before they pass it (the others' reads have a whole interval more).
  issue_a(0, 0);
  issue_w(0, 0);
  issue_w(1, 1);
  if (LW_ROW_MAJOR && nk == 2) {  // a contraction of 64: the prologue already reaches past the weight
    ad_setup();
    if (ad_rings) {
      issue_a_ad(0, 1);
      issue_w_ad(0, 2);
    } else {
      issue_a(1, 1);
      issue_w(2, 2);
    }
  } else {
    issue_a(1, 1);
    issue_w(2, 2);
    ad_setup();
  }
  asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");  // A(0), W(0) landed everywhere
  if (wm == 1) asm volatile("s_barrier" ::: "memory");
  // one copy of the loop per wave group: the two differ in one wait, and a branch per step costs 2 - 4 %
  auto main_loop = [&](auto lgkm) {
    constexpr bool kLgkm = decltype(lgkm)::value;
    int e0_running = 0;  // activation entry of the current pair of steps; the weight stage of step t is t % 4
    // The last two trips, whose requests reach past the weight, are copies of the loop that ask for the adapter's
    // operands instead (ad_rings; no trip of the first copy pays for the choice).  kTrip 1 (t = nk - 4) requests entry
    // nk2 and step nk where the others request the activations and the weight; kTrip 2 (t = nk - 2) requests step nk + 1,
    // entry nk2 + 1 and step nk + 1 again (the count of requests in flight stays what the waits assume) - or nothing
    // (ad_compact), and then waits by the counts of that case: newer than W(nk - 1) are A x4 and W(nk) x2, and by the end
    // of the last step everything has landed.
    // kWs: the weight stage of the trip's even step where the caller knows it (the loop below takes two trips at a time,
    // so that stage offsets are constants of the instructions: no arithmetic on them in the loop), -1: t % 4
    // kE0: the activation entry of the trip where the caller knows it, -1: the running one.  Both known: every LDS offset
    // of the trip is a constant of its instructions, and none of its requests reaches past the weight.
    auto pair = [&](int t, auto trip, auto stage, auto entry) {
      constexpr int kTrip = decltype(trip)::value;
      constexpr int kWs = decltype(stage)::value;
      constexpr int kE0 = decltype(entry)::value;
      constexpr bool kInside = kE0 >= 0;
      const int ws = kWs >= 0 ? kWs : (t & 3);
      const bool nothing = kTrip == 2 && ad_compact;
      const int e0 = kE0 >= 0 ? kE0 : e0_running;
      const int e1 = e0 == 2 ? 0 : e0 + 1, e2 = e1 == 2 ? 0 : e1 + 1;
      // ---- even step t
      if constexpr (kTrip == 2) {
        if (!nothing) {
          issue_w_ad(1, (ws + 3) & 3);
          issue_a_ad(1, e2);
        }
      } else {
        issue_w(t + 3, (ws + 3) & 3, kInside);
        if constexpr (kTrip == 1)
          issue_a_ad(0, e2);
        else
          issue_a((t >> 1) + 2, e2, kInside);
      }
      read_step(e0, 0, ws);
      __builtin_amdgcn_sched_barrier(0);
      if (nothing) {
        if constexpr (kLgkm)
          asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else
          asm volatile("s_waitcnt vmcnt(6)\n\ts_barrier" ::: "memory");
      } else {
        if constexpr (kLgkm)
          asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else
          asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");
      }
      compute();
      // ---- odd step t + 1
      if constexpr (kTrip == 0)
        issue_w(t + 4, ws, kInside);
      else if constexpr (kTrip == 1)
        issue_w_ad(0, ws);
      else if (!nothing)
        issue_w_ad(1, ws);
      read_step(e0, 1, (ws + 1) & 3);
      __builtin_amdgcn_sched_barrier(0);
      if (nothing) {
        if constexpr (kLgkm)
          asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else
          asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
      } else {
        if constexpr (kLgkm)
          asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else
          asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
      }
      compute();
      e0_running = e1;
    };
    using C0 = std::integral_constant<int, 0>;
    using C1 = std::integral_constant<int, 1>;
    using C2 = std::integral_constant<int, 2>;
    using Cr = std::integral_constant<int, -1>;
    const int t_tail = ad_rings ? nk - 4 : nk;
    if constexpr (SEGS == kSegWalk) {  // the walk's state on top of several trips' worth of code does not fit the registers
      for (int t = 0; t < t_tail; t += 2) pair(t, C0{}, Cr{}, Cr{});
    } else {
      // six trips at a time (the weight ring repeats every two, the activation ring every three), as long as all of
      // their requests stay inside the weight; the rest one by one with running indices and clamped requests
      int t = 0;
      for (; t + 12 <= t_tail && t + 16 <= nk; t += 12) {
        pair(t, C0{}, C0{}, C0{});
        pair(t + 2, C0{}, C2{}, C1{});
        pair(t + 4, C0{}, C0{}, C2{});
        pair(t + 6, C0{}, C2{}, C0{});
        pair(t + 8, C0{}, C0{}, C1{});
        pair(t + 10, C0{}, C2{}, C2{});
      }
      for (; t < t_tail; t += 2) pair(t, C0{}, Cr{}, Cr{});
    }
    if constexpr (LW_ROW_MAJOR) {
      if (ad_rings) {
        if (nk >= 4) pair(nk - 4, C1{}, Cr{}, Cr{});
        pair(nk - 2, C2{}, Cr{}, Cr{});
      }
    }
  };
  if (wm == 1)
    main_loop(std::true_type{});
  else
    main_loop(std::false_type{});
  if (wm == 0) asm volatile("s_barrier" ::: "memory");
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the clamped requests of the last steps

  // the adapter's scale goes onto the activation side, bf16(lscale * lX), as in the fused kernel; a power of two is
  // exact on either operand, and the weight side has half as many registers to scale
  auto scaled = [&](u32x4_t raw, float lscale) {
#pragma unroll
    for (int d = 0; d < 4; ++d)
      raw[d] = pack_bf16x2(bits_f32(raw[d] << 16) * lscale, bits_f32(raw[d] & 0xffff0000u) * lscale);
    return raw;
  };
  // ---- adapters from the rings (see issue_a_ad): steps nk, nk + 1 of the loop with the scale on one operand
  if (ad_rings) {
    __syncthreads();  // every wave's requests have landed
    const int a = GATED ? (wn >> 1) : 0;
    const int R = a ? ad_R[1] : ad_R[0];
    const float lscale = a ? ad_lscale[1] : ad_lscale[0];
    const bool on_w = (f32_bits(lscale) & 0x007fffffu) == 0;
    const int entry = (nk2 + (GATED && !ad_compact ? a : 0)) % 3;
    for (int step = 0; 32 * step < R; ++step) {
      read_step(entry, GATED && ad_compact ? a : step, (nk + step) & 3);
      bf16x8_t wfr[NT], xfr[MT];
#pragma unroll
      for (int j = 0; j < NT; ++j)
        wfr[j] = lscale != 1.0f && on_w ? __builtin_bit_cast(bf16x8_t, scaled(__builtin_bit_cast(u32x4_t, wf[j]), lscale)) : wf[j];
#pragma unroll
      for (int i = 0; i < MT; ++i)
        xfr[i] = lscale != 1.0f && !on_w ? __builtin_bit_cast(bf16x8_t, scaled(__builtin_bit_cast(u32x4_t, xf[i]), lscale)) : xf[i];
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wfr[j], xfr[i], acc[j][i], 0, 0, 0);
    }
  }

  // ---- adapters of the grad-input launches, whose lW lies the other way: one MFMA
  //      step per 32 ranks and segment, operands straight from global memory.  Lane (l15, g4) holds
  //      ranks rc + 8 g4 .. + 7 of weight column / activation row l15 of its tile; ranks beyond R are zero.
  for (int aidx = 0; aidx < (LW_ROW_MAJOR ? 0 : g.nad); ++aidx) {
    const int R = g.ad[aidx].R;
    const int nb = g.ad[aidx].n_begin, ncols = g.ad[aidx].n_end - nb;
    if constexpr (GATED) {
      if (R <= 0 || aidx != (wn >> 1)) continue;  // adapter i belongs to member i; uniform over the wave, no barrier below
    } else {
      if (R <= 0 || n0 < nb || n0 >= nb + ncols) continue;  // the same for every wave of the workgroup
    }
    const uint16_t* lX = g.ad[aidx].lX;
    const uint16_t* lW = g.ad[aidx].lW;
    const float lscale = g.ad[aidx].lscale;
    // first column of the tile among the adapter's columns (GATED: such that + 64 wn lands on the wave's own columns)
    const int nl0 = GATED ? 128 * tile_n - 128 * (wn >> 1) : n0 - nb;
    // Every request of a 32-rank step is issued before the first use of any of them: one trip to memory per step instead
    // of one per operand (with the scaling between two loads the compiler waited for each load in turn, ~5 us a tile).
    u32x4_t xraw[MT], wraw[NT];
    auto load_x = [&](int rc) {
      const int r0 = rc + 8 * g4;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        int row = m0 + 128 * wm + 16 * i + l15;
        row = row < g.M ? row : g.M - 1;
        xraw[i] = u32x4_t{0, 0, 0, 0};
        if (r0 < R) xraw[i] = *reinterpret_cast<const u32x4_t*>(lX + (int64_t)row * g.ldlx + r0);  // R % 8 == 0: 8 ranks all in or all out
      }
    };
    load_x(0);
    int pitch = 0;  // bytes per column of the staged adapter weights
    if constexpr (!LW_ROW_MAJOR) {
      // lW is [R, Nout]: a lane needs 8 ranks of one column, 8 elements Nout apart.  The workgroup copies the 256
      // columns of its tile into LDS column by column (the rings are free after the loop), 16 bytes of a rank row per
      // thread, and every lane then reads its operand as one 16-byte piece.
      pitch = (R + 8) * 2;
      __syncthreads();
      for (int idx = tid; idx < R * 32; idx += 512) {
        const int r = idx >> 5, c8 = (idx & 31) * 8;
        u32x4_t raw = {0, 0, 0, 0};
        if (nl0 + c8 < ncols) raw = *reinterpret_cast<const u32x4_t*>(lW + (int64_t)r * ncols + nl0 + c8);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          *reinterpret_cast<uint16_t*>(smem + (c8 + e) * pitch + 2 * r) = (uint16_t)(raw[e >> 1] >> (16 * (e & 1)));
      }
      __syncthreads();
    }
    for (int rc = 0; rc < R; rc += 32) {
      const int r0 = rc + 8 * g4;
      const bool in = r0 < R;
      if (rc > 0) load_x(rc);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        wraw[j] = u32x4_t{0, 0, 0, 0};
        if (in) {
          if constexpr (LW_ROW_MAJOR) {
            int col = nl0 + wn * 64 + 16 * j + l15;
            col = col < ncols ? col : ncols - 1;
            wraw[j] = *reinterpret_cast<const u32x4_t*>(lW + (int64_t)col * R + r0);
          } else {
            wraw[j] = *reinterpret_cast<const u32x4_t*>(smem + (wn * 64 + 16 * j + l15) * pitch + 2 * r0);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      bf16x8_t wfr[NT], xfr[MT];
      const bool on_w = (f32_bits(lscale) & 0x007fffffu) == 0;
#pragma unroll
      for (int j = 0; j < NT; ++j) wfr[j] = __builtin_bit_cast(bf16x8_t, lscale != 1.0f && on_w ? scaled(wraw[j], lscale) : wraw[j]);
#pragma unroll
      for (int i = 0; i < MT; ++i) xfr[i] = __builtin_bit_cast(bf16x8_t, lscale != 1.0f && !on_w ? scaled(xraw[i], lscale) : xraw[i]);
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wfr[j], xfr[i], acc[j][i], 0, 0, 0);
    }
  }

  // ---- epilogue: acc[j][i][v] = C[m][n], m = m0 + 128 wm + 16 i + l15, n = n0 + 64 wn + 16 j + 4 g4 + v.  Each wave
  //      transposes its 128 x 64 band through LDS (the rings are free now) and writes whole 128-byte row segments;
  //      16-byte chunk c of row r sits in slot c ^ (r & 7).
  __syncthreads();
  int oi = 0;
  if constexpr (GATED) {
    oi = wn >> 1;
  } else {
    while (oi + 1 < g.nout && n0 >= g.out[oi + 1].n_begin) ++oi;
  }
  // first column of this wave's band in its output tensor
  const int nlo = GATED ? 128 * tile_n + 64 * (wn & 1) : n0 - g.out[oi].n_begin + wn * 64;
  const int width = g.out[oi].width;
  if constexpr (!GATED) {
    if (nlo >= width) return;  // the whole band of this wave lies outside (no barrier follows)
  }
  {
    const uint16_t* bias = g.out[oi].bias;
    const uint16_t* cscale = g.out[oi].cscale;
    char* band = smem + wv * 16384;  // 128 rows x 128 bytes
    // SwiGLU backward: the pieces of gate and up that meet rows [64 half, + 64) of the band; those of the first half are
    // asked for before the band is staged, the others right after.  Rows beyond M read row M - 1 and are not stored.
    u32x4_t sw_g[EPI == kEpiSwigluBwd ? 16 : 1], sw_u[EPI == kEpiSwigluBwd ? 16 : 1];
    const int64_t sw_col = nlo + 8 * (lane & 7);
    auto sw_fetch = [&](int half) {
#pragma unroll
      for (int t = 0; t < (EPI == kEpiSwigluBwd ? 8 : 0); ++t) {
        const int row = m0 + 128 * wm + 64 * half + 8 * t + (lane >> 3);
        const int64_t at = (int64_t)(row < g.M ? row : g.M - 1) * width + sw_col;
        sw_g[8 * half + t] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(g.sw_gate + at));
        sw_u[8 * half + t] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(g.sw_up + at));
      }
    };
    if constexpr (EPI == kEpiSwigluBwd) sw_fetch(0);
    if (!bias && !cscale) {
      // nothing to add or scale: two conversions per four values instead of ten operations
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const int r = 16 * i + l15;
          u32x2_t o;
          o.x = pack_bf16x2(acc[j][i][0], acc[j][i][1]);
          o.y = pack_bf16x2(acc[j][i][2], acc[j][i][3]);
          *reinterpret_cast<u32x2_t*>(band + r * 128 + (((2 * j + (g4 >> 1)) ^ (r & 7)) << 4) + 8 * (g4 & 1)) = o;
        }
    } else
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      float b4[4] = {0.f, 0.f, 0.f, 0.f};
      if (bias) {
        const u32x2_t bb = *reinterpret_cast<const u32x2_t*>(bias + nlo + 16 * j + 4 * g4);
        b4[0] = bits_f32(bb.x << 16); b4[1] = bits_f32(bb.x & 0xffff0000u);
        b4[2] = bits_f32(bb.y << 16); b4[3] = bits_f32(bb.y & 0xffff0000u);
      }
      float c4[4] = {1.f, 1.f, 1.f, 1.f};
      if (cscale) {
        const u32x2_t cc = *reinterpret_cast<const u32x2_t*>(cscale + nlo + 16 * j + 4 * g4);
        c4[0] = bits_f32(cc.x << 16); c4[1] = bits_f32(cc.x & 0xffff0000u);
        c4[2] = bits_f32(cc.y << 16); c4[3] = bits_f32(cc.y & 0xffff0000u);
      }
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int r = 16 * i + l15;
        u32x2_t o;
        o.x = pack_bf16x2((acc[j][i][0] + b4[0]) * c4[0], (acc[j][i][1] + b4[1]) * c4[1]);
        o.y = pack_bf16x2((acc[j][i][2] + b4[2]) * c4[2], (acc[j][i][3] + b4[3]) * c4[3]);
        *reinterpret_cast<u32x2_t*>(band + r * 128 + (((2 * j + (g4 >> 1)) ^ (r & 7)) << 4) + 8 * (g4 & 1)) = o;
      }
    }
    if constexpr (GATED) {
      __syncthreads();  // the gate's and the up projection's bands are read across waves below (widths are multiples of 128: every wave is here)
    } else {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    const int c = lane & 7;
    uint16_t* crow = g.out[oi].C + nlo + 8 * c;
    const int mrow0 = m0 + 128 * wm;
    if constexpr (EPI == kEpiSwigluBwd) {
      sw_fetch(1);
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        const int r = 8 * t + (lane >> 3);
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(band + r * 128 + ((c ^ (r & 7)) << 4));
        u32x4_t og, ou;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          uint32_t dg, du;
          swiglu_bwd_pair(v[d], sw_g[t][d], sw_u[t][d], dg, du);
          og[d] = dg;
          ou[d] = du;
        }
        if (mrow0 + r < g.M) {
          const int64_t at = (int64_t)(mrow0 + r) * width + sw_col;
          *reinterpret_cast<u32x4_t*>(g.out[oi].C + at) = og;
          *reinterpret_cast<u32x4_t*>(g.sw_gup + at) = ou;
        }
      }
      return;
    }
    auto store_band = [&](auto streaming) {
#pragma unroll 8
      for (int t = 0; t < 16; ++t) {
        const int r = 8 * t + (lane >> 3);
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(band + r * 128 + ((c ^ (r & 7)) << 4));
        if (mrow0 + r < g.M) {
          u32x4_t* dst = reinterpret_cast<u32x4_t*>(crow + (int64_t)(mrow0 + r) * width);
          if constexpr (decltype(streaming)::value)
            __builtin_nontemporal_store(v, dst);
          else
            *dst = v;
        }
      }
    };
    // stream_members (gated launches): gate and up are not read again before the backward, act is read twice right away
    // (by the next layer's rank-r product and by its GEMM); written as streaming stores the two do not push act out of
    // the memory-side cache where act fits it
    if (GATED && g.stream_members)
      store_band(std::true_type{});
    else
      store_band(std::false_type{});
    if constexpr (GATED) {
      // act: the 128 x 64 piece (wm, wn & 1) is shared by the two waves that hold its gate and up bands, 64 rows each
      const char* gband = smem + (4 * wm + (wn & 1)) * 16384;
      const char* uband = gband + 2 * 16384;
      uint16_t* arow = g.act + nlo + 8 * c;
#pragma unroll 8
      for (int t = 0; t < 8; ++t) {
        const int r = 64 * (wn >> 1) + 8 * t + (lane >> 3);
        const int slot = r * 128 + ((c ^ (r & 7)) << 4);
        const u32x4_t gv = *reinterpret_cast<const u32x4_t*>(gband + slot);
        const u32x4_t uv = *reinterpret_cast<const u32x4_t*>(uband + slot);
        u32x4_t o;
#pragma unroll
        for (int d = 0; d < 4; ++d) o[d] = swiglu_gate_pair(gv[d], uv[d]);
        if (mrow0 + r < g.M) *reinterpret_cast<u32x4_t*>(arow + (int64_t)(mrow0 + r) * width) = o;
      }
    }
  }
#endif
}

template <bool LW_ROW_MAJOR, bool GATED = false>
__global__ __launch_bounds__(512) void nf4_gemm_dense_kernel(const DenseArgs g) {
  gemm_dense_tile<LW_ROW_MAJOR, GATED ? kEpiGated : kEpiPlain>(g);
}
// grad-input launches of a single layer (one segment) and, on forward tiles, of the gated pair (paired segments)
__global__ __launch_bounds__(512) void nf4_gemm_dense_dx1_kernel(const DenseArgs g) { gemm_dense_tile<false, kEpiPlain, false, kSegOne>(g); }
__global__ __launch_bounds__(512) void nf4_gemm_dense_tr1_kernel(const DenseArgs g) { gemm_dense_tile<false, kEpiPlain, true, kSegOne>(g); }
__global__ __launch_bounds__(512) void nf4_gemm_dense_trp_kernel(const DenseArgs g) { gemm_dense_tile<false, kEpiPlain, true, kSegPaired>(g); }
// grad-input launch of two members of equal width on transposed tiles (the gate / up pair)
__global__ __launch_bounds__(512) void nf4_gemm_dense_dx2_kernel(const DenseArgs g) { gemm_dense_tile<false, kEpiPlain, false, kSegHalves>(g); }
// grad-input launch (adapter weights [r, K]) whose result goes on through the backward of silu(gate) * up
__global__ __launch_bounds__(512) void nf4_gemm_dense_swiglu_bwd_kernel(const DenseArgs g) { gemm_dense_tile<false, kEpiSwigluBwd, false, kSegOne>(g); }
// grad-input launch on the forward launch's tiles
__global__ __launch_bounds__(512) void nf4_gemm_dense_tr_kernel(const DenseArgs g) { gemm_dense_tile<false, kEpiPlain, true>(g); }

// mode 0 / 2 / 1: nf4_expand_tiled_kernel<mode> over the members' stacked blocks of 16 output columns; mode 3: the
// transposed kernel over the members' 32-row steps (nout = K, kc = N of each member: codes and scalers in the weight's
// own layout).  blk_end is filled in here.
int launch_expand_group(int mode, ExpandGroup& eg, int64_t nk_total, hipStream_t s, bool paired = false) {
  const dim3 block(256);
  int64_t blocks = 0, max_chunks = 1;
  for (int i = 0; i < eg.n; ++i) {
    blocks += mode == 3 ? eg.m[i].kc >> 5 : eg.m[i].nout >> 4;
    eg.blk_end[i] = (int)blocks;
    const int64_t chunks = ((eg.m[i].kc >> 5) + 15) / 16;
    max_chunks = chunks > max_chunks ? chunks : max_chunks;
  }
  TT_REQUIRE(blocks > 0 && blocks < (int64_t(1) << 31), "nf4_expand_tiled: bad launch size");
  if (mode == 3) {
    const int64_t K = eg.m[0].nout;
    TT_REQUIRE(!paired, "nf4_expand_tiled: the paired layout exists for the forward modes only");
    TT_REQUIRE((K + 255) / 256 < 65536, "nf4_expand_tiled: K too large for one launch");
    nf4_expand_tiled_transposed_kernel<<<dim3((unsigned)blocks, (unsigned)((K + 255) / 256)), block, 0, s>>>(eg, (int)K, (int)nk_total);
    return check_launch("nf4_expand_tiled_transposed");
  }
  // One workgroup per 16 columns x 512 contraction indices (a single trip of its loop): a workgroup's load, expansion
  // and stores are a dependent chain, so the more of them are resident the more memory requests are in flight (235 M
  // elements: 129 us with 2048 workgroups that loop, 103 us with 28672 that do not; 4.7 -> 5.9 TB/s).
  int64_t ysplit = max_chunks;
  ysplit = ysplit < 1 ? 1 : (ysplit > 65535 ? 65535 : ysplit);
  const dim3 grid((unsigned)blocks, (unsigned)ysplit);
  const int pr = paired ? 1 : 0;
  if (mode == 1)
    nf4_expand_tiled_kernel<1><<<grid, block, 0, s>>>(eg, (int)nk_total, pr);
  else if (mode == 2)
    nf4_expand_tiled_kernel<2><<<grid, block, 0, s>>>(eg, (int)nk_total, pr);
  else
    nf4_expand_tiled_kernel<0><<<grid, block, 0, s>>>(eg, (int)nk_total, pr);
  return check_launch("nf4_expand_tiled");
}

int launch_expand(int mode, const uint8_t* codes, const float* scal, int64_t Nout, int64_t Kc, int64_t nk_total, int64_t t_off,
                  char* tiled, hipStream_t s, bool paired = false) {
  ExpandGroup eg = {};
  eg.n = 1;
  eg.m[0] = ExpandMember{codes, scal, tiled, (int)Nout, (int)Kc, (int)t_off};
  return launch_expand_group(mode, eg, nk_total, s, paired);
}

int launch_dense(DenseArgs& g, hipStream_t s) {
  g.tiles_m = (g.M + 255) / 256;
  g.tiles_n = (g.Nout + 255) / 256;
  // the LDS limit is a per-device attribute of the function: set it for the current device once (a race only repeats
  // the call)
  static bool attr_set[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
  if (dev < 0 || !attr_set[dev]) {
    for (const void* fn : {reinterpret_cast<const void*>(&nf4_gemm_dense_kernel<true>), reinterpret_cast<const void*>(&nf4_gemm_dense_kernel<false>),
                           reinterpret_cast<const void*>(&nf4_gemm_dense_kernel<true, true>),
                           reinterpret_cast<const void*>(&nf4_gemm_dense_swiglu_bwd_kernel),
                           reinterpret_cast<const void*>(&nf4_gemm_dense_tr_kernel),
                           reinterpret_cast<const void*>(&nf4_gemm_dense_dx1_kernel),
                           reinterpret_cast<const void*>(&nf4_gemm_dense_tr1_kernel),
                           reinterpret_cast<const void*>(&nf4_gemm_dense_trp_kernel),
                           reinterpret_cast<const void*>(&nf4_gemm_dense_dx2_kernel)}) {
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsDense);
      if (e != hipSuccess) return fail(TTAMD_ELAUNCH, "nf4_gemm_dense: cannot reserve %d bytes of LDS: %s", kLdsDense, hipGetErrorString(e));
    }
    if (dev >= 0) attr_set[dev] = true;
  }
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n)), block(512);
  TT_REQUIRE(!g.lw_row_major || g.nseg == 1, "nf4_gemm_dense: a forward launch contracts over one activation tensor (%d given)", g.nseg);
  if (g.lw_row_major)  // forward: the adapter's operands ride the rings behind the weight's last steps
    for (int i = 0; i < g.nad; ++i)
      TT_REQUIRE(g.ad[i].R <= 0 || (g.ad[i].R <= 64 && g.ad[i].R % 8 == 0 && g.ldlx % 8 == 0),
                 "nf4_gemm_dense: the adapter of a forward launch needs a rank that is a multiple of 8, at most 64 (%d)", g.ad[i].R);
  if (g.w_tr) {
    TT_REQUIRE(!g.lw_row_major && !g.act && !g.sw_gup && g.nout == 1 && g.Kc % 64 == 0 && g.Nout % 64 == 0,
               "nf4_gemm_dense: the launch on forward tiles is a plain grad-input launch");
    TT_REQUIRE(!g.w_paired || (g.nseg == 2 && g.seg[0].Kc == g.seg[1].Kc && g.seg[0].Kc % 128 == 0),
               "nf4_gemm_dense: paired forward tiles belong to two members of equal width, a multiple of 128");
    if (g.w_paired)
      nf4_gemm_dense_trp_kernel<<<grid, block, kLdsDense, s>>>(g);
    else if (g.nseg == 1)
      nf4_gemm_dense_tr1_kernel<<<grid, block, kLdsDense, s>>>(g);
    else
      nf4_gemm_dense_tr_kernel<<<grid, block, kLdsDense, s>>>(g);
    return check_launch("nf4_gemm_dense_tr");
  }
  if (g.act) {
    TT_REQUIRE(g.lw_row_major && g.nout == 2 && (g.nad == 2 || g.nad == 0) && g.nseg == 1 && g.out[0].width == g.out[1].width &&
                   g.out[0].width % 128 == 0 && g.Nout == 2 * g.out[0].width,
               "nf4_gemm_dense: the gated launch takes two members of equal width, a multiple of 128");
    // act alone must fit the 256 MB memory-side cache with room to spare (measured: 8192 x 8192 bf16, 134 MB: the gated
    // launch 449 -> 437 us and the step -1 %; 8192 x 14336, 235 MB: the launch 1366 -> 1382 us, the step unchanged)
    g.stream_members = (int64_t)g.M * g.out[0].width * 2 <= (int64_t(160) << 20) ? 1 : 0;
    nf4_gemm_dense_kernel<true, true><<<grid, block, kLdsDense, s>>>(g);
  } else if (g.sw_gup) {
    TT_REQUIRE(!g.lw_row_major && g.nout == 1 && g.out[0].n_begin == 0 && g.out[0].width == g.Nout && !g.out[0].bias &&
                   !g.out[0].cscale && g.sw_gate && g.sw_up && g.out[0].C,
               "nf4_gemm_dense: the SwiGLU-backward launch is a grad-input launch with one output, no bias or column scale");
    nf4_gemm_dense_swiglu_bwd_kernel<<<grid, block, kLdsDense, s>>>(g);
  } else if (g.lw_row_major)
    nf4_gemm_dense_kernel<true><<<grid, block, kLdsDense, s>>>(g);
  else if (g.nseg == 1)
    nf4_gemm_dense_dx1_kernel<<<grid, block, kLdsDense, s>>>(g);
  else if (g.nseg == 2 && g.seg[0].Kc == g.seg[1].Kc)
    nf4_gemm_dense_dx2_kernel<<<grid, block, kLdsDense, s>>>(g);
  else
    nf4_gemm_dense_kernel<false><<<grid, block, kLdsDense, s>>>(g);
  return check_launch("nf4_gemm_dense");
}

}  // namespace

// When the expand-once path is taken, from its 256 x 256 output tiles against the 256 CUs (measured against the fused
// kernel, whose tiles have 128 rows, on 8B / 70B shapes):
//   * at least a full round of tiles and 2048 tokens: always (below 2048 tokens the expansion, which costs as much as
//     the GEMM of ~360 tokens, and the second round eat the gain);
//   * between half a round and a full one, from 1280 tokens: the fused kernel needs a second round of its tiles there
//     (+ 60 %), one partly filled round of this kernel is 15 - 30 % faster;
//   * up to half a round the fused kernel fills the chip in one round of its own and wins.
constexpr int64_t kDenseMinRows = 2048, kDenseMinRowsPartRound = 1280;

bool dense_tiles_apply(int64_t M, int64_t tiles) {
  return (M >= kDenseMinRows && tiles >= 256) || (M >= kDenseMinRowsPartRound && tiles > 128 && tiles < 256);
}

bool dense_path_applies(int64_t M, int64_t Nout, int64_t Kc) {
  if (Nout % 64 != 0 || Kc % 64 != 0) return false;
  if (!dense_tiles_apply(M, ((M + 255) / 256) * ((Nout + 255) / 256))) return false;
  // per-lane byte offsets inside the kernel are 32-bit
  return M * Kc * 2 < (int64_t(1) << 32) && Kc * 2 * 256 < (int64_t(1) << 32);
}

size_t dense_workspace_bytes(int64_t M, int64_t Nout, int64_t Kc) {
  return dense_path_applies(M, Nout, Kc) ? (size_t)Nout * (size_t)Kc * 2 : 0;
}

// One layer: the ordinary forward (mode 0 / 2) or grad-input (mode 1).  Arguments as run_gemm_rs.
int run_gemm_dense(const void* X, const uint8_t* codes, const void* scal, int mode, const void* lX, int ldlx, const void* lW,
                   bool lw_row_major, int R, float lscale, const void* bias, const void* cscale, void* C, int64_t M, int64_t Nout,
                   int64_t Kc, void* workspace, hipStream_t s, const DenseSwigluBwd* swiglu_bwd) {
  TT_REQUIRE(dense_path_applies(M, Nout, Kc), "nf4_gemm_dense: shape not served (M=%lld Nout=%lld Kc=%lld)", (long long)M,
             (long long)Nout, (long long)Kc);
  TT_REQUIRE(aligned16(workspace) && aligned16(X) && aligned16(codes) && aligned16(scal), "nf4_gemm_dense: pointers must be 16-byte aligned");
  if (int rc = launch_expand(mode, codes, reinterpret_cast<const float*>(scal), Nout, Kc, Kc >> 5, 0, reinterpret_cast<char*>(workspace), s))
    return rc;
  DenseArgs g = {};
  g.nseg = g.nout = 1;
  g.seg[0].X = reinterpret_cast<const uint16_t*>(X);
  g.seg[0].Kc = (int)Kc;
  g.nad = R > 0 ? 1 : 0;
  g.ad[0].lX = reinterpret_cast<const uint16_t*>(lX);
  g.ad[0].lW = reinterpret_cast<const uint16_t*>(lW);
  g.ad[0].R = R;
  g.ad[0].n_begin = 0;
  g.ad[0].n_end = (int)Nout;
  g.ad[0].lscale = lscale;
  g.out[0].C = reinterpret_cast<uint16_t*>(C);
  g.out[0].bias = reinterpret_cast<const uint16_t*>(bias);
  g.out[0].cscale = reinterpret_cast<const uint16_t*>(cscale);
  g.out[0].n_begin = 0;
  g.out[0].width = (int)Nout;
  g.Wt = reinterpret_cast<const char*>(workspace);
  g.M = (int)M; g.Nout = (int)Nout; g.Kc = (int)Kc;
  g.lw_row_major = lw_row_major ? 1 : 0;
  g.ldlx = ldlx;
  if (swiglu_bwd) {
    TT_REQUIRE(swiglu_bwd->gate && swiglu_bwd->up && swiglu_bwd->gup && aligned16(swiglu_bwd->gate) && aligned16(swiglu_bwd->up) &&
                   aligned16(swiglu_bwd->gup) && aligned16(C),
               "nf4_gemm_dense: gate, up and their gradients must be non-null and 16-byte aligned");
    g.sw_gate = reinterpret_cast<const uint16_t*>(swiglu_bwd->gate);
    g.sw_up = reinterpret_cast<const uint16_t*>(swiglu_bwd->up);
    g.sw_gup = reinterpret_cast<uint16_t*>(swiglu_bwd->gup);
  }
  return launch_dense(g, s);
}

// Forward of a group of layers with a common input as one launch over the members' concatenated output columns.
size_t dense_group_fwd_workspace_bytes(const GroupGemm& d) {
  int64_t n_total = 0;
  for (int i = 0; i < d.n; ++i) {
    if (d.N[i] % 256 != 0) return 0;  // a tile belongs to one member
    n_total += d.N[i];
  }
  return d.n >= 2 && dense_path_applies(d.M, n_total, d.K) ? (size_t)n_total * (size_t)d.K * 2 : 0;
}

bool dense_group_gated_applies(const GroupGemm& d) {
  return d.n == 2 && d.N[0] == d.N[1] && d.N[0] % 128 == 0 && dense_group_fwd_workspace_bytes(d) > 0;
}

// act != nullptr: the pair (gate, up) with act = silu(y_0) * y_1 written by the same launch (dense_group_gated_applies)
// tiles != nullptr: the members' weights as an earlier call of this function left them in its workspace (the same
// members, the same act-or-not): no expansion launch, workspace is not touched
int run_gemm_dense_group_fwd(const void* x, const GroupGemm& d, const void* h_cat, void* workspace, hipStream_t s, void* act,
                             const void* tiles) {
  TT_REQUIRE(d.n >= 2 && d.n <= kGroupMax && dense_group_fwd_workspace_bytes(d) > 0, "nf4_lora_group_fwd (expanded): shape not served");
  TT_REQUIRE(aligned16(tiles ? tiles : workspace) && aligned16(x), "nf4_lora_group_fwd (expanded): pointers must be 16-byte aligned");
  const bool gated = act != nullptr;
  TT_REQUIRE(!gated || (dense_group_gated_applies(d) && aligned16(act)), "nf4_lora_group_swiglu_fwd (expanded): shape not served");
  DenseArgs g = {};
  g.act = reinterpret_cast<uint16_t*>(act);
  g.nseg = 1;
  g.seg[0].X = reinterpret_cast<const uint16_t*>(x);
  g.seg[0].Kc = (int)d.K;
  g.nout = g.nad = d.n;
  int64_t n_off = 0;
  // the members' weights are expanded by one launch when they come in the same form (with or without transposed scalers)
  ExpandGroup eg = {};
  bool one_launch = true;
  for (int i = 0; i < d.n; ++i) one_launch = one_launch && (d.bscal_t[i] != nullptr) == (d.bscal_t[0] != nullptr);
  for (int i = 0; i < d.n; ++i) {
    const bool tr = d.bscal_t[i] != nullptr;
    // gated: the members' column blocks alternate 8 by 8, the second member starting 8 blocks (128 columns) in
    char* dst = reinterpret_cast<char*>(workspace) + (gated ? (int64_t)i * 128 : n_off) * d.K * 2;
    eg.m[i] = ExpandMember{d.codes[i], tr ? d.bscal_t[i] : d.bscal[i], dst, (int)d.N[i], (int)d.K, 0};
    if (!one_launch && !tiles)
      if (int rc = launch_expand(tr ? 2 : 0, eg.m[i].codes, eg.m[i].scal, d.N[i], d.K, d.K >> 5, 0, dst, s, gated)) return rc;
    g.ad[i].lX = reinterpret_cast<const uint16_t*>(h_cat) + d.r_off[i];
    g.ad[i].lW = d.lora_b[i];
    g.ad[i].R = d.rank[i];
    g.ad[i].n_begin = (int)n_off;
    g.ad[i].n_end = (int)(n_off + d.N[i]);
    g.ad[i].lscale = d.scale[i];
    g.out[i].C = d.y[i];
    g.out[i].bias = d.bias[i];
    g.out[i].cscale = nullptr;
    g.out[i].n_begin = (int)n_off;
    g.out[i].width = (int)d.N[i];
    n_off += d.N[i];
  }
  if (one_launch && !tiles) {
    eg.n = d.n;
    if (int rc = launch_expand_group(d.bscal_t[0] ? 2 : 0, eg, d.K >> 5, s, gated)) return rc;
  }
  g.Wt = reinterpret_cast<const char*>(tiles ? tiles : workspace);
  g.M = (int)d.M; g.Nout = (int)n_off; g.Kc = (int)d.K;
  g.lw_row_major = 1;
  g.ldlx = d.r_off[d.n];
  return launch_dense(g, s);
}

// Grad-input of a group of layers with a common input over the concatenated contraction (see run_gemm_rs_group_dx).
size_t dense_group_dx_workspace_bytes(const GroupDx& d) {
  int64_t n_total = 0;
  for (int i = 0; i < d.n; ++i) {
    if (d.N[i] % 64 != 0) return 0;
    n_total += d.N[i];
    if (d.M * d.N[i] * 2 >= (int64_t(1) << 32)) return 0;
  }
  // the launch contracts over all members' columns: the kernel's 32-bit lane offsets and step counts bound n_total as
  // they bound the contraction of a single layer
  if (!dense_path_applies(d.M, d.K, n_total)) return 0;
  return (size_t)d.K * (size_t)n_total * 2;
}

// tiles_fwd != nullptr: no expansion; the launch reads the tiles the forward launch of the same group left in its
// workspace (the members' weights stacked by rows, or - paired - the gated pair's 128-column alternation).
int run_gemm_dense_group_dx(const GroupDx& d, const void* gh_cat, void* gx, void* workspace, hipStream_t s, const void* tiles_fwd,
                            bool paired) {
  TT_REQUIRE(d.n >= 1 && d.n <= kGroupMax && dense_group_dx_workspace_bytes(d) > 0, "nf4_group_dx (expanded): shape not served");
  TT_REQUIRE(tiles_fwd ? aligned16(tiles_fwd) : aligned16(workspace), "nf4_group_dx (expanded): workspace / tiles must be 16-byte aligned");
  int64_t n_total = 0;
  for (int i = 0; i < d.n; ++i) n_total += d.N[i];
  DenseArgs g = {};
  g.nseg = d.n;
  g.nout = 1;
  int64_t t_off = 0;
  // one expansion launch for the members when all of them come with, or all without, the transposed copies
  ExpandGroup eg = {};
  bool one_launch = true;
  for (int i = 0; i < d.n; ++i) one_launch = one_launch && (d.codes_t[i] != nullptr) == (d.codes_t[0] != nullptr);
  for (int i = 0; i < d.n; ++i) {
    const bool tr = d.codes_t[i] != nullptr;
    TT_REQUIRE(aligned16(d.gy[i]) && (tiles_fwd || (tr ? aligned16(d.codes_t[i]) && aligned16(d.scal_t[i]) : aligned16(d.codes[i]) && d.bscal[i] != nullptr)),
               "nf4_group_dx (expanded): pointers must be 16-byte aligned");
    eg.m[i] = ExpandMember{tr ? d.codes_t[i] : d.codes[i], tr ? d.scal_t[i] : d.bscal[i], reinterpret_cast<char*>(workspace), (int)d.K,
                           (int)d.N[i], (int)t_off};
    if (!one_launch && !tiles_fwd)
      if (int rc = launch_expand(tr ? 1 : 3, eg.m[i].codes, eg.m[i].scal, d.K, d.N[i], n_total >> 5, t_off, reinterpret_cast<char*>(workspace), s))
        return rc;
    t_off += d.N[i] >> 5;
    g.seg[i].X = d.gy[i];
    g.seg[i].Kc = (int)d.N[i];
    if (d.rank[i] > 0) {
      DenseAdapter& a = g.ad[g.nad++];
      a.lX = reinterpret_cast<const uint16_t*>(gh_cat) + d.r_off[i];
      a.lW = d.lora_a[i];
      a.R = d.rank[i];
      a.n_begin = 0;
      a.n_end = (int)d.K;
      a.lscale = 1.0f;
    }
  }
  if (one_launch && !tiles_fwd) {
    eg.n = d.n;
    if (int rc = launch_expand_group(d.codes_t[0] ? 1 : 3, eg, n_total >> 5, s)) return rc;
  }
  g.out[0].C = reinterpret_cast<uint16_t*>(gx);
  g.out[0].n_begin = 0;
  g.out[0].width = (int)d.K;
  g.Wt = reinterpret_cast<const char*>(tiles_fwd ? tiles_fwd : workspace);
  g.M = (int)d.M; g.Nout = (int)d.K; g.Kc = (int)n_total;
  g.lw_row_major = 0;
  g.ldlx = d.r_off[d.n];
  g.w_tr = tiles_fwd ? 1 : 0;
  g.w_paired = tiles_fwd && paired ? 1 : 0;
  return launch_dense(g, s);
}

}  // namespace ttamd

using namespace ttamd;

extern "C" size_t ttamd_tiled_weight_bytes(int64_t N, int64_t K) { return N > 0 && K > 0 ? (size_t)N * (size_t)K * 2 : 0; }

extern "C" int ttamd_fq_per_group_int4_sym_tiled_at_bf16(const void* w, int64_t N, int64_t K, int group_size, int qparam_dtype, float eps,
                                                         void* tiled_fwd, int fwd_paired, void* tiled_bwd, int64_t bwd_n_total,
                                                         int64_t bwd_n_offset, float* scale, void* stream) {
  TT_REQUIRE(!fwd_paired || N % 128 == 0, "fq_per_group_int4_sym_tiled: the paired forward layout needs N (%lld) to be a multiple of 128", (long long)N);
  TT_REQUIRE(bwd_n_total % 64 == 0 && bwd_n_offset % 32 == 0 && bwd_n_offset >= 0 && bwd_n_offset + N <= bwd_n_total && bwd_n_total < (1 << 30),
             "fq_per_group_int4_sym_tiled: rows [%lld, + %lld) do not fit a contraction of %lld (multiples of 32 / 64)",
             (long long)bwd_n_offset, (long long)N, (long long)bwd_n_total);
  TT_REQUIRE(w && aligned16(w) && (tiled_fwd || tiled_bwd), "fq_per_group_int4_sym_tiled: w must be non-null and 16-byte aligned, one output given");
  TT_REQUIRE((!tiled_fwd || aligned16(tiled_fwd)) && (!tiled_bwd || aligned16(tiled_bwd)), "fq_per_group_int4_sym_tiled: outputs must be 16-byte aligned");
  TT_REQUIRE(N > 0 && K > 0 && N % 64 == 0 && K % 64 == 0 && N < (1 << 30) && K < (1 << 30),
             "fq_per_group_int4_sym_tiled: N (%lld) and K (%lld) must be positive multiples of 64", (long long)N, (long long)K);
  TT_REQUIRE(qparam_dtype == TTAMD_BF16 || qparam_dtype == TTAMD_F32, "fq_per_group_int4_sym_tiled: unknown qparam dtype code %d", qparam_dtype);
  TT_REQUIRE(eps > 0.0f, "fq_per_group_int4_sym_tiled: eps must be positive");
  if (!(group_size == 32 || group_size == 64 || group_size == 128 || group_size == 256) || K % group_size != 0)
    return fail(TTAMD_EUNSUPPORTED, "fq_per_group_int4_sym_tiled: group size %d (serves 32, 64, 128, 256 dividing K)", group_size);
  const int64_t gy = (K + 255) / 256;
  TT_REQUIRE(gy < 65536, "fq_per_group_int4_sym_tiled: K too large for one launch");
  fq_int4_sym_tiled_kernel<<<dim3((unsigned)(N / 32), (unsigned)gy), dim3(256), 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const uint16_t*>(w), (int)N, (int)K, group_size / 32, reinterpret_cast<char*>(tiled_fwd),
      reinterpret_cast<char*>(tiled_bwd), scale, (int)(K / group_size), qparam_dtype == TTAMD_BF16, eps, (int)(bwd_n_total >> 5),
      (int)(bwd_n_offset >> 5), fwd_paired ? 1 : 0);
  return check_launch("fq_per_group_int4_sym_tiled");
}

extern "C" int ttamd_fq_per_group_int4_sym_tiled_bf16(const void* w, int64_t N, int64_t K, int group_size, int qparam_dtype, float eps,
                                                      void* tiled_fwd, void* tiled_bwd, float* scale, void* stream) {
  return ttamd_fq_per_group_int4_sym_tiled_at_bf16(w, N, K, group_size, qparam_dtype, eps, tiled_fwd, 0, tiled_bwd, N, 0, scale, stream);
}

namespace {
int tiled_linear(const void* x, const void* tiled_weight, const void* lx, const void* lw, bool lw_row_major, int rank, float lscale,
                 const void* bias, void* y, int64_t M, int64_t n_out, int64_t k_contract, void* stream) {
  TT_REQUIRE(x && tiled_weight && y && aligned16(x) && aligned16(tiled_weight) && aligned16(y), "tiled_linear: pointers must be non-null and 16-byte aligned");
  TT_REQUIRE(bias == nullptr || (reinterpret_cast<uintptr_t>(bias) & 7u) == 0, "tiled_linear: bias must be 8-byte aligned");
  TT_REQUIRE(M > 0 && n_out > 0 && k_contract > 0 && n_out % 64 == 0 && k_contract % 64 == 0,
             "tiled_linear: n_out (%lld) and k_contract (%lld) must be positive multiples of 64", (long long)n_out, (long long)k_contract);
  if (!(M * k_contract * 2 < (int64_t(1) << 32) && k_contract * 2 * 256 < (int64_t(1) << 32) && M < (1 << 30) && n_out < (1 << 30)))
    return fail(TTAMD_EUNSUPPORTED, "tiled_linear: operands too large for 32-bit offsets (M=%lld k=%lld)", (long long)M, (long long)k_contract);
  TT_REQUIRE(rank >= 0 && rank % 8 == 0 && rank <= 64, "tiled_linear: the adapter rank (%d) must be a multiple of 8, at most 64", rank);
  TT_REQUIRE(rank == 0 || (lx && lw && aligned16(lx) && aligned16(lw)), "tiled_linear: adapter operands must be non-null and 16-byte aligned");
  DenseArgs g = {};
  g.nseg = g.nout = 1;
  g.nad = rank > 0 ? 1 : 0;
  g.seg[0].X = reinterpret_cast<const uint16_t*>(x);
  g.seg[0].Kc = (int)k_contract;
  g.out[0].C = reinterpret_cast<uint16_t*>(y);
  g.out[0].bias = reinterpret_cast<const uint16_t*>(bias);
  g.out[0].n_begin = 0;
  g.out[0].width = (int)n_out;
  if (rank > 0) {
    g.ad[0].lX = reinterpret_cast<const uint16_t*>(lx);
    g.ad[0].lW = reinterpret_cast<const uint16_t*>(lw);
    g.ad[0].R = rank;
    g.ad[0].n_begin = 0;
    g.ad[0].n_end = (int)n_out;
    g.ad[0].lscale = lscale;
  }
  g.Wt = reinterpret_cast<const char*>(tiled_weight);
  g.M = (int)M; g.Nout = (int)n_out; g.Kc = (int)k_contract;
  g.lw_row_major = lw_row_major ? 1 : 0;
  g.ldlx = rank;
  return launch_dense(g, reinterpret_cast<hipStream_t>(stream));
}
}  // namespace

extern "C" int ttamd_tiled_linear_dx_bf16(const void* gy, const void* tiled_weight_fwd, const void* gh, const void* lora_a, int rank,
                                          void* gx, int64_t M, int64_t N, int64_t K, void* stream) {
  TT_REQUIRE(gy && tiled_weight_fwd && gx && aligned16(gy) && aligned16(tiled_weight_fwd) && aligned16(gx),
             "tiled_linear_dx: pointers must be non-null and 16-byte aligned");
  TT_REQUIRE(M > 0 && N > 0 && K > 0 && N % 64 == 0 && K % 64 == 0, "tiled_linear_dx: N (%lld) and K (%lld) must be positive multiples of 64",
             (long long)N, (long long)K);
  if (!(M * N * 2 < (int64_t(1) << 32) && N * 2 * 256 < (int64_t(1) << 32) && M < (1 << 30) && K < (1 << 30)))
    return fail(TTAMD_EUNSUPPORTED, "tiled_linear_dx: operands too large for 32-bit offsets (M=%lld N=%lld)", (long long)M, (long long)N);
  TT_REQUIRE(rank >= 0 && rank % 8 == 0 && rank <= 64, "tiled_linear_dx: the adapter rank (%d) must be a multiple of 8, at most 64", rank);
  TT_REQUIRE(rank == 0 || (gh && lora_a && aligned16(gh) && aligned16(lora_a)), "tiled_linear_dx: adapter operands must be non-null and 16-byte aligned");
  DenseArgs g = {};
  g.nseg = g.nout = 1;
  g.seg[0].X = reinterpret_cast<const uint16_t*>(gy);
  g.seg[0].Kc = (int)N;
  g.out[0].C = reinterpret_cast<uint16_t*>(gx);
  g.out[0].n_begin = 0;
  g.out[0].width = (int)K;
  if (rank > 0) {
    g.nad = 1;
    g.ad[0].lX = reinterpret_cast<const uint16_t*>(gh);
    g.ad[0].lW = reinterpret_cast<const uint16_t*>(lora_a);
    g.ad[0].R = rank;
    g.ad[0].n_begin = 0;
    g.ad[0].n_end = (int)K;
    g.ad[0].lscale = 1.0f;
  }
  g.Wt = reinterpret_cast<const char*>(tiled_weight_fwd);
  g.M = (int)M; g.Nout = (int)K; g.Kc = (int)N;
  g.lw_row_major = 0;
  g.ldlx = rank;
  g.w_tr = 1;
  return launch_dense(g, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int ttamd_tiled_linear_bf16(const void* x, const void* tiled_weight, const void* bias, void* y, int64_t M, int64_t n_out,
                                       int64_t k_contract, void* stream) {
  return tiled_linear(x, tiled_weight, nullptr, nullptr, true, 0, 1.0f, bias, y, M, n_out, k_contract, stream);
}

extern "C" int ttamd_tiled_lora_linear_bf16(const void* x, const void* tiled_weight, const void* lx, const void* lw, int lw_row_major,
                                            int rank, float lscale, const void* bias, void* y, int64_t M, int64_t n_out,
                                            int64_t k_contract, void* stream) {
  return tiled_linear(x, tiled_weight, lx, lw, lw_row_major != 0, rank, lscale, bias, y, M, n_out, k_contract, stream);
}

// Layers with a common input on weights in the tiled layout (q / k / v, gate / up of a fake-quantised model): the forward
// over the members' concatenated output columns, the grad-input over the concatenated contraction.
extern "C" int ttamd_tiled_linear_group_fwd_bf16(const void* x, const void* tiled_weights, int n_members, const int64_t* n_out,
                                                 const void* const* bias, void* const* y, void* act, int64_t M, int64_t k_contract,
                                                 void* stream) {
  TT_REQUIRE(act == nullptr || (n_members == 2 && n_out && n_out[0] == n_out[1] && aligned16(act)),
             "tiled_linear_group_fwd: the gated product takes two members of equal width (paired forward tiles) and a 16-byte aligned output");
  TT_REQUIRE(x && tiled_weights && n_out && y && aligned16(x) && aligned16(tiled_weights), "tiled_linear_group_fwd: pointers must be non-null and 16-byte aligned");
  TT_REQUIRE(n_members >= 1 && n_members <= kGroupMax, "tiled_linear_group_fwd: 1 to %d members (got %d)", kGroupMax, n_members);
  TT_REQUIRE(M > 0 && k_contract > 0 && k_contract % 64 == 0, "tiled_linear_group_fwd: k_contract (%lld) must be a positive multiple of 64", (long long)k_contract);
  DenseArgs g = {};
  g.nseg = 1;
  g.seg[0].X = reinterpret_cast<const uint16_t*>(x);
  g.seg[0].Kc = (int)k_contract;
  g.nout = n_members;
  int64_t n_off = 0;
  for (int i = 0; i < n_members; ++i) {
    TT_REQUIRE(n_out[i] > 0 && n_out[i] % 256 == 0, "tiled_linear_group_fwd: member %d: n_out (%lld) must be a positive multiple of 256 (a tile belongs to one member)", i, (long long)n_out[i]);
    TT_REQUIRE(y[i] && aligned16(y[i]) && (!bias || !bias[i] || (reinterpret_cast<uintptr_t>(bias[i]) & 7u) == 0), "tiled_linear_group_fwd: member %d: output must be non-null and 16-byte aligned, bias 8-byte aligned", i);
    g.out[i].C = reinterpret_cast<uint16_t*>(y[i]);
    g.out[i].bias = bias ? reinterpret_cast<const uint16_t*>(bias[i]) : nullptr;
    g.out[i].n_begin = (int)n_off;
    g.out[i].width = (int)n_out[i];
    n_off += n_out[i];
  }
  if (!(M * k_contract * 2 < (int64_t(1) << 32) && k_contract * 2 * 256 < (int64_t(1) << 32) && M < (1 << 30) && n_off < (1 << 30)))
    return fail(TTAMD_EUNSUPPORTED, "tiled_linear_group_fwd: operands too large for 32-bit offsets (M=%lld k=%lld)", (long long)M, (long long)k_contract);
  g.Wt = reinterpret_cast<const char*>(tiled_weights);
  g.M = (int)M; g.Nout = (int)n_off; g.Kc = (int)k_contract;
  g.lw_row_major = 1;
  g.act = reinterpret_cast<uint16_t*>(act);
  return launch_dense(g, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int ttamd_tiled_linear_group_dx_bf16(const void* const* gy, const int64_t* n_out, int n_members, const void* tiled_weights_t,
                                                void* gx, int64_t M, int64_t K, void* stream) {
  TT_REQUIRE(gy && n_out && tiled_weights_t && gx && aligned16(tiled_weights_t) && aligned16(gx), "tiled_linear_group_dx: pointers must be non-null and 16-byte aligned");
  TT_REQUIRE(n_members >= 1 && n_members <= kGroupMax, "tiled_linear_group_dx: 1 to %d members (got %d)", kGroupMax, n_members);
  TT_REQUIRE(M > 0 && K > 0 && K % 64 == 0, "tiled_linear_group_dx: K (%lld) must be a positive multiple of 64", (long long)K);
  DenseArgs g = {};
  g.nseg = n_members;
  g.nout = 1;
  int64_t n_total = 0;
  for (int i = 0; i < n_members; ++i) {
    TT_REQUIRE(gy[i] && aligned16(gy[i]) && n_out[i] > 0 && n_out[i] % 64 == 0, "tiled_linear_group_dx: member %d: gradient non-null and 16-byte aligned, n_out (%lld) a multiple of 64", i, (long long)n_out[i]);
    if (M * n_out[i] * 2 >= (int64_t(1) << 32)) return fail(TTAMD_EUNSUPPORTED, "tiled_linear_group_dx: member %d too large for 32-bit offsets", i);
    g.seg[i].X = reinterpret_cast<const uint16_t*>(gy[i]);
    g.seg[i].Kc = (int)n_out[i];
    n_total += n_out[i];
  }
  if (!(n_total * 2 * 256 < (int64_t(1) << 32) && M < (1 << 30) && K < (1 << 30)))
    return fail(TTAMD_EUNSUPPORTED, "tiled_linear_group_dx: operands too large for 32-bit offsets");
  g.out[0].C = reinterpret_cast<uint16_t*>(gx);
  g.out[0].n_begin = 0;
  g.out[0].width = (int)K;
  g.Wt = reinterpret_cast<const char*>(tiled_weights_t);
  g.M = (int)M; g.Nout = (int)K; g.Kc = (int)n_total;
  g.lw_row_major = 0;
  return launch_dense(g, reinterpret_cast<hipStream_t>(stream));
}
