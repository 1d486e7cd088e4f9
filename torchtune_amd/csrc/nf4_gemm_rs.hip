// Fused NF4-dequantise + bf16 MFMA GEMM, second generation: the weight operand never goes through LDS as bf16.
//
//     C[M, Nout] = X[M, Kc] . D(Wv)[Nout, Kc]^T  (+ bias)  + (lscale . lX)[M, R] . lW[Nout, R]^T
//
// `Wv` is a "weight view" whose rows are output columns and whose packed 4-bit codes run along the
// contraction dimension:
//   forward  : Wv = W   [N, K]  (the NF4 tensor as stored),   one scaler per row per 64 contraction elements
//   backward : Wv = W^T [K, N]  (a transposed copy of the codes), one scaler per contraction element per
//              64 output columns (NF4 blocks run along K, i.e. along the output columns of this view)
//
// Work split.  256 threads = 4 waves; the workgroup owns a BM x 256 tile of C, wave w the 64 output columns
// [64w, 64w+64) for ALL BM rows.  A lane of the MFMA weight operand needs 8 consecutive contraction elements
// of one output column: exactly one dword of codes.  Each lane expands its own code dwords in registers
// (byte -> pair of fp32 code points from a 256-entry LDS table, multiply by the scaler in fp32, round to bf16:
// bit-identical to the stand-alone dequantise kernel) one k-substep ahead of the MFMA that consumes them.
//
// Every global read of the main loop is a direct-to-LDS load (global_load_lds_*): the activation tile with an
// XOR swizzle applied on the global-address side, the code bytes and the scalers into wave-private slots.
// That keeps the vector-memory counter free of register-destination loads, so a single explicit
// `s_waitcnt vmcnt(one batch)` per k-step lets the next batch stay in flight (prefetch distance two k-steps;
// four activation stages so that one workgroup barrier per k-step suffices).
//
// Per 64-wide k-step a wave issues 64 v_mfma_f32_32x32x16_bf16 against ~2.5 VALU ops per weight element,
// 12 direct-to-LDS loads, BM/32 x 4 operand reads and 32 table reads.

#include "common.h"
#include "group.h"
#include "nf4_math.h"

namespace ttamd {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __constant__ float kNF4Rs[16] = TT_NF4_TABLE;

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2_t v;
  v.x = (__bf16)lo;
  v.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}

#define TT_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

struct RsArgs {
  const uint16_t* X;     // [M, Kc] bf16 activations
  const uint8_t* codes;  // [Nout, Kc/2] packed NF4 codes of the weight view
  const float* scal;     // block scalers, fp32: MODE 0 [Nout, Kc/64]; MODE 2 [Kc/64, Nout]; MODE 1 per element [Nout/64, Kc]
  const uint16_t* lX;    // adapter activations [M, R] bf16 (rows ldlx elements apart) or null
  const uint16_t* lW;    // adapter weights: [Nout, R] (lw_row_major) or [R, Nout] bf16, or null
  const uint16_t* bias;  // [Nout] bf16 or null
  const uint16_t* cscale;  // [Nout] bf16 or null: C = (acc + bias) * cscale per column (DoRA's magnitude / norm)
  uint16_t* C;           // [M, Nout] bf16
  float* part;           // SPLIT: fp32 partial products [splits, M, Nout], summed by nf4_gemm_rs_reduce_kernel
  int M, Nout, Kc, R;
  int ksteps;            // SPLIT: 64-wide k-steps per slice of the contraction (blockIdx.y = slice)
  int lw_row_major;
  int ldlx;
  float lscale;
  int tiles_m, tiles_n;
};

// SEG kernels: the contraction is the concatenation of up to kGroupMax segments, each with its own activation, weight
// view and adapter (the grad-input of a group of layers with a common input: gx = sum_i gy_i . D(W_i) + gh_i . A_i is
// one GEMM whose contraction runs over the members' output columns one member after the other).  g.X / codes / scal /
// Kc / lX / lW / R are then unused; M, Nout, C and ldlx are shared.
struct RsSegs {
  const uint16_t* X[kGroupMax];     // [M, Kc[i]]
  const uint8_t* codes[kGroupMax];  // [Nout, Kc[i] / 2]
  const float* scal[kGroupMax];     // MODE 1: [Nout / 64, Kc[i]]
  const uint16_t* lX[kGroupMax];    // adapter activations, rows g.ldlx apart, or null
  const uint16_t* lW[kGroupMax];    // adapter weights [R[i], Nout]
  int Kc[kGroupMax], R[kGroupMax];
  int n;
};

constexpr int kBN = 256;
constexpr int kLutBytes = 256 * 8;  // 256 byte values x (fp32 nf4[hi nibble], fp32 nf4[lo nibble])

// LDS: a ring of 4 activation tiles (shared by the waves), a ring of 3 wave-private {code bytes, scalers} slots, the table
template <int BM>
struct RsLayout {
  static constexpr int kStageA = BM * 128;   // activation tile: BM rows x 64 bf16
  static constexpr int kAStages = 4;
  static constexpr int kWOff = kAStages * kStageA;
  static constexpr int kStageW = 8192 + 2048;  // code bytes [wave][tile j][lane] x 16 B, then scalers [wave] x 512 B
  static constexpr int kWStages = 3;
  static constexpr int kLutOff = kWOff + kWStages * kStageW;
  static constexpr int kTotal = kLutOff;  // dynamic part; the table is a static LDS object of kLutBytes
};

// MODE 0: one scaler per (output column, 64-wide k-step), scaler tensor laid out like the weight's blocks
// MODE 2: the same scalers, tensor transposed so that the 64 columns of a wave are contiguous (one coalesced load)
// MODE 1: one scaler per contraction element, shared by the wave's 64 columns (the transposed weight of the backward)
// SPLIT: the contraction is cut into gridDim.y slices so that a launch with few output tiles still fills the chip; a
// workgroup then leaves its tile as fp32 in g.part (slice 0 includes the adapter) and bias, column scale and the
// rounding to bf16 happen in nf4_gemm_rs_reduce_kernel, which adds the slices in a fixed order.
// SEG: segmented contraction (see RsSegs); only with MODE 1 and without SPLIT.
template <int BM, int MODE, bool SPLIT, bool SEG = false>
__global__ __launch_bounds__(256) void nf4_gemm_rs_kernel(const RsArgs g, const RsSegs sg) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses LDS address-space casts and gfx950 builtins the host pass cannot parse
  static_assert(BM == 256 || BM == 128, "BM");
  static_assert(!SEG || (MODE == 1 && !SPLIT), "segments: grad-input kernels only");
  constexpr bool PER_ELEM = MODE == 1;
  constexpr bool SCAL_T = MODE == 2;
  using L = RsLayout<BM>;
  constexpr int MT = BM / 32;       // activation tiles (MFMA columns) per wave
  constexpr int NT = 2;             // weight tiles (MFMA rows) per wave
  constexpr int kALoads = BM / 32;  // direct-to-LDS instructions per wave per k-step for the activation tile (8 rows each)
  constexpr int kBatch = kALoads + NT + (MODE == 0 ? NT : 1);  // vector-memory operations per wave per k-step
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l31 = lane & 31, h = lane >> 5;

  int tile_m, tile_n;
  {
    // workgroup ids are dealt round-robin to the 8 XCDs (one L2 each): give every XCD a band of m-tiles and walk it
    // column by column, so the workgroups resident on an XCD share each weight tile through its L2 (the weight is
    // then fetched once per XCD instead of once per m-tile)
    const int id = blockIdx.x;
    if ((g.tiles_m & 7) == 0) {
      const int xcd = id & 7, slot = id >> 3, band = g.tiles_m >> 3;
      tile_m = xcd * band + slot % band;
      tile_n = slot / band;
    } else {
      tile_m = id / g.tiles_n;
      tile_n = id % g.tiles_n;
    }
  }
  const int m0 = tile_m * BM, n0 = tile_n * kBN;
  const int Kc = SEG ? sg.Kc[0] : g.Kc;
  const int nkf = Kc >> 6;  // k-steps of the whole contraction: the row stride of the MODE 0 scalers
  int kb = 0, nk = nkf;     // this workgroup's k-steps are [kb, kb + nk)
  if constexpr (SEG) {
    for (int q = 1; q < sg.n; ++q) nk += sg.Kc[q] >> 6;
  }
  if constexpr (SPLIT) {
    kb = blockIdx.y * g.ksteps;
    nk = nkf - kb < g.ksteps ? nkf - kb : g.ksteps;
  }

  // ---- table: entry(byte) = (nf4[byte >> 4], nf4[byte & 15]) as two fp32 (each exactly a bf16 value)
  //      It is a separate LDS object so that the compiler can tell table reads from the direct-to-LDS destinations.
  __shared__ float2 lut_s[256];
  lut_s[tid] = make_float2(round_to_bf16(kNF4Rs[tid >> 4]), round_to_bf16(kNF4Rs[tid & 15]));
  const char* lut = reinterpret_cast<const char*>(lut_s);

  // ---- activation tile.  A row is eight 16-byte chunks; chunk c of row r is stored in slot c ^ ((r >> 1) & 7), which
  //      makes the 128-bit operand reads below bank-conflict free.  A direct-to-LDS instruction writes lane l to
  //      linear slot l, so the lane fetches the chunk that belongs there.
  const int a_r8 = lane >> 3;
  uint32_t a_off[kALoads];  // byte offset of this lane's chunk from X + k0
  // ---- weight view rows of this lane: tile j -> output column n0 + 64 wv + 32 j + l31; half h owns code bytes [16h, 16h+16)
  uint32_t w_off[NT], s_off[NT];  // byte offsets from codes + k0/2 and from scal + tk
  // (the offsets depend on the row length kc of the operands: a SEG kernel recomputes them at every segment boundary)
  auto set_offsets = [&](int kc) {
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      const int trow = wv * (BM / 4) + 8 * i + a_r8;  // row inside the tile
      const int chunk = (lane & 7) ^ ((trow >> 1) & 7);
      int row = m0 + trow;
      row = row < g.M ? row : g.M - 1;
      a_off[i] = ((uint32_t)row * (uint32_t)kc + chunk * 8) * 2u;
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      int col = n0 + wv * 64 + 32 * j + l31;
      col = col < g.Nout ? col : g.Nout - 1;
      w_off[j] = (uint32_t)(((int64_t)col * kc) >> 1) + 16 * h;
      s_off[j] = (uint32_t)col * (uint32_t)(kc >> 6) * 4u;
    }
    if constexpr (SCAL_T) {
      int col = n0 + wv * 64 + lane;  // lane l fetches the scaler of the wave's column l
      col = col < g.Nout ? col : g.Nout - 1;
      s_off[0] = (uint32_t)col * 4u;
    }
    if constexpr (PER_ELEM) {
      // scalers of the wave's 64-column block for the 64 contraction elements of a k-step: lane l fetches element l
      int ob = (n0 >> 6) + wv;
      const int nob = g.Nout >> 6;
      ob = ob < nob ? ob : nob - 1;
      s_off[0] = ((uint32_t)ob * (uint32_t)kc + lane) * 4u;
    }
  };
  set_offsets(Kc);

  // Direct-to-LDS loads are written as inline assembly: `voff` is this lane's 32-bit byte offset from the uniform
  // `base`, the wave's 64 lanes land in LDS at `lds`, `lds` + size, ...  Issued this way the compiler keeps no
  // bookkeeping for them (it would otherwise wait for ALL outstanding loads before the next LDS read it cannot prove
  // disjoint); completion is awaited explicitly with s_waitcnt vmcnt below.
  // M0 (the LDS destination) is formed by the scalar add itself: `lds` is a wave-uniform base, `imm` a compile-time
  // offset.  One wait state must separate a scalar write of M0 from the load that reads it.
  auto dma16 = [&](uint32_t voff, const char* base, uint32_t lds, int imm) {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 ::"v"(voff), "s"(base), "s"(lds), "n"(imm) : "memory", "m0", "scc");
  };
  auto dma4 = [&](uint32_t voff, const char* base, uint32_t lds, int imm) {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                 ::"v"(voff), "s"(base), "s"(lds), "n"(imm) : "memory", "m0", "scc");
  };
  const uint32_t lds0 = (uint32_t)(uintptr_t)TT_LDS_PTR(smem);
  // A batch (k-step t) is kBatch loads: the activation tile -> A stage, this wave's code bytes and scalers -> W stage.
  // They are issued one at a time between MFMAs (slot d of the batch), never back to back: the address unit takes
  // tens of cycles per 64-lane load and a wave that finds its queue full cannot issue anything else meanwhile.
  struct BatchAddr {
    const char *xb, *cb, *sb;
    uint32_t abase, wcodes, wscal;  // LDS bases of this wave's share of the A stage, of its code bytes and of its scalers
  };
  // Global bases of k-step t are base + min(t, nk - 1) * stride (past the end the last tile is reloaded, never
  // consumed).  The main loop carries the three pointers and bumps them by a constant instead of recomputing them.
  const int64_t s_stride = PER_ELEM ? 256 : SCAL_T ? (int64_t)g.Nout * 4 : 4;
  auto batch_addr_at = [&](const char* xb, const char* cb, const char* sb, int sa, int sw) -> BatchAddr {
    BatchAddr b;
    b.xb = xb;
    b.cb = cb;
    b.sb = sb;
    b.abase = lds0 + sa * L::kStageA + wv * (BM / 4) * 128;
    b.wcodes = lds0 + L::kWOff + sw * L::kStageW + wv * NT * 1024;
    b.wscal = lds0 + L::kWOff + sw * L::kStageW + 8192 + wv * 512;
    return b;
  };
  auto batch_addr = [&](int t, int sa, int sw) -> BatchAddr {
    const int tk = kb + (t < nk ? t : nk - 1);
    return batch_addr_at(reinterpret_cast<const char*>(g.X) + ((int64_t)tk << 7),      // + k0 * 2 bytes
                         reinterpret_cast<const char*>(g.codes) + ((int64_t)tk << 5),  // + k0 / 2 bytes
                         reinterpret_cast<const char*>(g.scal) + tk * s_stride, sa, sw);
  };
  auto issue_one = [&](const BatchAddr& b, int d) {  // d is a compile-time constant after unrolling
    if (d < kALoads) {
      dma16(a_off[d], b.xb, b.abase, d * 1024);
    } else if (d < kALoads + NT) {
      const int j = d - kALoads;
      dma16(w_off[j], b.cb, b.wcodes, j * 1024);
    } else if (d < kBatch) {
      const int j = d - kALoads - NT;
      dma4(s_off[j], b.sb, b.wscal, j * 256);
    }
  };
  auto issue = [&](int t, int sa, int sw) {
    const BatchAddr b = batch_addr(t, sa, sw);
#pragma unroll
    for (int d = 0; d < kBatch; ++d) issue_one(b, d);
  };

  // weights of one k-substep: a code byte -> one fp32 pair from the table (fetch), scaled and rounded to bf16 (finish)
  uint32_t codes[NT][4];  // this lane's code dwords of the k-step being expanded: [tile][k-substep]
  float sc[NT], sc_next[NT];
  float2 pend[NT][4];     // table entries fetched in one phase, finished in the next: [tile][code byte]
  u32x4_t wfa[NT], wfb[NT];  // weight operands (8 bf16 each) of two consecutive k-substeps
  bf16x8_t xfa[MT], xfb[MT];

  auto fetch_byte = [&](int j, int ks, int b) {
    uint32_t off;
    if (b == 0) {
      // byte 0 as one sub-dword-addressed shift, like the compiler's own choice for bytes 1-3 (it would otherwise
      // emit a mask and a shift here)
      asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0"
          : "=v"(off) : "v"(3u), "v"(codes[j][ks]));
    } else {
      off = ((codes[j][ks] >> (8 * b)) & 0xffu) << 3;
    }
    pend[j][b] = *reinterpret_cast<const float2*>(lut + off);
  };
  // finish byte b of tile j into wf[j]; s8 = the eight per-element scalers of the substep (PER_ELEM), s = the row's scaler
  auto finish_byte = [&](u32x4_t (&wf)[NT], int j, int b, const float (&s)[NT], const float (&s8)[8]) {
    if constexpr (PER_ELEM)
      wf[j][b] = pack_bf16x2(pend[j][b].x * s8[2 * b], pend[j][b].y * s8[2 * b + 1]);
    else
      wf[j][b] = pack_bf16x2(pend[j][b].x * s[j], pend[j][b].y * s[j]);
  };
  auto load_s8 = [&](float (&s8)[8], int sw, int ks) {
    if constexpr (PER_ELEM) {
      const f32x4_t* sp = reinterpret_cast<const f32x4_t*>(smem + L::kWOff + sw * L::kStageW + 8192 + wv * 512 + (32 * h + 8 * ks) * 4);
      const f32x4_t a = sp[0], b = sp[1];
      s8[0] = a.x; s8[1] = a.y; s8[2] = a.z; s8[3] = a.w; s8[4] = b.x; s8[5] = b.y; s8[6] = b.z; s8[7] = b.w;
    }
  };
  auto load_codes = [&](int sw, float (&s_out)[NT]) {
    const char* wbase = smem + L::kWOff + sw * L::kStageW;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(wbase + (wv * NT + j) * 1024 + lane * 16);
      codes[j][0] = v.x; codes[j][1] = v.y; codes[j][2] = v.z; codes[j][3] = v.w;
      if constexpr (MODE == 0) s_out[j] = *reinterpret_cast<const float*>(wbase + 8192 + wv * 512 + j * 256 + lane * 4);
      if constexpr (SCAL_T) s_out[j] = *reinterpret_cast<const float*>(wbase + 8192 + wv * 512 + (32 * j + l31) * 4);
    }
  };

  f32x16_t acc[NT][MT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;

  // operand read offsets inside a stage: row 32 i + l31, chunk 4h + ks, slot = chunk ^ ((row >> 1) & 7)
  int x_off[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) x_off[ks] = l31 * 128 + (((4 * h + ks) ^ ((l31 >> 1) & 7)) << 4);

  // One phase = the 16 (NT x MT) MFMAs of a k-substep, cut into quarters.  Quarter q:
  //   MFMAs of weight tile q/2 against activation tiles [MT/2 (q%2), +MT/2)
  //   operand reads of the NEXT phase: activation tiles [MT/4 q, +MT/4)
  //   finish + fetch of code bytes 2(q%2), 2(q%2)+1 of weight tile q/2 (finish: previous fetch -> wf_next)
  //   up to two direct-to-LDS loads of batch `b` (slots d0, d0+1)
  // and the scheduler is asked to alternate MFMA / VALU / LDS inside the quarter.
  auto phase = [&](const bf16x8_t (&xf_use)[MT], const u32x4_t (&wf_use)[NT], bf16x8_t (&xf_next)[MT], int st_next, int ks_next,
                   u32x4_t (&wf_next)[NT], const float (&s_fin)[NT], int sw_fin, int ks_fin, int ks_fetch, const BatchAddr& b,
                   int d_first, int d_per_quarter_even, int d_per_quarter_odd) {
    float s8[8];
    load_s8(s8, sw_fin, ks_fin);
    const char* sA = smem + st_next * L::kStageA;
    int d = d_first;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int j = q >> 1;
      const int nd = (q & 1) ? d_per_quarter_odd : d_per_quarter_even;
#pragma unroll
      for (int u = 0; u < 2; ++u)
        if (u < nd) issue_one(b, d + u);
      d += nd;
#pragma unroll
      for (int i = (MT / 4) * q; i < (MT / 4) * (q + 1); ++i)
        xf_next[i] = *reinterpret_cast<const bf16x8_t*>(sA + i * 4096 + x_off[ks_next]);
#pragma unroll
      for (int i = (MT / 2) * (q & 1); i < (MT / 2) * ((q & 1) + 1); ++i)
        acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wf_use[j]), xf_use[i], acc[j][i], 0, 0, 0);
#pragma unroll
      for (int bb = 2 * (q & 1); bb < 2 * (q & 1) + 2; ++bb) {
        finish_byte(wf_next, j, bb, s_fin, s8);
        fetch_byte(j, ks_fetch, bb);
      }
#pragma unroll
      for (int r = 0; r < MT / 2; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);  // VALU
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- software pipeline.  Activation tile t lives in A stage t % 4, this wave's codes of k-step t in W stage t % 3.
  // Step t:
  //   phase 0,1 : MFMAs on substeps 0,1 of tile t; batch t+2 is issued, one load per quarter phase
  //   wait for this wave's batch t+1 (batch t+2 stays in flight); barrier: tile t+1 is visible to all waves
  //   phase 2,3 : MFMAs on substeps 2,3; codes of k-step t+1 are read back; phase 3 pre-reads the operands of step t+1
  // That one barrier per step also orders stage reuse: a wave issuing batch t+2 into the A stage of tile t-2 has
  // passed barrier t-1, which every wave reaches only after finishing step t-2.  W stages are wave-private.
  // Weights are expanded just in time: substep ks is fetched two phases and finished one phase before its MFMAs.
  // Global bases of the next batch to issue, carried through the main loop and bumped by a constant per k-step.
  const char *pxb, *pcb, *psb;
  auto seg_base = [&](int q, int step) {
    pxb = reinterpret_cast<const char*>(sg.X[q]) + ((int64_t)step << 7);
    pcb = reinterpret_cast<const char*>(sg.codes[q]) + ((int64_t)step << 5);
    psb = reinterpret_cast<const char*>(sg.scal[q]) + (int64_t)step * 256;
  };
  if constexpr (SEG) {  // segment 0 has at least two k-steps (the host puts the widest first): batches 0 and 1 are its
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      seg_base(0, t);
      const BatchAddr bt = batch_addr_at(pxb, pcb, psb, t, t);
#pragma unroll
      for (int d = 0; d < kBatch; ++d) issue_one(bt, d);
    }
  } else {
    issue(0, 0, 0);
    issue(1, 1, 1);
  }
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kBatch) : "memory");  // batch 0 landed everywhere, table written
  load_codes(0, sc);
  {
    float s8[8];
    load_s8(s8, 0, 0);
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        fetch_byte(j, 0, b);
        finish_byte(wfa, j, b, sc, s8);
        fetch_byte(j, 1, b);
      }
  }
#pragma unroll
  for (int i = 0; i < MT; ++i) xfa[i] = *reinterpret_cast<const bf16x8_t*>(smem + i * 4096 + x_off[0]);

  constexpr int kDEven = (kBatch + 7) / 8 > 1 ? 2 : 1;  // loads per even quarter over the 8 quarters of phases 0 and 1
  constexpr int kDOdd = (kBatch - 4 * kDEven + 3) / 4;  // and per odd quarter
  static_assert(4 * kDEven + 4 * kDOdd >= kBatch && kDOdd <= 2 && kDOdd >= 0, "batch does not fit the 8 quarter phases");
  int a0 = 0, w0 = 0;  // A / W stage of the k-step being multiplied
  // One k-step: multiplies tile kt, issues batch kt + 2 from the carried bases, then moves them on by `adv` k-steps
  // (0 past the end of the contraction: the last tile is reloaded, never consumed).
  auto k_step = [&](int64_t adv) {
    const int a1 = (a0 + 1) & 3, a2 = (a0 + 2) & 3;
    const int w1 = w0 == 2 ? 0 : w0 + 1, w2 = w1 == 2 ? 0 : w1 + 1;
    const BatchAddr b = batch_addr_at(pxb, pcb, psb, a2, w2);
    pxb += adv << 7;
    pcb += adv << 5;
    psb += adv * s_stride;
    phase(xfa, wfa, xfb, a0, 1, wfb, sc, w0, 1, 2, b, 0, kDEven, kDOdd);
    phase(xfb, wfb, xfa, a0, 2, wfa, sc, w0, 2, 3, b, 2 * (kDEven + kDOdd), kDEven, kDOdd);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kBatch) : "memory");
    load_codes(w1, sc_next);
    phase(xfa, wfa, xfb, a0, 3, wfb, sc, w0, 3, 0, b, kBatch, 0, 0);
    phase(xfb, wfb, xfa, a1, 0, wfa, sc_next, w1, 0, 1, b, kBatch, 0, 0);
#pragma unroll
    for (int j = 0; j < NT; ++j) sc[j] = sc_next[j];
    a0 = a1;
    w0 = w1;
  };
  if constexpr (!SEG) {
    const BatchAddr b2 = batch_addr(2, 0, 0);  // global bases of k-step 2
    pxb = b2.xb; pcb = b2.cb; psb = b2.sb;
    for (int kt = 0; kt < nk; ++kt) k_step(kt + 3 < nk ? 1 : 0);
  } else {
    // The batches are issued segment by segment; inside a segment the lane offsets are loop constants.  The k-steps
    // multiplied meanwhile lag two batches behind and do not care which segment their tile came from.  The last
    // segment runs the two extra steps that drain the pipeline.
    int issued = 2;  // index of the next batch to issue
    for (int q = 0; q < sg.n; ++q) {
      int steps = sg.Kc[q] >> 6;
      if (q == 0) {
        steps -= 2;
        seg_base(0, nk > 2 ? 2 : 1);
      } else {
        set_offsets(sg.Kc[q]);
        seg_base(q, 0);
      }
      if (q == sg.n - 1) steps += 2;
      for (int it = 0; it < steps; ++it) {
        k_step(issued + 1 < nk ? 1 : 0);
        ++issued;
      }
    }
  }

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the clamped batches issued by the last two steps
  // ---- adapter: R extra contraction steps, operands straight from global memory
  //      (a SEG kernel has one adapter per segment)
  const int n_adapters = SEG ? sg.n : 1;
  for (int ad = 0; ad < n_adapters; ++ad) {
    const uint16_t* __restrict__ lX = SEG ? sg.lX[ad] : g.lX;
    const uint16_t* __restrict__ lW = SEG ? sg.lW[ad] : g.lW;
    const int R = SEG ? sg.R[ad] : g.R;
    if (!(R > 0 && lX != nullptr && (!SPLIT || blockIdx.y == 0))) continue;
    for (int rc = 0; rc < R; rc += 16) {
      const int r0 = rc + 8 * h;
      const bool in = r0 < R;  // R % 8 == 0: a lane's 8 indices are all in or all out
      bf16x8_t wfr[NT], xfr[MT];
      // every request of the step first, then their uses: one trip to memory per step (with the scaling between two
      // loads the compiler waited for each of them in turn)
      u32x4_t xraw[MT];
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        int row = m0 + 32 * i + l31;
        row = row < g.M ? row : g.M - 1;
        xraw[i] = u32x4_t{0, 0, 0, 0};
        if (in) xraw[i] = *reinterpret_cast<const u32x4_t*>(lX + (int64_t)row * g.ldlx + r0);
      }
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        int col = n0 + wv * 64 + 32 * j + l31;
        col = col < g.Nout ? col : g.Nout - 1;
        u32x4_t raw = {0, 0, 0, 0};
        if (in) {
          if (g.lw_row_major) {
            raw = *reinterpret_cast<const u32x4_t*>(lW + (int64_t)col * R + r0);
          } else {
            uint32_t e[8];
#pragma unroll
            for (int d = 0; d < 8; ++d) e[d] = lW[(int64_t)(r0 + d) * g.Nout + col];
#pragma unroll
            for (int d = 0; d < 4; ++d) raw[d] = e[2 * d] | (e[2 * d + 1] << 16);
          }
        }
        wfr[j] = __builtin_bit_cast(bf16x8_t, raw);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        u32x4_t raw = xraw[i];
        if (g.lscale != 1.0f) {
#pragma unroll
          for (int d = 0; d < 4; ++d)
            raw[d] = pack_bf16x2(bits_f32(raw[d] << 16) * g.lscale, bits_f32(raw[d] & 0xffff0000u) * g.lscale);
        }
        xfr[i] = __builtin_bit_cast(bf16x8_t, raw);
      }
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int i = 0; i < MT; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wfr[j], xfr[i], acc[j][i], 0, 0, 0);
    }
  }

  // ---- epilogue.  acc[j][i][v] = C[m][n] with m = m0 + 32 i + l31 and n = n0 + 64 wv + 32 j + 8 (v/4) + 4 h + v%4.
  //      Stored straight from these registers a wave would write 16-byte pieces of 32 different rows per instruction,
  //      which the memory system turns into partial-line read-modify-writes.  Instead each wave transposes its
  //      BM x 64 band through LDS (the activation ring is free now: BM x 128 bytes per wave) and writes whole
  //      128-byte row segments.  16-byte chunk c of row r sits in slot c ^ (r & 7): both sides are conflict-free.
  if constexpr (SPLIT) {
    // fp32 partial tile, straight from the registers: a lane holds four consecutive columns of a row (16 bytes), the
    // two halves of a wave make 32 bytes and the four q of a weight tile complete the row's 128-byte line
    if (n0 + wv * 64 >= g.Nout) return;
    float* P = g.part + (int64_t)blockIdx.y * g.M * g.Nout + n0 + wv * 64 + 4 * h;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int row = m0 + 32 * i + l31;
      if (row >= g.M) continue;
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<f32x4_t*>(P + (int64_t)row * g.Nout + 32 * j + 8 * q) =
              f32x4_t{acc[j][i][4 * q], acc[j][i][4 * q + 1], acc[j][i][4 * q + 2], acc[j][i][4 * q + 3]};
    }
    return;
  }
  __syncthreads();                      // every wave is done reading the activation ring
  if (n0 + wv * 64 >= g.Nout) return;  // the whole 64-column band of this wave lies outside (no barrier follows)
  {
    char* band = smem + wv * (BM * 128);
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float b4[4] = {0.f, 0.f, 0.f, 0.f};
        if (g.bias) {
          const u32x2_t bb = *reinterpret_cast<const u32x2_t*>(g.bias + n0 + wv * 64 + 32 * j + 8 * q + 4 * h);
          b4[0] = bits_f32(bb.x << 16); b4[1] = bits_f32(bb.x & 0xffff0000u);
          b4[2] = bits_f32(bb.y << 16); b4[3] = bits_f32(bb.y & 0xffff0000u);
        }
        float c4[4] = {1.f, 1.f, 1.f, 1.f};
        if (g.cscale) {
          const u32x2_t cc = *reinterpret_cast<const u32x2_t*>(g.cscale + n0 + wv * 64 + 32 * j + 8 * q + 4 * h);
          c4[0] = bits_f32(cc.x << 16); c4[1] = bits_f32(cc.x & 0xffff0000u);
          c4[2] = bits_f32(cc.y << 16); c4[3] = bits_f32(cc.y & 0xffff0000u);
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const int r = 32 * i + l31;
          u32x2_t o;
          o.x = pack_bf16x2((acc[j][i][4 * q + 0] + b4[0]) * c4[0], (acc[j][i][4 * q + 1] + b4[1]) * c4[1]);
          o.y = pack_bf16x2((acc[j][i][4 * q + 2] + b4[2]) * c4[2], (acc[j][i][4 * q + 3] + b4[3]) * c4[3]);
          *reinterpret_cast<u32x2_t*>(band + r * 128 + (((4 * j + q) ^ (r & 7)) << 4) + 8 * h) = o;
        }
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int c = lane & 7;
    uint16_t* crow = g.C + n0 + wv * 64 + 8 * c;
#pragma unroll 8
    for (int t = 0; t < BM / 8; ++t) {
      const int r = 8 * t + (lane >> 3);
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(band + r * 128 + ((c ^ (r & 7)) << 4));
      if (m0 + r < g.M) *reinterpret_cast<u32x4_t*>(crow + (int64_t)(m0 + r) * g.Nout) = v;
    }
  }
#endif
}

// The same kernel on v_mfma_f32_16x16x32_bf16.  This part is power-limited under matrix load and the 16 x 16 x 32 shape
// sustains 13 % more FLOP/s than 32 x 32 x 16 at the same power (2.04 against 1.80 PFLOP/s for MFMA-only loops), so the
// loop is re-cut for it: a lane (l15, lg) of the weight operand holds row l15 of a 16-column tile and the 8 contraction
// elements [16 lg + 8 ks, + 8) of substep ks - still exactly one dword of codes - and a 64-wide k-step is two substeps
// of NT (4) x MT (BM / 16) MFMAs.  Loads, LDS stages and the table are those of the kernel above; what changes is who
// reads what: the code bytes a direct-to-LDS instruction leaves as 16 bytes per (row, half) are read back as 8 bytes per
// (row, quarter), the activation operand is chunk 2 lg + ks of its row.
//   phase p = (substep ks = p / 2, half ih = p % 2): the NT x MT/2 MFMAs of substep ks against activation tiles
//     [MT/2 ih, + MT/2), the operand reads of the next phase, the finish of the 8 table entries fetched in the previous
//     phase and the fetch of the next 8 (tiles 0, 1 of a substep in one phase, tiles 2, 3 in the next);
//   the workgroup barrier of a k-step stands after phase 0: from phase 1 on the entries fetched belong to the next
//     k-step's codes, which are read back right after it.
template <int BM, int MODE, bool SPLIT, bool SEG = false>
__global__ __launch_bounds__(256) void nf4_gemm_rs16_kernel(const RsArgs g, const RsSegs sg) {
#if defined(__HIP_DEVICE_COMPILE__)
  static_assert(BM == 256 || BM == 128, "BM");
  static_assert(!SEG || (MODE == 1 && !SPLIT), "segments: grad-input kernels only");
  constexpr bool PER_ELEM = MODE == 1;
  constexpr bool SCAL_T = MODE == 2;
  using L = RsLayout<BM>;
  constexpr int MT = BM / 16;       // 16-row activation tiles (MFMA columns) per wave
  constexpr int MH = MT / 2;        // of which a phase takes half
  constexpr int NT = 4;             // 16-column weight tiles (MFMA rows) per wave
  constexpr int ND = 2;             // direct-to-LDS instructions per k-step for the wave's code bytes (32 rows each)
  constexpr int kALoads = BM / 32;  // and for its share of the activation tile (8 rows each)
  constexpr int kBatch = kALoads + ND + (MODE == 0 ? ND : 1);
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l31 = lane & 31, h = lane >> 5;    // roles on the load side
  const int l15 = lane & 15, lg = lane >> 4;   // roles on the MFMA side

  int tile_m, tile_n;
  {
    const int id = blockIdx.x;
    if ((g.tiles_m & 7) == 0) {
      const int xcd = id & 7, slot = id >> 3, band = g.tiles_m >> 3;
      tile_m = xcd * band + slot % band;
      tile_n = slot / band;
    } else {
      tile_m = id / g.tiles_n;
      tile_n = id % g.tiles_n;
    }
  }
  const int m0 = tile_m * BM, n0 = tile_n * kBN;
  const int Kc = SEG ? sg.Kc[0] : g.Kc;
  const int nkf = Kc >> 6;
  int kb = 0, nk = nkf;
  if constexpr (SEG) {
    for (int q = 1; q < sg.n; ++q) nk += sg.Kc[q] >> 6;
  }
  if constexpr (SPLIT) {
    kb = blockIdx.y * g.ksteps;
    nk = nkf - kb < g.ksteps ? nkf - kb : g.ksteps;
  }

  __shared__ float2 lut_s[256];
  lut_s[tid] = make_float2(round_to_bf16(kNF4Rs[tid >> 4]), round_to_bf16(kNF4Rs[tid & 15]));
  const char* lut = reinterpret_cast<const char*>(lut_s);

  // ---- load side: as in nf4_gemm_rs_kernel
  const int a_r8 = lane >> 3;
  uint32_t a_off[kALoads];
  uint32_t w_off[ND], s_off[ND];
  auto set_offsets = [&](int kc) {
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      const int trow = wv * (BM / 4) + 8 * i + a_r8;
      const int chunk = (lane & 7) ^ ((trow >> 1) & 7);
      int row = m0 + trow;
      row = row < g.M ? row : g.M - 1;
      a_off[i] = ((uint32_t)row * (uint32_t)kc + chunk * 8) * 2u;
    }
#pragma unroll
    for (int j = 0; j < ND; ++j) {
      int col = n0 + wv * 64 + 32 * j + l31;
      col = col < g.Nout ? col : g.Nout - 1;
      w_off[j] = (uint32_t)(((int64_t)col * kc) >> 1) + 16 * h;
      s_off[j] = (uint32_t)col * (uint32_t)(kc >> 6) * 4u;
    }
    if constexpr (SCAL_T) {
      int col = n0 + wv * 64 + lane;
      col = col < g.Nout ? col : g.Nout - 1;
      s_off[0] = (uint32_t)col * 4u;
    }
    if constexpr (PER_ELEM) {
      int ob = (n0 >> 6) + wv;
      const int nob = g.Nout >> 6;
      ob = ob < nob ? ob : nob - 1;
      s_off[0] = ((uint32_t)ob * (uint32_t)kc + lane) * 4u;
    }
  };
  set_offsets(Kc);

  auto dma16 = [&](uint32_t voff, const char* base, uint32_t lds, int imm) {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 ::"v"(voff), "s"(base), "s"(lds), "n"(imm) : "memory", "m0", "scc");
  };
  auto dma4 = [&](uint32_t voff, const char* base, uint32_t lds, int imm) {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                 ::"v"(voff), "s"(base), "s"(lds), "n"(imm) : "memory", "m0", "scc");
  };
  const uint32_t lds0 = (uint32_t)(uintptr_t)TT_LDS_PTR(smem);
  struct BatchAddr {
    const char *xb, *cb, *sb;
    uint32_t abase, wcodes, wscal;
  };
  const int64_t s_stride = PER_ELEM ? 256 : SCAL_T ? (int64_t)g.Nout * 4 : 4;
  auto batch_addr_at = [&](const char* xb, const char* cb, const char* sb, int sa, int sw) -> BatchAddr {
    BatchAddr b;
    b.xb = xb;
    b.cb = cb;
    b.sb = sb;
    b.abase = lds0 + sa * L::kStageA + wv * (BM / 4) * 128;
    b.wcodes = lds0 + L::kWOff + sw * L::kStageW + wv * ND * 1024;
    b.wscal = lds0 + L::kWOff + sw * L::kStageW + 8192 + wv * 512;
    return b;
  };
  auto batch_addr = [&](int t, int sa, int sw) -> BatchAddr {
    const int tk = kb + (t < nk ? t : nk - 1);
    return batch_addr_at(reinterpret_cast<const char*>(g.X) + ((int64_t)tk << 7),
                         reinterpret_cast<const char*>(g.codes) + ((int64_t)tk << 5),
                         reinterpret_cast<const char*>(g.scal) + tk * s_stride, sa, sw);
  };
  auto issue_one = [&](const BatchAddr& b, int d) {
    if (d < kALoads) {
      dma16(a_off[d], b.xb, b.abase, d * 1024);
    } else if (d < kALoads + ND) {
      const int j = d - kALoads;
      dma16(w_off[j], b.cb, b.wcodes, j * 1024);
    } else if (d < kBatch) {
      const int j = d - kALoads - ND;
      dma4(s_off[j], b.sb, b.wscal, j * 256);
    }
  };
  auto issue = [&](int t, int sa, int sw) {
    const BatchAddr b = batch_addr(t, sa, sw);
#pragma unroll
    for (int d = 0; d < kBatch; ++d) issue_one(b, d);
  };

  // ---- weights: tile j is rows 16 j + l15 of the wave's 64; substep ks of this lane is code dword 2 lg + ks of the
  //      row's eight.  A load instruction left row 32 J + r, bytes [16 H, + 16) at lane r + 32 H of piece J.
  uint32_t codes[NT][2];
  float sc[NT], sc_next[NT];
  float2 pend[2][4];  // the eight table entries in flight: [tile of the pair][code byte]
  u32x4_t wfa[NT], wfb[NT];
  bf16x8_t xfa[MH], xfb[MH];

  auto fetch_byte = [&](int jj, int j, int ks, int b) {
    uint32_t off;
    if (b == 0) {
      asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0"
          : "=v"(off) : "v"(3u), "v"(codes[j][ks]));
    } else {
      off = ((codes[j][ks] >> (8 * b)) & 0xffu) << 3;
    }
    pend[jj][b] = *reinterpret_cast<const float2*>(lut + off);
  };
  auto finish_byte = [&](u32x4_t (&wf)[NT], int jj, int j, int b, const float (&s)[NT], const float (&s8)[8]) {
    if constexpr (PER_ELEM)
      wf[j][b] = pack_bf16x2(pend[jj][b].x * s8[2 * b], pend[jj][b].y * s8[2 * b + 1]);
    else
      wf[j][b] = pack_bf16x2(pend[jj][b].x * s[j], pend[jj][b].y * s[j]);
  };
  auto load_s8 = [&](float (&s8)[8], int sw, int ks) {
    if constexpr (PER_ELEM) {
      const f32x4_t* sp = reinterpret_cast<const f32x4_t*>(smem + L::kWOff + sw * L::kStageW + 8192 + wv * 512 + (16 * lg + 8 * ks) * 4);
      const f32x4_t a = sp[0], b = sp[1];
      s8[0] = a.x; s8[1] = a.y; s8[2] = a.z; s8[3] = a.w; s8[4] = b.x; s8[5] = b.y; s8[6] = b.z; s8[7] = b.w;
    }
  };
  auto load_codes = [&](int sw, float (&s_out)[NT]) {
    const char* wbase = smem + L::kWOff + sw * L::kStageW;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const u32x2_t v = *reinterpret_cast<const u32x2_t*>(wbase + (wv * ND + (j >> 1)) * 1024 +
                                                          (16 * (j & 1) + l15 + 32 * (lg >> 1)) * 16 + 8 * (lg & 1));
      codes[j][0] = v.x; codes[j][1] = v.y;
      if constexpr (MODE == 0) s_out[j] = *reinterpret_cast<const float*>(wbase + 8192 + wv * 512 + (j >> 1) * 256 + (16 * (j & 1) + l15) * 4);
      if constexpr (SCAL_T) s_out[j] = *reinterpret_cast<const float*>(wbase + 8192 + wv * 512 + (16 * j + l15) * 4);
    }
  };

  f32x4_t acc[NT][MT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[j][i][v] = 0.f;

  // operand read offsets inside a stage: row 16 i + l15, chunk 2 lg + ks, slot = chunk ^ ((row >> 1) & 7)
  int x_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) x_off[ks] = l15 * 128 + (((2 * lg + ks) ^ ((l15 >> 1) & 7)) << 4);

  // One phase, in quarters.  Quarter q:
  //   MFMAs of weight tile q against the MH activation tiles of the phase's half
  //   operand reads of the NEXT phase: activation tiles [MH/4 q, + MH/4) of its half
  //   finish + fetch of code bytes 2 (q % 2), 2 (q % 2) + 1 of tile q / 2 of the pair (finish: what the previous phase
  //     fetched, into wf_next of the pair jp_fin; fetch: the pair jp_fetch of substep ks_fetch)
  //   up to two direct-to-LDS loads of batch `b`
  auto phase = [&](const bf16x8_t (&xf_use)[MH], int ih_use, const u32x4_t (&wf_use)[NT], bf16x8_t (&xf_next)[MH], int st_next,
                   int ks_next, int ih_next, u32x4_t (&wf_next)[NT], int jp_fin, const float (&s_fin)[NT], int sw_fin, int ks_fin,
                   int jp_fetch, int ks_fetch, const BatchAddr& b, int d_first, int d_even, int d_odd) {
    float s8[8];
    load_s8(s8, sw_fin, ks_fin);
    const char* sA = smem + st_next * L::kStageA + (MH * ih_next) * 2048;
    int d = d_first;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int nd = (q & 1) ? d_odd : d_even;
      const int jj = q >> 1, b0 = 2 * (q & 1);
      // The MFMAs are written in assembly with the accumulator tied to itself in the AGPR file: left to the register
      // allocator, the 64 four-register accumulators of this loop get different source and destination registers and are
      // copied around the loop's back edge (700 v_accvgpr moves per k-step).  The scheduler does not know such a
      // statement for a matrix instruction, so the interleaving is spelled out: one MFMA, one piece of the quarter's
      // other work, a scheduling barrier.  A 16 x 16 x 32 MFMA keeps the pipe for 16 cycles and the wave issues in
      // order: whatever follows it in program order rides in the 12 cycles before the next one can start.
      auto mfma = [&](int i) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[q][MH * ih_use + i]) : "v"(wf_use[q]), "v"(xf_use[i]));
      };
      auto other = [&](int slot) {  // the quarter's other work in eight pieces
        constexpr int kReads = MH / 4;  // operand reads of the next phase per quarter: 2 (BM = 256) or 1
        switch (slot) {
          case 0:
            xf_next[kReads * q] = *reinterpret_cast<const bf16x8_t*>(sA + (kReads * q) * 2048 + x_off[ks_next]);
            break;
          case 1: finish_byte(wf_next, jj, 2 * jp_fin + jj, b0, s_fin, s8); break;
          case 2: fetch_byte(jj, 2 * jp_fetch + jj, ks_fetch, b0); break;
          case 3:
            if (kReads > 1) xf_next[kReads * q + 1] = *reinterpret_cast<const bf16x8_t*>(sA + (kReads * q + 1) * 2048 + x_off[ks_next]);
            break;
          case 4: finish_byte(wf_next, jj, 2 * jp_fin + jj, b0 + 1, s_fin, s8); break;
          case 5: fetch_byte(jj, 2 * jp_fetch + jj, ks_fetch, b0 + 1); break;
          case 6:
            if (nd > 0) issue_one(b, d);
            break;
          default:
            if (nd > 1) issue_one(b, d + 1);
            break;
        }
      };
      constexpr int kPer = 8 / MH;  // pieces per MFMA: 1 (BM = 256) or 2
#pragma unroll
      for (int i = 0; i < MH; ++i) {
        mfma(i);
#pragma unroll
        for (int u = 0; u < kPer; ++u) other(kPer * i + u);
        __builtin_amdgcn_sched_barrier(0);
      }
      d += nd;
    }
  };

  // ---- software pipeline: as in nf4_gemm_rs_kernel (activation tile t in A stage t % 4, this wave's codes in W stage
  //      t % 3, batch t + 2 issued during phases 0 and 1 of step t), with the barrier of step t after phase 0.  There
  //      this wave's batch t + 1 has landed (it was issued a step ago; the loads phase 0 just issued may be in flight)
  //      and, past the barrier, everybody's.  A wave that issues batch t + 2 into the A stage of tile t - 2 has passed
  //      barrier t - 1, which every wave reaches only after its last read of tile t - 2.
  const char *pxb, *pcb, *psb;
  auto seg_base = [&](int q, int step) {
    pxb = reinterpret_cast<const char*>(sg.X[q]) + ((int64_t)step << 7);
    pcb = reinterpret_cast<const char*>(sg.codes[q]) + ((int64_t)step << 5);
    psb = reinterpret_cast<const char*>(sg.scal[q]) + (int64_t)step * 256;
  };
  if constexpr (SEG) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      seg_base(0, t);
      const BatchAddr bt = batch_addr_at(pxb, pcb, psb, t, t);
#pragma unroll
      for (int d = 0; d < kBatch; ++d) issue_one(bt, d);
    }
  } else {
    issue(0, 0, 0);
    issue(1, 1, 1);
  }
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kBatch) : "memory");  // batch 0 landed everywhere, table written
  load_codes(0, sc);
  {
    // substep 0 in full, and the first pair of substep 1 on its way
    float s8[8];
    load_s8(s8, 0, 0);
#pragma unroll
    for (int jp = 0; jp < 2; ++jp) {
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
#pragma unroll
        for (int b = 0; b < 4; ++b) fetch_byte(jj, 2 * jp + jj, 0, b);
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
#pragma unroll
        for (int b = 0; b < 4; ++b) finish_byte(wfa, jj, 2 * jp + jj, b, sc, s8);
    }
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int b = 0; b < 4; ++b) fetch_byte(jj, jj, 1, b);
  }
#pragma unroll
  for (int i = 0; i < MH; ++i) xfa[i] = *reinterpret_cast<const bf16x8_t*>(smem + i * 2048 + x_off[0]);

  constexpr int kDEven = (kBatch + 7) / 8 > 1 ? 2 : 1;
  constexpr int kDOdd = (kBatch - 4 * kDEven + 3) / 4;
  static_assert(4 * kDEven + 4 * kDOdd >= kBatch && kDOdd <= 2 && kDOdd >= 0, "batch does not fit the 8 quarter phases");
  constexpr int kInPhase0 = 2 * (kDEven + kDOdd) < kBatch ? 2 * (kDEven + kDOdd) : kBatch;  // loads phase 0 issues
  int a0 = 0, w0 = 0;
  auto k_step = [&](int64_t adv) {
    const int a1 = (a0 + 1) & 3, a2 = (a0 + 2) & 3;
    const int w1 = w0 == 2 ? 0 : w0 + 1, w2 = w1 == 2 ? 0 : w1 + 1;
    const BatchAddr b = batch_addr_at(pxb, pcb, psb, a2, w2);
    pxb += adv << 7;
    pcb += adv << 5;
    psb += adv * s_stride;
    //    use        use   next operands          builds  finish: pair, scalers, stage, substep   fetch: pair, substep
    phase(xfa, 0, wfa, xfb, a0, 0, 1, wfb, 0, sc, w0, 1, 1, 1, b, 0, kDEven, kDOdd);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kInPhase0) : "memory");
    load_codes(w1, sc_next);
    phase(xfb, 1, wfa, xfa, a0, 1, 0, wfb, 1, sc, w0, 1, 0, 0, b, kInPhase0, kDEven, kDOdd);
    phase(xfa, 0, wfb, xfb, a0, 1, 1, wfa, 0, sc_next, w1, 0, 1, 0, b, kBatch, 0, 0);
    phase(xfb, 1, wfb, xfa, a1, 0, 0, wfa, 1, sc_next, w1, 0, 0, 1, b, kBatch, 0, 0);
#pragma unroll
    for (int j = 0; j < NT; ++j) sc[j] = sc_next[j];
    a0 = a1;
    w0 = w1;
  };
  if constexpr (!SEG) {
    const BatchAddr b2 = batch_addr(2, 0, 0);
    pxb = b2.xb; pcb = b2.cb; psb = b2.sb;
    for (int kt = 0; kt < nk; ++kt) k_step(kt + 3 < nk ? 1 : 0);
  } else {
    int issued = 2;
    for (int q = 0; q < sg.n; ++q) {
      int steps = sg.Kc[q] >> 6;
      if (q == 0) {
        steps -= 2;
        seg_base(0, nk > 2 ? 2 : 1);
      } else {
        set_offsets(sg.Kc[q]);
        seg_base(q, 0);
      }
      if (q == sg.n - 1) steps += 2;
      for (int it = 0; it < steps; ++it) {
        k_step(issued + 1 < nk ? 1 : 0);
        ++issued;
      }
    }
  }

  // the clamped batches issued by the last two steps; and the last MFMAs of the loop (assembly: the compiler does not
  // know they are matrix instructions) have left the pipeline before anything reads their accumulators
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  // ---- adapter: one MFMA step per 32 ranks, operands straight from global memory; lane (l15, lg) holds ranks
  //      rc + 8 lg .. + 7 of weight column / activation row l15 of its tile
  const int n_adapters = SEG ? sg.n : 1;
  for (int ad = 0; ad < n_adapters; ++ad) {
    const uint16_t* __restrict__ lX = SEG ? sg.lX[ad] : g.lX;
    const uint16_t* __restrict__ lW = SEG ? sg.lW[ad] : g.lW;
    const int R = SEG ? sg.R[ad] : g.R;
    if (!(R > 0 && lX != nullptr && (!SPLIT || blockIdx.y == 0))) continue;
    for (int rc = 0; rc < R; rc += 32) {
      const int r0 = rc + 8 * lg;
      const bool in = r0 < R;  // R % 8 == 0: a lane's 8 indices are all in or all out
      bf16x8_t wfr[NT];
      // the requests of half a step first, then their uses: two trips to memory per step (with the scaling between two
      // loads the compiler waited for each of them in turn)
      u32x4_t xraw[MH];
      auto load_x = [&](int ih) {
#pragma unroll
        for (int i = 0; i < MH; ++i) {
          int row = m0 + 16 * (MH * ih + i) + l15;
          row = row < g.M ? row : g.M - 1;
          xraw[i] = u32x4_t{0, 0, 0, 0};
          if (in) xraw[i] = *reinterpret_cast<const u32x4_t*>(lX + (int64_t)row * g.ldlx + r0);
        }
      };
      load_x(0);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        int col = n0 + wv * 64 + 16 * j + l15;
        col = col < g.Nout ? col : g.Nout - 1;
        u32x4_t raw = {0, 0, 0, 0};
        if (in) {
          if (g.lw_row_major) {
            raw = *reinterpret_cast<const u32x4_t*>(lW + (int64_t)col * R + r0);
          } else {
            uint32_t e[8];
#pragma unroll
            for (int d = 0; d < 8; ++d) e[d] = lW[(int64_t)(r0 + d) * g.Nout + col];
#pragma unroll
            for (int d = 0; d < 4; ++d) raw[d] = e[2 * d] | (e[2 * d + 1] << 16);
          }
        }
        wfr[j] = __builtin_bit_cast(bf16x8_t, raw);
      }
#pragma unroll
      for (int ih = 0; ih < 2; ++ih) {
        bf16x8_t xfr[MH];
        if (ih == 1) load_x(1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < MH; ++i) {
          u32x4_t raw = xraw[i];
          if (g.lscale != 1.0f) {
#pragma unroll
            for (int d = 0; d < 4; ++d)
              raw[d] = pack_bf16x2(bits_f32(raw[d] << 16) * g.lscale, bits_f32(raw[d] & 0xffff0000u) * g.lscale);
          }
          xfr[i] = __builtin_bit_cast(bf16x8_t, raw);
        }
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int i = 0; i < MH; ++i)
            acc[j][MH * ih + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wfr[j], xfr[i], acc[j][MH * ih + i], 0, 0, 0);
      }
    }
  }

  // ---- epilogue.  acc[j][i][v] = C[m][n] with m = m0 + 16 i + l15 and n = n0 + 64 wv + 16 j + 4 lg + v.
  if constexpr (SPLIT) {
    // fp32 partial tile straight from the registers: a lane holds four consecutive columns of a row (16 bytes), the
    // four lane groups make the 64 bytes of a weight tile's columns
    if (n0 + wv * 64 >= g.Nout) return;
    float* P = g.part + (int64_t)blockIdx.y * g.M * g.Nout + n0 + wv * 64 + 4 * lg;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int row = m0 + 16 * i + l15;
      if (row >= g.M) continue;
#pragma unroll
      for (int j = 0; j < NT; ++j) *reinterpret_cast<f32x4_t*>(P + (int64_t)row * g.Nout + 16 * j) = acc[j][i];
    }
    return;
  }
  __syncthreads();                      // every wave is done reading the activation ring
  if (n0 + wv * 64 >= g.Nout) return;  // the whole 64-column band of this wave lies outside (no barrier follows)
  {
    // each wave transposes its BM x 64 band through LDS (BM x 128 bytes per wave) and writes whole 128-byte row
    // segments; 16-byte chunk c of row r sits in slot c ^ (r & 7)
    char* band = smem + wv * (BM * 128);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      float b4[4] = {0.f, 0.f, 0.f, 0.f};
      if (g.bias) {
        const u32x2_t bb = *reinterpret_cast<const u32x2_t*>(g.bias + n0 + wv * 64 + 16 * j + 4 * lg);
        b4[0] = bits_f32(bb.x << 16); b4[1] = bits_f32(bb.x & 0xffff0000u);
        b4[2] = bits_f32(bb.y << 16); b4[3] = bits_f32(bb.y & 0xffff0000u);
      }
      float c4[4] = {1.f, 1.f, 1.f, 1.f};
      if (g.cscale) {
        const u32x2_t cc = *reinterpret_cast<const u32x2_t*>(g.cscale + n0 + wv * 64 + 16 * j + 4 * lg);
        c4[0] = bits_f32(cc.x << 16); c4[1] = bits_f32(cc.x & 0xffff0000u);
        c4[2] = bits_f32(cc.y << 16); c4[3] = bits_f32(cc.y & 0xffff0000u);
      }
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int r = 16 * i + l15;
        u32x2_t o;
        o.x = pack_bf16x2((acc[j][i][0] + b4[0]) * c4[0], (acc[j][i][1] + b4[1]) * c4[1]);
        o.y = pack_bf16x2((acc[j][i][2] + b4[2]) * c4[2], (acc[j][i][3] + b4[3]) * c4[3]);
        *reinterpret_cast<u32x2_t*>(band + r * 128 + (((2 * j + (lg >> 1)) ^ (r & 7)) << 4) + 8 * (lg & 1)) = o;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int c = lane & 7;
    uint16_t* crow = g.C + n0 + wv * 64 + 8 * c;
#pragma unroll 8
    for (int t = 0; t < BM / 8; ++t) {
      const int r = 8 * t + (lane >> 3);
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(band + r * 128 + ((c ^ (r & 7)) << 4));
      if (m0 + r < g.M) *reinterpret_cast<u32x4_t*>(crow + (int64_t)(m0 + r) * g.Nout) = v;
    }
  }
#endif
}

// C[m][n] = bf16((sum over slices of part[s][m][n] + bias[n]) * cscale[n]); a thread takes 8 consecutive columns.
__global__ __launch_bounds__(256) void nf4_gemm_rs_reduce_kernel(const float* __restrict__ part, int splits, int64_t mn,
                                                                 int Nout, const uint16_t* __restrict__ bias,
                                                                 const uint16_t* __restrict__ cscale, uint16_t* __restrict__ C) {
  const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (e >= mn) return;
  float v[8];
  {
    const f32x4_t a = *reinterpret_cast<const f32x4_t*>(part + e), b = *reinterpret_cast<const f32x4_t*>(part + e + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  for (int sidx = 1; sidx < splits; ++sidx) {
    const float* p = part + (int64_t)sidx * mn + e;
    const f32x4_t a = *reinterpret_cast<const f32x4_t*>(p), b = *reinterpret_cast<const f32x4_t*>(p + 4);
    v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w; v[4] += b.x; v[5] += b.y; v[6] += b.z; v[7] += b.w;
  }
  const int n = (int)(e % Nout);  // Nout % 8 == 0: the 8 columns share a row
  if (bias) {
    const u32x4_t bb = *reinterpret_cast<const u32x4_t*>(bias + n);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      v[2 * d] += bits_f32(bb[d] << 16);
      v[2 * d + 1] += bits_f32(bb[d] & 0xffff0000u);
    }
  }
  if (cscale) {
    const u32x4_t cc = *reinterpret_cast<const u32x4_t*>(cscale + n);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      v[2 * d] *= bits_f32(cc[d] << 16);
      v[2 * d + 1] *= bits_f32(cc[d] & 0xffff0000u);
    }
  }
  u32x4_t o;
#pragma unroll
  for (int d = 0; d < 4; ++d) o[d] = pack_bf16x2(v[2 * d], v[2 * d + 1]);
  *reinterpret_cast<u32x4_t*>(C + e) = o;
}

template <int BM, int MODE, bool SPLIT, bool SEG = false>
int launch_rs(RsArgs& g, int splits, hipStream_t s, const RsSegs* segs = nullptr) {
  using L = RsLayout<BM>;
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.Nout + kBN - 1) / kBN;
  // Full tiles of a single layer run the 16 x 16 x 32 form of the loop: 1 - 5 % faster there (the part clocks 15 % higher
  // on that MFMA shape, and the loop needs 15 % more cycles for the 64 extra MFMA issues of a k-step); with 128-row tiles
  // it is 1 - 5 % slower and with segments it spills, so those keep the 32 x 32 x 16 form.
  constexpr bool kMfma16 = BM == 256 && !SPLIT && !SEG;
  const void* fn;
  if constexpr (kMfma16)
    fn = reinterpret_cast<const void*>(&nf4_gemm_rs16_kernel<BM, MODE, SPLIT, SEG>);
  else
    fn = reinterpret_cast<const void*>(&nf4_gemm_rs_kernel<BM, MODE, SPLIT, SEG>);
  // the LDS limit is a per-device attribute of the function: set it for the current device once (a race only repeats the call)
  static bool attr_set[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
  if (dev < 0 || !attr_set[dev]) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, L::kTotal);
    if (e != hipSuccess)
      return fail(TTAMD_ELAUNCH, "nf4_gemm_rs: cannot reserve %d bytes of LDS: %s", L::kTotal, hipGetErrorString(e));
    if (dev >= 0) attr_set[dev] = true;
  }
  static const RsSegs no_segs = {};
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)splits), block(256);
  if constexpr (kMfma16)
    nf4_gemm_rs16_kernel<BM, MODE, SPLIT, SEG><<<grid, block, L::kTotal, s>>>(g, segs ? *segs : no_segs);
  else
    nf4_gemm_rs_kernel<BM, MODE, SPLIT, SEG><<<grid, block, L::kTotal, s>>>(g, segs ? *segs : no_segs);
  return check_launch("nf4_gemm_rs");
}

// Slices of the contraction for a launch that would leave half of the chip or more idle: enough to reach about one
// workgroup per CU, at least four k-steps (256 elements) each, at most 16.  1 = do not split.
int choose_splits(int64_t M, int64_t Nout, int64_t Kc) {
  const int64_t tiles = ((M + 127) / 128) * ((Nout + kBN - 1) / kBN);  // small launches use 128-row tiles
  if (tiles > 128) return 1;
  if (tiles > 64 && Kc < 4096) return 1;  // two slices of a short contraction: the reduction costs what the slicing gains
  int64_t sp = 256 / tiles;
  const int64_t by_k = (Kc / 64) / 4;
  sp = sp < by_k ? sp : by_k;
  sp = sp < 16 ? sp : 16;
  return sp < 2 ? 1 : (int)sp;
}

}  // namespace

// Bytes of workspace run_gemm_rs can use: slices of the contraction for a small launch, or the expanded copy of the
// weight for a launch of many tokens (nf4_gemm_dense.hip); the two cases exclude each other.  0: it would use none.
size_t gemm_rs_workspace_bytes(int64_t M, int64_t Nout, int64_t Kc) {
  const int sp = choose_splits(M, Nout, Kc);
  if (sp > 1) return (size_t)sp * (size_t)M * (size_t)Nout * sizeof(float);
  return dense_workspace_bytes(M, Nout, Kc);
}

// Entry used by the C-ABI wrappers.  `workspace` may be null: then small launches are not sliced.  The rows of the
// adapter activation lX are ldlx elements apart (a group keeps its members' activations side by side).
int run_gemm_rs(const void* X, const uint8_t* codes, const void* scal, int mode, const void* lX, int ldlx, const void* lW,
                bool lw_row_major, int R, float lscale, const void* bias, const void* cscale, void* C, int64_t M, int64_t Nout,
                int64_t Kc, void* workspace, size_t workspace_bytes, hipStream_t s) {
  // per-lane byte offsets inside the kernel are 32-bit: the weight must fit them, and a token dimension too long for
  // them is cut into row ranges (multiples of the 256-row tile) that are launched one after the other
  TT_REQUIRE(Nout * Kc / 2 < (int64_t(1) << 32) && Nout * (Kc / 64) * 4 < (int64_t(1) << 32) && Kc * 2 * 256 < (int64_t(1) << 32),
             "nf4_gemm: weight too large for 32-bit offsets (Nout=%lld Kc=%lld)", (long long)Nout, (long long)Kc);
  const int64_t max_rows = (((int64_t(1) << 32) - 1) / (Kc * 2)) / 256 * 256;
  if (M > max_rows) {
    for (int64_t r0 = 0; r0 < M; r0 += max_rows) {
      const int64_t rows = M - r0 < max_rows ? M - r0 : max_rows;
      const int rc = run_gemm_rs(reinterpret_cast<const uint16_t*>(X) + r0 * Kc, codes, scal, mode,
                                 lX ? reinterpret_cast<const uint16_t*>(lX) + r0 * ldlx : nullptr, ldlx, lW, lw_row_major, R, lscale, bias,
                                 cscale, reinterpret_cast<uint16_t*>(C) + r0 * Nout, rows, Nout, Kc, nullptr, 0, s);
      if (rc != TTAMD_OK) return rc;
    }
    return TTAMD_OK;
  }
  // many tokens and room for the expanded weight: expand once, then the plain bf16 GEMM
  if (workspace != nullptr && dense_path_applies(M, Nout, Kc) && workspace_bytes >= dense_workspace_bytes(M, Nout, Kc))
    return run_gemm_dense(X, codes, scal, mode, lX, ldlx, lW, lw_row_major, R, lscale, bias, cscale, C, M, Nout, Kc, workspace, s);
  RsArgs g;
  g.X = reinterpret_cast<const uint16_t*>(X);
  g.codes = codes;
  g.scal = reinterpret_cast<const float*>(scal);
  g.lX = reinterpret_cast<const uint16_t*>(lX);
  g.lW = reinterpret_cast<const uint16_t*>(lW);
  g.bias = reinterpret_cast<const uint16_t*>(bias);
  g.cscale = reinterpret_cast<const uint16_t*>(cscale);
  g.C = reinterpret_cast<uint16_t*>(C);
  g.M = (int)M; g.Nout = (int)Nout; g.Kc = (int)Kc; g.R = R;
  g.lw_row_major = lw_row_major ? 1 : 0;
  g.ldlx = ldlx;
  g.lscale = lscale;
  g.part = nullptr;
  g.ksteps = 0;
  const int splits = choose_splits(M, Nout, Kc);
  if (splits > 1 && workspace != nullptr && workspace_bytes >= gemm_rs_workspace_bytes(M, Nout, Kc)) {
    TT_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15u) == 0, "nf4_gemm: workspace must be 16-byte aligned");
    g.part = reinterpret_cast<float*>(workspace);
    g.ksteps = (int)(((Kc >> 6) + splits - 1) / splits);
    const int used = (int)(((Kc >> 6) + g.ksteps - 1) / g.ksteps);  // slices that hold at least one k-step
    int rc = mode == 1 ? launch_rs<128, 1, true>(g, used, s)
             : mode == 2 ? launch_rs<128, 2, true>(g, used, s)
                         : launch_rs<128, 0, true>(g, used, s);
    if (rc != TTAMD_OK) return rc;
    const int64_t mn = M * Nout;
    nf4_gemm_rs_reduce_kernel<<<dim3((unsigned)((mn / 8 + 255) / 256)), dim3(256), 0, s>>>(g.part, used, mn, (int)Nout, g.bias,
                                                                                          g.cscale, g.C);
    return check_launch("nf4_gemm_rs_reduce");
  }
  const int64_t tiles256 = ((M + 255) / 256) * ((Nout + kBN - 1) / kBN);
  const bool big = tiles256 >= 256;
  if (mode == 1) return big ? launch_rs<256, 1, false>(g, 1, s) : launch_rs<128, 1, false>(g, 1, s);
  if (mode == 2) return big ? launch_rs<256, 2, false>(g, 1, s) : launch_rs<128, 2, false>(g, 1, s);
  return big ? launch_rs<256, 0, false>(g, 1, s) : launch_rs<128, 0, false>(g, 1, s);
}


// Grad-input of a group of layers with a common input, as one GEMM over the concatenated contraction:
//   gx[M, K] = sum_i gy_i[M, N_i] . D(W_i)[N_i, K] + gh_i[M, R_i] . A_i[R_i, K]
// with the members' transposed copies (codes [K, N_i / 2], per-element scalers [K / 64, N_i]); gh_i = columns
// [r_off[i], r_off[i + 1]) of gh_cat.  The sum over members is taken in fp32, before the one rounding to bf16.
int run_gemm_rs_group_dx(const GroupDx& d, const void* gh_cat, void* gx, hipStream_t s) {
  TT_REQUIRE(d.n >= 1 && d.n <= kGroupMax, "nf4_group_dx: %d members", d.n);
  RsSegs sg = {};
  sg.n = d.n;
  int64_t max_n = 0;
  int first = 0;  // the widest member goes first: the kernel takes its first two batches from segment 0
  for (int i = 0; i < d.n; ++i) {
    TT_REQUIRE(d.N[i] > 0 && d.N[i] % 64 == 0, "nf4_group_dx: N (%lld) must be a positive multiple of 64", (long long)d.N[i]);
    TT_REQUIRE(aligned16(d.gy[i]) && aligned16(d.codes_t[i]) && aligned16(d.scal_t[i]), "nf4_group_dx: pointers must be 16-byte aligned");
    if (d.N[i] > max_n) {
      max_n = d.N[i];
      first = i;
    }
  }
  if (max_n < 128) return fail(TTAMD_EUNSUPPORTED, "nf4_group_dx: the widest member must have at least 128 outputs (has %lld)", (long long)max_n);
  for (int k = 0; k < d.n; ++k) {
    const int i = k == 0 ? first : (k <= first ? k - 1 : k);  // first, then the others in their order
    sg.X[k] = d.gy[i];
    sg.codes[k] = d.codes_t[i];
    sg.scal[k] = d.scal_t[i];
    sg.lX[k] = d.rank[i] > 0 ? reinterpret_cast<const uint16_t*>(gh_cat) + d.r_off[i] : nullptr;
    sg.lW[k] = d.lora_a[i];
    sg.Kc[k] = (int)d.N[i];
    sg.R[k] = d.rank[i];
  }
  // per-lane byte offsets inside the kernel are 32-bit
  if (!(d.K * max_n / 2 < (int64_t(1) << 32) && d.K / 64 * max_n * 4 < (int64_t(1) << 32) && d.M * max_n * 2 < (int64_t(1) << 32)))
    return fail(TTAMD_EUNSUPPORTED, "nf4_group_dx: operands too large for 32-bit offsets (M=%lld K=%lld N=%lld)", (long long)d.M,
                (long long)d.K, (long long)max_n);
  RsArgs g = {};
  g.C = reinterpret_cast<uint16_t*>(gx);
  g.M = (int)d.M; g.Nout = (int)d.K;
  g.lw_row_major = 0;
  g.ldlx = d.r_off[d.n];
  g.lscale = 1.0f;
  const int64_t tiles256 = ((d.M + 255) / 256) * ((d.K + kBN - 1) / kBN);
  return tiles256 >= 256 ? launch_rs<256, 1, false, true>(g, 1, s, &sg) : launch_rs<128, 1, false, true>(g, 1, s, &sg);
}

}  // namespace ttamd
