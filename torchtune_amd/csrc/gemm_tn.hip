// Weight gradient of a linear layer over many tokens: C[N, K] = A[M, N]^T . B[M, K] for bf16 A = gy and B = x as they lie in
// memory (rows = tokens), the third matmul of FakeQuantizedLinear's training step (autograd of F.linear(fq(x), fq(W)),
// torchao; reached from recipes/qat_single_device.py:378-386).  The contraction runs over the rows of both operands, so
// neither has the 8 consecutive contraction elements per lane that v_mfma_f32_16x16x32_bf16 wants: the LDS transposes them
// (ds_read_b64_tr_b16 returns to lane i of a 16-lane group column i of the four rows the group points at).
//
// Skeleton of nf4_gemm_dense.hip: workgroup = 8 waves (two per SIMD), tile 256 x 256 of C, step = 32 rows of A and B, both
// tiles (32 rows x 512 bytes each) into a ring of four LDS stages by direct-to-LDS loads; wave (wm, wn) owns rows
// [128 wm, +128) x columns [64 wn, +64) of the tile (128 accumulators per lane); the two waves of a SIMD run half a step
// apart, one in its MFMA part while the other requests loads and reads operands, swapping at workgroup barriers.
// LDS layout of a stage: row r of the 32 at r * 512, its 16-byte chunk c in slot c ^ (2 (r % 4)) ^ (8 ((r / 8) % 2)) -
// applied on the global-address side of the loads.  The first term puts the four rows a 16-lane group reads together on
// disjoint banks; the second moves the rows of the odd 16-lane groups 128 bytes aside, so that the two groups the LDS
// serves in one pass (lanes 0 - 31, then 32 - 63; 64 banks of 4 bytes) use different halves of the banks (without it
// every transposing read takes two passes: SQ_LDS_BANK_CONFLICT = half of SQ_LDS_IDX_ACTIVE).
//
// Last partial round.  256 CUs take 256 tiles at a time; a launch of, say, 3.5 rounds of tiles leaves half the chip idle
// for the length of one tile (220 us at 8192 tokens).  With a workspace the tiles beyond the last whole round have their
// contraction cut into 2 - 8 slices, one workgroup per tile and slice, so that the last round fills the chip with
// shorter pieces of work; each leaves its tile as fp32 in the workspace and gemm_tn_reduce_kernel adds the slices of a
// tile in slice order (deterministic), rounds once and stores through the same epilogue.  Taken where the time saved
// pays for the 256 KiB per tile and slice that go to memory and back (long contractions: training token counts).
#include <type_traits>

#include "common.h"
#include "group.h"
#include "nf4_math.h"

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

// One launch serves the weight gradients of up to kGroupMax layers with a common input (q / k / v, gate / up): they share
// B and differ in A and C; row tiles [tile_end[i - 1], tile_end[i]) of the stacked outputs belong to member i.
struct TnArgs {
  const uint16_t* A[kGroupMax];  // [M, N[i]] bf16
  uint16_t* C[kGroupMax];        // [N[i], K] bf16
  int N[kGroupMax], tile_end[kGroupMax];
  int n;
  const uint16_t* B;  // [M, K] bf16
  int M, K;
  int tiles_n, tiles_k;  // tiles_n: all members
  // workgroups [0, full_tiles) run tiles [0, full_tiles) over the whole contraction; workgroup full_tiles + u runs slice
  // u / tail_tiles of tile full_tiles + u % tail_tiles and leaves it in slabs (slices == 1: no tile is cut, tail_tiles == 0)
  int full_tiles, tail_tiles, slices;
  float* slabs;  // [tail_tiles][slices][NT * MT][512 threads][4] fp32
};

constexpr int kTnStage = 32768;  // 32 rows x 512 bytes of A, then the same of B
constexpr int kTnLds = 4 * kTnStage;

constexpr int kTnMT = 8, kTnNT = 4;  // 16 x 16 MFMA tiles per wave: MT along the rows of C (columns of A), NT along its columns

// Tile `id` of a launch: the member it belongs to and its first row (within the member) and column.
__device__ __forceinline__ void tn_locate(const TnArgs& g, int id, int& which, int& n0, int& k0) {
  int tile_n, tile_k;
  // Tile ids are dealt round-robin to the 8 XCDs (one L2 each), 32 at a time.  Where the grid divides into blocks of
  // 4 x 8 tiles, eight at a time, an XCD works on one block at a time: 4 + 8 operand panels of 256 columns through its L2
  // per round (bands of two row tiles walked column by column would be 2 + 16); the XCDs of a round take different rows of
  // the same eight columns.
  // The blocks beyond the last whole eight (the tiles of a last partial round, ids from 256 * rounds on) follow in order.
  const int super_rows = g.tiles_n >> 2, runs = g.tiles_k >> 3;
  if ((g.tiles_n & 3) == 0 && (g.tiles_k & 7) == 0) {
    const int whole = (super_rows * runs) & ~7;  // blocks in whole rounds
    int block, t;
    if (id < 32 * whole) {
      const int xcd = id & 7, slot = id >> 3;
      block = (slot >> 5) * 8 + xcd;
      t = slot & 31;
    } else {
      block = whole + ((id - 32 * whole) >> 5);
      t = id & 31;
    }
    tile_n = 4 * (block % super_rows) + (t & 3);
    tile_k = 8 * (block / super_rows) + (t >> 2);
  } else if ((g.tiles_n & 7) == 0) {
    // otherwise every XCD gets a band of row tiles and walks it column by column
    const int xcd = id & 7, slot = id >> 3, band = g.tiles_n >> 3;
    tile_n = xcd * band + slot % band;
    tile_k = slot / band;
  } else {
    tile_n = id / g.tiles_k;
    tile_k = id % g.tiles_k;
  }
  which = 0;  // uniform over the workgroup
#pragma unroll
  for (int q = 0; q < kGroupMax - 1; ++q)
    if (q < g.n - 1 && tile_n >= g.tile_end[q]) which = q + 1;
  n0 = (tile_n - (which ? g.tile_end[which - 1] : 0)) * 256;
  k0 = tile_k * 256;
}

// acc[j][i][v] = C[n][k], n = n0 + 128 wm + 16 i + l15, k = k0 + 64 wn + 16 j + 4 g4 + v.  Each wave transposes its
// 128 x 64 band through LDS (128 KiB for the eight waves) and writes whole 128-byte row segments.
__device__ __forceinline__ void tn_store_tile(const f32x4_t (&acc)[kTnNT][kTnMT], char* smem, uint16_t* C, int K, int n0, int k0) {
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wv >> 2, wn = wv & 3;
  const int l15 = lane & 15, g4 = lane >> 4;
  char* band = smem + wv * 16384;  // 128 rows x 128 bytes
#pragma unroll
  for (int j = 0; j < kTnNT; ++j)
#pragma unroll
    for (int i = 0; i < kTnMT; ++i) {
      const int r = 16 * i + l15;
      u32x2_t o;
      o.x = pack_bf16x2(acc[j][i][0], acc[j][i][1]);
      o.y = pack_bf16x2(acc[j][i][2], acc[j][i][3]);
      *reinterpret_cast<u32x2_t*>(band + r * 128 + (((2 * j + (g4 >> 1)) ^ (r & 7)) << 4) + 8 * (g4 & 1)) = o;
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int c = lane & 7;
  uint16_t* crow = C + k0 + wn * 64 + 8 * c;
  const int nrow0 = n0 + 128 * wm;
#pragma unroll 8
  for (int t = 0; t < 16; ++t) {
    const int r = 8 * t + (lane >> 3);
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(band + r * 128 + ((c ^ (r & 7)) << 4));
    *reinterpret_cast<u32x4_t*>(crow + (int64_t)(nrow0 + r) * K) = v;
  }
}

// Steps [begin, end) of slice `slice` of `slices` over nk steps (every slice non-empty when slices <= nk).
__device__ __forceinline__ int tn_slice_begin(int slice, int slices, int nk) { return (int)(((int64_t)slice * nk) / slices); }

__global__ __launch_bounds__(512) void gemm_tn_kernel(const TnArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int MT = kTnMT, NT = kTnNT;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wv >> 2, wn = wv & 3;
  const int l15 = lane & 15, g4 = lane >> 4;

  const int nk_all = g.M >> 5;  // steps of 32 rows
  int id = blockIdx.x, t_begin = 0, nk = nk_all;  // this workgroup runs steps [t_begin, nk)
  int slab = -1;
  if (id >= g.full_tiles) {
    const int u = id - g.full_tiles;
    const int slice = u / g.tail_tiles, tl = u - slice * g.tail_tiles;
    id = g.full_tiles + tl;
    t_begin = tn_slice_begin(slice, g.slices, nk_all);
    nk = tn_slice_begin(slice + 1, g.slices, nk_all);
    slab = tl * g.slices + slice;
  }
  int which, n0, k0;
  tn_locate(g, id, which, n0, k0);
  const uint16_t* const A = g.A[which];
  uint16_t* const C = g.C[which];
  const int N = g.N[which];

  // ---- loads: per step and wave two instructions for A (rows 4 wv .. + 3 of the 32, two rows of 512 bytes each) and two
  //      for B; lane l of an instruction fetches chunk (l % 32) ^ (2 (row % 4)) ^ (8 ((row / 8) % 2)) of row l / 32 of its pair
  uint32_t a_off[2], b_off[2];
#pragma unroll
  for (int d = 0; d < 2; ++d) {
    const int rl = 4 * wv + 2 * d + (lane >> 5);
    const int chunk = (lane & 31) ^ ((rl & 3) << 1) ^ (((rl >> 3) & 1) << 3);
    a_off[d] = (uint32_t)rl * (uint32_t)N * 2u + (uint32_t)n0 * 2u + (uint32_t)chunk * 16u;
    b_off[d] = (uint32_t)rl * (uint32_t)g.K * 2u + (uint32_t)k0 * 2u + (uint32_t)chunk * 16u;
  }
  // The two requests of an operand name their LDS destinations through the instruction's offset field, which moves the
  // global address along with the LDS address: one M0 write per operand and step.  The second request therefore carries
  // offset 1024 and a lane offset that is 1024 short; both are lifted by 1024 against a base lowered by as much, so that
  // neither is negative.
  const uint32_t a_v0 = a_off[0] + 1024u, a_v1 = a_off[1], b_v0 = b_off[0] + 1024u, b_v1 = b_off[1];
  const char* const a_base = reinterpret_cast<const char*>(A) - 1024;
  const char* const b_base = reinterpret_cast<const char*>(g.B) - 1024;
  const int64_t a_step = (int64_t)N * 64, b_step = (int64_t)g.K * 64;  // 32 rows of the operand
  const uint32_t lds0 = (uint32_t)(uintptr_t)TT_LDS_PTR(smem);
  auto request = [&](const char* ab, const char* bb, int stage) {
    const uint32_t st = lds0 + stage * kTnStage + wv * 2048;
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, %2\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:1024"
                 ::"v"(a_v0), "v"(a_v1), "s"(ab), "s"(st) : "memory", "m0");
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, %2\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:1024"
                 ::"v"(b_v0), "v"(b_v1), "s"(bb), "s"(st + 16384u) : "memory", "m0");
  };
  auto issue = [&](int t, int stage) {  // past the end: the last step again (the waits count a fixed number in flight)
    const int tk = t < nk ? t : nk - 1;
    request(a_base + (int64_t)tk * a_step, b_base + (int64_t)tk * b_step, stage);
  };

  // ---- operand reads.  Lane (l15, g4) of ds_read_b64_tr_b16 points at row 8 g4 + l15 / 4 (+ 4 for the second half of the
  //      operand), columns 4 (l15 % 4) .. + 3 of a 16-column group e, and receives column l15 of that group for rows
  //      8 g4 .. + 3 (+ 4): with both halves the 8 contraction elements of an MFMA operand.  Group e of a row with
  //      row % 4 = q and (row / 8) % 2 = sb sits at byte 32 ((e ^ q) ^ 4 sb) of the row; sb = g4 % 2 for both halves of an
  //      operand.  A groups of this wave: 8 wm + i (ra[i % 4] + ah[i / 4]); B groups: 4 wn + j.
  //      The reads go through the compiler's builtin, so that everything of an address that is the same for all lanes
  //      (stage, half, group of four) rides in the instruction's offset field: eight address additions per two steps.
  //      With one register operand per read, as hand-written assembly takes it, every read cost a vector-ALU addition
  //      of its own (24 per step), issued from the memory part of one wave into the MFMA part of the other wave of
  //      its SIMD.
  int ra[4], rb[4], ah[2];  // byte offsets from the start of a stage
  {
    const int q = (l15 >> 2) & 3, sb = g4 & 1;
    const int rowbase = (8 * g4 + (l15 >> 2)) * 512 + 8 * (l15 & 3);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ra[e] = rowbase + 32 * (8 * wm) + 32 * (e ^ q);
      rb[e] = 16384 + rowbase + 32 * (4 * (wn ^ sb)) + 32 * (e ^ q);
    }
    ah[0] = 128 * sb;
    ah[1] = 128 * (1 - sb);
  }
  typedef short s16x4_t __attribute__((ext_vector_type(4)));
  auto tr16 = [&](const char* at) {
    return __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)(at)));
  };

  f32x4_t acc[NT][MT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[j][i][v] = 0.f;

  u32x2_t alo[MT], ahi[MT], blo[NT], bhi[NT];
  // pa[e], pb[e]: the lane's addresses in the even stage of the current pair; `odd` adds one stage as a constant
  auto read_step = [&](const char* const (&pa)[4], const char* const (&pb)[4], int odd) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      blo[j] = tr16(pb[j] + odd * kTnStage);
      bhi[j] = tr16(pb[j] + odd * kTnStage + 2048);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      alo[i] = tr16(pa[i & 3] + ah[i >> 2] + odd * kTnStage);
      ahi[i] = tr16(pa[i & 3] + ah[i >> 2] + odd * kTnStage + 2048);
    }
  };
  auto compute = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const u32x4_t aop = {alo[i].x, alo[i].y, ahi[i].x, ahi[i].y};
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const u32x4_t bop = {blo[j].x, blo[j].y, bhi[j].x, bhi[j].y};
        acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, bop), __builtin_bit_cast(bf16x8_t, aop),
                                                           acc[j][i], 0, 0, 0);
      }
    }
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- pipeline, as in nf4_gemm_dense.hip: memory part M(t) / barrier / compute part C(t) / barrier, the waves with wm = 1
  //      one barrier behind.  M(t) requests step t + 3 (four loads) into the stage step t - 1 was read from and reads the
  //      operands of step t.  At the end of M(t) a wave's own loads of step t + 1 must have landed (the other waves read
  //      them after the next barrier): they came from M(t - 2), newer are the 4 + 4 loads of M(t - 1) and M(t).  Stages
  //      are counted from the workgroup's first step (a slice may start anywhere); the loop takes two steps per trip.
  issue(t_begin, 0);
  issue(t_begin + 1, 1);
  issue(t_begin + 2, 2);
  asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");  // the first step landed everywhere
  if (wm == 1) asm volatile("s_barrier" ::: "memory");
  // one copy of the loop per wave group: the two differ in one wait, and a branch per step costs 2 - 4 %
  auto main_loop = [&](auto lgkm) {
    constexpr bool kLgkm = decltype(lgkm)::value;
    // what the waves with wm = 1 read in a memory part is overwritten by requests the waves with wm = 0 issue right after
    // the next barrier: they let their reads complete before they pass it (the others' reads have a whole interval more)
    auto end_of_memory_part = [&]() {
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kLgkm)
        asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      else
        asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
    };
    int t = t_begin;
    // four steps at a time (the ring has four stages: every stage is then a constant of the instructions), as long as
    // all of their requests stay inside the operands; the rest two by two with a running stage and clamped requests
    {
      const char* pa0[4];
      const char* pb0[4];
      const char* pa2[4];
      const char* pb2[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        pa0[e] = smem + ra[e];
        pb0[e] = smem + rb[e];
        pa2[e] = smem + 2 * kTnStage + ra[e];
        pb2[e] = smem + 2 * kTnStage + rb[e];
      }
      // the requests of the block run three steps ahead of t, on pointers of their own
      const char* ap = a_base + (int64_t)(t + 3) * a_step;
      const char* bp = b_base + (int64_t)(t + 3) * b_step;
      auto next = [&](int stage) {
        request(ap, bp, stage);
        ap += a_step;
        bp += b_step;
      };
      for (; t + 8 <= nk; t += 4) {
        next(3);
        read_step(pa0, pb0, 0);
        end_of_memory_part();
        compute();
        next(0);
        read_step(pa0, pb0, 1);
        end_of_memory_part();
        compute();
        next(1);
        read_step(pa2, pb2, 0);
        end_of_memory_part();
        compute();
        next(2);
        read_step(pa2, pb2, 1);
        end_of_memory_part();
        compute();
      }
    }
    int ws = 0;  // stage of the even step of the current pair: 0 or 2 (whole rounds of the ring lie behind)
    for (; t + 1 < nk; t += 2) {
      const char* pa[4];
      const char* pb[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        pa[e] = smem + ws * kTnStage + ra[e];
        pb[e] = smem + ws * kTnStage + rb[e];
      }
      issue(t + 3, (ws + 3) & 3);
      read_step(pa, pb, 0);
      end_of_memory_part();
      compute();
      issue(t + 4, ws);
      read_step(pa, pb, 1);
      end_of_memory_part();
      compute();
      ws ^= 2;
    }
    if (t < nk) {  // an odd number of steps: the last one on its own
      const char* pa[4];
      const char* pb[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        pa[e] = smem + ws * kTnStage + ra[e];
        pb[e] = smem + ws * kTnStage + rb[e];
      }
      issue(t + 3, (ws + 3) & 3);
      read_step(pa, pb, 0);
      end_of_memory_part();
      compute();
    }
  };
  if (wm == 1)
    main_loop(std::true_type{});
  else
    main_loop(std::false_type{});
  if (wm == 0) asm volatile("s_barrier" ::: "memory");
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the clamped requests of the last steps

  // ---- a slice leaves its partial tile as fp32, in the accumulators' own order: 16 bytes per lane, whole lines per wave
  if (slab >= 0) {
    f32x4_t* dst = reinterpret_cast<f32x4_t*>(g.slabs) + (int64_t)slab * (NT * MT * 512) + tid;
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < MT; ++i) dst[(j * MT + i) * 512] = acc[j][i];
    return;
  }
  // ---- epilogue
  __syncthreads();
  tn_store_tile(acc, smem, C, g.K, n0, k0);
#endif
}

// Adds the slices of one tail tile in slice order and stores the tile (one workgroup per tile, the lanes as in gemm_tn_kernel).
__global__ __launch_bounds__(512) void gemm_tn_reduce_kernel(const TnArgs g) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int MT = kTnMT, NT = kTnNT;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x;
  const int tl = blockIdx.x;
  int which, n0, k0;
  tn_locate(g, g.full_tiles + tl, which, n0, k0);
  f32x4_t acc[NT][MT];
  const f32x4_t* src = reinterpret_cast<const f32x4_t*>(g.slabs) + (int64_t)tl * g.slices * (NT * MT * 512) + tid;
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[j][i] = __builtin_nontemporal_load(src + (j * MT + i) * 512);
  for (int sl = 1; sl < g.slices; ++sl) {
    src += NT * MT * 512;
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const f32x4_t v = __builtin_nontemporal_load(src + (j * MT + i) * 512);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[j][i][e] += v[e];
      }
  }
  tn_store_tile(acc, smem, g.C[which], g.K, n0, k0);
#endif
}

}  // namespace

bool gemm_tn_applies(int64_t M, int64_t N, int64_t K) {
  if (M < 32 || M % 32 != 0 || N <= 0 || K <= 0 || N % 256 != 0 || K % 256 != 0) return false;
  // per-lane byte offsets inside the kernel are 32-bit: a step of 32 rows of either operand
  return N * 2 * 32 < (int64_t(1) << 31) && K * 2 * 32 < (int64_t(1) << 31) && (N / 256) * (K / 256) < (int64_t(1) << 31);
}

}  // namespace ttamd

using namespace ttamd;

extern "C" int ttamd_gemm_tn_applies(int64_t M, int64_t N, int64_t K) { return gemm_tn_applies(M, N, K) ? 1 : 0; }

namespace {
// How the tiles beyond the last whole round of 256 are cut.  A tile of nk steps takes about 0.8 us per step; cutting the
// tail's contraction into `slices` saves (1 - 1 / slices) of that once per launch and costs a reduce launch plus
// 256 KiB per tile and slice written and read back (about 0.1 us each at the rate such a burst moves).  Taken when the
// saving is at least one and a half times the cost; slices of fewer than 32 steps are not made.
struct TnPlan {
  int full_tiles, tail_tiles, slices;
};
constexpr int kTnChipTiles = 256;
TnPlan plan_tn(int64_t tiles, int64_t nk) {
  const int tail = (int)(tiles % kTnChipTiles);
  TnPlan none = {(int)tiles, 0, 1};
  if (tail == 0) return none;
  int slices = kTnChipTiles / tail;
  slices = slices > 8 ? 8 : slices;
  while (slices > 1 && nk / slices < 32) --slices;
  if (slices < 2) return none;
  const double saved = 0.8 * (double)nk * (1.0 - 1.0 / slices);
  const double cost = 16.0 + 0.105 * (double)tail * slices;
  if (saved < 1.5 * cost) return none;
  return TnPlan{(int)(tiles - tail), tail, slices};
}
size_t tn_slab_bytes(const TnPlan& p) { return (size_t)p.tail_tiles * (p.slices > 1 ? p.slices : 0) * 256 * 256 * sizeof(float); }

int launch_gemm_tn(TnArgs& g, void* workspace, size_t workspace_bytes, hipStream_t s) {
  const int64_t tiles = (int64_t)g.tiles_n * g.tiles_k;
  TnPlan plan = plan_tn(tiles, g.M >> 5);
  if (plan.slices > 1 && (workspace == nullptr || workspace_bytes < tn_slab_bytes(plan))) plan = TnPlan{(int)tiles, 0, 1};
  TT_REQUIRE(plan.slices == 1 || aligned16(workspace), "gemm_tn: workspace must be 16-byte aligned");
  g.full_tiles = plan.full_tiles;
  g.tail_tiles = plan.tail_tiles;
  g.slices = plan.slices;
  g.slabs = reinterpret_cast<float*>(workspace);
  const int64_t units = (int64_t)plan.full_tiles + (int64_t)plan.tail_tiles * (plan.slices > 1 ? plan.slices : 0);
  // the LDS limit is a per-device attribute of the function: set it for the current device once (a race only repeats the call)
  static bool attr_set[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
  if (dev < 0 || !attr_set[dev]) {
    for (const void* fn : {reinterpret_cast<const void*>(&gemm_tn_kernel), reinterpret_cast<const void*>(&gemm_tn_reduce_kernel)}) {
      hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kTnLds);
      if (e != hipSuccess) return fail(TTAMD_ELAUNCH, "gemm_tn: cannot reserve %d bytes of LDS: %s", kTnLds, hipGetErrorString(e));
    }
    if (dev >= 0) attr_set[dev] = true;
  }
  gemm_tn_kernel<<<dim3((unsigned)units), dim3(512), kTnLds, s>>>(g);
  if (int rc = check_launch("gemm_tn")) return rc;
  if (plan.slices > 1) {
    gemm_tn_reduce_kernel<<<dim3((unsigned)plan.tail_tiles), dim3(512), kTnLds, s>>>(g);
    return check_launch("gemm_tn_reduce");
  }
  return TTAMD_OK;
}
}  // namespace

extern "C" size_t ttamd_gemm_tn_workspace_bytes(int64_t M, int64_t n_total, int64_t K) {
  if (M < 32 || n_total <= 0 || K <= 0 || n_total % 256 != 0 || K % 256 != 0) return 0;
  return tn_slab_bytes(plan_tn((n_total / 256) * (K / 256), M >> 5));
}

extern "C" int ttamd_gemm_tn_ws_bf16(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, void* workspace,
                                     size_t workspace_bytes, void* stream) {
  TT_REQUIRE(a && b && c && aligned16(a) && aligned16(b) && aligned16(c), "gemm_tn: pointers must be non-null and 16-byte aligned");
  TT_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_tn: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (!gemm_tn_applies(M, N, K))
    return fail(TTAMD_EUNSUPPORTED, "gemm_tn: M (%lld) must be a multiple of 32, N (%lld) and K (%lld) multiples of 256", (long long)M,
                (long long)N, (long long)K);
  TnArgs g = {};
  g.n = 1;
  g.A[0] = reinterpret_cast<const uint16_t*>(a);
  g.C[0] = reinterpret_cast<uint16_t*>(c);
  g.N[0] = (int)N;
  g.B = reinterpret_cast<const uint16_t*>(b);
  g.M = (int)M; g.K = (int)K;
  g.tiles_n = g.tile_end[0] = (int)(N / 256);
  g.tiles_k = (int)(K / 256);
  return launch_gemm_tn(g, workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int ttamd_gemm_tn_bf16(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, void* stream) {
  return ttamd_gemm_tn_ws_bf16(a, b, c, M, N, K, nullptr, 0, stream);
}

extern "C" int ttamd_gemm_tn_group_ws_bf16(const void* const* a, const void* b, void* const* c, int n_members, int64_t M,
                                           const int64_t* N, int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  TT_REQUIRE(a && b && c && N && aligned16(b), "gemm_tn_group: null or misaligned pointer argument");
  TT_REQUIRE(n_members >= 1 && n_members <= kGroupMax, "gemm_tn_group: %d members (1 .. %d)", n_members, kGroupMax);
  TT_REQUIRE(M > 0 && K > 0, "gemm_tn_group: bad shape M=%lld K=%lld", (long long)M, (long long)K);
  TnArgs g = {};
  g.n = n_members;
  int64_t tiles = 0;
  for (int i = 0; i < n_members; ++i) {
    TT_REQUIRE(a[i] && c[i] && aligned16(a[i]) && aligned16(c[i]), "gemm_tn_group: member %d: pointers must be non-null and 16-byte aligned", i);
    if (N[i] <= 0 || !gemm_tn_applies(M, N[i], K))
      return fail(TTAMD_EUNSUPPORTED, "gemm_tn_group: M (%lld) must be a multiple of 32, N[%d] (%lld) and K (%lld) multiples of 256",
                  (long long)M, i, (long long)N[i], (long long)K);
    g.A[i] = reinterpret_cast<const uint16_t*>(a[i]);
    g.C[i] = reinterpret_cast<uint16_t*>(c[i]);
    g.N[i] = (int)N[i];
    tiles += N[i] / 256;
    g.tile_end[i] = (int)tiles;
  }
  if (tiles * (K / 256) >= (int64_t(1) << 31)) return fail(TTAMD_EUNSUPPORTED, "gemm_tn_group: too many tiles for one launch");
  g.B = reinterpret_cast<const uint16_t*>(b);
  g.M = (int)M; g.K = (int)K;
  g.tiles_n = (int)tiles;
  g.tiles_k = (int)(K / 256);
  return launch_gemm_tn(g, workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int ttamd_gemm_tn_group_bf16(const void* const* a, const void* b, void* const* c, int n_members, int64_t M,
                                        const int64_t* N, int64_t K, void* stream) {
  return ttamd_gemm_tn_group_ws_bf16(a, b, c, n_members, M, N, K, nullptr, 0, stream);
}
