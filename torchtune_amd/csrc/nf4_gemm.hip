// Fused NF4-dequantise + bf16 MFMA GEMM for gfx950, with the LoRA adapter folded in as extra k-steps.
//
//   forward  (TRANS_W = false):  C[M,N] = A[M,K] . D(W)[N,K]^T  (+ bias[N])  + (s.h)[M,R] . B[N,R]^T
//   backward (TRANS_W = true):   C[M,K] = A[M,N] . D(W)[N,K]                  +  gh[M,R]  . La[R,K]
//
// D(W) never exists in HBM: each workgroup expands the 4-bit codes of its weight tile straight into LDS
// (code-pair lookup in a 256-entry fp32 table, one multiply by the block's bf16 scaler, one round to bf16 —
// bit-identical to the stand-alone dequantise kernel) and the MFMA operands are read from there.
//
// Tiling: 256 threads = 4 waves in a 2x2 grid; workgroup tile BM x BN (256 or 128 each), k-step 64;
// v_mfma_f32_32x32x16_bf16, so a wave owns (BM/64) x (BN/64) accumulator tiles of 32x32 fp32.
// LDS holds two stages of {A tile, W tile}, each row = 64 bf16 = eight 16-byte chunks stored at
// chunk ^ (row & 7) so that both the 128-bit fills and the 128-bit operand reads are bank-conflict free.
//
// In the backward the contraction runs over N while NF4 blocks run along K, so the tile is transposed in
// registers: a thread expands an 8(n) x 8(k) patch (one dword of codes from each of 8 rows) and writes it
// as eight 16-byte chunks of 8 consecutive n.
#include "common.h"
#include "group.h"
#include "nf4_math.h"

namespace ttamd {
namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__device__ __constant__ float kNF4Gemm[16] = TT_NF4_TABLE;

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2_t v;
  v.x = (__bf16)lo;
  v.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float bf16lo(uint32_t d) { return bits_f32(d << 16); }
__device__ __forceinline__ float bf16hi(uint32_t d) { return bits_f32(d & 0xffff0000u); }

struct GemmArgs {
  const uint16_t* A;      // [M, Kc] bf16: x (forward) or gy (backward)
  const uint8_t* qdata;   // NF4 codes of W [N, K]
  const float* bscal;     // dequantised block scalers, fp32 [N*K/64]
  const uint16_t* lA;     // adapter operand on the A side: h (forward) or gh (backward), [M, R] bf16, or null
  const uint16_t* lB;     // adapter operand on the W side: lora_b [N, R] (forward) or lora_a [R, K] (backward)
  const uint16_t* bias;   // [N] bf16 or null (forward only)
  uint16_t* C;            // [M, Nout] bf16
  int M, N, K, R;
  float lscale;           // alpha / rank, applied to h in the forward
  int tiles_m, tiles_n;
};

constexpr int kRowBytes = 128;  // one LDS tile row: 64 bf16

__device__ __forceinline__ int swz(int row, int chunk) { return row * kRowBytes + ((chunk ^ (row & 7)) << 4); }

template <int BM, int BN, bool TRANS_W>
__global__ __launch_bounds__(256) void nf4_gemm_kernel(const GemmArgs g) {
  static_assert(BM == 256 || BM == 128, "BM");
  static_assert(BN == 256 || BN == 128, "BN");
  constexpr int TM = BM / 64, TN = BN / 64;
  constexpr int kStageBytes = (BM + BN) * kRowBytes;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  float2* lut = reinterpret_cast<float2*>(smem + 2 * kStageBytes);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int l31 = lane & 31, lhi = lane >> 5;
  const int wm0 = (wave >> 1) * (BM / 2), wn0 = (wave & 1) * (BN / 2);

  // workgroup -> tile.  Workgroup ids are dealt round-robin to the 8 XCDs, each with a private L2: give
  // every XCD a contiguous band of m-tiles so an A row band is fetched into exactly one L2.
  int tile_m, tile_n;
  {
    const int id = blockIdx.x;
    if ((g.tiles_m & 7) == 0) {
      const int xcd = id & 7, slot = id >> 3;
      const int band = g.tiles_m >> 3;
      tile_m = xcd * band + slot / g.tiles_n;
      tile_n = slot % g.tiles_n;
    } else {
      tile_m = id / g.tiles_n;
      tile_n = id % g.tiles_n;
    }
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;  // n0: first output column (n in forward, k in backward)
  const int Kc = TRANS_W ? g.N : g.K;             // contraction length
  const int Nout = TRANS_W ? g.K : g.N;
  const int kblocks_per_row = g.K >> 6;

  lut[tid] = make_float2(round_to_bf16(kNF4Gemm[tid >> 4]), round_to_bf16(kNF4Gemm[tid & 15]));

  // ---- per-thread global->register staging ---------------------------------------------------------
  // A tile: thread owns chunk (tid & 7) of rows (tid >> 3) + 32 i.
  constexpr int kARows = BM / 32;
  u32x4_t ra[kARows];
  const int a_chunk = tid & 7, a_row0 = tid >> 3;
  const uint16_t* a_src[kARows];
#pragma unroll
  for (int i = 0; i < kARows; ++i) {
    int row = m0 + a_row0 + 32 * i;
    row = row < g.M ? row : g.M - 1;
    a_src[i] = g.A + (int64_t)row * Kc + a_chunk * 8;
  }

  // W tile staging
  constexpr int TPR = TRANS_W ? 1 : 256 / BN;        // forward: threads per weight row
  constexpr int kWDwords = TRANS_W ? 8 : 8 / TPR;    // dwords of codes per thread per k-step
  uint32_t wq[kWDwords];
  float wscal[TRANS_W ? 8 : 1];
  // forward: row n = n0 + tid / TPR, dwords [part*kWDwords, ...) of the row's 8
  const int f_row = tid / TPR, f_part = tid % TPR;
  int f_n = n0 + f_row;
  f_n = f_n < g.N ? f_n : g.N - 1;
  // backward: patch of rows ng*8..+7 (contraction n), columns kg*8..+7 (output k)
  constexpr int kKGroups = BN / 8;
  const int b_kg = tid % kKGroups, b_ng = tid / kKGroups;  // b_ng < 8 only when BN == 256; else upper threads idle
  const bool b_active = !TRANS_W || (b_ng < 8);
  int b_kcol = n0 + b_kg * 8;
  b_kcol = b_kcol < g.K ? b_kcol : g.K - 8;

  auto load_tiles = [&](int kt) {
    const int k0 = kt * 64;
#pragma unroll
    for (int i = 0; i < kARows; ++i) ra[i] = *reinterpret_cast<const u32x4_t*>(a_src[i] + k0);
    if constexpr (!TRANS_W) {
      const uint32_t* src =
          reinterpret_cast<const uint32_t*>(g.qdata + (((int64_t)f_n * g.K + k0) >> 1)) + f_part * kWDwords;
      if constexpr (kWDwords == 8) {
        u32x4_t v0 = reinterpret_cast<const u32x4_t*>(src)[0], v1 = reinterpret_cast<const u32x4_t*>(src)[1];
        wq[0] = v0.x; wq[1] = v0.y; wq[2] = v0.z; wq[3] = v0.w;
        wq[4] = v1.x; wq[5] = v1.y; wq[6] = v1.z; wq[7] = v1.w;
      } else if constexpr (kWDwords == 4) {
        u32x4_t v0 = reinterpret_cast<const u32x4_t*>(src)[0];
        wq[0] = v0.x; wq[1] = v0.y; wq[2] = v0.z; wq[3] = v0.w;
      } else {
        u32x2_t v0 = reinterpret_cast<const u32x2_t*>(src)[0];
        wq[0] = v0.x; wq[1] = v0.y;
      }
      wscal[0] = g.bscal[(int64_t)f_n * kblocks_per_row + kt];
    } else {
      if (b_active) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int n = k0 + b_ng * 8 + i;  // contraction index: always < N because N % 64 == 0
          wq[i] = *reinterpret_cast<const uint32_t*>(g.qdata + (((int64_t)n * g.K + b_kcol) >> 1));
          wscal[i] = g.bscal[(int64_t)n * kblocks_per_row + (b_kcol >> 6)];
        }
      }
    }
  };

  auto store_tiles = [&](int stage) {
    char* sA = smem + stage * kStageBytes;
    char* sB = sA + BM * kRowBytes;
#pragma unroll
    for (int i = 0; i < kARows; ++i)
      *reinterpret_cast<u32x4_t*>(sA + swz(a_row0 + 32 * i, a_chunk)) = ra[i];
    if constexpr (!TRANS_W) {
      const float s = wscal[0];
#pragma unroll
      for (int j = 0; j < kWDwords; ++j) {
        u32x4_t o;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const float2 pr = lut[(wq[j] >> (8 * b)) & 0xffu];
          o[b] = pack_bf16x2(pr.x * s, pr.y * s);
        }
        *reinterpret_cast<u32x4_t*>(sB + swz(f_row, f_part * kWDwords + j)) = o;
      }
    } else {
      if (b_active) {
        // v[i][e]: row i of the patch (n), element e (k); written out as 8 chunks of 8 consecutive n.
        float v[8][8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            const float2 pr = lut[(wq[i] >> (8 * b)) & 0xffu];
            v[i][2 * b] = pr.x * wscal[i];
            v[i][2 * b + 1] = pr.y * wscal[i];
          }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          u32x4_t o;
          o.x = pack_bf16x2(v[0][e], v[1][e]);
          o.y = pack_bf16x2(v[2][e], v[3][e]);
          o.z = pack_bf16x2(v[4][e], v[5][e]);
          o.w = pack_bf16x2(v[6][e], v[7][e]);
          *reinterpret_cast<u32x4_t*>(sB + swz(b_kg * 8 + e, b_ng)) = o;
        }
      }
    }
  };

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int nk = Kc >> 6;
  load_tiles(0);
  __syncthreads();  // lut ready
  store_tiles(0);
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const bool more = kt + 1 < nk;
    if (more) load_tiles(kt + 1);
    const char* sA = smem + (kt & 1) * kStageBytes;
    const char* sB = sA + BM * kRowBytes;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      bf16x8_t af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const bf16x8_t*>(sA + swz(wm0 + i * 32 + l31, ks * 2 + lhi));
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bfr[j] = *reinterpret_cast<const bf16x8_t*>(sB + swz(wn0 + j * 32 + l31, ks * 2 + lhi));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    if (more) store_tiles((kt + 1) & 1);
    __syncthreads();
  }

  // ---- adapter: R extra contraction steps, operands straight from global memory ---------------------
  if (g.R > 0) {
    for (int rc = 0; rc < g.R; rc += 16) {
      const int r0 = rc + 8 * lhi;  // this lane's 8 contraction indices; R % 8 == 0 so all-in or all-out
      const bool in = r0 < g.R;
      bf16x8_t af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        int row = m0 + wm0 + i * 32 + l31;
        row = row < g.M ? row : g.M - 1;
        u32x4_t raw = {0, 0, 0, 0};
        if (in) raw = *reinterpret_cast<const u32x4_t*>(g.lA + (int64_t)row * g.R + r0);
        if constexpr (!TRANS_W) {
#pragma unroll
          for (int d = 0; d < 4; ++d) raw[d] = pack_bf16x2(bf16lo(raw[d]) * g.lscale, bf16hi(raw[d]) * g.lscale);
        }
        af[i] = __builtin_bit_cast(bf16x8_t, raw);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        int col = n0 + wn0 + j * 32 + l31;
        col = col < Nout ? col : Nout - 1;
        u32x4_t raw = {0, 0, 0, 0};
        if (in) {
          if constexpr (!TRANS_W) {
            raw = *reinterpret_cast<const u32x4_t*>(g.lB + (int64_t)col * g.R + r0);
          } else {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              const uint32_t lo = g.lB[(int64_t)(r0 + 2 * d) * g.K + col];
              const uint32_t hi = g.lB[(int64_t)(r0 + 2 * d + 1) * g.K + col];
              raw[d] = lo | (hi << 16);
            }
          }
        }
        bfr[j] = __builtin_bit_cast(bf16x8_t, raw);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
  }

  // ---- epilogue: (+bias) -> bf16 -> global.  acc[i][j][v] is C[row][col] with
  //      row = 8*(v/4) + 4*(lane/32) + v%4, col = lane%32 inside its 32x32 tile.
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn0 + j * 32 + l31;
    if (col >= Nout) continue;
    float bias = 0.f;
    if constexpr (!TRANS_W) {
      if (g.bias) bias = bf16_bits_to_f32(g.bias[col]);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm0 + i * 32 + 8 * (v >> 2) + 4 * lhi + (v & 3);
        if (row < g.M) g.C[(int64_t)row * Nout + col] = f32_to_bf16_bits(acc[i][j][v] + bias);
      }
  }
}

// block scalers: scaler[b] = dtype(dtype(int8[b] / factor[b / SB]) + mean), widened to fp32 (exact).
template <bool BF16>
__global__ __launch_bounds__(256) void nf4_block_scalers_kernel(const int8_t* __restrict__ qs, const void* __restrict__ qf,
                                                                const void* __restrict__ mean, int64_t n_blocks, int SB,
                                                                float* __restrict__ out) {
  const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (b >= n_blocks) return;
  float f, m;
  if constexpr (BF16) {
    f = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(qf)[b / SB]);
    m = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(mean)[0]);
  } else {
    f = reinterpret_cast<const float*>(qf)[b / SB];
    m = reinterpret_cast<const float*>(mean)[0];
  }
  out[b] = nf4_block_scaler<BF16>((int)qs[b], f, m);
}

// Transposed copy of the codes for the grad-input GEMM: out[k][n] = code of W[n][k], packed along n
// (byte (k*N + n)/2, even n in the high nibble).  A workgroup moves a tile of 64 rows n x 128 columns k through LDS:
// it reads 64-byte row pieces and writes 32-byte row pieces of the transposed tensor, so both sides use whole sectors
// (reading single bytes down a column fetched eight times the tensor).
constexpr int kTrTileK = 128;  // columns k per tile = 64 bytes of a row
constexpr int kTrPitch = 68;   // LDS row pitch in bytes (64 + 4: rows of a column land in different banks)

__global__ __launch_bounds__(256) void nf4_transpose_codes_kernel(const uint8_t* __restrict__ q, int N, int K,
                                                                  uint32_t* __restrict__ qt) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[64 * kTrPitch];
  const int t = threadIdx.x;
  const int n0 = blockIdx.x * 64, k0 = blockIdx.y * kTrTileK;
  {
    const int r = t >> 2, piece = t & 3;  // row of the tile, 16-byte piece (32 codes) of its 64 bytes
    uint32_t v[4] = {0, 0, 0, 0};
    if (k0 + 32 * piece < K) {            // K % 64 == 0: a piece is in or out as a whole
      const uint4 ld = *reinterpret_cast<const uint4*>(q + (((int64_t)(n0 + r) * K + k0) >> 1) + 16 * piece);
      v[0] = ld.x; v[1] = ld.y; v[2] = ld.z; v[3] = ld.w;
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) *reinterpret_cast<uint32_t*>(tile + r * kTrPitch + 16 * piece + 4 * d) = v[d];
  }
  __syncthreads();
  const int n8s = N >> 3;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int o = t + 256 * j;       // output dword of the tile: row k, eight consecutive n
    const int k = o >> 3, n8 = o & 7;
    if (k0 + k >= K) continue;
    const int shift = (k & 1) ? 0 : 4;
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t code = ((uint32_t)tile[(n8 * 8 + i) * kTrPitch + (k >> 1)] >> shift) & 0xfu;
      packed |= code << (8 * (i >> 1) + ((i & 1) ? 0 : 4));
    }
    qt[(int64_t)(k0 + k) * n8s + (n0 >> 3) + n8] = packed;
  }
}

// Transposed block scalers: out[kb][n] = scalers[n][kb]
__global__ __launch_bounds__(256) void nf4_transpose_scalers_kernel(const float* __restrict__ sc, int N, int KB,
                                                                    float* __restrict__ out) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // = kb * N + n
  if (idx >= (int64_t)N * KB) return;
  const int kb = (int)(idx / N), n = (int)(idx % N);
  out[idx] = sc[(int64_t)n * KB + kb];
}

template <int BM, int BN, bool TRANS_W>
int launch_gemm(GemmArgs& g, hipStream_t s) {
  const int Nout = TRANS_W ? g.K : g.N;
  g.tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (Nout + BN - 1) / BN;
  const size_t smem = 2 * (BM + BN) * kRowBytes + 256 * sizeof(float2);
  // the limit is a per-device attribute of the function: set it for the current device once (a race only repeats the call)
  static bool attr_set_dev[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
  if (dev < 0 || !attr_set_dev[dev]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&nf4_gemm_kernel<BM, BN, TRANS_W>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return fail(TTAMD_ELAUNCH, "nf4_gemm: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
    if (dev >= 0) attr_set_dev[dev] = true;
  }
  nf4_gemm_kernel<BM, BN, TRANS_W><<<dim3((unsigned)(g.tiles_m * g.tiles_n)), dim3(256), smem, s>>>(g);
  return check_launch("nf4_gemm");
}

// Pick the largest tile that still gives every CU something to do.
template <bool TRANS_W>
int dispatch_gemm(GemmArgs& g, hipStream_t s) {
  const int Nout = TRANS_W ? g.K : g.N;
  auto tiles = [&](int bm, int bn) { return (int64_t)((g.M + bm - 1) / bm) * ((Nout + bn - 1) / bn); };
  constexpr int kCUs = 256;
  if (tiles(256, 256) >= kCUs) return launch_gemm<256, 256, TRANS_W>(g, s);
  if (tiles(128, 256) >= kCUs) return launch_gemm<128, 256, TRANS_W>(g, s);
  return launch_gemm<128, 128, TRANS_W>(g, s);
}

int check_gemm_args(const char* who, const void* a, const uint8_t* qdata, const void* bscal, void* c, int64_t M, int64_t N,
                    int64_t K, int rank, const void* l1, const void* l2) {
  TT_REQUIRE(a && qdata && bscal && c, "%s: null pointer argument", who);
  TT_REQUIRE(aligned16(a) && aligned16(qdata) && aligned16(c), "%s: pointers must be 16-byte aligned", who);
  TT_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1 << 30) && N < (1 << 30) && K < (1 << 30), "%s: bad shape M=%lld N=%lld K=%lld",
             who, (long long)M, (long long)N, (long long)K);
  TT_REQUIRE(K % 64 == 0, "%s: K (%lld) must be a multiple of the NF4 block size 64", who, (long long)K);
  TT_REQUIRE(N % 64 == 0, "%s: N (%lld) must be a multiple of 64", who, (long long)N);
  TT_REQUIRE(rank >= 0 && rank <= 64 && rank % 8 == 0, "%s: rank (%d) must be a multiple of 8 in [0, 64]", who, rank);
  TT_REQUIRE((rank == 0) == (l1 == nullptr) && (rank == 0) == (l2 == nullptr),
             "%s: adapter pointers must be given exactly when rank > 0", who);
  TT_REQUIRE(rank == 0 || (aligned16(l1) && aligned16(l2)), "%s: adapter pointers must be 16-byte aligned", who);
  return TTAMD_OK;
}

}  // namespace

// nf4_small_m.hip (run_gemm_rs, gemm_rs_workspace_bytes and small_m_limit: group.h)
int run_small_m(const void* x, const uint8_t* codes, const void* bscal, const void* h, int ldh, const void* lora_b, int R,
                float lscale, const void* bias, const void* cscale, void* y, int64_t M, int64_t N, int64_t K, hipStream_t s);
}  // namespace ttamd

using namespace ttamd;

extern "C" int ttamd_nf4_block_scalers(const int8_t* quantized_scalers, const void* quantization_factor,
                                       const void* scaler_mean, int dtype, int64_t n_blocks, int scaler_block_size,
                                       void* block_scalers, void* stream) {
  TT_REQUIRE(dtype == TTAMD_BF16 || dtype == TTAMD_F32, "nf4_block_scalers: unknown dtype code %d", dtype);
  TT_REQUIRE(quantized_scalers && quantization_factor && scaler_mean && block_scalers, "nf4_block_scalers: null pointer");
  TT_REQUIRE(n_blocks > 0 && scaler_block_size > 0 && n_blocks % scaler_block_size == 0,
             "nf4_block_scalers: n_blocks (%lld) must be a positive multiple of scaler_block_size (%d)", (long long)n_blocks,
             scaler_block_size);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)((n_blocks + 255) / 256)), block(256);
  if (dtype == TTAMD_BF16)
    nf4_block_scalers_kernel<true><<<grid, block, 0, s>>>(quantized_scalers, quantization_factor, scaler_mean, n_blocks,
                                                          scaler_block_size, reinterpret_cast<float*>(block_scalers));
  else
    nf4_block_scalers_kernel<false><<<grid, block, 0, s>>>(quantized_scalers, quantization_factor, scaler_mean, n_blocks,
                                                           scaler_block_size, reinterpret_cast<float*>(block_scalers));
  return check_launch("nf4_block_scalers");
}

namespace {
int lora_linear_fwd(const char* who, const void* x, const uint8_t* quantized_data, const void* block_scalers,
                    const void* block_scalers_t, const void* h, const void* lora_b, int rank, float scale, const void* bias,
                    const void* col_scale, void* y, int64_t M, int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                    void* stream) {
  if (int rc = check_gemm_args(who, x, quantized_data, block_scalers, y, M, N, K, rank, h, lora_b)) return rc;
  TT_REQUIRE((bias == nullptr || (reinterpret_cast<uintptr_t>(bias) & 7u) == 0) &&
                 (col_scale == nullptr || (reinterpret_cast<uintptr_t>(col_scale) & 7u) == 0),
             "%s: bias / col_scale must be 8-byte aligned", who);
  // a handful of tokens: stream the packed weight once (nf4_small_m.hip)
  if (small_m_applies(M, N, K, workspace != nullptr && workspace_bytes > 0 && workspace_bytes >= gemm_rs_workspace_bytes(M, N, K)))
    return run_small_m(x, quantized_data, block_scalers, h, rank, lora_b, rank, scale, bias, col_scale, y, M, N, K,
                       reinterpret_cast<hipStream_t>(stream));
  if (block_scalers_t) {
    TT_REQUIRE(aligned16(block_scalers_t), "%s: block_scalers_t must be 16-byte aligned", who);
    return run_gemm_rs(x, quantized_data, block_scalers_t, 2, h, rank, lora_b, true, rank, scale, bias, col_scale, y, M, N, K,
                       workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
  }
  return run_gemm_rs(x, quantized_data, block_scalers, 0, h, rank, lora_b, true, rank, scale, bias, col_scale, y, M, N, K,
                     workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}
}  // namespace

extern "C" int ttamd_nf4_lora_linear_fwd_bf16(const void* x, const uint8_t* quantized_data, const void* block_scalers,
                                              const void* block_scalers_t, const void* h, const void* lora_b, int rank,
                                              float scale, const void* bias, void* y, int64_t M, int64_t N, int64_t K,
                                              void* stream) {
  return lora_linear_fwd("nf4_lora_linear_fwd", x, quantized_data, block_scalers, block_scalers_t, h, lora_b, rank, scale, bias,
                         nullptr, y, M, N, K, nullptr, 0, stream);
}

extern "C" size_t ttamd_nf4_gemm_workspace_bytes(int64_t M, int64_t n_out, int64_t k_contract) {
  if (M <= 0 || n_out <= 0 || k_contract <= 0 || small_m_applies(M, n_out, k_contract, true)) return 0;
  return gemm_rs_workspace_bytes(M, n_out, k_contract);
}

extern "C" int ttamd_nf4_gemm_expands_weight(int64_t M, int64_t n_out, int64_t k_contract) {
  return M > small_m_limit() && n_out > 0 && k_contract > 0 && dense_path_applies(M, n_out, k_contract) ? 1 : 0;
}

extern "C" int ttamd_nf4_lora_linear_fwd_ws_bf16(const void* x, const uint8_t* quantized_data, const void* block_scalers,
                                                 const void* block_scalers_t, const void* h, const void* lora_b, int rank,
                                                 float scale, const void* bias, const void* col_scale, void* y, int64_t M,
                                                 int64_t N, int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  return lora_linear_fwd("nf4_lora_linear_fwd_ws", x, quantized_data, block_scalers, block_scalers_t, h, lora_b, rank, scale,
                         bias, col_scale, y, M, N, K, workspace, workspace_bytes, stream);
}

extern "C" int ttamd_nf4_dora_linear_fwd_bf16(const void* x, const uint8_t* quantized_data, const void* block_scalers,
                                              const void* block_scalers_t, const void* h, const void* lora_b, int rank,
                                              float scale, const void* bias, const void* col_scale, void* y, int64_t M,
                                              int64_t N, int64_t K, void* stream) {
  TT_REQUIRE(col_scale, "nf4_dora_linear_fwd: col_scale is null");
  return lora_linear_fwd("nf4_dora_linear_fwd", x, quantized_data, block_scalers, block_scalers_t, h, lora_b, rank, scale, bias,
                         col_scale, y, M, N, K, nullptr, 0, stream);
}

extern "C" int ttamd_nf4_transpose_for_backward(const uint8_t* quantized_data, const void* block_scalers, int64_t N, int64_t K,
                                                uint8_t* quantized_data_t, void* block_scalers_t, void* stream) {
  TT_REQUIRE(quantized_data && block_scalers && quantized_data_t && block_scalers_t, "nf4_transpose_for_backward: null pointer");
  TT_REQUIRE(N > 0 && K > 0 && N % 64 == 0 && K % 64 == 0 && N < (1 << 30) && K < (1 << 30),
             "nf4_transpose_for_backward: N (%lld) and K (%lld) must be positive multiples of 64", (long long)N, (long long)K);
  TT_REQUIRE((reinterpret_cast<uintptr_t>(quantized_data_t) & 3u) == 0, "nf4_transpose_for_backward: output must be 4-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int64_t n2 = N * (K / 64);
  TT_REQUIRE((K + kTrTileK - 1) / kTrTileK < 65536, "nf4_transpose_for_backward: K too large for one launch");
  TT_REQUIRE(aligned16(quantized_data), "nf4_transpose_for_backward: quantized_data must be 16-byte aligned");
  nf4_transpose_codes_kernel<<<dim3((unsigned)(N / 64), (unsigned)((K + kTrTileK - 1) / kTrTileK)), dim3(256), 0, s>>>(
      quantized_data, (int)N, (int)K, reinterpret_cast<uint32_t*>(quantized_data_t));
  nf4_transpose_scalers_kernel<<<dim3((unsigned)((n2 + 255) / 256)), dim3(256), 0, s>>>(
      reinterpret_cast<const float*>(block_scalers), (int)N, (int)(K / 64), reinterpret_cast<float*>(block_scalers_t));
  return check_launch("nf4_transpose_for_backward");
}

extern "C" int ttamd_nf4_linear_bwd_dx_ws_bf16(const void* gy, const uint8_t* quantized_data, const void* block_scalers,
                                               const uint8_t* quantized_data_t, const void* block_scalers_t, const void* gh,
                                               const void* lora_a, int rank, void* gx, int64_t M, int64_t N, int64_t K,
                                               void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_gemm_args("nf4_linear_bwd_dx", gy, quantized_data, block_scalers, gx, M, N, K, rank, gh, lora_a)) return rc;
  TT_REQUIRE((quantized_data_t == nullptr) == (block_scalers_t == nullptr),
             "nf4_linear_bwd_dx: the transposed codes and scalers must be given together");
  if (quantized_data_t != nullptr) {
    TT_REQUIRE(aligned16(quantized_data_t) && aligned16(block_scalers_t), "nf4_linear_bwd_dx: transposed copies must be 16-byte aligned");
    return run_gemm_rs(gy, quantized_data_t, block_scalers_t, 1, gh, rank, lora_a, false, rank, 1.0f, nullptr, nullptr, gx, M, K, N,
                       workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
  }
  // no transposed copy, many tokens and room for the expanded weight: W^T is expanded from the weight's own codes
  if (workspace != nullptr && dense_path_applies(M, K, N) && workspace_bytes >= dense_workspace_bytes(M, K, N))
    return run_gemm_dense(gy, quantized_data, block_scalers, 3, gh, rank, lora_a, false, rank, 1.0f, nullptr, nullptr, gx, M, K, N,
                          workspace, reinterpret_cast<hipStream_t>(stream));
  GemmArgs g;
  g.A = reinterpret_cast<const uint16_t*>(gy);
  g.qdata = quantized_data;
  g.bscal = reinterpret_cast<const float*>(block_scalers);
  g.lA = reinterpret_cast<const uint16_t*>(gh);
  g.lB = reinterpret_cast<const uint16_t*>(lora_a);
  g.bias = nullptr;
  g.C = reinterpret_cast<uint16_t*>(gx);
  g.M = (int)M; g.N = (int)N; g.K = (int)K; g.R = rank;
  g.lscale = 1.0f;
  return dispatch_gemm<true>(g, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int ttamd_nf4_linear_bwd_dx_swiglu_ws_bf16(const void* gy, const uint8_t* quantized_data, const void* block_scalers,
                                                      const uint8_t* quantized_data_t, const void* block_scalers_t, const void* gh,
                                                      const void* lora_a, int rank, const void* gate, const void* up, void* ggate,
                                                      void* gup, int64_t M, int64_t N, int64_t K, void* workspace,
                                                      size_t workspace_bytes, void* stream) {
  if (int rc = check_gemm_args("nf4_linear_bwd_dx_swiglu", gy, quantized_data, block_scalers, ggate, M, N, K, rank, gh, lora_a)) return rc;
  TT_REQUIRE(gate && up && gup, "nf4_linear_bwd_dx_swiglu: null pointer argument");
  TT_REQUIRE(aligned16(gate) && aligned16(up) && aligned16(ggate) && aligned16(gup), "nf4_linear_bwd_dx_swiglu: pointers must be 16-byte aligned");
  TT_REQUIRE((quantized_data_t == nullptr) == (block_scalers_t == nullptr),
             "nf4_linear_bwd_dx_swiglu: the transposed codes and scalers must be given together");
  if (workspace != nullptr && dense_path_applies(M, K, N) && workspace_bytes >= dense_workspace_bytes(M, K, N)) {
    const DenseSwigluBwd sw = {gate, up, gup};
    const bool tr = quantized_data_t != nullptr;
    TT_REQUIRE(!tr || (aligned16(quantized_data_t) && aligned16(block_scalers_t)), "nf4_linear_bwd_dx_swiglu: transposed copies must be 16-byte aligned");
    return run_gemm_dense(gy, tr ? quantized_data_t : quantized_data, tr ? block_scalers_t : block_scalers, tr ? 1 : 3, gh, rank, lora_a,
                          false, rank, 1.0f, nullptr, nullptr, ggate, M, K, N, workspace, reinterpret_cast<hipStream_t>(stream), &sw);
  }
  // other sizes: the grad-input as usual, parked in ggate, then the stand-alone kernel in place
  if (int rc = ttamd_nf4_linear_bwd_dx_ws_bf16(gy, quantized_data, block_scalers, quantized_data_t, block_scalers_t, gh, lora_a, rank, ggate,
                                               M, N, K, workspace, workspace_bytes, stream))
    return rc;
  return ttamd_swiglu_bwd_bf16(ggate, gate, up, ggate, gup, M * K, stream);
}

extern "C" int ttamd_nf4_linear_bwd_dx_bf16(const void* gy, const uint8_t* quantized_data, const void* block_scalers,
                                            const uint8_t* quantized_data_t, const void* block_scalers_t, const void* gh,
                                            const void* lora_a, int rank, void* gx, int64_t M, int64_t N, int64_t K,
                                            void* stream) {
  return ttamd_nf4_linear_bwd_dx_ws_bf16(gy, quantized_data, block_scalers, quantized_data_t, block_scalers_t, gh, lora_a, rank,
                                         gx, M, N, K, nullptr, 0, stream);
}
