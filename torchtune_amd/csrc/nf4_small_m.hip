// y = x . D(W)^T (+ bias) + scale . h . lora_b^T, times an optional column scale, for a handful of tokens (M <= 64):
// the decode / evaluation regime of linear_nf4 and LoRALinear.forward (torchtune/modules/peft/lora.py:128-147,
// torchtune/modules/low_precision/nf4_linear.py:56-70).
//
// With so few rows the work is streaming the packed weight once: 0.5625 bytes per weight element against 2 for a
// dense bf16 weight.  A workgroup owns 16 or 32 weight rows and the whole contraction; its waves (up to sixteen) take
// groups of 128-wide chunks of K in turn, all of a group's loads in flight together, expand the codes in registers
// exactly as the large-M kernel does (byte -> fp32 pair from an LDS table, times the fp32 block scaler, one rounding to
// bf16 - the bits of ttamd_nf4_dequantize) and feed v_mfma_f32_16x16x32_bf16 with the weight rows as the row operand
// and up to four 16-token tiles of x as the column operand.  A lane reads 16 contiguous bytes of codes (32 elements of
// its row: the four lane groups of a row cover one 64-byte piece) and uses one dword of them per MFMA; x is small and
// comes from the cache.  The waves' partial sums meet in LDS in a fixed order, and wave 0 adds the adapter, the bias
// and the column scale and stores.  What the kernel reaches is 1.4 - 2.4 TB/s of packed weight, short of the HBM
// bound: a launch lives for a few trips to memory, and the expansion (about three vector instructions per element) is
// not hidden behind them.
#include "common.h"
#include "group.h"
#include "nf4_math.h"

namespace ttamd {
namespace {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  bf16x2_t v;
  v.x = (__bf16)lo;
  v.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float lo_of(uint32_t d) { return bits_f32(d << 16); }
__device__ __forceinline__ float hi_of(uint32_t d) { return bits_f32(d & 0xffff0000u); }

struct SmallMArgs {
  const uint16_t* x;       // [M, K] bf16
  const uint8_t* codes;    // [N, K/2]
  const float* bscal;      // [N, K/64]
  const uint16_t* h;       // [M, R] bf16 (rows ldh elements apart) or null
  const uint16_t* lora_b;  // [N, R] bf16 or null
  const uint16_t* bias;    // [N] bf16 or null
  const uint16_t* cscale;  // [N] bf16 or null
  uint16_t* y;             // [M, N] bf16
  int M, N, K, R, ldh;
  float lscale;
};
// The layers of one launch: they share x, M and K (projections of a common input); workgroups [wg_end[i - 1], wg_end[i])
// work on layer i.
struct SmallMGroup {
  SmallMArgs m[kGroupMax];
  int wg_end[kGroupMax];
  int n;
};

constexpr int kSmMaxWaves = 16;

// U chunks (128 elements of K each) of RT 16-row tiles: what one wave has in flight.
template <int RT, int U>
struct WeightFrag {
  u32x4_t cd[U][RT];  // 32 codes of this lane's row per chunk
  float sc[U][RT];    // the block scaler of those 32 elements
};

// TAIL: the lane may lie beyond K (the last chunk of a K that is an odd multiple of 64 is half a chunk).
template <int RT, int U, bool TAIL>
__device__ __forceinline__ void load_weights(WeightFrag<RT, U>& f, const uint8_t* crow, const float* srow, int64_t ctile,
                                             int64_t stile, int c0, bool valid) {
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if (TAIL && !valid) {
        f.cd[u][rt] = u32x4_t{0, 0, 0, 0};
        f.sc[u][rt] = 0.f;
      } else {
        f.cd[u][rt] = *reinterpret_cast<const u32x4_t*>(crow + rt * ctile + (int64_t)(c0 + u) * 64);
        f.sc[u][rt] = srow[rt * stile + 2 * (c0 + u)];
      }
    }
}

template <int MT, int RT, int U, int NACC, bool TAIL>
__device__ __forceinline__ void multiply(const WeightFrag<RT, U>& f, const float2* lut, const uint16_t* const (&xrow)[MT], int c0,
                                         bool valid, f32x4_t (&acc)[MT][RT][NACC]) {
  u32x4_t xb[U][4][MT];
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (TAIL && !valid)
          xb[u][s][mt] = u32x4_t{0, 0, 0, 0};
        else
          xb[u][s][mt] = *reinterpret_cast<const u32x4_t*>(xrow[mt] + (c0 + u) * 128 + 8 * s);
      }
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        u32x4_t wf;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const float2 p = lut[(f.cd[u][rt][s] >> (8 * b)) & 0xffu];
          wf[b] = pack_pair(p.x * f.sc[u][rt], p.y * f.sc[u][rt]);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[mt][rt][s % NACC] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(bf16x8_t, wf), __builtin_bit_cast(bf16x8_t, xb[u][s][mt]), acc[mt][rt][s % NACC], 0, 0, 0);
      }
}

// One NF4 code as fp32 without touching memory (a chain of selects over the sixteen constants).
__device__ __forceinline__ float nf4_code_value(int k) {
  constexpr float tab[16] = TT_NF4_TABLE;
  float v = tab[0];
#pragma unroll
  for (int j = 1; j < 16; ++j) v = k == j ? tab[j] : v;
  return v;
}

// MT 16-token tiles of x, RT 16-row tiles of W per workgroup, U chunks of K in flight per wave, at most MAXW waves (the
// register budget of a lane follows from it: the four-wave shapes hold more tiles per lane).
template <int MT, int RT, int U, int MAXW>
__global__ __launch_bounds__(64 * MAXW) void nf4_small_m_kernel(const SmallMGroup grp) {
  int which = 0;  // uniform over the workgroup
#pragma unroll
  for (int q = 0; q < kGroupMax - 1; ++q)
    if (q < grp.n - 1 && (int)blockIdx.x >= grp.wg_end[q]) which = q + 1;
  const SmallMArgs& a = grp.m[which];
  const int wg = (int)blockIdx.x - (which ? grp.wg_end[which - 1] : 0);
  // independent MFMA chains per lane: at least four; one token tile always sums in four chains, whatever the row tiles,
  // so that a row of up to 16 tokens gets the same bits alone and in a batch
  constexpr int NACC = MT == 1 ? 4 : (MT * RT == 2 ? 2 : 1);
  __shared__ float2 lut[256];
  extern __shared__ float red[];  // [waves - 1][MT * RT * 4][64]
  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int nw = blockDim.x >> 6;
  const int i = lane & 15, g = lane >> 4;

  const int K = a.K;
  const int n0 = wg * (16 * RT);  // N % (16 RT) == 0: every row of the workgroup exists
  const uint8_t* crow = a.codes + (((int64_t)(n0 + i) * K) >> 1) + 16 * g;
  const float* srow = a.bscal + (int64_t)(n0 + i) * (K >> 6) + (g >> 1);
  const int64_t ctile = (int64_t)8 * K, stile = (int64_t)16 * (K >> 6);  // one 16-row tile further on
  const uint16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int m = 16 * mt + i;
    m = m < a.M ? m : a.M - 1;  // rows beyond M repeat the last one and are never stored
    xrow[mt] = a.x + (int64_t)m * K + 32 * g;
  }
  f32x4_t acc[MT][RT][NACC];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int q = 0; q < NACC; ++q) acc[mt][rt][q] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // Groups of U whole chunks go round the waves; what is left (fewer than U chunks, the last maybe half a chunk) follows
  // one chunk at a time.  The first group's weights are asked for before the code table is built: a workgroup lives
  // for little more than one trip to memory, and the table must not stand in front of it.
  const int n_groups = (K >> 7) / U;
  const int n_chunks = (K + 127) >> 7;
  WeightFrag<RT, U> f;
  int j = wave;
  if (j < n_groups) load_weights<RT, U, false>(f, crow, srow, ctile, stile, j * U, true);
  for (int e = t; e < 256; e += blockDim.x)
    lut[e] = make_float2(round_to_bf16(nf4_code_value(e >> 4)), round_to_bf16(nf4_code_value(e & 15)));
  __syncthreads();
  while (j < n_groups) {
    multiply<MT, RT, U, NACC, false>(f, lut, xrow, j * U, true, acc);
    j += nw;
    if (j < n_groups) load_weights<RT, U, false>(f, crow, srow, ctile, stile, j * U, true);
  }
  for (int c = n_groups * U + wave; c < n_chunks; c += nw) {
    const bool valid = c * 128 + 32 * g < K;
    WeightFrag<RT, 1> f1;
    load_weights<RT, 1, true>(f1, crow, srow, ctile, stile, c, valid);
    multiply<MT, RT, 1, NACC, true>(f1, lut, xrow, c, valid, acc);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int q = 1; q < NACC; ++q) acc[mt][rt][0] += acc[mt][rt][q];
  // acc[mt][rt][0][v] = sum over this wave's chunks of D(W)[n0 + 16 rt + 4 g + v][.] . x[16 mt + i][.]
  if (wave > 0) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[(((wave - 1) * MT + mt) * RT + rt) * 256 + v * 64 + lane] = acc[mt][rt][0][v];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int nb = n0 + 16 * rt + 4 * g;  // this lane's four output columns nb .. nb + 3
    float b4[4] = {0.f, 0.f, 0.f, 0.f}, c4[4] = {1.f, 1.f, 1.f, 1.f};
    if (a.bias) {
      const u32x2_t bb = *reinterpret_cast<const u32x2_t*>(a.bias + nb);
      b4[0] = lo_of(bb.x); b4[1] = hi_of(bb.x); b4[2] = lo_of(bb.y); b4[3] = hi_of(bb.y);
    }
    if (a.cscale) {
      const u32x2_t cc = *reinterpret_cast<const u32x2_t*>(a.cscale + nb);
      c4[0] = lo_of(cc.x); c4[1] = hi_of(cc.x); c4[2] = lo_of(cc.y); c4[3] = hi_of(cc.y);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = 16 * mt + i;
      if (m >= a.M) continue;
      float o[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        o[v] = acc[mt][rt][0][v];
        for (int w = 0; w < nw - 1; ++w) o[v] += red[((w * MT + mt) * RT + rt) * 256 + v * 64 + lane];
      }
      if (a.R > 0) {
        // adapter: sum_r bf16(h[m][r] * lscale) * lora_b[n][r], the operands the large-M kernel feeds its MFMA
        float l4[4] = {0.f, 0.f, 0.f, 0.f};
        for (int r0 = 0; r0 < a.R; r0 += 8) {
          const u32x4_t hv = *reinterpret_cast<const u32x4_t*>(a.h + (int64_t)m * a.ldh + r0);
          float hs[8];
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            hs[2 * d] = round_to_bf16(lo_of(hv[d]) * a.lscale);
            hs[2 * d + 1] = round_to_bf16(hi_of(hv[d]) * a.lscale);
          }
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const u32x4_t bv = *reinterpret_cast<const u32x4_t*>(a.lora_b + (int64_t)(nb + v) * a.R + r0);
#pragma unroll
            for (int d = 0; d < 4; ++d) l4[v] += hs[2 * d] * lo_of(bv[d]) + hs[2 * d + 1] * hi_of(bv[d]);
          }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) o[v] += l4[v];
      }
      u32x2_t out;
      out.x = pack_pair((o[0] + b4[0]) * c4[0], (o[1] + b4[1]) * c4[1]);
      out.y = pack_pair((o[2] + b4[2]) * c4[2], (o[3] + b4[3]) * c4[3]);
      *reinterpret_cast<u32x2_t*>(a.y + (int64_t)m * a.N + nb) = out;
    }
  }
}

// Shape of a launch: token tiles, row tiles per workgroup, chunks in flight per wave, most waves.  It fixes the order
// in which a row's products are summed, so a layer gets the same bits alone and inside a group.
struct SmallMConfig {
  int mt, rt, u, max_waves;
  bool operator==(const SmallMConfig& o) const { return mt == o.mt && rt == o.rt && u == o.u && max_waves == o.max_waves; }
};
// Measured on MI355X over the projections of an 8B model (kernel time, M = 1 / 8 / 32 / 64): 4096 x 4096
// 7 / 7 / 13 / 20 us, 14336 x 4096 15 / 17 / 26 / 43 us, 4096 x 14336 14 / 18 / 37 / 64 us.  Wide layers share an x
// fragment between two row tiles once x is more than one token tile (x comes from L2 once per workgroup); long
// contractions get sixteen waves, short ones four.  From 9 tokens on the wide layers take two row tiles per workgroup as
// well: every workgroup reads all of x (16 tokens x 4096: 128 KB, 3.5 times the packed weight bytes over the 896
// workgroups of a 14336-wide layer), and twice the rows per workgroup halve that (M = 16: 1.33 -> 1.65 TB/s of packed weight).
SmallMConfig small_m_config(int64_t M, int64_t N, int64_t K) {
  const bool wide = N >= 8192, deep = K >= 8192;
  if (M <= 8) return {1, 1, 4, 16};
  if (M <= 16) return wide ? SmallMConfig{1, 2, 4, 16} : SmallMConfig{1, 1, 4, 16};
  if (M <= 32) return wide ? SmallMConfig{2, 2, 4, 4} : SmallMConfig{2, 1, 4, 4};
  return wide ? SmallMConfig{4, 2, 2, 4} : SmallMConfig{4, 1, 4, deep ? 16 : 4};
}

template <int MT, int RT, int U, int MAXW>
int launch_small_m(SmallMGroup& g, hipStream_t s) {
  static_assert(MAXW <= kSmMaxWaves, "the partial sums are laid out for at most kSmMaxWaves waves");
  const int K = g.m[0].K;
  int nw = ((K >> 7) + U - 1) / U;  // one group of U chunks per wave when K is short enough
  nw = nw > 1 ? nw : 1;
  nw = nw < MAXW ? nw : MAXW;
  // the partial sums of waves 1 .. nw - 1 must fit the 64 KB of LDS a workgroup gets without asking for more
  const int per_wave = MT * RT * 4 * 64 * (int)sizeof(float);
  const int fit = 1 + (63 * 1024) / per_wave;
  nw = nw < fit ? nw : fit;
  int wgs = 0;
  for (int i = 0; i < g.n; ++i) {
    wgs += g.m[i].N / (16 * RT);
    g.wg_end[i] = wgs;
  }
  const dim3 grid((unsigned)wgs), block(64 * nw);
  nf4_small_m_kernel<MT, RT, U, MAXW><<<grid, block, (size_t)(nw - 1) * per_wave, s>>>(g);
  return check_launch("nf4_small_m");
}

int dispatch_small_m(SmallMGroup& g, const SmallMConfig& c, hipStream_t s) {
  if (c.mt == 1) return c.rt == 2 ? launch_small_m<1, 2, 4, 16>(g, s) : launch_small_m<1, 1, 4, 16>(g, s);
  if (c.mt == 2) return c.rt == 2 ? launch_small_m<2, 2, 4, 4>(g, s) : launch_small_m<2, 1, 4, 4>(g, s);
  if (c.rt == 2) return launch_small_m<4, 2, 2, 4>(g, s);
  return c.max_waves > 4 ? launch_small_m<4, 1, 4, 16>(g, s) : launch_small_m<4, 1, 4, 4>(g, s);
}

}  // namespace

// Largest token count the small-M kernel takes; above it the tiled kernel runs.
int small_m_limit() { return 64; }

// Whether a forward of M tokens on an [N, K] weight goes to this kernel.  sliced_ok: the caller brought the workspace
// that lets the tiled kernel cut its contraction into slices.  Without it the tiled kernel fills 16 - 56 workgroups at
// these sizes and this kernel wins up to 64 tokens.  With it (measured, us, few-token / sliced at 24, 32, 40, 64 tokens):
// 4096 x 4096 13 / 17, 14 / 18, 20 / 19, 25 / 22; 14336 x 4096 29 / 23, 31 / 24, 40 / 25, 50 / 27; 4096 x 14336 33 / 24,
// 37 / 25, 50 / 26, 66 / 28: every workgroup of this kernel reads all of x, which at 64 tokens is seven times the
// packed weight, so from 17 tokens on the large weights and from 33 on all of them are better off in slices.
bool small_m_applies(int64_t M, int64_t N, int64_t K, bool sliced_ok) {
  if (M > small_m_limit()) return false;
  if (M <= 16 || !sliced_ok) return true;
  return M <= 32 && N * K <= (int64_t(1) << 25);
}

// Entries used by the C-ABI wrappers (arguments already validated there: N % 64 == 0, K % 64 == 0, R % 8 == 0, pointers
// aligned).  `bscal` is the natural [N, K/64] scaler layout; the rows of `h` are ldh elements apart.
int run_small_m(const void* x, const uint8_t* codes, const void* bscal, const void* h, int ldh, const void* lora_b, int R,
                float lscale, const void* bias, const void* cscale, void* y, int64_t M, int64_t N, int64_t K, hipStream_t s) {
  TT_REQUIRE(M > 0 && M <= small_m_limit(), "nf4_small_m: M (%lld) out of range", (long long)M);
  TT_REQUIRE(N / 16 < (int64_t(1) << 31) && N * K < (int64_t(1) << 40), "nf4_small_m: weight too large");
  SmallMGroup g = {};
  g.n = 1;
  SmallMArgs& a = g.m[0];
  a.x = reinterpret_cast<const uint16_t*>(x);
  a.codes = codes;
  a.bscal = reinterpret_cast<const float*>(bscal);
  a.h = reinterpret_cast<const uint16_t*>(h);
  a.lora_b = reinterpret_cast<const uint16_t*>(lora_b);
  a.bias = reinterpret_cast<const uint16_t*>(bias);
  a.cscale = reinterpret_cast<const uint16_t*>(cscale);
  a.y = reinterpret_cast<uint16_t*>(y);
  a.M = (int)M; a.N = (int)N; a.K = (int)K; a.R = R; a.ldh = ldh;
  a.lscale = lscale;
  return dispatch_small_m(g, small_m_config(M, N, K), s);
}

// The members of a group (same x, M, K) in as few launches as their launch shapes allow: consecutive members with
// the same shape share one.
int run_small_m_group(const void* x, const GroupGemm& gg, const void* h_cat, hipStream_t s) {
  TT_REQUIRE(gg.M > 0 && gg.M <= small_m_limit(), "nf4_small_m: M (%lld) out of range", (long long)gg.M);
  int i = 0;
  while (i < gg.n) {
    const SmallMConfig c = small_m_config(gg.M, gg.N[i], gg.K);
    SmallMGroup g = {};
    int j = i;
    for (; j < gg.n && small_m_config(gg.M, gg.N[j], gg.K) == c; ++j) {
      TT_REQUIRE(gg.N[j] / 16 < (int64_t(1) << 27) && gg.N[j] * gg.K < (int64_t(1) << 40), "nf4_small_m: weight too large");
      SmallMArgs& a = g.m[j - i];
      a.x = reinterpret_cast<const uint16_t*>(x);
      a.codes = gg.codes[j];
      a.bscal = gg.bscal[j];
      a.h = reinterpret_cast<const uint16_t*>(h_cat) + gg.r_off[j];
      a.lora_b = gg.lora_b[j];
      a.bias = gg.bias[j];
      a.cscale = nullptr;
      a.y = gg.y[j];
      a.M = (int)gg.M; a.N = (int)gg.N[j]; a.K = (int)gg.K; a.R = gg.rank[j]; a.ldh = gg.r_off[gg.n];
      a.lscale = gg.scale[j];
    }
    g.n = j - i;
    if (int rc = dispatch_small_m(g, c, s)) return rc;
    i = j;
  }
  return TTAMD_OK;
}

}  // namespace ttamd
