// A plain C++ host of libtorchtune_amd.so: no Python, no torch.  It is what a compiled caller of the C ABI looks like
// (include/torchtune_amd.h, hipMalloc'd pointers, a HIP stream) and doubles as a parity test of the boundary:
//
//   1. to_nf4            ttamd_nf4_quantize      bytes must equal the scalar C oracle's (oracle/nf4_ref.c)
//   2. .to(bf16)         ttamd_nf4_dequantize    bits must equal the oracle's
//   3. LoRALinear.forward  ttamd_nf4_block_scalers + ttamd_lora_hidden_bf16 + ttamd_nf4_lora_linear_fwd_bf16
//                        within rtol/atol 1e-2 of a double-precision loop over the dequantised weight
//   4. LoRALinear backward ttamd_lora_bwd_bf16 + ttamd_nf4_transpose_for_backward + ttamd_nf4_linear_bwd_dx_bf16
//                        grad-input within 1e-2 of the same loop
//   5. error convention  a bad argument returns a negative code and leaves a message in ttamd_last_error()
//
// Test infrastructure: links the oracle, so it lives under tests/ and is never part of the shipped library.
// Build (done by __graft_entry__.build()):
//   hipcc -O2 -std=c++17 tests/c_abi_host.cpp -Iinclude -Ltorchtune_amd/lib -ltorchtune_amd -Loracle/_build -lttamd_oracle
//         -Wl,-rpath,$ORIGIN/../../torchtune_amd/lib -Wl,-rpath,$ORIGIN/../../oracle/_build -o tests/_build/c_abi_host
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "torchtune_amd.h"

extern "C" {
void ref_nf4_quantize(const void* w, int is_bf16, int64_t numel, int block_size, int scaler_block_size, uint8_t* qdata,
                      int8_t* qscalers, void* qfactor, void* mean, float* absmax_out);
void ref_nf4_dequantize(const uint8_t* qdata, const int8_t* qscalers, const void* qfactor, const void* mean, int is_bf16,
                        int64_t numel, int block_size, int scaler_block_size, void* out);
}

#define HIP_OK(call)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess) {                                                                 \
      std::fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      std::exit(2);                                                                         \
    }                                                                                       \
  } while (0)
#define TT_OK(call)                                                                              \
  do {                                                                                           \
    int rc_ = (call);                                                                            \
    if (rc_ != 0) {                                                                              \
      std::fprintf(stderr, "%s:%d: %s -> %d: %s\n", __FILE__, __LINE__, #call, rc_, ttamd_last_error()); \
      std::exit(3);                                                                              \
    }                                                                                            \
  } while (0)

static uint16_t to_bf16(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// seeded, roughly normal values (sum of four uniforms), no libc rand state involved
struct Rng {
  uint64_t s;
  float uniform() {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return (float)((s >> 40) & 0xffffff) / 16777216.0f;
  }
  float normalish() { return (uniform() + uniform() + uniform() + uniform() - 2.0f) * 1.7320508f; }
};

static std::vector<uint16_t> random_bf16(size_t n, float std_dev, uint64_t seed) {
  Rng r{seed};
  std::vector<uint16_t> v(n);
  for (auto& x : v) x = to_bf16(r.normalish() * std_dev);
  return v;
}

template <typename T>
static T* to_device(const std::vector<T>& h) {
  T* d = nullptr;
  HIP_OK(hipMalloc(&d, h.size() * sizeof(T)));
  HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
  return d;
}
template <typename T>
static T* device_alloc(size_t n) {
  T* d = nullptr;
  HIP_OK(hipMalloc(&d, (n ? n : 1) * sizeof(T)));
  return d;
}
template <typename T>
static std::vector<T> to_host(const T* d, size_t n) {
  std::vector<T> h(n);
  HIP_OK(hipMemcpy(h.data(), d, n * sizeof(T), hipMemcpyDeviceToHost));
  return h;
}

static int n_fail = 0;
static void check(bool ok, const char* what) {
  std::printf("%-72s %s\n", what, ok ? "ok" : "FAILED");
  if (!ok) ++n_fail;
}

static bool close_enough(const std::vector<uint16_t>& got, const std::vector<double>& want, double rtol, double atol,
                         const char* what) {
  double worst = 0;
  size_t bad = 0;
  for (size_t i = 0; i < got.size(); ++i) {
    const double g = from_bf16(got[i]), err = std::fabs(g - want[i]), lim = atol + rtol * std::fabs(want[i]);
    if (!(err <= lim)) ++bad;
    if (err - lim > worst) worst = err - lim;
  }
  if (bad) std::printf("  %s: %zu of %zu elements outside rtol %.0e / atol %.0e (worst excess %.3g)\n", what, bad, got.size(), rtol, atol, worst);
  return bad == 0;
}

int main() {
  int n_dev = 0;
  if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev == 0) {
    std::fprintf(stderr, "c_abi_host: no GPU visible\n");
    return 77;
  }
  HIP_OK(hipSetDevice(0));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  std::printf("library version %d\n", ttamd_version());

  const int64_t M = 300, K = 1024, N = 512;  // M is deliberately not a multiple of any tile
  const int rank = 16, BS = 64, SBS = 256;
  const float alpha = 32.0f, scale = alpha / rank;
  const int64_t numel = N * K, n_blocks = numel / BS, n_factors = n_blocks / SBS;

  const auto w = random_bf16(numel, 0.02f, 1), x = random_bf16(M * K, 1.0f, 2), a = random_bf16(rank * K, 0.03f, 3),
             b = random_bf16(N * rank, 0.05f, 4), bias = random_bf16(N, 0.1f, 5), gy = random_bf16(M * N, 1.0f, 6);

  // ---- 1. quantise -------------------------------------------------------------------------------------------
  uint16_t* d_w = to_device(w);
  uint8_t* d_codes = device_alloc<uint8_t>(numel / 2);
  int8_t* d_qs = device_alloc<int8_t>(n_blocks);
  uint16_t* d_qf = device_alloc<uint16_t>(n_factors);
  uint16_t* d_mean = device_alloc<uint16_t>(1);
  const size_t q_ws_bytes = ttamd_nf4_quantize_workspace_bytes(numel, BS);
  char* d_qws = device_alloc<char>(q_ws_bytes);
  TT_OK(ttamd_nf4_quantize(d_w, TTAMD_BF16, numel, BS, SBS, d_codes, d_qs, d_qf, d_mean, d_qws, q_ws_bytes, stream));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<uint8_t> o_codes(numel / 2);
  std::vector<int8_t> o_qs(n_blocks);
  std::vector<uint16_t> o_qf(n_factors), o_mean(1);
  std::vector<float> o_absmax(n_blocks);
  ref_nf4_quantize(w.data(), 1, numel, BS, SBS, o_codes.data(), o_qs.data(), o_qf.data(), o_mean.data(), o_absmax.data());
  check(to_host(d_codes, numel / 2) == o_codes, "nf4_quantize: codes equal the C oracle's, byte for byte");
  check(to_host(d_qs, n_blocks) == o_qs, "nf4_quantize: int8 block scalers equal the oracle's");
  check(to_host(d_qf, n_factors) == o_qf && to_host(d_mean, 1) == o_mean, "nf4_quantize: quantization_factor and scaler_mean equal the oracle's");

  // ---- 2. dequantise -----------------------------------------------------------------------------------------
  uint16_t* d_dense = device_alloc<uint16_t>(numel);
  TT_OK(ttamd_nf4_dequantize(d_codes, d_qs, d_qf, d_mean, TTAMD_BF16, numel, BS, SBS, d_dense, stream));
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<uint16_t> o_dense(numel);
  ref_nf4_dequantize(o_codes.data(), o_qs.data(), o_qf.data(), o_mean.data(), 1, numel, BS, SBS, o_dense.data());
  const auto dense = to_host(d_dense, numel);
  check(dense == o_dense, "nf4_dequantize: dense bf16 weight equals the oracle's, bit for bit");

  // ---- 3. forward --------------------------------------------------------------------------------------------
  float* d_bs = device_alloc<float>(n_blocks);
  TT_OK(ttamd_nf4_block_scalers(d_qs, d_qf, d_mean, TTAMD_BF16, n_blocks, SBS, d_bs, stream));
  uint16_t *d_x = to_device(x), *d_a = to_device(a), *d_b = to_device(b), *d_bias = to_device(bias);
  uint16_t *d_h = device_alloc<uint16_t>(M * rank), *d_y = device_alloc<uint16_t>(M * N);
  const size_t f_ws_bytes = ttamd_lora_fwd_workspace_bytes(M, K, rank);
  char* d_fws = device_alloc<char>(f_ws_bytes);
  TT_OK(ttamd_lora_hidden_bf16(d_x, d_a, d_h, M, K, rank, d_fws, f_ws_bytes, stream));
  TT_OK(ttamd_nf4_lora_linear_fwd_bf16(d_x, d_codes, d_bs, nullptr, d_h, d_b, rank, scale, d_bias, d_y, M, N, K, stream));
  HIP_OK(hipStreamSynchronize(stream));
  const auto h = to_host(d_h, M * rank);
  std::vector<double> h_ref(M * rank), y_ref(M * N);
  for (int64_t m = 0; m < M; ++m)
    for (int r = 0; r < rank; ++r) {
      double s = 0;
      for (int64_t k = 0; k < K; ++k) s += (double)from_bf16(x[m * K + k]) * from_bf16(a[r * K + k]);
      h_ref[m * rank + r] = s;
    }
  check(close_enough(h, h_ref, 1e-2, 1e-2, "h"), "lora_hidden: h = x . A^T within 1e-2");
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      double s = from_bf16(bias[n]);
      for (int64_t k = 0; k < K; ++k) s += (double)from_bf16(x[m * K + k]) * from_bf16(dense[n * K + k]);
      for (int r = 0; r < rank; ++r) s += (double)scale * from_bf16(h[m * rank + r]) * from_bf16(b[n * rank + r]);
      y_ref[m * N + n] = s;
    }
  check(close_enough(to_host(d_y, M * N), y_ref, 1e-2, 1e-2, "y"), "nf4_lora_linear_fwd: y = x.D(W)^T + bias + s.h.B^T within 1e-2");

  // the same forward with the workspace that lets the library slice the contraction of this six-tile launch
  const size_t g_ws_bytes = ttamd_nf4_gemm_workspace_bytes(M, N, K);
  check(g_ws_bytes >= 2 * (size_t)M * N * sizeof(float), "nf4_gemm_workspace_bytes: a launch of few tiles asks for at least two slices");
  char* d_gws = device_alloc<char>(g_ws_bytes);
  uint16_t* d_y2 = device_alloc<uint16_t>(M * N);
  TT_OK(ttamd_nf4_lora_linear_fwd_ws_bf16(d_x, d_codes, d_bs, nullptr, d_h, d_b, rank, scale, d_bias, nullptr, d_y2, M, N, K, d_gws,
                                          g_ws_bytes, stream));
  HIP_OK(hipStreamSynchronize(stream));
  check(close_enough(to_host(d_y2, M * N), y_ref, 1e-2, 1e-2, "y (sliced)"), "nf4_lora_linear_fwd_ws: the sliced contraction gives the same y within 1e-2");

  // ---- 4. backward -------------------------------------------------------------------------------------------
  uint16_t* d_gy = to_device(gy);
  uint16_t *d_gh = device_alloc<uint16_t>(M * rank), *d_ga = device_alloc<uint16_t>(rank * K), *d_gb = device_alloc<uint16_t>(N * rank);
  const size_t b_ws_bytes = ttamd_lora_bwd_workspace_bytes(M, N, K, rank);
  char* d_bws = device_alloc<char>(b_ws_bytes);
  TT_OK(ttamd_lora_bwd_bf16(d_gy, d_x, d_h, d_b, scale, d_gh, d_ga, d_gb, M, N, K, rank, d_bws, b_ws_bytes, stream));
  uint8_t* d_codes_t = device_alloc<uint8_t>(numel / 2);
  float* d_bs_t = device_alloc<float>(n_blocks);
  TT_OK(ttamd_nf4_transpose_for_backward(d_codes, d_bs, N, K, d_codes_t, d_bs_t, stream));
  uint16_t* d_gx = device_alloc<uint16_t>(M * K);
  TT_OK(ttamd_nf4_linear_bwd_dx_bf16(d_gy, d_codes, d_bs, d_codes_t, d_bs_t, d_gh, d_a, rank, d_gx, M, N, K, stream));
  HIP_OK(hipStreamSynchronize(stream));
  const auto gh = to_host(d_gh, M * rank);
  std::vector<double> gx_ref(M * K);
  for (int64_t m = 0; m < M; ++m)
    for (int64_t k = 0; k < K; ++k) {
      double s = 0;
      for (int64_t n = 0; n < N; ++n) s += (double)from_bf16(gy[m * N + n]) * from_bf16(dense[n * K + k]);
      for (int r = 0; r < rank; ++r) s += (double)from_bf16(gh[m * rank + r]) * from_bf16(a[r * K + k]);
      gx_ref[m * K + k] = s;
    }
  check(close_enough(to_host(d_gx, M * K), gx_ref, 1e-2, 1e-2, "gx"), "nf4_linear_bwd_dx: gx = gy.D(W) + gh.A within 1e-2");
  std::vector<double> gb_ref(N * rank);
  double gb_max = 0;
  for (int64_t n = 0; n < N; ++n)
    for (int r = 0; r < rank; ++r) {
      double s = 0;
      for (int64_t m = 0; m < M; ++m) s += (double)from_bf16(gy[m * N + n]) * from_bf16(h[m * rank + r]);
      gb_ref[n * rank + r] = scale * s;
      gb_max = std::fmax(gb_max, std::fabs(scale * s));
    }
  check(close_enough(to_host(d_gb, N * rank), gb_ref, 1e-2, 1e-2 * gb_max, "gB"), "lora_bwd: gB = s . gy^T . h within 1e-2 of its scale");

  // ---- 5. error convention -----------------------------------------------------------------------------------
  const int rc = ttamd_nf4_lora_linear_fwd_bf16(d_x, d_codes, d_bs, nullptr, d_h, d_b, rank, scale, d_bias, d_y, M, N, K + 8, stream);
  check(rc < 0 && std::strlen(ttamd_last_error()) > 0, "a K that is not a multiple of 64 is refused with a message");
  const int rc2 = ttamd_nf4_quantize(d_w, TTAMD_BF16, numel, BS, SBS, d_codes, d_qs, d_qf, d_mean, d_qws, 16, stream);
  check(rc2 < 0, "a workspace that is too small is refused");
  HIP_OK(hipDeviceSynchronize());

  std::printf(n_fail ? "c_abi_host: %d check(s) FAILED\n" : "c_abi_host: all checks passed\n", n_fail);
  return n_fail ? 1 : 0;
}
