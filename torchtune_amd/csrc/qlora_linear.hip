// One call per direction for a whole QLoRA layer: LoRALinear.forward (torchtune/modules/peft/lora.py:128-147) and the
// backward autograd derives for it.  The reference's unit is one Python call of the layer; the per-kernel entry points
// (ttamd_lora_hidden_bf16 -> ttamd_nf4_lora_linear_fwd_ws_bf16, ttamd_lora_bwd_bf16 -> ttamd_nf4_linear_bwd_dx_ws_bf16)
// need two calls per direction, each with a workspace query and a workspace of its own.  These two run the same
// launches in the same order out of ONE caller workspace, so the results are the two-call sequence's bit for bit and a
// binding crosses the ABI once per direction (at the single-layer size the host side of the calls is most of the wall
// time).  The stages of a direction run one after the other on the caller's stream, so their scratch regions share
// the workspace's bytes; only the backward's gh = scale . gy . B, which the second stage reads, has a region to itself.
#include "common.h"

namespace ttamd {
namespace {
size_t align256(size_t v) { return (v + 255) & ~size_t(255); }
size_t max2(size_t a, size_t b) { return a > b ? a : b; }

int check_layer(const char* who, int64_t M, int64_t N, int64_t K, int rank) {
  TT_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1 << 30) && N < (1 << 30) && K < (1 << 30), "%s: bad shape M=%lld N=%lld K=%lld", who,
             (long long)M, (long long)N, (long long)K);
  TT_REQUIRE(K % 64 == 0 && N % 64 == 0, "%s: K (%lld) and N (%lld) must be multiples of 64", who, (long long)K, (long long)N);
  TT_REQUIRE(rank >= 8 && rank <= 64 && rank % 8 == 0, "%s: the adapter rank (%d) must be a multiple of 8 in [8, 64]", who, rank);
  return TTAMD_OK;
}
}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" size_t ttamd_qlora_linear_fwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int rank) {
  if (M <= 0 || N <= 0 || K <= 0 || rank <= 0) return 0;
  return align256(max2(ttamd_lora_fwd_workspace_bytes(M, K, rank), ttamd_nf4_gemm_workspace_bytes(M, N, K)));
}

extern "C" int ttamd_qlora_linear_fwd_bf16(const void* x, const uint8_t* quantized_data, const void* block_scalers,
                                           const void* block_scalers_t, const void* lora_a, const void* lora_b, int rank, float scale,
                                           const void* bias, void* y, void* h, int64_t M, int64_t N, int64_t K, void* workspace,
                                           size_t workspace_bytes, void* stream) {
  if (int rc = check_layer("qlora_linear_fwd", M, N, K, rank)) return rc;
  TT_REQUIRE(x && quantized_data && block_scalers && lora_a && lora_b && y && h, "qlora_linear_fwd: null pointer argument");
  const size_t need = ttamd_qlora_linear_fwd_workspace_bytes(M, N, K, rank);
  TT_REQUIRE(need == 0 || (workspace && aligned16(workspace)), "qlora_linear_fwd: workspace must be non-null and 16-byte aligned");
  if (workspace_bytes < need) return fail(TTAMD_EWORKSPACE, "qlora_linear_fwd: workspace has %zu bytes, needs %zu", workspace_bytes, need);
  // stage 1: h = bf16(x . A^T); its partial sums are consumed before stage 2 starts on the same stream
  const size_t hid = ttamd_lora_fwd_workspace_bytes(M, K, rank);
  if (int rc = ttamd_lora_hidden_bf16(x, lora_a, h, M, K, rank, hid ? workspace : nullptr, hid, stream)) return rc;
  // stage 2: y = x . D(W)^T (+ bias) + scale . h . B^T
  const size_t gemm = ttamd_nf4_gemm_workspace_bytes(M, N, K);
  return ttamd_nf4_lora_linear_fwd_ws_bf16(x, quantized_data, block_scalers, block_scalers_t, h, lora_b, rank, scale, bias, nullptr, y, M,
                                           N, K, gemm ? workspace : nullptr, gemm, stream);
}

extern "C" size_t ttamd_qlora_linear_bwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int rank) {
  if (M <= 0 || N <= 0 || K <= 0 || rank <= 0) return 0;
  return align256((size_t)M * (size_t)rank * 2) +
         align256(max2(ttamd_lora_bwd_workspace_bytes(M, N, K, rank), ttamd_nf4_gemm_workspace_bytes(M, K, N)));
}

extern "C" int ttamd_qlora_linear_bwd_bf16(const void* gy, const void* x, const void* h, const uint8_t* quantized_data,
                                           const void* block_scalers, const uint8_t* quantized_data_t, const void* block_scalers_t,
                                           const void* tiles_fwd, const void* lora_a, const void* lora_b, int rank, float scale,
                                           void* gx, void* grad_lora_a, void* grad_lora_b, int64_t M, int64_t N, int64_t K,
                                           void* workspace, size_t workspace_bytes, void* stream) {
  if (int rc = check_layer("qlora_linear_bwd", M, N, K, rank)) return rc;
  TT_REQUIRE(gy && x && h && quantized_data && block_scalers && lora_a && lora_b && grad_lora_a && grad_lora_b,
             "qlora_linear_bwd: null pointer argument");
  TT_REQUIRE((quantized_data_t == nullptr) == (block_scalers_t == nullptr), "qlora_linear_bwd: pass both transposed copies or neither");
  // with the forward's tiles at hand (or no grad-input at all) the GEMM stage needs no scratch memory
  const size_t need = (tiles_fwd || !gx) ? align256((size_t)M * (size_t)rank * 2) + align256(ttamd_lora_bwd_workspace_bytes(M, N, K, rank))
                                         : ttamd_qlora_linear_bwd_workspace_bytes(M, N, K, rank);
  TT_REQUIRE(workspace && aligned16(workspace), "qlora_linear_bwd: workspace must be non-null and 16-byte aligned");
  if (workspace_bytes < need) return fail(TTAMD_EWORKSPACE, "qlora_linear_bwd: workspace has %zu bytes, needs %zu", workspace_bytes, need);
  char* ws = reinterpret_cast<char*>(workspace);
  void* gh = ws;
  char* rest = ws + align256((size_t)M * (size_t)rank * 2);
  // stage 1: gh = scale . gy . B, gA = gh^T . x, gB = scale . gy^T . h
  const size_t skinny = ttamd_lora_bwd_workspace_bytes(M, N, K, rank);
  if (int rc = ttamd_lora_bwd_bf16(gy, x, h, lora_b, scale, gh, grad_lora_a, grad_lora_b, M, N, K, rank, rest, skinny, stream)) return rc;
  if (gx == nullptr) return TTAMD_OK;  // the layer's input needs no gradient
  // the forward call's expanded weight is still at hand: the grad-input reads it (no expansion, no scratch memory)
  if (tiles_fwd) return ttamd_tiled_linear_dx_bf16(gy, tiles_fwd, gh, lora_a, rank, gx, M, N, K, stream);
  // stage 2: gx = gy . D(W) + gh . A.  Without the transposed copies only the expanded-weight launch takes a workspace.
  size_t gemm = ttamd_nf4_gemm_workspace_bytes(M, K, N);
  if (!quantized_data_t && !ttamd_nf4_gemm_expands_weight(M, K, N)) gemm = 0;
  return ttamd_nf4_linear_bwd_dx_ws_bf16(gy, quantized_data, block_scalers, quantized_data_t, block_scalers_t, gh, lora_a, rank, gx, M, N,
                                         K, gemm ? rest : nullptr, gemm, stream);
}
