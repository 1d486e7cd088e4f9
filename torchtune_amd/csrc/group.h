// Internal interface between the translation units that serve a group of LoRA linears with a common input
// (q/k/v of torchtune/modules/attention.py:234,262-263; gate/up of torchtune/modules/feed_forward.py:50-53).
#pragma once
#include "common.h"

namespace ttamd {

constexpr int kGroupMax = TTAMD_GROUP_MAX;  // most members of a group

// What the rank-r products need to know about a group.  The members' hidden activations lie side by side in one
// [M, r_off[n]] tensor (member i in columns [r_off[i], r_off[i + 1])), and so do their gradients.
struct GroupSkinny {
  int n;
  int64_t M, K;
  int64_t N[kGroupMax];
  int rank[kGroupMax], r_off[kGroupMax + 1];
  float scale[kGroupMax];
  const uint16_t* lora_a[kGroupMax];  // [rank, K]
  const uint16_t* lora_b[kGroupMax];  // [N, rank]
  const uint16_t* gy[kGroupMax];      // [M, N]        (backward)
  uint16_t* ga[kGroupMax];            // [rank, K] out (backward)
  uint16_t* gb[kGroupMax];            // [N, rank] out (backward)
};

// What the fused NF4 GEMMs need to know about a group (forward).
struct GroupGemm {
  int n;
  int64_t M, K;
  int64_t N[kGroupMax];
  int rank[kGroupMax], r_off[kGroupMax + 1];
  float scale[kGroupMax];
  const uint8_t* codes[kGroupMax];    // [N, K/2]
  const float* bscal[kGroupMax];      // [N, K/64]
  const float* bscal_t[kGroupMax];    // [K/64, N] or null
  const uint16_t* lora_b[kGroupMax];  // [N, rank]
  const uint16_t* bias[kGroupMax];    // [N] or null
  uint16_t* y[kGroupMax];             // [M, N] out
};

// What the grouped grad-input needs (backward): the members' transposed copies and gradients.
struct GroupDx {
  int n;
  int64_t M, K;
  int64_t N[kGroupMax];
  int rank[kGroupMax], r_off[kGroupMax + 1];
  const uint16_t* gy[kGroupMax];       // [M, N]
  const uint8_t* codes_t[kGroupMax];   // [K, N/2] or null (then codes / bscal serve the expanded-weight path)
  const float* scal_t[kGroupMax];      // [K/64, N] or null
  const uint8_t* codes[kGroupMax];     // [N, K/2]
  const float* bscal[kGroupMax];       // [N, K/64]
  const uint16_t* lora_a[kGroupMax];   // [rank, K]
};

// nf4_gemm_rs.hip
int run_gemm_rs(const void* X, const uint8_t* codes, const void* scal, int mode, const void* lX, int ldlx, const void* lW,
                bool lw_row_major, int R, float lscale, const void* bias, const void* cscale, void* C, int64_t M, int64_t Nout,
                int64_t Kc, void* workspace, size_t workspace_bytes, hipStream_t s);
size_t gemm_rs_workspace_bytes(int64_t M, int64_t Nout, int64_t Kc);
int run_gemm_rs_group_dx(const GroupDx& d, const void* gh_cat, void* gx, hipStream_t s);

// nf4_gemm_dense.hip: expand the weight once into scratch memory, then a plain bf16 GEMM (many tokens)
bool dense_path_applies(int64_t M, int64_t Nout, int64_t Kc);
size_t dense_workspace_bytes(int64_t M, int64_t Nout, int64_t Kc);
// The result taken as the gradient of silu(gate) * up (gate, up [M, Nout] bf16): C receives the gradient of gate, gup
// that of up, and the result itself is not stored.
struct DenseSwigluBwd {
  const void* gate;
  const void* up;
  void* gup;
};
int run_gemm_dense(const void* X, const uint8_t* codes, const void* scal, int mode, const void* lX, int ldlx, const void* lW,
                   bool lw_row_major, int R, float lscale, const void* bias, const void* cscale, void* C, int64_t M, int64_t Nout,
                   int64_t Kc, void* workspace, hipStream_t s, const DenseSwigluBwd* swiglu_bwd = nullptr);
size_t dense_group_fwd_workspace_bytes(const GroupGemm& d);
// act != nullptr: two members of equal width (gate, up); the launch also writes act = silu(y[0]) * y[1]
bool dense_group_gated_applies(const GroupGemm& d);
int run_gemm_dense_group_fwd(const void* x, const GroupGemm& d, const void* h_cat, void* workspace, hipStream_t s, void* act = nullptr,
                             const void* tiles = nullptr);
size_t dense_group_dx_workspace_bytes(const GroupDx& d);
int run_gemm_dense_group_dx(const GroupDx& d, const void* gh_cat, void* gx, void* workspace, hipStream_t s,
                            const void* tiles_fwd = nullptr, bool paired = false);

// nf4_small_m.hip: y[i] = x . D(W_i)^T (+ bias) + scale . h_i . lora_b[i]^T for a handful of tokens
int small_m_limit();
// the forward of M tokens on an [N, K] weight runs the few-token kernel (sliced_ok: a slicing workspace is at hand)
bool small_m_applies(int64_t M, int64_t N, int64_t K, bool sliced_ok);
int run_small_m_group(const void* x, const GroupGemm& g, const void* h_cat, hipStream_t s);

// lora_skinny.hip
size_t group_hidden_ws_bytes(int64_t M, int64_t K, int r_total);
// h_cat[:, r_off[i] : r_off[i + 1]] = x . lora_a[i]^T for every member, in one pass over x
int run_group_hidden(const uint16_t* x, const GroupSkinny& g, uint16_t* h_cat, float* ws, hipStream_t s);
size_t group_lora_bwd_ws_bytes(const GroupSkinny& g);
// gh_cat[:, member i] = scale[i] . gy[i] . lora_b[i];  ga[i] = gh_i^T . x (one pass over x for all members);
// gb[i] = scale[i] . gy[i]^T . h_i
// sw (optional; the gate / up pair of a SwiGLU feed-forward): g.gy[0] and g.gy[1] are then OUTPUTS, the gradients of gate
// and up, which this call derives from the gradient of silu(gate) * up first - in the same pass that forms the products
// reading them where that pass exists (two wide members of equal width), otherwise by the stand-alone kernel.
struct SwigluBwdInputs {
  const uint16_t* gact;  // [M, N]
  const uint16_t* gate;  // [M, N]
  const uint16_t* up;    // [M, N]
};
int run_group_lora_bwd(const uint16_t* x, const uint16_t* h_cat, const GroupSkinny& g, uint16_t* gh_cat, float* ws, hipStream_t s,
                       const SwigluBwdInputs* sw = nullptr);

}  // namespace ttamd
