// C entry points for a group of QLoRA linears that share their input: q/k/v of an attention layer
// (torchtune/modules/attention.py:234,262-263 calls q_proj, k_proj and v_proj on the same tensor) and gate/up of a
// feed-forward (torchtune/modules/feed_forward.py:50-53: w1 and w3).  The reference has no such call: each LoRALinear
// (torchtune/modules/peft/lora.py:128-147) is on its own there.  What a group saves over member-by-member calls:
//   forward   one pass over x for every member's h = x . A^T; a handful of tokens: one launch for the members' outputs
//   backward  one launch for the members' gh, one pass over x for every member's gA, one launch for all gA / gB sums,
//             one grad-input GEMM over the members' concatenated output columns instead of one GEMM per member plus
//             the additions of their results
#include "common.h"
#include "group.h"

namespace ttamd {
namespace {

struct Decoded {
  GroupSkinny sk;
  GroupGemm gm;
  GroupDx dx;
};

size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

int decode(const char* who, const ttamd_lora_group_member* m, int n, int64_t M, int64_t K, bool backward, Decoded& d) {
  TT_REQUIRE(m != nullptr && n >= 1 && n <= kGroupMax, "%s: a group has 1 to %d members (got %d)", who, kGroupMax, n);
  TT_REQUIRE(M > 0 && K > 0 && M < (1 << 30) && K < (1 << 30) && K % 64 == 0, "%s: bad shape M=%lld K=%lld (K must be a multiple of 64)",
             who, (long long)M, (long long)K);
  d = Decoded{};
  d.sk.n = d.gm.n = d.dx.n = n;
  d.sk.M = d.gm.M = d.dx.M = M;
  d.sk.K = d.gm.K = d.dx.K = K;
  int off = 0;
  for (int i = 0; i < n; ++i) {
    const ttamd_lora_group_member& e = m[i];
    TT_REQUIRE(e.N > 0 && e.N < (1 << 30) && e.N % 64 == 0, "%s: member %d: N (%lld) must be a positive multiple of 64", who, i, (long long)e.N);
    TT_REQUIRE(e.rank > 0 && e.rank % 8 == 0, "%s: member %d: rank (%d) must be a positive multiple of 8", who, i, e.rank);
    TT_REQUIRE(e.quantized_data && e.block_scalers && e.lora_a && e.lora_b && e.y, "%s: member %d: null pointer", who, i);
    TT_REQUIRE(aligned16(e.quantized_data) && aligned16(e.block_scalers) && aligned16(e.block_scalers_t) && aligned16(e.lora_a) &&
                   aligned16(e.lora_b) && aligned16(e.y) && (reinterpret_cast<uintptr_t>(e.bias) & 7u) == 0,
               "%s: member %d: pointers must be 16-byte aligned (bias: 8)", who, i);
    if (backward) TT_REQUIRE(e.grad_lora_a && e.grad_lora_b, "%s: member %d: null gradient output", who, i);
    d.sk.N[i] = d.gm.N[i] = d.dx.N[i] = e.N;
    d.sk.rank[i] = d.gm.rank[i] = d.dx.rank[i] = e.rank;
    d.sk.r_off[i] = d.gm.r_off[i] = d.dx.r_off[i] = off;
    off += e.rank;
    d.sk.scale[i] = d.gm.scale[i] = e.scale;
    d.sk.lora_a[i] = d.dx.lora_a[i] = reinterpret_cast<const uint16_t*>(e.lora_a);
    d.sk.lora_b[i] = d.gm.lora_b[i] = reinterpret_cast<const uint16_t*>(e.lora_b);
    d.sk.gy[i] = d.dx.gy[i] = reinterpret_cast<const uint16_t*>(e.y);
    d.sk.ga[i] = reinterpret_cast<uint16_t*>(e.grad_lora_a);
    d.sk.gb[i] = reinterpret_cast<uint16_t*>(e.grad_lora_b);
    d.gm.codes[i] = e.quantized_data;
    d.gm.bscal[i] = reinterpret_cast<const float*>(e.block_scalers);
    d.gm.bscal_t[i] = reinterpret_cast<const float*>(e.block_scalers_t);
    d.gm.bias[i] = reinterpret_cast<const uint16_t*>(e.bias);
    d.gm.y[i] = reinterpret_cast<uint16_t*>(e.y);
    d.dx.codes_t[i] = e.quantized_data_t;
    d.dx.scal_t[i] = e.quantized_data_t ? reinterpret_cast<const float*>(e.block_scalers_t) : nullptr;
    d.dx.codes[i] = e.quantized_data;
    d.dx.bscal[i] = reinterpret_cast<const float*>(e.block_scalers);
  }
  TT_REQUIRE(off <= 64, "%s: the ranks of a group sum to at most 64 (got %d)", who, off);
  d.sk.r_off[n] = d.gm.r_off[n] = d.dx.r_off[n] = off;
  return TTAMD_OK;
}

// slices of the largest sliced member GEMM, or the expanded weight(s) of the many-token path
// the few-token launch serves the group when it would serve the member with the largest weight
bool group_small_m(const Decoded& d, bool sliced_ok) {
  int64_t n_max = 0;
  for (int i = 0; i < d.gm.n; ++i) n_max = d.gm.N[i] > n_max ? d.gm.N[i] : n_max;
  return small_m_applies(d.gm.M, n_max, d.gm.K, sliced_ok);
}

size_t fwd_gemm_ws(const Decoded& d) {
  const bool tiled = !group_small_m(d, true);
  size_t w = tiled ? dense_group_fwd_workspace_bytes(d.gm) : 0;
  if (tiled)
    for (int i = 0; i < d.gm.n; ++i) {
      const size_t b = gemm_rs_workspace_bytes(d.gm.M, d.gm.N[i], d.gm.K);
      w = b > w ? b : w;
    }
  return w;
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" size_t ttamd_lora_group_hidden_workspace_bytes(const ttamd_lora_group_member* members, int n_members, int64_t M,
                                                          int64_t K) {
  Decoded d;
  if (decode("lora_group_hidden_workspace_bytes", members, n_members, M, K, false, d) != TTAMD_OK) return 0;
  return align256(group_hidden_ws_bytes(M, K, d.sk.r_off[d.sk.n]));
}

extern "C" int ttamd_lora_group_hidden_bf16(const void* x, const ttamd_lora_group_member* members, int n_members, void* h_cat,
                                            int64_t M, int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  Decoded d;
  if (int rc = decode("lora_group_hidden", members, n_members, M, K, false, d)) return rc;
  TT_REQUIRE(x && h_cat && aligned16(x) && aligned16(h_cat), "lora_group_hidden: x and h_cat must be non-null and 16-byte aligned");
  const size_t need = align256(group_hidden_ws_bytes(M, K, d.sk.r_off[d.sk.n]));
  if (need > 0) {
    TT_REQUIRE(workspace && aligned16(workspace), "lora_group_hidden: workspace must be non-null and 16-byte aligned");
    if (workspace_bytes < need)
      return fail(TTAMD_EWORKSPACE, "lora_group_hidden: workspace has %zu bytes, needs %zu", workspace_bytes, need);
  }
  return run_group_hidden(reinterpret_cast<const uint16_t*>(x), d.sk, reinterpret_cast<uint16_t*>(h_cat),
                          reinterpret_cast<float*>(workspace), reinterpret_cast<hipStream_t>(stream));
}

extern "C" size_t ttamd_lora_group_fwd_workspace_bytes(const ttamd_lora_group_member* members, int n_members, int64_t M, int64_t K) {
  Decoded d;
  if (decode("lora_group_fwd_workspace_bytes", members, n_members, M, K, false, d) != TTAMD_OK) return 0;
  return align256(fwd_gemm_ws(d));
}

namespace {
// The members' outputs; *act_done says whether a launch that was asked for the gated product (act != nullptr) wrote it.
int group_fwd(const char* who, const void* x, const ttamd_lora_group_member* members, int n_members, const void* h_cat, void* act,
              bool* act_done, int64_t M, int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  Decoded d;
  if (int rc = decode(who, members, n_members, M, K, false, d)) return rc;
  TT_REQUIRE(x && h_cat && aligned16(x) && aligned16(h_cat), "%s: x and h_cat must be non-null and 16-byte aligned", who);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // slices of the contraction for a member with few output tiles, when the caller brought the memory for them
  const size_t gem = align256(fwd_gemm_ws(d));
  const bool sliced = gem > 0 && workspace != nullptr && workspace_bytes >= gem;
  if (group_small_m(d, sliced)) return run_small_m_group(x, d.gm, h_cat, s);
  TT_REQUIRE(!sliced || aligned16(workspace), "%s: workspace must be 16-byte aligned", who);
  // many tokens: one launch over the members' concatenated output columns, every weight expanded once
  if (sliced && dense_group_fwd_workspace_bytes(d.gm) > 0) {
    const bool gated = act != nullptr && dense_group_gated_applies(d.gm);
    if (act_done) *act_done = gated;
    return run_gemm_dense_group_fwd(x, d.gm, h_cat, workspace, s, gated ? act : nullptr);
  }
  const int ldh = d.gm.r_off[d.gm.n];
  for (int i = 0; i < d.gm.n; ++i) {
    const void* sc = d.gm.bscal_t[i] ? d.gm.bscal_t[i] : d.gm.bscal[i];
    if (int rc = run_gemm_rs(x, d.gm.codes[i], sc, d.gm.bscal_t[i] ? 2 : 0, reinterpret_cast<const uint16_t*>(h_cat) + d.gm.r_off[i], ldh,
                             d.gm.lora_b[i], true, d.gm.rank[i], d.gm.scale[i], d.gm.bias[i], nullptr, d.gm.y[i], M, d.gm.N[i], K,
                             sliced ? workspace : nullptr, sliced ? workspace_bytes : 0, s))
      return rc;
  }
  return TTAMD_OK;
}
}  // namespace

extern "C" int ttamd_nf4_lora_group_fwd_bf16(const void* x, const ttamd_lora_group_member* members, int n_members,
                                             const void* h_cat, int64_t M, int64_t K, void* workspace, size_t workspace_bytes,
                                             void* stream) {
  return group_fwd("nf4_lora_group_fwd", x, members, n_members, h_cat, nullptr, nullptr, M, K, workspace, workspace_bytes, stream);
}

extern "C" int ttamd_nf4_lora_group_swiglu_fwd_bf16(const void* x, const ttamd_lora_group_member* members, int n_members,
                                                    const void* h_cat, void* act, int64_t M, int64_t K, void* workspace,
                                                    size_t workspace_bytes, void* stream) {
  TT_REQUIRE(n_members == 2 && members && members[0].N == members[1].N,
             "nf4_lora_group_swiglu_fwd: takes the gate and the up projection, two members of equal width");
  TT_REQUIRE(act && aligned16(act), "nf4_lora_group_swiglu_fwd: act must be non-null and 16-byte aligned");
  bool done = false;
  if (int rc = group_fwd("nf4_lora_group_swiglu_fwd", x, members, n_members, h_cat, act, &done, M, K, workspace, workspace_bytes, stream))
    return rc;
  if (done) return TTAMD_OK;
  // shapes the many-token launch does not serve: the same arithmetic as its own pass over the two outputs
  return ttamd_swiglu_fwd_bf16(members[0].y, members[1].y, act, M * members[0].N, stream);
}

extern "C" size_t ttamd_lora_group_bwd_workspace_bytes(const ttamd_lora_group_member* members, int n_members, int64_t M, int64_t K) {
  Decoded d;
  if (decode("lora_group_bwd_workspace_bytes", members, n_members, M, K, false, d) != TTAMD_OK) return 0;
  return group_lora_bwd_ws_bytes(d.sk);
}

extern "C" int ttamd_lora_group_bwd_bf16(const void* x, const void* h_cat, const ttamd_lora_group_member* members, int n_members,
                                         void* gh_cat, int64_t M, int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  Decoded d;
  if (int rc = decode("lora_group_bwd", members, n_members, M, K, true, d)) return rc;
  TT_REQUIRE(x && h_cat && gh_cat && workspace, "lora_group_bwd: null pointer argument");
  TT_REQUIRE(aligned16(x) && aligned16(h_cat) && aligned16(gh_cat) && aligned16(workspace), "lora_group_bwd: pointers must be 16-byte aligned");
  const size_t need = group_lora_bwd_ws_bytes(d.sk);
  if (workspace_bytes < need) return fail(TTAMD_EWORKSPACE, "lora_group_bwd: workspace has %zu bytes, needs %zu", workspace_bytes, need);
  return run_group_lora_bwd(reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint16_t*>(h_cat), d.sk,
                            reinterpret_cast<uint16_t*>(gh_cat), reinterpret_cast<float*>(workspace), reinterpret_cast<hipStream_t>(stream));
}

// The pair's adapter backward from the gradient of silu(gate) * up: members[0] = gate, members[1] = up, members[i].y = OUT
// (the gradients of the two projections, which the grouped grad-input then reads).
extern "C" int ttamd_lora_group_swiglu_bwd_bf16(const void* x, const void* h_cat, const ttamd_lora_group_member* members, int n_members,
                                                const void* gact, const void* gate, const void* up, void* gh_cat, int64_t M, int64_t K,
                                                void* workspace, size_t workspace_bytes, void* stream) {
  TT_REQUIRE(n_members == 2 && members && members[0].N == members[1].N,
             "lora_group_swiglu_bwd: takes the gate and the up projection, two members of equal width");
  Decoded d;
  if (int rc = decode("lora_group_swiglu_bwd", members, n_members, M, K, true, d)) return rc;
  TT_REQUIRE(x && h_cat && gh_cat && workspace && gact && gate && up, "lora_group_swiglu_bwd: null pointer argument");
  TT_REQUIRE(aligned16(x) && aligned16(h_cat) && aligned16(gh_cat) && aligned16(workspace), "lora_group_swiglu_bwd: pointers must be 16-byte aligned");
  const size_t need = group_lora_bwd_ws_bytes(d.sk);
  if (workspace_bytes < need) return fail(TTAMD_EWORKSPACE, "lora_group_swiglu_bwd: workspace has %zu bytes, needs %zu", workspace_bytes, need);
  const SwigluBwdInputs sw = {reinterpret_cast<const uint16_t*>(gact), reinterpret_cast<const uint16_t*>(gate),
                              reinterpret_cast<const uint16_t*>(up)};
  return run_group_lora_bwd(reinterpret_cast<const uint16_t*>(x), reinterpret_cast<const uint16_t*>(h_cat), d.sk,
                            reinterpret_cast<uint16_t*>(gh_cat), reinterpret_cast<float*>(workspace), reinterpret_cast<hipStream_t>(stream), &sw);
}

extern "C" int ttamd_nf4_group_bwd_dx_bf16(const ttamd_lora_group_member* members, int n_members, const void* gh_cat, void* gx,
                                           int64_t M, int64_t K, void* stream) {
  Decoded d;
  if (int rc = decode("nf4_group_bwd_dx", members, n_members, M, K, false, d)) return rc;
  TT_REQUIRE(gh_cat && gx && aligned16(gh_cat) && aligned16(gx), "nf4_group_bwd_dx: gh_cat and gx must be non-null and 16-byte aligned");
  for (int i = 0; i < n_members; ++i)
    TT_REQUIRE(d.dx.codes_t[i] && d.dx.scal_t[i] && aligned16(d.dx.codes_t[i]),
               "nf4_group_bwd_dx: member %d: needs the transposed copies (ttamd_nf4_transpose_for_backward), 16-byte aligned", i);
  return run_gemm_rs_group_dx(d.dx, gh_cat, gx, reinterpret_cast<hipStream_t>(stream));
}

extern "C" size_t ttamd_nf4_group_bwd_dx_workspace_bytes(const ttamd_lora_group_member* members, int n_members, int64_t M, int64_t K) {
  Decoded d;
  if (decode("nf4_group_bwd_dx_workspace_bytes", members, n_members, M, K, false, d) != TTAMD_OK) return 0;
  return dense_group_dx_workspace_bytes(d.dx);
}

extern "C" int ttamd_nf4_group_bwd_dx_ws_bf16(const ttamd_lora_group_member* members, int n_members, const void* gh_cat, void* gx,
                                              int64_t M, int64_t K, void* workspace, size_t workspace_bytes, void* stream) {
  Decoded d;
  if (int rc = decode("nf4_group_bwd_dx", members, n_members, M, K, false, d)) return rc;
  const size_t need = dense_group_dx_workspace_bytes(d.dx);
  if (need == 0 || workspace == nullptr || workspace_bytes < need)
    return ttamd_nf4_group_bwd_dx_bf16(members, n_members, gh_cat, gx, M, K, stream);
  TT_REQUIRE(gh_cat && gx && aligned16(gh_cat) && aligned16(gx), "nf4_group_bwd_dx: gh_cat and gx must be non-null and 16-byte aligned");
  // members without transposed copies are expanded from the weight's own codes
  return run_gemm_dense_group_dx(d.dx, gh_cat, gx, workspace, reinterpret_cast<hipStream_t>(stream));
}

// Which expanded tiles a forward call of the group leaves at the start of the workspace it was given (when that workspace
// was large enough): 0 none (few tokens, slices, the fused kernel), 1 the members' weights stacked by rows in forward
// tile order, 2 the gated pair's layout (swiglu != 0: 128 columns of the gate, then 128 of the up projection).
extern "C" int ttamd_nf4_group_fwd_leaves_tiles(const ttamd_lora_group_member* members, int n_members, int64_t M, int64_t K, int swiglu) {
  Decoded d;
  if (decode("nf4_group_fwd_leaves_tiles", members, n_members, M, K, false, d) != TTAMD_OK) return 0;
  if (group_small_m(d, true) || dense_group_fwd_workspace_bytes(d.gm) == 0) return 0;
  return swiglu && dense_group_gated_applies(d.gm) ? 2 : 1;
}

extern "C" int ttamd_nf4_group_bwd_dx_tiles_bf16(const ttamd_lora_group_member* members, int n_members, const void* gh_cat, void* gx,
                                                 int64_t M, int64_t K, const void* tiles_fwd, int paired, void* stream) {
  Decoded d;
  if (int rc = decode("nf4_group_bwd_dx_tiles", members, n_members, M, K, false, d)) return rc;
  TT_REQUIRE(gh_cat && gx && tiles_fwd && aligned16(gh_cat) && aligned16(gx) && aligned16(tiles_fwd),
             "nf4_group_bwd_dx_tiles: gh_cat, gx and tiles_fwd must be non-null and 16-byte aligned");
  TT_REQUIRE(!paired || (n_members == 2 && members[0].N == members[1].N && members[0].N % 128 == 0),
             "nf4_group_bwd_dx_tiles: paired tiles belong to two members of equal width, a multiple of 128");
  for (int i = 0; i < n_members; ++i)
    TT_REQUIRE(members[i].N % 256 == 0 || paired, "nf4_group_bwd_dx_tiles: member %d: N (%lld) must be a multiple of 256 (as the forward launch required)",
               i, (long long)members[i].N);
  if (dense_group_dx_workspace_bytes(d.dx) == 0)
    return fail(TTAMD_EUNSUPPORTED, "nf4_group_bwd_dx_tiles: shape not served by the many-token launch (M=%lld K=%lld)", (long long)M, (long long)K);
  return run_gemm_dense_group_dx(d.dx, gh_cat, gx, nullptr, reinterpret_cast<hipStream_t>(stream), tiles_fwd, paired != 0);
}

// The group's forward on tiles an earlier forward call of the same members left behind (layout 1 or 2 of
// ttamd_nf4_group_fwd_leaves_tiles): the many-token launch without its expansion launches.
extern "C" int ttamd_nf4_lora_group_fwd_tiles_bf16(const void* x, const ttamd_lora_group_member* members, int n_members,
                                                   const void* h_cat, void* act, int64_t M, int64_t K, const void* tiles_fwd,
                                                   int paired, void* stream) {
  Decoded d;
  if (int rc = decode("nf4_lora_group_fwd_tiles", members, n_members, M, K, false, d)) return rc;
  TT_REQUIRE(x && h_cat && tiles_fwd && aligned16(x) && aligned16(h_cat) && aligned16(tiles_fwd),
             "nf4_lora_group_fwd_tiles: x, h_cat and tiles_fwd must be non-null and 16-byte aligned");
  TT_REQUIRE((paired != 0) == (act != nullptr), "nf4_lora_group_fwd_tiles: paired tiles are those of the call that writes act, and only those");
  TT_REQUIRE(!act || aligned16(act), "nf4_lora_group_fwd_tiles: act must be 16-byte aligned");
  if (group_small_m(d, true) || dense_group_fwd_workspace_bytes(d.gm) == 0 || (paired && !dense_group_gated_applies(d.gm)))
    return fail(TTAMD_EUNSUPPORTED, "nf4_lora_group_fwd_tiles: shape not served by the many-token launch (M=%lld K=%lld)", (long long)M,
                (long long)K);
  return run_gemm_dense_group_fwd(x, d.gm, h_cat, nullptr, reinterpret_cast<hipStream_t>(stream), act, tiles_fwd);
}
