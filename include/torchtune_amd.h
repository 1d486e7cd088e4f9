/*
 * torchtune_amd C ABI — MI355X (gfx950) kernels for the QLoRA / QAT quantized-linear path.
 *
 * The reference (pytorch/torchtune) has no native layer: the arithmetic of this path lives in eager
 * PyTorch op sequences inside the third-party `torchao` package.  Each entry point below therefore
 * cites the Python call site(s) in the reference whose work it replaces, not an FFI declaration.
 *
 * Conventions (all entry points):
 *   - plain C, no torch types; every pointer is a caller-owned DEVICE pointer unless stated, 16-byte
 *     aligned, row-major contiguous;
 *   - `stream` is a `hipStream_t` passed as `void*` (NULL = the default stream); work is enqueued
 *     asynchronously on it, nothing synchronises the host;
 *   - the return value is 0 on success or a negative `TTAMD_E*` code; `ttamd_last_error()` then gives
 *     a thread-local, human-readable message;
 *   - nothing here allocates or frees device memory: scratch space is passed in as `workspace`,
 *     sized by the matching `*_workspace_bytes` query;
 *   - the calls are re-entrant and keep no stream or device state between calls.  The one piece of process-wide
 *     state: the GEMM kernels that use more than 64 KB of LDS record per device, in a flag, that the runtime has
 *     been told so (`hipFuncSetAttribute`, once per device and kernel); two threads racing on a device's first call
 *     both make that call, which is harmless.  ttamd_lora_hidden_static_bf16 alone owns device memory (a fixed
 *     2 MiB array per GPU, see there).
 *
 * dtype codes: TTAMD_BF16 = bfloat16, TTAMD_F32 = float32.
 */
#ifndef TORCHTUNE_AMD_H
#define TORCHTUNE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TTAMD_ABI_VERSION 1

#define TTAMD_BF16 0
#define TTAMD_F32 1

#define TTAMD_GROUP_MAX 4 /* most members of a group of linears with a common input (ttamd_lora_group_*) */

#define TTAMD_OK 0
#define TTAMD_EINVAL (-1)     /* bad argument: null pointer, misaligned pointer, shape or divisibility violation */
#define TTAMD_EUNSUPPORTED (-2) /* valid request this build has no kernel for (e.g. fused GEMM with block_size != 64) */
#define TTAMD_EWORKSPACE (-3) /* workspace too small */
#define TTAMD_ELAUNCH (-4)    /* the HIP runtime reported an error at launch */

/* ABI version of the loaded library (== TTAMD_ABI_VERSION it was built with). */
int ttamd_version(void);

/* Message for the last non-zero return on the calling thread ("" if none). Host pointer, valid until the
 * next failing call on the same thread. */
const char* ttamd_last_error(void);

/* ------------------------------------------------------------------------------------------------
 * NF4 double-quantisation codec
 * ---------------------------------------------------------------------------------------------- */

/*
 * to_nf4(tensor, block_size, scaler_block_size): replaces torchao's NF4Tensor.from_tensor as called at
 *   torchtune/modules/peft/lora.py:86, torchtune/modules/low_precision/nf4_linear.py:49,
 *   torchtune/modules/low_precision/_register_nf4_dispatch_ops.py:20, torchtune/training/_distributed.py:404.
 *
 * w                    [numel] `dtype` (the flattened [N,K] weight)
 * quantized_data  out  [numel/2] uint8, two 4-bit codes per byte, even element in the high nibble
 * quantized_scalers out [numel/block_size] int8
 * quantization_factor out [numel/block_size/scaler_block_size] `dtype`
 * scaler_mean     out  [1] `dtype`
 * workspace            ttamd_nf4_quantize_workspace_bytes(numel, block_size) bytes
 *
 * Requires numel % block_size == 0, (numel/block_size) % scaler_block_size == 0, block_size % 8 == 0.
 * All arithmetic is carried out in `dtype` with round-to-nearest-even after every operation, as the eager
 * reference does.  A block whose absmax is 0 (0/0 = NaN distances) gets code 0 for every element; a NaN
 * scaled scaler quantises to 0.
 */
size_t ttamd_nf4_quantize_workspace_bytes(int64_t numel, int block_size);
int ttamd_nf4_quantize(const void* w, int dtype, int64_t numel, int block_size, int scaler_block_size,
                       uint8_t* quantized_data, int8_t* quantized_scalers, void* quantization_factor,
                       void* scaler_mean, void* workspace, size_t workspace_bytes, void* stream);

/*
 * NF4Tensor.get_original_weight() / NF4Tensor.to(dtype): replaces the torchao dequantisation chain reached from
 *   torchtune/modules/common_utils.py:57 (state-dict hook), torchtune/modules/peft/dora.py:137,183,
 *   torchtune/modules/low_precision/_register_nf4_dispatch_ops.py:20, torchtune/training/_distributed.py:523,
 *   and implicitly by linear_nf4 (lora.py:138, nf4_linear.py:67) in every forward and backward.
 *
 * `dtype` is the dtype of quantization_factor / scaler_mean and of `out` (the tensor's original dtype).
 * out [numel] `dtype`.
 */
int ttamd_nf4_dequantize(const uint8_t* quantized_data, const int8_t* quantized_scalers,
                         const void* quantization_factor, const void* scaler_mean, int dtype, int64_t numel,
                         int block_size, int scaler_block_size, void* out, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Fused NF4 + LoRA linear (bf16 activations, fp32 accumulate, NF4 block_size 64)
 *
 * One LoRALinear.forward (torchtune/modules/peft/lora.py:128-147) is two calls: ttamd_lora_hidden_bf16, then
 * ttamd_nf4_lora_linear_fwd_bf16.  Its backward is ttamd_lora_bwd_bf16 followed by ttamd_nf4_linear_bwd_dx_bf16.
 * FrozenNF4Linear.forward / linear_nf4 (torchtune/modules/low_precision/nf4_linear.py:56-70) is the rank == 0 case
 * of the two GEMM entry points alone.
 * ---------------------------------------------------------------------------------------------- */

/*
 * Dequantised block scalers of an NF4 tensor, one fp32 per 64-element block (the value is the tensor-dtype
 * result, widened exactly):
 *     block_scalers[b] = float( dtype( dtype(quantized_scalers[b] / quantization_factor[b / SB]) + scaler_mean ) )
 * This is the `dequantize_scalers` step of NF4Tensor.get_original_weight (torchao; reached from lora.py:138 on
 * every call).  The weight is frozen, so callers compute it once per tensor and keep it; the GEMMs below take it
 * in place of the three scaler tensors.  `dtype` is the dtype of quantization_factor / scaler_mean.
 */
int ttamd_nf4_block_scalers(const int8_t* quantized_scalers, const void* quantization_factor, const void* scaler_mean,
                            int dtype, int64_t n_blocks, int scaler_block_size, void* block_scalers, void* stream);

/*
 * Merged checkpoint weight of one QLoRA linear in a single pass over the packed weight:
 *   out = bf16( D(W) + bf16( scale * bf16(lora_b . lora_a) ) )
 * replaces the state-dict hook's NF4Tensor.to(bf16) (torchtune/modules/common_utils.py:55-59) followed by
 * get_merged_lora_ckpt's `weight += (alpha / rank) * lora_b @ lora_a` (torchtune/modules/peft/_utils.py:264-266),
 * with the same three bf16 roundings; the rank-r sum is accumulated in fp32 in ascending r.
 *
 * quantized_data = NF4 codes of the [N,K] weight (block_size 64); block_scalers fp32 [N*K/64] from
 * ttamd_nf4_block_scalers; lora_a [rank,K] bf16; lora_b [N,rank] bf16; scale = alpha / rank; out [N,K] bf16.
 * Requires K % 64 == 0, rank a multiple of 8 in [8,64].
 */
int ttamd_nf4_dequantize_merge_bf16(const uint8_t* quantized_data, const void* block_scalers, const void* lora_a,
                                    const void* lora_b, int rank, float scale, void* out, int64_t N, int64_t K,
                                    void* stream);

/*
 * h = bf16(x . lora_a^T): the adapter's hidden activation `self.lora_a(self.dropout(x))` (lora.py:144).
 * x [M,K] bf16, lora_a [rank,K] bf16, h out [M,rank] bf16; rank a multiple of 8 in [8,64], K % 64 == 0.
 * workspace: ttamd_lora_fwd_workspace_bytes(M, K, rank) bytes.
 */
size_t ttamd_lora_fwd_workspace_bytes(int64_t M, int64_t K, int rank);
int ttamd_lora_hidden_bf16(const void* x, const void* lora_a, void* h, int64_t M, int64_t K, int rank, void* workspace,
                           size_t workspace_bytes, void* stream);

/*
 * ttamd_lora_hidden_bf16 for callers that cannot allocate device memory or pass a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * arguments and bit-identical result; the partial sums of a launch that is cut along K go to a device array built
 * into the library (ttamd_lora_hidden_static_max_bytes() = 2 MiB per GPU, held until the process ends) instead of a
 * workspace.  Neither call allocates, frees or synchronises.  Returns TTAMD_EWORKSPACE if the shape would need more
 * than the built-in array (the plan of this build never does for rank <= 64).  All calls on one GPU share that
 * array: calls that overlap on the same GPU (different streams or threads) race on it and must be serialised by the
 * caller; calls on different GPUs are independent.  Nothing in the array has to start at zero.
 * The first use on a device asks the runtime for the array's device address (hipGetSymbolAddress, possibly a lazy
 * load of the code object): that query must not fall inside a stream capture.  Call ttamd_lora_hidden_static_init()
 * once per device, with that device current, before capturing (one eager call of the entry point does the same);
 * later calls only launch kernels.  Returns TTAMD_ELAUNCH if the runtime refuses the query.
 */
size_t ttamd_lora_hidden_static_max_bytes(void);
int ttamd_lora_hidden_static_init(void);
int ttamd_lora_hidden_static_bf16(const void* x, const void* lora_a, void* h, int64_t M, int64_t K, int rank, void* stream);

/*
 * y = x . D(W)^T (+ bias) + scale . h . lora_b^T          (lora.py:137-147; nf4_linear.py:67-70 when rank == 0)
 *
 * x [M,K] bf16; quantized_data = NF4 codes of the [N,K] weight (block_size 64); block_scalers from
 * ttamd_nf4_block_scalers; block_scalers_t = NULL or the same scalers transposed, fp32 [K/64, N], as
 * ttamd_nf4_transpose_for_backward writes them (then a wave fetches the 64 scalers of a k-step with one coalesced
 * load instead of two gathers; results are identical); h [M,rank] bf16 from ttamd_lora_hidden_bf16 and lora_b [N,rank] bf16 (both NULL iff
 * rank == 0); bias [N] bf16 or NULL; scale = alpha / rank; y out [M,N] bf16.
 * Requires K % 64 == 0, N % 64 == 0, rank % 8 == 0, 0 <= rank <= 64.
 * D(W) is bit-identical to ttamd_nf4_dequantize's output; all products are accumulated in fp32 and the sum is
 * rounded to bf16 once (the eager reference rounds after each of its five ops).
 * M <= 64 (decode, evaluation) runs a kernel that streams the packed weight once instead of the tiled one; same
 * operands, same expansion of the weight, fp32 sums in a different but fixed order.  (Through the _ws entry point below,
 * with the workspace its query asks for, that kernel serves M <= 16, and M <= 32 on weights of at most 2^25 elements;
 * above that every one of its workgroups reads more of x than of the weight and the sliced tiled kernel is faster.)
 */
int ttamd_nf4_lora_linear_fwd_bf16(const void* x, const uint8_t* quantized_data, const void* block_scalers,
                                   const void* block_scalers_t, const void* h, const void* lora_b, int rank, float scale,
                                   const void* bias, void* y, int64_t M, int64_t N, int64_t K, void* stream);

/*
 * DoRALinear (torchtune/modules/peft/dora.py:156-192) over an NF4 base weight.
 *
 * ttamd_nf4_dora_weight_norm_bf16: weight_norm[n] = bf16(|| D(W)[n,:] + bf16(scale * bf16(lora_b . lora_a))[n,:] ||_2)
 *   (dora.py:141-144, called in every forward at :183 and by initialize_dora_magnitude at :139), computed in one pass
 *   over the packed weight without materialising it; if magnitude [N] bf16 is given, also
 *   mag_norm_scale[n] = bf16(magnitude[n] / weight_norm[n]) (:185).  workspace:
 *   ttamd_dora_weight_norm_workspace_bytes(N, K) bytes.
 * ttamd_nf4_dora_linear_fwd_bf16: y = (x . D(W)^T + bias + scale . h . lora_b^T) * col_scale per output column,
 *   col_scale = mag_norm_scale [N] bf16 (:187-191 rearranged: (s - 1) base + s lora scale + base = s (base + lora scale));
 *   otherwise identical to ttamd_nf4_lora_linear_fwd_bf16.
 * ttamd_dora_bwd_prologue_bf16: from gy [M,N] and the layer's saved output y [M,N]:
 *   gy0 = bf16(gy * mag_norm_scale), the gradient for ttamd_lora_bwd_bf16 / ttamd_nf4_linear_bwd_dx_bf16, and
 *   gmagnitude[n] = bf16(sum_m gy[m,n] * y[m,n] / magnitude[n]) (fixed summation order; the norm is a constant in the
 *   reference's graph, :184).  workspace: ttamd_dora_bwd_workspace_bytes(N) bytes.
 */
size_t ttamd_dora_weight_norm_workspace_bytes(int64_t N, int64_t K);
int ttamd_nf4_dora_weight_norm_bf16(const uint8_t* quantized_data, const void* block_scalers, const void* lora_a,
                                    const void* lora_b, int rank, float scale, const void* magnitude, void* weight_norm,
                                    void* mag_norm_scale, int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                                    void* stream);
int ttamd_nf4_dora_linear_fwd_bf16(const void* x, const uint8_t* quantized_data, const void* block_scalers,
                                   const void* block_scalers_t, const void* h, const void* lora_b, int rank, float scale,
                                   const void* bias, const void* col_scale, void* y, int64_t M, int64_t N, int64_t K,
                                   void* stream);
size_t ttamd_dora_bwd_workspace_bytes(int64_t N);
int ttamd_dora_bwd_prologue_bf16(const void* gy, const void* out, const void* mag_norm_scale, const void* magnitude, void* gy0,
                                 void* gmagnitude, int64_t M, int64_t N, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Optional transposed copy of an NF4 weight for the grad-input GEMM.  NF4 blocks run along K, the grad-input GEMM
 * contracts over N; with the codes re-packed along N (quantized_data_t [K, N/2], even n in the high nibble) and the
 * block scalers transposed (block_scalers_t fp32 [K/64, N]) that GEMM streams the weight exactly like the forward
 * one.  Costs another 0.5625 B per weight element of device memory; derived data, built once per frozen tensor.
 * The reference has no counterpart (its backward re-materialises the whole bf16 weight: torchao LinearNF4.backward,
 * reached from torchtune/modules/peft/lora.py:138).
 */
int ttamd_nf4_transpose_for_backward(const uint8_t* quantized_data, const void* block_scalers, int64_t N, int64_t K,
                                     uint8_t* quantized_data_t, void* block_scalers_t, void* stream);

/*
 * gx = gy . D(W) + gh . lora_a: LinearNF4.backward (torchao; reached from lora.py:138, nf4_linear.py:67) plus the
 * term autograd adds for lora_a's input.  gy [M,N] bf16; gh [M,rank] bf16 from ttamd_lora_bwd_bf16 and
 * lora_a [rank,K] bf16 (both NULL iff rank == 0); gx out [M,K] bf16.  Same divisibility rules as the forward.
 * quantized_data_t / block_scalers_t: the copies made by ttamd_nf4_transpose_for_backward, or both NULL to run
 * the variant that transposes the weight tile on the fly (slower, no extra memory).
 */
int ttamd_nf4_linear_bwd_dx_bf16(const void* gy, const uint8_t* quantized_data, const void* block_scalers,
                                 const uint8_t* quantized_data_t, const void* block_scalers_t, const void* gh,
                                 const void* lora_a, int rank, void* gx, int64_t M, int64_t N, int64_t K, void* stream);

/*
 * The same two GEMMs for token counts between the few-token kernel and a full grid (17 - 64 tokens where the slices beat
 * the few-token kernel, see above, and 64 < M; at most 128 output tiles of 128 x 256): with a workspace the contraction is cut into up to 16 slices, one workgroup per tile per slice, fp32
 * partial tiles in the workspace, and a second kernel adds the slices in a fixed order, then bias, column scale and
 * the rounding to bf16.  The plain entry points above are these with workspace = NULL (no slicing: a launch of few
 * tiles then leaves most of the chip idle).  The reference has no counterpart: it dequantises the weight and calls a
 * dense GEMM (nf4_linear.py:67-70, lora.py:138).
 *   ttamd_nf4_gemm_workspace_bytes(M, n_out, k_contract): bytes to pass (0: the launch is not sliced); n_out /
 *     k_contract = N / K for the forward, K / N for the grad-input.
 *   ttamd_nf4_lora_linear_fwd_ws_bf16: col_scale NULL = ttamd_nf4_lora_linear_fwd_bf16, else = ttamd_nf4_dora_linear_fwd_bf16.
 *   ttamd_nf4_linear_bwd_dx_ws_bf16: slices only the variant with the transposed copies.
 * A workspace smaller than ttamd_nf4_gemm_workspace_bytes says, or NULL, runs the unsliced kernel.
 *
 * Many tokens (M >= 2048 and at least 256 output tiles of 256 x 256, or M >= 1280 and more than 128 such tiles, where
 * the fused kernel would need a second round of its 128-row tiles): the same workspace argument then holds the
 * weight expanded ONCE per call to bf16 (2 * n_out * k_contract bytes, in the order the matrix cores read it), and a
 * plain bf16 GEMM with the adapter, bias and column scale in its epilogue runs on it: the reference's own order of
 * work, F.linear(x, weight.to(dtype)) (torchao linear_nf4, reached from torchtune/modules/peft/lora.py:138), for the
 * token counts at which the fused kernel's per-tile expansion costs more than one pass of the expansion kernel.
 * ttamd_nf4_gemm_workspace_bytes reports those bytes; passing less (or NULL) keeps the fused kernel.  The expanded
 * values are the bits ttamd_nf4_dequantize writes.  The grad-input takes this path with or without the transposed
 * copies (without them W^T is expanded from quantized_data / block_scalers themselves, at the same speed), so a
 * caller that only ever runs many-token calls need not build them.
 */
size_t ttamd_nf4_gemm_workspace_bytes(int64_t M, int64_t n_out, int64_t k_contract);
/* 1 when those bytes are the expanded weight of the many-token path, 0 when they are slices (or none) */
int ttamd_nf4_gemm_expands_weight(int64_t M, int64_t n_out, int64_t k_contract);
int ttamd_nf4_lora_linear_fwd_ws_bf16(const void* x, const uint8_t* quantized_data, const void* block_scalers,
                                      const void* block_scalers_t, const void* h, const void* lora_b, int rank, float scale,
                                      const void* bias, const void* col_scale, void* y, int64_t M, int64_t N, int64_t K,
                                      void* workspace, size_t workspace_bytes, void* stream);
int ttamd_nf4_linear_bwd_dx_ws_bf16(const void* gy, const uint8_t* quantized_data, const void* block_scalers,
                                    const uint8_t* quantized_data_t, const void* block_scalers_t, const void* gh,
                                    const void* lora_a, int rank, void* gx, int64_t M, int64_t N, int64_t K, void* workspace,
                                    size_t workspace_bytes, void* stream);

/*
 * The grad-input of the layer that consumes a gated product, act = silu(gate) * up (the w2 of
 * torchtune/modules/feed_forward.py:53 applied to the product of :50-53), carried on to the gradients of gate and up:
 *     gact  = bf16(gy . D(W) + gh . lora_a)                    (what ttamd_nf4_linear_bwd_dx_ws_bf16 writes as gx)
 *     ggate, gup = ttamd_swiglu_bwd_bf16(gact, gate, up)       bit for bit
 * gate, up, ggate, gup [M,K] bf16; the other arguments as for ttamd_nf4_linear_bwd_dx_ws_bf16.  On the many-token path
 * (the workspace holds the expanded weight) the GEMM's epilogue reads gate and up and writes the two gradients itself:
 * gact never reaches memory (one write and one read of [M,K] less, and no launch of the stand-alone kernel).  At other
 * sizes the call runs the two existing steps, with gact parked in ggate.  The reference has no counterpart: autograd
 * runs the backward of the linear, of the multiply and of silu one after the other.
 */
int ttamd_nf4_linear_bwd_dx_swiglu_ws_bf16(const void* gy, const uint8_t* quantized_data, const void* block_scalers,
                                           const uint8_t* quantized_data_t, const void* block_scalers_t, const void* gh,
                                           const void* lora_a, int rank, const void* gate, const void* up, void* ggate,
                                           void* gup, int64_t M, int64_t N, int64_t K, void* workspace, size_t workspace_bytes,
                                           void* stream);

/*
 * Adapter gradients (what autograd derives for lora.py:144-146):
 *     gh = scale . gy . B        [M,rank] bf16
 *     gA = gh^T . x              [rank,K] bf16
 *     gB = scale . gy^T . h      [N,rank] bf16
 * gy [M,N], x [M,K], h [M,rank] (from the forward), lora_b [N,rank]; all bf16, fp32 accumulation in a fixed order.
 * workspace: ttamd_lora_bwd_workspace_bytes(M,N,K,rank) bytes.
 */
size_t ttamd_lora_bwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int rank);
int ttamd_lora_bwd_bf16(const void* gy, const void* x, const void* h, const void* lora_b, float scale, void* gh, void* ga,
                        void* gb, int64_t M, int64_t N, int64_t K, int rank, void* workspace, size_t workspace_bytes,
                        void* stream);

/*
 * The whole layer in one call per direction: LoRALinear.forward (torchtune/modules/peft/lora.py:128-147; one Python
 * call of the module is the reference's unit) and the backward autograd derives for it.
 *   ttamd_qlora_linear_fwd_bf16 = ttamd_lora_hidden_bf16 -> ttamd_nf4_lora_linear_fwd_ws_bf16:
 *       h = bf16(x . lora_a^T)   [M,rank], written for the backward (lora.py:144)
 *       y = x . D(W)^T (+ bias) + scale . h . lora_b^T   [M,N]   (lora.py:137-147)
 *   ttamd_qlora_linear_bwd_bf16 = ttamd_lora_bwd_bf16 -> ttamd_nf4_linear_bwd_dx_ws_bf16:
 *       grad_lora_a [rank,K], grad_lora_b [N,rank], and gx = gy . D(W) + gh . lora_a [M,K] unless gx is NULL (the layer's
 *       input needs no gradient); gh = scale . gy . lora_b lives in the workspace.
 * The launches, their order and therefore every result bit are those of the two-call sequences, including the dispatch
 * by size (few tokens, slices of the contraction, the weight expanded once per call).  One workspace per call, sized
 * by the matching query (the stages of a direction reuse its bytes one after the other).  rank a multiple of 8 in
 * [8,64]; the other operands as for the entry points above; quantized_data_t / block_scalers_t: both or neither.
 * One expansion for both directions (optional): when ttamd_nf4_gemm_expands_weight(M, N, K) is 1, the forward call
 * leaves the weight expanded to bf16, in forward tile order, in the first 2 N K bytes of its workspace.  A caller that
 * keeps those bytes until the backward passes them as tiles_fwd (else NULL): the grad-input then runs
 * ttamd_tiled_linear_dx_bf16 on them instead of expanding the weight a second time (the same products summed in the
 * same order: the same gx bit for bit; pays when the expansion is a large share of the call, i.e. at a few thousand
 * tokens).
 * With tiles_fwd (or gx == NULL) the backward needs only the bytes of gh and of ttamd_lora_bwd_workspace_bytes, each
 * rounded up to 256; the query above is the size that serves every case.
 */
size_t ttamd_qlora_linear_fwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int rank);
int ttamd_qlora_linear_fwd_bf16(const void* x, const uint8_t* quantized_data, const void* block_scalers, const void* block_scalers_t,
                                const void* lora_a, const void* lora_b, int rank, float scale, const void* bias, void* y, void* h,
                                int64_t M, int64_t N, int64_t K, void* workspace, size_t workspace_bytes, void* stream);
size_t ttamd_qlora_linear_bwd_workspace_bytes(int64_t M, int64_t N, int64_t K, int rank);
int ttamd_qlora_linear_bwd_bf16(const void* gy, const void* x, const void* h, const uint8_t* quantized_data, const void* block_scalers,
                                const uint8_t* quantized_data_t, const void* block_scalers_t, const void* tiles_fwd, const void* lora_a,
                                const void* lora_b, int rank, float scale, void* gx, void* grad_lora_a, void* grad_lora_b, int64_t M,
                                int64_t N, int64_t K, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Groups of LoRA linears with a common input
 *
 * An addition above the per-linear interface; the reference has no such call.  Its modules call the members one after
 * the other on the same tensor: q_proj, k_proj, v_proj in torchtune/modules/attention.py:234,262-263 and w1 (gate), w3
 * (up) in torchtune/modules/feed_forward.py:50-53, each a LoRALinear.forward (torchtune/modules/peft/lora.py:128-147).
 * A group call computes exactly what the member-by-member calls compute, with fewer passes over the shared operands:
 *
 *   forward   h_cat[:, member i] = x . lora_a_i^T for all members in one pass over x (h_cat [M, sum of ranks] bf16,
 *             member i in columns [sum of the ranks before it, + rank_i); the caller keeps it for the backward);
 *             y_i = x . D(W_i)^T (+ bias_i) + scale_i . h_i . lora_b_i^T: where the few-token kernel serves the member
 *             with the largest weight (the rule of ttamd_nf4_lora_linear_fwd_ws_bf16) one launch for all members that
 *             get the same launch shape, otherwise one launch per member.  h_cat and every y_i are bit-identical to
 *             ttamd_lora_hidden_bf16 + ttamd_nf4_lora_linear_fwd_bf16 on the member alone.
 *   backward  gh_cat[:, member i] = scale_i . gy_i . lora_b_i (one launch, bit-identical to ttamd_lora_bwd_bf16's gh);
 *             grad_lora_a_i = gh_i^T . x for all members in one pass over x and grad_lora_b_i = scale_i . gy_i^T . h_i in
 *             the same launch (fp32 partial sums over row ranges chosen for the whole batch: the same values as the
 *             per-member call up to the order of fp32 additions);
 *             gx = sum_i gy_i . D(W_i) + gh_i . lora_a_i as ONE GEMM whose contraction runs through the members' output
 *             columns one member after the other, summed in fp32 and rounded to bf16 once (the member-by-member
 *             path rounds each member's product to bf16 and adds the rounded tensors).  Every member needs
 *             quantized_data_t and block_scalers_t for it.
 *
 * Requires K % 64 == 0, N_i % 64 == 0, rank_i a positive multiple of 8, sum of ranks <= 64, 1 <= n_members <=
 * TTAMD_GROUP_MAX, all pointers 16-byte aligned (bias: 8).
 * ---------------------------------------------------------------------------------------------- */
typedef struct ttamd_lora_group_member {
  const uint8_t* quantized_data;   /* NF4 codes of the [N, K] weight */
  const void* block_scalers;       /* fp32 [N, K/64] (ttamd_nf4_block_scalers) */
  const void* block_scalers_t;     /* fp32 [K/64, N] or NULL   (ttamd_nf4_transpose_for_backward, second output) */
  const uint8_t* quantized_data_t; /* codes of the transposed weight, [K, N/2], or NULL (same call, first output) */
  const void* lora_a;              /* bf16 [rank, K] */
  const void* lora_b;              /* bf16 [N, rank] */
  const void* bias;                /* bf16 [N] or NULL (forward only) */
  void* y;                         /* forward: out, bf16 [M, N].  backward: in, the gradient of that output */
  void* grad_lora_a;               /* backward: out, bf16 [rank, K] */
  void* grad_lora_b;               /* backward: out, bf16 [N, rank] */
  int64_t N;
  int rank;
  float scale;                     /* alpha / rank */
} ttamd_lora_group_member;

/* h_cat out, bf16 [M, sum of ranks] */
size_t ttamd_lora_group_hidden_workspace_bytes(const ttamd_lora_group_member* members, int n_members, int64_t M, int64_t K);
int ttamd_lora_group_hidden_bf16(const void* x, const ttamd_lora_group_member* members, int n_members, void* h_cat, int64_t M,
                                 int64_t K, void* workspace, size_t workspace_bytes, void* stream);
/* every member's y from x and h_cat; workspace may be NULL (then launches with few output tiles are not sliced) */
size_t ttamd_lora_group_fwd_workspace_bytes(const ttamd_lora_group_member* members, int n_members, int64_t M, int64_t K);
int ttamd_nf4_lora_group_fwd_bf16(const void* x, const ttamd_lora_group_member* members, int n_members, const void* h_cat,
                                  int64_t M, int64_t K, void* workspace, size_t workspace_bytes, void* stream);
/* The gate / up pair of a SwiGLU feed-forward (torchtune/modules/feed_forward.py:50-53: w2(silu(w1(x)) * w3(x)), w1 and
 * w3 LoRALinear over NF4): members[0] = w1 (gate), members[1] = w3 (up), equal N.  Writes both members' y as the call above
 * does and act, bf16 [M, N] = bf16(bf16(silu(y_0)) * y_1) - the bits ttamd_swiglu_fwd_bf16 gives on the two outputs.
 * With the workspace of ttamd_lora_group_fwd_workspace_bytes and a shape the many-token path serves, the product is
 * formed in the epilogue of the one GEMM launch (the two outputs are not read back); otherwise in a pass of its own. */
int ttamd_nf4_lora_group_swiglu_fwd_bf16(const void* x, const ttamd_lora_group_member* members, int n_members, const void* h_cat,
                                         void* act, int64_t M, int64_t K, void* workspace, size_t workspace_bytes, void* stream);
/* gh_cat out, bf16 [M, sum of ranks]; every member's grad_lora_a and grad_lora_b; members[i].y = gy_i */
size_t ttamd_lora_group_bwd_workspace_bytes(const ttamd_lora_group_member* members, int n_members, int64_t M, int64_t K);
int ttamd_lora_group_bwd_bf16(const void* x, const void* h_cat, const ttamd_lora_group_member* members, int n_members,
                              void* gh_cat, int64_t M, int64_t K, void* workspace, size_t workspace_bytes, void* stream);
/* The same for the gate / up pair of a SwiGLU feed-forward (torchtune/modules/feed_forward.py:50-53), starting one step
 * earlier: from gact, the gradient of silu(w1 x) * w3 x, and the two projections gate = w1 x, up = w3 x (bf16 [M, N]).
 * members[0] = w1 (gate), members[1] = w3 (up), equal N; members[i].y = OUT, the gradients of the two projections (the
 * bits of ttamd_swiglu_bwd_bf16), then everything ttamd_lora_group_bwd_bf16 writes (the same bits).  Wide members
 * (N >= 8192, rank <= 16, M >= 1024) get both from one pass: the gradients are formed and stored by the kernel that
 * multiplies them with lora_b and h, and are not read back; otherwise the two steps run one after the other.
 * Workspace: ttamd_lora_group_bwd_workspace_bytes.  No counterpart in the reference (autograd runs the two steps). */
int ttamd_lora_group_swiglu_bwd_bf16(const void* x, const void* h_cat, const ttamd_lora_group_member* members, int n_members,
                                     const void* gact, const void* gate, const void* up, void* gh_cat, int64_t M, int64_t K,
                                     void* workspace, size_t workspace_bytes, void* stream);
/* gx out, bf16 [M, K], from gh_cat and members[i].y = gy_i, quantized_data_t, block_scalers_t, lora_a */
int ttamd_nf4_group_bwd_dx_bf16(const ttamd_lora_group_member* members, int n_members, const void* gh_cat, void* gx, int64_t M,
                                int64_t K, void* stream);
/* the same with room for the members' weights expanded once (many tokens, see ttamd_nf4_gemm_workspace_bytes): bytes to
 * pass (0: the shape is served by the fused kernel), and the call; less workspace than that, or NULL, = the call above */
size_t ttamd_nf4_group_bwd_dx_workspace_bytes(const ttamd_lora_group_member* members, int n_members, int64_t M, int64_t K);
int ttamd_nf4_group_bwd_dx_ws_bf16(const ttamd_lora_group_member* members, int n_members, const void* gh_cat, void* gx, int64_t M,
                                   int64_t K, void* workspace, size_t workspace_bytes, void* stream);

/*
 * One expansion for both directions of a group.  ttamd_nf4_group_fwd_leaves_tiles says what the group's forward call
 * (ttamd_nf4_lora_group_fwd_bf16; swiglu != 0: ttamd_nf4_lora_group_swiglu_fwd_bf16) leaves at the start of a workspace
 * of the size its query asks for: 0 nothing reusable, 1 the members' weights expanded to bf16 and stacked by rows in
 * forward tile order (2 K sum(N[i]) bytes), 2 the gated pair's layout (128 columns of the gate, then 128 of the up
 * projection).  ttamd_nf4_group_bwd_dx_tiles_bf16 is ttamd_nf4_group_bwd_dx_ws_bf16 on those bytes (paired = 1 for
 * layout 2): no expansion launch, the weight operand is transposed on its way out of LDS.  No counterpart in the
 * reference (autograd re-materialises every dequantised weight for the backward).
 */
int ttamd_nf4_group_fwd_leaves_tiles(const ttamd_lora_group_member* members, int n_members, int64_t M, int64_t K, int swiglu);
int ttamd_nf4_group_bwd_dx_tiles_bf16(const ttamd_lora_group_member* members, int n_members, const void* gh_cat, void* gx, int64_t M,
                                      int64_t K, const void* tiles_fwd, int paired, void* stream);
/* The group's forward on tiles that an earlier forward call of the same members left behind (a caller that keeps them
 * across calls: the base weight of a QLoRA run never changes): ttamd_nf4_lora_group_fwd_bf16 (act NULL, paired 0) or
 * ttamd_nf4_lora_group_swiglu_fwd_bf16 (act non-NULL, paired 1) without the expansion launches, same bits.  Shapes for
 * which ttamd_nf4_group_fwd_leaves_tiles gives 0 return TTAMD_EUNSUPPORTED. */
int ttamd_nf4_lora_group_fwd_tiles_bf16(const void* x, const ttamd_lora_group_member* members, int n_members, const void* h_cat,
                                        void* act, int64_t M, int64_t K, const void* tiles_fwd, int paired, void* stream);


/* ------------------------------------------------------------------------------------------------
 * QAT fake quantisation (int8 dynamic per-token activations, int4 per-group symmetric weights)
 * ---------------------------------------------------------------------------------------------- */

/*
 * FakeQuantizer.forward for FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=False) — torchao; built by
 * Int8DynActInt4WeightQATQuantizer.prepare (recipes/qat_single_device.py:378-386) and at
 * torchtune/modules/peft/lora.py:232,258.
 *
 * x [rows,K] `dtype`; out [rows,K] `dtype` = dequantise(quantise(x)) with per-row asymmetric int8 qparams computed
 * in fp32; scale out [rows] fp32 and zero_point out [rows] int32 may be NULL.  K % 8 == 0.
 * qparam_dtype = the config's scale_precision (TTAMD_F32, the reference's default, or TTAMD_BF16): with bf16 the scale
 * is rounded to bf16 after the zero point has been chosen, and the rounded scale quantises and dequantises (it is also
 * what `scale` receives, widened).  The same argument of the two group-wise entry points below means the same.
 * The straight-through backward is the identity and needs no kernel.
 */
int ttamd_fq_per_token_int8_asym(const void* x, int dtype, int64_t rows, int64_t K, int qparam_dtype, void* out, float* scale,
                                 int32_t* zero_point, void* stream);

/*
 * FakeQuantizer.forward for FakeQuantizeConfig(torch.int4, group_size=g, is_symmetric=True) — torchao; same call
 * sites (weight side: lora.py:245,259).
 *
 * w [rows,K] `dtype`, groups of `group_size` consecutive elements along K (K % group_size == 0, group_size a
 * power of two in [8, 512]); out [rows,K] `dtype`; scale out [rows, K/group_size] fp32 may be NULL.
 */
int ttamd_fq_per_group_int4_sym(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype, void* out,
                                float* scale, void* stream);

/*
 * quantizer.convert(model) (recipes/quantize.py:92): the real int4 weights of an 8da4w linear.
 * q out [rows,K] int8 holding values in [-8,7]; scale out [rows,K/group_size] fp32; zero_point out
 * [rows,K/group_size] fp32 (all zero for the symmetric scheme; may be NULL).
 */
int ttamd_quantize_per_group_int4(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype,
                                  int8_t* q, float* scale, float* zero_point, void* stream);

/*
 * Dense weight of the converted 8da4w linear (what Int8DynActInt4WeightLinear.forward rebuilds before its matmul; the
 * converted model is what recipes/quantize.py:92-95 saves and evaluates): out = dtype((q - zero_point) * scale).
 * q [rows,K] int8 holding int4 values; scale, zero_point fp32 [rows, K/group_size] (zero_point may be NULL = 0);
 * out [rows,K] `dtype`.
 */
int ttamd_dequantize_per_group_int4(const int8_t* q, const float* scale, const float* zero_point, int dtype, int64_t rows,
                                    int64_t K, int group_size, void* out, void* stream);

/*
 * The weight-only "4w-qat" mode (Int4WeightOnlyQATQuantizer, re-exported and mapped to "4w-qat" at
 * torchtune/training/quantization.py:27,125-127): FakeQuantizer.forward for
 * FakeQuantizeConfig(torch.uint4, group_size=g, is_symmetric=False, zero_point_domain=FLOAT) — torchao.
 *
 * Per group: scale = clamp((max - min) / 15, 1e-6), zero_point = min + 8 * scale (a float), both rounded to
 * `qparam_dtype` (TTAMD_BF16 / TTAMD_F32); q = clamp(round((w - (zero_point - 8 * scale)) / scale), 0, 15);
 * out = (q - 8) * scale + zero_point.  Every operation is rounded to `dtype` like the eager sequence.
 * w, out [rows,K] `dtype`; scale / zero_point out [rows, K/group_size] fp32, may be NULL.
 */
int ttamd_fq_per_group_uint4_asym(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype,
                                  void* out, float* scale, float* zero_point, void* stream);

/*
 * Int4WeightOnlyQATQuantizer.convert (same quantizer; recipes/quantize.py:92): the codes of the scheme above packed
 * two per byte, even element in the high nibble: q out [rows, K/2] uint8; scale, zero_point out [rows, K/group_size] fp32.
 */
int ttamd_quantize_per_group_uint4(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype,
                                   uint8_t* q, float* scale, float* zero_point, void* stream);

/*
 * Dense weight of the converted weight-only int4 linear: out = dtype((q - 8) * scale + zero_point), each operation
 * rounded to `dtype`.  q [rows, K/2] uint8 as written by ttamd_quantize_per_group_uint4.
 */
int ttamd_dequantize_per_group_uint4(const uint8_t* q, const float* scale, const float* zero_point, int dtype, int64_t rows,
                                     int64_t K, int group_size, void* out, void* stream);

/*
 * Conventions of the fake-quant schemes that differ between versions of the third-party package the reference takes
 * them from (torchao; the reference pins no version).  The plain entry points above use the defaults below; the `_conv`
 * variants take the same arguments plus a pointer to this struct (NULL = defaults), so a deployment that pins another
 * convention needs no other kernel:
 *   eps_per_token            lower bound of the per-token int8 scale.  Default finfo(float32).eps = 2^-23.
 *   eps_per_group_sym        lower bound of the per-group symmetric int4 scale.  Default 2^-23; a version that takes
 *                            eps from the weight dtype uses finfo(bfloat16).eps = 2^-7 for bf16 weights.
 *   min_scale_uint4          lower bound in the weight-only uint4 scheme.  Default 1e-6.
 *   uint4_clamp_range_first  0 (default): scale = max((max - min) / 15, min_scale_uint4);
 *                            1: scale = max(max - min, min_scale_uint4) / 15.
 * All bounds must be positive.
 */
typedef struct ttamd_fq_conventions {
  float eps_per_token;
  float eps_per_group_sym;
  float min_scale_uint4;
  int uint4_clamp_range_first;
} ttamd_fq_conventions;

int ttamd_fq_per_token_int8_asym_conv(const void* x, int dtype, int64_t rows, int64_t K, int qparam_dtype, void* out, float* scale,
                                      int32_t* zero_point, const ttamd_fq_conventions* conventions, void* stream);
int ttamd_fq_per_group_int4_sym_conv(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype,
                                     void* out, float* scale, const ttamd_fq_conventions* conventions, void* stream);
int ttamd_quantize_per_group_int4_conv(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype,
                                       int8_t* q, float* scale, float* zero_point, const ttamd_fq_conventions* conventions,
                                       void* stream);
int ttamd_fq_per_group_uint4_asym_conv(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype,
                                       void* out, float* scale, float* zero_point, const ttamd_fq_conventions* conventions,
                                       void* stream);
int ttamd_quantize_per_group_uint4_conv(const void* w, int dtype, int64_t rows, int64_t K, int group_size, int qparam_dtype,
                                        uint8_t* q, float* scale, float* zero_point, const ttamd_fq_conventions* conventions,
                                        void* stream);

/*
 * The weight side of FakeQuantizedLinear.forward = F.linear(fq(x), fq(W)) (torchao; reached from
 * recipes/qat_single_device.py:378-386 through Int8DynActInt4WeightQATQuantizer.prepare) on this library's own GEMM:
 *   ttamd_fq_per_group_int4_sym_tiled_bf16: ttamd_fq_per_group_int4_sym of a bf16 weight [N, K] (same values bit for bit,
 *     same scales), written straight into the layout ttamd_tiled_linear_bf16 reads instead of row-major: tiled_fwd
 *     (fq(W), for y = x . fq(W)^T) and / or tiled_bwd (fq(W)^T, for gx = gy . fq(W)); either may be NULL, each holds
 *     ttamd_tiled_weight_bytes(N, K) = 2 N K bytes.  group_size 32, 64, 128 or 256 (else TTAMD_EUNSUPPORTED); eps: lower
 *     bound of the scale (2^-23 is what the plain entry point uses); scale out fp32 [N, K / group_size] or NULL.
 *   ttamd_tiled_linear_bf16: y[M, n_out] = x[M, k_contract] . Wd^T (+ bias) with Wd in the tiled layout
 *     (forward: n_out = N, k_contract = K, tiled_fwd; grad-input: n_out = K, k_contract = N, tiled_bwd, bias NULL).
 *     n_out and k_contract multiples of 64.  The kernel of the many-token NF4 path; meant for M of a few thousand rows.
 * Layout: for every block of 16 output columns T and every 32-wide step t of the contraction one 1 KiB piece,
 * piece (T, t) at byte ((T * k_contract / 32) + t) * 1024; in it lane l (0..63) finds, at byte 16 l, the eight bf16
 * values Wd[16 T + l % 16][32 t + 8 (l / 16) .. + 7] (the operand order of v_mfma_f32_16x16x32_bf16).
 */
size_t ttamd_tiled_weight_bytes(int64_t N, int64_t K);
/*
 * The third matmul of that layer's training step, the weight gradient c[N, K] = a[M, N]^T . b[M, K] (a = gy, b = fq(x),
 * both bf16 row-major as autograd hands them over; c bf16): both operands are transposed on their way through LDS.
 * M a multiple of 32, N and K multiples of 256 (ttamd_gemm_tn_applies: 1 / 0; otherwise TTAMD_EUNSUPPORTED).  Meant for
 * shapes with a few hundred output tiles of 256 x 256 or more.
 */
int ttamd_gemm_tn_applies(int64_t M, int64_t N, int64_t K);
int ttamd_gemm_tn_bf16(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, void* stream);
/*
 * The weight gradients of layers with a common input (q / k / v of torchtune/modules/attention.py:234,262-263, gate / up
 * of torchtune/modules/feed_forward.py:50-53) as one launch: c[i][N[i], K] = a[i][M, N[i]]^T . b[M, K] for up to
 * TTAMD_GROUP_MAX members, each result bit-equal to ttamd_gemm_tn_bf16 of that member (same tiles, same order of sums).
 * The members' row tiles share the launch's rounds of 256 tiles, so a narrow member (a 1024-wide k / v projection: 64
 * tiles) no longer needs a launch that leaves three quarters of the chip idle.  Every N[i] and K multiples of 256, M of 32.
 */
int ttamd_gemm_tn_group_bf16(const void* const* a, const void* b, void* const* c, int n_members, int64_t M, const int64_t* N,
                             int64_t K, void* stream);

/*
 * The same two products with a workspace for the last partial round of tiles.  The 256 CUs take 256 output tiles at a
 * time; when the tile count is not a multiple of 256 (3.5 rounds on a 4096 x 14336 gradient) part of the chip idles for
 * the length of one tile.  Given ttamd_gemm_tn_workspace_bytes(M, n_total, K) bytes (n_total: N, or the sum of the
 * members' N[i]), the tiles beyond the last whole round have their contraction cut into 2 - 8 slices (one workgroup per
 * tile and slice, fp32 partial tiles in the workspace) and a second launch adds a tile's slices in slice order, rounds
 * once and stores: deterministic; the sliced tiles differ from the unsliced launch in the order of their fp32 sums only.
 * The query returns 0 where slicing does not pay (short contractions, whole rounds); a smaller workspace, or NULL, runs
 * the unsliced launch (= the entry points above).  The reference has no counterpart (autograd calls a dense GEMM).
 */
size_t ttamd_gemm_tn_workspace_bytes(int64_t M, int64_t n_total, int64_t K);
int ttamd_gemm_tn_ws_bf16(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, void* workspace,
                          size_t workspace_bytes, void* stream);
int ttamd_gemm_tn_group_ws_bf16(const void* const* a, const void* b, void* const* c, int n_members, int64_t M, const int64_t* N,
                                int64_t K, void* workspace, size_t workspace_bytes, void* stream);

int ttamd_fq_per_group_int4_sym_tiled_bf16(const void* w, int64_t N, int64_t K, int group_size, int qparam_dtype, float eps,
                                           void* tiled_fwd, void* tiled_bwd, float* scale, void* stream);
int ttamd_tiled_linear_bf16(const void* x, const void* tiled_weight, const void* bias, void* y, int64_t M, int64_t n_out,
                            int64_t k_contract, void* stream);
/*
 * The same GEMM with a low-rank adapter in its epilogue, for QATLoRALinear.forward (torchtune/modules/peft/lora.py:248-264:
 * F.linear(fq(x), fq(W)) + (alpha / r) * lora_b(lora_a(x)), base weight frozen) and its grad-input:
 *   y[M, n_out] = x . Wd^T (+ bias) + lscale * lx[M, rank] . lw^T
 * forward:    x = fq(x), Wd = tiled_fwd, lx = x . lora_a^T (ttamd_lora_hidden_bf16 on the unquantised x), lw = lora_b [N, rank]
 *             (lw_row_major = 1), lscale = alpha / rank;
 * grad-input: x = gy, Wd = tiled_bwd, lx = gh (ttamd_lora_bwd_bf16), lw = lora_a [rank, K] (lw_row_major = 0), lscale = 1.
 * rank a multiple of 8, at most 64 (0: no adapter, = ttamd_tiled_linear_bf16).
 */
int ttamd_tiled_lora_linear_bf16(const void* x, const void* tiled_weight, const void* lx, const void* lw, int lw_row_major, int rank,
                                 float lscale, const void* bias, void* y, int64_t M, int64_t n_out, int64_t k_contract, void* stream);
/*
 * Fake-quantised layers that read the same input (q_proj / k_proj / v_proj, torchtune/modules/attention.py:234,262-263; w1 / w3,
 * torchtune/modules/feed_forward.py:50-53), as additions above the per-layer calls:
 *   ttamd_fq_per_group_int4_sym_tiled_at_bf16: ttamd_fq_per_group_int4_sym_tiled_bf16 with a place for the transposed tiles:
 *     tiled_bwd is the tile buffer of the members' weights stacked along N (bwd_n_total rows in all, 2 * bwd_n_total * K
 *     bytes) and this weight's rows start at bwd_n_offset (a multiple of 32).  The forward tiles of stacked weights need no
 *     such argument: member i's start at byte 2 * K * (rows before it) of the common buffer.
 *   ttamd_tiled_linear_group_fwd_bf16: y_i[M, n_out_i] = x . Wd_i^T (+ bias_i) for the stacked forward tiles, one launch
 *     (n_out_i multiples of 256; bias NULL or an array with NULL entries allowed).
 *     act != NULL (two members of equal width, the gate and the up projection of a SwiGLU feed-forward): the launch also
 *     writes act[M, n_out] = bf16(bf16(silu(y_0)) * y_1) from its epilogue, as ttamd_nf4_lora_group_swiglu_fwd_bf16 does;
 *     the forward tiles must then be in the paired layout: both members written with fwd_paired = 1, the second one's
 *     tiled_fwd starting 256 * K bytes (128 columns) after the first one's, so that the two weights' blocks of 128
 *     columns alternate.
 *   ttamd_tiled_linear_group_dx_bf16: gx[M, K] = sum_i gy_i[M, n_out_i] . Wd_i, one launch over the stacked transposed
 *     tiles (the sum is taken in fp32 inside the GEMM: no separate additions of the members' grad-inputs).
 */
int ttamd_fq_per_group_int4_sym_tiled_at_bf16(const void* w, int64_t N, int64_t K, int group_size, int qparam_dtype, float eps,
                                              void* tiled_fwd, int fwd_paired, void* tiled_bwd, int64_t bwd_n_total, int64_t bwd_n_offset,
                                              float* scale, void* stream);
int ttamd_tiled_linear_group_fwd_bf16(const void* x, const void* tiled_weights, int n_members, const int64_t* n_out,
                                      const void* const* bias, void* const* y, void* act, int64_t M, int64_t k_contract, void* stream);
int ttamd_tiled_linear_group_dx_bf16(const void* const* gy, const int64_t* n_out, int n_members, const void* tiled_weights_t, void* gx,
                                     int64_t M, int64_t K, void* stream);

/*
 * gx[M, K] = gy[M, N] . Wd (+ gh[M, rank] . lora_a[rank, K]) with Wd [N, K] given as the FORWARD tiles
 * (tiled[N / 16][K / 32][64 lanes][8], what the forward launch of the same layer read): the grad-input of
 * F.linear(x, Wd) (torchao LinearNF4.backward / autograd of FakeQuantizedLinear, reached from
 * torchtune/modules/peft/lora.py:138 and recipes/qat_single_device.py:378-386) without a second, transposed copy of the
 * weight.  The launch transposes the weight operand on its way out of LDS (ds_read_b64_tr_b16); products and their
 * order of summation are those of ttamd_tiled_lora_linear_bf16 on tiles of Wd^T, so the two results are equal bit for
 * bit.  rank a multiple of 8 in [0, 64] (0: gh and lora_a NULL); N and K multiples of 64.
 */
int ttamd_tiled_linear_dx_bf16(const void* gy, const void* tiled_weight_fwd, const void* gh, const void* lora_a, int rank, void* gx,
                               int64_t M, int64_t N, int64_t K, void* stream);


/* ------------------------------------------------------------------------------------------------
 * Neighbours of the quantized linears inside a decoder layer (one pass over HBM each, bf16 tensors, fp32 math).
 * Floating-point kernels: results agree with the eager sequences to a tolerance (summation order and hardware
 * exp / rsqrt differ), not bit for bit.
 * ---------------------------------------------------------------------------------------------- */

/*
 * RMSNorm.forward (torchtune/modules/rms_norm.py:28-41): y = bf16( bf16(x * rsqrt(mean(x^2) + eps)) * scale ).
 * x, y [rows, D] bf16; scale [D] bf16; rstd out [rows] fp32 (kept for the backward; may be NULL).
 * D a multiple of 8, at most 8192.
 */
int ttamd_rms_norm_fwd_bf16(const void* x, const void* scale, float eps, void* y, float* rstd, int64_t rows, int64_t D,
                            void* stream);

/*
 * Backward of the above: gx [rows, D] bf16, and (if gscale is not NULL) gscale [D] bf16 = sum over rows of
 * gy * bf16(x * rstd), summed in a fixed order.  workspace (only read when gscale is given):
 * ttamd_rms_norm_bwd_workspace_bytes(D) bytes.
 */
size_t ttamd_rms_norm_bwd_workspace_bytes(int64_t D);
int ttamd_rms_norm_bwd_bf16(const void* gy, const void* x, const void* scale, const float* rstd, void* gx, void* gscale,
                            int64_t rows, int64_t D, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The residual stream's addition in the same passes (h = attn_out + x and out = h + mlp_out of
 * torchtune/modules/transformer.py:129-141, each followed by an RMSNorm in the next sub-block):
 *   ttamd_add_rms_norm_fwd_bf16: h = bf16(x + residual) (written to h) and y = RMSNorm(h); the bits of the addition
 *     followed by ttamd_rms_norm_fwd_bf16, without reading h back.
 *   ttamd_rms_norm_bwd_add_bf16: gx = bf16( bf16(gx of ttamd_rms_norm_bwd_bf16) + g_add ), g_add [rows, D] bf16 being the
 *     gradient that reaches the norm's input on the residual way (NULL: ttamd_rms_norm_bwd_bf16): what autograd's
 *     accumulation of the two gradients gives, without writing and re-reading the first.
 * The reference has no counterpart (separate eager kernels).
 */
int ttamd_add_rms_norm_fwd_bf16(const void* x, const void* residual, const void* scale, float eps, void* h, void* y, float* rstd,
                                int64_t rows, int64_t D, void* stream);
int ttamd_rms_norm_bwd_add_bf16(const void* gy, const void* x, const void* scale, const float* rstd, const void* g_add, void* gx,
                                void* gscale, int64_t rows, int64_t D, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Rotary position embedding (torchtune/models/llama3_1/_position_embeddings.py:128-190, positions 0..S-1):
 * x, y [B, S, n_heads, head_dim] bf16; cache [S, head_dim/2, 2] fp32 (cos, sin); consecutive pairs are rotated in
 * fp32.  inverse != 0 rotates by the negative angle, which is the backward pass.  head_dim a multiple of 8.
 */
int ttamd_rope_bf16(const void* x, const float* cache, void* y, int64_t B, int64_t S, int64_t n_heads, int64_t head_dim,
                    int inverse, void* stream);

/*
 * Grouped-query expansion of the key / value heads before attention
 * (torchtune/modules/attention.py:284-290: k.unsqueeze(2).expand(...).flatten(1, 2), here on the [b, s, n_kv, h_d] layout):
 * y [tokens, n_kv * rep, head_dim] with y[t][kv * rep + r] = x[t][kv], and its backward
 * gx[t][kv] = bf16(sum_r gy[t][kv * rep + r]) (fp32 sums, r ascending).  All bf16, head_dim a multiple of 8.
 */
int ttamd_repeat_kv_bf16(const void* x, void* y, int64_t tokens, int64_t n_kv, int64_t rep, int64_t head_dim, void* stream);
int ttamd_repeat_kv_bwd_bf16(const void* gy, void* gx, int64_t tokens, int64_t n_kv, int64_t rep, int64_t head_dim,
                             void* stream);

/*
 * Everything between the q / k / v projections and the attention in one launch
 * (torchtune/modules/attention.py:255-290: the rotary embedding of q and k, then the expansion of the k / v heads):
 * q_out = rope(q), k_out = repeat(rope(k)), v_out = repeat(v) with q, q_out, k_out, v_out [B, S, n_heads, head_dim] and
 * k, v [B, S, n_kv, head_dim], rep = n_heads / n_kv (1: k_out = rope(k), v_out = v).  The backward takes the gradients of
 * the three outputs and writes those of q, k, v.  Both give the bits of ttamd_rope_bf16 and ttamd_repeat_kv(_bwd)_bf16
 * called one after the other.  n_heads a multiple of n_kv, head_dim a multiple of 8.
 */
int ttamd_qkv_rope_repeat_bf16(const void* q, const void* k, const void* v, const float* cache, void* q_out, void* k_out,
                               void* v_out, int64_t B, int64_t S, int64_t n_heads, int64_t n_kv, int64_t head_dim, void* stream);
int ttamd_qkv_rope_repeat_bwd_bf16(const void* gq_out, const void* gk_out, const void* gv_out, const float* cache, void* gq,
                                   void* gk, void* gv, int64_t B, int64_t S, int64_t n_heads, int64_t n_kv, int64_t head_dim,
                                   void* stream);

/*
 * FeedForward gate (torchtune/modules/feed_forward.py:50-53): out = bf16( bf16(silu(gate)) * up ), and its backward
 * ggate, gup from gout.  All [numel] bf16, numel a multiple of 8.
 */
int ttamd_swiglu_fwd_bf16(const void* gate, const void* up, void* out, int64_t numel, void* stream);
int ttamd_swiglu_bwd_bf16(const void* gout, const void* gate, const void* up, void* ggate, void* gup, int64_t numel,
                          void* stream);

/*
 * The per-chunk body of LinearCrossEntropyLoss (torchtune/modules/loss/cross_entropy_loss.py:86-112):
 * F.cross_entropy(logits.float(), target, reduction="sum", ignore_index), forward and backward in one pass.
 * logits [rows, V] bf16; target [rows] int64 (class index in [0, V), or ignore_index); loss out [rows] fp32 =
 * logsumexp - logit[target] (0 for an ignored row; the caller sums); grad_logits out [rows, V] bf16 =
 * grad_scale * (softmax - onehot) (0 for an ignored row).  V a multiple of 8, at most 131072.
 */
int ttamd_cross_entropy_fwd_bwd_bf16(const void* logits, const int64_t* target, int64_t ignore_index, float grad_scale,
                                     float* loss, void* grad_logits, int64_t rows, int64_t V, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TORCHTUNE_AMD_H */
