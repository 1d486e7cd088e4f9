"""A Llama-shaped decoder that drives the quantized linears the way the reference's model does.

The reference composes ``LoRALinear`` / ``FrozenNF4Linear`` inside ``MultiHeadAttention``
(``torchtune/modules/attention.py:228-303``), ``FeedForward`` (``torchtune/modules/feed_forward.py:50-54``),
``TransformerSelfAttentionLayer`` (``torchtune/modules/transformer.py:88-141``) and ``TransformerDecoder``
(``:574-689``), with a chunked output-projection + cross-entropy loss
(``torchtune/modules/loss/cross_entropy_loss.py:147-188``).  Those classes are not part of the quantized path;
this file reproduces only their call pattern with stock PyTorch ops so that the benchmark and the smoke test
exercise the seven projections per layer with the reference's shapes and order:

    RMSNorm -> q, k, v (same input) -> RoPE -> causal GQA attention -> o -> residual
            -> RMSNorm -> w2(silu(w1 x) * w3 x) -> residual

Shapes come from the reference's builders: ``llama3_2_1b`` (``torchtune/models/llama3_2/_model_builders.py:20-46``),
``llama3_1_8b`` / ``llama3_1_70b`` (``torchtune/models/llama3_1/_model_builders.py:20-59``); LoRA placement from
``lora_llama3_attention`` / ``lora_llama3_mlp`` (``torchtune/models/llama3_1/_component_builders.py:338-401,433-456``).
The output projection is a plain frozen bf16 linear, never NF4 (``_component_builders.py:251-257``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn
from torch.nn.attention import SDPBackend, sdpa_kernel
from torch.utils.checkpoint import checkpoint

from .modules import layer_ops
from .modules.peft import (LoRALinear, get_adapter_params, lora_feed_forward, lora_linear_group, lora_swiglu_group,
                           set_trainable_params)
from .qat import FakeQuantizedLinear, Int8DynActInt4WeightQATQuantizer, fake_quantized_linear_group, fake_quantized_swiglu_group


# True: projections that read the same tensor (q/k/v, gate/up) go through the group kernels; False: one call per
# projection, as the reference's modules make them (kept for A/B timing and for the tests that compare the two)
GROUP_SHARED_INPUT = True
# silu(w1 x) * w3 x formed in the epilogue of the gate / up GEMM launch instead of a pass of its own
GATED_EPILOGUE = True
# True: on the way back the gradients of w1 x and w3 x are written by the epilogue of w2's grad-input GEMM launch instead
# of the gradient of their product followed by a pass of its own.  Off by default: it saves the write and the read of
# that gradient (470 MB per 8B layer at 8192 tokens) but the reads of gate and up then sit in the GEMM's epilogue, where
# all workgroups wait for memory at once (+111 us per launch against the 187 us of the pass it replaces; 8B step
# 245.9 -> 245.4 ms, while the GEMM launches' own TFLOP/s drop by 2 %).
SWIGLU_BWD_EPILOGUE = False


def _shared_input(x, layers):
    """Projections that read the same tensor: the LoRA group kernels, the fake-quantised group, or the layers in turn."""
    if all(isinstance(layer, FakeQuantizedLinear) for layer in layers):
        return fake_quantized_linear_group(x, layers)
    return lora_linear_group(x, layers)


@dataclass(frozen=True)
class LlamaShape:
    name: str
    n_layers: int
    dim: int
    n_heads: int
    n_kv_heads: int
    hidden: int
    vocab: int = 128256
    rope_base: float = 500000.0
    norm_eps: float = 1e-5

    @property
    def head_dim(self) -> int:
        return self.dim // self.n_heads


SHAPES = {
    "llama3_2_1b": LlamaShape("llama3_2_1b", 16, 2048, 32, 8, 8192),
    "llama3_1_8b": LlamaShape("llama3_1_8b", 32, 4096, 32, 8, 14336),
    "llama3_1_70b": LlamaShape("llama3_1_70b", 80, 8192, 64, 8, 28672),
    # a toy shape for tests: same structure, every dimension still a multiple of 64
    "tiny": LlamaShape("tiny", 2, 256, 4, 2, 512, vocab=1024),
}


# True: the additions of the residual stream run inside the RMSNorm pass that follows each of them, forward and backward
# (same bits; one write and one read of the stream less per addition)
FUSED_ADD_NORM = True
# True: the rotary embedding of q and k and the grouped-query expansion of k and v run as one launch per direction
# (same bits; four launches and the intermediate rotated k less per layer and direction)
FUSED_QKV_POST = True
# A fake-quantised output projection and the loss of a chunk of rows as one autograd node
# (``FakeQuantizedLinear.cross_entropy_sum``): backward then scales the [rows, dim] operands by the incoming gradient instead
# of the [rows, vocabulary] gradient of the logits (False: the layer's output followed by ``layer_ops.cross_entropy_sum``).
FUSED_QAT_OUTPUT_LOSS = True
# True: RMSNorm, RoPE and the SwiGLU gate run as single-pass HIP kernels (bf16 on the GPU); False: the eager op chains
# of the reference.  The quantized linears are unaffected.
FUSED_LAYER_OPS = True


# Which of PyTorch's own scaled_dot_product_attention backends the stack asks for (attention is stock PyTorch here, as
# in the reference, which calls F.scaled_dot_product_attention and takes the dispatcher's first choice, "flash").  On
# this GPU the backward of the "efficient" backend takes 0.77 ms per 8B layer against 2.2 ms for "flash" (forward equal),
# so "efficient" is the default; "flash" restores the dispatcher's own choice, "default" leaves the dispatcher alone.
SDPA_BACKEND = "efficient"
_SDPA_CHOICES = {
    "efficient": [SDPBackend.EFFICIENT_ATTENTION, SDPBackend.MATH],
    "flash": [SDPBackend.FLASH_ATTENTION, SDPBackend.MATH],
}


def _sdpa(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    if SDPA_BACKEND == "default" or not q.is_cuda:
        return F.scaled_dot_product_attention(q, k, v, is_causal=True)
    with sdpa_kernel(_SDPA_CHOICES[SDPA_BACKEND]):
        return F.scaled_dot_product_attention(q, k, v, is_causal=True)


def _fused(x: torch.Tensor) -> bool:
    return FUSED_LAYER_OPS and x.is_cuda and x.dtype == torch.bfloat16


class RMSNorm(nn.Module):
    """fp32 RMS normalisation (``torchtune/modules/rms_norm.py:28-41``)."""

    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.eps = eps
        self.scale = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if _fused(x) and self.scale.dtype == torch.bfloat16 and x.shape[-1] % 8 == 0 and x.shape[-1] <= 8192:
            return layer_ops._RMSNormFn.apply(x, self.scale, self.eps)
        xf = x.float()
        x_normed = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)).type_as(x)
        return x_normed * self.scale


def rope_cache(seq_len: int, head_dim: int, base: float, device) -> torch.Tensor:
    """[seq, head_dim/2, 2] cos/sin table."""
    theta = 1.0 / (base ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
    idx = torch.outer(torch.arange(seq_len, device=device, dtype=torch.float32), theta)
    return torch.stack([idx.cos(), idx.sin()], dim=-1)


def apply_rope(x: torch.Tensor, cache: torch.Tensor) -> torch.Tensor:
    """x [b, s, n_h, h_d]; rotates interleaved pairs, fp32 math."""
    if _fused(x) and x.shape[-1] % 8 == 0:
        return layer_ops.apply_rope(x, cache)
    xs = x.float().reshape(*x.shape[:-1], -1, 2)
    c = cache.view(1, xs.size(1), 1, xs.size(3), 2)
    out = torch.stack(
        [xs[..., 0] * c[..., 0] - xs[..., 1] * c[..., 1], xs[..., 1] * c[..., 0] + xs[..., 0] * c[..., 1]], dim=-1
    )
    return out.flatten(3).to(x.dtype)


def _linear(in_dim: int, out_dim: int, rank: int, alpha: float, quantize_base: bool) -> nn.Module:
    if rank > 0:
        return LoRALinear(in_dim, out_dim, rank=rank, alpha=alpha, quantize_base=quantize_base)
    return nn.Linear(in_dim, out_dim, bias=False)


class Attention(nn.Module):
    def __init__(self, s: LlamaShape, rank: int, alpha: float, quantize_base: bool):
        super().__init__()
        self.n_heads, self.n_kv, self.head_dim = s.n_heads, s.n_kv_heads, s.head_dim
        self.q_proj = _linear(s.dim, s.n_heads * s.head_dim, rank, alpha, quantize_base)
        self.k_proj = _linear(s.dim, s.n_kv_heads * s.head_dim, rank, alpha, quantize_base)
        self.v_proj = _linear(s.dim, s.n_kv_heads * s.head_dim, rank, alpha, quantize_base)
        self.output_proj = _linear(s.dim, s.dim, rank, alpha, quantize_base)

    def forward(self, x: torch.Tensor, rope: torch.Tensor) -> torch.Tensor:
        b, sl, _ = x.shape
        # the three projections read the same tensor (torchtune/modules/attention.py:234,262-263): one group
        q, k, v = _shared_input(x, (self.q_proj, self.k_proj, self.v_proj)) if GROUP_SHARED_INPUT else (
            self.q_proj(x), self.k_proj(x), self.v_proj(x))
        q = q.view(b, sl, self.n_heads, self.head_dim)
        k = k.view(b, sl, self.n_kv, self.head_dim)
        v = v.view(b, sl, self.n_kv, self.head_dim)
        if FUSED_QKV_POST and self.n_kv != self.n_heads and _fused(q) and self.head_dim % 8 == 0:
            # rotary embedding of q and k and the expansion of the k / v heads: one launch per direction
            q, k, v = layer_ops.qkv_rope_repeat(q, k, v, rope)
            o = _sdpa(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
            return self.output_proj(o.transpose(1, 2).reshape(b, sl, -1))
        q = apply_rope(q, rope)
        k = apply_rope(k, rope)
        if self.n_kv != self.n_heads:  # expand kv heads to query heads, as the reference does before SDPA
            rep = self.n_heads // self.n_kv
            if _fused(k) and self.head_dim % 8 == 0:
                k, v = layer_ops.repeat_kv(k, rep), layer_ops.repeat_kv(v, rep)
            else:
                k = k.unsqueeze(3).expand(b, sl, self.n_kv, rep, self.head_dim).flatten(2, 3)
                v = v.unsqueeze(3).expand(b, sl, self.n_kv, rep, self.head_dim).flatten(2, 3)
        o = _sdpa(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
        return self.output_proj(o.transpose(1, 2).reshape(b, sl, -1))


class FeedForward(nn.Module):
    def __init__(self, s: LlamaShape, rank: int, alpha: float, quantize_base: bool):
        super().__init__()
        self.w1 = _linear(s.dim, s.hidden, rank, alpha, quantize_base)  # gate
        self.w2 = _linear(s.hidden, s.dim, rank, alpha, quantize_base)  # down
        self.w3 = _linear(s.dim, s.hidden, rank, alpha, quantize_base)  # up

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # gate and up read the same tensor (torchtune/modules/feed_forward.py:50-53): one group
        if GROUP_SHARED_INPUT and GATED_EPILOGUE:
            if SWIGLU_BWD_EPILOGUE and not isinstance(self.w1, FakeQuantizedLinear):
                # also the way back: w2's grad-input GEMM writes the gradients of the two projections
                y = lora_feed_forward(x, self.w1, self.w3, self.w2)
                if y is not None:
                    return y
            # the product written by the pair's GEMM launch
            act = (fake_quantized_swiglu_group(x, self.w1, self.w3) if isinstance(self.w1, FakeQuantizedLinear)
                   else lora_swiglu_group(x, self.w1, self.w3))
            if act is not None:
                return self.w2(act)
        g, u = _shared_input(x, (self.w1, self.w3)) if GROUP_SHARED_INPUT else (self.w1(x), self.w3(x))
        return self.w2(layer_ops.swiglu(g, u) if _fused(g) else F.silu(g) * u)


def _add_norm(x: torch.Tensor, delta: torch.Tensor, norm: RMSNorm):
    """``h = x + delta; return h, norm(h)``: one pass forward and one backward where the fused kernels apply."""
    if FUSED_ADD_NORM and _fused(x) and norm.scale.dtype == torch.bfloat16 and x.shape[-1] % 8 == 0 and x.shape[-1] <= 8192:
        return layer_ops.add_rms_norm(x, delta, norm)
    h = x + delta
    return h, norm(h)


class DecoderLayer(nn.Module):
    def __init__(self, s: LlamaShape, rank: int, alpha: float, quantize_base: bool):
        super().__init__()
        self.sa_norm = RMSNorm(s.dim, s.norm_eps)
        self.attn = Attention(s, rank, alpha, quantize_base)
        self.mlp_norm = RMSNorm(s.dim, s.norm_eps)
        self.mlp = FeedForward(s, rank, alpha, quantize_base)

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], rope: torch.Tensor):
        """``x``: the residual stream before the previous layer's feed-forward output ``delta`` is added (``None`` for the
        first layer).  Returns the stream after the attention sub-block and this layer's feed-forward output, not yet
        added: every addition of the stream (``torchtune/modules/transformer.py:129-141``) is followed by an RMSNorm and
        runs in that norm's pass (``_add_norm``)."""
        h, n = (x, self.sa_norm(x)) if delta is None else _add_norm(x, delta, self.sa_norm)
        h, n = _add_norm(h, self.attn(n, rope), self.mlp_norm)
        return h, self.mlp(n)


class Decoder(nn.Module):
    """Token ids -> final hidden states; ``loss`` adds the chunked output projection + cross entropy.

    ``loss_chunks`` = 2 (the reference default is 8): with 288 GB of HBM the fp32 logits of half the batch (2 GB for
    8192 tokens) are no burden, and the vocabulary GEMM runs 25 % faster on 4096-row chunks than on 1024-row ones."""

    def __init__(self, s: LlamaShape, rank: int, alpha: float, quantize_base: bool, activation_checkpointing: bool = False,
                 loss_chunks: int = 2):
        super().__init__()
        self.shape = s
        self.ac = activation_checkpointing
        self.loss_chunks = loss_chunks
        self.tok_embeddings = nn.Embedding(s.vocab, s.dim)
        self.layers = nn.ModuleList(DecoderLayer(s, rank, alpha, quantize_base) for _ in range(s.n_layers))
        self.norm = RMSNorm(s.dim, s.norm_eps)
        self.output = nn.Linear(s.dim, s.vocab, bias=False)
        self._rope = None  # (seq_len, device, table): built once per sequence length, as the reference keeps it in a buffer

    def _rope_cache(self, seq_len: int, device) -> torch.Tensor:
        if self._rope is None or self._rope[0] != seq_len or self._rope[1] != device:
            self._rope = (seq_len, device, rope_cache(seq_len, self.shape.head_dim, self.shape.rope_base, device))
        return self._rope[2]

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        rope = self._rope_cache(tokens.shape[1], tokens.device)
        h = self.tok_embeddings(tokens)
        delta = None
        for layer in self.layers:
            if self.ac and torch.is_grad_enabled():
                h, delta = checkpoint(layer, h, delta, rope, use_reentrant=False)
            else:
                h, delta = layer(h, delta, rope)
        return _add_norm(h, delta, self.norm)[1]

    def loss(self, tokens: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
        """Mean next-token cross entropy; the vocabulary projection is applied chunk by chunk over the sequence."""
        h = self.forward(tokens)
        hidden = h.reshape(-1, h.shape[-1])
        target = labels.reshape(-1)
        total = hidden.new_zeros((), dtype=torch.float32)
        n = target.numel()
        out = self.output
        plain = type(out) is nn.Linear and out.bias is None and out.weight.shape[0] % 8 == 0 and out.weight.shape[0] <= 131072
        for hc, tc in zip(hidden.chunk(self.loss_chunks), target.chunk(self.loss_chunks)):
            if plain and _fused(hc) and out.weight.dtype == hc.dtype:
                total = total + layer_ops.linear_cross_entropy_sum(hc, out.weight, tc, scale=1.0 / n)
                continue
            if FUSED_QAT_OUTPUT_LOSS and hasattr(out, "cross_entropy_sum") and _fused(hc):
                part = out.cross_entropy_sum(hc, tc, scale=1.0 / n)
                if part is not None:
                    total = total + part
                    continue
            logits = self.output(hc)
            if _fused(logits) and logits.shape[-1] % 8 == 0 and logits.shape[-1] <= 131072:
                total = total + layer_ops.cross_entropy_sum(logits, tc, scale=1.0 / n)
            else:
                total = total + F.cross_entropy(logits.float(), tc, reduction="sum") / n
        return total


@torch.no_grad()
def _init_weights(model: Decoder, seed: int, std: float = 0.02) -> None:
    """Base weights ~ N(0, std) generated on the device one tensor at a time (an NF4 parameter re-quantises on
    ``copy_``, so the dense model never exists); lora_b ~ N(0, 0.01) so the adapter path is not a no-op."""
    dev = model.tok_embeddings.weight.device
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    for name, p in model.named_parameters():
        if name.endswith("scale"):
            continue
        if "lora_a" in name:
            bound = 1.0 / (p.shape[1] ** 0.5)
            p.copy_(torch.empty(p.shape, device=dev, dtype=torch.float32).uniform_(-bound, bound, generator=gen))
        elif "lora_b" in name:
            p.copy_(torch.randn(p.shape, device=dev, dtype=torch.float32, generator=gen) * 0.01)
        else:
            p.copy_((torch.randn(p.shape, device=dev, dtype=torch.float32, generator=gen) * std).to(torch.bfloat16))


def build_qlora_decoder(shape: str | LlamaShape, rank: int, alpha: float, device="cuda", seed: int = 0,
                        activation_checkpointing: bool = False, dtype: torch.dtype = torch.bfloat16) -> Decoder:
    """QLoRA model: NF4 base + LoRA on all seven projections, everything but the adapters frozen."""
    s = SHAPES[shape] if isinstance(shape, str) else shape
    prev = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        with torch.device(device):
            model = Decoder(s, rank, alpha, quantize_base=True, activation_checkpointing=activation_checkpointing)
    finally:
        torch.set_default_dtype(prev)
    _init_weights(model, seed)
    set_trainable_params(model, get_adapter_params(model))
    return model


def build_qat_decoder(shape: str | LlamaShape, groupsize: int = 32, device="cuda", seed: int = 0,
                      activation_checkpointing: bool = False, dtype: torch.dtype = torch.bfloat16,
                      quantize_output: bool = True, scales_precision: torch.dtype = torch.float32) -> Decoder:
    """Full-finetune model prepared for 8da4w QAT: every linear swapped for the fake-quantised one.
    ``scales_precision`` float32 is the reference quantizer's default; bfloat16 rounds every scale before use."""
    s = SHAPES[shape] if isinstance(shape, str) else shape
    prev = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        with torch.device(device):
            model = Decoder(s, 0, 0.0, quantize_base=False, activation_checkpointing=activation_checkpointing)
    finally:
        torch.set_default_dtype(prev)
    _init_weights(model, seed)
    quantizer = Int8DynActInt4WeightQATQuantizer(groupsize=groupsize, precision=dtype, scales_precision=scales_precision)
    if quantize_output:
        quantizer.prepare(model)
    else:
        quantizer.prepare(model.layers)
    return model


def train_step(model: Decoder, tokens: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """One forward + backward; returns the detached loss."""
    loss = model.loss(tokens, labels)
    loss.backward()
    return loss.detach()
