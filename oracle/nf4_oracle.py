"""CPU oracle for the NF4 double-quantisation codec and ``linear_nf4``.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; it is the checker that
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` hold the HIP kernels
against.

It restates, op for op in eager PyTorch on the CPU, what the reference executes through the third-party
``torchao`` package (not vendored in the reference tree, version not pinned by it):

* ``nf4_quantize``    <- ``to_nf4`` / ``NF4Tensor.from_tensor``; reference call sites
  ``torchtune/modules/peft/lora.py:86``, ``torchtune/modules/low_precision/nf4_linear.py:49``,
  ``torchtune/modules/low_precision/_register_nf4_dispatch_ops.py:20``.
* ``nf4_dequantize``  <- ``NF4Tensor.get_original_weight`` / ``.to(dtype)``; reference call sites
  ``torchtune/modules/common_utils.py:57``, ``torchtune/modules/peft/dora.py:137``.
* ``linear_nf4_forward`` / ``linear_nf4_backward`` <- ``linear_nf4`` (``LinearNF4`` autograd function);
  reference call sites ``torchtune/modules/peft/lora.py:138``, ``torchtune/modules/low_precision/nf4_linear.py:67``.

Parity status.  ``torchao`` cannot be imported where this was written, and no test of the reference pins NF4
codes, scaler bytes or dequantised values, so bit-level agreement with torchao itself is PARITY UNPINNED for
``nf4_quantize`` and ``nf4_dequantize``.  What pins this restatement instead (see tests/test_oracle_nf4.py):
the 16 published NF4 code points; closed forms (a block equal to absmax*table quantises to codes 0..15, +-c
blocks to 15/0, arithmetic-progression absmaxes give known scaler bytes); brute force over every bf16 bit
pattern; the reference's own invariant quantise(dequantise(q)) == q (tests/torchtune/modules/peft/test_lora.py:229-237);
the nibble order by single-element perturbation; and an independent scalar C restatement (oracle/nf4_ref.c) that
emulates bf16 rounding with integer arithmetic.  ``linear_nf4`` reduces to ``F.linear`` on the dequantised
weight, which is the reference's own definition (tests/torchtune/modules/peft/test_lora.py:157-182).

One deliberate definition: ``scaler_mean``.  The eager reference calls ``absmax.mean()``, whose fp32
summation order differs between CPU and GPU builds of PyTorch and can flip the last bf16 bit.  The oracle
(and the kernels) define it order-independently: the exact sum (fp64 accumulation), divided by the count in
fp64, rounded to fp32 and then to the tensor dtype.  ``tests/test_oracle_nf4.py`` checks it equals
``absmax.mean()`` on the seeded inputs used here.

Degenerate inputs: an all-zero block has absmax 0, every scaled value is NaN and ``argmin`` over an all-NaN
row returns 0, so every code is 0; a NaN scaled scaler quantises to 0.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F

# The NormalFloat4 code points (QLoRA, Dettmers et al. 2023, appendix E); all exactly representable in fp32.
NF4_TABLE = (
    -1.0,
    -0.6961928009986877,
    -0.5250730514526367,
    -0.39491748809814453,
    -0.28444138169288635,
    -0.18477343022823334,
    -0.09105003625154495,
    0.0,
    0.07958029955625534,
    0.16093020141124725,
    0.24611230194568634,
    0.33791524171829224,
    0.44070982933044434,
    0.5626170039176941,
    0.7229568362236023,
    1.0,
)

_ARGMIN_CHUNK = 1024**2  # the reference processes the [chunk, 16] distance matrix in pieces of this size


@dataclass
class NF4Parts:
    """The inner tensors and metadata of an NF4 tensor (attribute names as pinned by
    tests/torchtune/modules/low_precision/test_nf4_dispatch_registration.py:22-31)."""

    block_size: int
    n_blocks: int
    scaler_block_size: int
    quantized_scalers: torch.Tensor  # int8  [n_blocks]
    quantization_factor: torch.Tensor  # dtype [n_blocks / scaler_block_size]
    scaler_mean: torch.Tensor  # dtype 0-dim
    quantized_data: torch.Tensor  # uint8 [numel / 2]
    nf4: torch.Tensor  # dtype [16]
    shape: torch.Size
    dtype: torch.dtype


def order_independent_mean(absmax: torch.Tensor) -> torch.Tensor:
    """mean of the block absmaxes: exact sum / n in fp64 -> fp32 -> tensor dtype."""
    s = absmax.to(torch.float64).sum()
    return (s / absmax.numel()).to(torch.float32).to(absmax.dtype)


def nf4_quantize(tensor: torch.Tensor, block_size: int = 64, scaler_block_size: int = 256,
                 mean: torch.Tensor | None = None) -> NF4Parts:
    """``mean``: the scaler mean to use instead of this tensor's own.  The mean is the only quantity of the algorithm
    that couples distant parts of a tensor, so a slice of whole scaler blocks of a large tensor quantises, given the
    large tensor's mean, to exactly the corresponding slice of the large tensor's parts (how the tests check tensors too
    large for an eager CPU pass)."""
    assert tensor.dim() <= 2, "NF4 supports at most 2-D tensors"
    assert tensor.is_contiguous()
    assert tensor.dtype in (torch.bfloat16, torch.float32)
    numel = tensor.numel()
    assert numel % block_size == 0
    n_blocks = numel // block_size
    assert n_blocks % scaler_block_size == 0
    dtype = tensor.dtype
    tensor = tensor.detach().cpu()
    nf4 = torch.tensor(NF4_TABLE, dtype=dtype)

    flat = tensor.flatten()
    blocks = flat.view(n_blocks, block_size)
    absmax = blocks.abs().max(dim=1).values  # [n_blocks], dtype

    # double quantisation of the block scalers
    mean = order_independent_mean(absmax) if mean is None else mean.detach().cpu().to(dtype).reshape(())
    centred = absmax - mean
    n_sb = n_blocks // scaler_block_size
    centred_sb = centred.view(n_sb, scaler_block_size)
    absmax2 = centred_sb.abs().max(dim=1).values
    factor = 256 / (2 * absmax2)  # dtype
    scaled_scalers = (centred_sb * factor[:, None]).round()
    scaled_scalers = torch.nan_to_num(scaled_scalers, nan=0.0, posinf=127.0, neginf=-128.0)
    quantized_scalers = scaled_scalers.clamp(-128, 127).to(torch.int8).flatten()

    # 4-bit codes: divide by the UNquantised absmax, nearest code with distances rounded in dtype
    scaled = (blocks / absmax[:, None]).flatten()
    codes = torch.empty(numel, dtype=torch.uint8)
    for lo in range(0, numel, _ARGMIN_CHUNK):
        piece = scaled[lo : lo + _ARGMIN_CHUNK]
        diff = (piece[:, None] - nf4[None, :]).abs()
        codes[lo : lo + _ARGMIN_CHUNK] = diff.argmin(dim=-1).to(torch.uint8)
    packed = (codes[0::2] << 4) | codes[1::2]

    return NF4Parts(
        block_size=block_size,
        n_blocks=n_blocks,
        scaler_block_size=scaler_block_size,
        quantized_scalers=quantized_scalers,
        quantization_factor=factor,
        scaler_mean=mean,
        quantized_data=packed,
        nf4=nf4,
        shape=tensor.shape,
        dtype=dtype,
    )


def nf4_dequantize_scalers(p: NF4Parts) -> torch.Tensor:
    n_sb = p.n_blocks // p.scaler_block_size
    q = p.quantized_scalers.view(n_sb, p.scaler_block_size)
    return (q / p.quantization_factor[:, None]).flatten().to(p.dtype) + p.scaler_mean


def nf4_dequantize(p: NF4Parts) -> torch.Tensor:
    scalers = nf4_dequantize_scalers(p)  # [n_blocks], dtype
    hi = (p.quantized_data >> 4).to(torch.long)
    lo = (p.quantized_data & 0xF).to(torch.long)
    per_elem = scalers.repeat_interleave(p.block_size // 2)
    out = torch.empty(p.quantized_data.numel() * 2, dtype=p.dtype)
    out[0::2] = p.nf4[hi] * per_elem
    out[1::2] = p.nf4[lo] * per_elem
    return out.view(p.shape)


def linear_nf4_forward(x: torch.Tensor, p: NF4Parts) -> torch.Tensor:
    return F.linear(x, nf4_dequantize(p).to(x.dtype))


def linear_nf4_backward(grad_out: torch.Tensor, p: NF4Parts) -> torch.Tensor:
    return grad_out @ nf4_dequantize(p).to(grad_out.dtype)
