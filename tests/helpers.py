"""Shared helpers for the tests: ctypes access to the C oracle with torch tensors, seeded inputs."""
import ctypes

import torch

from oracle import nf4_oracle


def ptr(t: torch.Tensor):
    return ctypes.c_void_p(t.data_ptr())


def c_nf4_quantize(lib, w: torch.Tensor, block_size: int, scaler_block_size: int) -> nf4_oracle.NF4Parts:
    w = w.contiguous()
    numel = w.numel()
    n_blocks = numel // block_size
    qdata = torch.empty(numel // 2, dtype=torch.uint8)
    qs = torch.empty(n_blocks, dtype=torch.int8)
    qf = torch.empty(n_blocks // scaler_block_size, dtype=w.dtype)
    mean = torch.empty((), dtype=w.dtype)
    absmax = torch.empty(n_blocks, dtype=torch.float32)
    lib.ref_nf4_quantize(ptr(w), int(w.dtype == torch.bfloat16), numel, block_size, scaler_block_size, ptr(qdata), ptr(qs),
                         ptr(qf), ptr(mean), ptr(absmax))
    return nf4_oracle.NF4Parts(block_size, n_blocks, scaler_block_size, qs, qf, mean, qdata,
                               torch.tensor(nf4_oracle.NF4_TABLE, dtype=w.dtype), w.shape, w.dtype)


def c_nf4_dequantize(lib, p: nf4_oracle.NF4Parts) -> torch.Tensor:
    numel = p.quantized_data.numel() * 2
    out = torch.empty(numel, dtype=p.dtype)
    lib.ref_nf4_dequantize(ptr(p.quantized_data), ptr(p.quantized_scalers), ptr(p.quantization_factor), ptr(p.scaler_mean),
                           int(p.dtype == torch.bfloat16), numel, p.block_size, p.scaler_block_size, ptr(out))
    return out.view(p.shape)


def c_fq_per_token(lib, x: torch.Tensor, qp_bf16: bool = False):
    x = x.contiguous()
    rows, K = x.shape
    out = torch.empty_like(x)
    scale = torch.empty(rows, dtype=torch.float32)
    zp = torch.empty(rows, dtype=torch.int32)
    lib.ref_fq_per_token_qp(ptr(x), int(x.dtype == torch.bfloat16), int(qp_bf16), rows, K,
                            ptr(out), ptr(scale), ptr(zp))
    return out, scale, zp


def c_fq_per_group(lib, w: torch.Tensor, g: int, qp_bf16: bool = False):
    w = w.contiguous()
    rows, K = w.shape
    fq = torch.empty_like(w)
    q = torch.empty(w.shape, dtype=torch.int8)
    scale = torch.empty(rows, K // g, dtype=torch.float32)
    lib.ref_fq_per_group_qp(ptr(w), int(w.dtype == torch.bfloat16), int(qp_bf16), rows, K, g,
                            ptr(fq), ptr(q), ptr(scale))
    return fq, q, scale


def c_fq_per_group_uint4_asym(lib, w: torch.Tensor, g: int, qp_bf16: bool = True):
    w = w.contiguous()
    rows, K = w.shape
    fq = torch.empty_like(w)
    q = torch.empty(w.shape, dtype=torch.uint8)
    scale = torch.empty(rows, K // g, dtype=torch.float32)
    zero = torch.empty(rows, K // g, dtype=torch.float32)
    lib.ref_fq_per_group_uint4_asym(ptr(w), int(w.dtype == torch.bfloat16), int(qp_bf16), rows, K, g, ptr(fq), ptr(q), ptr(scale), ptr(zero))
    return fq, q, scale, zero


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Bit-for-bit equality (distinguishes -0.0 from 0.0, treats equal NaN payloads as equal)."""
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    if a.dtype == torch.bfloat16:
        return torch.equal(a.view(torch.int16), b.view(torch.int16))
    if a.dtype == torch.float32:
        return torch.equal(a.view(torch.int32), b.view(torch.int32))
    return torch.equal(a, b)


def seeded_weight(shape, dtype, seed=0, std=0.02):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def parts_equal(a: nf4_oracle.NF4Parts, b: nf4_oracle.NF4Parts) -> bool:
    return (
        torch.equal(a.quantized_data, b.quantized_data)
        and torch.equal(a.quantized_scalers, b.quantized_scalers)
        and bits_equal(a.quantization_factor, b.quantization_factor)
        and bits_equal(a.scaler_mean.reshape(1), b.scaler_mean.reshape(1))
    )
