#!/usr/bin/env python3
"""Benchmark of the QLoRA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3_1_8b]

A "step" is one forward + backward of a Llama-3.1-8B-shaped QLoRA decoder (32 layers, all seven projections
NF4 + LoRA r=16 alpha=32, batch 4 x 2048, bf16, synthetic token ids, random-init weights).  Prints ONE JSON
line: tokens/s for the whole step, the roofline of the dominant kernel (the fused NF4 + LoRA MFMA GEMM; flops
per launch = 2*M*N*K + 2*M*r*min(N or K), timed live with HIP events on the launch stream) and a CPU baseline
(the eager-PyTorch oracle timed on this box's host cores on a bounded sample of the same workload).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (shape, rank, alpha, batch, seq, activation checkpointing)
    "llama3_2_1b": ("llama3_2_1b", 8, 16.0, 4, 2048, False),
    "llama3_1_8b": ("llama3_1_8b", 16, 32.0, 4, 2048, False),
    "llama3_1_70b": ("llama3_1_70b", 16, 32.0, 1, 4096, True),
    # 8da4w QAT of the 8B shape (rank/alpha unused): every linear fake-quantised, group size 32, batch 2 x 4096
    "llama3_1_8b_qat": ("llama3_1_8b", 0, 0.0, 2, 4096, False),
}
HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
# HBM-side bytes per launch of the workload's dominant kernel (fused GEMM; fake quant for the QAT workload), average over
# the launches of one step.  Counters cannot be read from inside this process: the figure comes from the FETCH_SIZE /
# WRITE_SIZE counter runs summarised under profiles/, each of which ends with a line
#     bench.traffic_bytes_per_launch[<workload>] = <bytes>
# that is read back here, so the bench line always quotes the committed measurement (null when there is none).
TRAFFIC_SUMMARIES = {
    "llama3_1_8b": "profiles/nf4_gemm_dense_kernel_hbm_traffic.txt",             # weight expanded once per call (default)
    "llama3_1_8b/fused": "profiles/nf4_gemm_rs_kernel_hbm_traffic.txt",           # --no-expanded-weight
    "llama3_1_8b_qat": "profiles/fake_quant_and_layer_kernels_hbm_traffic.txt",
}


def measured_traffic(workload: str):
    """-> (bytes per launch or None, the summary file it was read from or None)"""
    rel = TRAFFIC_SUMMARIES.get(workload)
    if rel is None:
        return None, None
    try:
        with open(os.path.join(ROOT, rel)) as f:
            for line in f:
                line = line.strip()
                if line.startswith(f"bench.traffic_bytes_per_launch[{workload}]"):
                    return float(line.split("=", 1)[1]), rel
    except (OSError, ValueError):
        pass
    return None, rel


class GemmTimer:
    """HIP-event timing of the fused-GEMM launches while installed in ``ops``.

    An event pair costs the stream about 6 us per timed launch (the GPU idles around the markers), 1.6 % of a step if
    every one of its 255 calls is timed.  So every ``stride``-th launch of each (kind, shape) is timed and the
    others only counted: the averages still come from the timed region itself, the step pays a quarter of the cost."""

    def __init__(self, stride: int = 4):
        self.stride = max(1, stride)
        self.records = []
        self.counts = {}
        self.expanded_calls = 0

    def __call__(self, kind, M, N, K, rank, on_tiles=False):
        # on_tiles (grad-input calls): the GEMM reads the expanded weight its layer's forward call left behind - no expansion
        # launch, and 2 B per weight element instead of the packed weight plus a copy written and read back
        # "fwd" / "bwd": one layer, one call of the library.  "fwd_group" / "bwd_group": the layers of a group with a common
        # input (N and rank are lists), one call; "fwd_gated": the gate / up pair with its gated product in the same call;
        # "bwd_swiglu": the grad-input of the layer after the gated product, carried on to the gradients of gate and up.  Between the events lie all launches of the call: with the weight expanded
        # once per call (many tokens) one expansion launch (the weights of a group together) and one GEMM launch; otherwise one fused launch per
        # member (forward) or the single fused grad-input launch over all members' output columns.
        from torchtune_amd import _lib, ops

        Ns = tuple(N) if isinstance(N, (list, tuple)) else (N,)
        ranks = tuple(rank) if isinstance(rank, (list, tuple)) else (rank,) * len(Ns)
        fwd = kind.startswith("fwd")
        if kind in ("tiled", "tn"):  # QAT: the plain GEMM on a bf16 weight already in tile order, y [M, N] = x [M, K] . Wd^T,
            # and the weight gradient c [N, K] = a [M, N]^T . b [M, K]
            key = (kind, M, Ns[0], K)
            seen = self.counts.get(key, [0, 2.0 * M * Ns[0] * K, 2.0 * (M * K + M * Ns[0] + Ns[0] * K), 1])
            self.counts[key] = [seen[0] + 1] + seen[1:]
            if seen[0] % self.stride:
                return None
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            self.records.append((key, start, end))
            return start, end
        flops = sum(2.0 * M * n * K + 2.0 * M * r * (n if fwd else K) for n, r in zip(Ns, ranks))
        n_out, k_contract = (sum(Ns), K) if fwd else (K, sum(Ns))
        expanded = bool(ops.EXPANDED_WEIGHT_PATH and _lib.load().ttamd_nf4_gemm_expands_weight(M, n_out, k_contract)
                        and (len(Ns) == 1 or not fwd or all(n % 256 == 0 for n in Ns)))
        # algorithmic bytes of a call: both activation tensors once, the packed weight with its fp32 block scalers
        # (0.5 + 4/64 B per element), the adapter operands; with the weight expanded once also the bf16 copy written and
        # read back (4 B per element)
        per_w = 2.0 if on_tiles else 0.5625 + (4.0 if expanded else 0.0)
        if fwd:
            launches = 1 if expanded else len(Ns)
            nbytes = (2.0 * M * K if expanded else 2.0 * M * K * len(Ns)) + sum(2.0 * M * n + per_w * n * K + 2.0 * r * (M + n) for n, r in zip(Ns, ranks))
            if kind == "fwd_gated":  # the gate / up pair: silu(gate) * up written as well (by a pass of its own when not expanded)
                nbytes += 2.0 * M * Ns[0] * (1 if expanded else 3)
        else:
            launches = 1
            nbytes = 2.0 * M * K + sum(2.0 * M * n + per_w * n * K + 2.0 * r * (M + K) for n, r in zip(Ns, ranks))
            if kind == "bwd_swiglu":  # gate and up read, their two gradients written in place of the one grad-input (expanded);
                # otherwise the grad-input written, then read again with gate and up by the pass that writes the two gradients
                nbytes += 2.0 * M * K * (3 if expanded else 5)
        self.expanded_calls += 1 if expanded else 0
        key = (kind, M, Ns if len(Ns) > 1 else Ns[0], K)
        seen = self.counts.get(key, [0, flops, nbytes, launches])
        self.counts[key] = [seen[0] + 1, flops, nbytes, launches]
        if seen[0] % self.stride:
            return None
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        self.records.append((key, start, end))
        return start, end

    def summary(self):
        """-> (launches, launches timed, estimated ms of all launches, flops of all launches, per-shape table); the
        algorithmic bytes of all launches are left in ``self.total_bytes``"""
        timed = {}
        for key, s, e in self.records:
            acc = timed.setdefault(key, [0, 0.0])
            acc[0] += 1
            acc[1] += s.elapsed_time(e)
        total_ms = total_flops = 0.0
        self.total_bytes = 0.0
        per_shape = {}
        n_launches = 0
        for key, (n, flops, nbytes, launches) in self.counts.items():
            self.total_bytes += nbytes * n
            n_launches += launches * n
            n_timed, ms = timed[key]
            avg_ms = ms / n_timed
            total_ms += avg_ms * n
            total_flops += flops * n
            shape_n = "+".join(map(str, key[2])) if isinstance(key[2], tuple) else key[2]
            per_shape[f"{key[0]} M{key[1]} N{shape_n} K{key[3]}"] = {
                "calls": n, "launches": launches * n, "timed": n_timed, "avg_us": round(1e3 * avg_ms, 1),
                "tflops": round(flops / avg_ms / 1e9, 1)}
        return n_launches, len(self.records), total_ms, total_flops, per_shape


class FqTimer:
    """HIP-event timing of the fake-quant launches while installed in ``ops``; every ``stride``-th launch of each
    (kind, shape) is timed, like the GEMM launches.  Algorithmic bytes: one read and one write of the tensor, plus
    the fp32 qparams the launch writes."""

    def __init__(self, stride: int = 4):
        self.stride = max(1, stride)
        self.records = []
        self.counts = {}

    def __call__(self, kind, rows, K, group_size, elem_bytes):
        n = rows * K
        # "per_group_tiled1" / "per_group_tiled2": the weight fake-quantised into one / both tile orders of the library's GEMM
        outputs = 2 if kind == "per_group_tiled2" else 1
        nbytes = (1 + outputs) * n * elem_bytes + (rows * 8 if kind == "per_token" else n // group_size * 4)
        key = (kind, rows, K, group_size, elem_bytes)
        seen = self.counts.get(key, [0, nbytes])
        self.counts[key] = [seen[0] + 1, nbytes]
        if seen[0] % self.stride:
            return None
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        self.records.append((key, start, end))
        return start, end

    def summary(self):
        timed = {}
        for key, s, e in self.records:
            acc = timed.setdefault(key, [0, 0.0])
            acc[0] += 1
            acc[1] += s.elapsed_time(e)
        by = {}
        for key, (n, nbytes) in self.counts.items():
            n_timed, ms = timed[key]
            acc = by.setdefault(key[0], [0, 0.0, 0.0])
            acc[0] += n
            acc[1] += ms / n_timed * n
            acc[2] += float(nbytes) * n
        return {k: {"launches": v[0], "avg_us": round(1e3 * v[1] / v[0], 1), "gbps": round(v[2] / v[1] / 1e6, 1),
                    "ms": v[1], "bytes": v[2]} for k, v in by.items()}


def cpu_baseline_qat(shape_name: str, group: int, layers: int, max_tokens: int, min_seconds: float = 10.0):
    """CPU oracle of the fake-quantised linear (eager PyTorch: fq(x), fq(W), F.linear, straight-through backward) on
    one decoder layer's seven linears at the workload's token count, repeated until `min_seconds`; tokens/s for the
    full depth."""
    from oracle import fake_quant_oracle as fqo
    from torchtune_amd.harness import SHAPES

    s = SHAPES[shape_name]
    kv = s.n_kv_heads * s.head_dim
    dims = [(s.dim, s.dim), (kv, s.dim), (kv, s.dim), (s.dim, s.dim), (s.hidden, s.dim), (s.hidden, s.dim), (s.dim, s.hidden)]
    gen = torch.Generator().manual_seed(0)
    cores = torch.get_num_threads()
    ws = [(torch.randn(N, K, generator=gen) * 0.02).to(torch.bfloat16).requires_grad_() for N, K in dims]
    xs = [torch.randn(max_tokens, K, generator=gen).to(torch.bfloat16).requires_grad_() for _, K in dims]
    reps, dt = 0, 0.0
    t0 = time.perf_counter()
    while dt < min_seconds:
        for w, x in zip(ws, xs):
            y = fqo.fake_quantized_linear(x, w, group)
            (y.float() ** 2).sum().backward()
        reps += 1
        dt = time.perf_counter() - t0
    return {
        "value": round(max_tokens * reps / (dt * layers), 3),
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"eager-PyTorch oracle, fwd+bwd of one {shape_name} layer's seven 8da4w fake-quantised linears (group {group}) "
                  f"at {max_tokens} tokens x {reps} passes ({dt:.1f} s on {cores} threads), extrapolated x{layers} layers",
    }


def cpu_baseline(shape_name: str, rank: int, alpha: float, tokens_sample: int, layers: int, max_tokens: int,
                 min_seconds: float = 10.0):
    """Time the CPU oracle (eager PyTorch, the op sequence the reference executes) on one decoder layer's seven
    QLoRA linears, forward + backward, and scale to tokens/s for the full depth.  The token count of the sample
    starts at `tokens_sample` and is quadrupled up to the workload's tokens per step, then the pass is repeated, until
    the sample takes at least `min_seconds`."""
    from oracle import lora_oracle, nf4_oracle
    from torchtune_amd.harness import SHAPES

    s = SHAPES[shape_name]
    kv = s.n_kv_heads * s.head_dim
    dims = [(s.dim, s.dim), (kv, s.dim), (kv, s.dim), (s.dim, s.dim), (s.hidden, s.dim), (s.hidden, s.dim), (s.dim, s.hidden)]
    gen = torch.Generator().manual_seed(0)
    cores = torch.get_num_threads()
    weights = []
    for N, K in dims:
        W = (torch.randn(N, K, generator=gen) * 0.02).to(torch.bfloat16)
        parts = nf4_oracle.nf4_quantize(W, 64, 256)
        A = lora_oracle.lora_a_init_(torch.empty(rank, K), gen).to(torch.bfloat16).requires_grad_()
        B = (torch.randn(N, rank, generator=gen) * 0.01).to(torch.bfloat16).requires_grad_()
        weights.append((K, parts, A, B))
    tokens = tokens_sample
    reps = 1
    while True:
        xs = [torch.randn(tokens, K, generator=gen).to(torch.bfloat16).requires_grad_() for K, _, _, _ in weights]
        t0 = time.perf_counter()
        for _ in range(reps):
            for (K, parts, A, B), x in zip(weights, xs):
                y = lora_oracle.lora_linear_forward(x, parts, A, B, alpha, rank)
                (y.float() ** 2).sum().backward()
        dt = time.perf_counter() - t0
        if dt >= min_seconds:
            break
        if tokens < max_tokens:
            tokens = min(max_tokens, tokens * 4)
        else:
            reps = max(reps + 1, int(reps * 1.2 * min_seconds / dt) + 1)
    return {
        "value": round(tokens * reps / (dt * layers), 3),
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "sample": f"eager-PyTorch oracle, fwd+bwd of one {shape_name} layer's seven NF4+LoRA linears at {tokens} tokens x {reps} passes "
                  f"({dt:.1f} s on {cores} threads), extrapolated x{layers} layers; attention, norms and loss not included",
    }


def gemm_kernels(dev, tokens=(256, 512, 1024, 1536)) -> dict:
    """The GEMM kernels of the path in isolation, each against its alternative in the same process (HIP events, best of
    two rounds of 30 launches, microseconds):

    * ``dispatch_vs_dequantise_plus_vendor_gemm``: what the library's dispatch runs for a forward and a grad-input of the
      8B projections at evaluation / short-batch token counts against the reference's order of work with the vendor
      library's GEMM (``ttamd_nf4_dequantize`` into a dense bf16 weight + ``F.linear`` / ``gy @ W``);
    * ``weight_gradient``: ``gemm_tn`` with and without contraction slices for the last partial round of tiles, and the
      vendor library's ``a.T @ b``, at the 8B shapes of the 8da4w QAT step (8192 tokens);
    * ``grad_input_tiles``: the plain GEMM's grad-input on tiles of the transposed weight against the same launch on the
      forward launch's tiles (transposing LDS reads, no second copy of the weight)."""
    import torch.nn.functional as F

    from torchtune_amd import ops, to_nf4

    def timed(fn, iters=30):
        best = None
        for _ in range(2):
            for _ in range(5):
                fn()
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(iters):
                fn()
            end.record()
            torch.cuda.synchronize()
            us = start.elapsed_time(end) / iters * 1e3
            best = us if best is None else min(best, us)
        return round(best, 1)

    BF = torch.bfloat16
    gen = torch.Generator(device=dev).manual_seed(4)
    warm = torch.randn(8192, 8192, device=dev, dtype=BF)
    for _ in range(30):
        warm @ warm
    del warm
    out = {"dispatch_vs_dequantise_plus_vendor_gemm": [], "weight_gradient": [], "grad_input_tiles": []}
    for N, K in ((4096, 4096), (14336, 4096), (4096, 14336)):
        t = to_nf4((torch.randn(N, K, device=dev, generator=gen) * 0.02).to(BF))
        bs = t.block_scalers()
        A = (torch.randn(16, K, device=dev, generator=gen) * 0.05).to(BF)
        B = (torch.randn(N, 16, device=dev, generator=gen) * 0.05).to(BF)
        for M in tokens:
            x = torch.randn(M, K, device=dev, generator=gen).to(BF)
            gy = torch.randn(M, N, device=dev, generator=gen).to(BF)
            h = torch.randn(M, 16, device=dev, generator=gen).to(BF)
            gh = torch.randn(M, 16, device=dev, generator=gen).to(BF)
            trf, trb = t.backward_copy_for(M, True), t.backward_copy_for(M, False)
            out["dispatch_vs_dequantise_plus_vendor_gemm"].append({
                "weight": f"{N}x{K}", "tokens": M,
                "fwd_own_us": timed(lambda: ops.nf4_lora_linear_fwd(x, t.quantized_data, bs, N, h, B, 2.0, block_scalers_t=trf[1] if trf else None)),
                "fwd_dequant_vendor_us": timed(lambda: F.linear(x, t.get_original_weight())),
                "dx_own_us": timed(lambda: ops.nf4_linear_bwd_dx(gy, t.quantized_data, bs, K, gh, A, transposed=trb)),
                "dx_dequant_vendor_us": timed(lambda: gy @ t.get_original_weight()),
            })
        del t, bs
    M = 8192
    for Ns, K in (((4096,), 4096), ((4096, 1024, 1024), 4096), ((14336, 14336), 4096), ((4096,), 14336)):
        a = [torch.randn(M, N, device=dev, generator=gen).to(BF) for N in Ns]
        b = torch.randn(M, K, device=dev, generator=gen).to(BF)
        run = (lambda: ops.gemm_tn_group(a, b)) if len(Ns) > 1 else (lambda: ops.gemm_tn(a[0], b))
        row = {"a_columns": "+".join(str(n) for n in Ns), "b_columns": K, "tokens": M, "tiles": sum(Ns) // 256 * (K // 256),
               "flop": 2.0 * M * sum(Ns) * K}
        ops.TN_TAIL_SLICES = True
        row["own_us"] = timed(run, 20)
        ops.TN_TAIL_SLICES = False
        row["own_unsliced_us"] = timed(run, 20)
        ops.TN_TAIL_SLICES = True
        row["vendor_us"] = timed(lambda: [m.t().matmul(b) for m in a], 20)
        row["own_tflops"] = round(row["flop"] / row["own_us"] / 1e6, 1)
        out["weight_gradient"].append(row)
        del a, b
    for N, K in ((4096, 4096), (14336, 4096), (4096, 14336)):
        w = (torch.randn(N, K, device=dev, generator=gen) * 0.02).to(BF)
        tf, tb, _ = ops.fq_per_group_int4_sym_tiled(w, 32)
        gy = torch.randn(M, N, device=dev, generator=gen).to(BF)
        row = {"weight": f"{N}x{K}", "tokens": M, "flop": 2.0 * M * N * K,
               "on_transposed_tiles_us": timed(lambda: ops.tiled_linear(gy, tb, K), 20),
               "on_forward_tiles_us": timed(lambda: ops.tiled_linear_dx(gy, tf, K), 20)}
        row["bit_equal"] = bool(torch.equal(ops.tiled_linear(gy, tb, K), ops.tiled_linear_dx(gy, tf, K)))
        out["grad_input_tiles"].append(row)
        del w, tf, tb, gy
    return out


def secondary_kernels(dev, offload_leg: bool = True) -> dict:
    """Achieved HBM GB/s of the bandwidth-bound kernels of the path on the largest 8B weight / activation shapes:
    algorithmic bytes (2.515747 B/element for the NF4 codec, 4 B/element for fake quant) / HIP-event time."""
    from torchtune_amd import ops, to_nf4

    def timed(fn, iters=30):
        for _ in range(10):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / iters * 1e-3

    out = {}
    gen = torch.Generator(device=dev).manual_seed(2)
    W = (torch.randn(14336, 4096, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    t = to_nf4(W)
    n = W.numel()
    dense = torch.empty_like(W)  # preallocated: with the allocator in the loop the host barely keeps ahead of a 25 us kernel
    out["nf4_dequantize 14336x4096 bf16"] = round(n * 2.515747 / timed(lambda: t.get_original_weight(out=dense)) / 1e9, 1)
    del dense
    # the 70B gate / up weight: 118 MB of codes in, 470 MB out — more than the 256 MB last-level cache holds, so this is
    # the rate against HBM itself (the 8B weight above can live in that cache between launches)
    Wb = (torch.randn(28672, 8192, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    tb = to_nf4(Wb)
    nb = Wb.numel()
    out["nf4_dequantize 28672x8192 bf16 (235 M elements, beyond the last-level cache)"] = round(
        nb * 2.515747 / timed(lambda: tb.get_original_weight(out=Wb), iters=20) / 1e9, 1)
    del Wb, tb
    out["nf4_quantize 14336x4096 bf16"] = round(n * 2.515747 / timed(lambda: ops.nf4_quantize(W, 64, 256)) / 1e9, 1)
    out["fq_per_group_int4_sym g32 14336x4096 bf16"] = round(
        (n * 4 + n / 32 * 4) / timed(lambda: ops.fq_per_group_int4_sym(W, 32)) / 1e9, 1)
    out["fq_per_group_uint4_asym g256 14336x4096 bf16 (4w-qat)"] = round(
        (n * 4 + n / 256 * 8) / timed(lambda: ops.fq_per_group_uint4_asym(W, 256, want_qparams=True)) / 1e9, 1)
    x = torch.randn(8192, 14336, device=dev, generator=gen).to(torch.bfloat16)
    out["fq_per_token_int8_asym 8192x14336 bf16"] = round(
        x.numel() * 4 / timed(lambda: ops.fq_per_token_int8_asym(x, want_qparams=False)) / 1e9, 1)
    if offload_leg:
        host = torch.empty(14336, 4096, dtype=torch.bfloat16, pin_memory=True)
        out["checkpoint offload: nf4_dequantize 14336x4096 written into pinned host memory (PCIe-bound, host bytes only)"] = round(
            n * 2 / timed(lambda: t.get_original_weight(out=host), iters=5) / 1e9, 1)
    # forward for a handful of tokens (decode): the packed weight is streamed once, 0.5625 B per element.  The kernels
    # take 7-15 us, less than a launch from Python costs, so 20 launches are captured in a HIP graph and the replay timed.
    bs = t.block_scalers()
    bst = t.backward_copy()[1] if t.backward_copy() is not None else None
    for m_tok in (1, 16):
        xs = torch.randn(m_tok, 4096, device=dev, generator=gen).to(torch.bfloat16)
        ys = ops.nf4_lora_linear_fwd(xs, t.quantized_data, bs, 14336, block_scalers_t=bst)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(20):
                yg = ops.nf4_lora_linear_fwd(xs, t.quantized_data, bs, 14336, block_scalers_t=bst)
        sec = timed(graph.replay, iters=10) / 20
        torch.cuda.synchronize()
        if not torch.equal(yg, ys):
            raise RuntimeError("bench: the graph replay of the few-token forward differs from the eager result")
        out[f"nf4_lora_linear_fwd M={m_tok} 14336x4096 (few-token kernel, packed-weight bytes)"] = round(n * 0.5625 / sec / 1e9, 1)
        del graph
    # the same for two layers with a common input (gate / up: 2 x 14336 x 4096, rank 16) as one group call: one launch for
    # both hidden products, one for both outputs
    t2 = to_nf4((torch.randn(14336, 4096, device=dev, generator=gen) * 0.02).to(torch.bfloat16))
    members = []
    for tt in (t, t2):
        la = (torch.randn(16, 4096, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        lb = (torch.randn(14336, 16, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        members.append(ops.GroupMember(tt.quantized_data, tt.block_scalers(), tt.backward_copy(), la, lb, None, 2.0, 14336))
    for m_tok in (1, 16):
        xs = torch.randn(m_tok, 4096, device=dev, generator=gen).to(torch.bfloat16)
        _, ys = ops.lora_group_fwd(xs, members)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(20):
                _, yg = ops.lora_group_fwd(xs, members)
        sec = timed(graph.replay, iters=10) / 20
        torch.cuda.synchronize()
        if not all(torch.equal(a, b) for a, b in zip(yg, ys)):
            raise RuntimeError("bench: the graph replay of the grouped few-token forward differs from the eager result")
        out[f"lora_group_fwd M={m_tok} 2 x 14336x4096 r=16 (gate / up as one group, packed-weight bytes, both launches)"] = round(
            2 * n * 0.5625 / sec / 1e9, 1)
        del graph
    return {"unit": "GB/s (algorithmic bytes / HIP-event time, HBM peak 8000)", **out}


def config1_leg(dev, runs: int = 15, warmups: int = 3) -> dict:
    """The single-layer configuration (one QLoRA ``LoRALinear``: bf16 [2048, 2048] N(0, 0.02) base weight quantised with
    ``to_nf4`` (64 / 256), rank 8, alpha 16, A Kaiming-uniform, B ~ N(0, 0.01), x bf16 [4, 512, 2048] ~ N(0, 1), seed 0,
    forward + backward of sum(y^2)), timed in full on the GPU and on the host: median of ``runs`` after ``warmups``
    warm-ups each.  The CPU figure is the eager-PyTorch oracle (the reference's op sequence) on this box's host cores."""
    import statistics

    from oracle import lora_oracle, nf4_oracle
    from torchtune_amd.modules.peft import LoRALinear

    torch.manual_seed(0)
    W = (torch.randn(2048, 2048) * 0.02).to(torch.bfloat16)
    A = lora_oracle.lora_a_init_(torch.empty(8, 2048)).to(torch.bfloat16)
    B = (torch.randn(2048, 8) * 0.01).to(torch.bfloat16)
    x = torch.randn(4, 512, 2048).to(torch.bfloat16)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            layer = LoRALinear(2048, 2048, rank=8, alpha=16.0, quantize_base=True)
    finally:
        torch.set_default_dtype(prev)
    with torch.no_grad():
        layer.weight.copy_(W.to(dev))
        layer.lora_a.weight.copy_(A.to(dev))
        layer.lora_b.weight.copy_(B.to(dev))
    xd = x.to(dev).requires_grad_()

    grads = (layer.lora_a.weight, layer.lora_b.weight, xd)

    def gpu_run():
        y = layer(xd)
        (y.float() ** 2).sum().backward()
        for p in grads:  # the three tensors that received a gradient (Module.zero_grad walks the module tree: 20 us)
            p.grad = None

    gpu_ms = []
    for i in range(warmups + runs):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        gpu_run()
        torch.cuda.synchronize()
        if i >= warmups:
            gpu_ms.append(1e3 * (time.perf_counter() - t0))
    # kernel time alone (the layer is a handful of launches, so wall time above is mostly launch latency)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(runs):
        gpu_run()
    end.record()
    torch.cuda.synchronize()
    stream_ms = start.elapsed_time(end) / runs

    # The launches of the layer alone: its forward, the loss gradient 2 y and its backward are captured once in a HIP graph
    # (the library's entry points only launch on the stream they are given) and replayed back to back, so that no host work
    # lies between the kernels.  34.76 GFLOP per replay (2 M N K per direction + the rank-8 products).
    from torchtune_amd import ops

    wq = layer.weight
    qd, bs = wq.quantized_data, wq.block_scalers()
    tr_f, tr_b = wq.backward_copy_for(2048, True), wq.backward_copy_for(2048, False)
    Ad, Bd = layer.lora_a.weight.detach(), layer.lora_b.weight.detach()
    x2 = xd.detach().reshape(-1, 2048)

    def launches():
        y, h = ops.qlora_linear_fwd(x2, qd, bs, 2048, Ad, Bd, 2.0, None, block_scalers_t=tr_f[1] if tr_f else None)
        gy = (y.float() * 2.0).to(torch.bfloat16)
        return ops.qlora_linear_bwd(gy, x2, h, qd, bs, Ad, Bd, 2.0, transposed=tr_b)

    launches()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launches()
    replays = 50
    for _ in range(5):
        graph.replay()
    start.record()
    for _ in range(replays):
        graph.replay()
    end.record()
    torch.cuda.synchronize()
    kernel_us = 1e3 * start.elapsed_time(end) / replays
    del graph
    flops = 2 * (2 * 2048 * 2048 * 2048) + 6 * 2048 * 8 * (2048 + 2048)

    parts = nf4_oracle.nf4_quantize(W, 64, 256)
    xo = x.clone().requires_grad_()
    Ao, Bo = A.clone().requires_grad_(), B.clone().requires_grad_()
    cpu_ms = []
    for i in range(warmups + runs):
        t0 = time.perf_counter()
        yo = lora_oracle.lora_linear_forward(xo, parts, Ao, Bo, 16.0, 8)
        (yo.float() ** 2).sum().backward()
        if i >= warmups:
            cpu_ms.append(1e3 * (time.perf_counter() - t0))
        xo.grad = Ao.grad = Bo.grad = None
    tokens = 4 * 512
    g, c = statistics.median(gpu_ms), statistics.median(cpu_ms)
    return {
        "workload": "one QLoRA LoRALinear 2048x2048 r=8 alpha=16, x [4, 512, 2048], fwd+bwd of sum(y^2), seed 0",
        "runs": runs, "warmups": warmups,
        "gpu_ms_median": round(g, 3), "gpu_ms_back_to_back": round(stream_ms, 3), "gpu_tokens_per_s": round(tokens / g * 1e3, 1),
        "gpu_kernels_us_graph_replay": round(kernel_us, 1), "kernels_tflops": round(flops / kernel_us / 1e6, 1),
        "kernels_frac_of_bf16_mfma_peak": round(flops / kernel_us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
        "kernels_note": "forward + loss gradient + backward launches of the layer replayed from one HIP graph, "
                        "34.76 GFLOP per replay; gpu_ms_* above include Python, autograd and the ABI calls",
        "cpu_ms_median": round(c, 2), "cpu_tokens_per_s": round(tokens / c * 1e3, 1), "cpu_cores": torch.get_num_threads(),
        "cpu_kind": "port (eager-PyTorch oracle, timed in full)",
    }


def memory_leg(build, step, dev) -> dict:
    """Peak device memory of one forward + backward (``torch.cuda.max_memory_allocated``) for the three ways the NF4 GEMMs
    can run: the weight expanded once per call (the default at training sizes: scratch memory of one weight or group at a
    time, no transposed copy ever built), the fused kernel with the transposed copy of the codes its grad-input streams
    (0.5625 B per weight element), and the fused kernel without it (first-generation grad-input kernel)."""
    from torchtune_amd import nf4_tensor, ops

    out = {}
    keep_expanded, keep_copy = ops.EXPANDED_WEIGHT_PATH, nf4_tensor.BACKWARD_COPY
    for name, expanded, copy in (("expanded_weight_per_call", True, True), ("fused_with_backward_copy", False, True),
                                 ("fused_without_backward_copy", False, False)):
        ops.EXPANDED_WEIGHT_PATH, nf4_tensor.BACKWARD_COPY = expanded, copy
        try:
            model = build()
            step(model)  # builds the derived copies, warms the allocator
            torch.cuda.synchronize()
            resident = torch.cuda.memory_allocated(dev)
            torch.cuda.reset_peak_memory_stats(dev)
            step(model)
            torch.cuda.synchronize()
            out[name] = {"resident_gib": round(resident / 2**30, 3), "peak_gib": round(torch.cuda.max_memory_allocated(dev) / 2**30, 3)}
            del model
            torch.cuda.empty_cache()
        finally:
            ops.EXPANDED_WEIGHT_PATH, nf4_tensor.BACKWARD_COPY = keep_expanded, keep_copy
    out["unit"] = "GiB (torch.cuda.memory_allocated after a step = weights + derived copies; max_memory_allocated over one fwd+bwd)"
    return out


def optimizer_leg(model, tokens, labels, train_step, qat: bool, steps: int, tokens_per_step: int):
    """fwd + bwd + optimizer step, with the optimizer of the reference's configs: ``torch.optim.AdamW(fused=True)``,
    lr 3e-4 / weight decay 0.01 for QLoRA (``recipes/configs/llama3_1/8B_qlora_single_device.yaml:60-64``), lr 2e-5
    for QAT (``recipes/configs/llama3_1/8B_qat_full.yaml:66-69``).  The reference's own ``tokens_per_second_per_gpu``
    includes the optimizer (``recipes/lora_finetune_single_device.py:666-671``); the headline metric does not."""
    if steps <= 0:
        return None
    params = [p for p in model.parameters() if p.requires_grad]
    opt = (torch.optim.AdamW(params, lr=2e-5, fused=True) if qat
           else torch.optim.AdamW(params, lr=3e-4, weight_decay=0.01, fused=True))

    def opt_step():
        loss = train_step(model, tokens, labels)
        opt.step()
        opt.zero_grad(set_to_none=True)
        return loss

    opt_step()  # allocates the optimizer state
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = opt_step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    out = {
        "value": round(tokens_per_step * steps / dt, 1),
        "unit": "tokens/s",
        "ms_per_step": round(1e3 * dt / steps, 2),
        "steps": steps,
        "optimizer": "torch.optim.AdamW(fused=True) over %d tensors / %.1f M trainable parameters" % (
            len(params), sum(p.numel() for p in params) / 1e6),
        "loss_after": float(loss),
    }
    del opt
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="llama3_1_8b", choices=sorted(WORKLOADS) + ["hbm_kernels", "config1_single_layer", "gemm_kernels"],
                    help="a decoder configuration, or 'hbm_kernels': only the bandwidth-bound kernels in isolation (NF4 "
                         "dequantise / quantise, fake quant, few-token forward), the launches a kernel trace of them should hold; "
                         "'gemm_kernels': the GEMM kernels in isolation beside their alternatives (dispatch at a few hundred tokens "
                         "against dequantise + vendor GEMM, the weight-gradient GEMM with and without slices of its last partial "
                         "round, the grad-input on forward tiles); 'config1_single_layer': one 2048 x 2048 QLoRA layer")
    ap.add_argument("--no-offload-leg", action="store_true",
                    help="hbm_kernels: skip the dequantise-into-pinned-host-memory leg (PCIe-bound launches of the same kernel)")
    ap.add_argument("--cpu-tokens", type=int, default=512,
                    help="starting token count of the CPU-baseline sample, grown until it takes >= 10 s (0 = skip)")
    ap.add_argument("--optimizer-steps", type=int, default=3,
                    help="after the timed fwd+bwd steps, time this many steps that also run the recipe's fused AdamW "
                         "(reported beside the metric as `with_adamw`; 0 = skip)")
    ap.add_argument("--qat-scales", default="float32", choices=["float32", "bfloat16"],
                    help="scales_precision of the QAT workload: float32 is the reference quantizer's default, bfloat16 rounds "
                         "every scale before it quantises and dequantises")
    ap.add_argument("--sdpa", default="efficient", choices=["efficient", "flash", "default"],
                    help="which of PyTorch's scaled_dot_product_attention backends the stack asks for (attention is stock "
                         "PyTorch; 'flash' is what the dispatcher picks by itself)")
    ap.add_argument("--gemm-timing-stride", type=int, default=4,
                    help="time every n-th fused-GEMM / fake-quant launch of each shape with HIP events (1 = every launch)")
    ap.add_argument("--no-memory-leg", action="store_true",
                    help="skip the peak-memory measurement (two extra model builds with one step each)")
    ap.add_argument("--no-config1", action="store_true", help="skip the single-layer configuration timed on GPU and CPU")
    ap.add_argument("--no-gated-epilogue", action="store_true",
                    help="A/B: silu(gate) * up as a pass of its own instead of the epilogue of the gate / up GEMM launch")
    ap.add_argument("--swiglu-bwd-epilogue", action="store_true",
                    help="A/B: the backward of silu(gate) * up from the epilogue of the down projection's grad-input GEMM launch "
                         "instead of a pass of its own (QLoRA workloads)")
    ap.add_argument("--no-qat-tn-group", action="store_true",
                    help="A/B (QAT workloads): one weight-gradient launch per member of a group instead of one for the group")
    ap.add_argument("--no-fused-qkv-post", action="store_true",
                    help="rotary embedding and key / value head expansion as four launches per layer and direction instead of one")
    ap.add_argument("--no-fused-output-loss", action="store_true",
                    help="QAT workload: the fake-quantised output projection and the loss as two autograd nodes (the gradient of the "
                         "logits is then rescaled by the incoming gradient in a pass of its own) instead of one")
    ap.add_argument("--no-fused-swiglu-bwd", action="store_true",
                    help="the backward of silu(gate) * up as a pass of its own ahead of the gate / up pair's adapter backward, instead "
                         "of inside the pass that multiplies its results with the adapters")
    ap.add_argument("--no-fused-add-norm", action="store_true",
                    help="A/B: the additions of the residual stream as passes of their own instead of inside the RMSNorm that "
                         "follows each of them")
    ap.add_argument("--no-group", action="store_true",
                    help="one call per projection, as the reference's modules make them, instead of the group kernels for the "
                         "projections that share an input (q/k/v, gate/up): for A/B timing")
    ap.add_argument("--no-expanded-weight", action="store_true",
                    help="keep the fused NF4 GEMM (expansion repeated per tile, no scratch memory) also for many tokens, "
                         "instead of expanding the weight once per call and running the plain bf16 GEMM")
    ap.add_argument("--no-qat-tiled-gemm", action="store_true",
                    help="QAT workload: row-major fq(W) and the vendor library's GEMM for every matmul, instead of fake-quantising "
                         "the weights straight into the tile order of the library's own GEMM for forward and grad-input")
    ap.add_argument("--keep-forward-tiles", type=int, default=None, metavar="TOKENS",
                    help="calls of at most this many tokens hand their expanded weight to the backward of the same layer, whose "
                         "grad-input GEMM reads it instead of expanding the weight again (0: never; default: the library's rule, "
                         "torchtune_amd.ops.KEEP_FORWARD_TILES_MAX_TOKENS = 8192)")
    ap.add_argument("--resident-tiles-gib", type=float, default=0.0, metavar="GIB",
                    help="keep up to this many GiB of expanded NF4 weights across calls (2 B per weight element; the frozen base "
                         "weight never changes, so later steps run their GEMMs on the kept tiles and launch no expansion; "
                         "torchtune_amd.ops.RESIDENT_TILES_MAX_BYTES). Default 0: every call expands its weight, as the "
                         "reference dequantises it in every call")
    ap.add_argument("--no-backward-copy", action="store_true",
                    help="keep no transposed copy of the NF4 codes (0.5625 B per weight element less): the expanded-weight path then "
                         "builds W^T from the weight's own codes, the fused path falls back to its first-generation grad-input kernel")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="before the steps, run one elementwise kernel that reads and writes this many MiB: the known-size "
                         "dispatch that FETCH_SIZE / WRITE_SIZE counter runs are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); multi-GPU runs are not part of it", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the hot path has no CPU implementation", file=sys.stderr)
        return 2

    from torchtune_amd import ops
    from torchtune_amd import harness
    from torchtune_amd.harness import SHAPES, build_qat_decoder, build_qlora_decoder, train_step

    harness.SDPA_BACKEND = args.sdpa
    harness.GROUP_SHARED_INPUT = not args.no_group
    harness.GATED_EPILOGUE = not args.no_gated_epilogue
    harness.FUSED_ADD_NORM = not args.no_fused_add_norm
    harness.FUSED_QKV_POST = not args.no_fused_qkv_post
    harness.FUSED_QAT_OUTPUT_LOSS = not args.no_fused_output_loss
    from torchtune_amd.modules.peft import group as _peft_group
    _peft_group.FUSED_SWIGLU_BWD = not args.no_fused_swiglu_bwd
    harness.SWIGLU_BWD_EPILOGUE = args.swiglu_bwd_epilogue
    ops.EXPANDED_WEIGHT_PATH = not args.no_expanded_weight
    if args.keep_forward_tiles is not None:
        ops.KEEP_FORWARD_TILES_MAX_TOKENS = args.keep_forward_tiles
    ops.RESIDENT_TILES_MAX_BYTES = int(args.resident_tiles_gib * 2**30)
    if args.no_qat_tiled_gemm:
        from torchtune_amd import qat as qat_module
        qat_module.TILED_GEMM = False
    if args.no_qat_tn_group:
        from torchtune_amd import qat as qat_module
        qat_module.TN_GROUP_GEMM = False
    if args.no_backward_copy:
        from torchtune_amd import nf4_tensor
        nf4_tensor.BACKWARD_COPY = False

    if args.workload == "gemm_kernels":
        dev = torch.device("cuda", 0)
        torch.cuda.set_device(dev)
        table = gemm_kernels(dev)
        best = max(table["weight_gradient"], key=lambda r: r["own_tflops"])
        print(json.dumps({
            "metric": "weight-gradient GEMM TFLOP/s (gemm_tn, 8192 tokens, 1 GPU)", "value": best["own_tflops"], "unit": "TFLOP/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic (random operands)",
            "config": {"workload": "the GEMM kernels of the path in isolation, each beside its alternative"},
            "roofline": {"bound": "mfma", "kernel": "gemm_tn_kernel", "achieved": best["own_tflops"], "peak": MFMA_BF16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(best["own_tflops"] / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None},
            "gemm_kernels": table}))
        return 0
    if args.workload == "config1_single_layer":
        dev = torch.device("cuda", 0)
        torch.cuda.set_device(dev)
        leg = config1_leg(dev)
        print(json.dumps({
            "metric": "QLoRA LoRALinear fwd+bwd tokens/sec (one 2048x2048 layer, 1 GPU)", "value": leg["gpu_tokens_per_s"], "unit": "tokens/s",
            "n_gpus": 1, "steps": leg["runs"], "warmup": leg["warmups"], "ms_per_step": leg["gpu_ms_median"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic (seed 0)", "config": {"workload": leg["workload"]},
            "roofline": {"bound": "mfma", "kernel": "the layer's launches replayed from one HIP graph", "achieved": leg["kernels_tflops"],
                         "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": leg["kernels_frac_of_bf16_mfma_peak"], "traffic": None},
            "cpu_baseline": {"value": leg["cpu_tokens_per_s"], "unit": "tokens/s", "cores": leg["cpu_cores"], "kind": "port",
                             "sample": "the whole configuration, median of %d runs" % leg["runs"]},
            "config1_single_layer": leg}))
        return 0
    if args.workload == "hbm_kernels":
        dev = torch.device("cuda", 0)
        torch.cuda.set_device(dev)
        table = secondary_kernels(dev, offload_leg=not args.no_offload_leg)
        key = "nf4_dequantize 28672x8192 bf16 (235 M elements, beyond the last-level cache)"
        print(json.dumps({
            "metric": "NF4 dequantise GB/s beyond the last-level cache (28672x8192, 1 GPU)", "value": table[key], "unit": "GB/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic (random-init N(0,0.02) weights)",
            "config": {"workload": "bandwidth-bound kernels of the path in isolation"},
            "roofline": {"bound": "hbm", "kernel": "nf4_dequantize_kernel", "achieved": table[key], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": round(table[key] / HBM_PEAK_GBPS, 4), "traffic": None},
            "hbm_bound_kernels": table}))
        return 0
    shape_name, rank, alpha, batch, seq, ac = WORKLOADS[args.workload]
    qat = args.workload.endswith("_qat")
    qat_group = 32
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if qat:
        model = build_qat_decoder(shape_name, groupsize=qat_group, device=dev, seed=0, activation_checkpointing=ac,
                                  scales_precision=getattr(torch, args.qat_scales))
    else:
        model = build_qlora_decoder(shape_name, rank, alpha, device=dev, seed=0, activation_checkpointing=ac)
    gen = torch.Generator(device=dev).manual_seed(1)
    vocab = SHAPES[shape_name].vocab
    tokens = torch.randint(0, vocab, (batch, seq), device=dev, generator=gen)
    labels = torch.randint(0, vocab, (batch, seq), device=dev, generator=gen)

    def step():
        loss = train_step(model, tokens, labels)
        model.zero_grad(set_to_none=True)
        return loss

    if args.calibration_copy_mib > 0:
        src = torch.ones(args.calibration_copy_mib << 18, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.add(src, 1.0, out=dst)  # one vectorized_elementwise_kernel dispatch: reads and writes exactly src.nbytes
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timer = GemmTimer(args.gemm_timing_stride)
    fq_timer = FqTimer(args.gemm_timing_stride)
    ops.set_gemm_timer(timer)
    ops.set_fq_timer(fq_timer)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats(dev)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    peak_timed = torch.cuda.max_memory_allocated(dev)
    ops.set_gemm_timer(None)
    ops.set_fq_timer(None)
    ms_per_step = 1e3 * dt / args.steps
    with_adamw = optimizer_leg(model, tokens, labels, train_step, qat, args.optimizer_steps, batch * seq)

    if qat:
        fq = fq_timer.summary()
        own_gemm = None
        if timer.counts:
            g_launches, g_timed, g_ms, g_flops, g_shapes = timer.summary()
            own_gemm = {"kernel": "nf4_gemm_dense_kernel on weights fake-quantised straight into its tile order (forward and "
                                  "grad-input) and gemm_tn_kernel (weight gradients) for every linear that gives a full round of "
                                  "256 x 256 tiles; q / k / v and gate / up run as groups (one forward and one grad-input launch "
                                  "each) unless --no-group; the weight gradients of the 1024-wide k / v projections run on the "
                                  "vendor library",
                        "launches": g_launches, "tflops": round(g_flops / g_ms / 1e9, 1), "frac_of_bf16_mfma_peak":
                        round(g_flops / g_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4), "gemm_ms_per_step": round(g_ms / args.steps, 2),
                        "per_shape": g_shapes}
        fq_ms = sum(v["ms"] for v in fq.values())
        fq_bytes = sum(v["bytes"] for v in fq.values())
        achieved = fq_bytes / fq_ms / 1e6 if fq_ms > 0 else 0.0
        result = {
            "metric": "8da4w QAT fwd+bwd tokens/sec (Llama-3.1-8B, 1 GPU)",
            "value": round(batch * seq * args.steps / dt, 1),
            "unit": "tokens/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(ms_per_step, 2),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "bf16",
            "data": "synthetic (uniform random token ids, random-init N(0,0.02) bf16 weights)",
            "config": {
                "workload": f"{shape_name}-shaped decoder, every linear (incl. output) 8da4w fake-quantised as the reference's "
                            "quantizer does it: per-token asymmetric int8 activations (min/max with zero point), "
                            f"per-group({qat_group}) symmetric int4 weights, {args.qat_scales} scales, batch {batch} x seq {seq}, "
                            "fwd+bwd with weight gradients, output projection and cross-entropy; "
                            f"attention = torch SDPA, backend '{args.sdpa}'",
                "global_batch": batch,
                "seq_len": seq,
                "loss": float(loss),
            },
            "roofline": {
                "bound": "hbm",
                "kernel": "fq_per_token_regs_kernel / fq_per_token_wg_kernel + fq_int4_sym_tiled_kernel / fq_per_group_kernel (the fake-quant launches of "
                          "the step; the matmuls: see own_gemm)",
                "achieved": round(achieved, 1),
                "peak": HBM_PEAK_GBPS,
                "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": measured_traffic(args.workload)[0],
                "traffic_unit": "bytes per launch, average over a step's fake-quant launches (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 "
                                f"from the rocprofv3 --pmc runs summarised in {measured_traffic(args.workload)[1]}); "
                                f"algorithmic {fq_bytes / max(1, sum(v['launches'] for v in fq.values())) / 1e6:.1f}e6",
                "fq_ms_per_step": round(fq_ms / args.steps, 2),
                "timing": f"HIP events on the launch stream around every {fq_timer.stride}th launch of each shape inside the "
                          "timed steps; achieved = sum(bytes) / sum(average duration x launches)",
                "per_kernel": {k: {kk: vv for kk, vv in v.items() if kk in ("launches", "avg_us", "gbps")} for k, v in fq.items()},
            },
        }
        result["own_gemm"] = own_gemm
        result["with_adamw"] = with_adamw
        result["peak_memory_gib_timed_steps"] = round(peak_timed / 2**30, 3)
        del model
        torch.cuda.empty_cache()
        if args.cpu_tokens > 0:
            result["cpu_baseline"] = cpu_baseline_qat(shape_name, qat_group, SHAPES[shape_name].n_layers, batch * seq)
        print(json.dumps(result))
        return 0

    launches, launches_timed, gemm_ms, gemm_flops, per_shape = timer.summary()
    gemm_bytes = timer.total_bytes
    calls = sum(v["calls"] for v in per_shape.values())
    traffic_key = args.workload if timer.expanded_calls * 2 > calls else args.workload + "/fused"
    achieved = gemm_flops / gemm_ms / 1e9 if gemm_ms > 0 else 0.0
    result = {
        "metric": "QLoRA fwd+bwd tokens/sec (Llama-3.1-8B, 1 GPU)" if args.workload == "llama3_1_8b"
        else f"QLoRA fwd+bwd tokens/sec ({args.workload}, 1 GPU)",
        "value": round(batch * seq * args.steps / dt, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 2),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic (uniform random token ids, random-init N(0,0.02) weights quantised to NF4)",
        "config": {
            "workload": f"{args.workload}-shaped QLoRA decoder, all 7 projections NF4(64/256)+LoRA r={rank} alpha={alpha:g}, "
                        f"batch {batch} x seq {seq}, fwd+bwd incl. output projection and cross-entropy"
                        + (", activation checkpointing" if ac else "")
                        + f"; attention = torch SDPA, backend '{args.sdpa}'",
            "global_batch": batch,
            "seq_len": seq,
            "loss": float(loss),
        },
        "roofline": {
            "bound": "mfma",
            "kernel": ("nf4_gemm_dense_kernel with the nf4_expand_tiled_kernel launches that precede it in the same call (NF4 weight "
                       "expanded once per call into scratch memory, then a bf16 MFMA GEMM with the LoRA adapter in its epilogue"
                       + ("; the gate / up launch also forms silu(gate) * up there, counted as zero FLOPs" if harness.GATED_EPILOGUE
                          and harness.GROUP_SHARED_INPUT else "")
                       + (", and the down projection's grad-input launch the backward of that product" if harness.GATED_EPILOGUE
                          and harness.GROUP_SHARED_INPUT and harness.SWIGLU_BWD_EPILOGUE and not qat else "")
                       + "; forward and grad-input calls)"
                       if timer.expanded_calls * 2 > calls else
                       "nf4_gemm_rs_kernel (fused NF4-dequant + LoRA bf16 MFMA GEMM, forward and grad-input launches)"),
            "achieved": round(achieved, 1),
            "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
            "traffic": measured_traffic(traffic_key)[0],
            "traffic_unit": ("bytes per GEMM launch, average over a step's launches, expansion launches included with their GEMM "
                             "(FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 from the "
                             f"rocprofv3 --pmc runs summarised in {measured_traffic(traffic_key)[1]}); algorithmic "
                             f"{gemm_bytes / max(1, launches) / 1e6:.1f}e6") if measured_traffic(traffic_key)[1] else None,
            "launches": launches,
            "calls_with_expanded_weight": timer.expanded_calls,
            "launches_timed": launches_timed,
            "timing": f"HIP events on the launch stream around every {timer.stride}th call of each shape inside the timed steps "
                      "(an event pair idles the GPU for about 6 us); achieved = sum(flops) / sum(average duration x calls)",
            "gemm_ms_per_step": round(gemm_ms / args.steps, 2),
            "per_shape": per_shape,
        },
    }
    result["with_adamw"] = with_adamw
    result["peak_memory_gib_timed_steps"] = round(peak_timed / 2**30, 3)
    if ops.resident_tiles_enabled():
        result["resident_tiles"] = {
            "budget_gib": args.resident_tiles_gib, "held_gib": round(ops.resident_tiles_bytes() / 2**30, 3),
            "note": "expanded NF4 weights kept across steps (opt-in): the timed steps launch no expansion for the layers held"}
    del model
    torch.cuda.empty_cache()
    if not args.no_memory_leg:
        def one_step(m):
            train_step(m, tokens, labels)
            m.zero_grad(set_to_none=True)

        result["memory"] = memory_leg(
            lambda: build_qlora_decoder(shape_name, rank, alpha, device=dev, seed=0, activation_checkpointing=ac), one_step, dev)
    if not args.no_config1:
        result["config1_single_layer"] = config1_leg(dev)
    result["hbm_bound_kernels"] = secondary_kernels(dev)
    if args.cpu_tokens > 0:
        result["cpu_baseline"] = cpu_baseline(shape_name, rank, alpha, args.cpu_tokens, SHAPES[shape_name].n_layers, batch * seq)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
