"""Pins the NF4 oracle (oracle/nf4_oracle.py, oracle/nf4_ref.c) without the reference's third-party arithmetic:
published constants, closed forms, brute force, invariants, and agreement of two independent restatements."""
from fractions import Fraction

import pytest
import torch

from oracle import nf4_oracle
from tests.helpers import bits_equal, c_nf4_dequantize, c_nf4_quantize, parts_equal, seeded_weight

DTYPES = [torch.bfloat16, torch.float32]


def test_table_matches_the_papers_construction():
    # QLoRA (Dettmers et al. 2023), appendix E / bitsandbytes create_normal_map: 8 positive and 7 negative
    # quantiles of N(0,1) at evenly spaced probabilities from `offset` to 0.5, plus an exact zero, normalised.
    from scipy.stats import norm

    offset = 0.9677083
    pos = norm.ppf(torch.linspace(offset, 0.5, 9)[:-1].double().numpy()).tolist()
    neg = (-norm.ppf(torch.linspace(offset, 0.5, 8)[:-1].double().numpy())).tolist()
    vals = sorted(pos + [0.0] + neg)
    vals = [v / max(vals) for v in vals]
    assert len(vals) == 16
    for got, want in zip(nf4_oracle.NF4_TABLE, vals):
        assert abs(got - want) < 2e-6
    t = nf4_oracle.NF4_TABLE
    assert t[0] == -1.0 and t[7] == 0.0 and t[15] == 1.0
    assert all(a < b for a, b in zip(t, t[1:]))
    assert all(torch.tensor(v, dtype=torch.float32).item() == v for v in t)  # exactly representable in fp32


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_of_scaled_code_points_quantises_to_identity(dtype):
    # closed form: a block equal to absmax * table must give codes 0..15 (four times per 64-block)
    table = torch.tensor(nf4_oracle.NF4_TABLE, dtype=dtype)
    for absmax in (1.0, 0.5, 0.03125):
        w = (table * absmax).repeat(4 * 256)  # 256 identical blocks of 64 -> one scaler block
        p = nf4_oracle.nf4_quantize(w.contiguous(), 64, 256)
        codes = torch.stack([p.quantized_data >> 4, p.quantized_data & 0xF], dim=1).flatten()
        assert torch.equal(codes.view(-1, 16), torch.arange(16, dtype=torch.uint8).expand(4 * 256, 16))
        # identical absmaxes: centred scalers are 0, factor = 256/0 = inf, 0*inf = NaN -> scaler byte 0,
        # and 0/inf + mean reproduces the absmax exactly
        assert torch.all(p.quantized_scalers == 0)
        assert bits_equal(nf4_oracle.nf4_dequantize(p), w)


@pytest.mark.parametrize("dtype", DTYPES)
def test_plus_minus_c_block(dtype):
    w = torch.full((64 * 256,), 0.25, dtype=dtype)
    w[1::2] = -0.25
    p = nf4_oracle.nf4_quantize(w, 64, 256)
    assert torch.all(p.quantized_data == 0xF0)  # even element (+c) -> code 15 in the HIGH nibble, odd (-c) -> code 0


def test_nibble_order_by_single_element_perturbation():
    w = torch.zeros(64 * 256, dtype=torch.float32)
    w[0] = 1.0  # keeps block 0's absmax at 1 so other elements scale to themselves
    base = nf4_oracle.nf4_quantize(w, 64, 256).quantized_data.clone()
    for e, expect_shift in ((2, 4), (3, 0), (10, 4), (11, 0)):
        w2 = w.clone()
        w2[e] = -1.0  # code 0 instead of code 7
        q = nf4_oracle.nf4_quantize(w2, 64, 256).quantized_data
        changed = (q != base).nonzero().flatten().tolist()
        assert changed == [e // 2]
        assert ((int(q[e // 2]) >> expect_shift) & 0xF) == 0
        assert ((int(base[e // 2]) >> expect_shift) & 0xF) == 7


def test_every_bf16_pattern_brute_force(c_oracle):
    # all 65536 bf16 bit patterns as the "scaled" value: the torch oracle's rule (rounded distances, first
    # minimum) evaluated by an explicit python loop over the 16 codes must agree with both restatements
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    table = torch.tensor(nf4_oracle.NF4_TABLE, dtype=torch.bfloat16)
    best = torch.full((65536,), float("inf"))
    arg = torch.zeros(65536, dtype=torch.long)
    nan_rows = pats.isnan()
    for j in range(16):
        d = (pats - table[j]).abs().float()  # subtraction rounds to bf16 before abs
        better = d < best
        arg[better] = j
        best[better] = d[better]
    arg[nan_rows] = 0
    vec = (pats[:, None] - table[None, :]).abs().argmin(dim=-1)
    assert torch.equal(vec, arg)
    # C restatement: quantise blocks whose first element is 1.0 (absmax 1) and whose second is the pattern
    finite = pats[~nan_rows & (pats.abs() <= 1)]
    w = torch.zeros(finite.numel(), 64, dtype=torch.bfloat16)
    w[:, 0] = 1.0
    w[:, 1] = finite
    pad = (-w.shape[0]) % 256
    w = torch.cat([w, torch.ones(pad, 64, dtype=torch.bfloat16)])
    pc = c_nf4_quantize(c_oracle, w.flatten(), 64, 256)
    got = (pc.quantized_data.view(-1, 32)[: finite.numel(), 0] & 0xF).long()
    want = (finite[:, None] - table[None, :]).abs().argmin(dim=-1)
    assert torch.equal(got, want)
    # monotone: a larger scaled value never gets a smaller code
    order = finite.float().argsort(stable=True)
    assert torch.all(want[order][1:] >= want[order][:-1])
    # and exact code points map to themselves
    assert torch.equal((table[:, None] - table[None, :]).abs().argmin(dim=-1), torch.arange(16))


def test_double_quant_closed_form_with_clamp():
    # block absmaxes a_i = 1 + i/256, i = 0..255 (exact in fp32): mean = 1 + 255/512,
    # factor = 256 / (2 * 127.5/256) = 65536/255, byte_i = round((i - 127.5) * 256/255) clamped to [-128, 127]
    w = torch.zeros(256, 64, dtype=torch.float32)
    for i in range(256):
        w[i, i % 64] = 1.0 + i / 256.0
    p = nf4_oracle.nf4_quantize(w.flatten(), 64, 256)
    assert p.scaler_mean.item() == 1.0 + 255.0 / 512.0
    assert abs(p.quantization_factor.item() - 65536.0 / 255.0) < 1e-4
    want = []
    for i in range(256):
        v = Fraction(2 * i - 255, 2) * Fraction(256, 255)
        r = round(v)  # python rounds half to even, and no value here is a tie
        want.append(max(-128, min(127, r)))
    assert want[0] == -128 and want[255] == 127 and round(Fraction(255, 2) * Fraction(256, 255)) == 128  # clamp is exercised
    assert p.quantized_scalers.tolist() == want
    assert int(p.quantized_scalers.abs().max()) <= 128


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape,bs,sbs", [((512, 512), 64, 256), ((512, 512), 8, 4), ((512, 512), 16, 256), ((64, 2048), 128, 32)])
def test_two_restatements_agree(c_oracle, dtype, shape, bs, sbs):
    w = seeded_weight(shape, dtype, seed=3)
    w[5, 7] = 0.3  # an outlier block
    pt = nf4_oracle.nf4_quantize(w, bs, sbs)
    pc = c_nf4_quantize(c_oracle, w, bs, sbs)
    assert parts_equal(pt, pc)
    assert bits_equal(nf4_oracle.nf4_dequantize(pt), c_nf4_dequantize(c_oracle, pc))


@pytest.mark.parametrize("dtype", DTYPES)
def test_dequantise_exhaustive_lut(c_oracle, dtype):
    # every (code, int8 scaler) pair for several factor/mean choices: 16 x 256 values each
    for factor, mean in ((257.0, 0.0625), (1000.0, 0.02), (3.0, -0.5)):
        codes = torch.arange(16, dtype=torch.uint8)
        packed = ((codes[:, None] << 4) | codes[None, :]).flatten()  # all 256 byte values = 512 elements
        qs = torch.arange(-128, 128, dtype=torch.int8)
        # 256 blocks of 512 elements: block b uses scaler byte qs[b] and contains every byte value once
        p = nf4_oracle.NF4Parts(512, 256, 256, qs, torch.tensor([factor], dtype=dtype), torch.tensor(mean, dtype=dtype),
                                packed.repeat(256), torch.tensor(nf4_oracle.NF4_TABLE, dtype=dtype), torch.Size([256, 512]), dtype)
        dt = nf4_oracle.nf4_dequantize(p)
        dc = c_nf4_dequantize(c_oracle, p)
        assert bits_equal(dt, dc)
        # spot-check the formula itself in python floats for fp32 (each op is then a single IEEE operation)
        if dtype == torch.float32:
            f32 = lambda v: torch.tensor(v, dtype=torch.float64).to(torch.float32).item()
            fac, mn = f32(factor), f32(mean)
            for b in (0, 77, 255):
                scaler = f32(f32(int(qs[b]) / fac) + mn)
                for e in (0, 1, 100, 511):
                    byte = int(packed[e // 2])
                    code = (byte >> 4) if e % 2 == 0 else (byte & 0xF)
                    assert dt[b, e].item() == f32(nf4_oracle.NF4_TABLE[code] * scaler)


@pytest.mark.parametrize("dtype", DTYPES)
def test_requantise_is_idempotent(dtype):
    # the reference's own invariant (tests/torchtune/modules/peft/test_lora.py:229-237)
    w = seeded_weight((512, 512), dtype, seed=5)
    p1 = nf4_oracle.nf4_quantize(w, 64, 256)
    p2 = nf4_oracle.nf4_quantize(nf4_oracle.nf4_dequantize(p1), 64, 256)
    assert torch.equal(p1.quantized_data, p2.quantized_data)


@pytest.mark.parametrize("dtype", DTYPES)
def test_reconstruction_error_bound(dtype):
    w = seeded_weight((512, 512), dtype, seed=6)
    p = nf4_oracle.nf4_quantize(w, 64, 256)
    d = nf4_oracle.nf4_dequantize(p).float()
    absmax = w.float().view(-1, 64).abs().max(dim=1).values
    scaler = nf4_oracle.nf4_dequantize_scalers(p).float()
    half_gap = 0.5 * max(b - a for a, b in zip(nf4_oracle.NF4_TABLE, nf4_oracle.NF4_TABLE[1:]))  # 0.1519
    bound = absmax * half_gap * 1.02 + (scaler - absmax).abs() + 1e-3 * absmax
    err = (d - w.float()).abs().view(-1, 64)
    assert torch.all(err <= bound[:, None])
    # the element that defines a block's absmax always lands on code 0 or 15
    codes = torch.stack([p.quantized_data >> 4, p.quantized_data & 0xF], dim=1).flatten().view(-1, 64)
    idx = w.float().view(-1, 64).abs().argmax(dim=1)
    at = codes[torch.arange(codes.shape[0]), idx]
    assert torch.all((at == 0) | (at == 15))


def test_order_independent_mean_against_torch_mean_on_seeded_inputs():
    # bf16: the exactly rounded mean equals what torch's fp32-accumulated mean rounds to on these inputs.
    # fp32: torch's own result depends on its summation order; the exactly rounded mean is within one ulp of it.
    for seed in range(4):
        w = seeded_weight((1024, 1024), torch.bfloat16, seed=seed)
        absmax = w.view(-1, 64).abs().max(dim=1).values
        assert nf4_oracle.order_independent_mean(absmax).item() == absmax.mean().item()
        w = seeded_weight((1024, 1024), torch.float32, seed=seed)
        absmax = w.view(-1, 64).abs().max(dim=1).values
        exact = nf4_oracle.order_independent_mean(absmax)
        assert exact.item() == (absmax.double().sum() / absmax.numel()).float().item()
        assert abs(exact.view(torch.int32).item() - absmax.mean().view(torch.int32).item()) <= 1


def test_all_zero_tensor_does_not_raise():
    # tests/torchtune/modules/peft/test_lora.py:218-228 builds to_nf4(zeros)
    for dtype in DTYPES:
        p = nf4_oracle.nf4_quantize(torch.zeros(512, 512, dtype=dtype), 64, 256)
        assert torch.all(p.quantized_data == 0) and torch.all(p.quantized_scalers == 0)


def test_linear_nf4_is_linear_on_dequantised_weight():
    w = seeded_weight((128, 256), torch.float32, seed=7)
    p = nf4_oracle.nf4_quantize(w, 64, 32)
    x = torch.randn(5, 256, generator=torch.Generator().manual_seed(1))
    g = torch.randn(5, 128, generator=torch.Generator().manual_seed(2))
    d = nf4_oracle.nf4_dequantize(p)
    torch.testing.assert_close(nf4_oracle.linear_nf4_forward(x, p), x @ d.T)
    torch.testing.assert_close(nf4_oracle.linear_nf4_backward(g, p), g @ d)


def test_shared_reciprocal_division_is_exact_for_bf16(c_oracle):
    """The bf16 quantise kernel divides 1/absmax once per block and forms each quotient with two fused
    multiply-adds.  Enumerate EVERY pair of bf16 operands 0 <= x <= a with a >= 2^-119 (the kernel's guard): the
    bf16-rounded quotient must equal that of the correctly rounded division.  Below the guard the shortcut does
    fail, which is why the guard exists."""
    from concurrent.futures import ThreadPoolExecutor

    lo, hi = 0x0400, 0x7F80  # 2^-119 .. the largest finite bf16
    edges = [lo + (hi - lo) * i // 32 for i in range(33)]
    with ThreadPoolExecutor(max_workers=8) as pool:  # ctypes releases the GIL
        bad = list(pool.map(lambda i: c_oracle.ref_check_shared_reciprocal_division(edges[i], edges[i + 1]), range(32)))
    assert sum(bad) == 0
    assert c_oracle.ref_check_shared_reciprocal_division(0x0001, 0x0100) > 0


def test_shared_reciprocal_division_is_exact_for_uint4_group_offsets(c_oracle):
    """The weight-only uint4 fake-quant kernel uses the same shortcut for (w - lowest) / scale: divisors are bf16
    scales >= 1e-6, quotients of interest reach 15.5 (larger ones clamp to 15).  Enumerate every bf16 divisor from
    2^-20 up and every bf16 numerator up to 17 times the divisor."""
    import ctypes
    from concurrent.futures import ThreadPoolExecutor

    fn = c_oracle.ref_check_shared_reciprocal_division_upto
    fn.restype = ctypes.c_int64
    fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float]
    lo, hi = 0x3580, 0x7F80  # 2^-20 (below bf16(1e-6) = 0x3586) .. the largest finite bf16
    edges = [lo + (hi - lo) * i // 32 for i in range(33)]
    with ThreadPoolExecutor(max_workers=8) as pool:
        bad = list(pool.map(lambda i: fn(edges[i], edges[i + 1], 17.0), range(32)))
    assert sum(bad) == 0


def test_code_table_premises_and_monotone_codes(c_oracle):
    """Every bf16 scaled value below 2^-5 is the zero code and NaN is code 0 (what lets the kernel's table span only
    2^-5..1); inside the table the code never decreases with the value."""
    import ctypes

    buf = (ctypes.c_uint8 * (2 * 641))()
    assert c_oracle.ref_check_code_table(ctypes.cast(buf, ctypes.c_void_p)) == 0
    pos, neg = list(buf[:641]), list(buf[641:])
    assert pos == sorted(pos) and neg == sorted(neg, reverse=True)
    assert pos[0] == 7 and neg[0] == 7 and pos[-1] == 15 and neg[-1] == 0
    # the same table from the eager-PyTorch oracle
    bits = torch.arange(0x3D00, 0x3F81, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    for sign, want in ((1.0, pos), (-1.0, neg)):
        blocks = torch.zeros(641, 64, dtype=torch.bfloat16)
        blocks[:, 0] = 1.0
        blocks[:, 1] = bits * sign
        p = nf4_oracle.nf4_quantize(blocks, 64, 1)
        assert (p.quantized_data.view(641, 32)[:, 0] & 0xF).tolist() == want


def test_exact_scaler_mean_against_eager_mean_on_every_benchmark_weight_shape(record_property):
    """The oracle (and the kernels) define ``scaler_mean`` as the exact mean of the block absmaxes, rounded once; the
    reference computes ``absmax.mean()``, whose fp32 summation order belongs to the library version.  On every projection
    shape of the 1B / 8B / 70B configurations with the benchmark's N(0, 0.02) weights (seed 0) the two are compared in
    bf16 and the number of mismatches is reported; a mismatch would be one bf16 ulp of the mean and would move every scaler
    byte of that tensor."""
    shapes = [(2048, 2048), (512, 2048), (8192, 2048), (2048, 8192), (4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336),
              (8192, 8192), (1024, 8192), (28672, 8192), (8192, 28672)]
    mismatches = []
    for N, K in shapes:
        g = torch.Generator().manual_seed(0)
        w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
        absmax = w.view(-1, 64).abs().max(dim=1).values
        del w
        exact, eager = nf4_oracle.order_independent_mean(absmax), absmax.mean()
        if exact.view(torch.int16).item() != eager.view(torch.int16).item():
            mismatches.append((N, K, float(exact), float(eager)))
    # the same question where it is hardest: weight scales swept so that the mean crosses bf16 rounding boundaries
    near = []
    for i in range(48):
        g = torch.Generator().manual_seed(100 + i)
        w = (torch.randn(1024, 4096, generator=g) * (0.015 + 0.0005 * i)).to(torch.bfloat16)
        absmax = w.view(-1, 64).abs().max(dim=1).values
        exact, eager = nf4_oracle.order_independent_mean(absmax), absmax.mean()
        if exact.view(torch.int16).item() != eager.view(torch.int16).item():
            near.append((i, float(exact), float(eager)))
            assert abs(int(exact.view(torch.int16)) - int(eager.view(torch.int16))) == 1  # never more than one ulp
    record_property("scaler_mean_mismatches_benchmark_shapes", len(mismatches))
    record_property("scaler_mean_mismatches_scale_sweep", len(near))
    print(f"scaler_mean: {len(mismatches)} of {len(shapes)} benchmark shapes differ from eager mean(); "
          f"{len(near)} of 48 tensors of the scale sweep differ (by one bf16 ulp)")
    assert mismatches == [], mismatches
