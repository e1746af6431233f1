"""Pins the quantize / fp8-matmul oracle (CPU only).

Checks, in order of independence from the oracle's own formula:
  * golden vectors written by the reference's ``_to_fp8`` (tests/golden/quantize_reference.json)
  * the C encoder vs torch's library cast over every bf16 bit pattern
  * OCP e4m3 known answers (ties to even, subnormals, saturation)
  * invariants (sign symmetry, max code, idempotence)
  * matmul: ``torch._scaled_mm`` on CPU, exact power-of-two cases, brute force
"""
import ctypes
import json
import os

import numpy as np
import pytest
import torch

from oracle import fp8_ref
from oracle.build_oracle import load as load_c_oracle

GOLD = os.path.join(os.path.dirname(__file__), "golden", "quantize_reference.json")


def bits_to_tensor(d):
    if d["dtype"] == "bf16":
        return torch.tensor(d["bits"], dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    a = np.array(d["bits"], dtype=np.uint32).view(np.float32)
    return torch.from_numpy(a.copy())


@pytest.fixture(scope="module")
def golden():
    with open(GOLD) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def clib():
    return load_c_oracle()


def c_quantize(clib, x):
    n = x.numel()
    out = np.zeros(n, dtype=np.uint8)
    scale = ctypes.c_float()
    inv = ctypes.c_float()
    if x.dtype == torch.bfloat16:
        src = x.contiguous().view(torch.int16).numpy()
        clib.oracle_quantize_bf16(src.ctypes.data, n, out.ctypes.data, ctypes.addressof(scale), ctypes.addressof(inv))
    else:
        src = x.contiguous().numpy()
        clib.oracle_quantize_f32(src.ctypes.data, n, out.ctypes.data, ctypes.addressof(scale), ctypes.addressof(inv))
    return out, scale.value, inv.value


def f32_bits(v):
    return int(np.array([v], dtype=np.float32).view(np.uint32)[0])


def test_golden_vectors_torch_oracle(golden):
    for name, case in golden.items():
        x = bits_to_tensor(case["input"])
        payload, inv, _ = fp8_ref.to_fp8(x)
        assert payload.view(torch.uint8).tolist() == case["payload"], name
        assert f32_bits(inv.item()) == case["inv_scale_bits"], name


def test_golden_vectors_c_oracle(golden, clib):
    for name, case in golden.items():
        x = bits_to_tensor(case["input"])
        payload, _, inv = c_quantize(clib, x)
        assert payload.tolist() == case["payload"], name
        assert f32_bits(inv) == case["inv_scale_bits"], name


@pytest.mark.parametrize("scale", [1.0, 0.37, 448.0 / 5.1875, 3.0e-3, 1.7e4, 4.48e14])
def test_c_encoder_exhaustive_vs_library_cast(clib, scale):
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16)
    finite = torch.isfinite(x.float())
    x = x[finite]
    want = (x.float() * scale).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.zeros(x.numel(), dtype=np.uint8)
    src = x.contiguous().view(torch.int16).numpy()
    clib.oracle_encode_bf16_with_scale(src.ctypes.data, x.numel(), ctypes.c_float(scale), got.ctypes.data)
    # -0.0 * scale keeps its sign in both; compare all bytes
    assert np.array_equal(got, want)


def test_e4m3_known_answers(clib):
    # value -> byte, from the OCP e4m3fn definition
    table = {
        0.0: 0x00, 2.0 ** -9: 0x01, 2.0 ** -10: 0x00, 1.5 * 2.0 ** -10: 0x01, 3 * 2.0 ** -10: 0x02,
        2.0 ** -6: 0x08, 1.0: 0x38, 1.0625: 0x38, 1.1875: 0x3A, 17.0: 0x58, 19.0: 0x5A, 21.0: 0x5A, 23.0: 0x5C,
        448.0: 0x7E, 440.0: 0x7E, 432.0: 0x7E, 400.0: 0x7C, 416.0: 0x7D, -448.0: 0xFE, -1.0: 0xB8, 0.875 * 2.0 ** -6: 0x07,
        0.9375 * 2.0 ** -6: 0x08,
    }
    for v, b in table.items():
        assert clib.oracle_e4m3_encode(v) == b, (v, hex(b))
        t = torch.tensor([v]).to(torch.float8_e4m3fn).view(torch.uint8).item()
        assert t == b, (v, hex(b), hex(t))
    for b in range(256):
        if b & 0x7F == 0x7F:
            continue
        v = clib.oracle_e4m3_decode(b)
        assert clib.oracle_e4m3_encode(v) == b
        assert torch.tensor([b], dtype=torch.uint8).view(torch.float8_e4m3fn).float().item() == v


def test_scale_closed_forms():
    # amax == 448 -> scale exactly 1; all-zero -> floor 1e-12 -> 4.48e14; power-of-two amax -> exact
    p, inv, s = fp8_ref.to_fp8(torch.tensor([448.0, 1.0]))
    assert s.item() == 1.0 and inv.item() == 1.0
    p, inv, s = fp8_ref.to_fp8(torch.zeros(8))
    assert s.item() == np.float32(448.0 / 1e-12) and p.view(torch.uint8).sum().item() == 0
    p, inv, s = fp8_ref.to_fp8(torch.tensor([0.5, -0.25]))
    assert s.item() == 896.0 and inv.item() == np.float32(1.0) / np.float32(896.0)
    assert p.view(torch.uint8).tolist() == [0x7E, 0xF6]      # 448, -224


def test_quantize_invariants():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(5000, generator=g).bfloat16()
    p, inv, s = fp8_ref.to_fp8(x)
    pn, invn, _ = fp8_ref.to_fp8(-x)
    b, bn = p.view(torch.uint8), pn.view(torch.uint8)
    assert torch.equal(b ^ 0x80, bn) and inv == invn
    assert (b & 0x7F).max().item() == 0x7E
    # re-quantizing the dequantized payload at the same scale is the identity
    deq = p.float()
    again = deq.clamp(-448, 448).to(torch.float8_e4m3fn)
    assert torch.equal(again.view(torch.uint8), b)


def test_matmul_matches_library_scaled_mm():
    g = torch.Generator().manual_seed(3)
    a = torch.randn(24, 64, generator=g).bfloat16()
    w = ((torch.rand(48, 64, generator=g) * 2 - 1) * 0.2).bfloat16()
    a8, ia, _ = fp8_ref.to_fp8(a)
    w8, iw, _ = fp8_ref.to_fp8(w)
    lib = fp8_ref.scaled_mm_library(a8, w8, ia, iw)
    emu = fp8_ref.scaled_mm_emulated(a8, w8, ia, iw)
    assert torch.equal(lib, emu)


def test_matmul_power_of_two_exact_and_bruteforce():
    g = torch.Generator().manual_seed(5)
    # power-of-two entries: every product and partial sum is exact in fp32
    ea = torch.randint(-3, 4, (8, 16), generator=g).float()
    ew = torch.randint(-3, 4, (12, 16), generator=g).float()
    sa = torch.randint(0, 2, (8, 16), generator=g).float() * 2 - 1
    a = (sa * 2.0 ** ea)
    w = 2.0 ** ew
    a[0, 0] = 8.0   # amax 8 -> scale 56, not a power of two but 56*2^k is e4m3-exact
    w[0, 0] = 8.0
    a8, ia, _ = fp8_ref.to_fp8(a.bfloat16())
    w8, iw, _ = fp8_ref.to_fp8(w.bfloat16())
    assert torch.equal(a8.float() * ia, a) and torch.equal(w8.float() * iw, w)
    out = fp8_ref.scaled_mm_emulated(a8, w8, ia, iw, out_dtype=torch.float32)
    # brute force in python floats (double): tiny K
    af, wf = a8.float().double(), w8.float().double()
    for i in range(8):
        for j in range(12):
            acc = sum(float(af[i, k]) * float(wf[j, k]) for k in range(16))
            want = np.float32(np.float32(np.float32(acc) * np.float32(ia.item())) * np.float32(iw.item()))
            assert out[i, j].item() == want


def test_float8_linear_shapes_and_filter():
    x = torch.randn(2, 3, 128)
    w = torch.randn(256, 128) * 0.05
    y = fp8_ref.float8_linear(x, w)
    assert y.shape == (2, 3, 256) and y.dtype == torch.bfloat16
    exact = x.bfloat16().float() @ w.t()
    rel = (y.float() - exact).norm() / exact.norm()
    assert rel < 0.06      # e4m3 has 3 mantissa bits: ~3-4% rms error is expected
    assert fp8_ref.fp8_module_filter(256, 1024) and not fp8_ref.fp8_module_filter(12, 2)
    assert not fp8_ref.fp8_module_filter(24, 1) and not fp8_ref.fp8_module_filter(130, 256)


# ---------------------------------------------------------------- gradient format and the backward GEMMs (nanochat/fp8.py:156-192)
def test_e5m2_cast_pinned_by_integer_encoder_exhaustively():
    """Every bf16 value the clamp lets through, and random fp32 values: torch's e5m2 cast (the library routine the reference
    calls at fp8.py:103) against an integer restatement of OCP e5m2 round-to-nearest-even."""
    allb = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    x = allb[allb.abs() <= fp8_ref.E5M2_MAX]
    assert torch.equal(x.to(torch.float8_e5m2).view(torch.uint8), fp8_ref.e5m2_encode_bits(x))
    g = torch.Generator().manual_seed(0)
    y = (torch.randn(500_000, generator=g) * torch.exp(torch.randn(500_000, generator=g) * 6)).clamp(-fp8_ref.E5M2_MAX, fp8_ref.E5M2_MAX)
    assert torch.equal(y.to(torch.float8_e5m2).view(torch.uint8), fp8_ref.e5m2_encode_bits(y))
    # ties to even, the subnormal boundary and the saturation point
    probe = torch.tensor([1.125, 1.375, 2.0 ** -16, 2.0 ** -17, 1.5 * 2.0 ** -16, 57344.0, 60000.0])
    assert probe.clamp(max=fp8_ref.E5M2_MAX).to(torch.float8_e5m2).float().tolist() == [1.0, 1.5, 2.0 ** -16, 0.0, 2.0 ** -15, 57344.0, 57344.0]


def test_to_fp8_e5m2_closed_form_and_invariants():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(4096, generator=g) * 3).bfloat16()
    p, inv, scale = fp8_ref.to_fp8(x, torch.float8_e5m2)
    amax = x.float().abs().max().double()
    assert scale.item() == np.float32(57344.0 / amax.item()) and inv.item() == np.float32(1.0) / np.float32(scale.item())
    assert (p.view(torch.uint8) & 0x7F).max().item() == 0x7B                 # the largest entry lands on 57344
    p2, _, _ = fp8_ref.to_fp8(-x, torch.float8_e5m2)
    assert torch.equal(p.view(torch.uint8) ^ 0x80, p2.view(torch.uint8))
    z, _, sz = fp8_ref.to_fp8(torch.zeros(64).bfloat16(), torch.float8_e5m2)
    assert z.view(torch.uint8).sum().item() == 0 and sz.item() == np.float32(57344.0 / 1e-12)


def test_backward_restatement_against_library_and_exact_case():
    g = torch.Generator().manual_seed(2)
    B, K, N = 64, 128, 96
    x = torch.randn(B, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    go = (torch.randn(B, N, generator=g) * 1e-3).bfloat16()
    a8, ia, _ = fp8_ref.to_fp8(x)
    w8, iw, _ = fp8_ref.to_fp8(w)
    gi, gw, go8, igo = fp8_ref.float8_matmul_backward(go, a8, ia, w8, iw)
    gi_lib, gw_lib = fp8_ref.float8_matmul_backward_library(go, a8, ia, w8, iw)      # the reference's own three calls, on CPU
    for got, want in ((gi, gi_lib), (gw, gw_lib)):
        assert got.shape == want.shape and got.dtype == torch.bfloat16
        rel = ((got.float() - want.float()).norm() / want.float().norm()).item()
        assert rel < 2e-3, rel                                                       # same fp8 inputs: summation order + one bf16 rounding
    # against the unquantized gradients, fp8 noise only
    gi_exact = go.float() @ w.float()
    gw_exact = go.float().t() @ x.float()
    assert ((gi.float() - gi_exact).norm() / gi_exact.norm()).item() < 0.1
    assert ((gw.float() - gw_exact).norm() / gw_exact.norm()).item() < 0.1
    # signed powers of two with power-of-two scales: every product and partial sum is exact, so the result is the exact gradient
    sgn = lambda *s: torch.randint(0, 2, s, generator=g).float() * 2 - 1
    xe = sgn(B, K) * 2.0 ** torch.randint(-2, 3, (B, K), generator=g).float()
    we = sgn(N, K) * 2.0 ** torch.randint(-2, 3, (N, K), generator=g).float()
    ge = sgn(B, N) * 2.0 ** torch.randint(-2, 3, (B, N), generator=g).float()
    xe[0, 0], we[0, 0], ge[0, 0] = 7.0, 7.0, 7.0                                     # amax 7: 448/7 = 64 and 57344/7 = 8192
    a8, ia, _ = fp8_ref.to_fp8(xe.bfloat16())
    w8, iw, _ = fp8_ref.to_fp8(we.bfloat16())
    gi, gw, _, _ = fp8_ref.float8_matmul_backward(ge.bfloat16(), a8, ia, w8, iw)
    assert torch.equal(gi, (ge @ we).bfloat16()) and torch.equal(gw, (ge.t() @ xe).bfloat16())

