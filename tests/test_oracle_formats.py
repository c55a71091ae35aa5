"""Pins the oracle's number formats against library routines that are independent of it (numpy float16,
torch bfloat16 / float8_e4m3fn) and against closed forms.  CPU only."""
import json
from pathlib import Path

import numpy as np
import pytest
import torch

from tests.gpu_util import bf16_safe as _bf16_safe

GOLD = Path(__file__).parent / "golden"


def test_f16_decode_all_codes(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib.orc_f16_to_f32(int(b)) for b in bits], np.float32)
    both_nan = np.isnan(ref) & np.isnan(got)
    assert np.array_equal(ref.view(np.uint32)[~both_nan], got.view(np.uint32)[~both_nan])


def test_f16_encode_rne(oracle):
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(20000) * 10.0 ** rng.uniform(-8, 5, 20000),
        # exact ties between neighbouring halfs and values one ulp(f64) either side
        (np.arange(1, 2047, dtype=np.float64) + 0.5) * 2.0 ** -14, (np.arange(1, 2047) + 0.5) * 2.0 ** -24 * 1024,
        np.nextafter((np.arange(1, 2047, dtype=np.float64) + 0.5) * 2.0 ** -3, 0), np.nextafter((np.arange(1, 2047, dtype=np.float64) + 0.5) * 2.0 ** -3, 9e9),
        [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 5.96e-8, 6.1e-5],
    ])
    ref = x.astype(np.float16).view(np.uint16)           # numpy converts binary64 -> binary16 with one rounding
    got = np.array([oracle.lib.orc_f64_to_f16(float(v)) for v in x], np.uint16)
    assert np.array_equal(ref, got)


def test_bf16_rne_vs_torch(oracle):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(50000) * 10.0 ** rng.uniform(-6, 6, 50000)).astype(np.float32)
    ties = (np.arange(0x3f80, 0x4080, dtype=np.uint32) << 16 | 0x8000).view(np.float32)   # exact ties
    x = np.concatenate([x, ties, np.nextafter(ties, 0), np.nextafter(ties, np.float32(9e9))]).astype(np.float32)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([oracle.lib.orc_f32_to_bf16(float(v)) for v in x], np.uint16)
    assert np.array_equal(ref, got)
    assert np.array_equal(oracle.bf16_bits(x), ref)      # the numpy helper used by the generators


def test_e4m3_decode_all_codes_vs_torch(oracle):
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float().numpy()
    got = np.array([oracle.lib.orc_e4m3_to_f32(int(c)) for c in range(256)], np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(nan, np.isnan(got)) and nan.sum() == 2
    assert np.array_equal(ref[~nan], got[~nan])
    assert got[0x7e] == 448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9      # OCP FP8 anchors


def test_e4m3_encode_rne_vs_torch(oracle):
    rng = np.random.default_rng(2)
    vals = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    vals = np.sort(vals[np.isfinite(vals)])
    mids = (vals[:-1].astype(np.float64) + vals[1:]) / 2                  # exact ties (representable in binary32)
    x = np.concatenate([vals, mids, np.nextafter(mids.astype(np.float32), -9e9), np.nextafter(mids.astype(np.float32), 9e9),
                        rng.uniform(-448, 448, 40000), rng.standard_normal(20000) * 10.0 ** rng.uniform(-5, 0, 20000)]).astype(np.float32)
    x = x[np.abs(x) <= 448.0]
    ref = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.array([oracle.lib.orc_f32_to_e4m3(float(v)) for v in x], np.uint8)
    # +0 and -0 both decode to zero; compare the codes exactly except the sign of zero
    z = (ref & 0x7f) == 0
    assert np.array_equal(ref[~z], got[~z]) and np.all((got[z] & 0x7f) == 0)
    # saturation: beyond the largest finite value the conversion gives +-448 (the clamp of the reference kernels)
    assert oracle.lib.orc_f32_to_e4m3(1e9) == 0x7e and oracle.lib.orc_f32_to_e4m3(-500.0) == 0xfe


def test_e8m0_and_e2m1(oracle):
    for b in range(1, 255):
        assert oracle.lib.orc_e8m0_to_f32(b) == 2.0 ** (b - 127)
    assert oracle.lib.orc_e8m0_to_f32(0) == 0.0            # reference ops.rs:22 / ds41.cu:23: the bits b << 23
    table = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]       # OCP MX E2M1 magnitudes
    for c in range(16):
        v = oracle.lib.orc_e2m1_to_f32(c)
        assert abs(v) == table[c & 7] and (np.signbit(v) == bool(c & 8))


def test_mxfp4_dequant_exhaustive(oracle):
    # every byte (two codes) x every usable scale byte, against the closed form table[nibble] * 2^(s - 127)
    table = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], np.float64)
    scales = np.arange(1, 253, dtype=np.uint8)                 # 6 * 2^(253-127) would overflow binary32
    w = np.tile(np.arange(256, dtype=np.uint8).reshape(16, 16), (len(scales), 1))        # [252*16, 16] -> K = 32
    s = np.repeat(scales, 16).reshape(-1, 1)
    got = oracle.mxfp4_dequant(w, s)
    lo, hi = w & 15, w >> 4
    ref = np.stack([table[lo], table[hi]], -1).reshape(w.shape[0], 32) * 2.0 ** (s.astype(np.float64) - 127)
    assert np.array_equal(got.astype(np.float64), ref)     # low nibble = even k


def test_fp8_block_dequant_closed_form(oracle):
    rng = np.random.default_rng(3)
    w = rng.integers(0, 256, (256, 384), dtype=np.uint8)
    w[(w & 0x7f) == 0x7f] = 0
    s = np.exp(rng.uniform(np.log(1e-3), np.log(1e-1), (2, 3))).astype(np.float32)
    got = oracle.fp8_block_dequant(w, s, 128)
    ref = torch.from_numpy(w).view(torch.float8_e4m3fn).float().numpy() * np.repeat(np.repeat(s, 128, 0), 128, 1)
    assert np.array_equal(got, ref.astype(np.float32))
    s8 = rng.integers(100, 130, (8, 12), dtype=np.uint8)
    got = oracle.fp8_e8m0_dequant(w, s8)
    ref = torch.from_numpy(w).view(torch.float8_e4m3fn).float().numpy() * np.repeat(np.repeat(2.0 ** (s8.astype(np.float32) - 127), 32, 0), 32, 1)
    assert np.array_equal(got, ref.astype(np.float32))


def _act_quant_torch(x):
    """act_quant with UE8M0 scales per 32 from library pieces only (torch float8 cast, frexp): the closed form
    scale = 2^ceil(log2(max(amax, 1e-4) / 448)), q = e4m3_rn(clamp(x / scale))."""
    xb = x.float().reshape(-1, 32)
    amax = xb.abs().amax(-1).clamp_min(1e-4)
    t = amax * torch.tensor(1.0 / 448.0)
    m, e = torch.frexp(t)                                   # t = m * 2^e, m in [0.5, 1)
    ce = torch.where(m == 0.5, e - 1, e)                    # ceil(log2 t)
    s = torch.ldexp(torch.ones_like(t), ce)
    q = (xb / s[:, None]).clamp(-448, 448).to(torch.float8_e4m3fn)
    return q.view(torch.uint8).reshape(x.shape).numpy(), (ce + 127).to(torch.uint8).reshape(*x.shape[:-1], -1).numpy(), \
        (q.float() * s[:, None]).reshape(x.shape).to(torch.bfloat16)


def test_act_quant_vs_library(oracle):
    g = torch.Generator().manual_seed(4)
    # blocks whose amax sweeps many binades (incl. below the 1e-4 floor and exact powers of two times 448)
    x = torch.randn(4096, 32, generator=g) * (10.0 ** torch.empty(4096, 1).uniform_(-6, 3, generator=g))
    x[:64] = 0.0
    x[64:128, 0] = 448.0 * 2.0 ** torch.arange(-32, 32).float()[:64]
    x = x.to(torch.bfloat16)
    q_ref, s_ref, d_ref = _act_quant_torch(x)
    bits = x.view(torch.int16).numpy().view(np.uint16)
    q, s = oracle.act_quant_fp8(bits)
    assert np.array_equal(s, s_ref)
    z = (q_ref & 0x7f) == 0
    assert np.array_equal(q[~z], q_ref[~z]) and np.all((q[z] & 0x7f) == 0)
    d = oracle.act_quant32(bits)
    assert np.array_equal(oracle.bf16_to_f32(d), d_ref.float().numpy())


def test_act_quant_scale_exhaustive_exponents(oracle):
    # aq_scale over every binade and mantissa pattern class: exact power of two vs not
    for e in range(-20, 12):
        for man in (1.0, 1.0 + 2.0 ** -23, 1.5, 2.0 - 2.0 ** -23):
            amax = np.float32(man * 2.0 ** e)
            t = np.float32(max(amax, np.float32(1e-4))) * np.float32(1.0 / 448.0)
            expect = int(np.ceil(np.log2(np.float64(t)))) + 127
            assert oracle.lib.orc_aq_scale(float(amax)) == expect, (e, man)


def test_requant_fp8_vs_library(oracle):
    # stored E4M3 rows with an E8M0 byte per 32 -> act_quant of their bf16 dequantisation (reference ds41_mx.cu:333-353), against the
    # library's types end to end (torch float8 decode, bf16 cast, the torch act_quant above) and two values worked by hand
    g = torch.Generator().manual_seed(9)
    wq = torch.randint(0, 256, (512, 64), generator=g, dtype=torch.uint8)
    wq[(wq & 0x7f) == 0x7f] = 0x3c
    ws = torch.randint(90, 150, (512, 2), generator=g, dtype=torch.uint8)
    x = (wq.view(torch.float8_e4m3fn).float().view(512, 2, 32) * torch.ldexp(torch.ones(512, 2, 1), ws.int().view(512, 2, 1) - 127)).view(512, 64).to(torch.bfloat16)
    q_ref, s_ref, _ = _act_quant_torch(x)
    q, s = oracle.requant_fp8(wq.numpy(), ws.numpy())
    assert np.array_equal(s, s_ref)
    z = (q_ref & 0x7f) == 0
    assert np.array_equal(q[~z], q_ref[~z]) and np.all((q[z] & 0x7f) == 0)
    # 1.0 (0x38) under scale 2^3: the block maximum 8 gives the scale 2^-5 (8 / 448 rounded up to a power of two) and the byte of 256 (0x78);
    # -1.5 (0xbc) beside it: -1.5 * 8 / 2^-5 = -384 (0xfc)
    one = np.zeros((1, 32), np.uint8); one[0, 0] = 0x38; one[0, 1] = 0xbc
    q1, s1 = oracle.requant_fp8(one, np.array([[130]], np.uint8))
    assert s1[0, 0] == 122 and q1[0, 0] == 0x78 and q1[0, 1] == 0xfc and not q1[0, 2:].any()


# ---------------------------------------------------------------- weight-only FP8 with a scale per output row (GLM dense projections)

def test_fp8_rowscale_quant_and_gemv_vs_library(oracle):
    # quantiser (reference dense_fp8.rs:59-62) against torch's own float8 cast, the product against a binary64 matmul of the library's
    # f16 / bf16 roundings; hand-worked values pin the scale rule and the order "sum, then scale, then round"
    g = torch.Generator().manual_seed(11)
    n, k, m = 96, 320, 5
    w = torch.randn(n, k, generator=g) * (10.0 ** torch.empty(n, 1).uniform_(-3, 2, generator=g))
    w[7] = 0.0                                                          # an all-zero row: the scale floor 1e-12 / 448, codes 0
    q, s = oracle.fp8_rowscale_quant(w.numpy())
    s_ref = (w.abs().amax(dim=1).clamp_min(1e-12) / 448.0)
    assert np.array_equal(s, s_ref.numpy())
    q_ref = (w / s_ref[:, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(q, q_ref)
    assert (np.abs(torch.from_numpy(q).view(torch.float8_e4m3fn).float().numpy()).max(axis=1)[np.arange(n) != 7] == 448.0).all()   # every row uses the full range
    x = torch.randn(m, k, generator=g) * 3.0
    wd = torch.from_numpy(q).view(torch.float8_e4m3fn).double()
    for act, cast in ((0, torch.float16), (1, torch.bfloat16)):
        ref = ((x.to(cast).double() @ wd.T).float() * torch.from_numpy(s)[None]).numpy()
        got = oracle.fp8_rowscale_gemv(x.numpy(), q, s, act=act)
        assert np.array_equal(got, ref)                                 # binary64 sums of exact products: the same value whatever the order
        assert not np.array_equal(got, oracle.fp8_rowscale_gemv(x.numpy(), q, s, act=2))          # the rounding of the activations is there
    rounded = oracle.fp8_rowscale_gemv(x.numpy(), q, s, act=0, rounded=True)
    ref = ((x.half().double() @ wd.T).float() * torch.from_numpy(s)[None]).half().float().numpy()
    assert np.array_equal(rounded, ref)
    # by hand: w row (2, -1), x (3, 5) -> scale 2 / 448, codes 448 and -224, sum 3 * 448 - 5 * 224 = 224, y = 224 * 2 / 448 = 1
    q1, s1 = oracle.fp8_rowscale_quant(np.array([[2.0, -1.0] + [0.0] * 6], np.float32))
    assert s1[0] == np.float32(2.0) / np.float32(448.0) and q1[0, 0] == 0x7e and q1[0, 1] == 0xf6
    y1 = oracle.fp8_rowscale_gemv(np.array([[3.0, 5.0] + [0.0] * 6], np.float32), q1, s1, act=0)
    assert abs(y1[0, 0] - 1.0) < 1e-6


# ---------------------------------------------------------------- shared-expert glue

def test_swiglu_quant_vs_float64_and_act_quant(oracle):
    g = torch.Generator().manual_seed(7)
    T, I = 16, 256
    gu = torch.randn(T, 2 * I, generator=g) * (10.0 ** torch.empty(T, 1).uniform_(-2, 1.5, generator=g))
    gu[0, :4] = torch.tensor([3.0, -20.0, 40.0, 11.0]); gu[0, I:I + 4] = torch.tensor([0.5, 40.0, -40.0, 2.0])   # the clamp cases of the reference's test
    for lim in (10.0, 0.0, 7.0):
        gb = gu[:, :I].to(torch.bfloat16).double(); ub = gu[:, I:].to(torch.bfloat16).double()      # library bf16 rounding
        if lim > 0:
            gb = gb.clamp(max=lim); ub = ub.clamp(min=-lim, max=lim)
        v64 = (gb / (1.0 + torch.exp(-gb)) * ub).numpy()
        vb = torch.from_numpy(v64).to(torch.float32).to(torch.bfloat16)
        ref = oracle.act_quant32(vb.view(torch.int16).numpy().view(np.uint16))                        # pinned above against the library
        got = oracle.swiglu_quant(gu.numpy(), lim)
        safe = _bf16_safe(v64).reshape(T, I // 32, 32).all(-1)                                        # blocks every element of which rounds robustly
        assert safe.mean() > 0.9
        eq = (got == ref).reshape(T, I // 32, 32).all(-1)
        assert eq[safe].all(), f"lim {lim}: {np.argwhere(safe & ~eq)[:4]}"
        # the other blocks may differ where one value sat on a rounding boundary; they still agree to one step of the block's grid
        d = np.abs(oracle.bf16_to_f32(got) - oracle.bf16_to_f32(ref))
        assert (d <= 2.0 ** -3 * np.abs(oracle.bf16_to_f32(ref)).reshape(T, I // 32, 32).max(-1, keepdims=True).repeat(32, -1).reshape(T, I) + 1e-30).all()
    # clamp semantics (reference glm53_tests/test_moe.py:34-40): gate one-sided, up two-sided; lim = 0 switches the clamp off
    one = np.zeros((1, 64), np.float32); one[0, 0] = 40.0; one[0, 32] = 40.0
    assert oracle.bf16_to_f32(oracle.swiglu_quant(one, 10.0))[0, 0] <= 100.0 < oracle.bf16_to_f32(oracle.swiglu_quant(one, 0.0))[0, 0]
    one[0, 0] = 3.0; one[0, 32] = -40.0
    assert abs(oracle.bf16_to_f32(oracle.swiglu_quant(one, 10.0))[0, 0] + 10.0 * 3.0 / (1 + np.exp(-3.0))) <= 1.0     # half a step of the E4M3 grid at 228 x 2^-3


def test_silu_mul_and_gate_scale_vs_float64(oracle):
    rng = np.random.default_rng(8)
    gv = (rng.standard_normal(5000) * 10.0 ** rng.uniform(-3, 1.3, 5000)).astype(np.float32)
    uv = rng.standard_normal(5000).astype(np.float32)
    ref = gv.astype(np.float64) / (1.0 + np.exp(-gv.astype(np.float64))) * uv.astype(np.float64)
    got = oracle.silu_mul(gv, uv)
    assert np.all(np.abs(got - ref) <= 4e-7 * np.abs(ref) + 1e-38)
    assert oracle.silu_mul(np.array([0.0], np.float32), np.array([5.0], np.float32))[0] == 0.0
    gl = (rng.standard_normal((7, 13)) * 4).astype(np.float32)
    d = rng.standard_normal((7, 96)).astype(np.float32)
    for col in (0, 5, 12):
        ref = (1.0 / (1.0 + np.exp(-gl[:, col].astype(np.float64))))[:, None] * d.astype(np.float64)
        got = oracle.gate_scale(gl, col, d)
        assert np.all(np.abs(got - ref) <= 4e-7 * np.abs(ref))
    # a transposed / mis-strided gate would pick another element: rows must use their own gate
    z = np.zeros((3, 4), np.float32); z[1, 2] = 50.0; z[0, 2] = -50.0
    o = oracle.gate_scale(z, 2, np.ones((3, 8), np.float32))
    assert np.allclose(o[0], 0.0, atol=1e-20) and np.allclose(o[1], 1.0) and np.allclose(o[2], 0.5)
