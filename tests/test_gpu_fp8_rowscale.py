"""GPU parity of the weight-only FP8 GEMV with one scale per output row (the reference's GLM dense / shared-expert projections,
engine-rs/shim/fp8.cu:13-22,110-151) against the CPU oracle.  Bound: max |diff| / max |ref| < 1e-5, the reference's own bar for its
dense GEMVs against a dequantise + FP32 matmul (engine-rs/src/ds41/kern.rs:1863-1867)."""
import numpy as np
import pytest
import torch

from spark_engine_amd import synth
from tests.gpu_util import DEV, dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from spark_engine_amd import ops
    return ops


def _maxrel(a, b):
    return float(np.abs(a.astype(np.float64) - b).max() / np.abs(b).max())


def _case(ops, g, n, k, m):
    w = torch.from_numpy(g.standard_normal((n, k)).astype(np.float32) * 10.0 ** g.uniform(-2, 1, (n, 1)).astype(np.float32)).to(DEV)
    q, s = ops.fp8_rowscale_quantize(w)
    x = (g.standard_normal((m, k)) * 2.0).astype(np.float32)
    return q, s, x, host(w)


@pytest.mark.parametrize("n,k", [(4096, 4096), (2048, 6144), (320, 1280), (192, 320), (64, 64), (6144, 512)])
@pytest.mark.parametrize("m", [1, 4, 16])
def test_dense_f16_activations_vs_oracle(ops, oracle, n, k, m):
    g = synth.rng(900 + m)
    q, s, x, w = _case(ops, g, n, k, m)
    qh, sh = host(q), host(s)
    oq, osc = oracle.fp8_rowscale_quant(w)
    assert np.array_equal(osc, sh) and np.array_equal(oq, qh)           # the host-side mirror of the reference's quantiser and the oracle's agree
    ref = oracle.fp8_rowscale_gemv(x, qh, sh, act=0)
    y = host(ops.glm_fp8_dense(dev(x), q, s))
    assert _maxrel(y, ref) < 1e-5, _maxrel(y, ref)
    yr = host(ops.glm_fp8_dense(dev(x), q, s, rounded=True))
    assert np.array_equal(yr, host(torch.from_numpy(y).half().float()))  # the rounded form is the binary16 rounding of what the plain form stores
    # a row's value does not depend on the rows beside it
    if m > 1:
        assert np.array_equal(host(ops.glm_fp8_dense(dev(x[m - 1:]), q, s))[0], y[m - 1])


@pytest.mark.parametrize("n,k", [(4096, 4096), (320, 1280), (128, 192)])
def test_bf16_activations_and_skinny_rows(ops, oracle, n, k):
    g = synth.rng(910)
    q, s, x, _ = _case(ops, g, n, k, 32)
    qh, sh = host(q), host(s)
    ref = oracle.fp8_rowscale_gemv(x, qh, sh, act=1)
    y16 = host(ops.glm_fp8_dense(dev(x[:16]), q, s, act="bf16"))
    assert _maxrel(y16, ref[:16]) < 1e-5
    # exact in the activations' scale: a power of two scales every product and every sum (bf16 has binary32's exponent range;
    # binary16 activations would lose bits of their smallest values)
    assert np.array_equal(host(ops.glm_fp8_dense(dev(x[:16] * 4.0), q, s, act="bf16")), y16 * 4.0)
    xb = dev(x).to(torch.bfloat16)                                       # the same rounding, done by the caller: the skinny entry reads bf16 rows
    y32 = host(ops.glm_fp8_dense(xb, q, s))
    assert _maxrel(y32, ref) < 1e-5
    assert np.array_equal(y32[:16], y16)
    for lo, hi in ((0, 2), (5, 8), (29, 32)):                            # rows 17..32 and small calls give a row the same bits (reference fp8.cu:136-137)
        assert np.array_equal(host(ops.glm_fp8_dense(xb[lo:hi], q, s)), y32[lo:hi])


def test_shapes_outside_the_limits_are_refused(ops):
    q = torch.zeros(128, 128, dtype=torch.uint8, device=DEV)
    s = torch.ones(128, device=DEV)
    x = torch.zeros(17, 128, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.glm_fp8_dense(x, q, s)                                       # more than 16 rows
    with pytest.raises(ops.KernelError):
        ops.glm_fp8_dense(x[:1].to(torch.bfloat16), q, s)                # the skinny entry starts at two rows
    with pytest.raises(ops.KernelError):
        ops.glm_fp8_dense(torch.zeros(2, 96, device=DEV), q[:, :96].contiguous(), s)       # k not a multiple of 64
    with pytest.raises(ops.KernelError):
        ops.glm_fp8_dense(x[:2], q[:100].contiguous(), s[:100].contiguous())               # n not a multiple of 64
