"""Seeded sweeps over the shapes the expert layers accept (hidden and intermediate widths, expert counts, top-k, shared experts,
row counts on both sides of the single-launch limit), each case against the CPU oracle through the C ABI.  The fixed-shape tests
pin named cases; these draw the combinations nobody thought of.  Tolerance: rel-L2 <= 1e-3 on the FP32 output
(reference kern.rs:2206-2208, test_kern_moe.py:24)."""
import numpy as np
import pytest
import torch

from spark_engine_amd import synth
from tests.gpu_util import dev, dev_bf16, dev_f16, host, rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def ops():
    from spark_engine_amd import ops
    return ops


def _mx_cases(n, seed):
    g = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        H = int(g.choice([512, 768, 1024, 1280, 1536, 2048, 2560, 3072, 4096, 4608, 5120]))
        I = int(g.choice([128, 256, 384, 512, 640, 768, 1024, 1152, 2048, 2304]))
        E = int(g.integers(2, 24))
        ns = int(g.integers(0, 3))
        topk = int(g.integers(1, min(E, 8) + 1))
        R = int(g.choice([1, 1, 2, 3, 4, 5, 7, 8, 9, 12, 17, 33]))
        if H * I > 3 * 2 ** 20:                                        # the oracle walks every pair on the CPU: bound the big ones
            R = min(R, 4)
        out.append((R, H, I, E, topk, ns))
    return out


@pytest.mark.parametrize("R,H,I,E,topk,ns", _mx_cases(24, 9001))
def test_mxfp4_layer_random_shapes(ops, oracle, R, H, I, E, topk, ns):
    g = synth.rng(R * 7 + H + I + E)
    ws = synth.mxfp4_experts(g, E + ns, H, I, 117)
    x = synth.randn_bf16(g, (R, H))
    idx = np.stack([g.permutation(E)[:topk] for _ in range(R)]).astype(np.int64)
    rw = g.uniform(0.1, 1.0, (R, topk)).astype(np.float32)
    add = g.standard_normal((R, H)).astype(np.float32) if (R + E) % 2 else None
    ex = ops.Mxfp4Experts(*[dev(a) for a in ws], n_shared=ns)
    ref = oracle.mxfp4_moe(x, idx, rw, *ws, n_shared=ns, add=add)
    y = host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ex, add=None if add is None else dev(add)))
    assert rel_l2(y, ref) <= TOL, rel_l2(y, ref)
    # a row's bits do not depend on the path or on the other rows: the first row alone (single launch) against the call's first row
    y1 = host(ops.mxfp4_moe(dev_bf16(x[:1]), dev(idx[:1]), dev(rw[:1]), ex, add=None if add is None else dev(add[:1])))
    assert np.array_equal(y1[0], y[0])


def _exl3_cases(n, seed):
    g = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        H = int(g.choice([128, 256, 384, 512, 768, 1024, 1536, 2048]))
        I = int(g.choice([128, 256, 384, 512, 640, 1024]))
        E = int(g.integers(2, 20))
        topk = int(g.integers(1, min(E, 10) + 1))
        R = int(g.choice([1, 1, 2, 3, 4, 6, 8, 9, 13, 20]))
        if H * I > 2 ** 19:
            R = min(R, 4)
        out.append((R, H, I, E, topk, int(g.choice([1, 2])), int(g.integers(0, 2))))
    return out


@pytest.mark.parametrize("R,H,I,E,topk,cbk,act", _exl3_cases(16, 9002))
def test_exl3_layer_random_shapes(ops, oracle, R, H, I, E, topk, cbk, act):
    g = synth.rng(R * 11 + H + I + E)
    logits = g.standard_normal((R, E)).astype(np.float32)
    idx, w = oracle.qwen_route(logits, topk)
    used = sorted(set(idx.ravel().tolist()))
    experts = {e: synth.exl3_expert(g, H, I) for e in used}
    xb = synth.randn_bf16(g, (R, H))
    ref = oracle.exl3_moe(synth.bf16_to_f32(xb), idx, w, experts, E, H, I, 4, cbk, act)
    table = ops.ExpertTable({e: [dev(t[0]), dev(t[1]), dev(t[2])] + [dev_f16(a) for a in t[3:]] for e, t in experts.items()}, E)
    out = host(ops.exl3_moe(dev_bf16(xb), dev(idx), dev(w), table, H, I, cbk, act))
    assert rel_l2(out, ref) <= TOL, rel_l2(out, ref)
    if R <= 8:                                                         # within the single launch a row's bits do not depend on the batch
        o1 = host(ops.exl3_moe(dev_bf16(xb[:1]), dev(idx[:1]), dev(w[:1]), table, H, I, cbk, act))
        assert np.array_equal(o1[0], out[0])
