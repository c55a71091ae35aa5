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


def _ds41_cases(n, seed):
    g = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        I = int(g.choice([128, 256, 512, 640, 768, 1024, 1536, 2048, 2304]))
        E = int(g.integers(2, 12))
        topk = int(g.integers(1, min(E, 6) + 1))
        R = int(g.choice([1, 2, 3, 4, 5, 8, 9, 16, 17, 31, 40, 70]))
        if I > 1024:
            R = min(R, 17)
        out.append((R, I, E, topk))
    return out


@pytest.mark.parametrize("R,I,E,topk", _ds41_cases(10, 9003))
def test_ds41_entry_points_random_shapes(ops, oracle, R, I, E, topk):
    # the reference-named entry points (hidden width 5120) on the reference's two tile layouts, raw scale bytes: against the oracle, and
    # bit for bit against the record layout (every path and layout gives a row the same bits)
    H = 5120
    g = synth.rng(R * 13 + I + E)
    ws = synth.mxfp4_experts(g, E, H, I, 119)
    x = synth.randn_bf16(g, (R, H))
    idx = np.stack([g.permutation(E)[:topk] for _ in range(R)]).astype(np.int64)
    rw = g.uniform(0.1, 1.0, (R, topk)).astype(np.float32)
    add = g.standard_normal((R, H)).astype(np.float32)
    ref = oracle.mxfp4_moe(x, idx, rw, *ws, add=add)
    d = [dev(a) for a in ws]
    p1, ps1 = ops.moe_pack(d[0], d[1]); p3, ps3 = ops.moe_pack(d[2], d[3]); p2, ps2 = ops.moe_pack(d[4], d[5])
    xq, xs = ops.act_quant_fp8(dev_bf16(x))
    y_mx, _ = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), (ops.moe_pack_mx(p1), ps1, ops.moe_pack_mx(p3), ps3, ops.moe_pack_mx(p2), ps2), I, add=dev(add))
    assert rel_l2(host(y_mx), ref) <= TOL, rel_l2(host(y_mx), ref)
    y_p8 = ops.ds41_moe(ops.act_quant(dev_bf16(x)), dev(idx), dev(rw), (p1, ps1, p3, ps3, p2, ps2), I, add=dev(add))
    assert np.array_equal(host(y_p8), host(y_mx))
    y_rec = host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ops.Mxfp4Experts(*d), add=dev(add)))
    assert np.array_equal(y_rec, host(y_mx))
