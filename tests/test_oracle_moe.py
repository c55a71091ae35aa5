"""Pins the oracle's routers and MoE compositions against library routines (torch softmax / topk / softplus / sigmoid,
float8 casts) and special cases that reduce to a dense MLP.  CPU only."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from spark_engine_amd import synth


def test_qwen_route_vs_torch(oracle):
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(7, 512, generator=g)
    idx, w = oracle.qwen_route(logits.numpy(), 10)
    p = torch.softmax(logits, -1)
    wr, ir = torch.topk(p, 10, -1)                                    # reference test_kern_moe.py:17
    wr = wr / wr.sum(-1, keepdim=True)
    assert np.array_equal(idx, ir.numpy())
    assert np.allclose(w, wr.numpy(), rtol=1e-5)
    # ties -> lower index first (reference qwen_moe.cu:44,53)
    t = torch.zeros(1, 512); t[0, [400, 17, 300]] = 1.0
    idx, w = oracle.qwen_route(t.numpy(), 10)
    assert idx[0, :3].tolist() == [17, 300, 400] and idx[0, 3:].tolist() == list(range(7))


def test_ds41_route_vs_torch(oracle):
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(5, 384, generator=g) * 3
    logits[0, 3] = 25.0                                               # above the softplus threshold
    bias = torch.randn(384, generator=g) * 0.1
    idx, w = oracle.ds41_route(logits.numpy(), bias.numpy(), 6, 1.5)
    s = torch.sqrt(F.softplus(logits))                                # torch's threshold is 20 as well
    ir = (s + bias).topk(6, -1).indices
    wr = torch.gather(s, 1, ir)
    wr = wr / (wr.sum(-1, keepdim=True) + 1e-20) * 1.5                # reference kern.rs:1965-1977
    assert np.array_equal(idx, ir.numpy())
    assert np.allclose(w, wr.numpy(), rtol=2e-6)
    idx1, w1 = oracle.ds41_route(logits.numpy(), bias.numpy(), 1, 2.0)   # k = 1: not normalised
    assert np.allclose(w1[:, 0], torch.gather(s, 1, torch.from_numpy(idx1))[:, 0].numpy() * 2.0, rtol=2e-6)
    z = np.zeros((1, 384), np.float32)
    idxz, _ = oracle.ds41_route(z, np.zeros(384, np.float32), 6, 1.0)
    assert idxz[0].tolist() == [0, 1, 2, 3, 4, 5]                      # ties -> lower index


def test_glm_route_noaux_tc_math(oracle):
    # reference glm53_tests/test_moe.py:20-31 restated on logits
    torch.manual_seed(0)
    h = torch.randn(1, 8); wg = torch.randn(5, 8); bias = torch.randn(5)
    logits = (h @ wg.T)
    idx, w = oracle.glm_route(logits.numpy(), bias.numpy(), 3, 2.5)
    scores = torch.sigmoid(logits)[0]
    sel = (scores + bias).topk(3).indices.tolist()
    assert idx[0].tolist() == sel
    raw = torch.tensor([scores[i] for i in sel])
    assert np.allclose(w[0], (raw / raw.sum() * 2.5).numpy(), atol=1e-6)


def _dense_mlp64(x, Wg, Wu, Wd, clamp):
    g = x @ Wg; u = x @ Wu
    if clamp:
        g = np.minimum(g, 10.0); u = np.clip(u, -10.0, 10.0)
    return (g / (1 + np.exp(-g)) * u) @ Wd


@pytest.mark.parametrize("cbk,act", [(2, 0), (1, 1)])
def test_exl3_moe_reduces_to_dense_mlp(oracle, cbk, act):
    # topk = 1, weight 1: the routed layer is one dense 3-matrix MLP on the dequantised weights (float64 here)
    g = synth.rng(3)
    H, I, E = 256, 128, 4
    experts = {e: synth.exl3_expert(g, H, I) for e in range(E)}
    x = g.standard_normal((2, H)).astype(np.float32) * 3
    idx = np.array([[2], [0]], np.int32); w = np.ones((2, 1), np.float32)
    out = oracle.exl3_moe(x, idx, w, experts, E, H, I, 4, cbk, act)
    for r in range(2):
        t = experts[int(idx[r, 0])]
        Wg = oracle.decode_weight(t[0], t[3], t[6], cbk).astype(np.float64)
        Wu = oracle.decode_weight(t[1], t[4], t[7], cbk).astype(np.float64)
        Wd = oracle.decode_weight(t[2], t[5], t[8], cbk).astype(np.float64)
        ref = _dense_mlp64(x[r].astype(np.float64), Wg, Wu, Wd, act == 1)
        assert np.linalg.norm(out[r] - ref) / np.linalg.norm(ref) < 1e-5


def test_exl3_moe_weighted_sum_add_and_row_invariance(oracle):
    g = synth.rng(4)
    H, I, E = 256, 128, 6
    experts = {e: synth.exl3_expert(g, H, I) for e in range(E)}
    x = g.standard_normal((3, H)).astype(np.float32)
    idx = np.array([[1, 4], [4, 1], [5, 0]], np.int32)
    w = g.uniform(0.1, 1, (3, 2)).astype(np.float32)
    add = g.standard_normal((3, H)).astype(np.float32)
    out = oracle.exl3_moe(x, idx, w, experts, E, H, I, 4, 2, 0, add)
    # linearity in the route weights and the add term
    single = [[oracle.exl3_moe(x[r:r + 1], idx[r:r + 1, k:k + 1], np.ones((1, 1), np.float32), experts, E, H, I, 4, 2, 0)[0]
               for k in range(2)] for r in range(3)]
    for r in range(3):
        ref = add[r] + w[r, 0] * single[r][0] + w[r, 1] * single[r][1]
        assert np.allclose(out[r], ref, rtol=1e-5, atol=1e-5)
    # a row's result does not depend on the other rows in the call
    assert np.array_equal(oracle.exl3_moe(x[1:2], idx[1:2], w[1:2], experts, E, H, I, 4, 2, 0, add[1:2])[0], out[1])


def _ds41_pair_torch(xd, w1, s1, w3, s3, w2, s2, rw, oracle):
    """reference ds41/kern.rs:1116-1133 (moe_ref) for one pair, with torch ops."""
    bf = lambda t: t.to(torch.bfloat16).float()
    deq = lambda w, s: torch.from_numpy(oracle.mxfp4_dequant(w, s))
    x = torch.from_numpy(xd)[None]
    g = bf(x @ deq(w1, s1).T).clamp_max(10.0)
    u = bf(x @ deq(w3, s3).T).clamp(-10.0, 10.0)
    hm = (F.silu(g) * u * rw).to(torch.bfloat16)
    hb = hm.view(torch.int16).numpy().view(np.uint16)
    hq = torch.from_numpy(oracle.bf16_to_f32(oracle.act_quant32(hb)))
    return (hq @ deq(w2, s2).T)[0].numpy()


def test_mxfp4_moe_vs_torch_restatement(oracle):
    g = synth.rng(5)
    H, I, E, topk, R = 256, 128, 5, 2, 3
    ws = synth.mxfp4_experts(g, E + 1, H, I, smin=119)
    x = synth.randn_bf16(g, (R, H))
    idx = np.array([[0, 3], [3, 4], [1, 2]], np.int64)
    rw = g.uniform(0.2, 1.0, (R, topk)).astype(np.float32)
    add = g.standard_normal((R, H)).astype(np.float32)
    y, pairs = oracle.mxfp4_moe(x, idx, rw, *ws, n_shared=1, add=add, want_pairs=True)
    xd = oracle.bf16_to_f32(oracle.act_quant32(x))
    for r in range(R):
        acc = np.zeros(H, np.float32)
        for k in range(topk):
            e = int(idx[r, k])
            ref = _ds41_pair_torch(xd[r], ws[0][e], ws[1][e], ws[2][e], ws[3][e], ws[4][e], ws[5][e], float(rw[r, k]), oracle)
            assert np.linalg.norm(pairs[r * topk + k] - ref) <= 2e-3 * np.linalg.norm(ref)   # bf16 / e4m3 roundings may flip on summation order
            acc = acc + pairs[r * topk + k]
        sh = _ds41_pair_torch(xd[r], ws[0][E], ws[1][E], ws[2][E], ws[3][E], ws[4][E], ws[5][E], 1.0, oracle)
        full = add[r] + sh + acc
        assert np.linalg.norm(y[r] - full) <= 2e-3 * np.linalg.norm(full)
    # zero codes -> zero expert output: y == add
    zw = [np.zeros_like(a) if i % 2 == 0 else a for i, a in enumerate(ws)]
    y0 = oracle.mxfp4_moe(x, idx, rw, *zw, n_shared=1, add=add)
    assert np.array_equal(y0, add)


def test_dense_gemvs_vs_float64(oracle):
    g = synth.rng(6)
    w, s = synth.mxfp4_matrix(g, 64, 256, 119)
    x = synth.randn_bf16(g, (2, 256))
    y = oracle.mxfp4_gemv(x, w, s)
    ref = oracle.bf16_to_f32(x).astype(np.float64) @ oracle.mxfp4_dequant(w, s).astype(np.float64).T
    assert np.allclose(y, ref, rtol=1e-5, atol=1e-5)
    w8, s8 = synth.fp8_block_matrix(g, 256, 384)
    x = synth.randn_bf16(g, (3, 384))
    y = oracle.fp8_block_gemv(x, w8, s8)
    ref = oracle.bf16_to_f32(x).astype(np.float64) @ oracle.fp8_block_dequant(w8, s8).astype(np.float64).T
    assert np.allclose(y, ref, rtol=1e-5, atol=1e-6)
