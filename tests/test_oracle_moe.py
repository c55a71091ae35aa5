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


def _ds41_pair_stages(xd, w1, s1, w3, s3, w2, s2, rw, oracle):
    """reference ds41/kern.rs:1116-1133 (moe_ref) for one pair, stage by stage with library routines: the gate / up sums in
    binary64 (exact for these terms, whatever the order), the activation in binary64 too, the quantiser through
    torch.float8_e4m3fn.  -> E4M3 codes [I], scale bytes [I / 32], and which 32-blocks are robust: no element's product within 1e-6
    of a bf16 rounding boundary, so that a last-place difference of expf cannot change a code or the block's scale."""
    from tests.gpu_util import bf16_safe
    bf = lambda t: t.float().to(torch.bfloat16).double()
    deq = lambda w, s: torch.from_numpy(oracle.mxfp4_dequant(w, s)).double()
    x = torch.from_numpy(xd).double()[None]
    g = bf(x @ deq(w1, s1).T).clamp_max(10.0)[0]
    u = bf(x @ deq(w3, s3).T).clamp(-10.0, 10.0)[0]
    y64 = g / (1.0 + torch.exp(-g)) * u * float(np.float32(rw))
    # element by element: none of its three roundings within 1e-6 of a rounding boundary (gate / up sums: of the norm of their terms; product: of itself)
    tnorm = lambda w, s: torch.sqrt((x * x) @ (deq(w, s) ** 2).T)[0].numpy()                       # the norm of each sum's terms
    esafe = (bf16_safe(y64.numpy(), margin=1e-6) & bf16_safe((x @ deq(w1, s1).T)[0].numpy(), margin=1e-6, size=tnorm(w1, s1)) &
             bf16_safe((x @ deq(w3, s3).T)[0].numpy(), margin=1e-6, size=tnorm(w3, s3)))
    safe = torch.from_numpy(bf16_safe(y64.numpy(), margin=1e-6)).view(-1, 32).all(dim=1).numpy()
    yb = y64.float().to(torch.bfloat16).float().view(-1, 32)
    amax = yb.abs().amax(dim=1).clamp_min(1e-4)
    e = torch.ceil(torch.log2(amax.double() / 448.0)).to(torch.int32)              # scale = 2^ceil(log2(amax / 448)), reference kernel.py:59-73
    q = (yb.double() / torch.pow(2.0, e.double())[:, None]).clamp(-448.0, 448.0).float().to(torch.float8_e4m3fn)
    return q.view(torch.uint8).view(-1).numpy(), (e + 127).to(torch.uint8).numpy(), safe, esafe


def test_mxfp4_moe_stage_by_stage_vs_library_routines(oracle):
    g = synth.rng(5)
    H, I, E, topk, R = 512, 256, 5, 2, 3
    ws = synth.mxfp4_experts(g, E + 1, H, I, smin=119)
    x = synth.randn_bf16(g, (R, H))
    idx = np.array([[0, 3], [3, 4], [1, 2]], np.int64)
    rw = g.uniform(0.2, 1.0, (R, topk)).astype(np.float32)
    add = g.standard_normal((R, H)).astype(np.float32)
    y, pairs, hq, hs, hmargin = oracle.mxfp4_moe(x, idx, rw, *ws, n_shared=1, add=add, want_pairs=True, want_h=True)
    xd = oracle.bf16_to_f32(oracle.act_quant32(x))
    P = R * topk
    nblocks = nsafe = 0
    for p in range(P + R):                                             # routed pairs, then the shared expert of every row
        r, e, w = (p // topk, int(idx.ravel()[p]), float(rw.ravel()[p])) if p < P else (p - P, E, 1.0)
        q, sb, safe, esafe = _ds41_pair_stages(xd[r], *[a[e] for a in ws], w, oracle)
        # the oracle's own rounding margins say the same, element by element (elements right at the threshold aside)
        clear = np.abs(hmargin[p] - 1e-6) > 1e-7
        assert np.array_equal((hmargin[p] > 1e-6)[clear], esafe[clear])
        nblocks += safe.size; nsafe += int(safe.sum())
        # the intermediate: codes and scale bytes equal on every robust block (a dropped rounding, a missing route weight, a wrong
        # clamp or scale rule changes nearly every block)
        assert np.array_equal(hs[p][safe], sb[safe])
        assert np.array_equal(hq[p].reshape(-1, 32)[safe], q.reshape(-1, 32)[safe])
        # the down product of the oracle's own codes, in binary64
        hm = torch.from_numpy(hq[p].copy()).view(torch.float8_e4m3fn).double() * torch.pow(2.0, torch.from_numpy(hs[p].astype(np.float64)) - 127.0).repeat_interleave(32)
        out = (hm[None] @ torch.from_numpy(oracle.mxfp4_dequant(ws[4][e], ws[5][e])).double().T)[0].numpy()
        if p < P:
            assert np.linalg.norm(pairs[p] - out) <= 1e-5 * np.linalg.norm(out)
        else:
            routed = np.zeros(H, np.float32)
            for k in range(topk):
                routed = routed + pairs[r * topk + k]                  # slot order, then added to add + shared (reference ds41_mx.cu:302-317)
            full = (add[r].astype(np.float64) + out) + routed
            assert np.linalg.norm(y[r] - full) <= 1e-5 * np.linalg.norm(full)
    assert nsafe >= 0.9 * nblocks, (nsafe, nblocks)                   # the exact comparison covers nearly everything
    assert (hmargin < 1e-6).sum() >= 1                                # and the margins do flag something at this size
    # the second half alone, on the oracle's own intermediate, is the whole: same operations in the same order
    assert np.array_equal(oracle.mxfp4_moe_from_h(hq, hs, idx, ws[4], ws[5], n_shared=1, add=add), y)
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
