"""GPU parity: dequantisation surfaces (bit-exact), act_quant (bit-exact), routers (exact indices), dense GEMVs.
Every call goes through the C ABI of libspark_shim_hip.so."""
import numpy as np
import pytest
import torch

from spark_engine_amd import synth
from tests.gpu_util import DEV, dev, dev_bf16, dev_f16, host, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from spark_engine_amd import ops
    return ops


@pytest.mark.parametrize("cbk", [2, 1])
@pytest.mark.parametrize("bits", [4, 3, 5, 6])
def test_exl3_reconstruct_bit_exact(ops, oracle, cbk, bits):
    g = synth.rng(100 + bits)
    tr = g.integers(-32768, 32768, (24, 9, 16 * bits), dtype=np.int16)
    got = host(ops.exl3_reconstruct(dev(tr), cbk))
    assert np.array_equal(got, oracle.decode_inner(tr, cbk))


def test_exl3_reconstruct_all_codebook_states(ops, oracle):
    # a 4-bit tile stream visits the states of its nibble 4-grams: cover the whole codebook with a De Bruijn-free trick,
    # 4096 tiles of random bits and compare the multiset of decoded values against the tables
    g = synth.rng(7)
    tr = g.integers(-32768, 32768, (64, 64, 64), dtype=np.int16)
    for cbk in (1, 2):
        assert np.array_equal(host(ops.exl3_reconstruct(dev(tr), cbk)), oracle.decode_inner(tr, cbk))


@pytest.mark.parametrize("cbk,bits", [(2, 4), (1, 4), (2, 5)])
def test_exl3_fold_bit_exact(ops, oracle, cbk, bits):
    g = synth.rng(110 + bits + cbk)
    K, N = 256, 384
    tr, suh, svh = synth.exl3_matrix(g, K, N, bits)
    got = host(ops.exl3_fold(dev(tr), dev_f16(suh), dev_f16(svh), cbk))
    assert np.array_equal(got, oracle.fold(tr, suh, svh, cbk))


def test_mxfp4_dequant_bit_exact(ops, oracle):
    g = synth.rng(120)
    w, s = synth.mxfp4_matrix(g, 96, 512, 1, 250)
    assert np.array_equal(host(ops.mxfp4_dequant(dev(w), dev(s))), oracle.mxfp4_dequant(w, s))
    # every byte value under one scale
    w = np.tile(np.arange(256, dtype=np.uint8), (4, 1)).reshape(4, 256)[:, :64].copy(); w = np.arange(256, dtype=np.uint8).reshape(16, 16)
    s = np.full((16, 1), 125, np.uint8)
    assert np.array_equal(host(ops.mxfp4_dequant(dev(w), dev(s))), oracle.mxfp4_dequant(w, s))


def test_fp8_dequant_bit_exact(ops, oracle):
    g = synth.rng(121)
    w = g.integers(0, 256, (256, 384), dtype=np.uint8)
    w[(w & 0x7f) == 0x7f] = 0x12
    w[0, :256] = np.arange(256, dtype=np.uint8); w[0, 0x7f] = 0; w[0, 0xff] = 0   # every finite code
    s = np.exp(g.uniform(np.log(1e-3), np.log(1e-1), (2, 3))).astype(np.float32)
    assert np.array_equal(host(ops.fp8_block_dequant(dev(w), dev(s), 128)), oracle.fp8_block_dequant(w, s, 128))
    s8 = g.integers(100, 135, (8, 12), dtype=np.uint8)
    assert np.array_equal(host(ops.fp8_e8m0_dequant(dev(w), dev(s8))), oracle.fp8_e8m0_dequant(w, s8))


def test_act_quant_bit_exact(ops, oracle):
    g = synth.rng(122)
    x = g.standard_normal((512, 64), np.float32) * (10.0 ** g.uniform(-6, 3, (512, 1))).astype(np.float32)
    x[:8] = 0
    x[8:72, 0] = (448.0 * 2.0 ** np.arange(-32, 32)).astype(np.float32)
    xb = synth.bf16_bits(x)
    q, s = ops.act_quant_fp8(dev_bf16(xb))
    qo, so = oracle.act_quant_fp8(xb)
    assert np.array_equal(host(s), so)
    qh = host(q)
    z = (qo & 0x7f) == 0
    assert np.array_equal(qh[~z], qo[~z]) and np.all((qh[z] & 0x7f) == 0)
    d = host(ops.act_quant(dev_bf16(xb)))
    assert np.array_equal(synth.bf16_to_f32(d), synth.bf16_to_f32(oracle.act_quant32(xb)))


def test_requant_fp8_is_act_quant_of_the_dequantised_rows(ops, oracle):
    """The reference's own check (kern.rs:1820-1828): random E4M3 bytes (no NaN) under every scale byte 0 .. 254; the bytes and scales
    of act_quant_fp8 of the bf16 dequantisation, from this library's act_quant_fp8 and from the oracle."""
    g = synth.rng(123)
    R = 255 * 8
    wq = g.integers(0, 256, (R, 64), dtype=np.uint8)
    wq[(wq & 0x7f) == 0x7f] = 0x3c
    ws = np.repeat(np.arange(255, dtype=np.uint8), 8)[:, None].repeat(2, axis=1).copy()
    ws[::3, 1] = g.integers(96, 140, len(ws[::3]), dtype=np.uint8)
    wq[:4] = 0                                             # blocks of zeros
    q, s = ops.requant_fp8(dev(wq), dev(ws))
    # the dequantised rows as bf16 (exact products of a 4-bit significand and a power of two, rounded to bf16 only where they leave its range)
    # (scale byte 0 stands for the factor 0, not 2^-127: a negative byte then gives -0, reference ops::e8m0)
    f = np.where(ws == 0, 0.0, np.exp2(ws.astype(np.float64) - 127.0)).repeat(32, axis=1)
    with np.errstate(over="ignore"):
        W = (torch.from_numpy(wq.copy()).view(torch.float8_e4m3fn).to(torch.float64).numpy() * f).astype(np.float32)
    xb = synth.bf16_bits(W)
    q2, s2 = ops.act_quant_fp8(dev_bf16(xb))
    assert torch.equal(s, s2) and torch.equal(q, q2)
    fin = (ws <= 240).all(axis=1)                          # the oracle on the rows whose values are finite
    qo, so = oracle.requant_fp8(wq[fin], ws[fin])
    assert np.array_equal(host(s)[fin], so)
    qh = host(q)[fin]; z = (qo & 0x7f) == 0
    assert np.array_equal(qh[~z], qo[~z]) and np.all((qh[z] & 0x7f) == 0)
    assert ops._lib().ds41_requant_fp8(ops._p(dev(wq)), ops._p(dev(ws)), ops._p(q), ops._p(s), 33, ops._st()) == 1


def test_act_quant_every_bf16_value(ops, oracle):
    # all 65536 bf16 patterns (finite ones) in blocks that share a large amax, and alone in a block
    bits = np.arange(65536, dtype=np.uint16)
    f = synth.bf16_to_f32(bits)
    ok = np.isfinite(f) & (np.abs(f) < 1e30)
    bits = bits[ok]
    pad = (-len(bits)) % 32
    bits = np.concatenate([bits, np.zeros(pad, np.uint16)]).reshape(-1, 32)
    q, s = ops.act_quant_fp8(dev_bf16(bits))
    qo, so = oracle.act_quant_fp8(bits)
    assert np.array_equal(host(s), so)
    qh = host(q); z = (qo & 0x7f) == 0
    assert np.array_equal(qh[~z], qo[~z]) and np.all((qh[z] & 0x7f) == 0)


def test_routers_exact_indices(ops, oracle):
    g = synth.rng(130)
    lq = g.standard_normal((5, 512)).astype(np.float32)
    idx, w = ops.qwen_moe_route(dev(lq))
    io, wo = oracle.qwen_route(lq, 10)
    assert np.array_equal(host(idx), io) and np.allclose(host(w), wo, rtol=1e-5)
    idx, w = ops.softmax_route(dev(lq[:, :300].copy()), 6)
    io, wo = oracle.qwen_route(lq[:, :300].copy(), 6)
    assert np.array_equal(host(idx), io) and np.allclose(host(w), wo, rtol=1e-5)
    ld = g.standard_normal((7, 384)).astype(np.float32) * 3
    ld[0, 3] = 25.0
    bias = (g.standard_normal(384) * 0.1).astype(np.float32)
    idx, w = ops.route(dev(ld), dev(bias), 6, 1.5)
    io, wo = oracle.ds41_route(ld, bias, 6, 1.5)
    assert np.array_equal(host(idx), io) and np.allclose(host(w), wo, rtol=2e-6)
    idx, w = ops.sigmoid_route(dev(ld[:, :288].copy()), dev(bias[:288].copy()), 8, 2.5)
    io, wo = oracle.glm_route(ld[:, :288].copy(), bias[:288].copy(), 8, 2.5)
    assert np.array_equal(host(idx), io) and np.allclose(host(w), wo, rtol=2e-6)
    # ties go to the lower expert id
    t = np.zeros((1, 512), np.float32); t[0, [400, 17, 300]] = 1.0
    idx, _ = ops.qwen_moe_route(dev(t))
    assert host(idx)[0].tolist() == [17, 300, 400, 0, 1, 2, 3, 4, 5, 6]
    idx, _ = ops.route(dev(np.zeros((2, 384), np.float32)), dev(np.zeros(384, np.float32)), 6, 1.0)
    assert host(idx).tolist() == [[0, 1, 2, 3, 4, 5]] * 2


@pytest.mark.parametrize("E,K", [(8, 1), (8, 8), (64, 6), (100, 16), (256, 10), (257, 10), (384, 6), (512, 16), (513, 2), (1000, 10), (1024, 16)])
def test_routers_expert_counts_and_ties(ops, oracle, E, K):
    """Every split of the experts over the router's four waves, with logits on a coarse grid so that most picks are decided by
    the tie rule (lower expert id), within a wave and across waves; then continuous logits.  Picks of a row are distinct."""
    g = synth.rng(1300 + E + K)
    for grid in (True, False):
        lg = g.standard_normal((6, E)).astype(np.float32) * 2
        if grid:
            lg = np.round(lg * 2) / 2
            lg[1] = 0.0                                   # one row of nothing but ties
            lg[2, E // 2:] = lg[2, :E - E // 2]           # every value twice, in different waves
        lg = lg.astype(np.float32)
        zb = np.zeros(E, np.float32)
        for name, got, want in (("softmax", ops.softmax_route(dev(lg), K), oracle.qwen_route(lg, K)),
                                ("sqrt-softplus", ops.route(dev(lg), dev(zb), K, 1.5), oracle.ds41_route(lg, zb, K, 1.5)),
                                ("sigmoid", ops.sigmoid_route(dev(lg), dev(zb), K, 2.5), oracle.glm_route(lg, zb, K, 2.5))):
            ids = host(got[0])
            assert np.array_equal(ids, want[0]), (name, E, K, grid)
            assert np.allclose(host(got[1]), want[1], rtol=1e-5), (name, E, K, grid)
            assert all(len(set(r.tolist())) == K for r in ids) and ids.min() >= 0 and ids.max() < E


def test_routers_picks_are_distinct_whatever_the_logits(ops):
    """NaNs, infinities and constant rows: the picks of a row are K different experts in range (what the expert kernels rely on)."""
    g = synth.rng(1399)
    for E, K in ((512, 10), (384, 6), (288, 8), (100, 16)):
        lg = g.standard_normal((8, E)).astype(np.float32)
        lg[0] = np.nan; lg[1] = np.inf; lg[2] = -np.inf; lg[3, ::3] = np.nan; lg[4, ::2] = np.inf; lg[5, 1::2] = -np.inf
        lg[6] = np.float32(np.uint32(0xffffffff).view(np.float32))
        zb = np.zeros(E, np.float32); nb = zb.copy(); nb[::5] = np.nan
        for got in (ops.softmax_route(dev(lg), K), ops.route(dev(lg), dev(zb), K, 1.5), ops.sigmoid_route(dev(lg), dev(nb), K, 2.5)):
            ids = host(got[0])
            assert ids.min() >= 0 and ids.max() < E and all(len(set(r.tolist())) == K for r in ids), (E, K, ids)


def test_glm_router_fused(ops, oracle):
    g = synth.rng(131)
    h = g.standard_normal((3, 1024)).astype(np.float32)
    wg = (g.standard_normal((288, 1024)) * 0.05).astype(np.float32)
    bias = (g.standard_normal(288) * 0.1).astype(np.float32)
    ids, wt = ops.glm_router_fused(dev(h), dev(wg), dev(bias), 2.5)
    logits = (h.astype(np.float64) @ wg.astype(np.float64).T).astype(np.float32)
    io, wo = oracle.glm_route(logits, bias, 8, 2.5)
    assert np.array_equal(host(ids), io) and np.allclose(host(wt), wo, rtol=1e-4)
    # one and two rows, call after call with fresh inputs in between (nothing is carried from one call to the next)
    for it in range(40):
        rows = 1 + it % 2
        h2 = g.standard_normal((rows, 1024)).astype(np.float32)
        i2, w2 = ops.glm_router_fused(dev(h2), dev(wg), dev(bias), 2.5)
        lo, wo2 = oracle.glm_route((h2.astype(np.float64) @ wg.astype(np.float64).T).astype(np.float32), bias, 8, 2.5)
        assert np.array_equal(host(i2), lo) and np.allclose(host(w2), wo2, rtol=1e-4), it
    i1, w1 = ops.glm_router_fused(dev(h[:1].copy()), dev(wg), dev(bias), 2.5)
    assert np.array_equal(host(i1), host(ids)[:1]) and np.array_equal(host(w1), host(wt)[:1])
    # bf16 gate weights, 4096 wide (the reference model's shape)
    h4 = g.standard_normal((2, 4096)).astype(np.float32)
    wb = synth.bf16_bits((g.standard_normal((288, 4096)) * 0.05).astype(np.float32))
    ib, wbt = ops.glm_router_fused(dev(h4), dev_bf16(wb), dev(bias), 2.5)
    lo, wo3 = oracle.glm_route((h4.astype(np.float64) @ synth.bf16_to_f32(wb).astype(np.float64).T).astype(np.float32), bias, 8, 2.5)
    assert np.array_equal(host(ib), lo) and np.allclose(host(wbt), wo3, rtol=1e-4)
    # the form that also writes the binary16 copy of the weights (what glm_moe_experts takes): the same picks and weights, and the
    # copy is the weights' own rounding to nearest even
    ih, wf, wh = ops.glm_router_fused(dev(h4), dev_bf16(wb), dev(bias), 2.5, half_w=True)
    assert np.array_equal(host(ih), host(ib)) and np.array_equal(host(wf), host(wbt))
    assert np.array_equal(wh.cpu().numpy().view(np.uint16), host(wf).astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("m", [1, 2, 4, 7])
def test_mxfp4_gemv(ops, oracle, m):
    # config 1 shape at m = 1: W 2048 x 2048, scales 2^-8 .. 2^0
    g = synth.rng(0)
    n, k = (2048, 2048) if m == 1 else (200, 1024)
    w, s = synth.mxfp4_matrix(g, n, k, 119)
    x = synth.randn_bf16(g, (m, k))
    y = host(ops.mxfp4_gemv(dev_bf16(x), dev(w), dev(s)))
    ref = oracle.mxfp4_gemv(x, w, s)
    assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5         # the reference's own GEMV threshold (kern.rs:1863-1867)
    assert rel_l2(y, ref) < 1e-5


def _t16_pack_np(w):
    """The packed layout restated with numpy index arithmetic: tile (16 rows x 128 k) -> [half h][lane = 16 g + i][16 bytes] with
    bytes 0-7 = W[i][64 h + 8 g ..], bytes 8-15 = W[i][64 h + 32 + 8 g ..]."""
    n, k = w.shape
    t = w.reshape(n // 16, 16, k // 128, 2, 2, 4, 8)          # nt, i, kb, h, step, g, byte
    return np.ascontiguousarray(t.transpose(0, 2, 3, 5, 1, 4, 6)).reshape(-1)      # nt, kb, h, g, i, step, byte


@pytest.mark.parametrize("n,k", [(16, 128), (48, 1152), (128, 2048), (384, 8192)])
def test_fp8_t16_pack_is_the_stated_permutation(ops, n, k):
    g = synth.rng(1500 + n)
    w = g.integers(0, 256, (n, k), dtype=np.uint8)
    assert np.array_equal(host(ops.fp8_t16_pack(dev(w))), _t16_pack_np(w))


@pytest.mark.parametrize("n,k,ms", [(16, 128, (1, 16)), (48, 1152, (1, 2, 3, 5, 16)), (384, 1024, (1, 4, 8)), (144, 8192, (4, 8, 11))])
def test_fp8_block128_gemv_on_packed_weights(ops, oracle, n, k, ms):
    """Every split of K over the waves (one block; a full span and a ragged one; eight spans), every row count class."""
    g = synth.rng(1510 + n + k)
    w8, s = synth.fp8_block_matrix(g, n, k)
    wt = ops.fp8_t16_pack(dev(w8))
    for m in ms:
        x = synth.randn_bf16(g, (m, k))
        y = host(ops.fp8_block128_gemv_t16(dev_bf16(x), wt, dev(s), n))
        ref = oracle.fp8_block_gemv(x, w8, s)
        assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(y, ref) < 1e-5, (n, k, m)
        # a row's value does not depend on the rows beside it
        if m > 1:
            assert np.array_equal(host(ops.fp8_block128_gemv_t16(dev_bf16(x[:1].copy()), wt, dev(s), n))[0], y[0])
        # the row-major call with the same split of K over the waves (four chunks a wave) runs the same arithmetic (its kernel
        # brings a chunk into this order through LDS): the same bits; with its own split the sums differ in their order only
        if 3 <= m <= 8 and k % 256 == 0:
            assert rel_l2(host(ops.fp8_block128_gemv(dev_bf16(x), dev(w8), dev(s))), y) < 1e-6
            ops._lib().spark_debug_rm_span(4)
            try:
                assert np.array_equal(host(ops.fp8_block128_gemv(dev_bf16(x), dev(w8), dev(s))), y)
            finally:
                ops._lib().spark_debug_rm_span(0)
    # shapes outside the layout are refused, not launched
    lib = ops._lib()
    assert lib.spark_fp8_block128_gemv_t16(ops._p(dev_bf16(x)), ops._p(wt), ops._p(dev(s)), ops._p(dev(np.zeros((1, n), np.float32))), 17, n, k, ops._st()) == 1
    assert lib.spark_fp8_block128_gemv_t16(ops._p(dev_bf16(x)), ops._p(wt), ops._p(dev(s)), ops._p(dev(np.zeros((1, n), np.float32))), 1, n, 128 * 65, ops._st()) == 1
    assert lib.spark_fp8_t16_pack(ops._p(wt), ops._p(wt), n + 8, k, ops._st()) == 1


@pytest.mark.parametrize("m", [1, 4])
def test_fp8_gemvs(ops, oracle, m):
    g = synth.rng(140 + m)
    n, k = 384, 1024
    w8, s = synth.fp8_block_matrix(g, n, k)
    x = synth.randn_bf16(g, (m, k))
    y = host(ops.fp8_block128_gemv(dev_bf16(x), dev(w8), dev(s)))
    ref = oracle.fp8_block_gemv(x, w8, s)
    assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(y, ref) < 1e-5
    s8 = g.integers(110, 128, (n // 32, k // 32), dtype=np.uint8)
    y = host(ops.fp8_gemv(dev_bf16(x), dev(w8), dev(s8)))
    ref = oracle.fp8_e8m0_gemv(x, w8, s8)
    assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(y, ref) < 1e-5
    wb = synth.randn_bf16(g, (n, k))
    y = host(ops.bf16_gemv(dev_bf16(x), dev_bf16(wb)))
    ref = synth.bf16_to_f32(x).astype(np.float64) @ synth.bf16_to_f32(wb).astype(np.float64).T
    assert rel_l2(y, ref) < 1e-5


@pytest.mark.parametrize("m,n,k", [(3, 208, 1536), (5, 64, 512), (8, 128, 4096), (4, 7168, 4096), (6, 96, 1280), (8, 64, 768), (3, 48, 256)])
def test_matrix_unit_gemvs(ops, oracle, m, n, k):
    # three or more rows of an eligible shape (k % 512 == 0, n % 16 == 0) run on the matrix unit in all three formats; the E8M0
    # scales span 50 binades inside a K block (they are applied relative to the block's largest)
    g = synth.rng(160 + m)
    x = synth.randn_bf16(g, (m, k))
    w4, s4 = synth.mxfp4_matrix(g, n, k, 119)
    s4 = g.integers(80, 131, s4.shape, dtype=np.uint8)
    y = host(ops.mxfp4_gemv(dev_bf16(x), dev(w4), dev(s4)))
    ref = oracle.mxfp4_gemv(x, w4, s4)
    assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(y, ref) < 1e-5
    w8, sb = synth.fp8_block_matrix(g, n, k)
    y = host(ops.fp8_block128_gemv(dev_bf16(x), dev(w8), dev(sb)))
    ref = oracle.fp8_block_gemv(x, w8, sb)
    assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(y, ref) < 1e-5
    s8 = g.integers(80, 131, ((n + 31) // 32, k // 32), dtype=np.uint8)
    y = host(ops.fp8_gemv(dev_bf16(x), dev(w8), dev(s8)))
    ref = oracle.fp8_e8m0_gemv(x, w8, s8)
    assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(y, ref) < 1e-5
    # a row's value does not depend on the other rows of a call within a kernel family (up to four rows / five to eight)
    sub = 3 if m == 4 else 5 if m > 5 else 0
    if sub:
        ys = host(ops.fp8_gemv(dev_bf16(x[:sub]), dev(w8), dev(s8)))
        assert np.array_equal(ys, y[:sub])


@pytest.mark.parametrize("n,k", [(384, 5120), (512, 2048), (100, 1032), (288, 4096), (3000, 1024)])
def test_bf16_gemv_matrices_of_few_rows(ops, n, k):
    """Router-logit sized matrices: a workgroup per row, K split over its waves (every wave count from two to eight, a ragged last piece)."""
    g = synth.rng(1530 + n)
    wb = synth.randn_bf16(g, (n, k))
    x = synth.randn_bf16(g, (8, k))
    ref = synth.bf16_to_f32(x).astype(np.float64) @ synth.bf16_to_f32(wb).astype(np.float64).T
    y8 = host(ops.bf16_gemv(dev_bf16(x), dev_bf16(wb)))
    assert rel_l2(y8, ref) < 1e-5
    for m in (1, 2, 3, 5):
        y = host(ops.bf16_gemv(dev_bf16(x[:m].copy()), dev_bf16(wb)))
        assert np.array_equal(y, y8[:m])                                  # a row's value does not depend on the row count


def test_bf16_gemv_up_to_16_rows(ops):
    # ds41_bf16_gemv_mx: the rows of ds41_bf16_gemv, eight at a time
    g = synth.rng(149)
    n, k = 384, 5120
    wb = synth.randn_bf16(g, (n, k))
    x = synth.randn_bf16(g, (13, k))
    y = host(ops.bf16_gemv_rows(dev_bf16(x), dev_bf16(wb)))
    ref = synth.bf16_to_f32(x).astype(np.float64) @ synth.bf16_to_f32(wb).astype(np.float64).T
    assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5
    assert np.array_equal(y[:8], host(ops.bf16_gemv(dev_bf16(x[:8]), dev_bf16(wb))))
    assert np.array_equal(y[8:], host(ops.bf16_gemv(dev_bf16(x[8:]), dev_bf16(wb))))
    assert ops._lib().ds41_bf16_gemv_mx(ops._p(dev_bf16(x)), ops._p(dev_bf16(wb)), ops._p(dev(np.zeros((17, n), np.float32))), 17, n, k, ops._st()) == 1


def test_bf16_gemv_tall_matrix_rows(ops):
    # three or more rows of a tall matrix take the row-tile kernel, four rows per launch
    g = synth.rng(170)
    n, k, m = 8192, 1024, 7
    wb = synth.randn_bf16(g, (n, k))
    x = synth.randn_bf16(g, (m, k))
    y = host(ops.bf16_gemv(dev_bf16(x), dev_bf16(wb)))
    ref = synth.bf16_to_f32(x).astype(np.float64) @ synth.bf16_to_f32(wb).astype(np.float64).T
    assert rel_l2(y, ref) < 1e-5
    y3 = host(ops.bf16_gemv(dev_bf16(x[:3]), dev_bf16(wb)))
    assert np.array_equal(y3, y[:3])


def test_fp8_gemv_bx_up_to_16_rows_and_groups(ops, oracle):
    g = synth.rng(150)
    n, k, m = 256, 512, 13
    w8, _ = synth.fp8_block_matrix(g, n, k)
    s8 = g.integers(110, 128, (n // 32, k // 32), dtype=np.uint8)
    x = synth.randn_bf16(g, (m, k))
    y = host(ops.fp8_gemv_bx(dev_bf16(x), dev(w8), dev(s8)))
    ref = oracle.fp8_e8m0_gemv(x, w8, s8)
    assert rel_l2(y, ref) < 1e-5
    y8 = host(ops.fp8_gemv(dev_bf16(x[:8]), dev(w8), dev(s8)))
    assert np.array_equal(y[:8], y8)                                   # a row's value does not depend on the row count
    # block-diagonal: weight rows [64 j, 64 j + 64) read input elements [j k, (j + 1) k) of their row
    groups = n // 64
    xg = synth.randn_bf16(g, (3, groups * k))
    yg = host(ops.fp8_gemv_bx(dev_bf16(xg), dev(w8), dev(s8), rpg=64))
    for j in range(groups):
        refj = oracle.fp8_e8m0_gemv(np.ascontiguousarray(xg[:, j * k:(j + 1) * k]), w8, s8)[:, 64 * j:64 * j + 64]
        assert rel_l2(yg[:, 64 * j:64 * j + 64], refj) < 1e-5


@pytest.mark.parametrize("n,k,m", [(256, 1024, 11), (208, 2048, 21), (64, 4096, 3), (7168, 4096, 16), (160, 1280, 5), (128, 3072, 9), (1280, 5120, 3), (96, 768, 4),
                                   (64, 1152, 4), (200, 1024, 5), (8, 256, 2)])
def test_fp8_gemv_with_quantised_activations(ops, oracle, n, k, m):
    # FP8 weights x act-quantised activations: every product is exact, the reference is the same sum in float64.  K in whole
    # 256-wide chunks runs on the matrix unit with the activations staged as exact bf16 (the reference model's 1280 / 3072 / 5120
    # among them; a last tile of 8 rows too), (64, 1152) on the dot-product kernel.  The threshold is the reference's own for this
    # product (kern.rs:1863-1867, 1908-1912): max |diff| / max |ref| < 1e-5.
    g = synth.rng(151)
    w8, _ = synth.fp8_block_matrix(g, n, k)
    s8 = g.integers(110, 128, ((n + 31) // 32, k // 32), dtype=np.uint8)
    x = synth.randn_bf16(g, (m, k))
    q, s = oracle.act_quant_fp8(x)
    W = oracle.fp8_e8m0_dequant(w8, s8).astype(np.float64)
    codes = torch.from_numpy(q.copy()).view(torch.float8_e4m3fn).to(torch.float64).numpy()          # library decode of E4M3
    xq = codes * np.exp2(s.astype(np.float64) - 127.0).repeat(32, axis=1)
    ref = xq @ W.T
    close = lambda got: np.abs(got - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(got, ref) < 1e-6
    given = lambda rows=slice(None), **kw: host(ops.fp8_gemv_mx(None, dev(w8), dev(s8), aq=dev(q[rows].copy()), as_=dev(s[rows].copy()), **kw))
    y2 = given()
    assert close(y2)
    r = min(2, m - 1)
    assert np.array_equal(given(bf16_out=True), synth.bf16_bits(y2))
    assert np.array_equal(given(slice(r, r + 1))[0], y2[r])                     # a row's value does not depend on the row count
    # the other kernel family (switched by the diagnostics call): the same products, the binary32 sums in another order
    ops._lib().spark_debug_fp8q_rowmajor(0)
    try:
        yd = given()
        assert close(yd) and rel_l2(yd, y2) <= 1e-6
        assert np.array_equal(given(slice(r, r + 1))[0], yd[r])
        if m <= 16:
            assert np.array_equal(host(ops.fp8_gemv_mx(dev_bf16(x), dev(w8), dev(s8))), yd)       # quantised inside = quantised by the caller
    finally:
        ops._lib().spark_debug_fp8q_rowmajor(1)
    # bf16 rows handed over are quantised by the kernel itself (the same codes): the bits of the codes-given call, at any row count
    if m <= 16:
        y = host(ops.fp8_gemv_mx(dev_bf16(x), dev(w8), dev(s8)))
        assert np.array_equal(y, y2)
        assert np.array_equal(host(ops.fp8_gemv_mx(dev_bf16(x), dev(w8), dev(s8), bf16_out=True)), synth.bf16_bits(y))
    y1 = host(ops.fp8_gemv_mx(dev_bf16(x[r:r + 1]), dev(w8), dev(s8)))
    assert np.array_equal(y1[0], y2[r])


def test_fp8_gemv_mx_row_does_not_depend_on_the_other_rows(ops, oracle):
    """The reference's own sweep (kern.rs:1885-1898): every (n, k) its ranks use, the caller's rule for who quantises (kern.rs:899-917);
    row 0 of a 2- and a 5-row call carries the bits of the one-row call.  The smallest n of every k is checked against the oracle."""
    gen = torch.Generator(device=DEV).manual_seed(77)
    for n in (512, 1024, 1536, 1792, 2048, 3072, 4096, 5120, 8192, 8536, 12288, 25600):
        for k in (512, 768, 1024, 1280, 2048, 3072, 4096, 5120, 6144, 15360):
            w = torch.randint(0, 120, (n, k), dtype=torch.uint8, device=DEV, generator=gen)
            s = torch.randint(100, 130, ((n + 31) // 32, k // 32), dtype=torch.uint8, device=DEV, generator=gen)
            x1 = torch.randn(1, k, device=DEV, generator=gen).to(torch.bfloat16)
            r1 = ops.gemv_mx(x1, w, s)
            for m in (2, 5):
                ym = ops.gemv_mx(x1.expand(m, k).contiguous(), w, s)
                assert torch.equal(ym[:1], r1), (n, k, m)
                assert torch.equal(ym[m - 1:], r1), (n, k, m)
            assert torch.equal(ops.gemv_mx(x1, w, s, bf16_out=True), r1.to(torch.bfloat16)), (n, k)
            if n == 512:
                xb = host(x1.view(torch.int16)).view(np.uint16)
                q, sq = oracle.act_quant_fp8(xb)
                W = oracle.fp8_e8m0_dequant(host(w), host(s)).astype(np.float64)
                codes = torch.from_numpy(q.copy()).view(torch.float8_e4m3fn).to(torch.float64).numpy()
                ref = (codes * np.exp2(sq.astype(np.float64) - 127.0).repeat(32, axis=1)) @ W.T
                assert np.abs(host(r1) - ref).max() / np.abs(ref).max() < 1e-5, (n, k)          # the reference's threshold (kern.rs:1863-1867)
            del w, s


@pytest.mark.parametrize("k", [15360, 15424, 20480])
def test_gemvs_of_long_rows(ops, oracle, k):
    """K beyond what a workgroup stages at once (the reference's kernels stage nothing: no limit on K; its largest is the
    15360 of mtp main_proj, kern.rs:1330): every dense GEMV at its largest row count, against the oracle."""
    g = synth.rng(4100 + k)
    n = 96
    w8, sb = synth.fp8_block_matrix(g, n, k)
    s8 = g.integers(110, 128, (n // 32, k // 32), dtype=np.uint8)
    x = synth.randn_bf16(g, (16, k))
    for m in (1, 3, 8):
        y = host(ops.fp8_gemv(dev_bf16(x[:m]), dev(w8), dev(s8)))
        ref = oracle.fp8_e8m0_gemv(x[:m], w8, s8)
        assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(y, ref) < 1e-5, (k, m)
        y = host(ops.fp8_block128_gemv(dev_bf16(x[:m]), dev(w8), dev(sb)))
        ref = oracle.fp8_block_gemv(x[:m], w8, sb)
        assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(y, ref) < 1e-5, (k, m)
    y = host(ops.fp8_gemv_bx(dev_bf16(x), dev(w8), dev(s8)))
    assert rel_l2(y, oracle.fp8_e8m0_gemv(x, w8, s8)) < 1e-5
    w4, s4 = synth.mxfp4_matrix(g, n, k, 119)
    y = host(ops.mxfp4_gemv(dev_bf16(x[:8]), dev(w4), dev(s4)))
    assert rel_l2(y, oracle.mxfp4_gemv(x[:8], w4, s4)) < 1e-5
    wb = synth.randn_bf16(g, (n, k))
    y = host(ops.bf16_gemv(dev_bf16(x[:8]), dev_bf16(wb)))
    assert rel_l2(y, synth.bf16_to_f32(x[:8]).astype(np.float64) @ synth.bf16_to_f32(wb).astype(np.float64).T) < 1e-5
    # act-quantised activations: codes given at 32 rows, bf16 rows quantised inside at 8
    x32 = synth.randn_bf16(g, (32, k))
    q, sq = oracle.act_quant_fp8(x32)
    W = oracle.fp8_e8m0_dequant(w8, s8).astype(np.float64)
    codes = torch.from_numpy(q.copy()).view(torch.float8_e4m3fn).to(torch.float64).numpy()
    ref = (codes * np.exp2(sq.astype(np.float64) - 127.0).repeat(32, axis=1)) @ W.T
    y = host(ops.fp8_gemv_mx(None, dev(w8), dev(s8), aq=dev(q), as_=dev(sq)))
    assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5
    y = host(ops.fp8_gemv_mx(dev_bf16(x32[:8]), dev(w8), dev(s8)))
    assert np.abs(y - ref[:8]).max() / np.abs(ref).max() < 1e-5


@pytest.mark.parametrize("n,k,rpg,ms", [(3072, 4096, 1024, (1, 2, 4, 8, 16)), (160, 512, 64, (2, 5)), (96, 15360, 32, (3,)), (200, 1088, 96, (1, 4))])
def test_fp8_gemv_bx_block_diagonal_shapes(ops, oracle, n, k, rpg, ms):
    """wo_a's block-diagonal projection (kern.rs:165-180; three groups of 1024 x 4096 a rank in the reference's benchmark, kern.rs:1396-1421),
    a last group of fewer rows, a long K and a shape outside the matrix-unit kernel's grid: group t of rpg weight rows reads the
    inputs [t k, +k) of its row."""
    g = synth.rng(4200 + n)
    w8, _ = synth.fp8_block_matrix(g, n, k)
    s8 = g.integers(110, 128, ((n + 31) // 32, k // 32), dtype=np.uint8)
    groups = (n + rpg - 1) // rpg
    for m in ms:
        xg = synth.randn_bf16(g, (m, groups * k))
        y = host(ops.fp8_gemv_bx(dev_bf16(xg), dev(w8), dev(s8), rpg=rpg))
        for t in range(groups):
            r0, r1 = t * rpg, min(n, (t + 1) * rpg)
            ref = oracle.fp8_e8m0_gemv(np.ascontiguousarray(xg[:, t * k:(t + 1) * k]), w8, s8)[:, r0:r1]
            assert rel_l2(y[:, r0:r1], ref) < 1e-5, (m, t)


@pytest.mark.parametrize("n,k,ms", [(32, 128, (1, 16)), (96, 1152, (1, 2, 3, 5, 16)), (384, 1024, (1, 4, 8)), (160, 8192, (4, 9)), (12288, 1280, (2,))])
def test_fp8_e8m0_gemv_on_packed_weights(ops, oracle, n, k, ms):
    """ds41_fp8_gemv's product (E8M0 scales per 32 x 32, bf16 activations) on the packed matrix, against the oracle and the row-major call."""
    g = synth.rng(1540 + n + k)
    w8, _ = synth.fp8_block_matrix(g, n, k)
    s8 = g.integers(110, 128, (n // 32, k // 32), dtype=np.uint8)
    wt = ops.fp8_t16_pack(dev(w8))
    for m in ms:
        x = synth.randn_bf16(g, (m, k))
        y = host(ops.fp8_e8m0_gemv_t16(dev_bf16(x), wt, dev(s8), n))
        ref = oracle.fp8_e8m0_gemv(x, w8, s8)
        assert np.abs(y - ref).max() / np.abs(ref).max() < 1e-5 and rel_l2(y, ref) < 1e-5, (n, k, m)
        if m <= 8:
            assert rel_l2(y, host(ops.fp8_gemv(dev_bf16(x), dev(w8), dev(s8)))) < 1e-6                 # the row-major call: the same products, another order of the sums
        if m > 1:
            assert np.array_equal(host(ops.fp8_e8m0_gemv_t16(dev_bf16(x[:1].copy()), wt, dev(s8), n))[0], y[0])


def test_gemv_rejects_bad_shapes(ops):
    x = torch.zeros(9, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(8, 32, dtype=torch.uint8, device=DEV)
    s = torch.zeros(8, 2, dtype=torch.uint8, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.mxfp4_gemv(x, w, s)                                       # m > 8 -> return code 1 (reference ds41.cu:230)


# ---------------------------------------------------------------- shared-expert glue (reference ds41_ops.cu:421-442,615; qwen_moe.cu:69-84,101-110)

@pytest.mark.parametrize("T,I,lim", [(1, 2048, 10.0), (5, 768, 10.0), (3, 256, 0.0), (2, 32, 7.0)])
def test_swiglu_quant_bit_exact(ops, oracle, T, I, lim):
    from tests.gpu_util import bf16_safe
    g = synth.rng(280 + T)
    gu = (g.standard_normal((T, 2 * I)) * 10.0 ** g.uniform(-2, 1.5, (T, 1))).astype(np.float32)
    gu[0, :4] = [3.0, -20.0, 40.0, 11.0]; gu[0, I:I + 4] = [0.5, 40.0, -40.0, 2.0]
    got = host(ops.swiglu_quant(dev(gu), lim))
    ref = oracle.swiglu_quant(gu, lim)
    # The bytes must be the oracle's.  The one licence: the GPU's and the host's exponential may differ in the last place, which
    # can move a product that sits on a bf16 rounding boundary; blocks that hold such a value are compared to one step instead.
    gb = torch.from_numpy(gu[:, :I]).to(torch.bfloat16).double(); ub = torch.from_numpy(gu[:, I:]).to(torch.bfloat16).double()
    if lim > 0:
        gb = gb.clamp(max=lim); ub = ub.clamp(min=-lim, max=lim)
    safe = bf16_safe((gb / (1.0 + torch.exp(-gb)) * ub).numpy()).reshape(T, I // 32, 32).all(-1)
    eq = (got == ref).reshape(T, I // 32, 32).all(-1)
    assert safe.mean() > 0.85 and eq[safe].all(), np.argwhere(safe & ~eq)[:4]
    d = np.abs(synth.bf16_to_f32(got) - synth.bf16_to_f32(ref)).reshape(T, I // 32, 32)
    top = np.abs(synth.bf16_to_f32(ref)).reshape(T, I // 32, 32).max(-1, keepdims=True)
    assert (d <= 2.0 ** -3 * top + 1e-30).all()
    # an unaligned output (odd element offset is refused, a 4-byte aligned one takes the narrow stores) gives the same bytes
    big = torch.zeros(T * I + 2, dtype=torch.bfloat16, device=DEV)
    L = ops._lib()
    assert L.ds41_swiglu_quant(dev(gu).data_ptr(), big[2:].data_ptr(), T, I, float(lim), ops._st()) == 0
    torch.cuda.synchronize()
    assert np.array_equal(host(big[2:]).reshape(T, I), got)
    assert L.ds41_swiglu_quant(dev(gu).data_ptr(), big.data_ptr(), 0, I, float(lim), ops._st()) == 0      # no rows: nothing to do (reference :616)
    assert L.ds41_swiglu_quant(dev(gu).data_ptr(), big.data_ptr(), T, 48, float(lim), ops._st()) == 1     # I not whole 32-blocks (reference :617)


def _ulps(a, b):
    ia = a.view(np.int32).astype(np.int64); ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7fffffff), ia); ib = np.where(ib < 0, -(ib & 0x7fffffff), ib)
    return np.abs(ia - ib)


@pytest.mark.parametrize("n", [1, 3, 640, 2563, 10240])
def test_silu_mul_last_places(ops, oracle, n):
    g = synth.rng(290 + n)
    gv = (g.standard_normal(n) * 10.0 ** g.uniform(-3, 1.3, n)).astype(np.float32)
    uv = g.standard_normal(n).astype(np.float32)
    ref = oracle.silu_mul(gv, uv)
    got = host(ops.silu_mul(dev(gv), dev(uv)))
    # the device's and the host's exponential differ by up to two units in the last place; one division and one product carry that on
    assert _ulps(got, ref).max() <= 4, _ulps(got, ref).max()
    true = gv.astype(np.float64) / (1.0 + np.exp(-gv.astype(np.float64))) * uv.astype(np.float64)
    assert np.all(np.abs(got - true) <= 6e-7 * np.abs(true) + 1e-38)
    # arrays that do not start on 16 bytes take the element-wise form: same values
    gp = torch.zeros(n + 1, device=DEV); up = torch.zeros(n + 1, device=DEV)
    gp[1:] = dev(gv); up[1:] = dev(uv)
    assert np.array_equal(host(ops.silu_mul(gp[1:], up[1:])), got)


@pytest.mark.parametrize("R,N,ldg,col", [(1, 2560, 513, 512), (4, 2560, 513, 512), (3, 130, 7, 2), (2, 8, 1, 0)])
def test_gate_scale_last_places(ops, oracle, R, N, ldg, col):
    g = synth.rng(295 + R + N)
    gl = (g.standard_normal((R, ldg)) * 4).astype(np.float32)
    d = g.standard_normal((R, N)).astype(np.float32)
    ref = oracle.gate_scale(gl, col, d)
    got = host(ops.gate_scale(dev(gl), col, dev(d)))
    assert _ulps(got, ref).max() <= 4, _ulps(got, ref).max()
    true = (1.0 / (1.0 + np.exp(-gl[:, col].astype(np.float64))))[:, None] * d.astype(np.float64)
    assert np.all(np.abs(got - true) <= 6e-7 * np.abs(true))
