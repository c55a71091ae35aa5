"""GPU parity of the routed MXFP4 experts against the CPU oracle (dequantise + FP32 matmul with the reference's
roundings).  Tolerance: rel-L2 <= 1e-3 on the FP32 output (reference kern.rs:2206-2208)."""
import numpy as np
import pytest
import torch

from spark_engine_amd import synth
from tests.gpu_util import DEV, dev, dev_bf16, host, rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def ops():
    from spark_engine_amd import ops
    return ops


def _case(g, R, H, I, E, topk, n_shared, smin=117):
    ws = synth.mxfp4_experts(g, E + n_shared, H, I, smin)
    x = synth.randn_bf16(g, (R, H))
    idx = np.stack([g.permutation(E)[:topk] for _ in range(R)]).astype(np.int64)
    rw = g.uniform(0.1, 1.0, (R, topk)).astype(np.float32)
    rw = (rw / rw.sum(-1, keepdims=True) * 1.5).astype(np.float32)
    return ws, x, idx, rw


@pytest.mark.parametrize("R,H,I,E,topk,ns", [(1, 512, 256, 8, 2, 0), (1, 1024, 512, 12, 6, 1), (4, 512, 384, 6, 3, 1), (3, 640, 128, 5, 2, 2)])
def test_moe_small_vs_oracle(ops, oracle, R, H, I, E, topk, ns):
    g = synth.rng(200 + R + H)
    ws, x, idx, rw = _case(g, R, H, I, E, topk, ns)
    add = g.standard_normal((R, H)).astype(np.float32)
    ex = ops.Mxfp4Experts(*[dev(a) for a in ws], n_shared=ns, keep_natural=True)
    ref = oracle.mxfp4_moe(x, idx, rw, *ws, n_shared=ns, add=add)
    y = host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ex, add=dev(add)))
    assert rel_l2(y, ref) <= TOL, rel_l2(y, ref)
    y2 = host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ex, add=dev(add), natural=True))
    assert np.array_equal(y, y2)                                     # the record layout changes bytes in memory, not results
    y3 = host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ex, add=dev(add)))
    assert np.array_equal(y, y3)                                     # deterministic


def test_moe_rows_sharing_experts_and_row_invariance(ops, oracle):
    g = synth.rng(210)
    R, H, I, E, topk = 4, 512, 256, 4, 2
    ws, x, idx, rw = _case(g, R, H, I, E, topk, 0)
    idx[:] = [[0, 1], [1, 0], [0, 3], [1, 2]]                        # experts shared by several rows
    ex = ops.Mxfp4Experts(*[dev(a) for a in ws])
    y = host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ex))
    assert rel_l2(y, oracle.mxfp4_moe(x, idx, rw, *ws)) <= TOL
    for r in range(R):                                                # a row's bits do not depend on the other rows
        yr = host(ops.mxfp4_moe(dev_bf16(x[r:r + 1]), dev(idx[r:r + 1]), dev(rw[r:r + 1]), ex))
        assert np.array_equal(yr[0], y[r])


def test_moe_zero_codes_give_add(ops):
    g = synth.rng(211)
    R, H, I, E, topk = 2, 512, 256, 3, 2
    ws, x, idx, rw = _case(g, R, H, I, E, topk, 0)
    ws = [np.zeros_like(a) if i % 2 == 0 else a for i, a in enumerate(ws)]
    add = g.standard_normal((R, H)).astype(np.float32)
    ex = ops.Mxfp4Experts(*[dev(a) for a in ws])
    assert np.array_equal(host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ex, add=dev(add))), add)


@pytest.mark.parametrize("R,H,I,E,topk,ns", [(1, 1024, 512, 12, 6, 1), (2, 512, 384, 6, 3, 1), (4, 1024, 256, 5, 2, 2), (8, 512, 256, 4, 2, 0),
                                             # nine and ten 512-wide K groups for the eight waves of a gate / up block (ten: the reference's
                                             # hidden width), a ragged last group, and more K groups than the balanced split covers
                                             (1, 5120, 256, 6, 3, 1), (4, 4608, 128, 5, 2, 0), (2, 4224, 128, 4, 2, 1), (3, 5120, 128, 4, 2, 0),
                                             (2, 6144, 128, 4, 2, 0)])
def test_single_launch_equals_several_kernel_path_bitwise(ops, oracle, R, H, I, E, topk, ns):
    # the decode entry runs the whole layer as one launch with the same summation orders as the several-kernel path;
    # a prepared workspace is reused call after call (the exchanged words clear themselves)
    g = synth.rng(230 + R)
    ws, x, idx, rw = _case(g, R, H, I, E, topk, ns)
    ex = ops.Mxfp4Experts(*[dev(a) for a in ws], n_shared=ns)
    wsd = ops.mxfp4_moe_ws_alloc(R, ex, topk)
    for it in range(3):
        x = synth.randn_bf16(g, (R, H))
        idx = np.stack([g.permutation(E)[:topk] for _ in range(R)]).astype(np.int64)
        add = g.standard_normal((R, H)).astype(np.float32)
        ref = oracle.mxfp4_moe(x, idx, rw, *ws, n_shared=ns, add=add)
        one = host(ops.mxfp4_moe_x(dev_bf16(x), dev(idx), dev(rw), ex, add=dev(add), ws=wsd, ws_clean=True))
        assert rel_l2(one, ref) <= TOL, rel_l2(one, ref)
        xq, xs = ops.act_quant_fp8(dev_bf16(x))
        several = host(ops.mxfp4_moe_x(xq, dev(idx), dev(rw), ex, xs=xs, add=dev(add), multi_kernel=True))
        assert np.array_equal(one, several)
        given = host(ops.mxfp4_moe_x(xq, dev(idx), dev(rw), ex, xs=xs, add=dev(add), ws=wsd, ws_clean=True))   # activations quantised by the caller
        assert np.array_equal(one, given)
    assert int(wsd.view(torch.int32)[0].item()) == 0                  # no wait expired


@pytest.mark.parametrize("R,multi", [(1, False), (4, False), (8, False), (4, True)])
def test_moe_bf16_output_is_the_rounded_f32_output(ops, oracle, R, multi):
    # the reference's decode graphs add the experts' result into a bf16 hidden state (engine-rs/src/ds41/kern.rs:1439-1445): with the
    # bf16-output flag the single-launch and the several-kernel paths store round-to-nearest-even of what they store in binary32
    g = synth.rng(240 + R)
    H, I, E, topk, ns = 1024, 512, 6, 2, 1
    ws, x, idx, rw = _case(g, R, H, I, E, topk, ns)
    ex = ops.Mxfp4Experts(*[dev(a) for a in ws], n_shared=ns)
    add = dev(g.standard_normal((R, H)).astype(np.float32))
    xd, xs = dev_bf16(x), None
    if multi:
        xd, xs = ops.act_quant_fp8(xd)
    f32 = ops.mxfp4_moe_x(xd, dev(idx), dev(rw), ex, xs=xs, add=add, multi_kernel=multi)
    b16 = ops.mxfp4_moe_x(xd, dev(idx), dev(rw), ex, xs=xs, add=add, multi_kernel=multi, out_bf16=True)
    assert b16.dtype == torch.bfloat16 and b16.shape == (R, H)
    assert torch.equal(b16, f32.to(torch.bfloat16))


def test_moe_many_rows_multi_column_groups(ops, oracle):
    # more than 16 rows on one expert: several MFMA column groups per item, items of 64 rows
    g = synth.rng(212)
    R, H, I, E, topk = 70, 1024, 512, 3, 2
    ws, x, idx, rw = _case(g, R, H, I, E, topk, 0)
    ex = ops.Mxfp4Experts(*[dev(a) for a in ws])
    y = host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ex))
    assert rel_l2(y, oracle.mxfp4_moe(x, idx, rw, *ws)) <= TOL


# the last three: a ragged last K group in the down product (I = 768, 640) and in both products (H = 1280: two and a half K groups)
@pytest.mark.parametrize("R,H,I", [(45, 2048, 1024), (45, 5120, 512), (45, 6144, 512), (12, 1024, 512), (9, 5120, 512), (45, 2048, 768),
                                   (12, 1280, 640), (40, 4352, 1920),
                                   # more K groups in the down product than its four waves along K: 2304 is the reference's whole intermediate width
                                   (20, 1024, 2304), (12, 512, 4096)])
def test_grouped_gemm_rows_equal_decode_rows_bitwise(ops, oracle, R, H, I):
    # more than 8 rows run as a grouped GEMM over 32-row items: a shared expert (every row), ragged tails, several K groups (more than
    # the eight waves of a decode block at the wider shapes); every row must come out with the bits the single-launch decode path
    # gives the row alone
    g = synth.rng(213)
    E, topk, ns = 5, 2, 1
    ws, x, idx, rw = _case(g, R, H, I, E, topk, ns)
    ex = ops.Mxfp4Experts(*[dev(a) for a in ws], n_shared=ns)
    xd, idxd, rwd = dev_bf16(x), dev(idx), dev(rw)
    add = g.standard_normal((R, H)).astype(np.float32)
    y = host(ops.mxfp4_moe(xd, idxd, rwd, ex, add=dev(add)))
    assert rel_l2(y, oracle.mxfp4_moe(x, idx, rw, *ws, n_shared=ns, add=add)) <= TOL
    for r in sorted({0, 17 % R, 31 % R, 32 % R, R - 1}):
        one = host(ops.mxfp4_moe_x(xd[r:r + 1], idxd[r:r + 1], rwd[r:r + 1], ex, add=dev(add[r:r + 1])))
        assert np.array_equal(one[0], y[r]), r


def test_one_prepared_workspace_serves_calls_of_every_size(ops, oracle):
    g = synth.rng(214)
    H, I, E, topk, ns = 1024, 512, 6, 2, 1
    ws, _, _, _ = _case(g, 1, H, I, E, topk, ns)
    ex = ops.Mxfp4Experts(*[dev(a) for a in ws], n_shared=ns)
    wsd = ops.mxfp4_moe_ws_alloc(40, ex, topk)

    def call(R, seed):
        gg = synth.rng(seed)
        x = synth.randn_bf16(gg, (R, H))
        idx = np.stack([gg.permutation(E)[:topk] for _ in range(R)]).astype(np.int64)
        rw = gg.uniform(0.1, 1.0, (R, topk)).astype(np.float32)
        if R <= 8:
            y = host(ops.mxfp4_moe_x(dev_bf16(x), dev(idx), dev(rw), ex, ws=wsd, ws_clean=True))
        else:
            y = host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ex, ws=wsd))
        assert rel_l2(y, oracle.mxfp4_moe(x, idx, rw, *ws, n_shared=ns)) <= TOL, R
        return y
    first = call(1, 1)
    for R in (4, 12, 40, 8):
        call(R, 20 + R)
    assert np.array_equal(call(1, 1), first)
    assert int(wsd.view(torch.int32)[0].item()) == 0                  # no wait expired


def test_ds41_reference_symbols_tile_layouts(ops, oracle):
    # the reference's own entry points: hidden 5120, weights repacked as kern.rs moe_pack / moe_pack_mx do
    g = synth.rng(213)
    R, H, I, E, topk = 2, 5120, 128, 4, 2
    ws, x, idx, rw = _case(g, R, H, I, E, topk, 0, smin=119)
    add = g.standard_normal((R, H)).astype(np.float32)
    ref = oracle.mxfp4_moe(x, idx, rw, *ws, add=add)
    d = [dev(a) for a in ws]
    p1, ps1 = ops.moe_pack(d[0], d[1]); p3, ps3 = ops.moe_pack(d[2], d[3]); p2, ps2 = ops.moe_pack(d[4], d[5])
    xq, xs = ops.act_quant_fp8(dev_bf16(x))
    y, wsb = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), (ops.moe_pack_mx(p1), ps1, ops.moe_pack_mx(p3), ps3, ops.moe_pack_mx(p2), ps2), I, add=dev(add))
    assert rel_l2(host(y), ref) <= TOL
    xdq = ops.act_quant(dev_bf16(x))
    y2 = ops.ds41_moe(xdq, dev(idx), dev(rw), (p1, ps1, p3, ps3, p2, ps2), I, add=dev(add))
    assert np.array_equal(host(y2), host(y))                          # same operands, same instruction sequence
    # skip_combine + combine_rows leave the same rows behind (reference ds41_mx.cu:1471-1487)
    from spark_engine_amd import lib
    import ctypes as C
    L = lib.load()
    y3, wsb3 = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), (ops.moe_pack_mx(p1), ps1, ops.moe_pack_mx(p3), ps3, ops.moe_pack_mx(p2), ps2), I, add=dev(add), skip_combine=True)
    y4 = torch.zeros(R, H, dtype=torch.float32, device=DEV)
    add_d = dev(add)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for r0 in range(R):
        assert L.ds41_moe_mx_combine_rows(C.c_void_p(wsb3.data_ptr()), R, I, topk, E, C.c_void_p(add_d.data_ptr()), C.c_void_p(y4.data_ptr()), r0, 1, st) == 0
    torch.cuda.synchronize()
    assert np.array_equal(host(y4), host(y))


# the reference symbols are compiled for hidden width 5120; 768 is the reference's intermediate width per rank (2304 over three
# ranks, engine-rs/src/ds41/kern.rs:2179-2190): one and a half K groups in the down product
@pytest.mark.parametrize("H,I", [(5120, 512), (5120, 1024), (5120, 768), (5120, 2304)])
def test_ds41_reference_symbols_prefill_sizes(ops, oracle, H, I):
    # more than 16 rows: the reference's tile layouts go through the grouped GEMM too (their 8-row tiles are read in place), and a
    # row's bits are those of the record layout's grouped GEMM and of the decode path
    g = synth.rng(215)
    R, E, topk = 45, 5, 2
    ws, x, idx, rw = _case(g, R, H, I, E, topk, 0, smin=119)
    add = g.standard_normal((R, H)).astype(np.float32)
    ref = oracle.mxfp4_moe(x, idx, rw, *ws, add=add)
    d = [dev(a) for a in ws]
    p1, ps1 = ops.moe_pack(d[0], d[1]); p3, ps3 = ops.moe_pack(d[2], d[3]); p2, ps2 = ops.moe_pack(d[4], d[5])
    xq, xs = ops.act_quant_fp8(dev_bf16(x))
    y_mx, _ = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), (ops.moe_pack_mx(p1), ps1, ops.moe_pack_mx(p3), ps3, ops.moe_pack_mx(p2), ps2), I, add=dev(add))
    assert rel_l2(host(y_mx), ref) <= TOL
    y_p8 = ops.ds41_moe(ops.act_quant(dev_bf16(x)), dev(idx), dev(rw), (p1, ps1, p3, ps3, p2, ps2), I, add=dev(add))
    assert np.array_equal(host(y_p8), host(y_mx))
    ex = ops.Mxfp4Experts(*d)
    y_rec = host(ops.mxfp4_moe(dev_bf16(x), dev(idx), dev(rw), ex, add=dev(add)))
    assert np.array_equal(y_rec, host(y_mx))
    for r in (0, 33, R - 1):
        one, _ = ops.ds41_moe_mx(xq[r:r + 1], xs[r:r + 1], dev(idx[r:r + 1]), dev(rw[r:r + 1]),
                                 (ops.moe_pack_mx(p1), ps1, ops.moe_pack_mx(p3), ps3, ops.moe_pack_mx(p2), ps2), I, add=dev(add[r:r + 1]))
        assert np.array_equal(host(one)[0], host(y_mx)[r]), r
    # two to eight rows on the tile layouts run as the grouped GEMM too (faster there than the single launch): same bits, and the
    # single launch forced for the same rows gives them as well
    L = ops._lib()
    for n in (2, 5, 8):
        args = (xq[:n], xs[:n], dev(idx[:n]), dev(rw[:n]), (ops.moe_pack_mx(p1), ps1, ops.moe_pack_mx(p3), ps3, ops.moe_pack_mx(p2), ps2), I)
        few, _ = ops.ds41_moe_mx(*args, add=dev(add[:n]))
        assert np.array_equal(host(few), host(y_mx)[:n]), n
        L.spark_debug_mx_fused_rows(8)
        try:
            one_launch, _ = ops.ds41_moe_mx(*args, add=dev(add[:n]))
        finally:
            L.spark_debug_mx_fused_rows(-1)
        assert np.array_equal(host(one_launch), host(few)), n


def test_ds41_two_bit_coded_scales(ops, oracle):
    # the reference's lossless 2-bit scale coding (kern.rs moe_scales_s2): nearly constant scales are coded, a tile with a wide
    # row keeps its raw words; the kernels must see the same scale bytes either way
    g = synth.rng(214)
    R, H, I, E, topk = 3, 5120, 128, 4, 2
    ws, x, idx, rw = _case(g, R, H, I, E, topk, 0, smin=119)
    ws = [a.copy() for a in ws]
    for s in (ws[1], ws[3], ws[5]):
        s[:] = g.integers(120, 123, s.shape, dtype=np.uint8)           # span <= 3 everywhere: coded tiles
    ws[1][1, 9, 5] = 110                                                # one wide row: its tile stays raw
    ws[5][2, 700, 1] = 127
    ref = oracle.mxfp4_moe(x, idx, rw, *ws)
    d = [dev(a) for a in ws]
    p1, ps1 = ops.moe_pack(d[0], d[1]); p3, ps3 = ops.moe_pack(d[2], d[3]); p2, ps2 = ops.moe_pack(d[4], d[5])
    xq, xs = ops.act_quant_fp8(dev_bf16(x))
    packed = (ops.moe_pack_mx(p1), ops.moe_pack_mx(p3), ops.moe_pack_mx(p2))
    y_raw, _ = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), (packed[0], ps1, packed[1], ps3, packed[2], ps2), I)
    b1, n1, t1 = ops.moe_scales_s2(ps1); b3, n3, _ = ops.moe_scales_s2(ps3); b2, n2, t2 = ops.moe_scales_s2(ps2)
    assert (n1, n3, n2) == (1, 0, 1) and t1 == E * I // 8 and t2 == E * H // 8
    assert b3.numel() == t1 * 16 + t1 * (H // 128) * 8                  # a quarter of the raw bytes + 16 per tile
    ops.moe_s2_set(True)
    try:
        y_s2, _ = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), (packed[0], b1, packed[1], b3, packed[2], b2), I)
    finally:
        ops.moe_s2_set(False)
    assert np.array_equal(host(y_s2), host(y_raw))
    assert rel_l2(host(y_s2), ref) <= TOL
    # more than 8 rows: the grouped GEMM decodes the same blobs (coded tiles and the raw one)
    R2 = 40
    x2 = synth.randn_bf16(g, (R2, H))
    idx2 = np.stack([g.permutation(E)[:topk] for _ in range(R2)]).astype(np.int64)
    rw2 = g.uniform(0.1, 1.0, (R2, topk)).astype(np.float32)
    xq2, xs2 = ops.act_quant_fp8(dev_bf16(x2))
    y2_raw, _ = ops.ds41_moe_mx(xq2, xs2, dev(idx2), dev(rw2), (packed[0], ps1, packed[1], ps3, packed[2], ps2), I)
    ops.moe_s2_set(True)
    try:
        y2_s2, _ = ops.ds41_moe_mx(xq2, xs2, dev(idx2), dev(rw2), (packed[0], b1, packed[1], b3, packed[2], b2), I)
    finally:
        ops.moe_s2_set(False)
    assert np.array_equal(host(y2_s2), host(y2_raw))
    assert rel_l2(host(y2_s2), oracle.mxfp4_moe(x2, idx2, rw2, *ws)) <= TOL



def _ds41_weights(ops, ws):
    d = [dev(a) for a in ws]
    p1, ps1 = ops.moe_pack(d[0], d[1]); p3, ps3 = ops.moe_pack(d[2], d[3]); p2, ps2 = ops.moe_pack(d[4], d[5])
    return (ops.moe_pack_mx(p1), ps1, ops.moe_pack_mx(p3), ps3, ops.moe_pack_mx(p2), ps2)


@pytest.mark.parametrize("R", [3, 20])
def test_ds41_ws_ptrs_hand_out_the_per_pair_outputs(ops, oracle, R):
    # reference ds41_mx.cu:1494-1505, kern.rs:1043-1050: after ds41_moe_mx_ex(skip_combine = 1) the caller (the prefill
    # reduce-scatter) sums out[pairmap[r * topk + k]] itself; the two arrays live inside ws
    import ctypes as C
    g = synth.rng(216 + R)
    H, I, E, topk = 5120, 512, 5, 2
    ws, x, idx, rw = _case(g, R, H, I, E, topk, 0, smin=119)
    ref, pairs = oracle.mxfp4_moe(x, idx, rw, *ws, want_pairs=True)
    w = _ds41_weights(ops, ws)
    xq, xs = ops.act_quant_fp8(dev_bf16(x))
    _, wsb = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), w, I, skip_combine=True)
    L = ops._lib()
    po, pm = C.c_void_p(), C.c_void_p()
    assert L.ds41_moe_mx_ws_ptrs(C.c_void_p(wsb.data_ptr()), R, I, topk, E, C.byref(po), C.byref(pm)) == 0
    lo, hi = wsb.data_ptr(), wsb.data_ptr() + wsb.numel()
    P = R * topk
    assert lo <= pm.value and pm.value + 4 * P <= hi and lo <= po.value and po.value + 4 * P * H <= hi     # both inside the caller's workspace
    torch.cuda.synchronize()
    off_m, off_o = pm.value - lo, po.value - lo
    pairmap = wsb[off_m:off_m + 4 * P].view(torch.int32).cpu().numpy()
    out = wsb[off_o:off_o + 4 * P * H].view(torch.float32).view(P, H).cpu().numpy()
    assert sorted(pairmap.tolist()) == list(range(P))                                                     # a permutation of the pair rows
    got = out[pairmap]                                                                                     # row r * topk + k = pair (r, k)
    assert rel_l2(got, pairs) <= TOL, rel_l2(got, pairs)
    # the caller's own sum in slot order reproduces the call with the combine inside, bit for bit
    y_in, _ = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), w, I)
    acc = np.zeros((R, H), np.float32)
    for k in range(topk):
        acc = acc + got[k::topk]
    assert np.array_equal(acc, host(y_in))
    assert rel_l2(acc, ref) <= TOL


def test_ds41_column_passes_under_a_small_cap(ops, oracle):
    # reference ds41_mx.cu:1416-1425: a prefill-sized call whose per-pair outputs exceed the cap runs down + combine in column
    # passes over a smaller buffer; the values are those of the one-pass call.  The cap is lowered here so that 40 rows reach it.
    g = synth.rng(218)
    R, H, I, E, topk = 40, 5120, 512, 5, 2
    ws, x, idx, rw = _case(g, R, H, I, E, topk, 0, smin=119)
    add = g.standard_normal((R, H)).astype(np.float32)
    w = _ds41_weights(ops, ws)
    xq, xs = ops.act_quant_fp8(dev_bf16(x))
    L = ops._lib()
    assert L.ds41_moe_mx_col_passes(R, topk, E) == 1 and L.ds41_moe_mx_pair_b16(R, topk, E) == 0
    one, _ = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), w, I, add=dev(add))
    one = host(one)
    assert rel_l2(one, oracle.mxfp4_moe(x, idx, rw, *ws, add=add)) <= TOL
    full = L.ds41_moe_mx_ws_bytes(R, I, topk, E)
    try:
        for cap, passes in ((4 * R * topk * H // 2, 2), (4 * R * topk * H // 4, 4), (1024, 4)):
            L.spark_debug_mx_out_cap(cap)
            assert L.ds41_moe_mx_col_passes(R, topk, E) == passes
            assert L.ds41_moe_mx_col_passes(8, topk, E) == 1                                               # decode sizes never split
            small = L.ds41_moe_mx_ws_bytes(R, I, topk, E)
            assert small < full - 4 * R * topk * H * (passes - 1) // passes + 4096
            wsb = torch.empty(small, dtype=torch.uint8, device=DEV)
            y, _ = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), w, I, add=dev(add), ws=wsb)
            assert np.array_equal(host(y), one), passes
            with pytest.raises(ops.KernelError):                                                           # no skip_combine with passes (reference :1445)
                ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), w, I, add=dev(add), ws=wsb, skip_combine=True)
    finally:
        L.spark_debug_mx_out_cap(0)


def test_ds41_bf16_pair_outputs_switch(ops, oracle):
    # reference ds41_mx.cu:1245-1255 (DS41_MOE_PAIR_BF16, off by default): calls of more than 64 rows keep every pair's down output as
    # bf16; the buffer ds41_moe_mx_ws_ptrs hands out then holds the bf16 rounding of what the binary32 form holds, and the sum over the
    # pairs is the binary32 sum of those in slot order
    import ctypes as C
    g = synth.rng(219)
    R, H, I, E, topk = 70, 5120, 512, 5, 2
    ws, x, idx, rw = _case(g, R, H, I, E, topk, 0, smin=119)
    add = g.standard_normal((R, H)).astype(np.float32)
    w = _ds41_weights(ops, ws)
    xq, xs = ops.act_quant_fp8(dev_bf16(x))
    L = ops._lib()
    assert L.ds41_moe_mx_pair_b16(R, topk, E) == 0
    y32, wsb32 = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), w, I, add=dev(add), skip_combine=True)
    po, pm = C.c_void_p(), C.c_void_p()
    assert L.ds41_moe_mx_ws_ptrs(C.c_void_p(wsb32.data_ptr()), R, I, topk, E, C.byref(po), C.byref(pm)) == 0
    torch.cuda.synchronize()
    P = R * topk
    o32 = wsb32[po.value - wsb32.data_ptr():po.value - wsb32.data_ptr() + 4 * P * H].view(torch.float32).view(P, H).clone()
    pmap32 = wsb32[pm.value - wsb32.data_ptr():pm.value - wsb32.data_ptr() + 4 * P].view(torch.int32).clone()
    L.spark_debug_mx_pair_b16(1)
    try:
        assert L.ds41_moe_mx_pair_b16(R, topk, E) == 1 and L.ds41_moe_mx_pair_b16(64, topk, E) == 0
        y16, wsb16 = ops.ds41_moe_mx(xq, xs, dev(idx), dev(rw), w, I, add=dev(add))
        assert L.ds41_moe_mx_ws_ptrs(C.c_void_p(wsb16.data_ptr()), R, I, topk, E, C.byref(po), C.byref(pm)) == 0
        torch.cuda.synchronize()
        o16 = wsb16[po.value - wsb16.data_ptr():po.value - wsb16.data_ptr() + 2 * P * H].view(torch.bfloat16).view(P, H)
        pmap16 = wsb16[pm.value - wsb16.data_ptr():pm.value - wsb16.data_ptr() + 4 * P].view(torch.int32)
        # (which compact row a pair gets may differ from call to call - the grouping hands rows out with atomics -: compare pair by pair)
        assert torch.equal(o16[pmap16.long()], o32[pmap32.long()].to(torch.bfloat16))
        acc = torch.zeros(R, H, dtype=torch.float32, device=DEV)
        for k in range(topk):
            acc = acc + o16.float()[pmap16.view(R, topk)[:, k].long()]
        assert torch.equal(y16, dev(add) + acc)                         # add + (the pairs in slot order), binary32
        assert rel_l2(host(y16), oracle.mxfp4_moe(x, idx, rw, *ws, add=add)) <= 4e-3      # the bf16 rounding of the pairs: the reference's class L1
        small, _ = ops.ds41_moe_mx(xq[:40], xs[:40], dev(idx[:40]), dev(rw[:40]), w, I, add=dev(add[:40]))
    finally:
        L.spark_debug_mx_pair_b16(0)
    plain, _ = ops.ds41_moe_mx(xq[:40], xs[:40], dev(idx[:40]), dev(rw[:40]), w, I, add=dev(add[:40]))
    assert torch.equal(small, plain)                                    # calls of up to 64 rows are not touched by the switch
    L.spark_debug_mx_pair_b16(-1)
