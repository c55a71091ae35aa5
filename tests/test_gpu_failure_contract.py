"""What the single-launch decode kernels do when a call breaks the routes' contract (a token row that names an expert twice: the
item would hold more rows than the kernels' arrays, so it is cut at what they hold) or a bounded wait expires: nothing is written
outside the arrays, the workspace's error flag is set, every output element whose sum could not be completed holds NaN - a caller
that only looks at return codes cannot take stale bytes for a result - later calls on that workspace give NaN until it is prepared
again, and spark_moe_ws_status makes the next call prepare it.  Every kernel here runs to its normal end."""
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


def test_exl3_duplicated_expert_is_contained_and_reported(ops, oracle):
    g = synth.rng(950)
    H, I, E, topk, R = 512, 256, 8, 2, 2
    experts = {e: synth.exl3_expert(g, H, I) for e in range(E)}
    table = ops.ExpertTable({e: [dev(t[0]), dev(t[1]), dev(t[2])] + [dev_f16(a) for a in t[3:]] for e, t in experts.items()}, E)
    xb = synth.randn_bf16(g, (R, H))
    w = g.uniform(0.2, 1.0, (R, topk)).astype(np.float32)
    good = np.array([[5, 3], [3, 7]], np.int32)
    bad = np.array([[5, 5], [5, 7]], np.int32)                          # expert 5 three times in a call of two rows
    xd, wd = dev_bf16(xb), dev(w)
    ws = ops.exl3_moe_ws_alloc(R, H, I, E, topk)
    want = host(ops.exl3_moe(xd, dev(good), wd, table, H, I, ws=ws, ws_clean=True))
    assert rel_l2(want, oracle.exl3_moe(synth.bf16_to_f32(xb), good, w, experts, E, H, I, 4, 2, 0)) <= 1e-3
    assert ops.ws_status(ws) == 0
    out = torch.full((R, H), 123.0, dtype=torch.float32, device=DEV)
    ops.exl3_moe(xd, dev(bad), wd, table, H, I, ws=ws, ws_clean=True, out=out)
    got = host(out)
    assert ops.ws_status(ws) == 1                                       # reported (and the workspace is no longer known as prepared)
    assert not (got == 123.0).any()                                     # no stale bytes: every element was written
    assert np.isnan(got[1]).all()                                       # the row whose pair was cut away
    # the other row's pairs were all served: a column block of it holds either the right sums or, where its summing block started after
    # the flag was raised (the flag is sticky and read as a summing block starts), NaN - never anything else
    real = ~np.isnan(got[0])
    one = oracle.exl3_moe(synth.bf16_to_f32(xb[:1]), np.array([[5]], np.int32), np.array([[1.0]], np.float32), experts, E, H, I, 4, 2, 0)
    exp0 = (w[0, 0] + w[0, 1]) * one[0]
    assert np.abs(got[0][real] - exp0[real]).max(initial=0.0) <= 2e-3 * np.abs(exp0).max()
    # while the flag stands, a caller that keeps promising "prepared" gets NaN, not sums of the words the failed call left behind
    again = host(ops.exl3_moe(xd, dev(good), wd, table, H, I, ws=ws, ws_clean=True))
    assert np.isnan(again).all()
    # a call that does not promise it prepares the workspace itself (the status call forgot it) and is right again
    assert np.array_equal(host(ops.exl3_moe(xd, dev(good), wd, table, H, I, ws=ws)), want)
    assert ops.ws_status(ws) == 0
    # the entry point on the library's own array: the same containment, its own status call, and the next call starts clean
    L = ops._lib()
    st_out = torch.full((R, H), 123.0, dtype=torch.float32, device=DEV)
    ops.exl3_moe_static(xd, dev(bad), wd, table, H, I, out=st_out)
    assert L.spark_exl3_moe_static_status(ops._st()) == 1 and np.isnan(host(st_out)[1]).all() and not (host(st_out) == 123.0).any()
    assert np.array_equal(host(ops.exl3_moe_static(xd, dev(good), wd, table, H, I)), want)
    assert L.spark_exl3_moe_static_status(ops._st()) == 0


def test_exl3_item_kernels_take_a_duplicated_expert_as_a_second_item(ops, oracle):
    # the several-kernel path groups by the instance's row count, so the repeated expert gets a second item and every pair is computed
    g = synth.rng(951)
    H, I, E, topk, R = 512, 256, 8, 2, 2
    experts = {e: synth.exl3_expert(g, H, I) for e in range(E)}
    table = ops.ExpertTable({e: [dev(t[0]), dev(t[1]), dev(t[2])] + [dev_f16(a) for a in t[3:]] for e, t in experts.items()}, E)
    xb = synth.randn_bf16(g, (R, H))
    w = g.uniform(0.2, 1.0, (R, topk)).astype(np.float32)
    bad = np.array([[5, 5], [5, 7]], np.int32)
    y = host(ops.exl3_moe(dev_bf16(xb), dev(bad), dev(w), table, H, I, multi_kernel=True))
    assert rel_l2(y, oracle.exl3_moe(synth.bf16_to_f32(xb), bad, w, experts, E, H, I, 4, 2, 0)) <= 1e-3


def test_mxfp4_duplicated_expert_is_contained_and_reported(ops, oracle):
    g = synth.rng(952)
    H, I, E, topk, ns, R = 1024, 512, 6, 2, 1, 2
    wts = synth.mxfp4_experts(g, E + ns, H, I)
    ex = ops.Mxfp4Experts(*[dev(a) for a in wts], n_shared=ns)
    x = synth.randn_bf16(g, (R, H))
    rw = g.uniform(0.2, 1.0, (R, topk)).astype(np.float32)
    good = np.array([[4, 1], [1, 3]], np.int64)
    bad = np.array([[4, 4], [4, 3]], np.int64)
    xd, rwd = dev_bf16(x), dev(rw)
    ws = ops.mxfp4_moe_ws_alloc(R, ex, topk)
    want = host(ops.mxfp4_moe_x(xd, dev(good), rwd, ex, ws=ws, ws_clean=True))
    assert rel_l2(want, oracle.mxfp4_moe(x, good, rw, *wts, n_shared=ns)) <= 1e-3
    assert ops.ws_status(ws) == 0
    y = torch.full((R, H), 123.0, dtype=torch.float32, device=DEV)
    ops.mxfp4_moe_x(xd, dev(bad), rwd, ex, ws=ws, ws_clean=True, y=y)
    got = host(y)
    assert ops.ws_status(ws) == 1
    assert not (got == 123.0).any() and np.isnan(got[1]).all()
    assert np.isnan(host(ops.mxfp4_moe_x(xd, dev(good), rwd, ex, ws=ws, ws_clean=True))).all()       # sticky while the caller promises "prepared"
    assert np.array_equal(host(ops.mxfp4_moe_x(xd, dev(good), rwd, ex, ws=ws)), want)                 # prepared again by the call itself
    assert ops.ws_status(ws) == 0


def test_empty_and_malformed_calls_are_refused_with_the_reference_codes(ops):
    # No rows, no top-k, an intermediate width that is not whole 128-blocks, too many experts: refused on the host with the reference's
    # codes before anything is launched (1 from the ds41 / MXFP4 entry points, engine-rs/shim/ds41_mx.cu:1439, ds41_moe.cu:268; negative
    # from the EXL3 ones, qwen_exl3.cu:72-128), so null pointers never reach a kernel.
    L = ops._lib()
    st = ops._st()
    N = None
    assert L.ds41_moe_mx(N, N, 0, N, N, N, N, N, N, N, N, 768, N, N, N, 6, 384, st) == 1           # no rows
    assert L.ds41_moe_mx(N, N, 1, N, N, N, N, N, N, N, N, 700, N, N, N, 6, 384, st) == 1           # I not a multiple of 128
    assert L.ds41_moe_mx(N, N, 1, N, N, N, N, N, N, N, N, 768, N, N, N, 0, 384, st) == 1           # no top-k
    assert L.ds41_moe_mx(N, N, 1, N, N, N, N, N, N, N, N, 768, N, N, N, 6, 385, st) == 1           # more experts than the reference's EMAX
    assert L.ds41_moe(N, 0, N, N, N, N, N, N, N, N, 768, N, N, N, 6, 384, st) == 1
    assert L.spark_mxfp4_moe_x(N, N, 0, N, N, N, N, N, N, N, N, 0, 4096, 2048, 6, 384, 1, N, N, N, 0, st) == 1
    assert L.spark_mxfp4_moe_x(N, N, 1, N, N, N, N, N, N, N, N, 0, 4100, 2048, 6, 384, 1, N, N, N, 0, st) == 1     # H not a multiple of 128
    assert L.qwen_moe_experts(N, 2560, 0, N, N, N, N, N, N, 4, st) < 0
    assert L.glm_moe_experts(N, 4096, 0, N, N, N, N, N, N, 4, N, 1 << 4, st) < 0
    assert L.spark_exl3_moe(N, 0, 2048, 0, N, 0, N, 0, N, N, N, N, 2048, 512, 512, 10, 2, 0, 0, st) < 0
    assert L.spark_exl3_moe(N, 0, 2048, 1, N, 0, N, 0, N, N, N, N, 2000, 512, 512, 10, 2, 0, 0, st) < 0            # H not a multiple of 128
    assert L.spark_exl3_moe(N, 0, 2048, 1, N, 0, N, 0, N, N, N, N, 2048, 512, 512, 10, 7, 0, 0, st) < 0            # no such codebook
    import torch
    torch.cuda.synchronize()
