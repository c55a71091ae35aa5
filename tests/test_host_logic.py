"""Host-side logic of the C ABI that needs no GPU: workspace sizing, packed sizes, argument checks that return before any launch."""
import ctypes as C

import pytest


@pytest.fixture(scope="module")
def L():
    from spark_engine_amd import lib
    if not lib.SO.exists():
        pytest.fail(f"{lib.SO} is not built")
    return lib.load()


def test_exl3_workspace_sizes(L):
    sizes = [L.spark_exl3_moe_ws_bytes(R, 2048, 512, 512, 10) for R in (1, 4, 16, 17, 64, 65, 2048)]
    assert all(s > 0 for s in sizes)
    assert sizes == sorted(sizes)                                   # more rows never need less
    assert sizes[-1] > 2048 * 10 * 2048 * 4                         # the prefill path holds the per-pair outputs
    assert L.spark_exl3_moe_ws_bytes(1, 2000, 512, 512, 10) == 0    # H not a multiple of 128
    assert L.spark_exl3_moe_ws_bytes(1, 2048, 500, 512, 10) == 0
    assert L.spark_exl3_moe_ws_bytes(0, 2048, 512, 512, 10) == 0
    assert L.spark_exl3_moe_ws_bytes(1, 2048, 512, 512, 0) == 0
    # the fixed-size entry points size for their models
    assert L.qwen_moe_ws_bytes(3, 4) == L.spark_exl3_moe_ws_bytes(3, 2560, 640, 512, 10)
    assert L.glm_moe_ws_bytes(3, 2) == L.spark_exl3_moe_ws_bytes(3, 4096, 1024, 288, 8)
    assert L.glm_moe3_ws_bytes(3, 2) == L.spark_exl3_moe_ws_bytes(3, 4096, 768, 288, 8)


def test_mxfp4_workspace_and_packed_sizes(L):
    sizes = [L.spark_mxfp4_moe_ws_bytes(R, 4096, 2048, 6, 384, 1) for R in (1, 2, 4, 8, 9, 64, 2048)]
    assert all(s > 0 for s in sizes) and sizes == sorted(sizes)
    assert sizes[-1] > 2048 * 7 * 4096 * 4                          # per-pair outputs [P, H] binary32
    assert L.spark_mxfp4_moe_ws_bytes(1, 4000, 2048, 6, 384, 1) == 0
    # one 4352-byte record per 16 rows x 512 K
    assert L.spark_mxfp4_packed_bytes(16, 512) == 4352
    assert L.spark_mxfp4_packed_bytes(385 * 2048, 4096) == (385 * 2048 // 16) * 8 * 4352
    assert L.spark_mxfp4_packed_bytes(32, 640) == 2 * 2 * 4352      # a partial K group takes a whole record
    # the reference-named sizing calls (H fixed at 7168 there)
    assert L.ds41_moe_mx_ws_bytes(1, 2048, 6, 384) > 0
    assert L.ds41_moe_ws_bytes(1, 2048, 6, 384) > 0


def test_switches(L):
    L.ds41_moe_mx_set_s2(1)
    assert L.ds41_moe_mx_get_s2() == 1
    L.ds41_moe_mx_set_s2(0)
    assert L.ds41_moe_mx_get_s2() == 0
    assert L.ds41_fp8_gemv_mx_smem_max() > 0


def test_argument_checks_return_before_any_launch(L):
    null = None
    # GEMVs: 1 = bad shape (reference ds41.cu:230)
    assert L.ds41_mxfp4_gemv(null, null, null, null, 9, 16, 64, null) == 1          # more than 8 rows
    assert L.ds41_mxfp4_gemv(null, null, null, null, 1, 16, 48, null) == 1          # k not a multiple of 32
    assert L.ds41_fp8_gemv(null, null, null, null, 0, 16, 64, null) == 1
    assert L.spark_fp8_block128_gemv(null, null, null, null, 1, 16, 24, null) == 1
    assert L.ds41_act_quant_fp8(null, null, null, 33, null) == 1                    # not whole blocks of 32
    assert L.ds41_act_quant32(null, null, 0, null) == 0                             # nothing to do
    # routers
    assert L.ds41_route(null, null, null, null, 1, 2048, 6, C.c_float(1.0), null) == 1   # too many experts
    assert L.ds41_route(null, null, null, null, 1, 384, 17, C.c_float(1.0), null) == 1   # top-k above 16
    # EXL3: -1 dimensions, -4 kmask (reference qwen_exl3.cu:72-128)
    assert L.spark_exl3_moe(null, 2, 2000, 1, null, 0, null, 0, null, null, null, null, 2000, 512, 512, 10, 2, 0, 0, null) == -1
    assert L.spark_exl3_moe(null, 2, 2048, 1, null, 0, null, 0, null, null, null, null, 2048, 512, 512, 10, 7, 0, 0, null) == -1   # codebook id
    assert L.spark_exl3_moe(null, 2, 2049, 1, null, 0, null, 0, null, null, null, null, 2048, 512, 512, 10, 2, 0, 0, null) == -1   # odd row stride
    assert L.glm_moe_experts(null, 4096, 1, null, null, null, null, null, null, 2, null, 0, null) == -4
    assert L.glm_moe_experts(null, 4096, 1, null, null, null, null, null, null, 2, null, 1 << 7, null) == -4
    assert L.glm_moe3_experts(null, 4096, 1, null, null, null, null, null, null, 2, 1 << 2, null) == -4
    # MXFP4 MoE: 1 = bad shape (reference ds41_mx.cu:1439)
    assert L.spark_mxfp4_moe_x(null, null, 1, null, null, null, null, null, null, null, null, 0, 4000, 2048, 6, 384, 1, null, null, null, 0, null) == 1
    assert L.spark_mxfp4_moe_x(null, null, 1, null, null, null, null, null, null, null, null, 9, 4096, 2048, 6, 384, 1, null, null, null, 0, null) == 1   # layout id


def test_fixed_width_entry_points_reject_other_widths():
    # ds41_moe_mx / ds41_moe carry no hidden-width argument (they are compiled for 5120): the wrappers check the operands' shapes
    # before anything is launched
    import torch
    from spark_engine_amd import ops
    xq = torch.zeros(2, 1024, dtype=torch.uint8)
    xs = torch.zeros(2, 32, dtype=torch.uint8)
    idx = torch.zeros(2, 2, dtype=torch.int64)
    rw = torch.ones(2, 2)
    w = tuple(torch.zeros(4, 8, dtype=torch.uint8) for _ in range(6))
    with pytest.raises(ValueError):
        ops.ds41_moe_mx(xq, xs, idx, rw, w, 128)
    with pytest.raises(ValueError):
        ops.ds41_moe(torch.zeros(2, 1024, dtype=torch.bfloat16), idx, rw, w, 128)


def _wave_items(experts, cap, nj=2):
    """Restatement of the one-wave item logic of the single-launch kernels (wave_items_init / wave_items_pick: lane l holds pairs
    l, l + 64, ...; an owner table gives every expert its first pair; ballots rank the first pairs and collect an item's pairs) as
    the 64 lanes execute it, with the cap on an item's rows.  -> list of (expert, rows written, n reported, over)."""
    P = len(experts)
    e = [[experts[l + 64 * j] if l + 64 * j < P else -1 for j in range(nj)] for l in range(64)]
    owner = {}
    for l in range(64):
        for j in range(nj):
            if e[l][j] >= 0:
                owner[e[l][j]] = min(owner.get(e[l][j], 1 << 30), l + 64 * j)
    first = [[e[l][j] >= 0 and owner[e[l][j]] == l + 64 * j for j in range(nj)] for l in range(64)]
    rank, base = [[0] * nj for _ in range(64)], 0
    for j in range(nj):
        m = [first[l][j] for l in range(64)]
        for l in range(64):
            rank[l][j] = base + sum(m[:l])
        base += sum(m)
    out = []
    for g in range(base + 1):
        eg = -1
        for j in range(nj):
            hit = [l for l in range(64) if first[l][j] and rank[l][j] == g]
            if hit:
                eg = e[hit[0]][j]
        if eg < 0:
            out.append((-1, [], 0, False))
            continue
        rows, n = [None] * cap, 0
        for j in range(nj):
            m = [e[l][j] == eg for l in range(64)]
            for l in range(64):
                if m[l] and n + sum(m[:l]) < cap:
                    assert 0 <= n + sum(m[:l]) < cap                        # the store the kernel makes: always inside rows[cap]
                    rows[n + sum(m[:l])] = l + 64 * j
            n += sum(m)
        over = n > cap
        out.append((eg, rows[:min(n, cap)], min(n, cap), over))
    return out


def test_item_rows_never_exceed_the_cap():
    # items = a call's distinct experts in order of first appearance, their pairs ascending (brute force below); a token row that names
    # an expert twice can give an item more pairs than the call has rows: the item keeps its first `cap` pairs and reports `over`
    import random
    rnd = random.Random(3)
    for trial in range(300):
        R, topk, E = rnd.choice([1, 2, 3, 4, 8]), rnd.choice([1, 2, 6, 10, 16]), rnd.choice([4, 17, 64])
        if R * topk > 128:
            continue
        dup = trial % 3 == 0
        ex = []
        for r in range(R):
            row = [rnd.randrange(E) for _ in range(topk)] if dup else rnd.sample(range(E), min(topk, E)) + [0] * max(0, topk - E)
            ex += row[:topk]
        order, pairs = [], {}
        for p, x in enumerate(ex):
            if x not in pairs:
                order.append(x); pairs[x] = []
            pairs[x].append(p)
        got = _wave_items(ex, cap=R)
        assert [g[0] for g in got[:-1]] == order and got[-1][0] == -1
        for eg, rows, n, over in got[:-1]:
            assert rows == pairs[eg][:R] and n == min(len(pairs[eg]), R) and over == (len(pairs[eg]) > R)
            if not dup and topk <= E:
                assert not over and n == len(pairs[eg])                       # valid routes: never capped
