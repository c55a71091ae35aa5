"""Pins the oracle's EXL3 decode: codebooks against closed forms evaluated with numpy float16 / float64, the tile bit
layout against the reference's NIBMAP table (tests/golden/nibmap_4bit.json) and against a big-integer bitstream, the
Hadamard against the dense Sylvester matrix.  CPU only."""
import json
from pathlib import Path

import numpy as np
import pytest

GOLD = Path(__file__).parent / "golden"
NIBMAP = np.array(json.loads((GOLD / "nibmap_4bit.json").read_text())["nibmap"])


def test_mcg_codebook_all_states(oracle):
    # reference glm53_tests/test_exl3.py:23-29 anchor + the closed form in numpy float16 arithmetic
    F = oracle.codebook(1).view(np.float16).astype(np.float32)
    lo = np.uint16(0x3B60).view(np.float16).astype(np.float32)
    assert F[0] == pytest.approx(2.0 * lo, abs=1e-6)
    assert not np.isnan(F).any()
    x = (np.arange(65536, dtype=np.uint64) * np.uint64(0xCBAC1FED)) & np.uint64(0xFFFFFFFF)
    y = (x.astype(np.uint32) & np.uint32(0x8FFF8FFF)) ^ np.uint32(0x3B603B60)
    ref = (y & 0xFFFF).astype(np.uint16).view(np.float16) + (y >> 16).astype(np.uint16).view(np.float16)   # fp16 add
    assert np.array_equal(ref.view(np.uint16), oracle.codebook(1))


def test_mul1_codebook_all_states(oracle):
    x = (np.arange(65536, dtype=np.uint64) * np.uint64(0x83DCD12D)) & np.uint64(0xFFFFFFFF)
    b = (x & 255) + ((x >> 8) & 255) + ((x >> 16) & 255) + (x >> 24)
    c1 = np.float64(np.uint16(0x1eee).view(np.float16)); c2 = np.float64(np.uint16(0xc931).view(np.float16))
    ref = ((1024.0 + b.astype(np.float64)) * c1 + c2).astype(np.float16)      # exact in binary64, one rounding
    assert np.array_equal(ref.view(np.uint16), oracle.codebook(2))
    v = ref.astype(np.float64)
    assert abs(v.mean()) < 0.05 and 0.9 < v.std() < 1.1                        # the codebook is ~ N(0, 1)


def test_nibmap_invariants():
    # reference glm53_tests/test_exl3.py:32-35
    assert NIBMAP.shape == (16, 16, 4)
    assert sorted(np.bincount(NIBMAP.ravel(), minlength=256))[-1] == 4
    assert NIBMAP[0][0].tolist() == [0, 255, 254, 253] and NIBMAP[8][0].tolist() == [2, 1, 0, 255]


def _inner_via_nibmap(trellis, table):
    """The reference's table-driven statement of the 4-bit layout (glm53/exl3.py:8-13 steps 1-3), in numpy."""
    w16 = trellis.astype(np.uint16)
    u32 = w16[..., 0::2].astype(np.uint32) | (w16[..., 1::2].astype(np.uint32) << 16)
    pos = np.arange(256)
    nib = ((u32[..., pos // 8] >> (28 - 4 * (pos % 8)).astype(np.uint32)) & 0xF).astype(np.uint32)
    word = nib[..., NIBMAP[..., 0]] | (nib[..., NIBMAP[..., 1]] << 4) | (nib[..., NIBMAP[..., 2]] << 8) | (nib[..., NIBMAP[..., 3]] << 12)
    Kt, Nt = trellis.shape[:2]
    return table[word].transpose(0, 2, 1, 3).reshape(Kt * 16, Nt * 16)


@pytest.mark.parametrize("cbk", [1, 2])
def test_decode_inner_4bit_matches_nibmap(oracle, cbk):
    rng = np.random.default_rng(10 + cbk)
    tr = rng.integers(-32768, 32768, (5, 7, 64), dtype=np.int16)
    ref = _inner_via_nibmap(tr, oracle.codebook(cbk))
    assert np.array_equal(oracle.decode_inner(tr, cbk), ref)


@pytest.mark.parametrize("bits", [3, 4, 5, 6])
def test_tile_states_vs_bigint_bitstream(oracle, bits):
    # the definition: words little-endian uint32, read MSB-first; state p = 16 bits starting at ((p+1)*bits - 16) mod L
    rng = np.random.default_rng(20 + bits)
    tile = rng.integers(-32768, 32768, 16 * bits, dtype=np.int16)
    w16 = tile.astype(np.uint16).astype(object)
    L = 256 * bits
    stream = 0
    for j in range(8 * bits):
        stream = (stream << 32) | int(w16[2 * j] | (w16[2 * j + 1] << 16))
    stream2 = (stream << L) | stream                                           # tail-biting: the stream repeated
    ref = []
    for p in range(256):
        b0 = ((p + 1) * bits - 16) % L
        ref.append((stream2 >> (2 * L - b0 - 16)) & 0xFFFF)
    assert oracle.tile_states(tile, bits).tolist() == ref


def test_perm_is_tensor_core_order(oracle):
    # position 8t+j <-> row (t%4)*2 + {0,1,8,9}[j%4], col t/4 + 8*(j/4); a permutation of the 256 cells that agrees
    # with the NIBMAP table: cell (r, c)'s lowest nibble slot is the state's last nibble = position p
    seen = set()
    for p in range(256):
        el = oracle.lib.orc_exl3_perm(p)
        seen.add(el)
        assert NIBMAP[el >> 4][el & 15][0] == p
    assert len(seen) == 256


def _hadamard(n):
    h = np.ones((1, 1))
    while h.shape[0] < n:
        h = np.block([[h, h], [h, -h]])
    return h / np.sqrt(n)


def test_fwht128_vs_dense_sylvester(oracle):
    rng = np.random.default_rng(30)
    H = _hadamard(128)
    assert np.allclose(H @ H, np.eye(128), atol=1e-12)
    for _ in range(8):
        x = rng.standard_normal(128).astype(np.float32)
        got = oracle.fwht128(x)
        assert np.allclose(got, H @ x.astype(np.float64), atol=2e-6)
        assert np.allclose(oracle.fwht128(got), x, atol=2e-6)                  # involution
    # small integers: every butterfly is exact, so the result is float32(sum) * float32(1/sqrt(128)) bit for bit
    xi = rng.integers(-50, 50, 128).astype(np.float32)
    exact = (_hadamard(128) * np.sqrt(128)) @ xi.astype(np.float64)
    assert np.array_equal(oracle.fwht128(xi), exact.astype(np.float32) * np.float32(0.08838834764831845))
    # unit vectors give the Sylvester rows (ordering check)
    e5 = np.zeros(128, np.float32); e5[5] = 1
    assert np.array_equal(np.sign(oracle.fwht128(e5)), np.sign(H[:, 5]))


@pytest.mark.parametrize("cbk,bits", [(2, 4), (1, 4), (2, 3), (2, 6)])
def test_decode_weight_vs_dense_formula(oracle, cbk, bits):
    rng = np.random.default_rng(40 + bits)
    K, N = 256, 128
    tr = rng.integers(-32768, 32768, (K // 16, N // 16, 16 * bits), dtype=np.int16)
    suh = np.where(rng.random(K) < 0.5, -1, 1).astype(np.float16)
    svh = (np.where(rng.random(N) < 0.5, -1, 1) * rng.uniform(0.5, 1.5, N) / np.sqrt(K)).astype(np.float16)
    inner = oracle.decode_inner(tr, cbk).view(np.float16).astype(np.float64)
    H = _hadamard(128)
    w = np.einsum("ij,kjn->kin", H, inner.reshape(K // 128, 128, N)).reshape(K, N) * suh.astype(np.float64)[:, None]
    w = (w.reshape(K, N // 128, 128) @ H).reshape(K, N) * svh.astype(np.float64)[None, :]
    got = oracle.decode_weight(tr, suh.view(np.uint16), svh.view(np.uint16), cbk)
    assert np.allclose(got, w, rtol=0, atol=2e-6 * np.abs(w).max() * 50)
    # identity x @ W == had(had(x * suh) @ inner) * svh   (reference qwen_exl3.cuh:4-7)
    x = rng.standard_normal(K)
    xh = np.concatenate([H @ (x * suh.astype(np.float64))[i:i + 128] for i in range(0, K, 128)])
    y = np.concatenate([H @ (xh @ inner)[i:i + 128] for i in range(0, N, 128)]) * svh.astype(np.float64)
    assert np.allclose(x @ got.astype(np.float64), y, atol=1e-4)
    # fold = W^T rounded to fp16
    f = oracle.fold(tr, suh.view(np.uint16), svh.view(np.uint16), cbk)
    assert np.array_equal(f, got.T.astype(np.float16).view(np.uint16))


def test_had_in_rounds_to_fp16(oracle):
    rng = np.random.default_rng(50)
    K = 256
    x = rng.standard_normal(K).astype(np.float32)
    suh = np.where(rng.random(K) < 0.5, -1, 1).astype(np.float16)
    H = _hadamard(128)
    ref = np.concatenate([H @ (x.astype(np.float64) * suh)[i:i + 128] for i in range(0, K, 128)])
    got = oracle.had_in(x, suh.view(np.uint16)).view(np.float16).astype(np.float64)
    assert np.allclose(got, ref, atol=2e-3, rtol=1e-3)
    assert np.abs(got - ref).max() <= np.abs(ref).max() * 2.0 ** -11 + 1e-6      # within half an fp16 ulp of the largest
