"""Seeded synthetic inputs for the five benchmark configurations (numpy, host side).

Every tensor comes from numpy.random.Generator(PCG64(seed)) so the CPU oracle and the GPU path see identical bytes.
bf16 / fp16 tensors are carried as uint16 bit patterns.
"""
import numpy as np


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def bf16_bits(x):
    """float32 -> bfloat16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def randn_bf16(g, shape):
    return bf16_bits(g.standard_normal(shape, np.float32))


# ---------------------------------------------------------------- EXL3 (config 2)

def exl3_matrix(g, K, N, bits=4):
    """One EXL3 linear: trellis int16 [K/16, N/16, 16*bits] of uniform random bits, suh fp16 [K] random +-1,
    svh fp16 [N] = random sign * U[0.5, 1.5] / sqrt(K)."""
    tr = g.integers(-32768, 32768, (K // 16, N // 16, 16 * bits), dtype=np.int16)
    suh = np.where(g.random(K) < 0.5, -1.0, 1.0).astype(np.float16)
    svh = (np.where(g.random(N) < 0.5, -1.0, 1.0) * g.uniform(0.5, 1.5, N) / np.sqrt(K)).astype(np.float16)
    return tr, suh.view(np.uint16), svh.view(np.uint16)


def exl3_expert(g, H, I, bits=4):
    """(gate_tr, up_tr, down_tr, gate_suh, up_suh, down_suh, gate_svh, up_svh, down_svh) in the reference's table order."""
    gt, gs, gv = exl3_matrix(g, H, I, bits)
    ut, us, uv = exl3_matrix(g, H, I, bits)
    dt, ds, dv = exl3_matrix(g, I, H, bits)
    return (gt, ut, dt, gs, us, ds, gv, uv, dv)


# ---------------------------------------------------------------- MXFP4 (configs 1, 3, 5)

def mxfp4_matrix(g, N, K, smin, smax=127):
    """codes [N, K/2] uint8 (two uniform E2M1 codes per byte), scales [N, K/32] uint8 uniform in [smin, smax]."""
    w = g.integers(0, 256, (N, K // 2), dtype=np.uint8)
    s = g.integers(smin, smax + 1, (N, K // 32), dtype=np.uint8)
    return w, s


def mxfp4_experts(g, E, H, I, smin=117):
    """Stacked natural layout: w1, s1, w3, s3 [E, I, H/2 | H/32], w2, s2 [E, H, I/2 | I/32]."""
    w1 = g.integers(0, 256, (E, I, H // 2), dtype=np.uint8); s1 = g.integers(smin, 128, (E, I, H // 32), dtype=np.uint8)
    w3 = g.integers(0, 256, (E, I, H // 2), dtype=np.uint8); s3 = g.integers(smin, 128, (E, I, H // 32), dtype=np.uint8)
    w2 = g.integers(0, 256, (E, H, I // 2), dtype=np.uint8); s2 = g.integers(smin, 128, (E, H, I // 32), dtype=np.uint8)
    return w1, s1, w3, s3, w2, s2


# ---------------------------------------------------------------- FP8 (config 4)

def fp8_e4m3_bits(x):
    """float32 -> E4M3 (fn) codes, round to nearest even, saturating at +-448 (numpy only)."""
    x = np.clip(np.ascontiguousarray(x, np.float32), -448.0, 448.0)
    a = np.abs(x).astype(np.float64)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -20)))
    e = np.clip(e, -6, 8)                                    # subnormals share the exponent of the smallest normal
    q = np.rint(a / 2.0 ** (e - 3))                          # units of the last place; rint = ties to even
    bump = q >= 16
    e = np.where(bump, e + 1, e); q = np.where(bump, 8, q)
    code = np.where(q < 8, q, ((e + 7) * 8 + (q - 8))).astype(np.int64)
    code = np.minimum(code, 0x7E)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def fp8_block_matrix(g, N, K, bs=128):
    """W fp32 N(0,1) clipped to +-448 then cast to E4M3; scales fp32 [ceil(N/bs), ceil(K/bs)] log-uniform in [1e-3, 1e-1]."""
    w = fp8_e4m3_bits(g.standard_normal((N, K), np.float32))
    s = np.exp(g.uniform(np.log(1e-3), np.log(1e-1), ((N + bs - 1) // bs, (K + bs - 1) // bs))).astype(np.float32)
    return w, s


# ---------------------------------------------------------------- routing

def zipf_routes(g, tokens, E, topk, a=1.1):
    """Per token: topk distinct experts drawn without replacement with probability ~ rank^-a over a fixed random
    permutation of the experts; weights uniform(0, 1) normalised (config 5)."""
    perm = g.permutation(E)
    p = 1.0 / np.arange(1, E + 1) ** a
    p /= p.sum()
    # Gumbel top-k = sampling without replacement
    keys = np.log(p)[None, :] + g.gumbel(size=(tokens, E))
    ranks = np.argsort(-keys, axis=1)[:, :topk]
    idx = perm[ranks].astype(np.int64)
    w = g.uniform(0, 1, (tokens, topk)).astype(np.float32)
    w /= w.sum(-1, keepdims=True)
    return idx, w.astype(np.float32)
