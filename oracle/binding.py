"""ctypes binding of the CPU oracle (oracle/oracle.c).  TEST INFRASTRUCTURE ONLY.

Imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg; never by the shipped package.
"""
import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_SO = _DIR / "liboracle.so"


def build(force=False):
    src = _DIR / "oracle.c"
    if force or not _SO.exists() or src.stat().st_mtime > _SO.stat().st_mtime:
        subprocess.check_call(["make", "-C", str(_DIR), "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _SO


def _load():
    build()                                     # compiles only when the library is missing or older than its source
    lib = C.CDLL(str(_SO))
    f32, u16, u8, i32, i64, vp = C.c_float, C.c_uint16, C.c_uint8, C.c_int, C.c_int64, C.c_void_p
    sig = {
        "orc_f16_to_f32": (f32, [u16]), "orc_f64_to_f16": (u16, [C.c_double]), "orc_f32_to_f16": (u16, [f32]),
        "orc_bf16_to_f32": (f32, [u16]), "orc_f32_to_bf16": (u16, [f32]),
        "orc_e4m3_to_f32": (f32, [u8]), "orc_f32_to_e4m3": (u8, [f32]), "orc_e8m0_to_f32": (f32, [u8]),
        "orc_e2m1_to_f32": (f32, [u8]), "orc_mul1_decode": (u16, [C.c_uint32]), "orc_mcg_decode": (u16, [C.c_uint32]),
        "orc_exl3_codebook": (None, [i32, vp]), "orc_exl3_tile_states": (None, [vp, i32, vp]), "orc_exl3_perm": (i32, [i32]),
        "orc_exl3_decode_inner": (None, [vp, i32, i32, i32, i32, vp]), "orc_fwht128": (None, [vp, C.c_size_t]),
        "orc_exl3_had_in": (None, [vp, vp, i32, vp]),
        "orc_exl3_decode_weight": (None, [vp, vp, vp, i32, i32, i32, i32, vp]),
        "orc_exl3_fold": (None, [vp, vp, vp, i32, i32, i32, i32, vp, i64]),
        "orc_exl3_moe": (None, [vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, vp, vp]),
        "orc_qwen_route": (None, [vp, i64, i32, i32, i32, vp, vp]),
        "orc_ds41_route": (None, [vp, vp, vp, vp, i32, i32, i32, f32]),
        "orc_glm_route": (None, [vp, vp, vp, vp, i32, i32, i32, f32]),
        "orc_mxfp4_dequant": (None, [vp, vp, i32, i32, vp]), "orc_fp8_block_dequant": (None, [vp, vp, i32, i32, i32, vp]),
        "orc_fp8_e8m0_dequant": (None, [vp, vp, i32, i32, vp]), "orc_gemv_nk": (None, [vp, vp, i32, i32, i32, vp]),
        "orc_aq_scale": (u8, [f32]), "orc_aq_byte": (u8, [f32, u8]),
        "orc_act_quant_fp8": (None, [vp, vp, vp, i64]), "orc_act_quant32": (None, [vp, vp, i64]),
        "orc_swiglu_quant": (None, [vp, vp, i32, i32, f32]), "orc_silu_mul": (None, [vp, vp, vp, i32]),
        "orc_gate_scale": (None, [vp, i64, i32, vp, vp, i32, i32]),
        "orc_mxfp4_moe": (None, [vp, i32, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp, vp, vp, vp, vp, vp]),
        "orc_mxfp4_moe_from_h": (None, [vp, vp, i32, vp, vp, vp, i32, i32, i32, i32, i32, vp, vp]),
        "orc_mxfp4_gemv": (None, [vp, vp, vp, vp, i32, i32, i32]),
        "orc_fp8_block_gemv": (None, [vp, vp, vp, vp, i32, i32, i32, i32]),
        "orc_fp8_e8m0_gemv": (None, [vp, vp, vp, vp, i32, i32, i32]),
        "orc_fp8_rowscale_gemv": (None, [vp, vp, vp, vp, i32, i32, i32, i32, i32]),
        "orc_fp8_rowscale_quant": (None, [vp, vp, vp, i32, i32]),
        "orc_num_threads": (i32, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


lib = _load()


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.dtype(dt), (a.dtype, dt)
    return a


# ---------------------------------------------------------------- numpy-level helpers (bf16 / fp16 as uint16 bits)

def bf16_bits(x):
    """float32 array -> bfloat16 bit patterns (uint16), round to nearest even (numpy only; independent of oracle.c)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def codebook(cbk):
    out = np.empty(65536, np.uint16)
    lib.orc_exl3_codebook(cbk, _p(out))
    return out


def tile_states(tile, bits):
    tile = _c(tile, np.int16)
    out = np.empty(256, np.uint16)
    lib.orc_exl3_tile_states(_p(tile), bits, _p(out))
    return out


def decode_inner(trellis, cbk):
    trellis = _c(trellis, np.int16)
    Kt, Nt, W = trellis.shape
    bits = W // 16
    out = np.empty((Kt * 16, Nt * 16), np.uint16)
    lib.orc_exl3_decode_inner(_p(trellis), Kt, Nt, bits, cbk, _p(out))
    return out


def fwht128(v):
    v = np.array(v, np.float32).copy()
    assert v.shape == (128,)
    lib.orc_fwht128(_p(v), 1)
    return v


def had_in(x, suh):
    x, suh = _c(x, np.float32), _c(suh, np.uint16)
    out = np.empty(x.shape[0], np.uint16)
    lib.orc_exl3_had_in(_p(x), _p(suh), x.shape[0], _p(out))
    return out


def decode_weight(trellis, suh, svh, cbk):
    trellis, suh, svh = _c(trellis, np.int16), _c(suh, np.uint16), _c(svh, np.uint16)
    Kt, Nt, W = trellis.shape
    out = np.empty((Kt * 16, Nt * 16), np.float32)
    lib.orc_exl3_decode_weight(_p(trellis), _p(suh), _p(svh), Kt * 16, Nt * 16, W // 16, cbk, _p(out))
    return out


def fold(trellis, suh, svh, cbk):
    trellis, suh, svh = _c(trellis, np.int16), _c(suh, np.uint16), _c(svh, np.uint16)
    Kt, Nt, W = trellis.shape
    out = np.empty((Nt * 16, Kt * 16), np.uint16)
    lib.orc_exl3_fold(_p(trellis), _p(suh), _p(svh), Kt * 16, Nt * 16, W // 16, cbk, _p(out), Kt * 16)
    return out


def exl3_moe(x, idx, w, experts, E, H, I, bits, cbk, act, add=None):
    """experts: dict e -> 9 numpy arrays (gate_tr, up_tr, down_tr, gate_suh, up_suh, down_suh, gate_svh, up_svh, down_svh)
    for every expert id in idx.  x float32 [R, H]."""
    x, idx, w = _c(x, np.float32), _c(idx, np.int32), _c(w, np.float32)
    R, topk = idx.shape
    tab = (C.c_void_p * (9 * E))()
    keep = []
    for e, arrs in experts.items():
        for slot, a in enumerate(arrs):
            a = np.ascontiguousarray(a)
            keep.append(a)
            tab[slot * E + e] = a.ctypes.data
    out = np.empty((R, H), np.float32)
    if add is not None:
        add = _c(add, np.float32)
    lib.orc_exl3_moe(_p(x), R, _p(idx), _p(w), C.cast(tab, C.c_void_p), E, topk, H, I, bits, cbk, act, _p(add), _p(out))
    return out


def qwen_route(logits, topk):
    logits = _c(logits, np.float32)
    R, E = logits.shape
    idx, w = np.empty((R, topk), np.int32), np.empty((R, topk), np.float32)
    lib.orc_qwen_route(_p(logits), E, R, E, topk, _p(idx), _p(w))
    return idx, w


def ds41_route(logits, bias, K, scale):
    logits, bias = _c(logits, np.float32), _c(bias, np.float32)
    T, E = logits.shape
    idx, w = np.empty((T, K), np.int64), np.empty((T, K), np.float32)
    lib.orc_ds41_route(_p(logits), _p(bias), _p(idx), _p(w), T, E, K, scale)
    return idx, w


def glm_route(logits, bias, K, scaling):
    logits, bias = _c(logits, np.float32), _c(bias, np.float32)
    T, E = logits.shape
    idx, w = np.empty((T, K), np.int64), np.empty((T, K), np.float32)
    lib.orc_glm_route(_p(logits), _p(bias), _p(idx), _p(w), T, E, K, scaling)
    return idx, w


def mxfp4_dequant(w, s):
    w, s = _c(w, np.uint8), _c(s, np.uint8)
    N, K = w.shape[0], w.shape[1] * 2
    out = np.empty((N, K), np.float32)
    lib.orc_mxfp4_dequant(_p(w), _p(s), N, K, _p(out))
    return out


def fp8_block_dequant(w, s, bs=128):
    w, s = _c(w, np.uint8), _c(s, np.float32)
    N, K = w.shape
    out = np.empty((N, K), np.float32)
    lib.orc_fp8_block_dequant(_p(w), _p(s), N, K, bs, _p(out))
    return out


def fp8_e8m0_dequant(w, s):
    w, s = _c(w, np.uint8), _c(s, np.uint8)
    N, K = w.shape
    out = np.empty((N, K), np.float32)
    lib.orc_fp8_e8m0_dequant(_p(w), _p(s), N, K, _p(out))
    return out


def act_quant_fp8(x_bits):
    x_bits = _c(x_bits, np.uint16)
    q = np.empty(x_bits.shape, np.uint8)
    s = np.empty(x_bits.shape[:-1] + (x_bits.shape[-1] // 32,), np.uint8)
    lib.orc_act_quant_fp8(_p(x_bits), _p(q), _p(s), x_bits.size)
    return q, s


def requant_fp8(wq, ws):
    """reference ds41_mx.cu:333-353 (requant_fp8_kernel): E4M3 bytes [R, K] with an E8M0 byte per 32 [R, K/32] -> act_quant_fp8 of
    byte x 2^(scale - 127) rounded to bf16 (kern.rs:1820-1828 checks it against exactly that composition).  Test infrastructure."""
    wq, ws = _c(wq, np.uint8), _c(ws, np.uint8)
    e4 = np.array([lib.orc_e4m3_to_f32(b) for b in range(256)], np.float32)
    e8 = np.array([lib.orc_e8m0_to_f32(b) for b in range(256)], np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        v = e4[wq] * np.repeat(e8[ws], 32, axis=-1)
    return act_quant_fp8(bf16_bits(v))


def act_quant32(x_bits):
    x_bits = _c(x_bits, np.uint16)
    out = np.empty_like(x_bits)
    lib.orc_act_quant32(_p(x_bits), _p(out), x_bits.size)
    return out


def swiglu_quant(gu, lim):
    """gu f32 [T, 2I] -> bf16 bits [T, I]."""
    gu = _c(gu, np.float32)
    T, I2 = gu.shape
    out = np.empty((T, I2 // 2), np.uint16)
    lib.orc_swiglu_quant(_p(gu), _p(out), T, I2 // 2, float(lim))
    return out


def silu_mul(g, u):
    g, u = _c(g, np.float32), _c(u, np.float32)
    h = np.empty_like(g)
    lib.orc_silu_mul(_p(g), _p(u), _p(h), g.size)
    return h


def gate_scale(gl, col, d):
    """gl f32 [R, ldg], d f32 [R, N] -> sigmoid(gl[:, col])[:, None] * d."""
    gl, d = _c(gl, np.float32), _c(d, np.float32)
    out = np.empty_like(d)
    lib.orc_gate_scale(_p(gl), gl.shape[1], int(col), _p(d), _p(out), d.shape[0], d.shape[1])
    return out


def mxfp4_moe(x_bits, idx, rw, w1, s1, w3, s3, w2, s2, n_shared=0, add=None, want_pairs=False, want_h=False):
    """Stacked natural-layout weights [E(+n_shared), ...]; x bf16 bits [R, H].  want_h: also the act-quantised intermediate of
    every pair (routed pairs first, then the shared ones): E4M3 codes [P + R * n_shared, I], scale bytes [.., I / 32] and each
    element's rounding margin [.., I] (the relative error of its sums or product it takes to change one of its bf16 roundings)."""
    x_bits, idx, rw = _c(x_bits, np.uint16), _c(idx, np.int64), _c(rw, np.float32)
    arrs = [_c(a, np.uint8) for a in (w1, s1, w3, s3, w2, s2)]
    R, H = x_bits.shape
    topk = idx.shape[1]
    I = arrs[0].shape[1]
    E = arrs[0].shape[0] - n_shared
    y = np.empty((R, H), np.float32)
    pairs = np.empty((R * topk, H), np.float32) if want_pairs else None
    hq = np.empty((R * (topk + n_shared), I), np.uint8) if want_h else None
    hs = np.empty((R * (topk + n_shared), I // 32), np.uint8) if want_h else None
    hm = np.empty((R * (topk + n_shared), I), np.float32) if want_h else None
    if add is not None:
        add = _c(add, np.float32)
    lib.orc_mxfp4_moe(_p(x_bits), R, _p(idx), _p(rw), *[_p(a) for a in arrs], H, I, topk, E, n_shared, _p(add), _p(y), _p(pairs), _p(hq), _p(hs), _p(hm))
    out = (y,) + ((pairs,) if want_pairs else ()) + ((hq, hs, hm) if want_h else ())
    return out if len(out) > 1 else y


def mxfp4_moe_from_h(hq, hs, idx, w2, s2, n_shared=0, add=None):
    """The down products and the sum of a given intermediate (codes hq [R * topk + R * n_shared, I], scale bytes hs, pairs ordered as
    mxfp4_moe(want_h=True) returns them); w2, s2 stacked [E + n_shared, H, ...]."""
    hq, hs, idx = _c(hq, np.uint8), _c(hs, np.uint8), _c(idx, np.int64)
    w2, s2 = _c(w2, np.uint8), _c(s2, np.uint8)
    R, topk = idx.shape
    H, I = w2.shape[1], w2.shape[2] * 2
    E = w2.shape[0] - n_shared
    y = np.empty((R, H), np.float32)
    if add is not None:
        add = _c(add, np.float32)
    lib.orc_mxfp4_moe_from_h(_p(hq), _p(hs), R, _p(idx), _p(w2), _p(s2), H, I, topk, E, n_shared, _p(add), _p(y))
    return y


def mxfp4_gemv(x_bits, w, s):
    x_bits, w, s = _c(x_bits, np.uint16), _c(w, np.uint8), _c(s, np.uint8)
    m, k = x_bits.shape
    n = w.shape[0]
    y = np.empty((m, n), np.float32)
    lib.orc_mxfp4_gemv(_p(x_bits), _p(w), _p(s), _p(y), m, n, k)
    return y


def fp8_block_gemv(x_bits, w, s, bs=128):
    x_bits, w, s = _c(x_bits, np.uint16), _c(w, np.uint8), _c(s, np.float32)
    m, k = x_bits.shape
    n = w.shape[0]
    y = np.empty((m, n), np.float32)
    lib.orc_fp8_block_gemv(_p(x_bits), _p(w), _p(s), _p(y), m, n, k, bs)
    return y


def fp8_e8m0_gemv(x_bits, w, s):
    x_bits, w, s = _c(x_bits, np.uint16), _c(w, np.uint8), _c(s, np.uint8)
    m, k = x_bits.shape
    n = w.shape[0]
    y = np.empty((m, n), np.float32)
    lib.orc_fp8_e8m0_gemv(_p(x_bits), _p(w), _p(s), _p(y), m, n, k)
    return y


def fp8_rowscale_gemv(x, w, scale, act=0, rounded=False):
    """x f32 [m, k] (act 0: rounded to f16, 1: to bf16, 2: as given), w E4M3 [n, k], scale f32 [n] -> y f32 [m, n]."""
    x, w, scale = _c(x, np.float32), _c(w, np.uint8), _c(scale, np.float32)
    m, k = x.shape
    n = w.shape[0]
    y = np.empty((m, n), np.float32)
    lib.orc_fp8_rowscale_gemv(_p(x), _p(w), _p(scale), _p(y), m, n, k, act, int(rounded))
    return y


def fp8_rowscale_quant(w):
    """w f32 [n, k] -> (E4M3 codes [n, k], scales f32 [n]) by the reference's row-amax rule."""
    w = _c(w, np.float32)
    n, k = w.shape
    q = np.empty((n, k), np.uint8)
    s = np.empty(n, np.float32)
    lib.orc_fp8_rowscale_quant(_p(w), _p(q), _p(s), n, k)
    return q, s


def num_threads():
    return lib.orc_num_threads()
