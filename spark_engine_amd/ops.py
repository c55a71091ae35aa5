"""Host-side mirror of the reference engine's kernel wrappers (engine-rs/src/ds41/kern.rs, src/qwen/ffi.rs,
src/moe_own.rs): tensors in, raw device pointers + the current stream into the C ABI, a non-zero return code raises
(the Rust wrappers `assert_eq!(rc, 0)`).  torch is used for device memory and the stream only.
"""
import ctypes as C
import weakref

import torch

from . import lib as _l


class KernelError(RuntimeError):
    pass


def _lib():
    return _l.load()


def _st():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _ck(rc, name):
    if rc != 0:
        raise KernelError(f"{name} returned {rc}")


def _fresh_ws(nbytes, device):
    """A new, unprepared workspace.  The allocator may hand out the address of a prepared workspace that has been freed since:
    the library must not mistake it for that one."""
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    _lib().spark_moe_ws_release(_p(ws))
    return ws


def _prepared_ws(ws, init, name):
    """Prepares ws with the given *_ws_init and makes sure the library forgets the address when the tensor goes away."""
    _ck(init(_p(ws), ws.numel(), _st()), name)
    weakref.finalize(ws, _lib().spark_moe_ws_release, C.c_void_p(ws.data_ptr()))
    return ws


def _dev(t):
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensor expected"
    return t


# ---------------------------------------------------------------- dequantisation surfaces

def exl3_reconstruct(trellis, codebook=2):
    """trellis int16 [Kt, Nt, 16*bits] -> inner fp16 [K, N].  reference qwen_exl3.cu qwen_exl3_reconstruct."""
    Kt, Nt, W = trellis.shape
    out = torch.empty(Kt * 16, Nt * 16, dtype=torch.float16, device=trellis.device)
    _ck(_lib().spark_exl3_reconstruct(_p(_dev(trellis)), _p(out), Kt * 16, Nt * 16, W // 16, codebook, _st()), "spark_exl3_reconstruct")
    return out


def exl3_fold(trellis, suh, svh, codebook=2):
    """-> W^T fp16 [N, K].  reference qwen_exl3.cu qwen_exl3_fold."""
    Kt, Nt, W = trellis.shape
    K, N = Kt * 16, Nt * 16
    out = torch.empty(N, K, dtype=torch.float16, device=trellis.device)
    _ck(_lib().spark_exl3_fold(_p(_dev(trellis)), _p(_dev(suh)), _p(_dev(svh)), K, N, W // 16, codebook, _p(out), K, _st()), "spark_exl3_fold")
    return out


# ---------------------------------------------------------------- dense EXL3 linears (reference qwen/ffi.rs exl3_* wrappers)

def exl3_had_in(x, suh):
    """x f32 | f16 [M, K] -> xh f16 [M, K] = had128(x * suh)."""
    M, K = x.shape
    xh = torch.empty(M, K, dtype=torch.float16, device=x.device)
    _ck(_lib().qwen_exl3_had_in(_p(x), int(x.dtype == torch.float32), x.stride(0), _p(_dev(suh)), _p(xh), M, K, _st()), "qwen_exl3_had_in")
    return xh


def exl3_gemv(xh, trellis, S=4):
    """xh f16 [M, K], trellis int16 [K/16, N/16, 16*bits] -> part f32 [S, M, N]."""
    M, K = xh.shape
    Kt, Nt, W = trellis.shape
    part = torch.empty(S, M, Nt * 16, dtype=torch.float32, device=xh.device)
    _ck(_lib().qwen_exl3_gemv(_p(_dev(xh)), _p(_dev(trellis)), _p(part), M, K, Nt * 16, W // 16, S, _st()), "qwen_exl3_gemv")
    return part


def exl3_finish(part, svh, f32=True):
    S, M, N = part.shape
    y = torch.empty(M, N, dtype=torch.float32 if f32 else torch.float16, device=part.device)
    _ck(_lib().qwen_exl3_finish(_p(_dev(part)), S, _p(_dev(svh)), _p(y), int(f32), N, M, N, _st()), "qwen_exl3_finish")
    return y


def exl3_linear(x, suh, trellis, svh, S=4, counters=False):
    """x f32 [M, K] -> y f32 [M, N] (had_in + gemv + finish).  counters: hand the entry point its counter array (one launch
    where it can); returns (y, cnt)."""
    M, K = x.shape
    Kt, Nt, W = trellis.shape
    N = Nt * 16
    part = torch.empty(S, M, N, dtype=torch.float32, device=x.device)
    y = torch.empty(M, N, dtype=torch.float32, device=x.device)
    cnt = torch.zeros(N // 128, dtype=torch.int32, device=x.device) if counters else None      # zero before, zero after (reference qwen_exl3.cu:148-149)
    _ck(_lib().qwen_exl3_linear(_p(x), x.stride(0), _p(_dev(suh)), _p(_dev(trellis)), _p(_dev(svh)), _p(part), _p(y), N, _p(cnt), M, K, N, W // 16, S, _st()),
        "qwen_exl3_linear")
    if counters:
        return y, cnt
    return y


def exl3_multi(x, linears, S=4, silu=False, mix=None):
    """x f32 [M, K]; linears = [(suh, trellis, svh), ...] (at most 4) -> list of y f32 [M, N_i] (one tensor with silu).
    mix = (g, n), both f32 [M, 4, K]: the input is the gated mean of the four streams (x is ignored); returns (ys, xout)."""
    M, K = (mix[0].shape[0], mix[0].shape[2]) if mix is not None else x.shape
    n = len(linears)
    if mix is not None:
        xout = torch.empty(M, K, dtype=torch.float32, device=mix[0].device)
        x = xout
    Ns = [lin[1].shape[1] * 16 for lin in linears]
    bits = [lin[1].shape[2] // 16 for lin in linears]
    parts = [torch.empty(S, M, N, dtype=torch.float32, device=x.device) for N in Ns]
    ys = [torch.empty(M, N, dtype=torch.float32, device=x.device) for N in Ns]
    vpa = lambda ts: (C.c_void_p * n)(*[t.data_ptr() for t in ts])
    ia = lambda vs: (C.c_int * n)(*vs)
    mg, mn, xo = (_p(_dev(mix[0])), _p(_dev(mix[1])), _p(xout)) if mix is not None else (None, None, None)
    _ck(_lib().qwen_exl3_multi(_p(x), x.stride(0), mg, mn, xo, M, K, n, vpa([lin[0] for lin in linears]), None, vpa([lin[1] for lin in linears]),
                               vpa(parts), ia(Ns), ia([S] * n), vpa([lin[2] for lin in linears]), vpa(ys), (C.c_int64 * n)(*Ns), ia(bits), int(silu), _st()),
        "qwen_exl3_multi")
    res = ys[0] if (int(silu) & 1) else ys
    return (res, xout) if mix is not None else res


def mxfp4_dequant(w, s):
    N, K = w.shape[0], w.shape[1] * 2
    out = torch.empty(N, K, dtype=torch.float32, device=w.device)
    _ck(_lib().spark_mxfp4_dequant(_p(_dev(w)), _p(_dev(s)), _p(out), N, K, _st()), "spark_mxfp4_dequant")
    return out


def fp8_block_dequant(w, s, bs=128):
    N, K = w.shape
    out = torch.empty(N, K, dtype=torch.float32, device=w.device)
    _ck(_lib().spark_fp8_block_dequant(_p(_dev(w)), _p(_dev(s)), _p(out), N, K, bs, _st()), "spark_fp8_block_dequant")
    return out


def fp8_e8m0_dequant(w, s):
    N, K = w.shape
    out = torch.empty(N, K, dtype=torch.float32, device=w.device)
    _ck(_lib().spark_fp8_e8m0_dequant(_p(_dev(w)), _p(_dev(s)), _p(out), N, K, _st()), "spark_fp8_e8m0_dequant")
    return out


# ---------------------------------------------------------------- act_quant (reference kern.rs act_quant / act_quant_fp8)

def act_quant(x):
    """bf16 -> quantize-dequantize bf16 (UE8M0 per 32)."""
    out = torch.empty_like(x)
    _ck(_lib().ds41_act_quant32(_p(_dev(x)), _p(out), x.numel(), _st()), "ds41_act_quant32")
    return out


def act_quant_fp8(x):
    """bf16 [R, K] -> (q uint8 [R, K], s uint8 [R, K/32])."""
    x = _dev(x)
    q = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    s = torch.empty(*x.shape[:-1], x.shape[-1] // 32, dtype=torch.uint8, device=x.device)
    _ck(_lib().ds41_act_quant_fp8(_p(x), _p(q), _p(s), x.numel(), _st()), "ds41_act_quant_fp8")
    return q, s


def requant_fp8(wq, ws):
    """reference kern.rs:780-789 (requant_fp8): rows stored as E4M3 bytes wq [R, K] with E8M0 bytes ws [R, K/32] -> the bytes
    act_quant_fp8 gives their bf16 dequantisation, (q uint8 [R, K], s uint8 [R, K/32])."""
    wq, ws = _dev(wq), _dev(ws)
    assert wq.numel() == ws.numel() * 32
    q, s = torch.empty_like(wq), torch.empty_like(ws)
    _ck(_lib().ds41_requant_fp8(_p(wq), _p(ws), _p(q), _p(s), wq.numel(), _st()), "ds41_requant_fp8")
    return q, s


def swiglu_quant(gu, lim):
    T, I2 = gu.shape
    out = torch.empty(T, I2 // 2, dtype=torch.bfloat16, device=gu.device)
    _ck(_lib().ds41_swiglu_quant(_p(_dev(gu)), _p(out), T, I2 // 2, float(lim), _st()), "ds41_swiglu_quant")
    return out


def silu_mul(g, u):
    """reference qwen/ffi.rs moe_silu_mul (qwen_moe_silu_mul): h = silu(g) * u, f32."""
    h = torch.empty_like(g)
    _ck(_lib().qwen_moe_silu_mul(_p(_dev(g)), _p(_dev(u)), _p(h), g.numel(), _st()), "qwen_moe_silu_mul")
    return h


def gate_scale(gl, col, d):
    """reference qwen/ffi.rs moe_gate_scale (qwen_moe_gate_scale): out[r] = sigmoid(gl[r, col]) * d[r], f32."""
    R, N = d.shape
    out = torch.empty_like(d)
    _ck(_lib().qwen_moe_gate_scale(_p(gl), gl.stride(0), int(col), _p(_dev(d)), _p(out), R, N, _st()), "qwen_moe_gate_scale")
    return out


# ---------------------------------------------------------------- single-launch workspaces

def ws_status(ws):
    """Waits for the current stream and returns the workspace's bounded-wait flag (0 = no wait of any call has expired)."""
    return _lib().spark_moe_ws_status(_p(ws), _st())


def ws_check(ws, what="single-launch workspace"):
    """Raises if a bounded wait of a single-launch call expired on this workspace (its outputs are then stale)."""
    rc = ws_status(ws)
    if rc != 0:
        raise KernelError(f"{what}: spark_moe_ws_status returned {rc} (a bounded wait expired; prepare the workspace again)")


def ws_release(ws):
    _lib().spark_moe_ws_release(_p(ws))


# ---------------------------------------------------------------- routers

def softmax_route(logits, topk):
    """reference qwen/ffi.rs moe_route: logits f32 [R, E] -> (idx int32 [R, topk], w f32)."""
    R, E = logits.shape
    idx = torch.empty(R, topk, dtype=torch.int32, device=logits.device)
    w = torch.empty(R, topk, dtype=torch.float32, device=logits.device)
    _ck(_lib().spark_softmax_route(_p(_dev(logits)), logits.stride(0), R, E, topk, _p(idx), _p(w), _st()), "spark_softmax_route")
    return idx, w


def qwen_moe_route(logits):
    R = logits.shape[0]
    idx = torch.empty(R, 10, dtype=torch.int32, device=logits.device)
    w = torch.empty(R, 10, dtype=torch.float32, device=logits.device)
    _ck(_lib().qwen_moe_route_ld(_p(logits), logits.stride(0), R, _p(idx), _p(w), _st()), "qwen_moe_route_ld")
    return idx, w


def route(logits, bias, k, scale):
    """reference kern.rs route (ds41_route): -> (idx int64 [T, k], w f32 [T, k])."""
    T, E = logits.shape
    idx = torch.empty(T, k, dtype=torch.int64, device=logits.device)
    w = torch.empty(T, k, dtype=torch.float32, device=logits.device)
    _ck(_lib().ds41_route(_p(_dev(logits)), _p(_dev(bias)), _p(idx), _p(w), T, E, k, float(scale), _st()), "ds41_route")
    return idx, w


def sigmoid_route(logits, bias, k, scaling):
    T, E = logits.shape
    idx = torch.empty(T, k, dtype=torch.int64, device=logits.device)
    w = torch.empty(T, k, dtype=torch.float32, device=logits.device)
    _ck(_lib().spark_sigmoid_route(_p(_dev(logits)), _p(_dev(bias)), _p(idx), _p(w), T, E, k, float(scaling), _st()), "spark_sigmoid_route")
    return idx, w


def glm_router_fused(h, w, bias, scaling, half_w=False):
    """reference moe.rs route() -> rs_router_fused(_h) -> glm53_router_fused(_h)_cuda: h f32 [rows, k], w f32|bf16 [E, k].
    half_w: also returns the binary16 copy of the weights that glm_moe_experts takes (reference moe.rs:66-67)."""
    rows, k = h.shape
    E = w.shape[0]
    partial = torch.empty(rows, E, 2, dtype=torch.float32, device=h.device)
    ids = torch.empty(rows, 8, dtype=torch.int64, device=h.device)
    wt = torch.empty(rows, 8, dtype=torch.float32, device=h.device)
    if half_w:
        wh = torch.empty(rows, 8, dtype=torch.float16, device=h.device)
        _ck(_lib().glm53_router_fused_h_cuda(_p(_dev(h)), _p(_dev(w)), int(w.dtype == torch.bfloat16), _p(_dev(bias)), _p(partial), _p(ids), _p(wt),
                                             _p(wh), rows, E, k, float(scaling), _st()), "glm53_router_fused_h_cuda")
        return ids, wt, wh
    _ck(_lib().glm53_router_fused_cuda(_p(_dev(h)), _p(_dev(w)), int(w.dtype == torch.bfloat16), _p(_dev(bias)), _p(partial), _p(ids), _p(wt),
                                       rows, E, k, float(scaling), _st()), "glm53_router_fused_cuda")
    return ids, wt


# ---------------------------------------------------------------- dense GEMVs (reference kern.rs mxfp4_gemv / fp8_gemv)

def mxfp4_gemv(x, w, s):
    m, k = x.shape
    n = w.shape[0]
    y = torch.empty(m, n, dtype=torch.float32, device=x.device)
    _ck(_lib().ds41_mxfp4_gemv(_p(_dev(x)), _p(_dev(w)), _p(_dev(s)), _p(y), m, n, k, _st()), "ds41_mxfp4_gemv")
    return y


def fp8_gemv(x, w, s):
    m, k = x.shape
    n = w.shape[0]
    y = torch.empty(m, n, dtype=torch.float32, device=x.device)
    _ck(_lib().ds41_fp8_gemv(_p(_dev(x)), _p(_dev(w)), _p(_dev(s)), _p(y), m, n, k, _st()), "ds41_fp8_gemv")
    return y


def fp8_gemv_bx(x, w, s, rpg=0):
    """reference kern.rs fp8_gemv_bx (ds41_fp8_gemv_bx): up to 16 rows; rpg > 0 = block-diagonal groups of rpg weight rows."""
    m = x.shape[0]
    n = w.shape[0]
    k = w.shape[1]
    y = torch.empty(m, n, dtype=torch.float32, device=x.device)
    _ck(_lib().ds41_fp8_gemv_bx(_p(_dev(x)), _p(_dev(w)), _p(_dev(s)), _p(y), m, n, k, x.stride(0), rpg, _st()), "ds41_fp8_gemv_bx")
    return y


def fp8_gemv_mx(x, w, s, aq=None, as_=None, bf16_out=False):
    """reference kern.rs fp8_gemv_mx / fp8_gemv_mx_bf16 (ds41_fp8_gemv_mx_q): FP8 weights x act-quantised activations, up to 32 rows;
    x bf16 [m, k] is quantised inside unless the quantised pair (aq, as_) is given."""
    m = (x if aq is None else aq).shape[0]
    n, k = w.shape
    y = torch.empty(m, n, dtype=torch.bfloat16 if bf16_out else torch.float32, device=w.device)
    _ck(_lib().ds41_fp8_gemv_mx_q(_p(x), _p(aq), _p(as_), _p(_dev(w)), _p(_dev(s)), _p(y), m, n, k, int(bf16_out), _st()), "ds41_fp8_gemv_mx_q")
    return y


def gemv_mx(x, w, s, bf16_out=False, preq_rows=2, preq_k1=True):
    """The caller's side of fp8_gemv_mx as the reference has it (kern.rs:899-917 gemv_mx): x bf16 [m, k] is handed over to be
    quantised inside while m (k + k / 32) fits ds41_fp8_gemv_mx_smem_max(), m < preq_rows (DS41_GEMV_PREQ_ROWS, default 2) and
    not (m == 1 and k >= 4096, DS41_GEMV_PREQ_K1); else ds41_act_quant_fp8 runs first and the codes are handed over.  Both
    ways give a row the same bits, whatever m (the property kern.rs:1885-1898 tests over the model's shapes)."""
    m, k = x.shape
    fits = m * k + m * k // 32 <= _lib().ds41_fp8_gemv_mx_smem_max() and m < preq_rows and not (m == 1 and k >= 4096 and preq_k1)
    if fits:
        return fp8_gemv_mx(_dev(x).contiguous(), w, s, bf16_out=bf16_out)
    aq, as_ = act_quant_fp8(_dev(x).contiguous())
    return fp8_gemv_mx(None, w, s, aq=aq, as_=as_, bf16_out=bf16_out)


def fp8_block128_gemv(x, w, scales, y=None):
    m, k = x.shape
    n = w.shape[0]
    if y is None:
        y = torch.empty(m, n, dtype=torch.float32, device=x.device)
    _ck(_lib().spark_fp8_block128_gemv(_p(_dev(x)), _p(_dev(w)), _p(_dev(scales)), _p(y), m, n, k, _st()), "spark_fp8_block128_gemv")
    return y


def fp8_t16_pack(w):
    """E4M3 [n, k] (uint8) -> the same bytes in the matrix unit's operand order (tiles of 16 rows x 128 k), once per matrix."""
    n, k = w.shape
    out = torch.empty(n * k, dtype=torch.uint8, device=w.device)
    _ck(_lib().spark_fp8_t16_pack(_p(_dev(w)), _p(out), n, k, _st()), "spark_fp8_t16_pack")
    return out


def fp8_block128_gemv_t16(x, wt, scales, n, y=None):
    """x bf16 [m, k] times a matrix packed by fp8_t16_pack, fp32 scales per 128 x 128 block: up to 16 rows at one cost."""
    m, k = x.shape
    if y is None:
        y = torch.empty(m, n, dtype=torch.float32, device=x.device)
    _ck(_lib().spark_fp8_block128_gemv_t16(_p(_dev(x)), _p(wt), _p(_dev(scales)), _p(y), m, n, k, _st()), "spark_fp8_block128_gemv_t16")
    return y


def fp8_e8m0_gemv_t16(x, wt, scales, n, y=None):
    """x bf16 [m, k] times a matrix packed by fp8_t16_pack with E8M0 scales [n / 32, k / 32] (the product of fp8_gemv)."""
    m, k = x.shape
    if y is None:
        y = torch.empty(m, n, dtype=torch.float32, device=x.device)
    _ck(_lib().spark_fp8_e8m0_gemv_t16(_p(_dev(x)), _p(wt), _p(_dev(scales)), _p(y), m, n, k, _st()), "spark_fp8_e8m0_gemv_t16")
    return y


def fp8_rowscale_quantize(w):
    """reference engine-rs/src/dense_fp8.rs:59-62 (quantize): one scale per output row = row amax / 448, codes = E4M3 of w / scale.
    w [n, k] f32 | f16 | bf16 -> (E4M3 bytes [n, k] as uint8, scales f32 [n])."""
    wf = w.float()
    # the two binary32 divisions through binary64 (correctly rounded either way: a device division may be a multiplication by 1 / 448)
    scale = (wf.abs().amax(dim=1, keepdim=True).clamp_min(1e-12).double() / 448.0).float()
    q = (wf.double() / scale.double()).float().clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.view(torch.uint8), scale.view(-1).contiguous()


def glm_fp8_dense(x, wq, scales, rounded=False, act="f16"):
    """reference engine-rs/src/dense_fp8.rs run / cached -> glm53_fp8_dense_cuda (act f16) | glm53_fp8_bf16_cuda (act bf16) |
    glm53_fp8_bf16_skinny_cuda (x given as bf16): x [m, k] -> y f32 [m, n]."""
    m, k = x.shape
    n = wq.shape[0]
    y = torch.empty(m, n, dtype=torch.float32, device=x.device)
    L = _lib()
    if x.dtype == torch.bfloat16:
        _ck(L.glm53_fp8_bf16_skinny_cuda(_p(_dev(x)), _p(_dev(wq)), _p(_dev(scales)), _p(y), m, n, k, _st()), "glm53_fp8_bf16_skinny_cuda")
    elif act == "bf16":
        _ck(L.glm53_fp8_bf16_cuda(_p(_dev(x)), _p(_dev(wq)), _p(_dev(scales)), _p(y), None, m, n, k, 1, _st()), "glm53_fp8_bf16_cuda")
    else:
        _ck(L.glm53_fp8_dense_cuda(_p(_dev(x)), _p(_dev(wq)), _p(_dev(scales)), _p(y), None, m, n, k, int(rounded), 1, 0, _st()), "glm53_fp8_dense_cuda")
    return y


def bf16_gemv(x, w):
    m, k = x.shape
    n = w.shape[0]
    y = torch.empty(m, n, dtype=torch.float32, device=x.device)
    _ck(_lib().ds41_bf16_gemv(_p(_dev(x)), _p(_dev(w)), _p(y), m, n, k, _st()), "ds41_bf16_gemv")
    return y


def bf16_gemv_rows(x, w):
    """reference kern.rs:249-259 (bf16_gemv_rows): bf16_gemv for up to 16 rows (ds41_bf16_gemv_mx where the shape allows it)."""
    m, k = x.shape
    n = w.shape[0]
    if m == 1 or n % 8 != 0 or k % 32 != 0 or m > 16:
        return bf16_gemv(x, w)
    y = torch.empty(m, n, dtype=torch.float32, device=x.device)
    _ck(_lib().ds41_bf16_gemv_mx(_p(_dev(x)), _p(_dev(w)), _p(y), m, n, k, _st()), "ds41_bf16_gemv_mx")
    return y


# ---------------------------------------------------------------- MXFP4 MoE

class Mxfp4Experts:
    """Stacked expert weights of one layer resident on the GPU (E routed + n_shared shared experts), packed once into
    the matrix-unit record layout, like the reference packs at load (kern.rs moe_pack / moe_pack_mx)."""

    def __init__(self, w1, s1, w3, s3, w2, s2, n_shared=0, keep_natural=False):
        ET, I, H2 = w1.shape
        self.E, self.n_shared, self.I, self.H = ET - n_shared, n_shared, I, H2 * 2
        self.packed = [self._pack(w1, s1), self._pack(w3, s3), self._pack(w2, s2)]
        self.natural = (w1, s1, w3, s3, w2, s2) if keep_natural else None

    @staticmethod
    def _pack(w, s):
        rows, K = w.shape[0] * w.shape[1], w.shape[2] * 2
        nbytes = _lib().spark_mxfp4_packed_bytes(rows, K)
        if nbytes == 0:
            raise KernelError(f"spark_mxfp4_packed_bytes: unsupported shape rows {rows} K {K}")
        out = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
        _ck(_lib().spark_mxfp4_prepack(_p(_dev(w)), _p(_dev(s)), _p(out), rows, K, _st()), "spark_mxfp4_prepack")
        return out


def mxfp4_moe_ws(R, ex, topk):
    n = _lib().spark_mxfp4_moe_ws_bytes(R, ex.H, ex.I, topk, ex.E, ex.n_shared)
    if n == 0:
        raise KernelError("spark_mxfp4_moe_ws_bytes: unsupported shape")
    return n


def mxfp4_moe(x, idx, rw, ex, add=None, y=None, ws=None, scratch=None, natural=False):
    """x bf16 [R, H] -> y f32 [R, H] (reference kern.rs moe_mx: act_quant_fp8 + ds41_moe_mx, with runtime sizes and the
    shared experts folded in)."""
    R, H = x.shape
    topk = idx.shape[1]
    dev = x.device
    if y is None:
        y = torch.empty(R, H, dtype=torch.float32, device=dev)
    if ws is None:
        ws = _fresh_ws(mxfp4_moe_ws(R, ex, topk), dev)
    if scratch is None:
        scratch = (torch.empty(R, H, dtype=torch.uint8, device=dev), torch.empty(R, H // 32, dtype=torch.uint8, device=dev))
    if natural:
        w1, s1, w3, s3, w2, s2 = ex.natural
        layout = 1
    else:
        (w1, w3, w2), (s1, s3, s2), layout = ex.packed, (None, None, None), 0
    _ck(_lib().spark_mxfp4_moe(_p(_dev(x)), _p(scratch[0]), _p(scratch[1]), R, _p(_dev(idx)), _p(_dev(rw)), _p(w1), _p(s1), _p(w3), _p(s3), _p(w2), _p(s2),
                               layout, H, ex.I, topk, ex.E, ex.n_shared, _p(add), _p(y), _p(ws), _st()), "spark_mxfp4_moe")
    return y


def mxfp4_moe_ws_alloc(R, ex, topk, device="cuda:0"):
    """A workspace prepared once (spark_mxfp4_moe_ws_init): calls of mxfp4_moe_x with ws_clean=True then run as one launch."""
    return _prepared_ws(torch.empty(mxfp4_moe_ws(R, ex, topk), dtype=torch.uint8, device=device), _lib().spark_mxfp4_moe_ws_init, "spark_mxfp4_moe_ws_init")


def mxfp4_moe_x(x, idx, rw, ex, xs=None, add=None, y=None, ws=None, ws_clean=False, multi_kernel=False, natural=False, out_bf16=False):
    """The decode entry (R <= 8): x bf16 [R, H] (quantised inside the kernel) or E4M3 bytes with scales xs -> y f32 [R, H] (bf16 with out_bf16)."""
    R, H = x.shape
    topk = idx.shape[1]
    dev = x.device
    if y is None:
        y = torch.empty(R, H, dtype=torch.bfloat16 if out_bf16 else torch.float32, device=dev)
    if ws is None:
        ws = _fresh_ws(mxfp4_moe_ws(R, ex, topk), dev)
        ws_clean = False
    if natural:
        w1, s1, w3, s3, w2, s2 = ex.natural
        layout = 1
    else:
        (w1, w3, w2), (s1, s3, s2), layout = ex.packed, (None, None, None), 0
    flags = (1 if ws_clean else 0) | (2 if multi_kernel else 0) | (16 if out_bf16 else 0)
    _ck(_lib().spark_mxfp4_moe_x(_p(_dev(x)), _p(xs), R, _p(_dev(idx)), _p(_dev(rw)), _p(w1), _p(s1), _p(w3), _p(s3), _p(w2), _p(s2),
                                 layout, H, ex.I, topk, ex.E, ex.n_shared, _p(add), _p(y), _p(ws), flags, _st()), "spark_mxfp4_moe_x")
    return y


# reference tile layouts (kern.rs:718-734), restated with tensor view/permute exactly as the Rust does
def moe_pack(w, s):
    e, rows, kb = w.shape
    steps = kb // 64
    wp = w.view(e * rows // 8, 8, steps, 4, 16).permute(0, 2, 1, 3, 4).contiguous()
    sp = s.view(e * rows // 8, 8, steps, 4).permute(0, 2, 1, 3).contiguous()
    return wp.view(e, rows, kb), sp.view(e, rows, kb // 16)


def moe_pack_mx(wp):
    e, rows, kb = wp.shape
    steps = kb // 64
    return wp.view(e * rows // 8, steps, 8, 4, 4, 4).permute(0, 1, 2, 4, 3, 5).contiguous().view(e, rows, kb)


def moe_scales_s2(sp):
    """The 2-bit scale blob the ds41_moe_mx* entry points read after moe_s2_set(True) (the format of reference
    engine-rs/shim/ds41_mx.cu:64-91, written there by kern.rs moe_scales_s2).  sp: tile-packed scale bytes [E, rows, K/32] from
    moe_pack.  Per 8-row tile the blob holds a 16-byte descriptor (the eight rows' smallest scale byte, then a little-endian int32:
    the tile's position among the raw tiles, or -1), per tile and 128-wide K step eight code bytes (one per row: the four blocks'
    offsets above the row's smallest byte, two bits each, block 0 lowest), and, for tiles with a row whose bytes span more than 3, the
    tile's raw bytes.  Lossless.  Returns (blob uint8, number of raw tiles, number of tiles)."""
    n_exp, rows, n_blocks = sp.shape
    n_tiles, n_steps = n_exp * rows // 8, n_blocks // 4
    t = sp.reshape(n_tiles, n_steps, 8, 4)                               # [tile][K step][row of the tile][32-block of the step]
    row_min = t.amin(dim=(1, 3))                                         # [tile][row]
    keeps_raw = (t.amax(dim=(1, 3)).int() - row_min.int() > 3).any(dim=1)
    offs = (t - row_min[:, None, :, None]).clamp(max=3)                  # uint8; meaningless (and unread) in raw tiles
    code_bytes = offs[..., 0] | (offs[..., 1] << 2) | (offs[..., 2] << 4) | (offs[..., 3] << 6)
    raw_pos = torch.where(keeps_raw, torch.cumsum(keeps_raw.int(), 0) - 1, torch.full((n_tiles,), -1, device=sp.device)).to(torch.int32)
    desc = torch.zeros(n_tiles, 16, dtype=torch.uint8, device=sp.device)
    desc[:, :8] = row_min
    desc[:, 8:12] = raw_pos.contiguous().view(torch.uint8).view(n_tiles, 4)
    blob = torch.cat([desc.reshape(-1), code_bytes.contiguous().reshape(-1), t[keeps_raw].reshape(-1)])
    return blob.contiguous(), int(keeps_raw.sum().item()), n_tiles


def moe_s2_set(on):
    """reference kern.rs moe_s2_set: the scale tensors handed to ds41_moe_mx* are 2-bit coded blobs."""
    _lib().ds41_moe_mx_set_s2(int(bool(on)))


def ds41_moe_mx(xq, xs, idx, rw, w, I, add=None, skip_combine=False, ws=None):
    """reference kern.rs moe_mx_par / ds41_moe_mx_ex: hidden 5120, weights w = (w1, s1, w3, s3, w2, s2) in the mx tile layout."""
    R = xq.shape[0]
    topk, E = idx.shape[1], w[0].shape[0]
    if xq.shape[1] != 5120 or xs.shape[1] != 160 or (add is not None and tuple(add.shape) != (R, 5120)):
        raise ValueError("ds41_moe_mx is compiled for hidden width 5120 (reference ds41_mx.cu:30); use mxfp4_moe for other widths")
    y = torch.empty(R, 5120, dtype=torch.float32, device=xq.device)
    if ws is None:
        ws = _fresh_ws(_lib().ds41_moe_mx_ws_bytes(R, I, topk, E), xq.device)
    _ck(_lib().ds41_moe_mx_ex(_p(_dev(xq)), _p(_dev(xs)), R, _p(_dev(idx)), _p(_dev(rw)), *[_p(_dev(t)) for t in w], I, _p(add), _p(y), _p(ws), topk, E,
                              int(skip_combine), _st()), "ds41_moe_mx_ex")
    return y, ws


def ds41_moe(xq_bf16, idx, rw, w, I, add=None):
    """reference kern.rs moe (ds41_moe): weights in the moe_pack tile layout, xq the act-quantized input as bf16."""
    R = xq_bf16.shape[0]
    topk, E = idx.shape[1], w[0].shape[0]
    if xq_bf16.shape[1] != 5120 or (add is not None and tuple(add.shape) != (R, 5120)):
        raise ValueError("ds41_moe is compiled for hidden width 5120 (reference ds41_moe.cu:32); use mxfp4_moe for other widths")
    y = torch.empty(R, 5120, dtype=torch.float32, device=xq_bf16.device)
    ws = _fresh_ws(_lib().ds41_moe_ws_bytes(R, I, topk, E), xq_bf16.device)
    _ck(_lib().ds41_moe(_p(_dev(xq_bf16)), R, _p(_dev(idx)), _p(_dev(rw)), *[_p(_dev(t)) for t in w], I, _p(add), _p(y), _p(ws), topk, E, _st()), "ds41_moe")
    return y


# ---------------------------------------------------------------- EXL3 MoE (reference reference/qwen38/kern.py ExpertTable / moe_routed,
# engine-rs/src/qwen/ffi.rs moe_experts, src/moe_own.rs run_into)

class ExpertTable:
    """All experts of one layer resident on the GPU + the [9][E] device-pointer table (gate_tr, up_tr, down_tr,
    gate_suh, up_suh, down_suh, gate_svh, up_svh, down_svh)."""

    def __init__(self, experts, E, device="cuda:0", bits=None, widths=None):
        """experts: dict e -> 9 device tensors (or stacked tensors per slot, see from_stacked).  Missing experts get null pointers.
        bits: dict e -> trellis width of the expert (3..6): adds row 9 of the reference's mixed-width tables (moe_exl3.cuh:239-252).
        widths: dict e -> intermediate width of the expert: adds row 10 (and row 9, 4 bits unless bits is given) of the reference's
        variable-width tables (moe_exl3.cuh:63-67,132-136)."""
        self.E = E
        self.keep = experts
        if bits is not None:
            wrong = {e: b for e, b in bits.items() if int(b) not in (3, 4, 5, 6)}
            if wrong:
                raise ValueError(f"trellis widths are 3..6 bits: {wrong}")
        if widths is not None:
            wrong = {e: v for e, v in widths.items() if int(v) < 128 or int(v) % 128}
            if wrong:
                raise ValueError(f"an expert's intermediate width is a positive multiple of 128: {wrong}")
        rows = [[0] * E for _ in range(11 if widths is not None else 9 if bits is None else 10)]
        for e, ts in experts.items():
            for slot, t in enumerate(ts):
                assert t.is_cuda and t.is_contiguous()
                rows[slot][e] = t.data_ptr()
            if bits is not None or widths is not None:
                rows[9][e] = int(bits[e]) if bits is not None else 4
            if widths is not None:
                rows[10][e] = int(widths[e])
        self.mixed = bits is not None
        self.varw = widths is not None
        self.kmask = 1 << 4 if bits is None else sum({1 << int(b) for b in bits.values()})
        self.tab = torch.tensor(rows, dtype=torch.int64, device=device).contiguous()

    @classmethod
    def from_stacked(cls, stacked, device="cuda:0"):
        """stacked: 9 tensors [E, ...] (one per table slot)."""
        E = stacked[0].shape[0]
        return cls({e: [s[e] for s in stacked] for e in range(E)}, E, device)


_XT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def exl3_moe_ws(R, H, I, E, topk):
    n = _lib().spark_exl3_moe_ws_bytes(R, H, I, E, topk)
    if n == 0:
        raise KernelError("spark_exl3_moe_ws_bytes: unsupported shape")
    return n


def exl3_moe_ws_alloc(R, H, I, E, topk, device="cuda:0"):
    """A workspace zeroed once (spark_exl3_moe_ws_init): calls that pass it with ws_clean=True skip their zeroing launch."""
    return _prepared_ws(torch.empty(exl3_moe_ws(R, H, I, E, topk), dtype=torch.uint8, device=device), _lib().spark_exl3_moe_ws_init, "spark_exl3_moe_ws_init")


def exl3_moe(x, idx, w, table, H, I, codebook=2, act=0, add=None, out=None, ws=None, ws_clean=False, multi_kernel=False, out_bf16=False):
    """x [R, H] f32 | f16 | bf16, idx int32 | int64 [R, topk], w f32 | f16 [R, topk] -> out f32 [R, H] (bf16 with out_bf16)."""
    R, topk = idx.shape
    if out is None:
        out = torch.empty(R, H, dtype=torch.bfloat16 if out_bf16 else torch.float32, device=x.device)
    if ws is None:
        ws = _fresh_ws(exl3_moe_ws(R, H, I, table.E, topk), x.device)
        ws_clean = False
    flags = ((1 if ws_clean else 0) | (2 if multi_kernel else 0) | (4 if getattr(table, "mixed", False) else 0) | (8 if getattr(table, "varw", False) else 0) |
             (16 if out_bf16 else 0))
    _ck(_lib().spark_exl3_moe(_p(x), _XT[x.dtype], x.stride(0), R, _p(_dev(idx)), int(idx.dtype == torch.int64), _p(_dev(w)), int(w.dtype == torch.float16),
                              _p(table.tab), _p(add), _p(out), _p(ws), H, I, table.E, topk, codebook, act, flags, _st()), "spark_exl3_moe")
    return out


def exl3_moe_static(x, idx, w, table, H, I, codebook=2, act=0, add=None, out=None):
    """exl3_moe on the library's own scratch array (spark_exl3_moe_static): no workspace, nothing allocated by the library; decode sizes."""
    R, topk = idx.shape
    if out is None:
        out = torch.empty(R, H, dtype=torch.float32, device=x.device)
    _ck(_lib().spark_exl3_moe_static(_p(x), _XT[x.dtype], x.stride(0), R, _p(_dev(idx)), int(idx.dtype == torch.int64), _p(_dev(w)), int(w.dtype == torch.float16),
                                     _p(table.tab), _p(add), _p(out), H, I, table.E, topk, codebook, act, _st()), "spark_exl3_moe_static")
    return out


def qwen_moe_experts(x, idx, w, table, add=None, S=4):
    """reference qwen/ffi.rs moe_experts: x f32 [R, 2560], 512 experts, top-10."""
    R = x.shape[0]
    ws = _fresh_ws(_lib().qwen_moe_ws_bytes(R, S), x.device)
    out = torch.empty(R, 2560, dtype=torch.float32, device=x.device)
    _ck(_lib().qwen_moe_experts(_p(x), x.stride(0), R, _p(_dev(idx)), _p(_dev(w)), _p(table.tab), _p(add), _p(out), _p(ws), S, _st()), "qwen_moe_experts")
    return out


def glm_moe3_experts(x, idx, w, table, add=None, S=2, kmask=1 << 4):
    """reference moe_own.rs:44-46 (TP3): as glm_moe_experts with every expert 768 or 640 wide (table rows 9 and 10)."""
    R = x.shape[0]
    ws = _fresh_ws(_lib().glm_moe3_ws_bytes(R, S), x.device)
    out = torch.empty(R, 4096, dtype=torch.float32, device=x.device)
    _ck(_lib().glm_moe3_experts(_p(x), x.stride(0), R, _p(_dev(idx)), _p(_dev(w)), _p(table.tab), _p(add), _p(out), _p(ws), S, kmask, _st()), "glm_moe3_experts")
    return out


def glm_moe_experts(x, idx, w, table, add=None, S=2, kmask=1 << 4):
    """reference moe_own.rs run_into: x f16 [R, 4096], idx int64 / w f16 [R, 8], 288 experts, mcg codebook."""
    R = x.shape[0]
    ws = _fresh_ws(_lib().glm_moe_ws_bytes(R, S), x.device)
    out = torch.empty(R, 4096, dtype=torch.float32, device=x.device)
    _ck(_lib().glm_moe_experts(_p(x), x.stride(0), R, _p(_dev(idx)), _p(_dev(w)), _p(table.tab), _p(add), _p(out), _p(ws), S, None, kmask, _st()), "glm_moe_experts")
    return out
