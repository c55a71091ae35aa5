#!/usr/bin/env python3
"""Benchmark of the decode-time quantized MoE expert path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one MoE layer call (router top-k + routed experts) on one batch of synthetic input.  The headline workload
is the Qwen-style EXL3 4-bit layer at batch 1 (hidden 2048, expert intermediate 512, 512 experts, top-10).  Steps run
from a HIP graph of many layer instances with fresh routes each, so successive steps stream different experts and the
weights come from HBM, not from the L2 or the Infinity Cache.  Prints ONE JSON line.
"""
import argparse
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
FP8_PEAK_TFLOPS = 5000.0       # MI355X published dense FP8 matrix rate (the block-scaled FP8 x FP4 products run at it)
# HBM bytes per launch of the dominant kernel from hardware counters (FETCH_SIZE + WRITE_SIZE, scaled by a copy kernel of known
# size); filled in from the committed counter summaries, None where no counter run exists
TRAFFIC = {("c2", 1): 19782641, ("c3", 1): 99177977, ("c5", 1): 6406407843}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=640)
    ap.add_argument("--warmup", type=int, default=128)
    ap.add_argument("--batch", type=int, default=1, help="tokens per step of the headline workload (1 or 4)")
    ap.add_argument("--config", default="c2", choices=["c1", "c2", "c2q", "c2g", "c3", "c3w", "c4a", "c4b", "c5", "c5w", "c2p"],
                    help="headline workload: c2 EXL3 MoE (default, the metric's configuration), c3 MXFP4 MoE (c3w: the same at hidden width 5120), c4a/c4b FP8 dense 7168x4096 / 4096x7168")
    ap.add_argument("--only-headline", action="store_true", help="skip the other configurations' lines")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calib-copy", type=int, default=0, metavar="MIB",
                    help="run only a plain device copy of this many MiB, 10 times (the known-size kernel that scales the FETCH_SIZE / WRITE_SIZE counters)")
    return ap.parse_args()


# ---------------------------------------------------------------------------------------------- workloads

class Exl3Layer:
    """Config 2: EXL3 4-bit, H 2048, I 512, 512 experts top-10 (mul1 codebook)."""
    H, I, E, TOPK, LAYERS = 2048, 512, 512, 10, 48
    DTYPE = "f16 (4-bit trellis codes decoded to fp16 codebook values, fp32 accumulate)"
    SET = "805 MB expert set"
    TAG = "C2 qwen-style"

    def __init__(self, torch, ops, R, inst, seed=0):
        self.torch, self.ops, self.R, self.inst = torch, ops, R, inst
        dev = "cuda:0"
        g = torch.Generator(device=dev).manual_seed(seed)
        H, I, E = self.H, self.I, self.E
        self.BYTES_PER_EXPERT = 3 * (H * I // 2) + 3 * (H + I) * 2     # 4-bit trellis + suh / svh (fp16)

        def mat(K, N):
            tr = torch.randint(-32768, 32768, (E, K // 16, N // 16, 64), dtype=torch.int16, device=dev, generator=g)
            suh = (torch.randint(0, 2, (E, K), device=dev, generator=g) * 2 - 1).to(torch.float16)
            svh = ((torch.randint(0, 2, (E, N), device=dev, generator=g) * 2 - 1) *
                   (torch.rand(E, N, device=dev, generator=g) + 0.5) / math.sqrt(K)).to(torch.float16)
            return tr, suh, svh
        gt, gs, gv = mat(H, I); ut, us, uv = mat(H, I); dt, ds, dv = mat(I, H)
        self.stacked = [gt, ut, dt, gs, us, ds, gv, uv, dv]
        self.table = ops.ExpertTable.from_stacked(self.stacked)
        self.x = torch.randn(R, H, device=dev, generator=g).to(torch.bfloat16)
        self.logits = torch.randn(inst, R, E, device=dev, generator=g)
        self.idx = torch.empty(inst, R, self.TOPK, dtype=torch.int32, device=dev)
        self.w = torch.empty(inst, R, self.TOPK, dtype=torch.float32, device=dev)
        self.out = torch.empty(inst, R, H, dtype=torch.float32, device=dev)
        self.ws = ops.exl3_moe_ws_alloc(R, H, I, E, self.TOPK)
        self.name = f"{self.TAG} EXL3 4-bit MoE layer (H {H}, I {I}, {E} experts top-{self.TOPK}), batch {R}"

    def step(self, i):
        import ctypes as C
        ops, L = self.ops, self.ops._lib()
        st = ops._st()
        k = i % self.inst
        ops._ck(L.spark_softmax_route(ops._p(self.logits[k]), self.E, self.R, self.E, self.TOPK, ops._p(self.idx[k]), ops._p(self.w[k]), st), "route")
        ops._ck(L.spark_exl3_moe(ops._p(self.x), 2, self.H, self.R, ops._p(self.idx[k]), 0, ops._p(self.w[k]), 0, ops._p(self.table.tab), None,
                                 ops._p(self.out[k]), ops._p(self.ws), self.H, self.I, self.E, self.TOPK, 2, 0, 1, st), "exl3_moe")

    DOMINANT = "spk::fused_kernel (the single-launch routed-experts kernel of spark_exl3_moe)"

    def dominant(self, i):
        """only the dominant kernel: the routed-experts launch on the routes the full steps left behind"""
        ops, L = self.ops, self.ops._lib()
        k = i % self.inst
        ops._ck(L.spark_exl3_moe(ops._p(self.x), 2, self.H, self.R, ops._p(self.idx[k]), 0, ops._p(self.w[k]), 0, ops._p(self.table.tab), None,
                                 ops._p(self.out[k]), ops._p(self.ws), self.H, self.I, self.E, self.TOPK, 2, 0, 1, ops._st()), "exl3_moe")

    def bytes_per_step(self):
        """algorithmic bytes: each distinct active expert's codes and scales once + activations in and out."""
        idx = self.idx.cpu().numpy()
        d = np.mean([len(set(idx[k].ravel().tolist())) for k in range(self.inst)])
        return d * self.BYTES_PER_EXPERT + self.R * self.H * (2 + 4), float(d)

    def cpu_sample(self, orc, budget_s=12.0):
        """dequantise + FP32 matmul of the same layer on the host cores (the oracle), a few instances."""
        t = self.torch
        idx = self.idx.cpu().numpy(); w = self.w.cpu().numpy()
        x = self.x.float().cpu().numpy()
        times, n = [], 0
        while sum(times) < budget_s and n < 8:
            used = sorted(set(idx[n].ravel().tolist()))
            experts = {}
            for e in used:
                experts[e] = [s[e].cpu().numpy() if s.dtype != t.float16 else s[e].view(t.int16).cpu().numpy().view(np.uint16) for s in self.stacked]
            t0 = time.perf_counter()
            ref = orc.exl3_moe(x, idx[n], w[n], experts, self.E, self.H, self.I, 4, 2, 0)
            times.append(time.perf_counter() - t0)
            n += 1
        return float(np.median(times)) * 1e6, n, ref, self.out[n - 1].cpu().numpy()


class Exl3LayerQwen(Exl3Layer):
    """The sizes the reference's QwenMoe kernels are compiled for (reference engine-rs/shim/moe_exl3.cuh:24-32)."""
    H, I, E, TOPK = 2560, 640, 512, 10
    SET = "1.26 GB expert set"
    TAG = "reference-sized qwen"


class Exl3LayerGlm(Exl3Layer):
    """The sizes the reference's GlmMoe kernels are compiled for (reference engine-rs/shim/moe_exl3.cuh:35-61)."""
    H, I, E, TOPK = 4096, 1024, 288, 8
    SET = "1.81 GB expert set"
    TAG = "reference-sized glm"


class Exl3Prefill(Exl3Layer):
    """The config-2 layer at prefill size (2048 tokens): not one of the five configurations, timed next to them because the
    drop-in takes such calls too (the grouped GEMM of spark_exl3_moe: weights decoded once per 64 rows, fp16 MFMA)."""

    def __init__(self, torch, ops, R, inst, seed=4):
        super().__init__(torch, ops, R, inst, seed)
        self.name = f"C2 shape at prefill size: EXL3 4-bit MoE layer (H {self.H}, I {self.I}, {self.E} experts top-{self.TOPK}), {R} tokens"
        self.flops = 2.0 * R * self.TOPK * 3 * self.H * self.I
        self.MFMA_PEAK_TFLOPS = 2500.0

    def step(self, i):
        ops, L = self.ops, self.ops._lib()
        st = ops._st()
        k = i % self.inst
        ops._ck(L.spark_softmax_route(ops._p(self.logits[k]), self.E, self.R, self.E, self.TOPK, ops._p(self.idx[k]), ops._p(self.w[k]), st), "route")
        ops._ck(L.spark_exl3_moe(ops._p(self.x), 2, self.H, self.R, ops._p(self.idx[k]), 0, ops._p(self.w[k]), 0, ops._p(self.table.tab), None,
                                 ops._p(self.out[k]), ops._p(self.ws), self.H, self.I, self.E, self.TOPK, 2, 0, 0, st), "exl3_moe")

    dominant = None

    def bytes_per_step(self):
        idx = self.idx.cpu().numpy()
        d = np.mean([len(set(idx[k].ravel().tolist())) for k in range(self.inst)])
        P = self.R * self.TOPK
        # weights of the distinct experts once + x in, transformed rows out and in (fp16, twice for gate / up), partial sums, y out
        act = self.R * self.H * 2 + 2 * (2 * P * self.H * 2) + 2 * (2 * P * self.I * 4) + 2 * P * self.I * 2 + 2 * P * self.H * 4 + self.R * self.H * 4
        return d * self.BYTES_PER_EXPERT + act, float(d)


class Mxfp4Layer:
    """Config 3: MXFP4 experts, H 4096, I 2048, 384 experts top-6 + 1 shared (sqrt-softplus router)."""
    H, I, E, TOPK, NS, LAYERS = 4096, 2048, 384, 6, 1, 61
    DTYPE = "fp4 x fp8 (E2M1 weights x E4M3 activations, E8M0 block scales, block-scaled MFMA, fp32 accumulate)"
    SET = "5.1 GB expert set"
    TAG = "C3 deepseek-style"

    def __init__(self, torch, ops, R, inst, seed=1):
        self.torch, self.ops, self.R, self.inst = torch, ops, R, inst
        dev = "cuda:0"
        g = torch.Generator(device=dev).manual_seed(seed)
        H, I, ET = self.H, self.I, self.E + self.NS
        self.BYTES_PER_EXPERT = 3 * (H * I // 2 + H * I // 32)         # codes + one E8M0 byte per 32
        packed = []
        for rows, K in ((I, H), (I, H), (H, I)):
            w = torch.randint(0, 256, (ET, rows, K // 2), dtype=torch.uint8, device=dev, generator=g)
            s = torch.randint(117, 128, (ET, rows, K // 32), dtype=torch.uint8, device=dev, generator=g)
            packed.append(ops.Mxfp4Experts._pack(w, s))
            del w, s
        self.ex = ops.Mxfp4Experts.__new__(ops.Mxfp4Experts)
        self.ex.E, self.ex.n_shared, self.ex.I, self.ex.H, self.ex.packed, self.ex.natural = self.E, self.NS, I, H, packed, None
        self.x = torch.randn(R, H, device=dev, generator=g).to(torch.bfloat16)
        self.logits = torch.randn(inst, R, self.E, device=dev, generator=g)
        self.bias = torch.zeros(self.E, device=dev)
        self.idx = torch.empty(inst, R, self.TOPK, dtype=torch.int64, device=dev)
        self.rw = torch.empty(inst, R, self.TOPK, dtype=torch.float32, device=dev)
        self.y = torch.empty(inst, R, H, dtype=torch.float32, device=dev)
        self.ws = ops.mxfp4_moe_ws_alloc(R, self.ex, self.TOPK)
        self.name = f"{self.TAG} MXFP4 MoE layer (H {H}, I {I}, {self.E} experts top-{self.TOPK} + {self.NS} shared), batch {R}"

    def step(self, i):
        ops, L = self.ops, self.ops._lib()
        st = ops._st()
        k = i % self.inst
        ops._ck(L.ds41_route(ops._p(self.logits[k]), ops._p(self.bias), ops._p(self.idx[k]), ops._p(self.rw[k]), self.R, self.E, self.TOPK, 1.5, st), "route")
        ops.mxfp4_moe_x(self.x, self.idx[k], self.rw[k], self.ex, y=self.y[k], ws=self.ws, ws_clean=True)

    DOMINANT = "spk::mx::mx_fused_kernel (the single-launch routed-experts kernel of spark_mxfp4_moe_x)"

    def dominant(self, i):
        k = i % self.inst
        self.ops.mxfp4_moe_x(self.x, self.idx[k], self.rw[k], self.ex, y=self.y[k], ws=self.ws, ws_clean=True)

    def bytes_per_step(self):
        idx = self.idx.cpu().numpy()
        d = np.mean([len(set(idx[k].ravel().tolist())) for k in range(self.inst)]) + self.NS
        return d * self.BYTES_PER_EXPERT + self.R * self.H * (2 + 4), float(d)


class Mxfp4LayerWide(Mxfp4Layer):
    """The MXFP4 layer at the hidden width the reference's kernels are compiled for (reference engine-rs/shim/ds41_moe.cu:32, H = 5120):
    ten 512-wide K groups for the eight waves of a gate/up block."""
    H = 5120
    SET = "6.4 GB expert set"
    TAG = "reference-sized ds41"


class Mxfp4Prefill(Mxfp4Layer):
    """Config 5: the MXFP4 layer at prefill size: 2048 tokens, top-6 of 384 experts drawn Zipf(1.1), no shared expert.  The routes are
    inputs here (drawn on the host, as the configuration prescribes); a step = act_quant + grouped gate/up/down + weighted sum."""
    NS = 0

    def __init__(self, torch, ops, R, inst, seed=3):
        from spark_engine_amd import synth
        super().__init__(torch, ops, R, inst, seed)
        g = synth.rng(seed)
        for k in range(inst):
            idx, w = synth.zipf_routes(g, R, self.E, self.TOPK)
            self.idx[k].copy_(torch.from_numpy(idx)); self.rw[k].copy_(torch.from_numpy(w))
        self.ws = torch.empty(ops.mxfp4_moe_ws(R, self.ex, self.TOPK), dtype=torch.uint8, device="cuda:0")
        self.scratch = (torch.empty(R, self.H, dtype=torch.uint8, device="cuda:0"), torch.empty(R, self.H // 32, dtype=torch.uint8, device="cuda:0"))
        self.name = f"C5 prefill-sized MXFP4 grouped GEMM (H {self.H}, I {self.I}, {self.E} experts top-{self.TOPK}, Zipf(1.1) routing), {R} tokens"
        self.flops = 2.0 * R * self.TOPK * 3 * self.H * self.I

    def step(self, i):
        k = i % self.inst
        self.ops.mxfp4_moe(self.x, self.idx[k], self.rw[k], self.ex, y=self.y[k], ws=self.ws, scratch=self.scratch)

    dominant = None

    def bytes_per_step(self):
        idx = self.idx.cpu().numpy()
        d = np.mean([len(set(idx[k].ravel().tolist())) for k in range(self.inst)])
        P = self.R * self.TOPK
        # weights of the distinct experts once + x in, h out and in (codes + scales), per-pair outputs out and in, y out
        act = self.R * self.H * 2 + 2 * P * (self.I + self.I // 32) + 2 * P * self.H * 4 + self.R * self.H * 4
        return d * self.BYTES_PER_EXPERT + act, float(d)


class Mxfp4PrefillWide(Mxfp4Prefill):
    """Config 5 at the hidden width of the reference's kernels (H = 5120, reference engine-rs/shim/ds41_moe.cu:32)."""
    H = 5120
    SET = "6.4 GB expert set"


class Fp8Dense:
    """Config 4: FP8 E4M3 dense projection with 128x128 FP32 block scales."""
    LAYERS = 1
    DTYPE = "fp8 x bf16 (E4M3 weights, fp32 block scales, fp32 accumulate)"
    SET = "rotating over more than 512 MB of weight copies"

    def __init__(self, torch, ops, R, inst, N, K, seed=2):
        self.torch, self.ops, self.R, self.inst, self.N, self.K = torch, ops, R, inst, N, K
        dev = "cuda:0"
        g = torch.Generator(device=dev).manual_seed(seed)
        ncopy = max(2, min(inst, (768 << 20) // (N * K) + 1))           # rotate over > 512 MB of distinct weights
        self.w = torch.randn(ncopy, N, K, device=dev, generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
        self.s = torch.exp(torch.empty(ncopy, (N + 127) // 128, (K + 127) // 128, device=dev).uniform_(math.log(1e-3), math.log(1e-1), generator=g))
        self.x = torch.randn(R, K, device=dev, generator=g).to(torch.bfloat16)
        self.y = torch.empty(R, N, dtype=torch.float32, device=dev)
        self.ncopy = ncopy
        self.name = f"C4 FP8 E4M3 128x128-block dense GEMV {N}x{K}, batch {R}"

    def step(self, i):
        k = i % self.ncopy
        self.ops.fp8_block128_gemv(self.x, self.w[k], self.s[k], y=self.y)

    def bytes_per_step(self):
        return self.N * self.K + self.s[0].numel() * 4 + self.R * self.K * 2 + self.R * self.N * 4, 1.0


class Mxfp4Dense:
    """Config 1: MXFP4 dense GEMV 2048 x 2048, one row (the reference's own CPU-runnable case, reference ds41.cu:75-110, 236)."""
    LAYERS = 1
    DTYPE = "fp4 x bf16 (E2M1 weights, E8M0 block scales, fp32 accumulate)"
    SET = "rotating over 256 weight copies (570 MB)"

    def __init__(self, torch, ops, R, inst, N=2048, K=2048, seed=6):
        self.torch, self.ops, self.R, self.inst, self.N, self.K = torch, ops, R, inst, N, K
        dev = "cuda:0"
        g = torch.Generator(device=dev).manual_seed(seed)
        self.ncopy = inst
        self.w = torch.randint(0, 256, (self.ncopy, N, K // 2), dtype=torch.uint8, device=dev, generator=g)
        self.s = torch.randint(117, 128, (self.ncopy, N, K // 32), dtype=torch.uint8, device=dev, generator=g)
        self.x = torch.randn(R, K, device=dev, generator=g).to(torch.bfloat16)
        self.y = torch.empty(R, N, dtype=torch.float32, device=dev)
        self.name = f"C1 MXFP4 dense GEMV {N}x{K}, batch {R}"

    def step(self, i):
        ops, k = self.ops, i % self.ncopy
        ops._ck(ops._lib().ds41_mxfp4_gemv(ops._p(self.x), ops._p(self.w[k]), ops._p(self.s[k]), ops._p(self.y), self.R, self.N, self.K, ops._st()),
                "ds41_mxfp4_gemv")

    def bytes_per_step(self):
        return self.N * self.K // 2 + self.N * self.K // 32 + self.R * self.K * 2 + self.R * self.N * 4, 1.0


# ---------------------------------------------------------------------------------------------- timing

def time_steps(torch, wl, steps, warmup, inst, fn=None):
    """W untimed steps, then exactly K timed steps from HIP graphs (inst layer instances per graph), events on the
    launch stream.  Returns ms per step.  fn = the step function (default the whole layer call)."""
    fn = fn or wl.step
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(min(inst, 4)):
            fn(i)                                       # eager once: lazy module loads, function attributes
        stream.synchronize()

        def capture(n):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for i in range(n):
                    fn(i)
            return g
        per = min(inst, steps)
        g_main = capture(per)
        rem = steps % per
        g_rem = capture(rem) if rem else None
        for _ in range(max(1, math.ceil(warmup / per))):
            g_main.replay()
        stream.synchronize()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(steps // per):
            g_main.replay()
        if g_rem is not None:
            g_rem.replay()
        e1.record(stream)
        e1.synchronize()
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def line_for(wl, ms):
    by, d = wl.bytes_per_step()
    us = ms * 1e3
    gbs = by / (us * 1e-6) / 1e9
    out = {"workload": wl.name, "us_per_layer": round(us, 3), "algorithmic_bytes": int(by), "distinct_experts": round(d, 2),
           "achieved_GBps": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
           "tok_per_s_equiv": round(1e6 / (us * wl.LAYERS) * wl.R, 1), "layers_assumed": wl.LAYERS}
    if hasattr(wl, "flops"):                               # the contraction-sized configuration: matrix-unit rate next to the bandwidth
        tf = wl.flops / (us * 1e-6) / 1e12
        peak = getattr(wl, "MFMA_PEAK_TFLOPS", FP8_PEAK_TFLOPS)      # fp16 operands for the EXL3 GEMM, fp8 for the MXFP4 one
        out.update({"flops": wl.flops, "achieved_TFLOPs": round(tf, 1), "mfma_peak_TFLOPs": peak, "frac_of_mfma_peak": round(tf / peak, 4),
                    "time_at_hbm_peak_us": round(by / (HBM_PEAK_GBS * 1e9) * 1e6, 1), "time_at_mfma_peak_us": round(wl.flops / (peak * 1e12) * 1e6, 1)})
    return out


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py measures one GPU: every box of this build has one MI355X and the path uses no collectives (--gpus {a.gpus} is not supported)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    from spark_engine_amd import ops
    if not torch.cuda.is_available():
        print("bench.py needs the GPU (no CPU fallback exists for the product path)", file=sys.stderr)
        sys.exit(3)
    ops._lib()
    if a.calib_copy:
        src = torch.empty(a.calib_copy << 20, dtype=torch.uint8, device="cuda:0").random_(0, 256)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "device copy", "bytes_read": src.numel(), "bytes_written": src.numel(), "launches": 10}))
        return
    INST = 64
    if a.config == "c2":
        wl = Exl3Layer(torch, ops, a.batch, INST)
    elif a.config == "c1":
        INST = 256                                      # 2.2 MB per matrix: 256 copies so that a graph's reads exceed every cache
        wl = Mxfp4Dense(torch, ops, a.batch, INST)
    elif a.config == "c2q":
        wl = Exl3LayerQwen(torch, ops, a.batch, INST)
    elif a.config == "c2g":
        wl = Exl3LayerGlm(torch, ops, a.batch, INST)
    elif a.config == "c3":
        wl = Mxfp4Layer(torch, ops, a.batch, INST)
    elif a.config == "c3w":
        wl = Mxfp4LayerWide(torch, ops, a.batch, INST)
    elif a.config == "c5":
        INST = 4
        wl = Mxfp4Prefill(torch, ops, 2048, INST)
    elif a.config == "c5w":
        INST = 4
        wl = Mxfp4PrefillWide(torch, ops, 2048, INST)
    elif a.config == "c2p":
        INST = 4
        wl = Exl3Prefill(torch, ops, 2048, INST)
    else:
        wl = Fp8Dense(torch, ops, a.batch, INST, *((7168, 4096) if a.config == "c4a" else (4096, 7168)))
    dtype, wset = wl.DTYPE, wl.SET
    ms = time_steps(torch, wl, a.steps, a.warmup, INST)
    head = line_for(wl, ms)
    # the dominant kernel alone, same graphs and events: its average launch duration prices the roofline
    if getattr(wl, "dominant", None) is not None:
        k_us = time_steps(torch, wl, a.steps, a.warmup, INST, wl.dominant) * 1e3
        k_name = wl.DOMINANT
    else:
        k_us, k_name = head["us_per_layer"], "whole call"
    k_gbs = head["algorithmic_bytes"] / (k_us * 1e-6) / 1e9

    cpu = None
    if not a.no_cpu and a.config == "c2":
        from oracle import binding as orc
        cpu_us, n, ref, got = wl.cpu_sample(orc)
        rel = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
        cpu = {"value": round(cpu_us, 1), "unit": "us per MoE layer", "cores": orc.num_threads(), "kind": "port",
               "sample": f"{n} layer instances of the same workload (dequantise to FP32 + FP32 matmul per active expert, OpenMP), median",
               "gpu_vs_cpu_rel_l2": rel}
    others = []
    if not a.only_headline:
        del wl
        torch.cuda.empty_cache()
        todo = [lambda: Exl3Layer(torch, ops, 4 if a.batch == 1 else 1, INST)]
        todo += [lambda R=R: Mxfp4Layer(torch, ops, R, INST) for R in (1, 2, 4)]
        todo += [lambda R=R, N=N, K=K: Fp8Dense(torch, ops, R, INST, N, K) for (N, K) in ((7168, 4096), (4096, 7168)) for R in (1, 4)]
        todo += [lambda: Mxfp4Dense(torch, ops, 1, 256)]
        todo += [lambda: Mxfp4Prefill(torch, ops, 2048, 4), lambda: Exl3Prefill(torch, ops, 2048, 4)]
        # the sizes the reference's own kernels are compiled for
        todo += [lambda: Exl3LayerQwen(torch, ops, 1, INST), lambda: Exl3LayerGlm(torch, ops, 1, INST), lambda: Mxfp4LayerWide(torch, ops, 1, INST)]
        for mk in todo:
            w2 = mk()
            big = isinstance(w2, (Mxfp4Prefill, Exl3Prefill))
            others.append(line_for(w2, time_steps(torch, w2, 32 if big else 256, 8 if big else 64, w2.inst)))
            del w2
            torch.cuda.empty_cache()

    out = {
        "metric": "us per MoE layer (+ achieved HBM GB/s, % of peak) at batch 1/4", "value": head["us_per_layer"], "unit": "us per MoE layer",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": head["workload"], "timing": f"HIP graph of {INST} layer instances with fresh routes, weights cold ({wset})",
                   "tok_per_s_equiv": head["tok_per_s_equiv"], "layers_assumed": head["layers_assumed"]},
        "roofline": {"bound": "hbm", "achieved": round(k_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(k_gbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC.get((a.config, a.batch)),
                     "kernel": k_name, "kernel_us_per_launch": round(k_us, 3), "algorithmic_bytes_per_launch": head["algorithmic_bytes"],
                     "whole_layer_GBps": head["achieved_GBps"], "whole_layer_frac": head["frac_of_hbm_peak"]},
        "cpu_baseline": cpu,
        "all_configs": [head] + others,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
