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
INSTANCES = 64                 # layer instances per graph (decode configurations)
REPLAYS, WARM_REPLAYS = 20, 5  # timing protocol: 5 warm-up replays, median of 20 timed replays


def counter_traffic(tag):
    """HBM bytes per launch of a dominant kernel from the committed hardware-counter summary (FETCH_SIZE + WRITE_SIZE, each scaled
    by a copy kernel of known size): the line `traffic <tag> = <bytes>` of profiles/hbm_counters_*.txt.  (bytes, source) or (None, None)."""
    import glob
    import re
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "hbm_counters_*.txt"))):
        for line in open(path):
            m = re.match(r"\s*traffic\s+%s\s*=\s*([0-9,]+)" % re.escape(tag), line)
            if m:
                return int(m.group(1).replace(",", "")), os.path.relpath(path, ROOT)
    return None, None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--batch", type=int, default=1, help="tokens per step of the headline workload (1 or 4)")
    ap.add_argument("--config", default="c2", choices=["c1", "c2", "c2q", "c2g", "c2ref", "c2refp", "c3", "c3w", "c3ref", "c3refp", "c3rank", "c4a", "c4b", "c4ap", "c4bp", "p1", "p2", "p3", "g8", "c5", "c5w", "c2p"],
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
    SINGLE_LAUNCH = True

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
        while sum(times) < budget_s and n < 5:
            used = sorted(set(idx[n].ravel().tolist()))
            experts = {}
            for e in used:
                experts[e] = [s[e].cpu().numpy() if s.dtype != t.float16 else s[e].view(t.int16).cpu().numpy().view(np.uint16) for s in self.stacked]
            t0 = time.perf_counter()
            ref = orc.exl3_moe(x, idx[n], w[n], experts, self.E, self.H, self.I, 4, 2, 0)
            times.append(time.perf_counter() - t0)
            n += 1
        got = self.out[n - 1].cpu().numpy()
        return (float(np.median(times)) * 1e6, f"{n} layer instances of the same workload (every routed pair: dequantise the expert to FP32 + FP32 matmul, OpenMP), median",
                float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))


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
    SINGLE_LAUNCH = False
    cpu_sample = None

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
    SINGLE_LAUNCH = True

    def __init__(self, torch, ops, R, inst, seed=1):
        self.torch, self.ops, self.R, self.inst, self.seed = torch, ops, R, inst, seed
        dev = "cuda:0"
        g = torch.Generator(device=dev).manual_seed(seed)
        H, I = self.H, self.I
        self.BYTES_PER_EXPERT = 3 * (H * I // 2 + H * I // 32)         # codes + one E8M0 byte per 32
        self.build_weights(g)
        self.x = torch.randn(R, H, device=dev, generator=g).to(torch.bfloat16)
        self.logits = torch.randn(inst, R, self.E, device=dev, generator=g)
        self.bias = torch.zeros(self.E, device=dev)
        self.idx = torch.empty(inst, R, self.TOPK, dtype=torch.int64, device=dev)
        self.rw = torch.empty(inst, R, self.TOPK, dtype=torch.float32, device=dev)
        self.y = torch.empty(inst, R, H, dtype=torch.float32, device=dev)
        self.ws = ops.mxfp4_moe_ws_alloc(R, self.ex, self.TOPK)
        self.name = f"{self.TAG} MXFP4 MoE layer (H {H}, I {I}, {self.E} experts top-{self.TOPK} + {self.NS} shared), batch {R}"

    def natural_tensors(self, g):
        """the three stacked matrices in checkpoint layout, one at a time: (codes [ET, rows, K/2], scales [ET, rows, K/32])"""
        torch, ET = self.torch, self.E + self.NS
        for rows, K in ((self.I, self.H), (self.I, self.H), (self.H, self.I)):
            w = torch.randint(0, 256, (ET, rows, K // 2), dtype=torch.uint8, device="cuda:0", generator=g)
            s = torch.randint(117, 128, (ET, rows, K // 32), dtype=torch.uint8, device="cuda:0", generator=g)
            yield w, s

    def build_weights(self, g):
        ops = self.ops
        packed = [ops.Mxfp4Experts._pack(w, s) for w, s in self.natural_tensors(g)]
        self.ex = ops.Mxfp4Experts.__new__(ops.Mxfp4Experts)
        self.ex.E, self.ex.n_shared, self.ex.I, self.ex.H, self.ex.packed, self.ex.natural = self.E, self.NS, self.I, self.H, packed, None

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

    def host_experts(self, used):
        """checkpoint-layout weights of the experts `used` (+ the shared ones) on the host: the generator replayed from the seed"""
        g = self.torch.Generator(device="cuda:0").manual_seed(self.seed)
        sel = self.torch.tensor(list(used) + [self.E + j for j in range(self.NS)], device="cuda:0")
        out = []
        for w, s in self.natural_tensors(g):
            out += [w[sel].cpu().numpy(), s[sel].cpu().numpy()]
            del w, s
        return out

    def cpu_rows(self, orc, k, rows):
        """oracle on token rows `rows` of instance k: (seconds, reference, GPU rows)"""
        idx = self.idx[k].cpu().numpy()[rows]; rw = self.rw[k].cpu().numpy()[rows]
        used = sorted(set(idx.ravel().tolist()))
        remap = {e: i for i, e in enumerate(used)}
        sub = self.host_experts(used)
        xb = self.x.view(self.torch.int16).cpu().numpy().view(np.uint16)[rows]
        li = np.vectorize(remap.get)(idx).astype(np.int64)
        t0 = time.perf_counter()
        ref = orc.mxfp4_moe(xb, li, rw, *sub, n_shared=self.NS)
        return time.perf_counter() - t0, ref, self.y[k].cpu().numpy()[rows]

    def cpu_sample(self, orc, budget_s=12.0):
        times, n = [], 0
        while sum(times) < budget_s and n < 3:
            dt, ref, got = self.cpu_rows(orc, n, list(range(self.R)))
            times.append(dt); n += 1
        return (float(np.median(times)) * 1e6, f"{n} layer instances of the same workload (every routed or shared pair: dequantise the expert to FP32 + FP32 "
                "matmul with the reference's roundings, OpenMP), median", float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))


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
    SINGLE_LAUNCH = False

    def cpu_sample(self, orc, budget_s=12.0):
        rows = list(range(0, self.R, self.R // 12))[:12]               # rel-L2 over a dozen rows: single rows scatter between 1e-5 and 3e-3 (a flipped E4M3 step of the intermediate)
        dt, ref, got = self.cpu_rows(orc, 0, rows)
        return (dt / len(rows) * self.R * 1e6, f"{len(rows)} of the {self.R} token rows of one layer call ({dt * 1e3:.0f} ms: every pair dequantises its expert to FP32, "
                f"as the reference's CPU path does), scaled to {self.R} rows", float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))

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


class QwenReferenceEntry(Exl3LayerQwen):
    """The reference-named symbols at the sizes they are compiled for: qwen_moe_route + qwen_moe_experts (x fp32 [R, 2560], 512 experts top-10).
    prepared = False is a caller that changes nothing: the workspace holds undefined bytes and no *_ws_init call was made for it, so every call
    prepares it first (one more launch) and the kernels exchange through device-coherent accesses (no placement check has run in such a process).
    prepared = True adds the one call the integration notes describe: spark_exl3_moe_ws_init(ws, bytes) once after allocating ws."""
    TAG = "reference entry points (qwen_moe_route + qwen_moe_experts)"

    def __init__(self, torch, ops, R, inst, prepared, seed=0):
        super().__init__(torch, ops, R, inst, seed)
        self.prepared = prepared
        self.x = self.x.float()
        L = ops._lib()
        nbytes = L.qwen_moe_ws_bytes(R, 4)
        if prepared:
            self.ws = ops._prepared_ws(torch.empty(nbytes, dtype=torch.uint8, device="cuda:0"), L.spark_exl3_moe_ws_init, "spark_exl3_moe_ws_init")
        else:
            self.ws = ops._fresh_ws(nbytes, "cuda:0").random_(0, 256)
        self.SINGLE_LAUNCH = prepared
        self.name += " - workspace prepared once by spark_exl3_moe_ws_init" if prepared else " - unchanged caller (no *_ws_init, device-coherent exchange)"

    def step(self, i):
        ops, L = self.ops, self.ops._lib()
        st = ops._st()
        k = i % self.inst
        if not self.prepared:
            L.spark_debug_exl3_local(0)
        try:
            ops._ck(L.qwen_moe_route(ops._p(self.logits[k]), self.R, ops._p(self.idx[k]), ops._p(self.w[k]), st), "qwen_moe_route")
            ops._ck(L.qwen_moe_experts(ops._p(self.x), self.H, self.R, ops._p(self.idx[k]), ops._p(self.w[k]), ops._p(self.table.tab), None, ops._p(self.out[k]),
                                       ops._p(self.ws), 4, st), "qwen_moe_experts")
        finally:
            if not self.prepared:
                L.spark_debug_exl3_local(-1)

    dominant = None
    cpu_sample = None

    def bytes_per_step(self):
        by, d = super().bytes_per_step()
        return by + self.R * self.H * 2, d                     # x is fp32 here


class Ds41ReferenceEntry(Mxfp4LayerWide):
    """The reference-named DeepSeek symbols at their compiled hidden width (5120): ds41_act_quant_fp8 + ds41_route + ds41_moe_mx on weights in the
    reference's moe_pack_mx tile layout with raw scale bytes, no shared expert (the reference adds it through `add`).  prepared as above."""
    NS = 0
    TAG = "reference entry points (ds41_act_quant_fp8 + ds41_route + ds41_moe_mx, moe_pack_mx layout)"

    def __init__(self, torch, ops, R, inst, prepared, seed=1):
        self.prepared = prepared
        super().__init__(torch, ops, R, inst, seed)
        L = ops._lib()
        nbytes = L.ds41_moe_mx_ws_bytes(R, self.I, self.TOPK, self.E)
        if prepared:
            self.ws = ops._prepared_ws(torch.empty(nbytes, dtype=torch.uint8, device="cuda:0"), L.spark_mxfp4_moe_ws_init, "spark_mxfp4_moe_ws_init")
        else:
            self.ws = ops._fresh_ws(nbytes, "cuda:0").random_(0, 256)
        self.xq = torch.empty(R, self.H, dtype=torch.uint8, device="cuda:0")
        self.xs = torch.empty(R, self.H // 32, dtype=torch.uint8, device="cuda:0")
        self.SINGLE_LAUNCH = prepared
        self.name = (f"{self.TAG} (H {self.H}, I {self.I}, {self.E} experts top-{self.TOPK}), batch {R}" +
                     (" - workspace prepared once by spark_mxfp4_moe_ws_init" if prepared else " - unchanged caller (no *_ws_init, device-coherent exchange)"))

    def build_weights(self, g):
        ops = self.ops
        self.wt = []
        for w, s in self.natural_tensors(g):
            wp, sp = ops.moe_pack(w, s)
            self.wt += [ops.moe_pack_mx(wp), sp]
            del w, s, wp
        self.ex = ops.Mxfp4Experts.__new__(ops.Mxfp4Experts)
        self.ex.E, self.ex.n_shared, self.ex.I, self.ex.H, self.ex.packed, self.ex.natural = self.E, 0, self.I, self.H, None, None

    def step(self, i):
        ops, L = self.ops, self.ops._lib()
        st = ops._st()
        k = i % self.inst
        if not self.prepared:
            L.spark_debug_mx_local(0)
        try:
            ops._ck(L.ds41_act_quant_fp8(ops._p(self.x), ops._p(self.xq), ops._p(self.xs), self.R * self.H, st), "ds41_act_quant_fp8")
            ops._ck(L.ds41_route(ops._p(self.logits[k]), ops._p(self.bias), ops._p(self.idx[k]), ops._p(self.rw[k]), self.R, self.E, self.TOPK, 1.5, st), "ds41_route")
            ops._ck(L.ds41_moe_mx(ops._p(self.xq), ops._p(self.xs), self.R, ops._p(self.idx[k]), ops._p(self.rw[k]), *[ops._p(t) for t in self.wt], self.I, None,
                                  ops._p(self.y[k]), ops._p(self.ws), self.TOPK, self.E, st), "ds41_moe_mx")
        finally:
            if not self.prepared:
                L.spark_debug_mx_local(-1)

    dominant = None
    cpu_sample = None


class Ds41ReferenceEntryRank(Ds41ReferenceEntry):
    """The same entry points at the intermediate width one rank of the reference's three-way split holds (2304 / 3 = 768,
    reference engine-rs/src/ds41/kern.rs:2179-2190): the shape the reference's decode graphs actually launch."""
    I = 768
    SET = "2.4 GB expert set"


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

    def cpu_sample(self, orc, budget_s=4.0):
        t = self.torch
        xb = self.x.view(t.int16).cpu().numpy().view(np.uint16)
        w, sc = self.w[0].cpu().numpy(), self.s[0].cpu().numpy()
        times = []
        for _ in range(6):
            t0 = time.perf_counter()
            ref = orc.fp8_block_gemv(xb, w, sc)
            times.append(time.perf_counter() - t0)
        self.ops.fp8_block128_gemv(self.x, self.w[0], self.s[0], y=self.y)
        got = self.y.cpu().numpy()
        return (float(np.median(times[1:])) * 1e6, "the whole projection (dequantise to FP32 + FP32 GEMV, OpenMP), median of 5 after one warm-up",
                float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))


class Fp8DensePacked(Fp8Dense):
    """Config 4 on weights packed once at load into the matrix unit's operand order (spark_fp8_t16_pack): the same product, the
    same bytes per call; the row-major line above stays the one the reference's layout gets."""

    def __init__(self, torch, ops, R, inst, N, K, seed=2):
        super().__init__(torch, ops, R, inst, N, K, seed)
        self.wt = torch.stack([ops.fp8_t16_pack(self.w[c]) for c in range(self.ncopy)])
        self.name = f"C4 FP8 E4M3 128x128-block dense GEMV {N}x{K} on weights packed at load (16 x 128 operand tiles), batch {R}"

    def step(self, i):
        k = i % self.ncopy
        self.ops.fp8_block128_gemv_t16(self.x, self.wt[k], self.s[k], self.N, y=self.y)

    def cpu_sample(self, orc, budget_s=4.0):
        us, what, _ = super().cpu_sample(orc, budget_s)
        self.ops.fp8_block128_gemv_t16(self.x, self.wt[0], self.s[0], self.N, y=self.y)
        xb = self.x.view(self.torch.int16).cpu().numpy().view(np.uint16)
        ref = orc.fp8_block_gemv(xb, self.w[0].cpu().numpy(), self.s[0].cpu().numpy())
        got = self.y.cpu().numpy()
        return us, what, float(np.linalg.norm(got - ref) / np.linalg.norm(ref))


class Fp8MxProjection:
    """The reference model's dense projections at decode (reference engine-rs/shim/ds41_mx.cu:953-1100, fp8_gemv_mx): E4M3 weights with
    E8M0 scales per 32 x 32 times act-quantised activations, on the row-major matrix (ds41_fp8_gemv_mx_q).  Not one of the five
    configurations."""
    LAYERS = 1
    DTYPE = "fp8 x fp8 (E4M3 weights and act-quantised activations with E8M0 scales per 32, multiplied as exact bf16, fp32 accumulate)"
    SET = "rotating over more than 512 MB of weight copies"
    cpu_sample = None

    def __init__(self, torch, ops, R, inst, N, K, seed=7):
        self.torch, self.ops, self.R, self.inst, self.N, self.K = torch, ops, R, inst, N, K
        dev = "cuda:0"
        g = torch.Generator(device=dev).manual_seed(seed)
        ncopy = max(2, min(inst, (600 << 20) // (N * K) + 1))
        self.w = torch.randn(ncopy, N, K, device=dev, generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
        self.s = torch.randint(110, 128, (ncopy, N // 32, K // 32), dtype=torch.uint8, device=dev, generator=g)
        x = torch.randn(R, K, device=dev, generator=g).to(torch.bfloat16)
        self.aq, self.as_ = ops.act_quant_fp8(x)
        self.y = torch.empty(R, N, dtype=torch.float32, device=dev)
        self.ncopy = ncopy
        self.name = f"dense FP8 projection {N}x{K} on act-quantised activations, row-major weights (ds41_fp8_gemv_mx_q), batch {R}"

    def step(self, i):
        c = i % self.ncopy
        L, ops = self.ops._lib(), self.ops
        ops._ck(L.ds41_fp8_gemv_mx_q(None, ops._p(self.aq), ops._p(self.as_), ops._p(self.w[c]), ops._p(self.s[c]), ops._p(self.y), self.R, self.N, self.K, 0,
                                      ops._st()), "ds41_fp8_gemv_mx_q")

    def bytes_per_step(self):
        return self.N * self.K + self.s[0].numel() + self.R * (self.K + self.K // 32) + self.R * self.N * 4, 1.0


class GlmFp8Dense:
    """The reference's GLM dense / shared-expert projection format (reference engine-rs/shim/fp8.cu:13-22,110-128): E4M3 weights with one
    binary32 scale per output row, binary32 activations rounded to binary16 inside (glm53_fp8_dense_cuda).  Not one of the five configurations."""
    LAYERS = 1
    DTYPE = "fp8 x f16 (E4M3 weights with a scale per output row, binary16 activations, fp32 accumulate)"
    SET = "rotating over more than 512 MB of weight copies"

    def __init__(self, torch, ops, R, inst, N, K, seed=8):
        self.torch, self.ops, self.R, self.inst, self.N, self.K = torch, ops, R, inst, N, K
        dev = "cuda:0"
        g = torch.Generator(device=dev).manual_seed(seed)
        ncopy = max(2, min(inst, (600 << 20) // (N * K) + 1))
        self.w = torch.randn(ncopy, N, K, device=dev, generator=g).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
        self.s = torch.rand(ncopy, N, device=dev, generator=g) * 1e-2 + 1e-3
        self.x = torch.randn(R, K, device=dev, generator=g)
        self.y = torch.empty(R, N, dtype=torch.float32, device=dev)
        self.ncopy = ncopy
        self.name = f"GLM-format FP8 dense GEMV {N}x{K} (one scale per output row, glm53_fp8_dense_cuda), batch {R}"

    def step(self, i):
        c = i % self.ncopy
        L, ops = self.ops._lib(), self.ops
        ops._ck(L.glm53_fp8_dense_cuda(ops._p(self.x), ops._p(self.w[c]), ops._p(self.s[c]), ops._p(self.y), None, self.R, self.N, self.K, 0, 1, 0, ops._st()),
                "glm53_fp8_dense_cuda")

    def bytes_per_step(self):
        return self.N * self.K + self.N * 4 + self.R * self.K * 4 + self.R * self.N * 4, 1.0

    def cpu_sample(self, orc, budget_s=4.0):
        x, w, sc = self.x.cpu().numpy(), self.w[0].cpu().numpy(), self.s[0].cpu().numpy()
        times = []
        for _ in range(4):
            t0 = time.perf_counter()
            ref = orc.fp8_rowscale_gemv(x, w, sc, act=0)
            times.append(time.perf_counter() - t0)
        self.step(0)
        got = self.y.cpu().numpy()
        return (float(np.median(times[1:])) * 1e6, "the whole projection (E4M3 decode + dot products in binary64, OpenMP), median of 3 after one warm-up",
                float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))


class StreamFloor:
    """The stream floor of a line: a plain read (non-temporal 16-byte loads, one small store) of exactly the line's algorithmic bytes,
    timed in the same graph of instances, each instance on its own region of a buffer larger than the caches."""

    def __init__(self, torch, ops, nbytes, inst):
        self.torch, self.ops, self.inst = torch, ops, inst
        self.nbytes = int(nbytes) // 16 * 16
        span = max(self.nbytes * min(inst, 64), 1 << 30)
        self.regions = max(1, min(inst, span // self.nbytes))
        self.buf = torch.empty(self.regions * self.nbytes, dtype=torch.uint8, device="cuda:0")
        self.buf.view(torch.int32).random_(0, 1 << 30)
        self.out = torch.zeros(1024, dtype=torch.int32, device="cuda:0")

    def step(self, i):
        ops = self.ops
        ops._ck(ops._lib().spark_debug_stream_read(self.buf.data_ptr() + (i % self.regions) * self.nbytes, self.nbytes, ops._p(self.out), ops._st()),
                "spark_debug_stream_read")


def stream_floor(torch, ops, nbytes, inst):
    """us to read nbytes: median per instance of the timing protocol's graph"""
    f = StreamFloor(torch, ops, nbytes, inst)
    us = time_protocol(torch, f, replays=10, warm=3)[0]
    del f
    torch.cuda.empty_cache()
    return us


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

    def cpu_sample(self, orc, budget_s=4.0):
        t = self.torch
        xb = self.x.view(t.int16).cpu().numpy().view(np.uint16)
        w, sc = self.w[0].cpu().numpy(), self.s[0].cpu().numpy()
        times = []
        for _ in range(6):
            t0 = time.perf_counter()
            ref = orc.mxfp4_gemv(xb, w, sc)
            times.append(time.perf_counter() - t0)
        self.step(0)
        got = self.y.cpu().numpy()
        return (float(np.median(times[1:])) * 1e6, "the whole GEMV (dequantise to FP32 + FP32 GEMV, OpenMP: the configuration's own definition), median of 5 after one warm-up",
                float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))


# ---------------------------------------------------------------------------------------------- timing

def _capture(torch, stream, fn, n):
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        for i in range(n):
            fn(i)
    return g


def time_protocol(torch, wl, fn=None, replays=REPLAYS, warm=WARM_REPLAYS):
    """The stated protocol: one HIP graph of wl.inst layer instances (fresh routes per instance, weights rotating through more
    bytes than the caches hold), `warm` untimed replays, then `replays` replays timed one by one with events on the launch
    stream.  Returns (median us per layer, min, max, single-call latency us): the latency is one eager call between two events
    on an otherwise idle stream, median of 20."""
    fn = fn or wl.step
    torch.cuda.synchronize()                            # whatever built or warmed the workload on another stream has finished
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(min(wl.inst, 4)):
            fn(i)                                       # eager once: lazy module loads, function attributes
        stream.synchronize()
        lat = []
        for i in range(20):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream); fn(i % wl.inst); e1.record(stream)
            e1.synchronize()
            lat.append(e0.elapsed_time(e1) * 1e3)
        g = _capture(torch, stream, fn, wl.inst)
        for _ in range(warm):
            g.replay()
        stream.synchronize()
        per = []
        for _ in range(replays):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream); g.replay(); e1.record(stream)
            e1.synchronize()
            per.append(e0.elapsed_time(e1) * 1e3 / wl.inst)
        torch.cuda.synchronize()
    return float(np.median(per)), float(min(per)), float(max(per)), float(np.median(lat))


def time_steps(torch, wl, steps, warmup, fn=None):
    """W untimed steps, then EXACTLY K timed steps between two events on the launch stream: the steps run from graphs of wl.inst
    instances (whole graphs, then one of K % inst instances).  Returns ms per step."""
    fn = fn or wl.step
    inst = wl.inst
    torch.cuda.synchronize()                            # the workload's weights, routes and workspace are in place before the timing stream starts
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        full, rem = divmod(steps, inst)
        g_full = _capture(torch, stream, fn, inst) if full or warmup >= inst else None
        g_rem = _capture(torch, stream, fn, rem) if rem else None
        wfull, wrem = divmod(warmup, inst)
        for _ in range(wfull):
            g_full.replay()
        for i in range(wrem):
            fn(i)
        stream.synchronize()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(full):
            g_full.replay()
        if g_rem is not None:
            g_rem.replay()
        e1.record(stream)
        e1.synchronize()
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def line_for(wl, us, lo, hi, lat, tag=None, floor=None):
    """tag: the line's name in profiles/hbm_counters_*.txt (counter traffic of its dominant kernel or whole call); floor: (torch, ops) to time
    the stream floor of the line's algorithmic bytes"""
    by, d = wl.bytes_per_step()
    gbs = by / (us * 1e-6) / 1e9
    out = {"workload": wl.name, "us_per_layer": round(us, 3), "us_per_layer_min_max": [round(lo, 3), round(hi, 3)], "single_call_latency_us": round(lat, 2),
           "instances": wl.inst, "replays": REPLAYS, "algorithmic_bytes": int(by), "distinct_experts": round(d, 2),
           "achieved_GBps": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
           "tok_per_s_equiv": round(1e6 / (us * wl.LAYERS) * wl.R, 1), "layers_assumed": wl.LAYERS}
    if hasattr(wl, "flops"):                               # the contraction-sized configuration: matrix-unit rate next to the bandwidth
        tf = wl.flops / (us * 1e-6) / 1e12
        peak = getattr(wl, "MFMA_PEAK_TFLOPS", FP8_PEAK_TFLOPS)      # fp16 operands for the EXL3 GEMM, fp8 for the MXFP4 one
        out.update({"flops": wl.flops, "achieved_TFLOPs": round(tf, 1), "mfma_peak_TFLOPs": peak, "frac_of_mfma_peak": round(tf / peak, 4),
                    "time_at_hbm_peak_us": round(by / (HBM_PEAK_GBS * 1e9) * 1e6, 1), "time_at_mfma_peak_us": round(wl.flops / (peak * 1e12) * 1e6, 1)})
    if tag is not None:
        out["traffic"], out["traffic_source"] = counter_traffic(tag)
    if floor is not None:
        fl = stream_floor(floor[0], floor[1], by, wl.inst)
        out["stream_floor_us"] = round(fl, 3)
        out["frac_of_floor"] = round(fl / us, 4)
    return out


def check_ws(ops, wl):
    """no bounded wait of a single-launch call may have expired during the timed region (its outputs would be stale)"""
    ws = getattr(wl, "ws", None)
    if ws is not None and getattr(wl, "SINGLE_LAUNCH", False):
        ops.ws_check(ws, wl.name)


def cpu_leg(wl, orc, budget_s):
    """the oracle (dequantise + FP32 matmul on the host cores) on a bounded sample of the workload, next to the GPU number"""
    if getattr(wl, "cpu_sample", None) is None:
        return None
    us, sample, rel = wl.cpu_sample(orc, budget_s)
    out = {"value": round(us, 1), "unit": "us per MoE layer" if hasattr(wl, "TOPK") else "us per GEMV", "cores": orc.num_threads(), "kind": "port", "sample": sample}
    if rel is not None:
        out["gpu_vs_cpu_rel_l2"] = rel
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
    INST = INSTANCES
    make = {
        "c2": lambda: Exl3Layer(torch, ops, a.batch, INST),
        "c1": lambda: Mxfp4Dense(torch, ops, a.batch, 256),      # 2.2 MB per matrix: 256 copies so that a graph's reads exceed every cache
        "c2q": lambda: Exl3LayerQwen(torch, ops, a.batch, INST), "c2g": lambda: Exl3LayerGlm(torch, ops, a.batch, INST),
        "c2ref": lambda: QwenReferenceEntry(torch, ops, a.batch, INST, prepared=False), "c2refp": lambda: QwenReferenceEntry(torch, ops, a.batch, INST, prepared=True),
        "c3": lambda: Mxfp4Layer(torch, ops, a.batch, INST), "c3w": lambda: Mxfp4LayerWide(torch, ops, a.batch, INST),
        "c3ref": lambda: Ds41ReferenceEntry(torch, ops, a.batch, INST, prepared=False), "c3refp": lambda: Ds41ReferenceEntry(torch, ops, a.batch, INST, prepared=True),
        "c3rank": lambda: Ds41ReferenceEntryRank(torch, ops, a.batch, INST, prepared=True),
        "c5": lambda: Mxfp4Prefill(torch, ops, 2048, 4), "c5w": lambda: Mxfp4PrefillWide(torch, ops, 2048, 4), "c2p": lambda: Exl3Prefill(torch, ops, 2048, 4),
        "c4a": lambda: Fp8Dense(torch, ops, a.batch, INST, 7168, 4096), "c4b": lambda: Fp8Dense(torch, ops, a.batch, INST, 4096, 7168),
        "p1": lambda: Fp8MxProjection(torch, ops, a.batch, INST, 12288, 1280), "p2": lambda: Fp8MxProjection(torch, ops, a.batch, INST, 5120, 3072),
        "p3": lambda: Fp8MxProjection(torch, ops, a.batch, INST, 1280, 5120), "g8": lambda: GlmFp8Dense(torch, ops, a.batch, INST, 4096, 4096),
        "c4ap": lambda: Fp8DensePacked(torch, ops, a.batch, INST, 7168, 4096), "c4bp": lambda: Fp8DensePacked(torch, ops, a.batch, INST, 4096, 7168),
    }
    wl = make[a.config]()
    dtype, wset = wl.DTYPE, wl.SET
    orc = None
    if not a.no_cpu:
        from oracle import binding as orc
    # the contract's K steps after W warm-up steps, then the stated protocol (median of 20 replays of the whole graph)
    ms = time_steps(torch, wl, a.steps, a.warmup)
    us, lo, hi, lat = time_protocol(torch, wl)
    check_ws(ops, wl)
    head = line_for(wl, us, lo, hi, lat, tag=f"{a.config} batch{wl.R}", floor=(torch, ops))
    # the dominant kernel alone, same graph and events: its average launch duration prices the roofline
    if getattr(wl, "dominant", None) is not None:
        k_us = time_protocol(torch, wl, wl.dominant)[0]
        check_ws(ops, wl)
        k_name = wl.DOMINANT
    else:
        k_us, k_name = head["us_per_layer"], "whole call"
    k_gbs = head["algorithmic_bytes"] / (k_us * 1e-6) / 1e9
    cpu = cpu_leg(wl, orc, 12.0) if orc is not None else None
    if cpu is not None:
        head["cpu_baseline"] = cpu
    traffic, traffic_src = head["traffic"], head["traffic_source"]
    others = []
    if not a.only_headline:
        del wl
        torch.cuda.empty_cache()
        # (workload, its tag in profiles/hbm_counters_*.txt or None)
        todo = [(lambda: Mxfp4Dense(torch, ops, 1, 256), "c1 batch1")]                      # C1 first: it is defined as the CPU path
        ob = 4 if a.batch == 1 else 1
        todo += [(lambda: Exl3Layer(torch, ops, ob, INST), f"c2 batch{ob}")]
        todo += [(lambda R=R: Mxfp4Layer(torch, ops, R, INST), f"c3 batch{R}") for R in (1, 2, 4)]
        todo += [(lambda R=R, N=N, K=K: Fp8Dense(torch, ops, R, INST, N, K), f"{c} batch{R}") for (c, N, K) in (("c4a", 7168, 4096), ("c4b", 4096, 7168)) for R in (1, 4)]
        todo += [(lambda R=R, N=N, K=K: Fp8DensePacked(torch, ops, R, INST, N, K), f"{c} batch{R}") for (c, N, K) in (("c4ap", 7168, 4096), ("c4bp", 4096, 7168)) for R in (1, 4)]
        todo += [(lambda: Mxfp4Prefill(torch, ops, 2048, 4), "c5 batch2048"), (lambda: Exl3Prefill(torch, ops, 2048, 4), "c2p batch2048")]
        # the reference model's dense projections (not a configuration: the callers either side of the expert layer)
        todo += [(lambda N=N, K=K, R=R: Fp8MxProjection(torch, ops, R, INST, N, K), f"{c} batch{R}") for (c, N, K) in (("p1", 12288, 1280), ("p2", 5120, 3072), ("p3", 1280, 5120)) for R in (1, 8)]
        todo += [(lambda R=R: GlmFp8Dense(torch, ops, R, INST, 4096, 4096), f"g8 batch{R}") for R in (1, 4)]
        # the sizes the reference's own kernels are compiled for, through spark_* and through the reference-named entry points
        # (a caller that changes nothing: workspace contents undefined, no *_ws_init; and with the one added *_ws_init call)
        todo += [(lambda: Exl3LayerQwen(torch, ops, 1, INST), "c2q batch1"), (lambda: QwenReferenceEntry(torch, ops, 1, INST, prepared=False), "c2ref batch1"),
                 (lambda: QwenReferenceEntry(torch, ops, 1, INST, prepared=True), "c2refp batch1"), (lambda: Exl3LayerGlm(torch, ops, 1, INST), "c2g batch1"),
                 (lambda: Mxfp4LayerWide(torch, ops, 1, INST), "c3w batch1"), (lambda: Ds41ReferenceEntry(torch, ops, 1, INST, prepared=False), "c3ref batch1"),
                 (lambda: Ds41ReferenceEntry(torch, ops, 1, INST, prepared=True), "c3refp batch1"),
                 (lambda: Ds41ReferenceEntryRank(torch, ops, 1, INST, prepared=True), "c3rank batch1")]
        for mk, tag in todo:
            w2 = mk()
            ln = line_for(w2, *time_protocol(torch, w2), tag=tag, floor=(torch, ops))
            check_ws(ops, w2)
            if orc is not None:
                c2 = cpu_leg(w2, orc, 4.0)
                if c2 is not None:
                    ln["cpu_baseline"] = c2
            others.append(ln)
            del w2
            torch.cuda.empty_cache()

    out = {
        "metric": "us per MoE layer (+ achieved HBM GB/s, % of peak) at batch 1/4", "value": head["us_per_layer"], "unit": "us per MoE layer",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": head["workload"],
                   "timing": f"value = median of {REPLAYS} timed replays (after {WARM_REPLAYS} warm-up replays) of one HIP graph of {head['instances']} layer instances "
                             f"with fresh routes each, weights cold ({wset}); ms_per_step = the {a.steps} steps asked for, timed in one region after {a.warmup} "
                             f"warm-up steps, from the same kind of graph ({min(a.steps, head['instances'])} instances when fewer steps than a graph holds are asked for)",
                   "instances": head["instances"], "replays": REPLAYS, "warmup_replays": WARM_REPLAYS, "single_call_latency_us": head["single_call_latency_us"],
                   "tok_per_s_equiv": head["tok_per_s_equiv"], "layers_assumed": head["layers_assumed"]},
        "roofline": {"bound": "hbm", "achieved": round(k_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(k_gbs / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": traffic_src, "kernel": k_name, "kernel_us_per_launch": round(k_us, 3), "algorithmic_bytes_per_launch": head["algorithmic_bytes"],
                     "whole_layer_GBps": head["achieved_GBps"], "whole_layer_frac": head["frac_of_hbm_peak"],
                     # a plain read of the launch's algorithmic bytes in the same graph of instances, and the kernel's time against it
                     "stream_floor_us": head["stream_floor_us"], "frac_of_floor": round(head["stream_floor_us"] / k_us, 4)},
        "cpu_baseline": cpu,
        "all_configs": [head] + others,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
