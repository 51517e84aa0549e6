#!/usr/bin/env python3
"""Benchmark of the EXL3 projection path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--sweep]

A step is one `linear` call of the dense decode-row GEMV workload the headline metric is quoted on
(in=4096, out=12288, K=4 bits/weight, 1 row, MCG codebook, f16 activations with 1 % outliers x20; synthetic seeded
codes). Calls rotate over enough distinct weight copies (> 512 MB in total) that every call reads its codes from
HBM, not from the 256 MB Infinity Cache. Inputs are resident in HBM before the timed region starts.

Prints ONE JSON line: the whole-call rate as GB/s of trellis code bytes (`value`), the dominant kernel's roofline
(`roofline`: algorithmic code bytes of one launch / its average duration, timed alone with HIP events on the launch
stream, against 8 TB/s), and the CPU oracle (`format.project` restated in C) timed on this box's host cores
(`cpu_baseline`). The same line carries the other benchmark configurations as extra objects: `moe_decode`
(config 3: routed decode at 1 and 8 tokens), `moe_prefill` (config 4: the routed prefill chain, TFLOP/s against the
2.5 PFLOP/s dense f16 MFMA peak) and `dense_prefill` (config 5: 4096 rows); `--quick` leaves them out. `--sweep` adds
K = 3, 4, 5 x rows = 1, 4, 16, 32; `--in-f/--out-f/--k/--rows` time another dense shape (lm_head: --in-f 4096
--out-f 151936 --k 6).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

IN_F, OUT_F = 4096, 12288
HBM_PEAK = 8.0e12
MIN_ROTATION_BYTES = 512 << 20
# HBM bytes one chain-GEMV launch moves, from the profiler's FETCH_SIZE and WRITE_SIZE counters scaled by a 256 MiB
# copy (profiles/dense_gemv_in4096_out12288_k4_rows1.txt): keyed by (in, out, K, rows); other workloads report null
MEASURED_TRAFFIC = {(4096, 12288, 4, 1): 25_762_406}


def code_bytes(in_f: int, out_f: int, n: int) -> int:
    """Algorithmic bytes of one projection: (in/16)(out/16) tiles of n halfwords."""
    return (in_f // 16) * (out_f // 16) * n * 2


def make_weights(torch, n: int, copies: int, seed: int):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    trellis = torch.randint(-32768, 32768, (copies, IN_F // 16, OUT_F // 16, n), dtype=torch.int16, device="cuda",
                            generator=g)
    sign = lambda k: (torch.randint(0, 2, (k,), device="cuda", generator=g) * 2 - 1).to(torch.float32)
    suh = (sign(IN_F) * (1.0 + 0.1 * torch.randn(IN_F, device="cuda", generator=g))).to(torch.float16)
    svh = (sign(OUT_F) * (1.0 + 0.1 * torch.randn(OUT_F, device="cuda", generator=g)) / (IN_F ** 0.5)).to(torch.float16)
    return trellis, suh, svh


def make_x(torch, rows: int, seed: int):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    x = torch.randn(rows, IN_F, device="cuda", generator=g)
    outl = torch.rand(rows, IN_F, device="cuda", generator=g) < 0.01
    return torch.where(outl, x * 20.0, x).to(torch.float16)


class DenseRunner:
    """Pre-built descriptors for back-to-back C-ABI calls: nothing is allocated inside the timed region."""

    def __init__(self, torch, api, trellis, suh, svh, x, dec):
        import ctypes as C

        from turboexl3_amd import _lib
        self.C, self.L, self.torch = C, _lib.lib(), torch
        self.copies = trellis.shape[0]
        self.dec = dec.c()
        self.ax = api._arr(x)
        self.at = [api._arr(trellis[i]) for i in range(self.copies)]
        self.asu, self.asv = api._arr(suh), api._arr(svh)
        self.y = torch.empty(x.shape[0], OUT_F, dtype=x.dtype, device="cuda")
        self.ay = api._arr(self.y)
        need = C.c_size_t(0)
        st = self.L.t3_linear_workspace_bytes(C.byref(self.ax), C.byref(self.at[0]), self.dec, C.byref(need))
        assert st == 0, _lib.error_name(st)
        self.ws = torch.zeros(need.value, dtype=torch.uint8, device="cuda")
        self.stream = torch.cuda.current_stream().cuda_stream

    def call(self, i: int, stages: int = 0):
        C = self.C
        t = self.at[i % self.copies]
        if stages:
            st = self.L.t3_linear_stages(self.stream, C.byref(self.ax), C.byref(t), C.byref(self.asu), C.byref(self.asv),
                                         self.dec, C.byref(self.ay), self.ws.data_ptr(), self.ws.numel(), stages)
        else:
            st = self.L.t3_linear(self.stream, C.byref(self.ax), C.byref(t), C.byref(self.asu), C.byref(self.asv),
                                  self.dec, C.byref(self.ay), self.ws.data_ptr(), self.ws.numel())
        if st != 0:
            raise RuntimeError(self.L.t3_error_name(st).decode())

    def time(self, steps: int, warmup: int, stages: int = 0) -> float:
        """Seconds per call over exactly `steps` back-to-back calls. The calls are captured once into a HIP graph
        (as a serving loop would hold its decode step) so the host's per-launch cost stays out of the GPU's
        timeline; events bracket the replay on the launch stream."""
        torch = self.torch
        for i in range(max(warmup, 1)):
            self.call(i, stages)
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            self.stream = side.cuda_stream
            with torch.cuda.graph(graph, stream=side):
                for i in range(steps):
                    self.call(warmup + i, stages)
            torch.cuda.synchronize()
            graph.replay()  # untimed: the graph's first replay uploads it
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            graph.replay()
            e1.record(side)
            torch.cuda.synchronize()
        self.stream = torch.cuda.current_stream().cuda_stream
        return e0.elapsed_time(e1) * 1e-3 / steps


class MoeRunner:
    """Benchmark configuration 3: 512 experts, hidden 2048, inter 512, K3, top-10, clamp 7, one shared expert (inter 512) in the
    same launches. Every call routes to a fresh set of experts (a rotation of disjoint routings) so the codes come from
    HBM: the bank alone is 604 MB."""

    E, HIDDEN, INTER, K, TOPK, LIMIT = 512, 2048, 512, 3, 10, 7

    def __init__(self, torch, api, tokens: int, seed: int = 5):
        import ctypes as C

        from turboexl3_amd import _lib
        self.C, self.L, self.torch, self.api = C, _lib.lib(), torch, api
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        n = 16 * self.K

        def proj(experts, in_f, out_f):
            t = torch.randint(-32768, 32768, (experts, in_f // 16, out_f // 16, n), dtype=torch.int16, device="cuda",
                              generator=g)
            suh = (0.5 + torch.rand(experts, in_f, device="cuda", generator=g)).to(torch.float16)
            svh = ((0.5 + torch.rand(experts, out_f, device="cuda", generator=g)) / in_f ** 0.5).to(torch.float16)
            return api.Proj(t, suh, svh)

        def bank(experts):
            return api.Bank(proj(experts, self.HIDDEN, self.INTER), proj(experts, self.HIDDEN, self.INTER),
                            proj(experts, self.INTER, self.HIDDEN))

        self.bank, self.shared = bank(self.E), bank(1)
        self.tokens = tokens
        self.x = torch.randn(1, tokens, self.HIDDEN, device="cuda", generator=g).to(torch.bfloat16)
        # router logits ~ N(0,1) -> top-k -> softmax over the selected (harness side, as in the reference's benches)
        self.sets = 24
        logits = torch.randn(self.sets, tokens, self.E, device="cuda", generator=g)
        top = torch.topk(logits, self.TOPK, dim=-1)
        self.inds = top.indices.to(torch.int32).contiguous()
        self.scores = torch.softmax(top.values, dim=-1).to(torch.float32).contiguous()
        self.cb, self._k1 = api._cbank(self.bank)
        self.sb, self._k2 = api._cbank(self.shared)
        self.ax = api._arr(self.x)
        self.ai = [api._arr(self.inds[i:i + 1]) for i in range(self.sets)]
        self.asc = [api._arr(self.scores[i:i + 1]) for i in range(self.sets)]
        self.y = torch.empty_like(self.x)
        self.ay = api._arr(self.y)
        need = C.c_size_t(0)
        st = self.L.t3_moe_workspace_bytes(C.byref(self.ax), C.byref(self.cb), C.byref(self.ai[0]), C.byref(self.sb),
                                           C.byref(need))
        assert st == 0, _lib.error_name(st)
        self.ws = torch.zeros(need.value, dtype=torch.uint8, device="cuda")
        self.dec = api.Decode.mcg.c()
        self.stream = torch.cuda.current_stream().cuda_stream
        per_expert = 3 * (self.HIDDEN // 16) * (self.INTER // 16) * n * 2
        distinct = [len(set(self.inds[i].flatten().tolist())) for i in range(self.sets)]
        self.code_bytes = (sum(distinct) / self.sets + 1) * per_expert  # + the shared expert

    def call(self, i: int, stages: int = 0):
        C = self.C
        j = i % self.sets
        st = self.L.t3_moe_shared_expert(self.stream, C.byref(self.ax), C.byref(self.cb), C.byref(self.ai[j]),
                                         C.byref(self.asc[j]), self.dec, self.LIMIT, C.byref(self.sb), C.byref(self.ay),
                                         self.ws.data_ptr(), self.ws.numel())
        if st != 0:
            raise RuntimeError(self.L.t3_error_name(st).decode())

    time = DenseRunner.time


class PrefillRunner:
    """Benchmark configuration 4: 2048 tokens, 256 experts, top-8, hidden 7168, inter 2048, gate|up K2, down K3, bf16, clamp 7.
    flops = tokens * topk * 3 * 2 * hidden * inter. `scale` shrinks experts and tokens together (same rows an expert)."""

    def __init__(self, torch, api, tokens=2048, experts=256, topk=8, hidden=7168, inter=2048, k_gu=2, k_dn=3, seed=9):
        import ctypes as C

        from turboexl3_amd import _lib
        self.C, self.L, self.torch, self.api = C, _lib.lib(), torch, api
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)

        def proj(in_f, out_f, k):
            t = torch.randint(-32768, 32768, (experts, in_f // 16, out_f // 16, 16 * k), dtype=torch.int16,
                              device="cuda", generator=g)
            suh = (0.5 + torch.rand(experts, in_f, device="cuda", generator=g)).to(torch.float16)
            svh = ((0.5 + torch.rand(experts, out_f, device="cuda", generator=g)) / in_f ** 0.5).to(torch.float16)
            return api.Proj(t, suh, svh)

        self.bank = api.Bank(proj(hidden, inter, k_gu), proj(hidden, inter, k_gu), proj(inter, hidden, k_dn))
        self.x = torch.randn(1, tokens, hidden, device="cuda", generator=g).to(torch.bfloat16)
        logits = torch.randn(tokens, experts, device="cuda", generator=g)
        top = torch.topk(logits, topk, dim=-1)
        self.inds = top.indices.to(torch.int32).reshape(1, tokens, topk).contiguous()
        self.scores = torch.softmax(top.values, dim=-1).to(torch.float32).reshape(1, tokens, topk).contiguous()
        self.cb, self._k1 = api._cbank(self.bank)
        self.ax, self.ai, self.asc = api._arr(self.x), api._arr(self.inds), api._arr(self.scores)
        self.y = torch.empty_like(self.x)
        self.ay = api._arr(self.y)
        need = C.c_size_t(0)
        st = self.L.t3_moe_workspace_bytes(C.byref(self.ax), C.byref(self.cb), C.byref(self.ai), None, C.byref(need))
        assert st == 0, _lib.error_name(st)
        self.ws = torch.zeros(need.value, dtype=torch.uint8, device="cuda")
        self.dec = api.Decode.mcg.c()
        self.stream = torch.cuda.current_stream().cuda_stream
        self.flops = tokens * topk * 3 * 2 * hidden * inter
        self.code_bytes = experts * (2 * code_bytes_of(hidden, inter, 16 * k_gu) + code_bytes_of(inter, hidden, 16 * k_dn))

    def call(self, i: int, stages: int = 0):
        C = self.C
        st = self.L.t3_moe_clamped(self.stream, C.byref(self.ax), C.byref(self.cb), C.byref(self.ai), C.byref(self.asc),
                                   self.dec, 7, C.byref(self.ay), self.ws.data_ptr(), self.ws.numel())
        if st != 0:
            raise RuntimeError(self.L.t3_error_name(st).decode())

    time = DenseRunner.time


def code_bytes_of(in_f: int, out_f: int, n: int) -> int:
    return (in_f // 16) * (out_f // 16) * n * 2


def cpu_baseline(n: int, seed: int, budget_s: float = 20.0):
    """format.project (the C oracle) on the host: the same shape and seeded distributions, one row, one thread,
    re-decoding every tile as the reference does. A bounded sample: whole calls until ~budget_s is spent."""
    from oracle import oracle
    rng = np.random.default_rng(seed)
    trellis, suh, svh = oracle.synth_linear(rng, IN_F, OUT_F, n)
    x = rng.standard_normal(IN_F).astype(np.float32)
    oracle.project(x[:128], trellis[:8, :8], suh[:128], svh[:128], 128, 128, n, oracle.MCG)  # load the library
    times = []
    t_start = time.perf_counter()
    while len(times) < 5 and (time.perf_counter() - t_start < budget_s or not times):
        t0 = time.perf_counter()
        oracle.project(x, trellis, suh, svh, IN_F, OUT_F, n, oracle.MCG)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    cores = os.cpu_count() or 1
    threads = min(cores, 16)
    t0 = time.perf_counter()
    oracle.project_rows(x[None, :], trellis, suh, svh, IN_F, OUT_F, n, oracle.MCG, threads=threads)
    par = time.perf_counter() - t0
    return {
        "value": code_bytes(IN_F, OUT_F, n) / med / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"{len(times)} whole calls of the same workload (in={IN_F}, out={OUT_F}, n={n}, 1 row), median "
                  f"{med * 1e3:.1f} ms a call; scalar single thread as the reference's format.project",
        "ms_per_call": med * 1e3,
        "all_cores": {"value": code_bytes(IN_F, OUT_F, n) / par / 1e9, "unit": "GB/s", "threads": threads,
                      "note": "decode-once + OpenMP over output blocks, same bits"},
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--sweep", action="store_true", help="also time K = 3, 4, 5 x rows = 1, 4, 16, 32")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--k", type=int, default=4)
    ap.add_argument("--rows", type=int, default=1)
    ap.add_argument("--moe", action="store_true", help="(default on) time the routed-expert decode chain (config 3)")
    ap.add_argument("--quick", action="store_true", help="the headline workload only: no routed or prefill timings")
    ap.add_argument("--prefill", action="store_true",
                    help="(default on) time the routed prefill chain (config 4) and the dense 4096-row projection "
                         "(config 5)")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one 256 MiB device copy, the known-size kernel that scales the profiler's "
                         "FETCH_SIZE / WRITE_SIZE readings")
    ap.add_argument("--dense-rows", default="",
                    help="comma-separated row counts above 32: time the dense projection --in-f x --out-f at --k on the "
                         "trellis GEMM and on the W_hat form (dense_gemm_rows forced either way)")
    ap.add_argument("--in-f", type=int, default=4096)
    ap.add_argument("--out-f", type=int, default=12288)
    args = ap.parse_args()
    global IN_F, OUT_F
    IN_F, OUT_F = args.in_f, args.out_f
    if not args.quick:
        args.moe = args.prefill = True
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU (the path has no collective); --gpus {args.gpus} is not served",
              file=sys.stderr)
        return 2

    import torch

    from turboexl3_amd import api
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    dec = api.Decode.mcg

    def measure(k: int, rows: int, steps: int, warmup: int):
        n = 16 * k
        cb = code_bytes(IN_F, OUT_F, n)
        copies = -(-MIN_ROTATION_BYTES // cb) + 1
        trellis, suh, svh = make_weights(torch, n, copies, seed=1000 + k)
        x = make_x(torch, rows, seed=7)
        run = DenseRunner(torch, api, trellis, suh, svh, x, dec)
        t_call = run.time(steps, warmup)
        t_gemv = run.time(steps, warmup, stages=2)
        plan = api.linear_plan(x, trellis[0], dec)
        return {"k": k, "rows": rows, "code_bytes": cb, "copies": copies, "us_per_call": t_call * 1e6,
                "plan": {key: plan[key] for key in ("path", "launches", "tiles_a_load", "k_slices", "tiles_a_wave",
                                                    "workgroups")},
                "call_gbps": cb / t_call / 1e9, "gemv_us": t_gemv * 1e6, "gemv_gbps": cb / t_gemv / 1e9,
                "gemv_frac_of_hbm": cb / t_gemv / HBM_PEAK}

    if args.traffic_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    head = measure(args.k, args.rows, args.steps, args.warmup)
    out = {
        "metric": "EXL3 GEMV HBM GB/s (% of 8 TB/s) at decode rows; MoE prefill GEMM TFLOP/s",
        "value": head["call_gbps"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["us_per_call"] * 1e-3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"dense decode-row GEMV in={IN_F} out={OUT_F} K={args.k} rows={args.rows} MCG w16, "
                               f"f16 activations, {head['copies']} rotating weight copies",
                   "pct_of_8TBps": 100.0 * head["call_gbps"] * 1e9 / HBM_PEAK, "plan": head["plan"]},
        "roofline": {"bound": "hbm", "achieved": head["gemv_gbps"], "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": head["gemv_frac_of_hbm"],
                     "traffic": MEASURED_TRAFFIC.get((IN_F, OUT_F, args.k, args.rows)), "kernel": "t3::dense_gemv",
                     "us_per_launch": head["gemv_us"], "algorithmic_bytes_per_launch": head["code_bytes"]},
    }
    if args.moe:
        out["moe_decode"] = []
        for tokens in (1, 8):
            run = MoeRunner(torch, api, tokens)
            t = run.time(max(50, args.steps // 2), 10)
            out["moe_decode"].append({"tokens": tokens, "us_per_call": t * 1e6, "code_bytes": run.code_bytes,
                                      "gbps": run.code_bytes / t / 1e9, "frac_of_hbm": run.code_bytes / t / HBM_PEAK})
            del run
    if args.prefill:
        run = PrefillRunner(torch, api)
        t = run.time(5, 2)
        out["moe_prefill"] = {"workload": "2048 tokens, E256 top-8, 7168/2048, gate|up K2, down K3, bf16, clamp 7",
                              "ms_per_call": t * 1e3, "tflops": run.flops / t / 1e12,
                              "frac_of_f16_mfma_peak": run.flops / t / 2.5e15, "code_gbps": run.code_bytes / t / 1e9}
        del run
        torch.cuda.empty_cache()
        rows, in_f, out_f, k = 4096, 4096, 14336, 4
        g = torch.Generator(device="cuda")
        g.manual_seed(3)
        tr = torch.randint(-32768, 32768, (in_f // 16, out_f // 16, 16 * k), dtype=torch.int16, device="cuda", generator=g)
        suh = (0.5 + torch.rand(in_f, device="cuda", generator=g)).to(torch.float16)
        svh = ((0.5 + torch.rand(out_f, device="cuda", generator=g)) / in_f ** 0.5).to(torch.float16)
        x = torch.randn(rows, in_f, device="cuda", generator=g).to(torch.bfloat16)
        api.linear(x, tr, suh, svh, dec)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            api.linear(x, tr, suh, svh, dec)
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / 5
        out["dense_prefill"] = {"workload": "4096 rows x (4096 -> 14336) K4 bf16", "ms_per_call": t * 1e3,
                                "tflops": 2 * rows * in_f * out_f / t / 1e12,
                                "frac_of_f16_mfma_peak": 2 * rows * in_f * out_f / t / 2.5e15}
        # the same projection with its un-rotated weight resident (made once a weight): one plain GEMM a call
        e0.record()
        w_std, bad = api.unrot_weight(tr, suh, svh, dec, torch.bfloat16)
        e1.record()
        torch.cuda.synchronize()
        once = e0.elapsed_time(e1)
        api.linear_unrot(x, w_std)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(5):
            api.linear_unrot(x, w_std)
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / 5
        out["dense_prefill_unrot"] = {"workload": "the same, W_std bf16 resident (117 MB)", "ms_per_call": t * 1e3,
                                      "tflops": 2 * rows * in_f * out_f / t / 1e12,
                                      "frac_of_f16_mfma_peak": 2 * rows * in_f * out_f / t / 2.5e15,
                                      "ms_to_make_w_std_once": once, "nonfinite": bad}
        # and with the W_hat of the trellis kept (decoded once a weight): the call above without its decode
        w_hat = api.dequant(tr, dec)
        api.linear_resident(x, w_hat, suh, svh)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(5):
            api.linear_resident(x, w_hat, suh, svh)
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / 5
        out["dense_prefill_resident"] = {"workload": "the same, W_hat f16 resident (117 MB)", "ms_per_call": t * 1e3,
                                         "tflops": 2 * rows * in_f * out_f / t / 1e12,
                                         "frac_of_f16_mfma_peak": 2 * rows * in_f * out_f / t / 2.5e15}
        del w_hat, w_std
    if args.dense_rows:
        g = torch.Generator(device="cuda")
        g.manual_seed(5)
        tr = torch.randint(-32768, 32768, (IN_F // 16, OUT_F // 16, 16 * args.k), dtype=torch.int16, device="cuda",
                           generator=g)
        suh = (0.5 + torch.rand(IN_F, device="cuda", generator=g)).to(torch.float16)
        svh = ((0.5 + torch.rand(OUT_F, device="cuda", generator=g)) / IN_F ** 0.5).to(torch.float16)

        def dense_us(rows, gemm_rows):
            api.configure(dense_gemm_rows=gemm_rows)
            x = torch.randn(rows, IN_F, device="cuda", generator=g).to(torch.bfloat16)
            api.linear(x, tr, suh, svh, dec)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(5):
                api.linear(x, tr, suh, svh, dec)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / 5

        w_hat = api.dequant(tr, dec)

        def resident_us(rows):
            x = torch.randn(rows, IN_F, device="cuda", generator=g).to(torch.bfloat16)
            api.linear_resident(x, w_hat, suh, svh)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(5):
                api.linear_resident(x, w_hat, suh, svh)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / 5

        out["dense_rows"] = [{"rows": r, "trellis_gemm_us": dense_us(r, 1 << 30), "w_hat_form_us": dense_us(r, 33),
                              "resident_w_hat_us": resident_us(r)}
                             for r in (int(v) for v in args.dense_rows.split(","))]
        api.configure()
    if args.sweep:
        out["sweep"] = [measure(k, r, max(50, args.steps // 4), 10) for k in (3, 4, 5) for r in (1, 4, 16, 32)]
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(16 * args.k, seed=11)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
