#!/usr/bin/env python3
"""Benchmark of the EXL3 projection path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick] [--no-cpu]

A step is one `linear` call of the dense decode-row GEMV workload the headline metric is quoted on
(in=4096, out=12288, K=4 bits/weight, 1 row, MCG codebook, f16 activations with 1 % outliers x20; synthetic seeded
codes). Calls rotate over enough distinct weight copies (> 512 MB in total) that every call reads its codes from
HBM, not from the 256 MB Infinity Cache. Inputs are resident in HBM before the timed region starts. Every timing
captures its calls once into a HIP graph and brackets a replay with events on the launch stream.

Prints ONE JSON line. `value`: the whole call's rate as GB/s of trellis code bytes. `roofline`: the kernel that call
launches (one launch at one row: the call's time is that kernel's), its algorithmic code bytes over its duration
against 8 TB/s; `gemv_launch_alone` is the chain's GEMV launch without prepare and finish, for comparison, and
`launch_floor` what the chain's two small launches cost alone (what any launch costs in a replayed graph). Beside
them, unless --quick: `sweep` (the metric's K = 3, 4, 5 x rows = 1, 4, 16, 32), `lm_head` (4096 -> 151936 at K6, 1 and
256 rows), `moe_decode` (config 3 at 1 and 8 tokens, each launch timed alone as well), `moe_prefill` (config 4, each
stage timed alone, and the same call over MUL1's codebook; TFLOP/s against the 2.5 PFLOP/s f16 MFMA figure and against a
dense f16 GEMM measured in this process, `measured_dense_f16_peak`), `dense_prefill` (config 5's 4096 rows and its
resident-weight forms),
`measured_hbm_read_peak` (a plain 16-byte-a-lane read of 2 GiB in this process: every HBM fraction is also given against
it), `plain_read_of_the_same_bytes` (the same read kernel over the headline's own 25 MB weight copies, launch by launch:
what start, first bytes and drain cost a launch of this size whatever it computes), `streaming` (one row of 4096 -> 151936 at K = 3, 4, 5: matrices of 233 to 389 MB, where a launch's ramp, tail and
hand-off vanish and the kernel's steady state shows), `reference_workload` (the reference's own published workload:
2560 x 640, 512 experts, top-10, bf16, MUL1, K2..K8 at 1 and 4 rows as chains of 48 dependent calls over fresh experts,
prefill at 8192 and 1328 rows; context beside docs/models/qwen38/results.md, never the target),
`codebook_forms` (what the other codebook forms cost in the GEMV), `rates` (a fractional narrow rate and a wide one) and
`dense_rows` (few-row dense calls with and without the rows-alone partition), `shapes` (shapes beside the metric's own:
what the rules that pick a path from the shape serve, beside the other path). `cpu_baseline`: the CPU oracle
(`format.project` restated in C) timed on this box's host cores, and, in the same leg, one sampled output block (or row)
of every timed cell held against the oracle by the reference's bars (`parity_checks`).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

IN_F, OUT_F = 4096, 12288
HBM_PEAK = 8.0e12
MFMA_F16_PEAK = 2.5e15
MIN_ROTATION_BYTES = 512 << 20
READ_PEAK_GBPS = None  # measured at start-up (measured_hbm_read)
# HBM bytes one launch of the served one-row kernel (the one-launch form) moves, from the profiler's FETCH_SIZE and
# WRITE_SIZE counters scaled by a 256 MiB copy (profiles/dense_gemv_in4096_out12288_k4_rows1.txt): keyed by the sources
# of the kernel the figure was measured on (`kernel_sources_key`), then by (in, out, n, rows). A kernel whose sources
# have changed since reports null until it is measured again.
MEASURED_TRAFFIC = {
    # one launch: FETCH_SIZE 12641.6 x 1.99973 = 25279.9 KiB read + WRITE_SIZE 435.0 KiB = 1.046 x the code bytes
    "701b8c38984d9268": {(4096, 12288, 64, 1): 26332051},
}
GEMV_SOURCES = ("t3_dense.hip", "t3_gemv_core.hpp", "t3_lds_loads.hpp", "t3_decode.hpp", "t3_stages.hpp", "t3_common.hpp")


def kernel_sources_key() -> str:
    """The first 16 hex digits of sha256 over the dense GEMV's source files and the build script (its compiler flags)
    as they lie in the tree, comments and white space left out: what the compiler sees of them."""
    import hashlib
    import re
    h = hashlib.sha256()
    for path in [os.path.join("csrc", name) for name in GEMV_SOURCES] + ["build.py"]:
        with open(os.path.join(ROOT, "turboexl3_amd", path), "r") as f:
            text = f.read()
        if path.endswith(".py"):
            text = re.sub(r"#[^\n]*", "", text)
        else:
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            text = re.sub(r"//[^\n]*", "", text)
        h.update(" ".join(text.split()).encode())
    return h.hexdigest()[:16]
F32_BAR, BF16_DENSE_BAR, BF16_MOE_BAR = 5e-3, 2.5e-2, 1.5e-2

MCG_CB, MUL1_CB = 1, 0


def code_bytes(in_f: int, out_f: int, n: int) -> int:
    """Algorithmic bytes of one projection: (in/16)(out/16) tiles of n halfwords."""
    return (in_f // 16) * (out_f // 16) * n * 2


def graph_times(torch, call, steps: int, warmup: int, replays: int = 1) -> list:
    """Seconds a call, one figure a timed replay (sorted), over exactly `steps` back-to-back calls `call(i, stream)`
    captured once into a HIP graph (as a serving loop would hold its decode step) so the host's per-launch cost stays out
    of the GPU's timeline; events bracket each replay on the launch stream (the reference's bench reports its rounds'
    median and fastest the same way, src/core/bench.zig:193-225)."""
    cur = torch.cuda.current_stream().cuda_stream
    for i in range(max(warmup, 1)):
        call(i, cur)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for i in range(steps):
                call(warmup + i, side.cuda_stream)
        torch.cuda.synchronize()
        graph.replay()  # untimed: the graph's first replay uploads it
        torch.cuda.synchronize()
        took = []
        for _ in range(replays):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            graph.replay()
            e1.record(side)
            torch.cuda.synchronize()
            took.append(e0.elapsed_time(e1))
    return [t * 1e-3 / steps for t in sorted(took)]


def graph_time(torch, call, steps: int, warmup: int, replays: int = 1) -> float:
    """The median of `graph_times`."""
    took = graph_times(torch, call, steps, warmup, replays)
    return took[len(took) // 2]


def host_u16(t) -> np.ndarray:
    import torch
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


class Dense:
    """One dense shape at one rate: rotating weight copies, descriptors built once, nothing allocated while timing."""

    def __init__(self, torch, api, in_f, out_f, n, codebook, max_rows, act_dtype, seed, copies=None, outliers=True):
        from turboexl3_amd import _lib
        self.torch, self.api, self.L = torch, api, _lib.lib()
        self.in_f, self.out_f, self.n, self.codebook = in_f, out_f, n, codebook
        self.dec = api.Decode(codebook, 16)
        self.cb = code_bytes(in_f, out_f, n)
        self.copies = copies or (-(-MIN_ROTATION_BYTES // self.cb) + 1)
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)
        self.trellis = torch.randint(-32768, 32768, (self.copies, in_f // 16, out_f // 16, n), dtype=torch.int16,
                                     device="cuda", generator=g)
        sign = lambda k: (torch.randint(0, 2, (k,), device="cuda", generator=g) * 2 - 1).to(torch.float32)
        self.suh = (sign(in_f) * (1.0 + 0.1 * torch.randn(in_f, device="cuda", generator=g))).to(torch.float16)
        self.svh = (sign(out_f) * (1.0 + 0.1 * torch.randn(out_f, device="cuda", generator=g)) / (in_f ** 0.5)).to(torch.float16)
        x = torch.randn(max_rows, in_f, device="cuda", generator=g)
        if outliers:
            x = torch.where(torch.rand(max_rows, in_f, device="cuda", generator=g) < 0.01, x * 20.0, x)
        self.x = x.to(act_dtype)
        self.at = [api._arr(self.trellis[i]) for i in range(self.copies)]
        self.asu, self.asv = api._arr(self.suh), api._arr(self.svh)
        self.ws = None

    def bind(self, rows: int):
        api = self.api
        self.rows = rows
        self.xr = self.x[:rows]
        self.ax = api._arr(self.xr)
        self.y = self.torch.empty(rows, self.out_f, dtype=self.x.dtype, device="cuda")
        self.ay = api._arr(self.y)
        need = C.c_size_t(0)
        st = self.L.t3_linear_workspace_bytes(C.byref(self.ax), C.byref(self.at[0]), self.dec.c(), C.byref(need))
        assert st == 0, self.L.t3_error_name(st).decode()
        if self.ws is None or self.ws.numel() < need.value:
            self.ws = self.torch.zeros(need.value, dtype=self.torch.uint8, device="cuda")
        self.plan = api.linear_plan(self.xr, self.trellis[0], self.dec)

    def call(self, i: int, stream: int, stages: int = 0):
        t = self.at[i % self.copies]
        dec = self.dec.c()
        if stages:
            st = self.L.t3_linear_stages(stream, C.byref(self.ax), C.byref(t), C.byref(self.asu), C.byref(self.asv), dec,
                                         C.byref(self.ay), self.ws.data_ptr(), self.ws.numel(), stages)
        else:
            st = self.L.t3_linear(stream, C.byref(self.ax), C.byref(t), C.byref(self.asu), C.byref(self.asv), dec,
                                  C.byref(self.ay), self.ws.data_ptr(), self.ws.numel())
        if st != 0:
            raise RuntimeError(self.L.t3_error_name(st).decode())

    def sample(self, name: str, blk: int, rows_to_check, bar: float, half_ulp: float):
        """One eager call over copy 0, and what the CPU leg needs to hold output columns [128 blk, 128 blk + 128) of the
        chosen rows against format.project."""
        torch = self.torch
        self.call(0, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        rows_to_check = sorted(set(rows_to_check))
        return {"kind": "dense", "cell": name, "in_f": self.in_f, "n": self.n, "codebook": self.codebook, "bar": bar,
                "half_ulp": half_ulp, "rows": rows_to_check,
                "trellis": host_u16(self.trellis[0][:, 8 * blk:8 * blk + 8, :]), "suh": host_u16(self.suh.view(torch.int16)),
                "svh": host_u16(self.svh[128 * blk:128 * blk + 128].view(torch.int16)),
                "x": self.xr[rows_to_check].to(torch.float32).cpu().numpy(),
                "y": self.y[rows_to_check, 128 * blk:128 * blk + 128].to(torch.float32).cpu().numpy()}

    def time(self, steps: int, warmup: int, stages: int = 0, replays: int = 3) -> float:
        return graph_time(self.torch, lambda i, s: self.call(i, s, stages), steps, warmup, replays)

    def times(self, steps: int, warmup: int, replays: int) -> list:
        return graph_times(self.torch, lambda i, s: self.call(i, s, 0), steps, warmup, replays)


def dense_cell(d: Dense, rows: int, steps: int, warmup: int, todo: list, name: str, gemv_alone: bool = False,
               replays: int = 3) -> dict:
    import torch
    d.bind(rows)
    bf16 = d.x.dtype == torch.bfloat16
    todo.append(d.sample(name, blk=(d.out_f // 128) // 3, rows_to_check=[0, rows - 1],
                         bar=BF16_DENSE_BAR if bf16 else F32_BAR, half_ulp=2.0 ** -8 if bf16 else 2.0 ** -11))
    took = d.times(steps, warmup, replays)
    t = took[len(took) // 2]
    out = {"n": d.n, "k": d.n / 16, "rows": rows, "code_bytes": d.cb, "copies": d.copies, "us_per_call": t * 1e6,
           "us_per_call_min": took[0] * 1e6, "replays": replays,
           "call_gbps": d.cb / t / 1e9, "frac_of_hbm": d.cb / t / HBM_PEAK,
           "frac_of_measured_read_peak": d.cb / t / 1e9 / READ_PEAK_GBPS if READ_PEAK_GBPS else None,
           "plan": {key: d.plan[key] for key in ("path", "launches", "tiles_a_load", "k_slices", "tiles_a_wave", "workgroups")}}
    if gemv_alone and rows <= 32:
        tg = d.time(steps, warmup, stages=2)
        out.update({"gemv_us": tg * 1e6, "gemv_gbps": d.cb / tg / 1e9, "gemv_frac_of_hbm": d.cb / tg / HBM_PEAK,
                    "gemv_frac_of_measured_read_peak": d.cb / tg / 1e9 / READ_PEAK_GBPS if READ_PEAK_GBPS else None})
    return out


class Moe:
    """A routed call over a synthetic bank: config 3 (decode rows, a shared expert in the same launches, rotating routings
    so every call reads fresh experts from HBM) or config 4 (prefill)."""

    def __init__(self, torch, api, experts, hidden, inter, k_gu, k_dn, topk, tokens, limit, shared: bool, sets: int, seed: int):
        from turboexl3_amd import _lib
        self.torch, self.api, self.L = torch, api, _lib.lib()
        self.E, self.hidden, self.inter, self.topk, self.tokens, self.limit = experts, hidden, inter, topk, tokens, limit
        self.n_gu, self.n_dn = 16 * k_gu, 16 * k_dn
        g = torch.Generator(device="cuda")
        g.manual_seed(seed)

        def proj(e, in_f, out_f, n):
            t = torch.randint(-32768, 32768, (e, in_f // 16, out_f // 16, n), dtype=torch.int16, device="cuda", generator=g)
            suh = (0.5 + torch.rand(e, in_f, device="cuda", generator=g)).to(torch.float16)
            svh = ((0.5 + torch.rand(e, out_f, device="cuda", generator=g)) / in_f ** 0.5).to(torch.float16)
            return api.Proj(t, suh, svh)

        def bank(e):
            return api.Bank(proj(e, hidden, inter, self.n_gu), proj(e, hidden, inter, self.n_gu), proj(e, inter, hidden, self.n_dn))

        self.bank = bank(experts)
        self.shared = bank(1) if shared else None
        self.x = torch.randn(1, tokens, hidden, device="cuda", generator=g).to(torch.bfloat16)
        # router logits ~ N(0,1) -> top-k -> softmax over the selected (harness side, as in the reference's benches)
        self.sets = sets
        logits = torch.randn(sets, tokens, experts, device="cuda", generator=g)
        top = torch.topk(logits, topk, dim=-1)
        self.inds = top.indices.to(torch.int32).contiguous()
        self.scores = torch.softmax(top.values, dim=-1).to(torch.float32).contiguous()
        self.cb, self._k1 = api._cbank(self.bank)
        self.sb, self._k2 = api._cbank(self.shared) if shared else (None, None)
        self.ax = api._arr(self.x)
        self.ai = [api._arr(self.inds[i:i + 1]) for i in range(sets)]
        self.asc = [api._arr(self.scores[i:i + 1]) for i in range(sets)]
        self.y = torch.empty_like(self.x)
        self.ay = api._arr(self.y)
        need = C.c_size_t(0)
        sbp = C.byref(self.sb) if shared else None
        st = self.L.t3_moe_workspace_bytes(C.byref(self.ax), C.byref(self.cb), C.byref(self.ai[0]), sbp, C.byref(need))
        assert st == 0, self.L.t3_error_name(st).decode()
        self.ws = torch.zeros(need.value, dtype=torch.uint8, device="cuda")
        self.dec = api.Decode.mcg
        self.per_expert = code_bytes(hidden, inter, self.n_gu) * 2 + code_bytes(inter, hidden, self.n_dn)
        distinct = [len(set(self.inds[i].flatten().tolist())) for i in range(sets)]
        self.distinct = sum(distinct) / sets + (1 if shared else 0)
        self.flops = tokens * topk * 3 * 2 * hidden * inter
        self.plan = api.moe_plan(self.x, self.bank, self.inds[0:1], self.shared)

    def call(self, i: int, stream: int, stages: int = 63):
        j = i % self.sets
        sbp = C.byref(self.sb) if self.sb is not None else None
        st = self.L.t3_moe_stages(stream, C.byref(self.ax), C.byref(self.cb), C.byref(self.ai[j]), C.byref(self.asc[j]),
                                  self.dec.c(), self.limit, sbp, C.byref(self.ay), self.ws.data_ptr(), self.ws.numel(), stages)
        if st != 0:
            raise RuntimeError(self.L.t3_error_name(st).decode())

    def time(self, steps: int, warmup: int, stages: int = 63, replays: int = 3) -> float:
        return graph_time(self.torch, lambda i, s: self.call(i, s, stages), steps, warmup, replays)

    def sample(self, name: str, token: int, bar: float):
        """One eager call over routing 0, and the chosen token's experts for ref.moeRowClamped on the host."""
        torch = self.torch
        self.call(0, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        ids = self.inds[0, token].tolist()
        side = lambda t, sh: np.stack([host_u16(t[e].view(torch.int16)) for e in ids] +
                                      ([host_u16(sh[0].view(torch.int16))] if self.shared else []))
        b, s = self.bank, self.shared
        arrays = {}
        for nm in ("gate", "up", "down"):
            p, q = getattr(b, nm), getattr(s, nm) if s else None
            arrays[nm + "_t"] = np.stack([host_u16(p.trellis[e]) for e in ids] + ([host_u16(q.trellis[0])] if s else []))
            arrays[nm + "_suh"] = side(p.suh, q.suh if s else None)
            arrays[nm + "_svh"] = side(p.svh, q.svh if s else None)
        scores = self.scores[0, token].tolist() + ([1.0] if s else [])
        return {"kind": "moe", "cell": name, "codebook": self.dec.codebook, "hidden": self.hidden, "inter": self.inter, "n_gu": self.n_gu, "n_dn": self.n_dn,
                "limit": float(self.limit), "bar": bar, "arrays": arrays, "scores": np.asarray(scores, dtype=np.float32),
                "x": self.x[0, token].to(torch.float32).cpu().numpy(), "y": self.y[0, token].to(torch.float32).cpu().numpy()}


def measured_f16_peak(torch) -> dict:
    """A plain dense f16 GEMM (8192^3, the library GEMM torch dispatches to) in this process: the matrix cores' practical
    rate on this GPU at its sustained clock, beside the 2.5 PFLOP/s figure."""
    m = 8192
    a = torch.randn(m, m, device="cuda", dtype=torch.float16)
    b = torch.randn(m, m, device="cuda", dtype=torch.float16)
    for _ in range(3):
        torch.matmul(a, b)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    reps = 10
    for _ in range(reps):
        torch.matmul(a, b)
    e1.record()
    torch.cuda.synchronize()
    t = e0.elapsed_time(e1) * 1e-3 / reps
    return {"tflops": 2 * m ** 3 / t / 1e12, "shape": f"{m} x {m} x {m} f16, f32 accumulate", "ms": t * 1e3,
            "frac_of_2.5_pflops": 2 * m ** 3 / t / MFMA_F16_PEAK}


def measured_hbm_read(torch) -> dict:
    """A plain read of 2 GiB (eight times the Infinity Cache), 16 bytes a lane, by this library's own measurement kernel
    in this process: what HBM gives a kernel that does nothing with its bytes, beside the 8 TB/s figure. The best of a few
    workgroup counts, each the median of five launches."""
    from turboexl3_amd import _lib
    L = _lib.lib()
    nbytes = 2 << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda").random_()
    best = None
    for wgs in (2048, 4096, 8192, 16384):
        sink = torch.empty(wgs * 256, dtype=torch.int32, device="cuda")
        stream = torch.cuda.current_stream().cuda_stream
        took = []
        for it in range(7):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            st = L.t3_test_hbm_read(stream, src.data_ptr(), nbytes, sink.data_ptr(), wgs)
            e1.record()
            torch.cuda.synchronize()
            if st != 0:
                raise RuntimeError(L.t3_error_name(st).decode())
            if it >= 2:
                took.append(e0.elapsed_time(e1) * 1e-3)
        t = sorted(took)[len(took) // 2]
        if best is None or t < best[0]:
            best = (t, wgs)
    del src
    torch.cuda.empty_cache()
    return {"gbps": nbytes / best[0] / 1e9, "bytes": nbytes, "us": best[0] * 1e6, "workgroups": best[1],
            "frac_of_8TBps": nbytes / best[0] / HBM_PEAK,
            "kernel": "t3_test_hbm_read (global_load_dwordx4 a lane, eight in flight, folded and stored)"}


def eager_time(torch, fn, reps: int = 5) -> float:
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e-3 / reps


def shapes_section(torch, api) -> dict:
    """Shapes beside the metric's own, one cell each for a rule that picks a path from the shape: what the served call
    takes and what the other path would (the same bytes either way, or the same bars)."""
    out = {}
    # a small matrix: four tiles a load while eight would leave at most 128 workgroups
    cells = []
    for in_f, out_f, n, rows in ((2560, 640, 64, 1), (2048, 2048, 64, 1), (2048, 2048, 64, 32)):
        d = Dense(torch, api, in_f, out_f, n, MCG_CB, 32, torch.float16, seed=77)
        d.bind(rows)
        cells.append({"in": in_f, "out": out_f, "n": n, "rows": rows, "us_per_call": d.time(96, 8) * 1e6,
                      "plan": {k: d.plan[k] for k in ("launches", "tiles_a_load", "k_slices", "workgroups")}})
        del d
    out["dense_small"] = cells
    # above 32 rows: the trellis GEMM (K parts within one round of resident workgroups) or the W_hat form (where its
    # GEMM's tiles fill the GPU)
    cells = []
    for in_f, out_f, n, rows in ((7168, 2048, 48, 1024), (4096, 4096, 64, 640), (4096, 14336, 64, 640), (8192, 8192, 64, 1536)):
        d = Dense(torch, api, in_f, out_f, n, MCG_CB, rows, torch.bfloat16, seed=78, copies=2, outliers=False)
        took = {}
        for name, cfg in (("served", {}), ("trellis_gemm", {"dense_gemm_rows": 0}),
                          ("w_hat_form", {"dense_gemm_rows": 1})):
            api.configure(**cfg)
            try:
                d.bind(rows)
                took[name + "_us"] = d.time(8, 2) * 1e6
                if name == "served":
                    took["served_plan"] = {k: d.plan[k] for k in ("path", "k_slices", "workgroups")}
            finally:
                api.configure()
        cells.append({"in": in_f, "out": out_f, "n": n, "rows": rows, **took})
        del d
    out["dense_above_32_rows"] = cells
    # a call of few rows over a kept weight: the plain GEMM shares K out over the grid where its tiles are few
    d = Dense(torch, api, 4096, 14336, 64, MCG_CB, 64, torch.bfloat16, seed=81, copies=1, outliers=False)
    w_hat = api.dequant(d.trellis[0], d.dec)
    w_std, _ = api.unrot_weight(d.trellis[0], d.suh, d.svh, d.dec, torch.bfloat16)
    x = d.x[:64]
    took = {name: graph_time(torch, fn, 8, 2, 3) * 1e6 for name, fn in (
        ("linear_us", lambda i, st: api.linear(x, d.trellis[0], d.suh, d.svh, d.dec)),
        ("resident_w_hat_us", lambda i, st: api.linear_resident(x, w_hat, d.suh, d.svh)),
        ("w_std_us", lambda i, st: api.linear_unrot(x, w_std)),
        ("w_std_k_parts_us", lambda i, st: api.linear_unrot_parts(x, w_std)))}
    out["dense_64_rows_over_kept_weights"] = {"in": 4096, "out": 14336, "n": 64, "rows": 64, **took}
    del d, w_hat, w_std, x
    # routed decode over large experts: two launches up to 8192 gate|up workgroups; past it the five launches behind a
    # grouping launch (the row-slots of one expert served together); GLM's profile
    cells = []
    m = None
    for tokens in (1, 4, 8, 16):
        m = Moe(torch, api, 64, 4096, 2048, 4, 4, 8, tokens, 7, shared=False, sets=8, seed=79)
        took = {}
        for name, form in (("served", 9), ("five_launches", 3)):
            api.configure(decode_form=form)
            try:
                took[name + "_us"] = m.time(48, 6) * 1e6
            finally:
                api.configure()
        cells.append({"experts": 64, "hidden": 4096, "inter": 2048, "k": 4, "topk": 8, "tokens": tokens, **took,
                      "served_launches": m.plan["launches"], "distinct_experts": m.distinct})
        if tokens != 1:
            del m
            m = None
        else:
            # GLM's profile over the same bank at one token (the last slot of the row is the host's shared expert)
            y = torch.zeros(1, 1, m.topk, m.hidden, dtype=torch.float32, device="cuda")
            ay = api._arr(y)
            inds = [torch.cat([m.inds[j, :, :m.topk - 1], torch.full((1, 1), m.E, dtype=torch.int32, device="cuda")], dim=1)
                    .reshape(1, 1, m.topk).contiguous() for j in range(m.sets)]
            ai = [api._arr(t) for t in inds]

            def glm_call(i, stream, m=m, ai=ai, ay=ay):
                st = m.L.t3_moe_glm(stream, C.byref(m.ax), C.byref(m.cb), C.byref(ai[i % m.sets]), m.dec.c(), 7, C.byref(ay),
                                    m.ws.data_ptr(), m.ws.numel())
                if st != 0:
                    raise RuntimeError(m.L.t3_error_name(st).decode())

            glm = {}
            for name, form in (("two_launches", 9), ("five_launches", 3)):
                api.configure(decode_form=form)
                try:
                    glm[name + "_us"] = graph_time(torch, glm_call, 48, 6, 3) * 1e6
                finally:
                    api.configure()
            out["moe_glm_one_token"] = {"experts": 64, "hidden": 4096, "inter": 2048, "k": 4, "topk": 7, **glm}
            del m, y, inds, ai
            m = None
    # few experts, each very large (eight of 4096 x 14336, top-2): most row-slots of a call share their expert
    for tokens in (4, 16):
        m = Moe(torch, api, 8, 4096, 14336, 4, 4, 2, tokens, 0, shared=False, sets=8, seed=80)
        took = {}
        for name, form in (("served", 9), ("five_launches", 3)):
            api.configure(decode_form=form)
            try:
                took[name + "_us"] = m.time(24, 4) * 1e6
            finally:
                api.configure()
        cells.append({"experts": 8, "hidden": 4096, "inter": 14336, "k": 4, "topk": 2, "tokens": tokens, **took,
                      "served_launches": m.plan["launches"], "distinct_experts": m.distinct})
        del m
    out["moe_decode_large_experts"] = cells
    torch.cuda.empty_cache()
    return out


# docs/models/qwen38/results.md:293-317 (decode, captured routing: form 9, median us at 1 and 4 rows), :326-350 (synthetic
# routing), :359-372 (prefill: median us and TFLOPS at 8192 and 1328 rows), all measured on one Apple M5 Max
REFERENCE_M5_MAX = {
    "decode_captured_us": {2: (70.7, 189.9), 3: (74.3, 199.3), 4: (69.9, 188.0), 5: (76.8, 207.0), 6: (82.4, 231.4),
                           7: (93.4, 269.9), 8: (105.8, 282.8)},
    "decode_synthetic_us": {2: (70.8, 217.0), 3: (74.6, 228.5), 4: (70.8, 215.0), 5: (79.7, 248.9), 6: (88.1, 285.8),
                            7: (98.3, 326.3), 8: (111.1, 370.2)},
    "prefill_us": {2: (19682, 4524), 3: (19935, 4729), 4: (19799, 4507), 5: (20067, 4808), 6: (20168, 4987),
                   7: (20773, 5436), 8: (20662, 5702)},
    "prefill_tflops": {2: (40.9, 28.9), 3: (40.4, 27.6), 4: (40.7, 29.0), 5: (40.1, 27.2), 6: (39.9, 26.2),
                       7: (38.8, 24.0), 8: (39.0, 22.9)},
}


def reference_section(torch, api, todo: list, rates=(2, 3, 4, 5, 6, 7, 8)) -> dict:
    """The reference's own published workload (docs/models/qwen38/results.md:278-284): Qwen3.8-Flash-Next's MoE layer,
    hidden 2560, expert width 640, 512 experts, top-10, bf16, MUL1, random codes at each rate. Decode: a chain of 48
    dependent calls (a call's output is the next call's input, every call routes to fresh experts drawn at random, so its
    weights come from HBM) divided by 48; median and fastest of the timed replays. Prefill: 4 back-to-back calls at 8192
    and at 1328 rows. The M5 Max figures the reference publishes stand beside each cell as context: another machine,
    never a target."""
    hidden, inter, experts, topk = 2560, 640, 512, 10
    out = {"workload": "hidden 2560, expert width 640, 512 experts, top-10, bf16, MUL1, random codes; synthetic routing",
           "reference_hardware": "Apple M5 Max (docs/models/qwen38/results.md:3,246-247)", "decode": [], "prefill": []}
    for k in rates:
        for rows in (1, 4):
            m = Moe(torch, api, experts, hidden, inter, k, k, topk, rows, 0, shared=False, sets=48, seed=300 + k)
            m.dec = api.Decode(MUL1_CB, 16)
            todo.append(m.sample(f"reference workload decode K{k} rows {rows}, row 0", 0, BF16_MOE_BAR))
            # the dependent chain: call i reads buffer i % 2 and writes the other
            bufs = [m.x.clone(), torch.empty_like(m.x)]
            arrs = [api._arr(b) for b in bufs]

            def chained(i, stream, m=m, arrs=arrs):
                j = i % m.sets
                st = m.L.t3_moe_stages(stream, C.byref(arrs[i % 2]), C.byref(m.cb), C.byref(m.ai[j]), C.byref(m.asc[j]),
                                       m.dec.c(), 0, None, C.byref(arrs[(i + 1) % 2]), m.ws.data_ptr(), m.ws.numel(), 63)
                if st != 0:
                    raise RuntimeError(m.L.t3_error_name(st).decode())

            took = graph_times(torch, chained, 48, 48, 9)
            med, best = took[len(took) // 2], took[0]
            bytes_call = m.distinct * m.per_expert
            ri = 0 if rows == 1 else 1
            out["decode"].append({
                "k": k, "rows": rows, "us_per_call_median": med * 1e6, "us_per_call_fastest": best * 1e6,
                "distinct_experts": m.distinct, "code_bytes": bytes_call, "gbps": bytes_call / med / 1e9,
                "frac_of_hbm": bytes_call / med / HBM_PEAK, "launches": m.plan["launches"],
                "m5_max_form9_us_synthetic_routing": REFERENCE_M5_MAX["decode_synthetic_us"][k][ri],
                "m5_max_form9_us_captured_routing": REFERENCE_M5_MAX["decode_captured_us"][k][ri]})
            del m, bufs, arrs
        for ri, rows in enumerate((8192, 1328)):
            m = Moe(torch, api, experts, hidden, inter, k, k, topk, rows, 0, shared=False, sets=1, seed=400 + k)
            m.dec = api.Decode(MUL1_CB, 16)
            todo.append(m.sample(f"reference workload prefill K{k} rows {rows}, row 0", 0, BF16_MOE_BAR))
            took = graph_times(torch, lambda i, st, m=m: m.call(i, st), 4, 2, 5)
            med, best = took[len(took) // 2], took[0]
            out["prefill"].append({
                "k": k, "rows": rows, "us_per_call_median": med * 1e6, "us_per_call_fastest": best * 1e6,
                "tflops": m.flops / med / 1e12, "frac_of_f16_mfma_peak": m.flops / med / MFMA_F16_PEAK,
                "item_rows": m.plan["item_rows"],
                "m5_max_us": REFERENCE_M5_MAX["prefill_us"][k][ri], "m5_max_tflops": REFERENCE_M5_MAX["prefill_tflops"][k][ri]})
            del m
        torch.cuda.empty_cache()
    return out


def cpu_leg(n: int, seed: int, todo: list, budget_s: float = 20.0):
    """The only place this program touches the CPU oracle. (1) format.project (the C restatement) timed on the host: the
    headline workload's shape and seeded distributions, one row, one thread, re-decoding every tile as the reference does;
    a bounded sample: whole calls until ~budget_s is spent. (2) The sampled outputs of the timed cells held against it."""
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
    threads = min(os.cpu_count() or 1, 16)
    t0 = time.perf_counter()
    oracle.project_rows(x[None, :], trellis, suh, svh, IN_F, OUT_F, n, oracle.MCG, threads=threads)
    par = time.perf_counter() - t0
    base = {
        "value": code_bytes(IN_F, OUT_F, n) / med / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"{len(times)} whole calls of the same workload (in={IN_F}, out={OUT_F}, n={n}, 1 row), median "
                  f"{med * 1e3:.1f} ms a call; scalar single thread as the reference's format.project",
        "ms_per_call": med * 1e3,
        "all_cores": {"value": code_bytes(IN_F, OUT_F, n) / par / 1e9, "unit": "GB/s", "threads": threads,
                      "note": "decode-once + OpenMP over output blocks, same bits"},
    }
    checks = []
    for s in todo:
        if s["kind"] == "dense":
            ref = oracle.project_rows(s["x"], s["trellis"], s["suh"], s["svh"], s["in_f"], 128, s["n"], s["codebook"], 0xFFFF,
                                      threads=threads)
            err = max(oracle.compare(s["y"][i], ref[i], s["half_ulp"]) for i in range(len(s["rows"])))
        else:
            a = s["arrays"]
            bank = oracle.Bank(a["gate_t"].shape[0], s["hidden"], s["inter"], s["n_gu"], s["n_dn"], a["gate_t"], a["gate_suh"],
                               a["gate_svh"], a["up_t"], a["up_suh"], a["up_svh"], a["down_t"], a["down_suh"], a["down_svh"])
            want, _ = oracle.moe_row(bank, s["x"], np.arange(len(s["scores"]), dtype=np.int32), s["scores"], s["codebook"],
                                     0xFFFF, s["limit"])
            err = oracle.compare(s["y"], want, 2.0 ** -8)
        checks.append({"cell": s["cell"], "err_over_rms": err, "bar": s["bar"], "ok": bool(err <= s["bar"])})
    return base, checks


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU leg (the oracle's timing and the parity checks)")
    ap.add_argument("--k", type=int, default=4)
    ap.add_argument("--rows", type=int, default=1)
    ap.add_argument("--quick", action="store_true", help="the headline workload only")
    ap.add_argument("--only", default="", help="comma-separated sections to run beside the headline: sweep, forms, rates, "
                                               "streaming, lm_head, moe_decode, moe_prefill, dense_prefill, dense_rows, peak, shapes, reference")
    ap.add_argument("--sweep", action="store_true", help="(default on) K = 3, 4, 5 x rows = 1, 4, 16, 32")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one 256 MiB device copy, the known-size kernel that scales the profiler's "
                         "FETCH_SIZE / WRITE_SIZE readings")
    ap.add_argument("--in-f", type=int, default=4096)
    ap.add_argument("--out-f", type=int, default=12288)
    args = ap.parse_args()
    global IN_F, OUT_F
    IN_F, OUT_F = args.in_f, args.out_f
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU (the path has no collective); --gpus {args.gpus} is not served",
              file=sys.stderr)
        return 2
    sections = {"sweep", "forms", "rates", "streaming", "lm_head", "moe_decode", "moe_prefill", "dense_prefill", "dense_rows",
                "peak", "shapes", "reference"}
    if args.quick:
        sections = set()
    elif args.only:
        sections = set(args.only.split(","))

    import torch

    from turboexl3_amd import api
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    todo: list = []
    sub_steps = max(50, args.steps // 4)

    if args.traffic_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # what HBM gives a plain read in this process: every HBM-bound cell states its fraction of it beside 8 TB/s
    global READ_PEAK_GBPS
    hbm_read = measured_hbm_read(torch)
    READ_PEAK_GBPS = hbm_read["gbps"]

    # ---- the headline: one row of the q|k|v shape --------------------------------------------------------------
    n_head = 16 * args.k
    d = Dense(torch, api, IN_F, OUT_F, n_head, MCG_CB, 32, torch.float16, seed=1000 + args.k)
    # the headline: the same --steps calls (one captured graph) replayed five times, the median taken, the fastest beside it
    head = dense_cell(d, args.rows, args.steps, args.warmup, todo, f"headline K{args.k} rows {args.rows}", gemv_alone=True,
                      replays=5)
    one_launch = head["plan"]["launches"] == 1
    out = {
        "metric": "EXL3 GEMV HBM GB/s (% of 8 TB/s) at decode rows; MoE prefill GEMM TFLOP/s",
        "value": head["call_gbps"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["us_per_call"] * 1e-3, "ms_per_step_min": head["us_per_call_min"] * 1e-3,
        "timing": "median of 5 replays of one HIP graph of --steps calls; ms_per_step_min: the fastest replay",
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"dense decode-row GEMV in={IN_F} out={OUT_F} K={args.k} rows={args.rows} MCG w16, "
                               f"f16 activations, {head['copies']} rotating weight copies",
                   "pct_of_8TBps": 100.0 * head["frac_of_hbm"], "plan": head["plan"]},
        # the kernel the timed step launches: at one row the call is that one launch, so its duration is the call's
        "roofline": {"bound": "hbm", "achieved": head["call_gbps"], "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": head["frac_of_hbm"],
                     "traffic": MEASURED_TRAFFIC.get(kernel_sources_key(), {}).get((IN_F, OUT_F, n_head, args.rows)),
                     "kernel_sources_key": kernel_sources_key(),
                     "kernel": "t3::dense_gemv<kMcg, narrow, 1 row block, 8 tiles, one launch> (prepare, GEMV and finish "
                               "in the launch)" if one_launch else "t3::dense_gemv (the call's GEMV launch, see gemv_launch_alone)",
                     "us_per_launch": head["us_per_call"] if one_launch else head.get("gemv_us"),
                     "algorithmic_bytes_per_launch": head["code_bytes"]},
        "gemv_launch_alone": {"kernel": "t3::dense_gemv<..., chain> (t3_linear_stages, the GEMV stage only: planes out, no "
                                        "prepare, no finish)", "us_per_launch": head.get("gemv_us"),
                              "achieved": head.get("gemv_gbps"), "unit": "GB/s", "frac": head.get("gemv_frac_of_hbm")},
    }

    # what a launch costs here whatever it computes: the chain's prepare and finish launches alone (32 and 96 one-wave
    # workgroups), each replayed back to back in a graph like every other cell
    d.bind(args.rows)
    out["launch_floor"] = {"prepare_launch_alone_us": d.time(sub_steps, 10, stages=1) * 1e6,
                           "finish_launch_alone_us": d.time(sub_steps, 10, stages=4) * 1e6,
                           "chain_three_launches_us": d.time(sub_steps, 10, stages=7) * 1e6}

    out["measured_hbm_read_peak"] = hbm_read
    out["roofline"]["frac_of_measured_read_peak"] = head["call_gbps"] / READ_PEAK_GBPS
    # what a launch that only reads the headline's bytes takes: the same rotating copies, the same graph of back-to-back
    # launches, the plain read kernel (start, first bytes and drain of a 25 MB launch included, as in `value`)
    sink = torch.empty(4096 * 256, dtype=torch.int32, device="cuda")

    def plain(i, stream, wgs):
        st = d.L.t3_test_hbm_read(stream, d.trellis[i % d.copies].data_ptr(), d.cb, sink.data_ptr(), wgs)
        if st != 0:
            raise RuntimeError(d.L.t3_error_name(st).decode())

    reads = {wgs: graph_time(torch, lambda i, s2: plain(i, s2, wgs), sub_steps, 10, 3) for wgs in (768, 1536, 2048)}
    wgs = min(reads, key=reads.get)
    out["plain_read_of_the_same_bytes"] = {"us_per_launch": reads[wgs] * 1e6, "workgroups": wgs, "bytes": d.cb,
                                           "gbps": d.cb / reads[wgs] / 1e9,
                                           "kernel": "t3_test_hbm_read over the headline's rotating weight copies"}

    if "sweep" in sections:
        out["sweep"] = []
        for k in (3, 4, 5):
            dk = d if 16 * k == n_head else Dense(torch, api, IN_F, OUT_F, 16 * k, MCG_CB, 32, torch.float16, seed=1000 + k)
            for rows in (1, 4, 16, 32):
                out["sweep"].append(dense_cell(dk, rows, sub_steps, 10, todo, f"sweep K{k} rows {rows}", gemv_alone=True))
            if dk is not d:
                del dk
                torch.cuda.empty_cache()

    if "forms" in sections:
        # the GEMV's codebook forms: MCG's f16 weight (served) against its pair form fed unrounded (t3_configure's
        # mcg_pair: this library's opt-in), MUL1's deferred map (served, the reference's own form) against the weight
        # decoded one by one (mul1_defer = 0)
        out["codebook_forms"] = []
        d.bind(1)
        dm = Dense(torch, api, IN_F, OUT_F, n_head, MUL1_CB, 1, torch.float16, seed=77)
        dm.bind(1)
        for label, obj, cfg in (("MCG, the f16 weight (served)", d, {}), ("MCG, the hashed pair unrounded (mcg_pair = 1)", d, {"mcg_pair": 1}),
                                ("MUL1, the deferred map (served)", dm, {}), ("MUL1, the f16 weight", dm, {"mul1_defer": 0})):
            api.configure(**cfg)
            try:
                t = obj.time(sub_steps, 10)
            finally:
                api.configure()
            out["codebook_forms"].append({"form": label, "us_per_call": t * 1e6, "gbps": obj.cb / t / 1e9,
                                          "frac_of_hbm": obj.cb / t / HBM_PEAK})
        del dm
        torch.cuda.empty_cache()

    if "rates" in sections:
        # a fractional narrow rate (2.5 bits a weight) and a wide one (5.375: the two-register reader)
        out["rates"] = []
        for n in (40, 86):
            dn = Dense(torch, api, IN_F, OUT_F, n, MCG_CB, 1, torch.float16, seed=500 + n)
            out["rates"].append(dense_cell(dn, 1, sub_steps, 10, todo, f"rate n {n} rows 1", gemv_alone=True))
            del dn
            torch.cuda.empty_cache()
    del d
    torch.cuda.empty_cache()

    if "streaming" in sections:
        # One row over a matrix too large for a launch's fixed costs to show: 4096 -> 151936 at K = 3, 4, 5 (233, 311 and
        # 389 MB of codes, two rotating copies: every call from HBM). The GEMV launch timed alone is the kernel's steady
        # state, what the 70 % target is about; the call adds its prepare launch and the arriving finish.
        out["streaming"] = []
        for k in (3, 4, 5):
            ds = Dense(torch, api, 4096, 151936, 16 * k, MCG_CB, 1, torch.float16, seed=2000 + k, copies=2)
            cell = dense_cell(ds, 1, 24, 4, todo, f"streaming 4096 -> 151936 K{k} rows 1", gemv_alone=True)
            cell["roofline"] = {"bound": "hbm", "kernel": "t3::dense_gemv<kMcg, narrow, 1 row block, 8 tiles> (the GEMV launch alone)",
                                "us_per_launch": cell.get("gemv_us"), "algorithmic_bytes_per_launch": ds.cb,
                                "achieved": cell.get("gemv_gbps"), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                                "frac": cell.get("gemv_frac_of_hbm"),
                                "frac_of_measured_read_peak": cell.get("gemv_frac_of_measured_read_peak")}
            out["streaming"].append(cell)
            del ds
            torch.cuda.empty_cache()

    if "peak" in sections or "moe_prefill" in sections or "dense_prefill" in sections or "lm_head" in sections:
        out["measured_dense_f16_peak"] = measured_f16_peak(torch)
    peak_meas = out.get("measured_dense_f16_peak", {}).get("tflops")
    both = lambda flops, t: {"tflops": flops / t / 1e12, "frac_of_f16_mfma_peak": flops / t / MFMA_F16_PEAK,
                             "frac_of_measured_f16_peak": (flops / t / 1e12 / peak_meas) if peak_meas else None}

    if "lm_head" in sections:
        in_f, out_f, n = 4096, 151936, 96
        dl = Dense(torch, api, in_f, out_f, n, MCG_CB, 256, torch.bfloat16, seed=6, copies=2, outliers=False)
        one = dense_cell(dl, 1, 40, 4, todo, "lm_head K6 rows 1", gemv_alone=True)
        one["roofline"] = {"bound": "hbm", "kernel": "t3::dense_gemv<kMcg, two-word wide reader, 1 row block, 4 tiles>", "us_per_launch": one.get("gemv_us"),
                           "algorithmic_bytes_per_launch": dl.cb, "achieved": one.get("gemv_gbps"), "peak": HBM_PEAK / 1e9,
                           "unit": "GB/s", "frac": one.get("gemv_frac_of_hbm"),
                           "frac_of_measured_read_peak": one.get("gemv_frac_of_measured_read_peak")}
        many = dense_cell(dl, 256, 10, 2, todo, "lm_head K6 rows 256")
        flops = 2 * 256 * in_f * out_f
        t = many["us_per_call"] * 1e-6
        many.update(both(flops, t))
        many["roofline"] = {"bound": "mfma", "kernel": "t3::pf_gemm (the trellis GEMM; whole call)", "us_per_call": many["us_per_call"],
                            "flops": flops, "achieved": flops / t / 1e12, "peak": MFMA_F16_PEAK / 1e12, "unit": "TFLOP/s",
                            "frac": flops / t / MFMA_F16_PEAK, "frac_of_hbm_on_code_bytes": dl.cb / t / HBM_PEAK}
        out["lm_head"] = [one, many]
        del dl
        torch.cuda.empty_cache()

    if "moe_decode" in sections:
        out["moe_decode"] = []
        for tokens in (1, 8):
            m = Moe(torch, api, 512, 2048, 512, 3, 3, 10, tokens, 7, shared=True, sets=24, seed=5)
            todo.append(m.sample(f"moe_decode {tokens} token(s), token 0", 0, BF16_MOE_BAR))
            steps = max(50, args.steps // 2)
            t = m.time(steps, 10)
            t_gu, t_dn = m.time(steps, 10, stages=1), m.time(steps, 10, stages=2)
            bytes_call = m.distinct * m.per_expert
            gu_bytes = bytes_call * (2 * code_bytes(2048, 512, 48)) / m.per_expert
            out["moe_decode"].append({
                "tokens": tokens, "us_per_call": t * 1e6, "code_bytes": bytes_call, "distinct_experts": m.distinct,
                "gbps": bytes_call / t / 1e9, "frac_of_hbm": bytes_call / t / HBM_PEAK,
                "plan": {key: m.plan[key] for key in ("path", "launches", "row_slots", "k_slices_gu", "k_slices_dn")},
                # the launch that reads two thirds of the code bytes; up to two rows the mid stage runs inside the down
                # launch, above that the gate|up launch's last arriver at a block runs it
                "roofline": {"bound": "hbm",
                             "kernel": "t3::moe_gemv<gate|up, prepare in LDS" + (">" if tokens <= 4 else ", arriving mid>"),
                             "us_per_launch": t_gu * 1e6, "algorithmic_bytes_per_launch": gu_bytes,
                             "achieved": gu_bytes / t_gu / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                             "frac": gu_bytes / t_gu / HBM_PEAK},
                "launches": {("gate_up_us" if tokens <= 4 else "gate_up_mid_us"): t_gu * 1e6,
                             ("mid_down_combine_us" if tokens <= 4 else "down_combine_us"): t_dn * 1e6}})
            del m
            torch.cuda.empty_cache()

    if "moe_prefill" in sections:
        m = Moe(torch, api, 256, 7168, 2048, 2, 3, 8, 2048, 7, shared=False, sets=1, seed=9)
        todo.append(m.sample("moe_prefill token 0", 0, BF16_MOE_BAR))
        t = m.time(5, 2)
        names = ("route", "prepare", "gemm_gate_up", "mid", "gemm_down", "combine")
        stage_t = {nm: m.time(5, 1, stages=1 << i) for i, nm in enumerate(names)}
        gu_flops = m.flops * 2 / 3
        t_gu = stage_t["gemm_gate_up"]
        code = 256 * m.per_expert
        out["moe_prefill"] = {
            "workload": "2048 tokens, E256 top-8, 7168/2048, gate|up K2, down K3, bf16, clamp 7", "ms_per_call": t * 1e3,
            "flops": m.flops, **both(m.flops, t), "code_gbps": code / t / 1e9, "frac_of_hbm_on_code_bytes": code / t / HBM_PEAK,
            "plan": {key: m.plan[key] for key in ("path", "launches", "row_slots", "item_rows", "max_items")},
            "roofline": {"bound": "mfma", "kernel": "t3::pf_gemm<kMcg, narrow, 8 row blocks, 6 live> (gate|up, the call's longest "
                                                    "launch)",
                         "us_per_launch": t_gu * 1e6, "flops_per_launch": gu_flops, "achieved": gu_flops / t_gu / 1e12,
                         "peak": MFMA_F16_PEAK / 1e12, "unit": "TFLOP/s", "frac": gu_flops / t_gu / MFMA_F16_PEAK,
                         "frac_of_measured_f16_peak": (gu_flops / t_gu / 1e12 / peak_meas) if peak_meas else None},
            "stages_us": {nm: v * 1e6 for nm, v in stage_t.items()}}
        # the same call over the same codes read as MUL1 (the deferred map: h = 1024 + t as the weight, three vector
        # operations a weight in the GEMM's decode instead of MCG's four)
        m.dec = api.Decode(MUL1_CB, 16)
        todo.append(m.sample("moe_prefill MUL1 token 0", 0, BF16_MOE_BAR))
        t1 = m.time(5, 2)
        out["moe_prefill"]["mul1_codebook"] = {"ms_per_call": t1 * 1e3, **both(m.flops, t1)}
        del m
        torch.cuda.empty_cache()

    if "dense_prefill" in sections:
        rows, in_f, out_f, n = 4096, 4096, 14336, 64
        dp = Dense(torch, api, in_f, out_f, n, MCG_CB, rows, torch.bfloat16, seed=3, copies=1, outliers=False)
        cell = dense_cell(dp, rows, 5, 2, todo, "dense_prefill 4096 rows")
        flops = 2 * rows * in_f * out_f
        t = cell["us_per_call"] * 1e-6
        tr, suh, svh, x = dp.trellis[0], dp.suh, dp.svh, dp.xr
        out["dense_prefill"] = {"workload": "4096 rows x (4096 -> 14336) K4 bf16", "ms_per_call": t * 1e3, "flops": flops,
                                **both(flops, t), "plan": cell["plan"],
                                "roofline": {"bound": "mfma", "kernel": "the call (W_hat decode, prepare, f16 GEMM, finish)",
                                             "us_per_call": t * 1e6, "flops": flops, "achieved": flops / t / 1e12,
                                             "peak": MFMA_F16_PEAK / 1e12, "unit": "TFLOP/s", "frac": flops / t / MFMA_F16_PEAK,
                                             "frac_of_measured_f16_peak": (flops / t / 1e12 / peak_meas) if peak_meas else None}}
        # the same projection with its un-rotated weight resident (made once a weight): one plain GEMM a call
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        w_std, bad = api.unrot_weight(tr, suh, svh, dp.dec, torch.bfloat16)
        e1.record()
        torch.cuda.synchronize()
        once = e0.elapsed_time(e1)
        t = eager_time(torch, lambda: api.linear_unrot(x, w_std))
        out["dense_prefill_unrot"] = {"workload": "the same, W_std bf16 resident (117 MB)", "ms_per_call": t * 1e3,
                                      **both(flops, t), "ms_to_make_w_std_once": once, "nonfinite": bad}
        # and with the W_hat of the trellis kept (decoded once a weight): the call above without its decode
        w_hat = api.dequant(tr, dp.dec)
        t = eager_time(torch, lambda: api.linear_resident(x, w_hat, suh, svh))
        out["dense_prefill_resident"] = {"workload": "the same, W_hat f16 resident (117 MB)", "ms_per_call": t * 1e3,
                                         **both(flops, t)}
        del w_hat, w_std

        if "dense_rows" in sections:
            # few-row dense calls of the same shape: the served partition (K parts follow the rows) against the rows-alone
            # configuration (one K part whatever the rows: a row's bytes then ignore the call's other rows)
            out["dense_rows"] = []
            for r in (64, 256, 1024):
                xr = dp.x[:r]
                served = eager_time(torch, lambda: api.linear(xr, tr, suh, svh, dp.dec))
                api.configure(dense_rows_alone=1)
                try:
                    alone = eager_time(torch, lambda: api.linear(xr, tr, suh, svh, dp.dec))
                finally:
                    api.configure()
                out["dense_rows"].append({"rows": r, "served_us": served * 1e6, "rows_alone_us": alone * 1e6,
                                          "served_plan": {k: v for k, v in api.linear_plan(xr, tr, dp.dec).items()
                                                          if k in ("path", "k_slices", "workgroups")}})
        del dp
        torch.cuda.empty_cache()

    if "shapes" in sections:
        out["shapes"] = shapes_section(torch, api)

    if "reference" in sections:
        out["reference_workload"] = reference_section(torch, api, todo)

    if not args.no_cpu:
        out["cpu_baseline"], checks = cpu_leg(n_head, seed=11, todo=todo)
        out["parity_checks"] = {"ok": all(c["ok"] for c in checks), "cells": len(checks),
                                "worst": max(checks, key=lambda c: c["err_over_rms"] / c["bar"]) if checks else None,
                                "failed": [c for c in checks if not c["ok"]]}
    print(json.dumps(out))
    if not args.no_cpu and not out["parity_checks"]["ok"]:
        print("bench.py: a sampled output missed the reference's bar: " + json.dumps(out["parity_checks"]["failed"]),
              file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
