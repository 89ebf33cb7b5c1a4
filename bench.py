#!/usr/bin/env python3
"""Benchmark of the hip kernel backend on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|matmul|gpt|mlp|gpt-large|components] [--no-extra]

Prints ONE JSON line.  A "step" is one pass of the workload over one batch of synthetic,
seeded input that is already resident in HBM when the timed region starts.

  c2      (default)  element-wise / broadcast / reduce suite on fp32 N(0,1) tensors of
                     16384 x 8192: add sub mul div with a same-shape, (R,1), (1,C) and scalar
                     right operand; exp, relu on N(0,1); log, sqrt on |x|+1e-3; sum and max
                     over axis 0, axis 1 and everything.  value = algorithmic GB/s of the suite.
  matmul             4096^3 fp32 GEMM, entries N(0, 1/sqrt(K)).  value = TFLOP/s.
  gpt                char-GPT (vocab 65, block 128, 6 layers, 4 heads, n_embd 128, batch 16):
                     forward + backward + Adam step.  value = tokens/s.
  mlp                784-64-10 MLP, batch 128: forward + backward + SGD step.  value = samples/s.
  gpt-large          scaled GPT (vocab 50304, block 1024, 12 layers, 12 heads, n_embd 768, batch 8),
                     Zipf(1.1) ids: forward + backward + Adam step.  value = tokens/s.

  components         the kernel classes c2 does not reach, at sizes beyond the caches: transposes, head
                     permutes, argmax, selects, and the scaled GPT's embedding gather / scatter-add,
                     softmax and cross-entropy shapes.  value = algorithmic GB/s over all of them;
                     `roofline` names the one that takes longest.

Unless --no-extra is given, the default run also reports the matmul sweep, the GPT step and
the 4096^2 / 1024^2 suites under "extra", so one run carries every headline figure.

`roofline` describes the dominant kernel of the workload (same-shape add for c2, the GEMM for
matmul/gpt): algorithmic bytes or flops per launch divided by the average launch duration,
measured with HIP events on the stream the kernels run on, inside the timed region.
`cpu_baseline` is the single-threaded C restatement of the reference's CPU kernels (oracle/),
timed on this machine's host cores on a bounded sample of the same workload.
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

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_FP32_PEAK_TFLOPS = 157.3  # dense fp32 MFMA
# HBM bytes per launch of the same-shape add at 16384x8192, from two rocprofv3 --pmc runs
# (FETCH_SIZE x 2.0 and WRITE_SIZE x 1.0, the factors a plain copy kernel of known size gives):
# 1024.0 MiB read + 512.0 MiB written = the algorithmic 12 B per element.
C2_ADD_TRAFFIC_BYTES = 1610612736


def _imports():
    from dlgrad_amd import Tensor, nn
    from dlgrad_amd.buffer import Buffer
    from dlgrad_amd.device import Device
    from dlgrad_amd.runtime import hip
    return Tensor, nn, Buffer, Device, hip


class EventTimer:
    """Per-name accumulation of kernel time from HIP events on the library's stream."""

    def __init__(self, lib) -> None:
        self.lib, self.pending, self.pool = lib, [], []

    def _ev(self) -> int:
        return self.pool.pop() if self.pool else self.lib.event_create()

    def run(self, name: str, fn):
        e0, e1 = self._ev(), self._ev()
        self.lib.event_record(e0)
        out = fn()
        self.lib.event_record(e1)
        self.pending.append((name, e0, e1))
        return out

    def collect(self) -> dict:
        """name -> list of ms; call after a sync."""
        res: dict = {}
        for name, e0, e1 in self.pending:
            res.setdefault(name, []).append(self.lib.event_elapsed_ms(e0, e1))
            self.pool += [e0, e1]
        self.pending = []
        return res


# ---------------------------------------------------------------------------------------------
# c2: element-wise / broadcast / reduce suite
# ---------------------------------------------------------------------------------------------
def c2_ops(R: int, C: int):
    """(name, callable on a dict of operands, algorithmic bytes) for every op of the suite.
    Bytes per element: 12 same-shape binary, 8 binary with a broadcast/scalar operand
    (+ the small operand), 8 unary, 4 per element read + 4 per output for reductions."""
    n = R * C
    ops = []
    for name, f in (("add", lambda a, b: a + b), ("sub", lambda a, b: a - b),
                    ("mul", lambda a, b: a * b), ("div", lambda a, b: a / b)):
        ops.append((f"{name}_same", (lambda d, f=f: f(d["a"], d["b"])), 12 * n))
        ops.append((f"{name}_rowvec", (lambda d, f=f: f(d["a"], d["col"])), 8 * n + 4 * R))   # (R,1)
        ops.append((f"{name}_colvec", (lambda d, f=f: f(d["a"], d["row"])), 8 * n + 4 * C))   # (1,C)
        ops.append((f"{name}_scalar", (lambda d, f=f: f(d["a"], 1.5)), 8 * n))
    ops.append(("exp", lambda d: d["a"].exp(), 8 * n))
    ops.append(("relu", lambda d: d["a"].relu(), 8 * n))
    ops.append(("log", lambda d: d["pos"].log(), 8 * n))
    ops.append(("sqrt", lambda d: d["pos"].sqrt(), 8 * n))
    for red in ("sum", "max"):
        ops.append((f"{red}_axis0", (lambda d, r=red: getattr(d["a"], r)(0)), 4 * n + 4 * C))
        ops.append((f"{red}_axis1", (lambda d, r=red: getattr(d["a"], r)(1)), 4 * n + 4 * R))
        ops.append((f"{red}_all", (lambda d, r=red: getattr(d["a"], r)()), 4 * n + 4))
    return ops


def c2_inputs(R: int, C: int, seed: int = 2):
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((R, C), dtype=np.float32)
    b = rng.standard_normal((R, C), dtype=np.float32)
    return {"a": a, "b": b, "pos": np.abs(a) + np.float32(1e-3),
            "col": rng.standard_normal((R, 1), dtype=np.float32) + np.float32(3),
            "row": rng.standard_normal((1, C), dtype=np.float32) + np.float32(3)}


def run_c2(R: int, C: int, steps: int, warmup: int, events_in_timed_region: bool = True) -> dict:
    """events_in_timed_region: per-op durations come from HIP event pairs recorded around every op inside the
    timed steps.  For tensors small enough that a step is bound by issuing its launches, two event records per op
    are a sizeable part of that work; there the steps are timed bare and run once more with the events."""
    _, _, Buffer, Device, hip = _imports()
    lib = hip.lib()
    host = c2_inputs(R, C)
    d = {k: Buffer.from_numpy(v, Device.HIP) for k, v in host.items()}
    del host
    ops = c2_ops(R, C)
    timer = EventTimer(lib)
    for _ in range(warmup):
        for _, f, _ in ops:
            f(d)
    lib.sync()
    n0 = hip.launch_count
    t0 = time.perf_counter()
    for _ in range(steps):                                   # the timed region
        for name, f, _ in ops:
            if events_in_timed_region:
                timer.run(name, lambda f=f: f(d))
            else:
                f(d)
    lib.sync()
    wall = time.perf_counter() - t0
    launches = (hip.launch_count - n0) / steps
    if not events_in_timed_region:                           # the same steps again with an event pair around every op
        for _ in range(steps):
            for name, f, _ in ops:
                timer.run(name, lambda f=f: f(d))
        lib.sync()
    per = timer.collect()
    total_bytes = sum(b for _, _, b in ops)
    per_op = {name: {"ms": float(np.mean(per[name])), "GBps": b / np.mean(per[name]) / 1e6,
                     "frac_hbm": b / np.mean(per[name]) / 1e6 / HBM_PEAK_GBS}
              for name, _, b in ops}
    return {"ms_per_step": wall / steps * 1e3, "GBps": total_bytes * steps / wall / 1e9,
            "bytes_per_step": total_bytes, "per_op": per_op, "n_ops": len(ops), "launches_per_step": launches}


def run_c2_graph(R: int, C: int, steps: int) -> dict:
    """The same 26-op suite recorded once as a HIP graph and replayed: what the kernels do at a size where issuing them
    from Python one by one is what takes the time."""
    _, _, Buffer, Device, hip = _imports()
    lib = hip.lib()
    d = {k: Buffer.from_numpy(v, Device.HIP) for k, v in c2_inputs(R, C).items()}
    ops = c2_ops(R, C)

    def suite():
        for _, f, _ in ops:
            f(d)                                              # (each result goes back to the graph's arena at once)
    g = hip.Graph()
    with g.arena():
        suite()
    with g.capture():
        suite()
    for _ in range(5):
        g.replay()
    lib.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        g.replay()
    lib.sync()
    wall = time.perf_counter() - t0
    total_bytes = sum(b for _, _, b in ops)
    res = {"GBps": round(total_bytes * steps / wall / 1e9, 1), "ms_per_step": round(wall / steps * 1e3, 4), "graph_nodes": g.nodes,
           "us_per_node": round(wall / steps * 1e6 / max(g.nodes, 1), 2)}
    g.close()
    return res


def cpu_c2(R: int, C: int, reps: int = 2) -> dict:
    """The same suite on the C restatement of the reference's kernels, one thread."""
    from oracle import cref
    host = c2_inputs(R, C)
    n = R * C
    work = []
    for op in ("add", "sub", "mul", "div"):
        work += [(lambda op=op: cref.binary(op, host["a"], host["b"]), 12 * n),
                 (lambda op=op: cref.binary(op, host["a"], host["col"]), 8 * n + 4 * R),
                 (lambda op=op: cref.binary(op, host["a"], host["row"]), 8 * n + 4 * C),
                 (lambda op=op: cref.binary(op, host["a"], np.float32(1.5)), 8 * n)]
    work += [(lambda: cref.unary("exp", host["a"]), 8 * n),
             (lambda: cref.where(host["a"], host["a"], np.float32(0)), 8 * n),
             (lambda: cref.unary("log", host["pos"]), 8 * n), (lambda: cref.unary("sqrt", host["pos"]), 8 * n)]
    for red in ("sum", "max"):
        work += [(lambda r=red: cref.reduce(r, host["a"], 0), 4 * n + 4 * C),
                 (lambda r=red: cref.reduce(r, host["a"], 1), 4 * n + 4 * R),
                 (lambda r=red: cref.reduce(r, host["a"]), 4 * n + 4)]
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        for f, _ in work:
            f()
        best = min(best, time.perf_counter() - t0)
    return {"value": sum(b for _, b in work) / best / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"the same {len(work)}-op suite at {R}x{C}, single thread, min of {reps} passes "
                      f"({best:.2f} s per pass); host has {os.cpu_count()} logical cores"}


# ---------------------------------------------------------------------------------------------
# matmul
# ---------------------------------------------------------------------------------------------
def run_matmul(M: int, N: int, K: int, steps: int, warmup: int, seed: int = 3) -> dict:
    _, _, Buffer, Device, hip = _imports()
    lib = hip.lib()
    rng = np.random.default_rng(seed)
    a = Buffer.from_numpy(rng.standard_normal((M, K), dtype=np.float32) * np.float32(K ** -0.5), Device.HIP)
    b = Buffer.from_numpy(rng.standard_normal((K, N), dtype=np.float32) * np.float32(K ** -0.5), Device.HIP)
    for _ in range(warmup):
        a @ b
    lib.sync()
    # The sweep may follow a host-only phase (the CPU baseline): at least 50 ms of the product itself, untimed, so that
    # the device clocks are up (4096^3 measured 112 TFLOP/s right after the CPU baseline, 127 with this warm-up).
    t_warm = time.perf_counter()
    while time.perf_counter() - t_warm < 0.05:
        for _ in range(4):
            a @ b
        lib.sync()
    timer = EventTimer(lib)
    t0 = time.perf_counter()
    for _ in range(steps):
        timer.run("matmul", lambda: a @ b)
    lib.sync()
    wall = time.perf_counter() - t0
    ms = float(np.mean(timer.collect()["matmul"]))
    flops = 2.0 * M * N * K
    res = {"ms_per_step": wall / steps * 1e3, "kernel_ms": ms, "TFLOPs": flops / ms / 1e9,
           "TFLOPs_wall": flops * steps / wall / 1e12, "flops": flops,
           "bytes": 4.0 * (M * K + K * N + M * N)}
    if ms < 0.05:
        # A launch this short is over before the next one arrives from Python, and an event pair around it adds the
        # front end's own latency: the same launch 48 times in a recorded graph, replayed, is what the kernel itself takes.
        n = 48

        def many():
            for _ in range(n):
                a @ b
        g = hip.Graph()
        with g.arena():
            many()
        with g.capture():
            many()
        for _ in range(5):
            g.replay()
        lib.sync()
        t0 = time.perf_counter()
        reps = 50
        for _ in range(reps):
            g.replay()
        lib.sync()
        in_graph = (time.perf_counter() - t0) / reps / n * 1e3
        g.close()
        res["kernel_ms_in_graph"], res["TFLOPs_in_graph"] = in_graph, flops / in_graph / 1e9
    return res


def run_matmul_transposed(n: int) -> dict:
    """The backward shapes A^T.G and G.B^T, two ways: as the reference issues them (a
    materialised transpose -- a permute kernel -- followed by a plain GEMM, both launches
    timed together) and with the transposed operand read in place by the TN / NT kernels."""
    _, _, Buffer, Device, hip = _imports()
    lib = hip.lib()
    rng = np.random.default_rng(4)
    a = Buffer.from_numpy(rng.standard_normal((n, n), dtype=np.float32) * np.float32(n ** -0.5), Device.HIP)
    g = Buffer.from_numpy(rng.standard_normal((n, n), dtype=np.float32) * np.float32(n ** -0.5), Device.HIP)
    out = {}
    for name, f, key in ((f"{n}_TN_At.G", lambda: a.T @ g, "ms_permute_plus_gemm"),
                         (f"{n}_NT_G.Bt", lambda: g @ a.T, "ms_permute_plus_gemm"),
                         (f"{n}_TN_At.G_in_place", lambda: a.matmul_tn(g), "kernel_ms"),
                         (f"{n}_NT_G.Bt_in_place", lambda: g.matmul_nt(a), "kernel_ms")):
        f()
        lib.sync()
        t_warm = time.perf_counter()                      # the clock warm-up of run_matmul: 50 ms of the product itself, untimed
        while time.perf_counter() - t_warm < 0.05:
            for _ in range(4):
                f()
            lib.sync()
        timer = EventTimer(lib)
        for _ in range(10):
            timer.run("mm", f)
        lib.sync()
        ms = float(np.mean(timer.collect()["mm"]))
        out[name] = {"TFLOPs": round(2.0 * n ** 3 / ms / 1e9, 2), key: round(ms, 4)}
    return out


def cpu_matmul(n: int = 512) -> dict:
    from oracle import cref
    rng = np.random.default_rng(3)
    a = rng.standard_normal((n, n), dtype=np.float32)
    b = rng.standard_normal((n, n), dtype=np.float32)
    best = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        cref.matmul(a, b)
        best = min(best, time.perf_counter() - t0)
    return {"value": 2.0 * n ** 3 / best / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"{n}^3 fp32 matmul_2d (i-k-j loops), single thread, min of 3 ({best * 1e3:.1f} ms); "
                      f"host has {os.cpu_count()} logical cores"}


# ---------------------------------------------------------------------------------------------
# C5 components at the scaled-GPT shapes
# ---------------------------------------------------------------------------------------------
def run_c5(steps: int, warmup: int) -> dict:
    """Embedding gather / scatter-add on a 50304x768 table with 8192 Zipf(1.1) ids, fused softmax
    on (98304, 1024), fused cross-entropy forward and backward on (8192, 50304).  GB/s are
    algorithmic: gather 4n + 8nW; scatter 4VW + 4nW + 4n; softmax and CE bwd 8 B/elt; CE fwd 4 B/elt + 8 B/row; the scaled,
    causally masked attention softmax 6 B/elt forward and 8 B/elt backward (the masked half of each input
    row is not read)."""
    Tensor, _, Buffer, Device, hip = _imports()
    lib = hip.lib()
    rng = np.random.default_rng(5)
    V, W, n = 50304, 768, 8192
    ids = np.minimum(rng.zipf(1.1, n) - 1, V - 1).astype(np.float32)
    table = Buffer.from_numpy(rng.standard_normal((V, W), dtype=np.float32), Device.HIP)
    idx = Buffer.from_numpy(ids.reshape(8, 1024), Device.HIP)
    g = Buffer.from_numpy(rng.standard_normal((8, 1024, W), dtype=np.float32), Device.HIP)
    att = Buffer.from_numpy(rng.standard_normal((8 * 12 * 1024, 1024), dtype=np.float32), Device.HIP)
    logits = Buffer.from_numpy(rng.standard_normal((n, V), dtype=np.float32), Device.HIP)
    tgt = Buffer.from_numpy(ids.reshape(n, 1), Device.HIP)
    one = Buffer.from_scalar(1.0)
    row_max, row_logsum, _ = logits.ce_stats(tgt)
    att4 = att.reshape((8, 12, 1024, 1024))
    from dlgrad_amd.ops import causal_mask
    causal = causal_mask(1024, Device.HIP)                     # the mask the attention layers use (built once per size, kept)
    probs = att4.masked_softmax(causal, 0.125)
    work = [("embedding_gather", lambda: table.embedding(idx), 4 * n + 8 * n * W),
            ("embedding_scatter_add", lambda: table.embedding(idx, backward=True, upstream_grad=g),
             4 * V * W + 4 * n * W + 4 * n),
            ("softmax_98304x1024", lambda: att.softmax(1), 8 * att.numel),
            # items above the diagonal are exact zeros and are not read: half of each input row moves; the mask is the cached causal
            # mask, whose bits the kernel computes from the indices instead of reading them (6 and 8 B per element, not 8 and 12)
            ("scaled_causal_softmax_(8,12,1024,1024)", lambda: att4.masked_softmax(causal, 0.125), 6 * att.numel),
            ("scaled_causal_softmax_backward", lambda: probs.masked_softmax_bwd(att4, causal, 0.125), 8 * att.numel),
            # forward: one read of the logits, (max, log-sum) and the picked log-prob per row; backward: logits in, gradient out
            ("ce_forward_8192x50304", lambda: logits.ce_stats(tgt), 4 * n * V + 8 * n),
            ("ce_backward_8192x50304", lambda: logits.ce_grad_logits(row_max, row_logsum, tgt, one, float(n)), 8 * n * V)]
    timer = EventTimer(lib)
    for _ in range(warmup):
        for _, f, _ in work:
            f()
    for _ in range(steps):
        for name, f, _ in work:
            timer.run(name, f)
    lib.sync()
    per = timer.collect()
    return {name: {"ms": round(float(np.mean(per[name])), 4),
                   "GBps": round(b / float(np.mean(per[name])) / 1e6, 1),
                   "frac_hbm": round(b / float(np.mean(per[name])) / 1e6 / HBM_PEAK_GBS, 3)}
            for name, _, b in work}


def run_attention(steps: int, warmup: int) -> dict:
    """Causal self-attention of the scaled GPT, (8, 12, 1024, 64) read from one interleaved (8, 1024, 3 * 768) projection:
    forward, and backward (row sums, the key-side launch that writes dS, and the product dQ = dS K).  Matrix-core bound:
    flops are those of the causal half -- 2 products forward, 5 backward (S is recomputed) of T^2 / 2 * d * 2 each per
    head -- and the figure is against the fp32 MFMA peak.  DLGRAD_HIP_ATTENTION_FLASH=0 times the chain over stored
    T x T tensors instead."""
    _, _, Buffer, Device, hip = _imports()
    lib = hip.lib()
    rng = np.random.default_rng(9)
    B, T, h, d = 8, 1024, 12, 64
    C = h * d
    qkv = Buffer.from_numpy(rng.standard_normal((B, T, 3 * C), dtype=np.float32), Device.HIP)
    g = Buffer.from_numpy(rng.standard_normal((B, T, C), dtype=np.float32), Device.HIP)
    scale = d ** -0.5
    y, kept = qkv.causal_attention_qkv(h, scale)
    per_product = B * h * T * T * d                                   # 2 * (T^2 / 2) * d flops per head
    work = [("causal_attention_forward_(8,12,1024,64)", lambda: qkv.causal_attention_qkv(h, scale), 2 * per_product),
            ("causal_attention_backward_(8,12,1024,64)", lambda: qkv.causal_attention_qkv_bwd(kept, g, h, scale, y), 5 * per_product)]
    timer = EventTimer(lib)
    for _ in range(warmup):
        for _, f, _ in work:
            f()
    for _ in range(steps):
        for name, f, _ in work:
            timer.run(name, f)
    lib.sync()
    per = timer.collect()
    return {name: {"ms": round(float(np.mean(per[name])), 4), "TFLOPs": round(fl / float(np.mean(per[name])) / 1e9, 1),
                   "frac_mfma_fp32": round(fl / float(np.mean(per[name])) / 1e9 / MFMA_FP32_PEAK_TFLOPS, 3),
                   "kept_for_backward_MiB": round(kept.nbytes / 2 ** 20, 1)}
            for name, _, fl in work}


def run_layout_and_select(steps: int, warmup: int) -> dict:
    """The kernel classes the C2 suite does not touch, at sizes beyond the caches: transposes
    and head permutes (8 B/elt), argmax (4 B/elt + 4 B/output), comparisons, clamp, pow,
    masked_fill with the causal mask broadcast over (8, 12, 1024, 1024) (8 B/elt), where with
    three tensor operands (16 B/elt)."""
    _, _, Buffer, Device, hip = _imports()
    lib = hip.lib()
    rng = np.random.default_rng(6)
    sq = Buffer.from_numpy(rng.standard_normal((8192, 8192), dtype=np.float32), Device.HIP)
    heads = Buffer.from_numpy(rng.standard_normal((64, 1024, 12, 64), dtype=np.float32), Device.HIP)
    att = Buffer.from_numpy(rng.standard_normal((8, 12, 1024, 1024), dtype=np.float32), Device.HIP)
    mask = Buffer.from_numpy(np.triu(np.ones((1024, 1024), np.float32), 1), Device.HIP)
    logits = Buffer.from_numpy(rng.standard_normal((8192, 50304), dtype=np.float32), Device.HIP)
    tall = Buffer.from_numpy(rng.standard_normal((1000000, 10), dtype=np.float32), Device.HIP)
    n2, nh, na = sq.numel, heads.numel, att.numel
    cond, other = Buffer(logits.ptr, sq.shape, Device.HIP), Buffer(logits.ptr + n2, sq.shape, Device.HIP)   # views into logits
    work = [("transpose_8192x8192", lambda: sq.transpose(0, 1), 8 * n2),
            ("permute_heads_(64,1024,12,64)->(64,12,1024,64)", lambda: heads.permute((0, 2, 1, 3)), 8 * nh),
            ("transpose_last_two_(64,12,1024,64)", lambda: heads.reshape((64, 12, 1024, 64)).permute((0, 1, 3, 2)), 8 * nh),
            ("argmax_rows_8192x50304", lambda: logits.argmax(1), 4 * logits.numel + 4 * 8192),
            ("argmax_rows_1000000x10", lambda: tall.argmax(1), 4 * tall.numel + 4 * 1000000),
            ("argmax_cols_8192x8192", lambda: sq.argmax(0), 4 * n2 + 4 * 8192),
            ("gt_scalar_(8,12,1024,1024)", lambda: att > 0.0, 8 * na),
            ("clamp_(8,12,1024,1024)", lambda: att.clamp(-0.5, 0.5), 8 * na),
            ("pow3_(8,12,1024,1024)", lambda: att ** 3, 8 * na),
            ("masked_fill_causal_(8,12,1024,1024)", lambda: Buffer.masked_fill(att, mask, float("-inf")), 8 * na + 4 * mask.numel),
            ("where_3_tensors_8192x8192", lambda: cond.where(sq, other), 16 * n2)]
    timer = EventTimer(lib)
    for _ in range(warmup):
        for _, f, _ in work:
            f()
    for _ in range(steps):
        for name, f, _ in work:
            timer.run(name, f)
    lib.sync()
    per = timer.collect()
    return {name: {"ms": round(float(np.mean(per[name])), 4),
                   "GBps": round(b / float(np.mean(per[name])) / 1e6, 1),
                   "frac_hbm": round(b / float(np.mean(per[name])) / 1e6 / HBM_PEAK_GBS, 3)}
            for name, _, b in work}


# ---------------------------------------------------------------------------------------------
# GPT / MLP steps
# ---------------------------------------------------------------------------------------------
GPT_C4 = dict(vocab_size=65, block_size=128, n_layer=6, n_head=4, n_embd=128, batch_size=16)


def make_gpt(device: str, cfg: dict, seed: int = 0):
    Tensor, nn, *_ = _imports()
    from examples import gpt as G
    c = G.GPTConfig(device=device, **cfg)
    model = G.GPT(c)
    G.init_weights_(model, seed)
    rng = np.random.default_rng(seed + 1)
    idx = Tensor(rng.integers(0, c.vocab_size, (c.batch_size, c.block_size)).astype(np.float32), device=device)
    tgt = Tensor(rng.integers(0, c.vocab_size, (c.batch_size, c.block_size)).astype(np.float32), device=device)
    params = nn.utils.get_parameters(model)
    opt = nn.optim.Adam(params, lr=c.learning_rate)

    def step():
        opt.zero_grad()
        _, loss = model(idx, tgt)
        loss.backward()
        opt.step()
        return loss
    return model, step


def run_gpt_graph(steps: int, warmup: int, cfg: dict = GPT_C4) -> dict:
    """The same training step captured once into a HIP graph and replayed: identical kernels
    and results, one submission per step instead of ~900 launches."""
    Tensor, nn, _, _, hip = _imports()
    from examples import gpt as G
    lib = hip.lib()
    c = G.GPTConfig(device="hip", **cfg)
    model = G.GPT(c)
    G.init_weights_(model, 0)
    rng = np.random.default_rng(1)
    idx = Tensor(rng.integers(0, c.vocab_size, (c.batch_size, c.block_size)).astype(np.float32), device="hip")
    tgt = Tensor(rng.integers(0, c.vocab_size, (c.batch_size, c.block_size)).astype(np.float32), device="hip")
    opt = nn.optim.Adam(nn.utils.get_parameters(model), lr=c.learning_rate, graph_safe=True)

    def step():
        opt.zero_grad()
        _, loss = model(idx, tgt)
        loss.backward()
        opt.step()
        return loss
    g = hip.Graph()
    with g.arena():
        step()
    with g.capture():
        loss = step()
    for _ in range(warmup):
        opt.advance()
        g.replay()
    lib.sync()
    e0, e1 = lib.event_create(), lib.event_create()
    t0 = time.perf_counter()
    lib.event_record(e0)
    for _ in range(steps):
        opt.advance()
        g.replay()
    lib.event_record(e1)
    lib.sync()
    wall = time.perf_counter() - t0
    tokens = cfg["batch_size"] * cfg["block_size"]
    res = {"ms_per_step": wall / steps * 1e3, "tokens_per_s": tokens * steps / wall, "graph_nodes": g.nodes,
           "gpu_ms_per_step": lib.event_elapsed_ms(e0, e1) / steps,
           "loss_per_token": float(loss.numpy()) / tokens}
    g.close()
    return res


def run_gpt(steps: int, warmup: int, cfg: dict = GPT_C4) -> dict:
    *_, hip = _imports()
    lib = hip.lib()
    _, step = make_gpt("hip", cfg)
    for _ in range(warmup):
        step()
    lib.sync()
    n0 = hip.launch_count
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = step()
    lib.sync()
    wall = time.perf_counter() - t0
    tokens = cfg["batch_size"] * cfg["block_size"]
    return {"ms_per_step": wall / steps * 1e3, "tokens_per_s": tokens * steps / wall,
            "launches_per_step": (hip.launch_count - n0) / steps, "loss_sum": float(loss.numpy()),
            "loss_per_token": float(loss.numpy()) / tokens}


GPT_C5 = dict(vocab_size=50304, block_size=1024, n_layer=12, n_head=12, n_embd=768, batch_size=8)


def run_gpt_large(steps: int = 2) -> dict:
    """Scaled GPT (C5): one inference pass and `steps` training steps with Zipf(1.1) token ids.
    There is no CPU figure beside it: the naive single-thread loops need ~7 TFLOP per step."""
    Tensor, nn, _, _, hip = _imports()
    from examples import gpt as G
    lib = hip.lib()
    c = G.GPTConfig(device="hip", **GPT_C5)
    model = G.GPT(c)
    G.init_weights_(model, 0)
    rng = np.random.default_rng(7)
    ids = np.minimum(rng.zipf(1.1, (2, c.batch_size, c.block_size)) - 1, c.vocab_size - 1).astype(np.float32)
    idx, tgt = Tensor(ids[0], device="hip"), Tensor(ids[1], device="hip")
    params = nn.utils.get_parameters(model)
    opt = nn.optim.Adam(params, lr=c.learning_rate)
    tokens = c.batch_size * c.block_size
    model(idx)                                                    # warm-up, loads kernels
    lib.sync()
    t0 = time.perf_counter()
    logits, _ = model(idx)
    lib.sync()
    t_inf = time.perf_counter() - t0
    del logits
    times, loss, first_loss = [], None, None
    for _ in range(steps + 1):
        t0 = time.perf_counter()
        opt.zero_grad()
        _, loss = model(idx, tgt)
        loss.backward()
        opt.step()
        lib.sync()
        times.append(time.perf_counter() - t0)
        if first_loss is None:
            first_loss = float(loss.numpy()) / tokens             # the loss of the seeded weights: what the float64 parity test holds
    n_params = sum(p.numel for p in params)
    in_use, cached, _ = lib.pool_stats()
    step_s = sum(times[1:]) / steps                               # the first step (kernel loading, tile timing) is warm-up
    return {"params_M": round(n_params / 1e6, 1), "inference_ms": round(t_inf * 1e3, 2),
            "inference_tokens_per_s": round(tokens / t_inf, 1),
            "train_step_ms": round(step_s * 1e3, 2), "train_tokens_per_s": round(tokens / step_s, 1),
            "train_TFLOPs_est": round(6 * (n_params - c.vocab_size * c.n_embd - c.block_size * c.n_embd) * tokens
                                      / step_s / 1e12, 2),
            "loss_per_token_first_forward": round(first_loss, 6),
            "loss_per_token": round(float(loss.numpy()) / tokens, 4),
            "attention": "streaming kernels (no T x T tensor kept)" if hip.HIP.ATTENTION_FLASH else "products and softmax over stored T x T tensors",
            "pool_GiB": round((in_use + cached) / 2 ** 30, 1)}


def run_decode(n_tokens: int = 256) -> dict:
    """Greedy decode of the char-GPT from a 1-token prompt, three ways: the reference's loop with
    full-context recompute per token (context cropped to block_size); its key/value-cache loop
    inside the window; and both regimes as fixed-shape steps captured as HIP graphs (one token
    against the cache while the window fills, the whole model over the last block_size tokens once
    it is full, as the reference does there), replayed per token with no Python between tokens."""
    *_, hip = _imports()
    from examples import gpt as G
    model = G.GPT(G.GPTConfig(device="hip", **GPT_C4))
    G.init_weights_(model, 0)
    model.generate_greedy(0, 4)
    hip.lib().sync()
    t0 = time.perf_counter()
    ids = model.generate_greedy(0, n_tokens)
    dt = time.perf_counter() - t0
    out = {"tokens": n_tokens, "full_recompute_loop": {"ms_per_token": round(dt / n_tokens * 1e3, 3),
                                                         "tokens_per_s": round(n_tokens / dt, 1)}, "first_ids": ids[:8]}
    # the reference's generate loop: key/value cache (here resident on the device) until the
    # window of 128 is full; 120 tokens stay inside the window
    model.generate_greedy_cached(0, 4, reference_positions=False)
    hip.lib().sync()
    t0 = time.perf_counter()
    cached = model.generate_greedy_cached(0, 120, reference_positions=False)
    dt = time.perf_counter() - t0
    out["kv_cached_120_tokens"] = {"ms_per_token": round(dt / 120 * 1e3, 3), "tokens_per_s": round(120 / dt, 1)}
    dec = G.StaticDecoder(model, reference_positions=False, capacity=max(n_tokens, 120) + 1)
    if not hip.COMPILE_ONLY:
        dec.capture()
    dec.generate(0, 8)
    hip.lib().sync()
    t0 = time.perf_counter()
    ids2 = dec.generate(0, 120)
    dt = time.perf_counter() - t0
    out["fixed_shape_step_hipgraph_120_tokens"] = {
        "ms_per_token": round(dt / 120 * 1e3, 3), "tokens_per_s": round(120 / dt, 1),
        "graph_nodes": dec.graph.nodes if dec.graph else 0, "same_ids_as_cached_loop": ids2 == cached}
    t0 = time.perf_counter()
    ids3 = dec.generate(0, n_tokens)
    dt = time.perf_counter() - t0
    out["ms_per_token"], out["tokens_per_s"] = round(dt / n_tokens * 1e3, 3), round(n_tokens / dt, 1)      # the headline: graphs throughout
    out["hipgraph_steps"] = {"window_graph_nodes": dec.window_graph.nodes if dec.window_graph else 0,
                             "tokens_inside_window": GPT_C4["block_size"] - 1,
                             "tokens_by_full_window_steps": n_tokens - GPT_C4["block_size"] + 1,
                             "same_ids_as_full_recompute": ids3 == ids}
    out["positions"] = ("reference_positions=False: every token at its own position, which makes the cached and the captured steps "
                        "comparable with full recompute; the library default follows helpers.STRICT_REFERENCE (the reference numbers an "
                        "incremental token one too high), timed below")
    dec.close()
    # the same captured steps with the reference's position ids (the strict default), checked against its cache loop
    strict = G.StaticDecoder(model, reference_positions=True, capacity=n_tokens + 1)
    if not hip.COMPILE_ONLY:
        strict.capture()
    strict.generate(0, 8)
    hip.lib().sync()
    t0 = time.perf_counter()
    ids4 = strict.generate(0, n_tokens)
    dt = time.perf_counter() - t0
    out["reference_positions_true"] = {"ms_per_token": round(dt / n_tokens * 1e3, 3), "tokens_per_s": round(n_tokens / dt, 1),
                                       "same_ids_as_cached_loop": ids4 == model.generate_greedy_cached(0, n_tokens, reference_positions=True)}
    strict.close()
    # sampling (temperature 0.7, as the reference's generate_endless): the draw is the last launch of each captured step
    sampler = G.StaticDecoder(model, reference_positions=False, capacity=n_tokens + 1, temperature=0.7)
    if not hip.COMPILE_ONLY:
        sampler.capture()
    u = np.random.default_rng(8).random(n_tokens + 1).astype(np.float32)
    sampler.generate(0, 8, u=u)
    hip.lib().sync()
    t0 = time.perf_counter()
    ids5 = sampler.generate(0, n_tokens, u=u)
    dt = time.perf_counter() - t0
    out["sampling_temperature_0.7"] = {"ms_per_token": round(dt / n_tokens * 1e3, 3), "tokens_per_s": round(n_tokens / dt, 1),
                                        "distinct_tokens": len(set(ids5)), "graph_nodes": sampler.graph.nodes if sampler.graph else 0}
    sampler.close()
    return out


def cpu_gpt(cfg: dict = GPT_C4) -> dict:
    import oracle.cpu_runtime  # noqa: F401
    _, step = make_gpt("cpu", cfg)
    t0 = time.perf_counter()
    step()
    dt = time.perf_counter() - t0
    tokens = cfg["batch_size"] * cfg["block_size"]
    return {"value": tokens / dt, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"one full char-GPT step (fwd+bwd+Adam, {tokens} tokens) on the C restatement, "
                      f"single thread ({dt:.2f} s); host has {os.cpu_count()} logical cores"}


def run_mlp(steps: int, warmup: int) -> dict:
    Tensor, nn, _, _, hip = _imports()
    from examples import mlp as M
    lib = hip.lib()
    model = M.MLP(device="hip")
    M.init_weights_(model, 0)
    x, y = M.synthetic_batch(1)
    xt, yt = Tensor(x, device="hip"), Tensor(y, device="hip")
    params = [model.fc1.weight, model.fc1.bias, model.fc2.weight, model.fc2.bias]
    opt = nn.optim.SGD(params, lr=1e-3)

    def step():
        opt.zero_grad()
        loss = model(xt).cross_entropy_loss(yt)
        loss.backward()
        opt.step()
    for _ in range(warmup):
        step()
    lib.sync()
    n0 = hip.launch_count
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    lib.sync()
    wall = time.perf_counter() - t0
    return {"ms_per_step": wall / steps * 1e3, "samples_per_s": 128 * steps / wall,
            "launches_per_step": (hip.launch_count - n0) / steps}


def run_mlp_graph(steps: int, warmup: int) -> dict:
    """The MLP step with in-place SGD, captured once and replayed.  The batch is staged in
    page-locked host memory and its upload is part of the graph: per step the host refills the
    staging arrays (after the previous replay has read them) and launches the graph."""
    Tensor, nn, _, _, hip = _imports()
    from examples import mlp as M
    lib = hip.lib()
    model = M.MLP(device="hip")
    M.init_weights_(model, 0)
    batches = [M.synthetic_batch(s) for s in range(8)]
    sx, sy = hip.pinned_empty((128, 784)), hip.pinned_empty((128, 1))
    sx[:], sy[:] = batches[0]
    xt, yt = Tensor(sx, device="hip"), Tensor(sy, device="hip")
    params = [model.fc1.weight, model.fc1.bias, model.fc2.weight, model.fc2.bias]
    opt = nn.optim.SGD(params, lr=1e-3, graph_safe=True)

    def step():
        xt.data.upload_(sx)
        yt.data.upload_(sy)
        opt.zero_grad()
        loss = model(xt).cross_entropy_loss(yt)
        loss.backward()
        opt.step()
    g = hip.Graph()
    with g.arena():
        step()
    with g.capture():
        step()

    def replay(k):
        lib.sync()                                   # the previous replay has consumed the staging arrays
        sx[:], sy[:] = batches[k % len(batches)]
        g.replay()
    for k in range(warmup):
        replay(k)
    lib.sync()
    t0 = time.perf_counter()
    for k in range(steps):
        replay(k)
    lib.sync()
    wall = time.perf_counter() - t0
    res = {"ms_per_step": wall / steps * 1e3, "samples_per_s": 128 * steps / wall, "graph_nodes": g.nodes}
    g.close()
    return res


def run_transfers() -> dict:
    """Host <-> device rates at the boundary (never part of `value`): 256 MiB uploaded from
    pageable memory (copy + wait, what Tensor(np_array) does), from page-locked staging memory
    (enqueued DMA), and downloaded."""
    _, _, Buffer, Device, hip = _imports()
    lib = hip.lib()
    n = 64 * 2 ** 20
    host = np.ones(n, np.float32)
    stage = hip.pinned_empty((n,))
    stage[:] = 1.0
    dst = hip.alloc(n)
    out = {}
    for name, src in (("h2d_pageable_GBps", host), ("h2d_page_locked_GBps", stage)):
        hip._upload(dst.addr, src)
        lib.sync()
        t0 = time.perf_counter()
        for _ in range(3):
            hip._upload(dst.addr, src)
        lib.sync()
        out[name] = round(3 * 4 * n / (time.perf_counter() - t0) / 1e9, 1)
    back = np.empty(n, np.float32)
    lib.d2h(back.ctypes.data, dst.addr, 4 * n)
    t0 = time.perf_counter()
    for _ in range(3):
        lib.d2h(back.ctypes.data, dst.addr, 4 * n)
    out["d2h_pageable_GBps"] = round(3 * 4 * n / (time.perf_counter() - t0) / 1e9, 1)
    return out


def step_roofline(flops: float, ms: float, note: str) -> dict:
    achieved = flops / (ms * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": achieved, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / MFMA_FP32_PEAK_TFLOPS, "traffic": None, "note": note}


# ---------------------------------------------------------------------------------------------
def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c2", choices=["c2", "matmul", "gpt", "mlp", "gpt-large", "components"])
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch a plain 16384x8192 copy kernel three times before the timed region "
                         "(a known 512 MiB read + 512 MiB write, to scale rocprofv3's FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs on one GPU; --gpus must be 1 (nothing here uses a second device)")
    *_, hip = _imports()
    props = hip.props()
    base = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic"}
    device = {"name": props["name"], "arch": props["arch"], "compute_units": props["compute_units"],
              "clock_mhz": props["clock_khz"] / 1000}

    if args.calib_copy:
        from dlgrad_amd.buffer import Buffer
        from dlgrad_amd.device import Device
        src = Buffer.from_numpy(np.ones((16384, 8192), np.float32), Device.HIP)
        for _ in range(3):
            hip._map("copy", "x0", [src], src.shape)
        hip.lib().sync()
        del src
    if args.workload == "c2":
        R, C = 16384, 8192
        r = run_c2(R, C, args.steps, args.warmup)
        add = r["per_op"]["add_same"]
        out = {"metric": "elementwise/reduce HBM GB/s (1 GPU)", "value": r["GBps"], "unit": "GB/s", **base,
               "ms_per_step": r["ms_per_step"],
               "config": {"workload": f"C2 elementwise/broadcast/reduce suite, fp32 N(0,1), {R}x{C} "
                                      f"({r['n_ops']} kernels per step: add/sub/mul/div x same,(R,1),(1,C),scalar; "
                                      "exp relu log sqrt; sum/max x axis0,axis1,all)"},
               "roofline": {"bound": "hbm", "achieved": add["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": add["GBps"] / HBM_PEAK_GBS, "traffic": C2_ADD_TRAFFIC_BYTES,
                            "kernel": "map_add_vec_vec_v4u1nt" if R * C >= hip.NT_STORE_MIN_ELEMENTS else "map_add_vec_vec_v4u4",
                            "bytes_per_launch": 12 * R * C,
                            "avg_launch_ms": add["ms"]},
               "per_op_frac_hbm": {k: round(v["frac_hbm"], 3) for k, v in r["per_op"].items()}}
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_c2(R, C, reps=1)                 # the GPU's own size, one pass (~20 s)
        if not args.no_extra:
            # the other two thirds of the headline metric, each with its roofline and its CPU figure from this same run
            n = 4096
            m = run_matmul(n, n, n, max(3, min(args.steps, 10)), 2)
            out["matmul"] = {"metric": "matmul fp32 TFLOPS (1 GPU)", "value": round(m["TFLOPs"], 2), "unit": "TFLOP/s",
                             "config": {"workload": f"C3 fp32 matmul {n}x{n}x{n}, entries N(0, 1/sqrt(K))"},
                             "roofline": {"bound": "mfma", "achieved": round(m["TFLOPs"], 2), "peak": MFMA_FP32_PEAK_TFLOPS,
                                          "unit": "TFLOP/s", "frac": round(m["TFLOPs"] / MFMA_FP32_PEAK_TFLOPS, 4),
                                          "traffic": None, "kernel": hip.HIP.last_matmul_kernel,
                                          "flops_per_launch": m["flops"], "avg_launch_ms": round(m["kernel_ms"], 4)}}
            gg = run_gpt_graph(max(3, min(args.steps, 20)), 2)
            g = run_gpt(100, 20)
            out["gpt"] = {"metric": "GPT fwd+bwd tokens/s (1 GPU)", "value": round(gg["tokens_per_s"], 1), "unit": "tokens/s",
                          "config": {"workload": "C4 char-GPT vocab 65, block 128, 6 layers, 4 heads, n_embd 128, batch 16; forward + "
                                                 "backward + Adam step, captured once as a HIP graph and replayed per step"},
                          "ms_per_step": round(gg["ms_per_step"], 4), "graph_nodes": gg["graph_nodes"],
                          "loss_per_token": round(gg["loss_per_token"], 5),
                          "eager": {"tokens_per_s": round(g["tokens_per_s"], 1), "ms_per_step": round(g["ms_per_step"], 3),
                                    "launches_per_step": g["launches_per_step"],
                                    "us_per_launch": round(g["ms_per_step"] * 1e3 / g["launches_per_step"], 2)},
                          "roofline": {k: (round(v, 5) if isinstance(v, float) else v) for k, v in step_roofline(
                              6 * 1_187_968 * 2048, gg["ms_per_step"],
                              "whole replayed step against the fp32 MFMA peak (6 x 1.19 M matmul parameters x 2048 tokens); "
                              "every kernel is a few microseconds: bound by kernel-to-kernel latency").items()}}
            if not args.no_cpu:
                out["matmul"]["cpu_baseline"] = cpu_matmul(512)
                out["gpt"]["cpu_baseline"] = cpu_gpt()
            extra = {}
            for (r2, c2) in ((4096, 4096), (1024, 1024)):
                e = run_c2(r2, c2, args.steps, args.warmup, events_in_timed_region=False)
                extra[f"c2_{r2}x{c2}_cache_resident"] = {
                    "GBps": round(e["GBps"], 1), "ms_per_step": round(e["ms_per_step"], 4),
                    "add_same_GBps": round(e["per_op"]["add_same"]["GBps"], 1),
                    "us_per_launch": round(e["ms_per_step"] * 1e3 / e["launches_per_step"], 2),
                    "replayed_as_hipgraph": run_c2_graph(r2, c2, max(args.steps, 50))}
            sweep = {}
            for n in (128, 512, 1024, 2048, 4096, 8192):
                m = run_matmul(n, n, n, max(3, min(args.steps, 10)), 2)
                sweep[str(n)] = {"TFLOPs": round(m["TFLOPs"], 2), "kernel_ms": round(m["kernel_ms"], 4),
                                 "frac_mfma_fp32": round(m["TFLOPs"] / MFMA_FP32_PEAK_TFLOPS, 3)}
                if "TFLOPs_in_graph" in m:
                    sweep[str(n)].update(TFLOPs_in_graph=round(m["TFLOPs_in_graph"], 2), kernel_ms_in_graph=round(m["kernel_ms_in_graph"], 4))
            for name, (M_, K_, N_) in (("16384x128.128x512", (16384, 128, 512)), ("2048x128.128x128", (2048, 128, 128))):
                m = run_matmul(M_, N_, K_, 10, 2)
                sweep[name] = {"TFLOPs": round(m["TFLOPs"], 2), "kernel_ms": round(m["kernel_ms"], 4)}
                if "TFLOPs_in_graph" in m:
                    sweep[name].update(TFLOPs_in_graph=round(m["TFLOPs_in_graph"], 2), kernel_ms_in_graph=round(m["kernel_ms_in_graph"], 4))
            sweep.update(run_matmul_transposed(4096))
            extra["matmul_fp32_TFLOPs"] = sweep
            extra["gpt_char_greedy_decode_256"] = run_decode(256)
            extra["mlp_784_64_10_step"] = {k: round(v, 3) for k, v in run_mlp(50, 5).items()}
            extra["mlp_784_64_10_step_hipgraph"] = {k: round(v, 3) for k, v in run_mlp_graph(200, 10).items()}
            extra["c5_components"] = run_c5(max(3, min(args.steps, 10)), 2)
            extra["c5_attention"] = run_attention(max(3, min(args.steps, 10)), 2)
            extra["layout_and_select"] = run_layout_and_select(max(3, min(args.steps, 10)), 2)
            extra["host_device_transfers"] = run_transfers()
            extra["gpt_scaled_c5"] = run_gpt_large(2)
            out["extra"] = extra
    elif args.workload == "matmul":
        n = 4096
        m = run_matmul(n, n, n, args.steps, args.warmup)
        out = {"metric": "matmul fp32 TFLOPS (1 GPU)", "value": m["TFLOPs_wall"], "unit": "TFLOP/s", **base,
               "ms_per_step": m["ms_per_step"],
               "config": {"workload": f"C3 fp32 matmul {n}x{n}x{n}, entries N(0, 1/sqrt(K))"},
               "roofline": {"bound": "mfma", "achieved": m["TFLOPs"], "peak": MFMA_FP32_PEAK_TFLOPS,
                            "unit": "TFLOP/s", "frac": m["TFLOPs"] / MFMA_FP32_PEAK_TFLOPS, "traffic": None,
                            "flops_per_launch": m["flops"], "avg_launch_ms": m["kernel_ms"]}}
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_matmul(512)
    elif args.workload == "gpt":
        gg = run_gpt_graph(args.steps, args.warmup)               # the step as it is meant to be run on this device
        g = run_gpt(100, 20)                                      # the same step issued launch by launch from Python
        out = {"metric": "GPT fwd+bwd tokens/s (1 GPU)", "value": gg["tokens_per_s"], "unit": "tokens/s", **base,
               "ms_per_step": gg["ms_per_step"],
               "config": {"workload": "C4 char-GPT vocab 65, block 128, 6 layers, 4 heads, n_embd 128, batch 16; "
                                      "forward + backward + Adam step (RMSNorm, ReLU MLP, no bias, as examples/gpt.py), "
                                      "captured once as a HIP graph and replayed per step (same kernels, bit-identical)",
                          "graph_nodes": gg["graph_nodes"], "loss_per_token": gg["loss_per_token"],
                          "eager_ms_per_step": round(g["ms_per_step"], 3), "eager_tokens_per_s": round(g["tokens_per_s"], 1),
                          "eager_launches_per_step": g["launches_per_step"]},
               "roofline": step_roofline(6 * 1_187_968 * 2048, gg["ms_per_step"],
                                         "whole step against the fp32 MFMA peak; 6 x 1.19 M matmul parameters x 2048 tokens; "
                                         "at this size every kernel is a few microseconds and the step is bound by per-kernel "
                                         "latency, not by the matrix cores")}
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_gpt()
    elif args.workload == "gpt-large":
        g = run_gpt_large(max(1, min(args.steps, 5)))
        out = {"metric": "scaled GPT fwd+bwd tokens/s (1 GPU)", "value": g["train_tokens_per_s"], "unit": "tokens/s",
               **base, "ms_per_step": g["train_step_ms"],
               "config": {"workload": "C5 scaled GPT vocab 50304, block 1024, 12 layers, 12 heads, n_embd 768, batch 8; "
                                      "Zipf(1.1) token ids; forward + backward + Adam step", **g},
               "roofline": step_roofline(g["train_TFLOPs_est"] * 1e12 * g["train_step_ms"] * 1e-3, g["train_step_ms"],
                                         "whole step against the fp32 MFMA peak; 6 x 124 M matmul parameters x 8192 tokens "
                                         "(attention products not counted)")}
    elif args.workload == "components":
        # the kernel classes C2 does not reach, each at a size beyond the caches: C5's embedding, softmax
        # and cross-entropy shapes, transposes, permutes, argmax, selects
        comp = {**run_c5(args.steps, args.warmup), **run_layout_and_select(args.steps, args.warmup)}
        total_ms = sum(v["ms"] for v in comp.values())
        total_bytes = sum(v["GBps"] * v["ms"] * 1e6 for v in comp.values())
        worst = max(comp, key=lambda k: comp[k]["ms"])
        out = {"metric": "elementwise/reduce HBM GB/s (1 GPU)", "value": total_bytes / total_ms / 1e6, "unit": "GB/s",
               **base, "ms_per_step": total_ms,
               "config": {"workload": f"{len(comp)} layout, select, argmax, embedding, softmax and cross-entropy kernels at the "
                                      "scaled-GPT shapes, one launch each per step; value = algorithmic bytes / summed kernel time"},
               "roofline": {"bound": "hbm", "achieved": comp[worst]["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": comp[worst]["GBps"] / HBM_PEAK_GBS, "traffic": None, "kernel": worst,
                            "avg_launch_ms": comp[worst]["ms"]},
               "per_op": comp, "attention": run_attention(args.steps, args.warmup)}
    else:
        r = run_mlp(args.steps, args.warmup)
        out = {"metric": "MLP 784-64-10 step samples/s (1 GPU)", "value": r["samples_per_s"], "unit": "samples/s",
               **base, "ms_per_step": r["ms_per_step"],
               "config": {"workload": "C1 MLP 784-64-10, batch 128, fwd+bwd+SGD", "launches_per_step": r["launches_per_step"]},
               "roofline": None}
    out["device"] = device
    print(json.dumps(out))


if __name__ == "__main__":
    main()
