#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Headline workload (`config.workload`): the Q4_K decode GEMV sweep at Qwen3-8B layer shapes,
batch 1 — 36 layers x {q 4096x4096, k/v 1024x4096, o 4096x4096, gate/up 12288x4096,
down 4096x12288}, 252 distinct weight matrices (3.9 GB, so every launch streams from HBM, not
from the 256 MB Infinity Cache). One step = one execute of that 252-op plan. `value` is weight
bytes / wall time of the timed steps (inputs resident in HBM), the reference's GB/s convention
(crates/infr-vulkan/tests/decode_gemv_bw.rs:97,209).

The same JSON line carries `roofline` for the dominant kernel (the Q4_K GEMV; achieved = weight
bytes per launch / average launch duration from HIP events on the backend's stream), the
`cpu_baseline` (the C restatement of infr-cpu's scalar kernels on the host cores, bounded sample;
`cpu_baseline_mmq` and `cpu_baseline_moe` for the prefill half and the routed-expert path)
and `extra` with the secondary figures of the benchmark's other configurations: Q6_K / Q8_0 GEMV, batch 8, prefill
mmq int8 TOPS at M in {64, 512, 2048}, the ternary Q2_0 sweep and the MoE routed-expert GEMV.
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

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
# algorithmic bytes per launch -> measured HBM bytes per launch (profiles/gemv_q4k_decode_sweep.md); the
# figure holds for that launch shape only, so it is looked up by the bytes the timed launch really moved
MEASURED_TRAFFIC = {2887778304: 2905303356}
# prefill Op::Linear (quantizer + strip kernel) at M = 512, K = 4096, N = 12288: HBM bytes per op from the
# FETCH_SIZE / WRITE_SIZE runs in profiles/mmq_q4k_prefill.md, keyed by the op's integer operations
MEASURED_TRAFFIC_MMQ = {51539607552: 83607984}
INT8_PEAK_TOPS = 5000.0    # MI355X dense int8 MFMA, published

# (name, out_f, in_f) of one Qwen3-8B decoder layer
LAYER = [("q", 4096, 4096), ("k", 1024, 4096), ("v", 1024, 4096), ("o", 4096, 4096),
         ("gate", 12288, 4096), ("up", 12288, 4096), ("down", 4096, 12288)]
N_LAYERS = 36
RAMP_STEPS = 60            # untimed executes before the warmup steps: the clocks take ~30 ms of load to settle
VOCAB = 151936


def weight_bytes(dtype, out_f, in_f):
    from infr_amd import block_layout
    e, b = block_layout(dtype)
    return out_f * (in_f // e) * b


class Sweep:
    """A decode-step matvec sweep: every projection of `n_layers` layers (+ optional lm_head) as
    one plan of Op::Linear ops over distinct weight buffers.

    chain=False: every op reads the shared input and owns its output, so all ops are independent
    (the GEMV-bandwidth measurement; the backend groups them into one launch per in_f).
    chain=True: a decoder layer's dependency structure, {q,k,v}(x) -> o(q) -> {gate,up}(o) ->
    down(gate) -> next layer, i.e. four dependent launches per layer."""

    def __init__(self, be, dtype, m, n_layers, seed=0, head=False, sigma=0.02, chain=False):
        from infr_amd import (Bindings, BufferUsage, DType, Graph, Linear, TensorDesc,
                              synth_normal_f32, synth_weight)
        self.be, self.dtype, self.m = be, dtype, m
        g, binds = Graph(), Bindings()
        g4096 = Graph()            # the in_f = 4096 ops alone (same tensor ids, same buffers)
        self.bytes = self.bytes_4096 = 0
        self.launches = 0
        self.keep = []
        self.out_bufs = {}          # layer 0's outputs by projection name (for the parity gate)
        xs = {}
        for in_f in (4096, 12288):
            xid = g.input(TensorDesc((m, in_f), DType.F32))
            xb = be.upload_new(synth_normal_f32(1 + in_f, m * in_f))
            binds.bind(xid, xb)
            xs[in_f] = xid
            self.keep.append(xb)

        def new_out(out_f):
            # every projection has its own output, as in a real graph
            yid = g.output(TensorDesc((m, out_f), DType.F32))
            yb = be.alloc(m * out_f * 4)
            binds.bind(yid, yb)
            self.keep.append(yb)
            return yid
        # one layer's weights are generated on the host (seed 0 -> W) and uploaded; the other
        # layers are device copies: distinct HBM addresses are what keeps the sweep cold.
        protos = {}
        for i, (name, out_f, in_f) in enumerate(LAYER):
            protos[name] = be.upload_new(synth_weight(dtype, seed + i, out_f, in_f, sigma),
                                         BufferUsage.Weights)
        x_cur = xs[4096]
        for layer in range(n_layers):
            outs = {}
            for name, out_f, in_f in LAYER:
                nb = weight_bytes(dtype, out_f, in_f)
                if layer == 0:
                    wb = protos[name]
                else:
                    wb = be.alloc_uninit(nb, BufferUsage.Weights)
                    be.copy_buffer(protos[name], wb, nb)
                wid = g.weight(TensorDesc((out_f, in_f), dtype))
                binds.bind(wid, wb)
                self.keep.append(wb)
                if chain:
                    src = {"q": x_cur, "k": x_cur, "v": x_cur, "o": outs.get("q"), "gate": outs.get("o"),
                           "up": outs.get("o"), "down": outs.get("gate")}[name]
                else:
                    src = xs[in_f]
                outs[name] = new_out(out_f)
                if layer == 0:
                    self.out_bufs[name] = self.keep[-1]
                op = Linear(src, wid, outs[name], m, in_f, out_f)
                g.push(op)
                if in_f == 4096:
                    g4096.ops.append(op)
                    self.bytes_4096 += nb
                self.bytes += nb
                self.launches += 1
            x_cur = outs["down"]
        if head:
            nb = weight_bytes(dtype, VOCAB, 4096)
            wb = be.upload_new(synth_weight(dtype, seed + 99, VOCAB, 4096, sigma), BufferUsage.Weights)
            wid = g.weight(TensorDesc((VOCAB, 4096), dtype))
            binds.bind(wid, wb)
            self.keep.append(wb)
            g.push(Linear(x_cur if chain else xs[4096], wid, new_out(VOCAB), m, 4096, VOCAB))
            self.bytes += nb
            self.launches += 1
        be.sync()
        g4096.tensors, g4096.kinds = g.tensors, g.kinds
        self.plan, self.binds = be.compile(g), binds
        self.plan_4096 = be.compile(g4096) if not chain else None

    def step(self, plan=None):
        self.be.execute(plan or self.plan, self.binds)

    def time(self, steps, warmup, plan=None):
        for _ in range(warmup):
            self.step(plan)
        self.be.sync()
        t0 = time.perf_counter()
        self.be.timer_begin()
        for _ in range(steps):
            self.step(plan)
        dev_ms = self.be.timer_end()
        wall_ms = (time.perf_counter() - t0) * 1e3
        return dev_ms / steps, wall_ms / steps

    def free(self):
        self.plan = self.plan_4096 = None
        for b in self.keep:
            b.free()
        self.keep = []


def parity_gate_sweep(be, sw, dtype):
    """Untimed check of what the timed plan computed: sampled rows of three of its outputs (a q, a
    gate and a down projection of layer 0) against the CPU oracle on the same bytes. Q4_K decode
    outputs must be bit-identical. Returns "ok" or raises."""
    from infr_amd import DType, synth_normal_f32, synth_weight
    from oracle import oracle as orc
    for i, (name, out_f, in_f) in enumerate(LAYER):
        if name not in ("q", "gate", "down"):
            continue
        yb = sw.out_bufs[name]
        rows = 64
        w = synth_weight(dtype, i, out_f, in_f)
        x = synth_normal_f32(1 + in_f, sw.m * in_f)
        e, bpb = __import__("infr_amd").block_layout(dtype)
        bpr = in_f // e * bpb
        for row0 in (0, out_f - rows):
            got = be.download(yb, np.empty((sw.m, out_f), np.float32))[:, row0:row0 + rows]
            want = orc.linear(dtype, w[row0 * bpr:(row0 + rows) * bpr], x, sw.m, in_f, rows)
            if dtype in (DType.Q4K, DType.Q6K):
                if not np.array_equal(got.view(np.uint32), want.view(np.uint32)):
                    raise SystemExit(f"parity gate: {name} rows {row0}.. differ from the oracle")
            else:
                rel = np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want)
                if rel > 1e-4:
                    raise SystemExit(f"parity gate: {name} rel-L2 {rel:.2e}")
    return "ok"


def parity_gate_linear(be, dtype, m, in_f, out_f, tokens, rows=32):
    """Untimed: one Op::Linear at the timed shape, sampled tokens x rows against the oracle
    (bit-identical for the K-quants below 128 tokens, rel-L2 <= 2e-6 for Q4_K from 128 on, <= 1e-4 otherwise)."""
    from infr_amd import DType, synth_normal_f32, synth_weight
    from oracle import oracle as orc
    w = synth_weight(dtype, 0, out_f, in_f)
    x = synth_normal_f32(1, m * in_f)
    wb, xb, yb = be.upload_new(w), be.upload_new(x), be.alloc(m * out_f * 4)
    be.linear(dtype, wb, xb, yb, m, in_f, out_f)
    y = be.download(yb, np.empty((m, out_f), np.float32))
    for b in (wb, xb, yb):
        b.free()
    e, bpb = __import__("infr_amd").block_layout(dtype)
    bpr = in_f // e * bpb
    xs = x.reshape(m, in_f)[tokens].ravel()
    for row0 in (0, out_f // 2, out_f - rows):
        want = orc.linear(dtype, w[row0 * bpr:(row0 + rows) * bpr], xs, len(tokens), in_f, rows)
        got = y[tokens, row0:row0 + rows]
        if dtype == DType.Q4K and m >= 128:
            # the prefill strips contract the f32 epilogue (integers exact): ~1e-7 relative
            if np.linalg.norm(got.astype(np.float64) - want) > 2e-6 * np.linalg.norm(want):
                raise SystemExit(f"parity gate: Linear m={m} {in_f}->{out_f} outside rel-L2 2e-6")
        elif dtype in (DType.Q4K, DType.Q5K, DType.Q6K):
            if not np.array_equal(got.view(np.uint32), want.view(np.uint32)):
                raise SystemExit(f"parity gate: Linear m={m} {in_f}->{out_f} rows {row0}.. differ from the oracle")
        elif np.linalg.norm(got.astype(np.float64) - want) > 1e-4 * np.linalg.norm(want):
            raise SystemExit(f"parity gate: Linear m={m} {in_f}->{out_f} outside rel-L2 1e-4")
    return "ok"


def settle_clocks(be, plan, binds, seconds=0.03):
    """Untimed: keep the device loaded with `plan` for ~30 ms so that its clocks have settled
    (see RAMP_STEPS); every section's timing starts from the same state."""
    t0 = time.perf_counter()
    while True:
        be.execute(plan, binds)
        be.sync()
        if time.perf_counter() - t0 > seconds:
            break


def layer_bench(be, n_layers, dtype=None, rows=1):
    """A decode step through `n_layers` Qwen3-8B-shaped decoder layers without attention:
    RmsNorm -> {q, k, v} -> o(q) -> Add -> RmsNorm -> {gate, up} -> GatedAct -> down -> Add, every op
    reading what the previous one wrote. The plan absorbs the norms, the gated activation and the
    residual adds into the decode GEMVs (4 launches per layer instead of 9) at one token; `rows`
    tokens (a decode batch) run the ops as they are, Linears of a level grouped. Returns
    (ms per step, weight bytes, launches per step)."""
    from infr_amd import (Add, Bindings, BufferUsage, DType, GatedAct, Graph, Linear, RmsNorm, TensorDesc,
                          synth_normal_f32, synth_weight)
    dtype = dtype or DType.Q4K
    H, KV, FF = 4096, 1024, 12288
    g, binds, keep = Graph(), Bindings(), []

    def f32(shape, data=None, out=False):
        t = (g.output if out else g.input)(TensorDesc(shape, DType.F32))
        n = 1
        for d in shape:
            n *= d
        b = be.upload_new(data) if data is not None else be.alloc(n * 4)
        keep.append(b)
        binds.bind(t, b)
        return t
    R = rows
    x = f32((R, H), synth_normal_f32(1, R * H))
    protos = {name: be.upload_new(synth_weight(dtype, i, out_f, in_f), BufferUsage.Weights)
              for i, (name, out_f, in_f) in enumerate(LAYER)}
    keep += list(protos.values())
    total = 0
    for layer in range(n_layers):
        w = {}
        for name, out_f, in_f in LAYER:
            nb = weight_bytes(dtype, out_f, in_f)
            wb = protos[name]
            if layer:
                wb = be.alloc_uninit(nb, BufferUsage.Weights)
                be.copy_buffer(protos[name], wb, nb)
                keep.append(wb)
            w[name] = g.weight(TensorDesc((out_f, in_f), dtype))
            binds.bind(w[name], wb)
            total += nb
        n1, n2 = (f32((H,), synth_normal_f32(2 + i, H, mean=1.0, sigma=0.1)) for i in range(2))
        h1, q, k, v, o = (f32((R, d), out=True) for d in (H, H, KV, KV, H))
        h2, gt, up, act, dn = (f32((R, d), out=True) for d in (H, FF, FF, FF, H))
        g.push(RmsNorm(x, n1, h1, R, H, 1e-6))
        g.push(Linear(h1, w["q"], q, R, H, H))
        g.push(Linear(h1, w["k"], k, R, H, KV))
        g.push(Linear(h1, w["v"], v, R, H, KV))
        g.push(Linear(q, w["o"], o, R, H, H))
        g.push(Add(o, x, x, R * H))
        g.push(RmsNorm(x, n2, h2, R, H, 1e-6))
        g.push(Linear(h2, w["gate"], gt, R, H, FF))
        g.push(Linear(h2, w["up"], up, R, H, FF))
        g.push(GatedAct(gt, up, act, R, FF))
        g.push(Linear(act, w["down"], dn, R, FF, H))
        g.push(Add(dn, x, x, R * H))
    be.sync()
    plan = be.compile(g)
    settle_clocks(be, plan, binds)
    steps, t0 = 10, time.perf_counter()
    be.timer_begin()
    for _ in range(steps):
        be.execute(plan, binds)
    dev = be.timer_end() / steps
    wall = (time.perf_counter() - t0) * 1e3 / steps
    launches = plan.launches()
    plan = None
    for b in keep:
        b.free()
    return max(dev, wall), total, launches


def single_shape(be, dtype, m, in_f, out_f, reps=40, rotate_bytes=768 << 20, distinct_x=False):
    """One shape, cold: rotate through enough distinct copies of the weight to exceed the last
    level cache, `reps` back-to-back launches. Returns (ms per launch, weight bytes).
    distinct_x: every op multiplies its own activation tensor, so every op pays its own activation
    quantizer (a plan quantizes a tensor once for all the Linears of a level that read it)."""
    from infr_amd import Bindings, BufferUsage, DType, Graph, Linear, TensorDesc, synth_normal_f32, synth_weight
    nb = weight_bytes(dtype, out_f, in_f)
    # decode shapes: enough ops over distinct copies that a plan moves ~1.5 GB - the fixed cost of one
    # graph launch (~8 us) is then a few percent of the launch, and the 256 MB memory-side cache holds
    # a sixth of the weights at most when the plan runs again (at 384 MB per plan it held most of
    # them, and the launch cost was a fifth of a 1024 x 4096 group's time)
    if rotate_bytes > 1 and m <= 8:
        reps = max(reps, -(-(1536 << 20) // nb))
        rotate_bytes = max(rotate_bytes, reps * nb)
    copies = max(2, min(reps, -(-rotate_bytes // nb)))
    g, binds, keep = Graph(), Bindings(), []
    xid = g.input(TensorDesc((m, in_f), DType.F32))
    xb = be.upload_new(synth_normal_f32(1, m * in_f))
    binds.bind(xid, xb)
    xids = [xid]
    if distinct_x:
        for _ in range(reps - 1):
            xi = g.input(TensorDesc((m, in_f), DType.F32))
            xc = be.alloc_uninit(m * in_f * 4)
            be.copy_buffer(xb, xc, m * in_f * 4)
            binds.bind(xi, xc)
            xids.append(xi)
            keep.append(xc)
    proto = be.upload_new(synth_weight(dtype, 0, out_f, in_f), BufferUsage.Weights)
    keep += [xb, proto]
    wids = []
    for c in range(copies):
        wb = proto if c == 0 else be.alloc_uninit(nb, BufferUsage.Weights)
        if c:
            be.copy_buffer(proto, wb, nb)
            keep.append(wb)
        wid = g.weight(TensorDesc((out_f, in_f), dtype))
        binds.bind(wid, wb)
        wids.append(wid)
    for i in range(reps):
        # each launch owns its output: the launches are independent, as in the reference's
        # bandwidth probe (one recorder, `reps` dispatches, crates/infr-vulkan/tests/decode_gemv_bw.rs:186-210)
        yid = g.output(TensorDesc((m, out_f), DType.F32))
        yb = be.alloc(m * out_f * 4)
        keep.append(yb)
        binds.bind(yid, yb)
        g.push(Linear(xids[i % len(xids)], wids[i % copies], yid, m, in_f, out_f))
    plan = be.compile(g)
    settle_clocks(be, plan, binds)
    # three executes back to back per timing: the start-up of an execute (host-side checks, the graph
    # launch reaching an idle device) then overlaps the execute before
    best = 1e30
    for _ in range(4):
        be.timer_begin()
        for _ in range(3):
            be.execute(plan, binds)
        best = min(best, be.timer_end() / 3.0)
    plan = None
    for b in keep:
        b.free()
    return best / reps, nb


def prefill_layer_bench(be, m=512, n_layers=4, dtype=None):
    """The seven projections of `n_layers` Qwen3-8B-shaped layers at `m` tokens as a prefill chunk
    issues them: q, k and v read one tensor, gate and up another, o and down their own (no attention or
    elementwise ops in between, inputs are independent tensors). One plan; the Linears of a level that
    share an activation tensor share its quantization. Returns (us per layer, integer ops per layer)."""
    from infr_amd import Bindings, BufferUsage, DType, Graph, Linear, TensorDesc, synth_normal_f32, synth_weight
    dtype = dtype or DType.Q4K
    g, binds, keep = Graph(), Bindings(), []
    protos = {name: be.upload_new(synth_weight(dtype, i, out_f, in_f), BufferUsage.Weights)
              for i, (name, out_f, in_f) in enumerate(LAYER)}
    keep += list(protos.values())
    x_src = {4096: be.upload_new(synth_normal_f32(7, m * 4096)), 12288: be.upload_new(synth_normal_f32(8, m * 12288))}
    keep += list(x_src.values())
    ops = 0
    for layer in range(n_layers):
        xin = {}
        for grp, in_f in (("qkv", 4096), ("o", 4096), ("gu", 4096), ("down", 12288)):
            t = g.input(TensorDesc((m, in_f), DType.F32))
            b = be.alloc_uninit(m * in_f * 4)
            be.copy_buffer(x_src[in_f], b, m * in_f * 4)
            binds.bind(t, b)
            keep.append(b)
            xin[grp] = t
        for name, out_f, in_f in LAYER:
            nb = weight_bytes(dtype, out_f, in_f)
            wb = protos[name]
            if layer:
                wb = be.alloc_uninit(nb, BufferUsage.Weights)
                be.copy_buffer(protos[name], wb, nb)
                keep.append(wb)
            wid = g.weight(TensorDesc((out_f, in_f), dtype))
            yid = g.output(TensorDesc((m, out_f), DType.F32))
            yb = be.alloc(m * out_f * 4)
            keep.append(yb)
            binds.bind(wid, wb).bind(yid, yb)
            src = xin["qkv" if name in ("q", "k", "v") else "gu" if name in ("gate", "up") else name]
            g.push(Linear(src, wid, yid, m, in_f, out_f))
            ops += 2 * m * out_f * in_f
    be.sync()
    plan = be.compile(g)
    settle_clocks(be, plan, binds)
    best = 1e30
    for _ in range(4):
        be.timer_begin()
        be.execute(plan, binds)
        best = min(best, be.timer_end())
    plan = None
    for b in keep:
        b.free()
    return best * 1e3 / n_layers, ops / n_layers


def moe_bench(be, n_layers=6):
    """Routed-expert MoE at the Qwen3-30B-A3B shape (128 experts, top-8, hidden 2048, expert FFN
    768, Q4_K banks), 1 and 16 tokens, and prefill batches of 64 / 512 / 2048 tokens (pairs bucketed
    by expert, int8 MFMA): `n_layers` Op::MoeFfn with distinct banks in one plan, so the experts
    stream from HBM. Bytes = 2,654,208 per selected expert (gate+up+down); ops = 2 per weight and
    pair."""
    from infr_amd import Bindings, BufferUsage, DType, Graph, MoeFfn, TensorDesc, synth_normal_f32, synth_weight
    ne, n_expert, n_used, nff = 2048, 128, 8, 768
    per_expert = 3 * nff * ne * 144 // 256
    protos = [be.upload_new(synth_weight(DType.Q4K, 70 + i, n_expert * (nff if i < 2 else ne),
                                         ne if i < 2 else nff), BufferUsage.Weights) for i in range(3)]
    router = be.upload_new(synth_normal_f32(80, n_expert * ne, sigma=0.03))
    out, keep = {}, list(protos) + [router]
    for rows in (1, 16, 64, 512, 2048):
        g, binds = Graph(), Bindings()
        x = synth_normal_f32(81 + rows, rows * ne)
        xid = g.input(TensorDesc((rows, ne), DType.F32))
        rid = g.weight(TensorDesc((n_expert, ne), DType.F32))
        binds.bind(xid, be.upload_new(x)).bind(rid, router)
        for layer in range(n_layers):
            ids = []
            for i, proto in enumerate(protos):
                nb = proto.len_bytes()
                wb = proto if layer == 0 else be.alloc_uninit(nb, BufferUsage.Weights)
                if layer:
                    be.copy_buffer(proto, wb, nb)
                    keep.append(wb)
                shape = (n_expert, nff, ne) if i < 2 else (n_expert, ne, nff)
                wid = g.weight(TensorDesc(shape, DType.Q4K))
                binds.bind(wid, wb)
                ids.append(wid)
            yid = g.output(TensorDesc((rows, ne), DType.F32))
            yb = be.alloc(rows * ne * 4)
            keep.append(yb)
            binds.bind(yid, yb)
            g.push(MoeFfn(xid, xid, rid, ids[0], ids[1], ids[2], yid, ne, n_expert, n_used, nff, 1.0))
        plan = be.compile(g)
        settle_clocks(be, plan, binds)
        best = 1e30
        for _ in range(3):
            be.timer_begin()
            be.execute(plan, binds)
            best = min(best, be.timer_end())
        us = best * 1e3 / n_layers
        # every layer routes the same x through the same router: the distinct experts a layer
        # touches come from the routing itself (one untimed direct call)
        idx_b, y_b = be.alloc(rows * n_used * 4), be.alloc(rows * ne * 4)
        be.moe_ffn(binds.get(xid), router, protos[0], protos[1], protos[2], y_b, rows=rows, ne=ne, n_expert=n_expert,
                   n_used=n_used, n_ff_exp=nff, scale=1.0, sel_idx=idx_b)
        unique = int(np.unique(be.download(idx_b, np.empty(rows * n_used, np.int32))).size)
        idx_b.free()
        y_b.free()
        out[f"moe_q4k_t{rows}_us_per_layer"] = round(us, 2)
        out[f"moe_q4k_t{rows}_unique_experts"] = unique
        # HBM figure: the bytes of the distinct experts touched, each counted once
        out[f"moe_q4k_t{rows}_unique_expert_GBs"] = round(unique * per_expert / (us * 1e-6) / 1e9, 1)
        if rows <= 16:
            # no-reuse figure (every (token, expert) pair's bytes, as the reference's dense-equivalent
            # convention, crates/infr-metal/tests/moe_bw.rs:150-157): not a bandwidth once pairs share experts
            out[f"moe_q4k_t{rows}_per_pair_no_reuse_GBs"] = round(rows * n_used * per_expert / (us * 1e-6) / 1e9, 1)
        if rows >= 64:
            out[f"moe_q4k_t{rows}_TOPS"] = round(rows * n_used * 3 * nff * ne * 2 / (us * 1e-6) / 1e12, 1)
        plan = None
    for b in keep:
        b.free()
    return out


def moe_shapes_bench(be):
    """One token of Op::MoeFfn at the expert shapes of other MoE files (hidden x expert FFN, experts,
    top-k): Mixtral 8x7B, a 7168 x 2048 top-8 layer (32 experts standing in for 256), a 5120 x 8192
    top-1 layer and Qwen3-235B-A22B's. Q4_K banks (one synthetic expert repeated), direct calls
    that rotate over enough copies of the banks that the selected experts (71-198 MB) come from HBM.
    Bytes = the selected experts' gate + up + down."""
    from infr_amd import BufferUsage, DType, synth_normal_f32, synth_weight
    out = {}
    for name, ne, n_expert, n_used, nff in (("mixtral_8x7b", 4096, 8, 2, 14336), ("h7168_ff2048_top8", 7168, 32, 8, 2048),
                                            ("h5120_ff8192_top1", 5120, 16, 1, 8192), ("qwen3_235b", 4096, 128, 8, 1536)):
        protos = []
        for i in range(3):
            one = synth_weight(DType.Q4K, 90 + i, nff if i < 2 else ne, ne if i < 2 else nff)
            protos.append(be.upload_new(np.tile(one, n_expert), BufferUsage.Weights))
        active = n_used * 3 * nff * ne * 144 // 256
        copies = max(2, -(-600_000_000 // active))
        banks = [protos]
        for _ in range(copies - 1):
            layer = []
            for proto in protos:
                wb = be.alloc_uninit(proto.len_bytes(), BufferUsage.Weights)
                be.copy_buffer(proto, wb, proto.len_bytes())
                layer.append(wb)
            banks.append(layer)
        router = be.upload_new(synth_normal_f32(95, n_expert * ne, sigma=0.03))
        x, y = be.upload_new(synth_normal_f32(96, ne)), be.alloc(ne * 4)
        kw = dict(rows=1, ne=ne, n_expert=n_expert, n_used=n_used, n_ff_exp=nff, scale=1.0)
        best = 1e30
        for rep in range(4):
            be.timer_begin()
            for g, u, d in banks:
                be.moe_ffn(x, router, g, u, d, y, **kw)
            t = be.timer_end()
            if rep:
                best = min(best, t)
        us = best * 1e3 / copies
        out[f"moe_q4k_t1_{name}_us_per_layer"] = round(us, 1)
        out[f"moe_q4k_t1_{name}_selected_expert_GBs"] = round(active / (us * 1e-6) / 1e9, 1)
        for layer in banks:
            for b in layer:
                b.free()
        for b in (router, x, y):
            b.free()
    return out


def load_bench(be, n_layers=8):
    """A synthetic checkpoint of `n_layers` Qwen3-8B layers (Q4_K projections, Q6_K down) written
    as a GGUF file, then opened and uploaded tensor by tensor through the reader: page cache ->
    HBM over PCIe. Returns (open ms, upload ms, bytes)."""
    import tempfile
    from infr_amd import DType, synth_weight
    from infr_amd.gguf import Gguf, write_gguf
    tensors = []
    for l in range(n_layers):
        for name, out_f, in_f in LAYER:
            dt = DType.Q6K if name == "down" else DType.Q4K
            tensors.append((f"blk.{l}.{name}.weight", (in_f, out_f), int(dt), synth_weight(dt, 900 + l, out_f, in_f)))
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "synthetic.gguf")
        write_gguf(path, {"general.architecture": "qwen3", "qwen3.block_count": n_layers}, tensors)
        del tensors
        t0 = time.perf_counter()
        g = Gguf.open(path)
        t1 = time.perf_counter()
        infos = g.tensors()
        bufs = [g.upload(be, t.name) for t in infos]
        be.sync()
        t2 = time.perf_counter()
        nbytes = sum(t.nbytes for t in infos)
        for b in bufs:
            b.free()
        g.close()
    return (t1 - t0) * 1e3, (t2 - t1) * 1e3, nbytes


def cpu_baseline(dtype_name="Q4_K"):
    """The CPU oracle (C restatement of infr-cpu's scalar kernels, OpenMP over output rows with the
    reference's 16-row grain) on a bounded sample of the headline workload: one layer's seven
    projections, repeated for about 1.2 s of wall time on every thread OpenMP gives the process (all of
    the host's cores; ~20 core-seconds on 16), at least 3 passes; the best pass counts."""
    from infr_amd import DType, synth_normal_f32, synth_weight
    from oracle import oracle as orc
    threads = orc.max_threads()          # every core the host gives this process
    mats = []
    for i, (name, out_f, in_f) in enumerate(LAYER):
        mats.append((synth_weight(DType.Q4K, i, out_f, in_f), synth_normal_f32(1 + in_f, in_f), in_f, out_f))
    total = sum(w.size for w, _, _, _ in mats)
    for w, x, in_f, out_f in mats[:1]:
        orc.linear(DType.Q4K, w, x, 1, in_f, out_f, threads=threads)  # warm-up
    best, passes, t_start = 1e30, 0, time.perf_counter()
    while passes < 3 or (time.perf_counter() - t_start < 1.2 and passes < 2000):
        t0 = time.perf_counter()
        for w, x, in_f, out_f in mats:
            orc.linear(DType.Q4K, w, x, 1, in_f, out_f, threads=threads)
        best = min(best, time.perf_counter() - t0)
        passes += 1
    return {"value": round(total / best / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"one Qwen3-8B layer (7 Q4_K GEMVs, {total / 1e6:.1f} MB of weights), "
                      f"best of {passes} passes; C restatement of infr-cpu's scalar kernels"}


def cpu_baseline_mmq(m=512, in_f=4096, rows=512):
    """The prefill half on the CPU oracle: Op::Linear at M = 512 over a bounded slice of the 12288 x 4096
    Q4_K matrix (`rows` weight rows: the oracle's batch kernel walks output rows, so a row slice runs at
    the whole matrix's rate), every thread, best of at least 3 passes within ~1.5 s."""
    from infr_amd import DType, synth_normal_f32, synth_weight
    from oracle import oracle as orc
    threads = orc.max_threads()
    w = synth_weight(DType.Q4K, 0, rows, in_f)
    x = synth_normal_f32(1, m * in_f)
    orc.linear(DType.Q4K, w, x, m, in_f, rows, threads=threads)  # warm-up
    best, passes, t_start = 1e30, 0, time.perf_counter()
    while passes < 3 or (time.perf_counter() - t_start < 1.5 and passes < 200):
        t0 = time.perf_counter()
        orc.linear(DType.Q4K, w, x, m, in_f, rows, threads=threads)
        best = min(best, time.perf_counter() - t0)
        passes += 1
    ops = 2.0 * m * rows * in_f
    return {"value": round(ops / best / 1e12, 5), "unit": "TOP/s", "cores": threads, "kind": "port",
            "sample": f"Op::Linear Q4_K M={m}, K={in_f}, {rows} of 12288 weight rows ({ops / 1e9:.2f} GOP per pass, "
                      f"activation quantizer included), best of {passes} passes; C restatement of infr-cpu's scalar "
                      f"batch kernel, OpenMP over output rows"}


def cpu_baseline_moe(n_expert=16):
    """The routed-expert path on the CPU oracle: one token of Op::MoeFfn at the Qwen3-30B-A3B expert
    shape (hidden 2048, expert FFN 768, top-8, Q4_K banks; a token touches eight experts whatever the
    bank holds, so the sample's bank has `n_expert` of the 128 experts), every thread, best of at
    least 3 passes within ~1.5 s. The same unit as `moe_q4k_t1_us_per_layer`."""
    from infr_amd import DType, synth_normal_f32, synth_weight
    from oracle import oracle as orc
    threads = orc.max_threads()
    ne, n_used, nff = 2048, 8, 768
    banks = [synth_weight(DType.Q4K, 70 + i, n_expert * (nff if i < 2 else ne), ne if i < 2 else nff) for i in range(3)]
    router = synth_normal_f32(80, n_expert * ne, sigma=0.03)
    x = synth_normal_f32(81, ne)
    call = lambda: orc.moe_ffn(x, router, banks[0], banks[1], banks[2], ne=ne, n_expert=n_expert, n_used=n_used,
                               n_ff_exp=nff, threads=threads)
    call()  # warm-up
    best, passes, t_start = 1e30, 0, time.perf_counter()
    while passes < 3 or (time.perf_counter() - t_start < 1.5 and passes < 2000):
        t0 = time.perf_counter()
        call()
        best = min(best, time.perf_counter() - t0)
        passes += 1
    return {"value": round(best * 1e6, 1), "unit": "us per layer (1 token)", "cores": threads, "kind": "port",
            "sample": f"Op::MoeFfn, one token, hidden {ne}, expert FFN {nff}, top-{n_used} of a {n_expert}-expert Q4_K bank "
                      f"(8 experts touched as with 128), best of {passes} passes; C restatement of infr-cpu's MoeFfn arm"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=N_LAYERS)
    ap.add_argument("--no-extra", action="store_true", help="headline sweep only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-parity", action="store_true", help="skip the untimed oracle checks of the timed outputs")
    ap.add_argument("--sections", default="shapes,formats,mmq,chain,layer,ternary,moe,load",
                    help="comma list of secondary sections: shapes, formats, mmq, chain, layer, ternary, moe, load; mmq_scaling and moe_shapes (off by default)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)

    from infr_amd import DType, HipBackend
    be = HipBackend(0)
    caps = be.capabilities()

    sw = Sweep(be, DType.Q4K, 1, args.layers)
    # The device raises its clocks over the first ~30 ms of continuous load (the same plan runs at
    # 5.2 TB/s in its first five executes after an idle period and at 5.7 TB/s from the fortieth on),
    # and an idle half second resets that. A sustained figure is what the metric asks for, so an
    # untimed ramp of RAMP_STEPS executes precedes the W warmup steps; it is reported in `config`.
    sw.time(RAMP_STEPS, 0)
    dev_ms, wall_ms = sw.time(args.steps, args.warmup)
    ms = max(dev_ms, wall_ms)
    value = sw.bytes / (ms * 1e-3) / 1e9
    n_launch = max(1, sw.plan.launches())          # grouped: independent ops share a launch
    # Dominant kernel: the in_f = 4096 Q4_K GEMV (gemv_fused_kernel<FmtQ4K, 1, 8>), 216 of the 252
    # ops, timed alone with HIP events on the backend's stream: one launch per execute.
    k_ms, _ = sw.time(args.steps, 2, sw.plan_4096)
    k_launches = max(1, sw.plan_4096.launches())
    avg_launch_us = k_ms * 1e3 / k_launches
    bytes_per_launch = sw.bytes_4096 // k_launches
    achieved = bytes_per_launch / (avg_launch_us * 1e-6) / 1e9
    # HBM bytes per launch of that kernel at the default 36-layer sweep, from two rocprofv3 --pmc
    # runs of this command (FETCH_SIZE x 1.99788 and WRITE_SIZE x 1.0, the factors a plain
    # 28,311,552-byte device copy in the same runs gives); null for any other launch shape.
    traffic = MEASURED_TRAFFIC.get(bytes_per_launch)
    if traffic is None:
        print(f"bench.py: roofline.traffic is null - no counter run is recorded for a launch of {bytes_per_launch} "
              f"algorithmic bytes (MEASURED_TRAFFIC holds {sorted(MEASURED_TRAFFIC)})", file=sys.stderr)
    # what a kernel that only fetches reaches here: a read-only streaming pass over 2 GiB, same run
    probe = be.alloc_uninit(2 << 30)
    stream_read_plain = be.stream_read_gbs(probe, reps=10)
    stream_read = be.stream_read_gbs(probe, reps=10, nontemporal=True)  # as the streamed GEMV fetches
    probe.free()
    parity = "skipped (--no-parity)" if args.no_parity else parity_gate_sweep(be, sw, DType.Q4K)
    out = {
        "metric": "Q4_K GEMV HBM GB/s (% of peak) + prefill mmq int8 TOPS at M=512",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "i8", "data": "synthetic",
        "config": {"workload": f"Q4_K decode GEMV sweep, Qwen3-8B layer shapes x {args.layers} layers "
                               f"({sw.launches} independent Op::Linear over distinct matrices, "
                               f"{sw.bytes / 1e9:.2f} GB, one plan), batch 1",
                   "weights": "N(0,0.02^2) seed 0 -> Q4_K", "activations": "N(0,1) f32, quantized on GPU",
                   "clock_ramp_steps_untimed": RAMP_STEPS,
                   "parity": parity,
                   "device": caps["device_name"], "compute_units": caps["compute_units"]},
        "pct_of_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "launches_per_step": n_launch,
        "roofline": {"bound": "hbm", "kernel": "gemv_fused_kernel<FmtQ4K, 1, 8, false, true> (in_f 4096 group, rows streamed through LDS rings)",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "avg_launch_us": round(avg_launch_us, 3), "bytes_per_launch": bytes_per_launch,
                     "stream_read_GBs": round(stream_read, 1),
                     "stream_read_plain_loads_GBs": round(stream_read_plain, 1),
                     "frac_of_stream_read": round(achieved / stream_read, 4)},
    }
    sw.free()

    extra = {}
    sections = set() if args.no_extra else set(args.sections.split(","))
    if "shapes" in sections:
        for name, dt in (("Q4_K", DType.Q4K), ("Q6_K", DType.Q6K), ("Q8_0", DType.Q8_0)):
            for m in (1, 8):
                for (out_f, in_f) in ((4096, 4096), (1024, 4096), (12288, 4096), (4096, 12288)):
                    t, nb = single_shape(be, dt, m, in_f, out_f)
                    extra[f"gemv_{name}_m{m}_{out_f}x{in_f}_GBs"] = round(nb / (t * 1e-3) / 1e9, 1)
        # the same shapes warm: two copies of one matrix (19-57 MB), resident in the 256 MB Infinity
        # Cache, so these are cache figures and not HBM bandwidth
        for (out_f, in_f) in ((4096, 4096), (1024, 4096), (12288, 4096), (4096, 12288)):
            t, nb = single_shape(be, DType.Q4K, 1, in_f, out_f, rotate_bytes=1)
            extra[f"gemv_Q4_K_m1_{out_f}x{in_f}_warm_cache_resident_GBs"] = round(nb / (t * 1e-3) / 1e9, 1)
    if "formats" in sections:
        for name, dt in (("Q5_K", DType.Q5K), ("Q4_0", DType.Q4_0), ("Q4_1", DType.Q4_1), ("Q5_0", DType.Q5_0),
                         ("Q5_1", DType.Q5_1), ("IQ4_NL", DType.IQ4NL), ("Q2_0", DType.Q2_0), ("Q2_K", DType.Q2K),
                         ("Q3_K", DType.Q3K), ("IQ4_XS", DType.IQ4XS), ("MXFP4", DType.MXFP4), ("NVFP4", DType.NVFP4),
                         ("TQ2_0", DType.TQ2_0), ("TQ1_0", DType.TQ1_0)):
            for m in (1, 8):
                for (out_f, in_f) in ((4096, 4096), (12288, 4096), (4096, 12288)):
                    t, nb = single_shape(be, dt, m, in_f, out_f)
                    extra[f"gemv_{name}_m{m}_{out_f}x{in_f}_GBs"] = round(nb / (t * 1e-3) / 1e9, 1)
    if "mmq" in sections:
        for M in (64, 512, 2048):
            # (every op multiplies its own activation tensor: each pays its own quantizer launch)
            t, nb = single_shape(be, DType.Q4K, M, 4096, 12288, reps=10, distinct_x=True)
            extra[f"mmq_Q4_K_M{M}_TOPS"] = round(2.0 * M * 12288 * 4096 / (t * 1e-3) / 1e12, 2)
            extra[f"mmq_Q4_K_M{M}_pct_int8_peak"] = round(100 * extra[f"mmq_Q4_K_M{M}_TOPS"] / INT8_PEAK_TOPS, 2)
            if M == 512:
                # the prefill half of the metric: one Op::Linear = the activation quantizer's launch and
                # the int8-MFMA kernel's (ten back-to-back ops over rotated weight copies, HIP events
                # on the backend's stream); ops = 2 M N K
                ops = 2.0 * M * 12288 * 4096
                traffic_mmq = MEASURED_TRAFFIC_MMQ.get(int(ops))
                if traffic_mmq is None:
                    print("bench.py: roofline_mmq.traffic is null - no counter run is recorded for this op",
                          file=sys.stderr)
                out["roofline_mmq"] = {
                    "bound": "mfma", "kernel": "quantize_q8_tiled_kernel + mmq_strip_q4k_kernel<3> (M=512, K=4096, N=12288)",
                    "achieved": round(ops / (t * 1e-3) / 1e12, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                    "frac": round(ops / (t * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4), "traffic": traffic_mmq,
                    "avg_launch_us": round(t * 1e3, 2), "ops_per_launch": ops,
                    "parity": "skipped (--no-parity)" if args.no_parity else
                              parity_gate_linear(be, DType.Q4K, M, 4096, 12288, [0, 255, 256, 511])}
        # the other three projections of the layer at 512 tokens (crates/infr-vulkan/tests/decode_gemv_bw.rs:61-73
        # for the shape mix), one op = quantizer + GEMM as above
        for (out_f, in_f) in ((4096, 4096), (1024, 4096), (4096, 12288)):
            t, nb = single_shape(be, DType.Q4K, 512, in_f, out_f, reps=10, distinct_x=True)
            extra[f"mmq_Q4_K_M512_{out_f}x{in_f}_TOPS"] = round(2.0 * 512 * out_f * in_f / (t * 1e-3) / 1e12, 2)
        extra["mmq_Q4_K_M512_12288x4096_TOPS"] = extra["mmq_Q4_K_M512_TOPS"]
        # and the whole layer's seven projections as a prefill chunk issues them (q / k / v and gate / up
        # share their activation tensor and its quantization)
        us, ops_layer = prefill_layer_bench(be, 512)
        extra["prefill_layer_Q4_K_M512_us_per_layer"] = round(us, 1)
        extra["prefill_layer_Q4_K_M512_TOPS"] = round(ops_layer / (us * 1e-6) / 1e12, 1)
        # the matrix rate the device sustains on a register-only loop of the same MFMA (no memory
        # traffic): constant operands, and pseudo-random operands as the kernels feed it
        extra["mfma_i8_peak_const_operands_TOPS"] = round(be.mfma_i8_peak_tops(4, 4096, False), 1)
        extra["mfma_i8_peak_random_operands_TOPS"] = round(be.mfma_i8_peak_tops(4, 4096, True), 1)
        extra["mmq_Q4_K_M512_pct_of_measured_mfma_peak"] = round(
            100 * extra["mmq_Q4_K_M512_TOPS"] / extra["mfma_i8_peak_random_operands_TOPS"], 2)
        # the other formats with an MFMA prefill kernel, at the ffn_down shape 4096 x 12288 (Q6_K there
        # in a Q4_K_M file)
        for name, dt in (("Q6_K", DType.Q6K), ("Q5_K", DType.Q5K), ("Q8_0", DType.Q8_0), ("Q4_0", DType.Q4_0),
                         ("Q2_0", DType.Q2_0), ("IQ4_XS", DType.IQ4XS), ("Q2_K", DType.Q2K),
                         ("Q3_K", DType.Q3K), ("TQ2_0", DType.TQ2_0), ("TQ1_0", DType.TQ1_0), ("MXFP4", DType.MXFP4),
                         ("NVFP4", DType.NVFP4)):
            for M in (64, 512, 2048):
                t, nb = single_shape(be, dt, M, 12288, 4096, reps=10, distinct_x=True)
                extra[f"mmq_{name}_M{M}_TOPS"] = round(2.0 * M * 12288 * 4096 / (t * 1e-3) / 1e12, 2)
    if "mmq_scaling" in sections:
        # the same prefill kernel on grids of 64 .. 4096 workgroups (32 rows x 128 tokens each,
        # M = 512, K = 16384): TOPS per resident workgroup falls as the device fills, which with
        # the clock counters of a profiler run separates per-workgroup latency from the power limit
        for out_f in (512, 2048, 8192, 32768):
            t, nb = single_shape(be, DType.Q4K, 512, 16384, out_f, reps=6, rotate_bytes=1)
            extra[f"mmq_Q4_K_M512_K16384_N{out_f}_TOPS"] = round(2.0 * 512 * out_f * 16384 / (t * 1e-3) / 1e12, 2)
    if "chain" in sections:
        ch = Sweep(be, DType.Q4K, 1, args.layers, chain=True)
        settle_clocks(be, ch.plan, ch.binds)
        d, w = ch.time(10, 2)
        extra["decode_chain_Q4_K_GBs"] = round(ch.bytes / (max(d, w) * 1e-3) / 1e9, 1)
        extra["decode_chain_launches_per_step"] = ch.plan.launches()
        ch.free()
    if "layer" in sections:
        ms, nb, launches = layer_bench(be, args.layers)
        extra["decode_layer_Q4_K_GBs"] = round(nb / (ms * 1e-3) / 1e9, 1)
        extra["decode_layer_us_per_layer"] = round(ms * 1e3 / args.layers, 2)
        extra["decode_layer_launches_per_step"] = launches
        for rows in (8, 16):
            ms, nb, launches = layer_bench(be, args.layers, rows=rows)
            extra[f"decode_layer_m{rows}_us_per_layer"] = round(ms * 1e3 / args.layers, 2)
            extra[f"decode_layer_m{rows}_launches_per_step"] = launches
        if os.environ.get("INFR_HIP_FUSE", "1") != "0":
            # the same plan with the absorption switched off (a fresh process: the switch is read once)
            import subprocess
            env = dict(os.environ, INFR_HIP_FUSE="0")
            r = subprocess.run([sys.executable, os.path.abspath(__file__), "--no-cpu", "--sections", "layer",
                                "--layers", str(args.layers), "--steps", "1", "--warmup", "1"],
                               env=env, capture_output=True, text=True, timeout=600)
            for line in r.stdout.splitlines():
                if line.startswith("{"):
                    ex = json.loads(line)["extra"]
                    extra["decode_layer_unfused_Q4_K_GBs"] = ex["decode_layer_Q4_K_GBs"]
                    extra["decode_layer_unfused_us_per_layer"] = ex["decode_layer_us_per_layer"]
                    extra["decode_layer_unfused_launches_per_step"] = ex["decode_layer_launches_per_step"]
    if "ternary" in sections:
        tern = Sweep(be, DType.Q2_0, 1, N_LAYERS, head=True)
        settle_clocks(be, tern.plan, tern.binds)
        d, w = tern.time(5, 2)
        tms = max(d, w)
        extra["ternary_Q2_0_sweep_GBs"] = round(tern.bytes / (tms * 1e-3) / 1e9, 1)
        extra["ternary_Q2_0_tok_s_equiv"] = round(1e3 / tms, 1)
        tern.free()
    if "moe" in sections:
        extra.update(moe_bench(be))
    if "moe_shapes" in sections:
        extra.update(moe_shapes_bench(be))
    if "load" in sections:
        open_ms, up_ms, nb = load_bench(be)
        extra["gguf_open_ms"] = round(open_ms, 2)
        extra["gguf_upload_GBs_pcie_inclusive"] = round(nb / (up_ms * 1e-3) / 1e9, 2)
        extra["gguf_upload_bytes"] = nb
    out["extra"] = extra
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
        out["cpu_baseline_mmq"] = cpu_baseline_mmq()
        out["cpu_baseline_moe"] = cpu_baseline_moe()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
