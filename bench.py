#!/usr/bin/env python3
"""Benchmark of the target-verify hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload 27b|9b]

One "step" is one pass of the M=16 int4 verify_qmm over every projection of the dense
stack (27B-shaped by default: 64 layers x {qkv, o, gate, up, down} = 320 calls through
``verify_matmul``, x re-drawn per call, all operands resident in HBM), replayed from a
HIP graph so that host launch overhead is not what is measured.  The printed value is
aggregate weight bytes (packed codes + scales + biases) per second.

Also measured and reported in the same JSON line:
  roofline      algorithmic bytes of the qmm kernel per launch / average launch
                duration (HIP events around the timed region), against 8 TB/s HBM
  replay        GDN tape-replay rollback, 48 layers x 32 heads, 16 steps, one launch
  cpu_baseline  the oracle's C port of the reference arithmetic on the host cores,
                on a bounded sample of the same workload

Exactly one JSON line goes to stdout; progress goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # bytes/s, MI355X HBM3E
# HBM bytes per launch of the qmm kernel (mean over the launches of a stack) cannot be measured by
# this file: counters need the profiler.  The figure is read from the text summary of the two
# rocprofv3 --pmc runs of this file (FETCH_SIZE, WRITE_SIZE, scaled by the same counters' reading
# for a 1 GiB copy) kept under profiles/, which also states the SHA-256 of the kernel's source
# files as they were when the counters were taken.  If the sources have changed since, the figure
# describes another kernel and is not reported.
TRAFFIC_PROFILES = {"27b": "profiles/qmm_stream_kernel_27b_stack_pmc.txt"}
KERNEL_SOURCES = ("dflash-mlx_amd/csrc/qmm_m16_stream.hip", "dflash-mlx_amd/csrc/qmm_stream_device.h")


def kernel_sources_sha256() -> str:
    import hashlib

    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(workload: str):
    """(bytes per launch or None, where the figure comes from or why there is none)."""
    import re

    rel = TRAFFIC_PROFILES.get(workload)
    if rel is None or not os.path.exists(os.path.join(ROOT, rel)):
        return None, "no counter summary for this workload"
    text = open(os.path.join(ROOT, rel)).read()
    sha = re.search(r"^kernel_sources_sha256:\s*([0-9a-f]{64})", text, flags=re.M)
    traffic = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", text, flags=re.M)
    if not sha or not traffic:
        return None, f"{rel} does not state the kernel sources it was taken with"
    if sha.group(1) != kernel_sources_sha256():
        return None, f"{rel} was taken with other kernel sources"
    return float(traffic.group(1)), rel


LEGS = ("other_stack", "dependent", "gate_up", "packed", "chain", "mlp", "single", "moe", "replay", "forward", "sdpa", "glue")


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_stack(stack: str, device: str, join_gate_up: bool = False):
    """All operands of one pass over the stack, generated on the device.  ``join_gate_up``:
    the rows of gate_proj and up_proj (same values as in the separate form) laid end to end
    and served by one call on gate_proj's input, as ``fuse_shared_input_linears`` arranges
    them for projections that read the same activations."""
    import torch

    from dflash_mlx_amd.workloads import QmmCase, make_qmm_case, seed_for, stack_linears

    linears, layers, cfg = stack_linears(stack)
    calls = []
    for layer in range(layers):
        for i, (name, K, N) in enumerate(linears):
            case = make_qmm_case(K, N, seed_for(cfg, layer) * 8 + i, device=device)
            if join_gate_up and name == "up_proj":
                gate = calls.pop()
                case = QmmCase(gate.x, torch.cat([gate.w, case.w]), torch.cat([gate.scales, case.scales]),
                               torch.cat([gate.biases, case.biases]), case.group_size)
            calls.append(case)
    torch.cuda.synchronize()
    return calls


def run_pass(calls):
    from dflash_mlx_amd.verify_qmm import verify_matmul

    return [verify_matmul(c.x, c.w, c.scales, c.biases, group_size=c.group_size, bits=4) for c in calls]


def run_pass_packed(calls, packed):
    from dflash_mlx_amd.verify_qmm import verify_matmul_packed

    return [verify_matmul_packed(c.x, p) for c, p in zip(calls, packed)]


def time_region(fn, steps: int):
    """Wall time and HIP-event time (ms) of ``steps`` invocations of fn."""
    import torch

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms, start.elapsed_time(stop)


def capture(fn):
    """Run ``fn`` once on a side stream (so that every lazily created buffer exists), then
    record it into a HIP graph on that stream.  Returns (graph, outputs of the capture)."""
    from dflash_mlx_amd.graph_replay import record

    return record(fn)


def bench_qmm_stack(stack: str, steps: int, warmup: int, device: str, join_gate_up: bool = False,
                    packed: bool = False):
    """``packed``: every linear's weights also stored in the streaming kernel's order
    (``pack_weights``, done before the timed region as at model load) and the calls made through
    ``verify_matmul_packed``; the results must equal those of the row-major calls bit for bit."""
    import torch

    from dflash_mlx_amd.workloads import qmm_algorithmic_bytes, stack_bytes

    calls = build_stack(stack, device, join_gate_up)
    weight_bytes, total_bytes = stack_bytes(stack)
    if join_gate_up:  # x and the launch are shared: count what the calls made here move
        total_bytes = sum(qmm_algorithmic_bytes(c.K, c.N)[1] for c in calls)
    log(f"[bench] {stack} stack: {len(calls)} qmm calls/step, {weight_bytes / 1e9:.3f} GB weights")

    eager = run_pass(calls)  # also creates the split-K workspace outside of graph capture
    torch.cuda.synchronize()
    one_pass = lambda: run_pass(calls)  # noqa: E731
    if packed:
        from dflash_mlx_amd.verify_qmm import pack_weights

        images = [pack_weights(c.w, c.scales, c.biases) for c in calls]
        one_pass = lambda: run_pass_packed(calls, images)  # noqa: E731

    graph, captured = capture(one_pass)

    # every replay must reproduce the eager result bit for bit
    for r in range(2):
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(eager, captured):
            if not torch.equal(a, b):
                raise RuntimeError(f"graph replay {r} differs from the eager result")

    for _ in range(warmup):
        graph.replay()
    wall_ms, ev_ms = time_region(graph.replay, steps)
    ms_per_step = wall_ms / steps
    # eager launches through the Python surface, for the record (one pass first: the outputs of
    # a pass are new tensors, and the allocator's pool has to have grown to hold them)
    one_pass()
    e_wall, _ = time_region(one_pass, max(1, min(steps, 3)))
    res = dict(
        calls_per_step=len(calls), weight_bytes=weight_bytes, total_bytes=total_bytes,
        ms_per_step=ms_per_step, event_ms_per_step=ev_ms / steps,
        weight_gbps=weight_bytes / (ms_per_step * 1e-3) / 1e9,
        avg_launch_us=ev_ms / steps / len(calls) * 1e3,
        bytes_per_launch=total_bytes / len(calls),
        eager_ms_per_step=e_wall / max(1, min(steps, 3)),
    )
    del graph, captured, eager, calls
    torch.cuda.empty_cache()
    return res


def bench_qmm_chain_stack(stack: str, steps: int, warmup: int, device: str, layers_per_launch: int = 1,
                          join_gate_up: bool = False, joint_split: bool = False, packed: bool = False):
    """The same stack with the projections of ``layers_per_launch`` layers handed over as one list
    per launch (``QmmChain``, dflash_qmm_m16_chain): one persistent grid runs them back to back,
    each divided among the workgroups as a launch of its own would be.  Every projection has an
    input of its own here, as in the headline (no dependencies between them), and the outputs
    must equal those of the separate launches bit for bit.  ``join_gate_up``: gate_proj and
    up_proj as one problem of both matrices' rows (see ``build_stack``).  ``joint_split``: the units
    of a launch's problems divided among the workgroups as one range (hardly any row block then
    crosses workgroups); outputs must be within one step of the output type of the separate
    launches and equal on at least 99 % of the elements.  ``packed``: every problem's weights as the
    packed images of ``pack_weights`` (a second copy of the weights; same bits out)."""
    import torch

    from dflash_mlx_amd._native import QMM_CHAIN_MAX
    from dflash_mlx_amd.verify_qmm import ChainProblem, QmmChain
    from dflash_mlx_amd.workloads import stack_bytes, stack_linears

    calls = build_stack(stack, device, join_gate_up)
    per_layer = len(stack_linears(stack)[0]) - (1 if join_gate_up else 0)
    per_chain = per_layer * layers_per_launch
    assert per_chain <= QMM_CHAIN_MAX
    _, total_bytes = stack_bytes(stack)
    if join_gate_up:  # x is shared: count what the problems handed over here move
        from dflash_mlx_amd.workloads import qmm_algorithmic_bytes

        total_bytes = sum(qmm_algorithmic_bytes(c.K, c.N)[1] for c in calls)
    if packed:
        from dflash_mlx_amd.verify_qmm import pack_weights

        images = [pack_weights(c.w, c.scales, c.biases) for c in calls]
        problems = [ChainProblem(c.x, im) for c, im in zip(calls, images)]
    else:
        problems = [ChainProblem(c.x, c.w, c.scales, c.biases) for c in calls]
    chains = [QmmChain(problems[i:i + per_chain], joint_split=joint_split) for i in range(0, len(calls), per_chain)]

    def one_pass():
        return [chain() for chain in chains]

    separate = run_pass(calls[:per_chain])
    got = one_pass()
    torch.cuda.synchronize()
    for a, b in zip(separate, got[0]):
        if joint_split:
            a32, b32 = a.float(), b.float()
            close = (a32 - b32).abs() <= 2.0 ** -7 * torch.maximum(a32.abs(), b32.abs()) + 1e-5 * a32.abs().max()
            if not bool(close.all()) or float((a == b).float().mean()) < 0.99:
                raise RuntimeError("a jointly split chained launch is further from the separate launches than one rounding")
        elif not torch.equal(a, b):
            raise RuntimeError("a chained launch differs from the separate launches")
    graph, _ = capture(one_pass)
    for _ in range(warmup):
        graph.replay()
    wall_ms, ev_ms = time_region(graph.replay, steps)
    res = dict(launches_per_step=len(chains), projections_per_launch=per_chain,
               ms_per_step=wall_ms / steps, us_per_layer=ev_ms / steps / (len(calls) / per_layer) * 1e3,
               avg_launch_us=ev_ms / steps / len(chains) * 1e3, bytes_per_launch=total_bytes / len(chains),
               frac_hbm=total_bytes / (ev_ms / steps * 1e-3) / HBM_PEAK)
    del graph, chains, calls, got, separate, problems
    if packed:
        del images
    torch.cuda.empty_cache()
    return res


def bench_mlp_chain(stack: str, steps: int, warmup: int, device: str):
    """The MLP of every layer of the stack, four ways: (a) gate, up, silu * mul (array
    operators), down as four separate steps; (b) gate and up in one launch, silu * mul, down;
    (c) gate/up with the silu * mul epilogue as one chained launch of a single problem, then down
    as a launch of its own; (d) one launch per layer: gate/up with the epilogue, and down, which
    waits inside the launch for the hidden activation while its weights already stream."""
    import torch

    from dflash_mlx_amd.verify_qmm import ChainProblem, QmmChain, verify_matmul
    from dflash_mlx_amd.workloads import make_qmm_case, qmm_algorithmic_bytes, seed_for, stack_linears

    linears, layers, cfg = stack_linears(stack)
    dims = {name: (K, N) for name, K, N in linears}
    (H, I) = dims["gate_proj"]
    mlps, nbytes = [], 0
    for layer in range(layers):
        g = make_qmm_case(H, I, seed_for(cfg, layer) * 8 + 2, device=device)
        u = make_qmm_case(H, I, seed_for(cfg, layer) * 8 + 3, device=device)
        d = make_qmm_case(I, H, seed_for(cfg, layer) * 8 + 4, device=device)
        gu = tuple(torch.cat([a, b]) for a, b in ((g.w, u.w), (g.scales, u.scales), (g.biases, u.biases)))
        mlps.append((g, u, d, gu))
        nbytes += 2 * qmm_algorithmic_bytes(H, I)[1] + qmm_algorithmic_bytes(I, H)[1]
    torch.cuda.synchronize()
    silu = torch.nn.functional.silu

    def separate():
        out = []
        for g, u, d, _ in mlps:
            h = silu(verify_matmul(g.x, g.w, g.scales, g.biases)) * verify_matmul(g.x, u.w, u.scales, u.biases)
            out.append(verify_matmul(h, d.w, d.scales, d.biases))
        return out

    def joined():
        out = []
        for g, u, d, gu in mlps:
            both = verify_matmul(g.x, *gu)
            h = silu(both[:, :I]) * both[:, I:]
            out.append(verify_matmul(h, d.w, d.scales, d.biases))
        return out

    chains = []
    for g, u, d, gu in mlps:
        hidden = ChainProblem(g.x, *gu, epilogue="silu_mul")
        chains.append(QmmChain([hidden, ChainProblem(hidden, d.w, d.scales, d.biases)]))

    def chained():
        return [chain()[1] for chain in chains]

    hidden_only = [QmmChain([ChainProblem(g.x, *gu, epilogue="silu_mul")]) for g, u, d, gu in mlps]

    def epilogue_then_down():
        return [verify_matmul(chain()[0], d.w, d.scales, d.biases) for chain, (g, u, d, gu) in zip(hidden_only, mlps)]

    res = {}
    ref = joined()
    got = chained()
    torch.cuda.synchronize()
    if any(c.error_word() for c in chains):
        raise RuntimeError("a chained launch gave up waiting")
    # the hidden activation of (c) is that of (b) rounded once less between gate/up and silu:
    # the outputs agree to bf16 rounding of the hidden activation, not bit for bit
    rel = max(float((a.float() - b.float()).norm() / b.float().norm()) for a, b in zip(got, ref))
    if rel > 2e-2:
        raise RuntimeError(f"chained MLP differs from the separate launches (relative {rel:.3g})")
    res["rel_diff_chained_vs_joined"] = rel
    for name, fn in (("separate_launches", separate), ("gate_up_in_one_launch", joined),
                     ("gate_up_with_epilogue_then_down", epilogue_then_down), ("one_launch_per_layer", chained)):
        fn()
        graph, _ = capture(fn)
        for _ in range(warmup):
            graph.replay()
        _, ev_ms = time_region(graph.replay, steps)
        res[name] = dict(us_per_layer=ev_ms / steps / layers * 1e3,
                         frac_hbm=nbytes / (ev_ms / steps * 1e-3) / HBM_PEAK)
        del graph
    del chains, mlps, ref, got
    torch.cuda.empty_cache()
    return res


def bench_dependent_layers(stack: str, steps: int, warmup: int, device: str, packed: bool = False):
    """The stack in the order a model runs it (dflash_mlx/runtime.py:779-821, the layer loop of the
    verify forward): every launch consumes what the one before produced.  Per layer: the joined
    q/k/v projection of the layer's input; a copy of the first `hidden` columns of its output
    stands in for the attention between it and o_proj; o_proj; gate_proj and up_proj as one
    launch with the silu * mul epilogue on o_proj's output; down_proj on the hidden activation;
    its output is the next layer's input.  Four qmm launches and one small copy per layer, none
    of which can start before the previous one has ended.  Scales and biases are shrunk so that
    activations keep their magnitude from layer to layer; the bytes moved are the headline's minus
    the second read of x by up_proj.  ``packed``: every launch on the packed copy of its weights
    (what ``pack_verify_linears`` gives a model; the result must be the row-major one bit for bit)."""
    import torch

    from dflash_mlx_amd.verify_qmm import ChainProblem, QmmChain, pack_weights, verify_matmul, verify_matmul_packed
    from dflash_mlx_amd.workloads import qmm_algorithmic_bytes, stack_linears

    linears, layers, _ = stack_linears(stack)
    dims = {name: (K, N) for name, K, N in linears}
    H = dims["o_proj"][0]
    calls = build_stack(stack, device, join_gate_up=True)   # qkv, o, gate/up joined, down per layer
    per_layer = len(linears) - 1
    total_bytes = sum(qmm_algorithmic_bytes(c.K, c.N)[1] for c in calls)
    x0 = calls[0].x

    def unit_gain(c, x, halves=False):
        """Shrinks the scales and biases of c so that its output on x has unit rms (zero-mean
        weights: the benchmark's bias of -8 scale leaves a mean that would add up over K)."""
        c.biases.copy_(-7.5 * c.scales)
        y = verify_matmul(x, c.w, c.scales, c.biases).float()
        parts = (y[:, :c.N // 2], y[:, c.N // 2:]) if halves else (y,)
        for i, part in enumerate(parts):
            rows = slice(i * c.N // len(parts), (i + 1) * c.N // len(parts))
            rms = float(part.pow(2).mean().sqrt())
            c.scales[rows] /= rms
            c.biases[rows] /= rms
        return verify_matmul(x, c.w, c.scales, c.biases)

    x = x0
    for layer in range(layers):  # once, before anything is timed
        qkv, o, gu, down = calls[layer * per_layer:(layer + 1) * per_layer]
        a = unit_gain(qkv, x)[:, :H].contiguous()
        both = unit_gain(gu, unit_gain(o, a), halves=True)
        g, u = both[:, :gu.N // 2], both[:, gu.N // 2:]
        x = unit_gain(down, (g * torch.sigmoid(g)) * u)
    def plan(use_packed):
        gate_up, images = [], []
        for layer in range(layers):
            c = calls[layer * per_layer + 2]
            x_slot = torch.empty((16, c.K), dtype=x0.dtype, device=device)
            if use_packed:
                problem = ChainProblem(x_slot, pack_weights(c.w, c.scales, c.biases, gate_up=True), epilogue="silu_mul")
                images.append([pack_weights(d.w, d.scales, d.biases) if i != 2 else None
                               for i, d in enumerate(calls[layer * per_layer:(layer + 1) * per_layer])])
            else:
                problem = ChainProblem(x_slot, c.w, c.scales, c.biases, epilogue="silu_mul")
            gate_up.append(QmmChain([problem]))

        def product(x, layer, i):
            if use_packed:
                return verify_matmul_packed(x, images[layer][i])
            c = calls[layer * per_layer + i]
            return verify_matmul(x, c.w, c.scales, c.biases)

        def one_pass():
            x = x0
            for layer in range(layers):
                gu = calls[layer * per_layer + 2]
                a = product(x, layer, 0)[:, :H].contiguous()
                o_out = product(a, layer, 1)
                h = torch.empty((16, gu.N // 2), dtype=x0.dtype, device=device)
                chain = gate_up[layer]
                chain.rebind(0, x=o_out, out=h)
                chain()
                x = product(h, layer, 3)
            return x

        return one_pass, gate_up, images

    one_pass, gate_up, images = plan(False)
    eager = one_pass()
    torch.cuda.synchronize()
    if not bool(torch.isfinite(eager.float()).all()):
        raise RuntimeError("dependent layers: activations left the finite range")
    if packed:
        one_pass, gate_up, images = plan(True)
        again = one_pass()
        torch.cuda.synchronize()
        if not torch.equal(again, eager):
            raise RuntimeError("dependent layers: packed weights give other bits than the row-major triples")
    graph, captured = capture(one_pass)
    for r in range(2):
        graph.replay()
        torch.cuda.synchronize()
        if not torch.equal(captured, eager):
            raise RuntimeError(f"dependent layers: graph replay {r} differs from the eager result")
    for _ in range(warmup):
        graph.replay()
    wall_ms, ev_ms = time_region(graph.replay, steps)
    res = dict(launches_per_layer=per_layer, layers=layers, ms_per_step=wall_ms / steps,
               us_per_layer=ev_ms / steps / layers * 1e3, total_bytes=total_bytes,
               frac_hbm=total_bytes / (ev_ms / steps * 1e-3) / HBM_PEAK)
    del graph, captured, eager, calls, gate_up, images, one_pass
    torch.cuda.empty_cache()
    return res


def bench_single_call(device: str, launches: int = 200):
    """config[0]: one 16x4096x4096 call, cold (ring of distinct weight sets larger than
    the 256 MB Infinity Cache) and hot (same weights every launch)."""
    import torch

    from dflash_mlx_amd.verify_qmm import verify_matmul
    from dflash_mlx_amd.workloads import make_qmm_case, qmm_algorithmic_bytes, seed_for

    ring = [make_qmm_case(4096, 4096, seed_for(0) + i, device=device) for i in range(64)]
    _, total = qmm_algorithmic_bytes(4096, 4096)
    out = {}
    for name, cases in (("cold", ring), ("hot", ring[:1])):
        def one_round():
            for i in range(launches):
                c = cases[i % len(cases)]
                verify_matmul(c.x, c.w, c.scales, c.biases)
        g, _ = capture(one_round)
        g.replay()
        _, ev_ms = time_region(g.replay, 3)
        us = ev_ms / 3 / launches * 1e3
        out[name] = dict(us_per_call=us, gbps=total / us / 1e3, frac_hbm=total / (us * 1e-6) / HBM_PEAK)
        del g
    del ring
    torch.cuda.empty_cache()
    return out


def bench_moe(device: str, steps: int, warmup: int, layers: int = 40, join_gate_up: bool = False,
              shared_as_expert: bool = False):
    """config[4]: MoE-shaped verify step at M=16 - 256 experts of intermediate 512 (gate/up
    2048->512, down 512->2048), top-8 routing, gathered per-expert qmm, plus a shared expert
    through verify_matmul; `layers` layers replayed from a HIP graph.  Algorithmic bytes
    count the weights of the experts the seeded routing actually touches.  ``join_gate_up``:
    gate and up, which read the same rows, laid end to end per expert (and for the shared
    expert) and served by one launch each - four launches per layer instead of six.
    ``shared_as_expert`` (with ``join_gate_up``): the shared expert, which has the shape of a
    routed one, stored as expert 256 and its 16 rows appended to the 128 routed pairs - two
    launches per layer, over the same weight bytes."""
    import torch

    from dflash_mlx_amd.verify_qmm import (append_shared_expert, gather_qmm, join_expert_projections,
                                           shared_expert_rows, verify_matmul)
    from dflash_mlx_amd.workloads import MoeCase, QmmCase
    from dflash_mlx_amd.workloads import make_moe_case, make_qmm_case, qmm_algorithmic_bytes, seed_for

    per_expert = 3 * qmm_algorithmic_bytes(2048, 512)[0]
    calls, total = [], 0
    for layer in range(layers):
        gate = make_moe_case(2048, 512, seed_for(4, layer) * 8, device=device)
        up = make_moe_case(2048, 512, seed_for(4, layer) * 8 + 1, device=device)
        up.expert_ids = gate.expert_ids
        down = make_moe_case(512, 2048, seed_for(4, layer) * 8 + 2, device=device)
        down.expert_ids = gate.expert_ids
        shared = [make_qmm_case(2048, 512, seed_for(4, layer) * 8 + 3, device=device),
                  make_qmm_case(2048, 512, seed_for(4, layer) * 8 + 4, device=device),
                  make_qmm_case(512, 2048, seed_for(4, layer) * 8 + 5, device=device)]
        if join_gate_up:
            (w, sc, bi), _ = join_expert_projections((gate.w, gate.scales, gate.biases), (up.w, up.scales, up.biases))
            gate_up = MoeCase(gate.x, gate.expert_ids, w, sc, bi, 64)
            sg, su, sd = shared
            shared_gu = QmmCase(sg.x, torch.cat([sg.w, su.w]), torch.cat([sg.scales, su.scales]),
                                torch.cat([sg.biases, su.biases]), 64)
            if shared_as_expert:
                both = []
                for routed, sh in ((gate_up, shared_gu), (down, sd)):
                    (w, sc, bi), sid = append_shared_expert((routed.w, routed.scales, routed.biases),
                                                            (sh.w, sh.scales, sh.biases))
                    x, ids = shared_expert_rows(routed.x, routed.expert_ids, sh.x, sid)
                    both.append(MoeCase(x, ids, w, sc, bi, 64))
                calls.append((tuple(both), ()))
                del routed, sh, gate_up, shared_gu, sd
            else:
                calls.append(((gate_up, down), (shared_gu, sd)))
            del gate, up, sg, su
        else:
            calls.append(((gate, up, down), tuple(shared)))
        total += (int(torch.unique(down.expert_ids).numel()) + 1) * per_expert
    torch.cuda.synchronize()

    def one_pass():
        out = []
        for gathered, shared in calls:
            for c in gathered:
                out.append(gather_qmm(c.x, c.w, c.scales, c.biases, c.expert_ids, group_size=64))
            for c in shared:
                out.append(verify_matmul(c.x, c.w, c.scales, c.biases))
        return out

    launches_per_layer = len(calls[0][0]) + len(calls[0][1])
    g, _ = capture(one_pass)
    for _ in range(max(1, warmup)):
        g.replay()
    wall_ms, ev_ms = time_region(g.replay, steps)
    ms = wall_ms / steps
    del g, calls
    torch.cuda.empty_cache()
    return dict(layers=layers, launches_per_layer=launches_per_layer,
                ms_per_step=ms, weight_bytes=total, weight_gbps=total / (ms * 1e-3) / 1e9,
                frac_hbm=total / (ms * 1e-3) / HBM_PEAK)


def bench_replay(device: str, steps: int, warmup: int, tape_dtype: str = "bfloat16"):
    """config[2]: 48 layers x 32 value heads, fp32 128x128 state, 16 recorded steps, all
    applied; one launch per rollback.  Four state sets (800 MB) are rotated so that the
    Infinity Cache cannot hold the working set.  ``tape_dtype``: bfloat16 is what a bf16 model's
    forward hands over, float32 what the arena keeps by default."""
    import torch

    from dflash_mlx_amd.cache import KVCache
    from dflash_mlx_amd.kernels import replay_launch
    from dflash_mlx_amd.workloads import make_replay_case, replay_algorithmic_bytes

    L, H, T = 48, 32, 16
    dt = getattr(torch, tape_dtype)
    sets = [make_replay_case(L, steps=T, seed=7000 + i, tape_dtype=dt, device=device) for i in range(4)]
    outs = [torch.empty_like(s.state) for s in sets]
    steps_dev = sets[0].steps

    def one_pass(i):
        c = sets[i % 4]
        replay_launch(c.tape, c.k, c.g, c.state, outs[i % 4], steps=steps_dev, T_alloc=T, slots=L)

    for i in range(max(warmup, 4)):
        one_pass(i)
    n = max(steps * 10, 40)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(n):
        one_pass(i)
    stop.record()
    torch.cuda.synchronize()
    us = start.elapsed_time(stop) / n * 1e3
    total = replay_algorithmic_bytes(128, 128, T, tape_bytes=dt.itemsize) * L * H
    # KV trim of the 16 full-attention layers: offset arithmetic, no device work
    kv = [KVCache() for _ in range(16)]
    for c in kv:
        c.offset = 4096 + 16
    t0 = time.perf_counter_ns()
    for c in kv:
        c.trim(c.offset - (4096 + 7))
    trim_ns = time.perf_counter_ns() - t0
    assert all(c.offset == 4096 + 7 for c in kv)
    del sets, outs
    torch.cuda.empty_cache()
    return dict(us_per_rollback=us, us_per_layer=us / L, gbps=total / us / 1e3,
                frac_hbm=total / (us * 1e-6) / HBM_PEAK, bytes=total, layers=L, heads=H,
                steps=T, tape_dtype=tape_dtype, kv_trim_host_ns_16_layers=trim_ns)


def bench_rollback_per_layer(device: str, steps: int, warmup: int, tape_dtype: str = "float32"):
    """The same rollback as the engine makes it without an arena: 48 ``RecurrentRollbackCache``
    objects, each armed, handed its tape and rolled back on its own (one launch per layer: the
    replay with the conv-state rebuild riding along; dflash_mlx/recurrent_rollback_cache.py:149-171).  Arming and
    recording are reference bookkeeping (no device work) and are left out of the timed region."""
    import torch

    from dflash_mlx_amd.recurrent_rollback_cache import RecurrentRollbackCache
    from dflash_mlx_amd.workloads import make_replay_case, replay_algorithmic_bytes

    L, H, T, D, conv_dim = 48, 32, 16, 128, 3 * 32 * 128
    dt = getattr(torch, tape_dtype)
    case = make_replay_case(L, steps=T, seed=7100, tape_dtype=dt, device=device)
    qkv = torch.randn((L, 1, T, conv_dim), device=device, dtype=torch.bfloat16)
    conv0 = torch.randn((L, 1, 3, conv_dim), device=device, dtype=torch.bfloat16)
    caches = [RecurrentRollbackCache() for _ in range(L)]

    def arm():
        for i, c in enumerate(caches):
            c[0], c[1] = conv0[i], case.state[i]
            c.arm_rollback(prefix_len=4096)
            c.record_tape(tape=case.tape[i], k=case.k[i], g=case.g[i], qkv=qkv[i])

    def rollback():
        for c in caches:
            c.rollback(T - 1)

    for _ in range(max(warmup, 3)):
        arm(); rollback()
    n = max(steps * 3, 20)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev_us = wall_us = 0.0
    for _ in range(n):
        arm()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record()
        rollback()
        stop.record()
        torch.cuda.synchronize()
        wall_us += (time.perf_counter() - t0) * 1e6
        ev_us += start.elapsed_time(stop) * 1e3
    total = replay_algorithmic_bytes(D, D, T, tape_bytes=dt.itemsize) * L * H
    return dict(tape_dtype=tape_dtype, launches_per_rollback=L, us_per_rollback=ev_us / n,
                us_per_layer=ev_us / n / L, host_us_per_rollback=wall_us / n,
                frac_hbm=total / (ev_us / n * 1e-6) / HBM_PEAK, bytes=total)


def bench_gdn_forward(device: str, steps: int, warmup: int):
    """The producer of the tape: GatedDeltaNet forward over a block of 16 tokens with the
    innovation tape recorded, 48 layers x 32 value heads (16 key heads) of 128 x 128 fp32
    state in one launch, bf16 q/k/v.  Algorithmic bytes per value head: the state once in and
    once out, v, y (bf16) and the tape (fp32) once, its share of q and k, g and beta."""
    import torch

    from dflash_mlx_amd import _native
    from dflash_mlx_amd.kernels import _DTYPE_CODE

    lib = _native.lib()
    L, Hk, Hv, T, D = 48, 16, 32, 16, 128
    gen = torch.Generator(device=device).manual_seed(0xDF1A + 2500)
    sets = []
    for _ in range(4):   # four state sets (400 MB): the Infinity Cache cannot hold them
        q = torch.randn((L, T, Hk, D), generator=gen, device=device)
        k = torch.randn((L, T, Hk, D), generator=gen, device=device)
        q = (q / q.norm(dim=-1, keepdim=True) * D ** -0.5).to(torch.bfloat16)
        k = (k / k.norm(dim=-1, keepdim=True)).to(torch.bfloat16)
        v = torch.randn((L, T, Hv, D), generator=gen, device=device).to(torch.bfloat16)
        g = torch.exp(-torch.nn.functional.softplus(torch.randn((L, T, Hv), generator=gen, device=device)))
        beta = torch.sigmoid(torch.randn((L, T, Hv), generator=gen, device=device)).to(torch.bfloat16)
        state = torch.randn((L, Hv, D, D), generator=gen, device=device) * 0.1
        # outputs allocated once: the timed region holds kernel launches only
        outs = (torch.empty_like(state), torch.empty_like(v),
                torch.empty((L, T, Hv, D), dtype=torch.float32, device=device))
        sets.append((q, k, v, g, beta, state) + outs)
    stream = torch.cuda.current_stream(device).cuda_stream

    def one_pass(i):
        q, k, v, g, beta, state, state_out, y, tape = sets[i % 4]
        rc = lib.dflash_gdn_forward_tape(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), beta.data_ptr(),
            state.data_ptr(), state_out.data_ptr(), y.data_ptr(), tape.data_ptr(), None,
            L, T, Hk, Hv, D, D, _DTYPE_CODE[q.dtype], _DTYPE_CODE[g.dtype], _DTYPE_CODE[beta.dtype],
            _DTYPE_CODE[state.dtype], 0, stream)
        _native.check(rc, "dflash_gdn_forward_tape")

    for i in range(max(warmup, 4)):
        one_pass(i)
    n = max(steps * 10, 40)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(n):
        one_pass(i)
    stop.record()
    torch.cuda.synchronize()
    us = start.elapsed_time(stop) / n * 1e3
    per_head = 2 * D * D * 4 + T * (D * 2 + D * 2 + D * 4 + (Hk * 2 * D * 2) // Hv + 4 + 2)
    total = per_head * L * Hv

    # A model's forward reaches this kernel one layer at a time (the rollback, not the forward,
    # covers all layers at once): a launch over the 32 heads of a single layer, replayed from a
    # HIP graph that walks the 48 layers of a state set.
    def one_layer(i):
        q, k, v, g, beta, state, state_out, y, tape = sets[(i // L) % 4]
        l = i % L
        rc = lib.dflash_gdn_forward_tape(
            q[l].data_ptr(), k[l].data_ptr(), v[l].data_ptr(), g[l].data_ptr(), beta[l].data_ptr(),
            state[l].data_ptr(), state_out[l].data_ptr(), y[l].data_ptr(), tape[l].data_ptr(), None,
            1, T, Hk, Hv, D, D, _DTYPE_CODE[q.dtype], _DTYPE_CODE[g.dtype], _DTYPE_CODE[beta.dtype],
            _DTYPE_CODE[state.dtype], 0, torch.cuda.current_stream(device).cuda_stream)
        _native.check(rc, "dflash_gdn_forward_tape")

    graph, _ = capture(lambda: [one_layer(i) for i in range(4 * L)])
    graph.replay()
    _, ev_ms = time_region(graph.replay, 3)
    us_single = ev_ms / 3 / (4 * L) * 1e3
    del graph

    # ... and with the layer's gated output norm: as a launch of its own behind the forward, and
    # computed by the forward's launch (dflash_gdn_forward_tape_norm)
    z = torch.randn((L, T, Hv, D), generator=gen, device=device).to(torch.bfloat16)
    weight = torch.ones(D, dtype=torch.bfloat16, device=device)
    normed = torch.empty_like(z)
    cur = torch.cuda.current_stream

    def one_layer_then_norm(i):
        one_layer(i)
        y, l = sets[(i // L) % 4][7], i % L
        rc = lib.dflash_gdn_gated_norm(y[l].data_ptr(), z[l].data_ptr(), weight.data_ptr(), normed[l].data_ptr(),
                                       T * Hv, D, _DTYPE_CODE[y.dtype], _DTYPE_CODE[weight.dtype], 1e-6,
                                       cur(device).cuda_stream)
        _native.check(rc, "dflash_gdn_gated_norm")

    def one_layer_with_norm(i):
        q, k, v, g, beta, state, state_out, y, tape = sets[(i // L) % 4]
        l = i % L
        rc = lib.dflash_gdn_forward_tape_norm(
            q[l].data_ptr(), k[l].data_ptr(), v[l].data_ptr(), g[l].data_ptr(), beta[l].data_ptr(),
            state[l].data_ptr(), state_out[l].data_ptr(), z[l].data_ptr(), weight.data_ptr(), normed[l].data_ptr(),
            tape[l].data_ptr(), None, 1, T, Hk, Hv, D, D, _DTYPE_CODE[q.dtype], _DTYPE_CODE[g.dtype],
            _DTYPE_CODE[beta.dtype], _DTYPE_CODE[state.dtype], _DTYPE_CODE[weight.dtype], 0, 1e-6,
            cur(device).cuda_stream)
        _native.check(rc, "dflash_gdn_forward_tape_norm")

    timings = {}
    for name, fn in (("then_norm", one_layer_then_norm), ("with_norm", one_layer_with_norm)):
        graph, _ = capture(lambda: [fn(i) for i in range(4 * L)])
        graph.replay()
        _, ev_ms = time_region(graph.replay, 3)
        timings[name] = ev_ms / 3 / (4 * L) * 1e3
        del graph
    del sets
    torch.cuda.empty_cache()
    return dict(us_per_forward=us, us_per_layer=us / L, gbps=total / us / 1e3,
                frac_hbm=total / (us * 1e-6) / HBM_PEAK, bytes=total, layers=L, heads=Hv, steps=T,
                us_per_single_layer_launch=us_single,
                us_per_single_layer_forward_then_norm=timings["then_norm"],
                us_per_single_layer_forward_with_norm=timings["with_norm"])


def bench_gdn_glue(device: str, steps: int, warmup: int):
    """The operators around the recurrence of one GatedDeltaNet layer at the verify shape
    (1 x 16 tokens, 16 key and 32 value heads of 128, conv over 8192 channels): the two fused
    launches through the C ABI (outputs allocated beforehand), the same through the Python
    wrappers (allocations included), and the same operators one by one in torch on the device."""
    import torch

    from dflash_mlx_amd import _native
    from dflash_mlx_amd import gdn_layer as G
    from dflash_mlx_amd.kernels import _DTYPE_CODE

    lib = _native.lib()
    B, S, Hk, Hv, D, K = 1, 16, 16, 32, 128, 4
    C = 2 * Hk * D + Hv * D
    gen = torch.Generator(device=device).manual_seed(0xDF1A + 2600)
    bf = torch.bfloat16
    rnd = lambda *shape: torch.randn(shape, generator=gen, device=device)
    qkv, conv_state, conv_w = rnd(B, S, C).to(bf), rnd(B, K - 1, C).to(bf), (rnd(C, K) * 0.4).to(bf)
    a, b, A_log, dt_bias = rnd(B, S, Hv).to(bf), rnd(B, S, Hv).to(bf), rnd(Hv).to(bf), rnd(Hv).to(bf)
    x, z, w = rnd(B, S, Hv, D).to(bf), rnd(B, S, Hv, D).to(bf), (1 + 0.1 * rnd(D)).to(bf)
    conv_next = torch.empty((B, K - 1, C), dtype=bf, device=device)
    q, k = (torch.empty((B, S, Hk, D), dtype=bf, device=device) for _ in range(2))
    v, y = (torch.empty((B, S, Hv, D), dtype=bf, device=device) for _ in range(2))
    g = torch.empty((B, S, Hv), dtype=torch.float32, device=device)
    beta = torch.empty((B, S, Hv), dtype=bf, device=device)
    stream = torch.cuda.current_stream(device).cuda_stream
    code = _DTYPE_CODE[bf]

    def abi():
        rc = lib.dflash_gdn_prepare(qkv.data_ptr(), conv_state.data_ptr(), conv_w.data_ptr(), a.data_ptr(),
                                    b.data_ptr(), A_log.data_ptr(), dt_bias.data_ptr(), None, conv_next.data_ptr(),
                                    q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), beta.data_ptr(),
                                    B, S, Hk, Hv, D, D, K, code, code, 1e-6, stream)
        rc |= lib.dflash_gdn_gated_norm(x.data_ptr(), z.data_ptr(), w.data_ptr(), y.data_ptr(), B * S * Hv, D,
                                        code, code, 1e-6, stream)
        _native.check(rc, "gdn glue")

    def wrappers():
        G.gdn_prepare(qkv, conv_state, conv_w, a, b, A_log, dt_bias, None, Hk=Hk, Hv=Hv, Dk=D, Dv=D)
        G.gated_norm(x, z, w)

    def array_ops():
        G.gdn_prepare_ops(qkv, conv_state, conv_w, a, b, A_log, dt_bias, None, Hk=Hk, Hv=Hv, Dk=D, Dv=D)
        G.gated_norm_ops(x, z, w)

    out = {}
    n = max(steps * 10, 48)
    for name, fn in (("fused_c_abi", abi), ("fused_python_wrappers", wrappers), ("torch_array_ops", array_ops)):
        for _ in range(max(warmup, 3)):
            fn()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(n):
            fn()
        stop.record()
        torch.cuda.synchronize()
        out[name + "_us_per_layer"] = start.elapsed_time(stop) / n * 1e3
    out["launches_fused"] = 2
    return out


def bench_sdpa(device: str, steps: int, warmup: int, N: int = 4112, L: int = 16, with_torch: bool = True):
    """Attention of the 16-token verify block over the KV caches of config[2]'s full-attention
    layers: 8 key/value heads of 256 over N = 4096 + 16 positions (bf16, read in place from buffers
    of capacity N + 240), 32 query heads, L layers with caches of their own (16 in the model).
    Algorithmic bytes per layer: K and V once, q and out once."""
    import torch

    from dflash_mlx_amd import _native
    from dflash_mlx_amd.kernels import _DTYPE_CODE

    lib = _native.lib()
    B, Hq, Hk, D, cap = 1, 32, 8, 256, N + 240
    bf = torch.bfloat16
    gen = torch.Generator(device=device).manual_seed(0xDF1A + 2700)
    caches = [(torch.randn((B, Hk, cap, D), generator=gen, device=device).to(bf),
               torch.randn((B, Hk, cap, D), generator=gen, device=device).to(bf)) for _ in range(L)]
    q = torch.randn((B, Hq, 16, D), generator=gen, device=device).to(bf)
    out = torch.empty_like(q)
    need = int(lib.dflash_sdpa_q16_workspace_bytes(B, Hq, Hk, N, D))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    stream = torch.cuda.current_stream(device).cuda_stream
    scale = D ** -0.5

    def kernel_pass():
        for kbuf, vbuf in caches:
            rc = lib.dflash_sdpa_q16(q.data_ptr(), kbuf.data_ptr(), vbuf.data_ptr(), None, out.data_ptr(),
                                     ws.data_ptr(), ws.numel(), B, Hq, Hk, N, D, kbuf.stride(0), kbuf.stride(1),
                                     kbuf.stride(2), vbuf.stride(0), vbuf.stride(1), vbuf.stride(2), scale,
                                     _DTYPE_CODE[bf], stream)
            _native.check(rc, "dflash_sdpa_q16")

    allow = (torch.arange(N, device=device)[None, :] <= (N - 16 + torch.arange(16, device=device))[:, None])

    def torch_pass():
        for kbuf, vbuf in caches:
            torch.nn.functional.scaled_dot_product_attention(q, kbuf[:, :, :N], vbuf[:, :, :N], attn_mask=allow,
                                                             scale=scale, enable_gqa=True)

    res = {}
    for name, fn in (("kernel", kernel_pass), ("torch_sdpa", torch_pass))[:2 if with_torch else 1]:
        for _ in range(max(warmup, 2)):
            fn()
        n = max(steps, 5)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(n):
            fn()
        stop.record()
        torch.cuda.synchronize()
        res[name + "_us_per_layer"] = start.elapsed_time(stop) / n / L * 1e3
    per_layer = 2 * B * Hk * N * D * 2 + 2 * B * Hq * 16 * D * 2
    us = res["kernel_us_per_layer"]
    res.update(bytes_per_layer=per_layer, gbps=per_layer / us / 1e3, frac_hbm=per_layer / (us * 1e-6) / HBM_PEAK,
               workspace_bytes=need, layers=L, kv_len=N)
    del caches
    torch.cuda.empty_cache()
    return res


def bench_cpu_baseline(stack: str, budget_s: float = 12.0):
    """The oracle's C port of the reference kernel arithmetic (bf16-rounded dequantised
    weights, fp32 accumulation) on the host cores: whole layers of the same stack, one
    after the other, until the time budget is used up."""
    from dflash_mlx_amd.workloads import make_qmm_case, qmm_algorithmic_bytes, seed_for, stack_linears
    from oracle.c_binding import load_c_oracle
    import numpy as np
    import torch

    orc = load_c_oracle(build_if_missing=True)
    linears, layers, cfg = stack_linears(stack)
    done_bytes, spent, n_layers = 0, 0.0, 0
    for layer in range(layers):
        for i, (name, K, N) in enumerate(linears):
            c = make_qmm_case(K, N, seed_for(cfg, layer) * 8 + i)
            args = (c.x.view(torch.int16).numpy().view(np.uint16), c.w.numpy().view(np.uint32),
                    c.scales.view(torch.int16).numpy().view(np.uint16),
                    c.biases.view(torch.int16).numpy().view(np.uint16), 64)
            t0 = time.perf_counter()
            orc.qmm_m16(*args, flavour=1, k_parts=1)
            spent += time.perf_counter() - t0
            done_bytes += qmm_algorithmic_bytes(K, N)[0]
        n_layers += 1
        if spent > budget_s:
            break
    return dict(value=round(done_bytes / spent / 1e9, 3), unit="GB/s", cores=orc.num_threads(), kind="port",
                sample=f"{n_layers} of {layers} layers of the {stack} stack ({done_bytes / 1e9:.2f} GB of "
                       f"weights in {spent:.1f} s of compute; input generation not timed), C/OpenMP port "
                       f"of the reference kernel arithmetic")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="27b", choices=["27b", "9b"])
    ap.add_argument("--skip-cpu", action="store_true", help="leave out the cpu_baseline leg")
    ap.add_argument("--skip-extra", action="store_true", help="only the headline stack")
    ap.add_argument("--legs", default="", help="comma-separated subset of the extra measurements to run "
                                               f"(default all): {', '.join(LEGS)}")
    ap.add_argument("--packed-weights", action="store_true",
                    help="headline stack through verify_matmul_packed (weights stored in the streaming "
                         "kernel's order); off by default: the headline uses the reference's operands")
    ap.add_argument("--kernel-sources-sha256", action="store_true",
                    help="print the hash a counter summary under profiles/ has to state, and exit")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run three 1 GiB device-to-device copies (a kernel of known traffic, "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings) and exit")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the verify hot path is a single-device path and this "
              "build has no multi-GPU leg; run with --gpus 1", file=sys.stderr)
        return 2

    if args.kernel_sources_sha256:
        print(kernel_sources_sha256())
        return 0

    import torch

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").random_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": 1 << 30, "copy_bytes_written": 1 << 30, "copies": 3}))
        return 0

    import dflash_mlx_amd._native as nat

    nat.lib()  # no library, no benchmark: there is no fallback path to time
    os.environ["DFLASH_VERIFY_QMM"] = "1"
    os.environ.pop("DFLASH_VERIFY_VARIANT", None)
    device = "cuda:0"
    torch.cuda.set_device(0)

    main_res = bench_qmm_stack(args.workload, args.steps, args.warmup, device, packed=args.packed_weights)
    log(f"[bench] {args.workload}: {main_res['ms_per_step']:.3f} ms/step, "
        f"{main_res['weight_gbps']:.0f} GB/s weights, {main_res['avg_launch_us']:.2f} us/launch")
    extra = {}
    rnd = lambda d: {k: (round(v, 4) if isinstance(v, float) else v) for k, v in d.items()}  # noqa: E731
    legs = set() if args.skip_extra else set(args.legs.split(",")) if args.legs else set(LEGS)
    if legs - set(LEGS):
        print(f"unknown --legs {sorted(legs - set(LEGS))}; known: {', '.join(LEGS)}", file=sys.stderr)
        return 2
    if "other_stack" in legs:
        other = "9b" if args.workload == "27b" else "27b"
        o = bench_qmm_stack(other, args.steps, args.warmup, device)
        extra[f"stack_{other}"] = dict(ms_per_step=round(o["ms_per_step"], 4),
                                       weight_gbps=round(o["weight_gbps"], 1),
                                       frac_hbm=round(o["total_bytes"] / (o["event_ms_per_step"] * 1e-3) / HBM_PEAK, 4))
    if "dependent" in legs:
        dep = bench_dependent_layers(args.workload, args.steps, args.warmup, device)
        log(f"[bench] {args.workload} stack, every launch waiting for the one before: {dep['ms_per_step']:.3f} ms/step, "
            f"{dep['us_per_layer']:.2f} us/layer, {dep['frac_hbm']:.3f} of peak")
        extra[f"stack_{args.workload}_dependent_layer"] = rnd(dep)
        dep = bench_dependent_layers(args.workload, args.steps, args.warmup, device, packed=True)
        log(f"[bench] {args.workload} stack, every launch waiting for the one before, packed weights: "
            f"{dep['ms_per_step']:.3f} ms/step, {dep['us_per_layer']:.2f} us/layer, {dep['frac_hbm']:.3f} of peak")
        extra[f"stack_{args.workload}_dependent_layer_packed_weights"] = rnd(dep)
    stack_variants = []
    if "gate_up" in legs:
        stack_variants.append(("gate_up_in_one_launch", dict(join_gate_up=True)))
    if "packed" in legs:
        stack_variants += [("packed_weights", dict(packed=True)),
                           ("gate_up_in_one_launch_packed_weights", dict(packed=True, join_gate_up=True))]
    for label, kw in stack_variants:
        q = bench_qmm_stack(args.workload, args.steps, args.warmup, device, **kw)
        log(f"[bench] {args.workload} stack, {label}: {q['ms_per_step']:.3f} ms/step")
        extra[f"stack_{args.workload}_{label}"] = dict(
            calls_per_step=q["calls_per_step"], ms_per_step=round(q["ms_per_step"], 4),
            weight_gbps=round(q["weight_gbps"], 1), avg_launch_us=round(q["avg_launch_us"], 3),
            frac_hbm=round(q["total_bytes"] / (q["event_ms_per_step"] * 1e-3) / HBM_PEAK, 4))
    if "chain" in legs:
        for n_layers in (1, 3):
            ch = bench_qmm_chain_stack(args.workload, args.steps, args.warmup, device, layers_per_launch=n_layers)
            log(f"[bench] {args.workload} stack, {n_layers} layer(s) per chained launch: {ch['ms_per_step']:.3f} ms/step, "
                f"{ch['us_per_layer']:.2f} us/layer")
            extra[f"stack_{args.workload}_chained_{n_layers}_layer_per_launch"] = rnd(ch)
        for n_layers in (1, 4):
            ch = bench_qmm_chain_stack(args.workload, args.steps, args.warmup, device, layers_per_launch=n_layers,
                                       join_gate_up=True)
            log(f"[bench] {args.workload} stack, {n_layers} layer(s) per chained launch, gate/up as one problem: "
                f"{ch['ms_per_step']:.3f} ms/step, {ch['us_per_layer']:.2f} us/layer")
            extra[f"stack_{args.workload}_chained_{n_layers}_layer_per_launch_gate_up_as_one_problem"] = rnd(ch)
        for n_layers, join in ((1, False), (3, False), (4, True)):
            ch = bench_qmm_chain_stack(args.workload, args.steps, args.warmup, device, layers_per_launch=n_layers,
                                       join_gate_up=join, joint_split=True)
            name = f"stack_{args.workload}_chained_{n_layers}_layer_per_launch" + ("_gate_up_as_one_problem" if join else "")
            log(f"[bench] {name}, units of a launch divided as one range: {ch['ms_per_step']:.3f} ms/step, "
                f"{ch['us_per_layer']:.2f} us/layer, {ch['frac_hbm']:.3f} of peak")
            extra[name + "_joint_split"] = rnd(ch)
        ch = bench_qmm_chain_stack(args.workload, args.steps, args.warmup, device, layers_per_launch=4, join_gate_up=True,
                                   joint_split=True, packed=True)
        log(f"[bench] {args.workload} stack, 4 layers per chained launch, gate/up as one problem, joint split, packed "
            f"weights: {ch['ms_per_step']:.3f} ms/step, {ch['us_per_layer']:.2f} us/layer, {ch['frac_hbm']:.3f} of peak")
        extra[f"stack_{args.workload}_chained_4_layer_per_launch_gate_up_as_one_problem_joint_split_packed_weights"] = rnd(ch)
        other = "9b" if args.workload == "27b" else "27b"
        ch = bench_qmm_chain_stack(other, args.steps, args.warmup, device, layers_per_launch=3, join_gate_up=True)
        log(f"[bench] {other} stack, 3 layers per chained launch, gate/up as one problem: {ch['ms_per_step']:.3f} ms/step, "
            f"{ch['frac_hbm']:.3f} of peak")
        extra[f"stack_{other}_chained_3_layer_per_launch_gate_up_as_one_problem"] = rnd(ch)
        ch = bench_qmm_chain_stack(other, args.steps, args.warmup, device, layers_per_launch=4, join_gate_up=True,
                                   joint_split=True)
        log(f"[bench] {other} stack, 4 layers per chained launch, gate/up as one problem, units divided as one range: "
            f"{ch['ms_per_step']:.3f} ms/step, {ch['frac_hbm']:.3f} of peak")
        extra[f"stack_{other}_chained_4_layer_per_launch_gate_up_as_one_problem_joint_split"] = rnd(ch)
    if "mlp" in legs:
        mlp = bench_mlp_chain(args.workload, args.steps, args.warmup, device)
        extra[f"mlp_{args.workload}"] = {k: (rnd(v) if isinstance(v, dict) else round(v, 6)) for k, v in mlp.items()}
        log("[bench] mlp: " + ", ".join(f"{k} {v['us_per_layer']:.2f} us/layer" for k, v in mlp.items() if isinstance(v, dict)))
    if "single" in legs:
        extra["single_call_16x4096x4096"] = {k: rnd(v) for k, v in bench_single_call(device).items()}
    if "moe" in legs:
        mo = bench_moe(device, args.steps, args.warmup)
        extra["moe_35b_a3b_stack"] = rnd(mo)
        log(f"[bench] moe: {mo['ms_per_step']:.3f} ms/step, {mo['weight_gbps']:.0f} GB/s")
        extra["moe_35b_a3b_stack_gate_up_in_one_launch"] = rnd(bench_moe(device, args.steps, args.warmup, join_gate_up=True))
        ms = bench_moe(device, args.steps, args.warmup, join_gate_up=True, shared_as_expert=True)
        log(f"[bench] moe stack, shared expert stored as expert 256: {ms['ms_per_step']:.3f} ms/step")
        extra["moe_35b_a3b_stack_shared_expert_in_the_gathered_launch"] = rnd(ms)
    if "replay" in legs:
        rp = bench_replay(device, args.steps, args.warmup)
        extra["gdn_tape_replay"] = rnd(rp)
        log(f"[bench] replay: {rp['us_per_layer']:.3f} us/layer, {rp['gbps']:.0f} GB/s")
        extra["gdn_tape_replay_fp32_tape"] = rnd(bench_replay(device, args.steps, args.warmup, tape_dtype="float32"))
        for dt in ("float32", "bfloat16"):
            pl = bench_rollback_per_layer(device, args.steps, args.warmup, tape_dtype=dt)
            log(f"[bench] rollback through 48 per-layer caches ({dt} tape): {pl['us_per_rollback']:.1f} us on the device, "
                f"{pl['host_us_per_rollback']:.1f} us on the host")
            extra[f"gdn_rollback_per_layer_cache_{dt}_tape"] = rnd(pl)
    if "forward" in legs:
        fw = bench_gdn_forward(device, args.steps, args.warmup)
        log(f"[bench] forward with tape: {fw['us_per_layer']:.3f} us/layer, {fw['gbps']:.0f} GB/s")
        extra["gdn_forward_with_tape"] = rnd(fw)
    if "sdpa" in legs:
        extra["sdpa_q16_kv4112"] = rnd(bench_sdpa(device, args.steps, args.warmup))
        extra["sdpa_q16_kv32784"] = rnd(bench_sdpa(device, args.steps, args.warmup, N=32784, with_torch=False))
    if "glue" in legs:
        extra["gdn_layer_glue"] = {k: (round(v, 3) if isinstance(v, float) else v)
                                   for k, v in bench_gdn_glue(device, args.steps, args.warmup).items()}

    achieved = main_res["bytes_per_launch"] / (main_res["avg_launch_us"] * 1e-6) / 1e9
    traffic, traffic_source = (None, "packed weights: see the profile summary") if args.packed_weights \
        else measured_traffic(args.workload)
    roofline = dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK / 1e9, unit="GB/s",
                    frac=round(achieved * 1e9 / HBM_PEAK, 4),
                    traffic=traffic, traffic_source=traffic_source,
                    kernel="qmm_stream_kernel", bytes_per_launch=round(main_res["bytes_per_launch"]),
                    avg_launch_us=round(main_res["avg_launch_us"], 3))
    cpu = None if args.skip_cpu else bench_cpu_baseline(args.workload)

    out = {
        "metric": "verify_qmm M=16 GB/s (% HBM peak); GDN tape-replay us/layer at 16 steps",
        "value": round(main_res["weight_gbps"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_res["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 x int4 (fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}-shaped dense int4 verify stack, M=16, group 64, "
                               f"{main_res['calls_per_step']} verify_matmul calls per step (HIP graph replay)"
                               + (", packed weights" if args.packed_weights else ""),
                   "weight_bytes_per_step": main_res["weight_bytes"],
                   "eager_ms_per_step": round(main_res["eager_ms_per_step"], 3)},
        "pct_hbm_peak": round(100.0 * main_res["weight_gbps"] * 1e9 / HBM_PEAK, 2),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
