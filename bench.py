#!/usr/bin/env python3
"""Benchmark of the sparse MoE block on one MI355X.

Default workload: the Q4_K OLMoE-shaped layer at decode batch 1 (hidden 2048, 64 experts,
top-8, SwiGLU intermediate 1024, f16 router, norm_topk_prob=false) - the configuration the
headline metric is quoted on.  A "step" is one forward of one MoE layer over one batch of
tokens, inputs and weights already resident in HBM.  Steps rotate over `--layers` distinct
layer banks (16 x 226.5 MB) and over a pool of distinct tokens, so that no step finds its
expert weights in the 256 MB Infinity Cache from an earlier step: a layer is revisited only
after the other 15 have streamed >= 425 MB through the cache.  What a step does find warm is its
256 KB router: the library's one-launch decode form reads the router of the layer after its own ahead
while it ends (what a decode loop that walks the layers in order calls next, and what these
steps do); MUMMU_WARM_NEXT=0 in the environment measures without that (`config.warm_next_router`).

The timed steps are replays of a HIP graph that holds one rotation (or the whole timed region,
if that is shorter) - the serving-loop form; they start where the warm-up steps stopped, so no
(layer, token batch) pair of the warm-up is read again.  --no-graph times eager launches instead.
`steady` adds the median and p10 / p90 of the per-layer time over >= 200 event-timed replays.

Prints ONE JSON line (the contract the round driver reads), including
  roofline      the dominant kernel against the 8 TB/s HBM peak: its duration is the median of the
                event-timed graph replays per layer, less the layer's other launches (their eager
                event-bound averages); `avg_launch_us_eager` is the kernel's own event-bound average in
                eager launches, and `layer_frac` the whole layer's algorithmic bytes over the layer time,
  cpu_baseline  the CPU oracle (a C restatement of the reference's routed CPU path) timed on
                this host on a bounded sample of the same workload.

Two other modes print a JSON line of their own instead: --probe-read (what a read-only kernel streams on
this GPU) and --packed-gemv K,N,BITS,ROWS (the packed-GEMV op, microseconds per call).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# kernel-timing slot -> name of the kernel in the rocprofv3 summaries
PROFILE_KERNEL_NAMES = {"gate_up": ("gate_up_fused_kernel", "gate_up_q_kernel"), "down_combine": ("down_combine_q_kernel",),
                        "decode_layer": ("decode_layer_kernel",)}


def profiled_traffic(workload, tokens, slot):
    """HBM bytes per launch of the dominant kernel, read from the committed summary of the rocprofv3 FETCH_SIZE /
    WRITE_SIZE counter runs of this same command (profiles/<workload>_hbm_traffic.txt, column "traffic B": each
    counter scaled by what it reads for the library's 256 MiB copy kernel).  None for a workload or batch size
    no summary was taken on."""
    path = os.path.join(ROOT, "profiles", f"{workload}_hbm_traffic.txt" if tokens == 1 else f"{workload}_bt{tokens}_hbm_traffic.txt")
    names = PROFILE_KERNEL_NAMES.get(slot)
    if names is None or not os.path.exists(path):
        return None
    column = None
    for line in open(path):
        if line.startswith("kernel ") and "traffic B" in line:
            head = line.split("  ")
            column = [c.strip() for c in head if c.strip()].index("traffic B")
        elif column is not None and line.startswith(names):
            # the kernel name holds template arguments with spaces: count the numeric fields from the right
            fields = line[line.index(">") + 1:].split() if ">" in line else line.split()[1:]
            return int(float(fields[column - 1]))
    return None


WORKLOADS = {
    # name: (hidden, inter, experts, top_k, norm, bank type, router type)
    "olmoe_q4k_decode": dict(hidden=2048, inter=1024, experts=64, top_k=8, norm=False, bank="Q4_K", router="F16"),
    "olmoe_q8_0_decode": dict(hidden=2048, inter=1024, experts=64, top_k=8, norm=False, bank="Q8_0", router="F16"),
    "olmoe_q6k_decode": dict(hidden=2048, inter=1024, experts=64, top_k=8, norm=False, bank="Q6_K", router="F16"),
    "olmoe_f16_decode": dict(hidden=2048, inter=1024, experts=64, top_k=8, norm=False, bank="F16", router="F16"),
    "olmoe_bf16_decode": dict(hidden=2048, inter=1024, experts=64, top_k=8, norm=False, bank="BF16", router="F16"),
    "olmoe_f32_decode": dict(hidden=2048, inter=1024, experts=64, top_k=8, norm=False, bank="F32", router="F16"),
    "qwen3_a3b_q4k": dict(hidden=2048, inter=768, experts=128, top_k=8, norm=True, bank="Q4_K", router="F16"),
    # mixed bank types: llama.cpp's Q4_K_M recipe stores part of ffn_down as Q6_K; the shipped qwen4exp file has
    # Q4_K gate/up with Q5_1 downs, 512 experts, top-10 (models/qwen4exp/mod.rs:18-20, experts.rs:1838-1879)
    "olmoe_q4km_decode": dict(hidden=2048, inter=1024, experts=64, top_k=8, norm=False, bank="Q4_K", down="Q6_K", router="F16"),
    "qwen4exp_decode": dict(hidden=2560, inter=640, experts=512, top_k=10, norm=True, bank="Q4_K", down="Q5_1", router="F16",
                            flavour=1),
}
BANK_TYPES = {"Q4_K": 12, "Q8_0": 8, "F16": 1, "F32": 0, "Q6_K": 14, "Q5_1": 7, "Q5_K": 13, "BF16": 30}


def probe_read(M) -> int:
    """Times the library's read-only stream (mummu_probe_read) over a gate + up bank of the OLMoE Q4_K shape
    (64 experts x 1024 rows x 1152 bytes, twice: 151 MB), rotating over three such banks so that no launch finds its
    bytes in the 256 MB Infinity Cache: front to back, and 128 / 64 / 32 bytes of each of a workgroup's 128 rows per
    step (32 is what a 64-element K step of the grouped GEMM asks of a Q4_K row)."""
    row_bytes, rows = 1152, 2 * 64 * 1024
    bank = rows * row_bytes
    banks, reps = 3, 30
    buf = M.DeviceBuffer(banks * bank)
    buf.upload(np.zeros(banks * bank // 8, dtype=np.int64))
    out = {"metric": "read-only stream over a 151 MB bank (no compute)", "unit": "TB/s", "bytes_per_launch": bank,
           "row_bytes": row_bytes, "rows_per_workgroup": 128, "launches_timed": reps, "patterns": {}}
    with M.SparseMoe(M.SparseMoeConfig(64, 64, 2, 1), max_tokens=1) as moe:
        for piece in (0, 128, 64, 32):
            for i in range(banks):
                M.probe_read(buf, bank, row_bytes, piece, moe.stream, offset=i * bank)
            moe.timer_start()
            for i in range(reps):
                M.probe_read(buf, bank, row_bytes, piece, moe.stream, offset=(i % banks) * bank)
            ms = moe.timer_stop()
            us = ms * 1e3 / reps
            out["patterns"]["front_to_back" if piece == 0 else f"{piece}_bytes_per_row_and_step"] = {
                "us_per_launch": round(us, 2), "tb_per_s": round(bank / (us * 1e-6) / 1e12, 3)}
    best = max(v["tb_per_s"] for v in out["patterns"].values())
    out["value"] = best
    out["of_8_tb_per_s"] = round(best / 8.0, 3)
    print(json.dumps(out))
    return 0


def packed_gemv(M, lib, synth, spec: str) -> int:
    """Times the packed-GEMV op (Q4GemvOps::q4s_gemv, nn/packed_gemv.rs) with device-resident inputs:
    `--packed-gemv K,N,BITS,ROWS[,REPS]` (5120,17408,4,1 is the Q4S weight the reference quotes).  Several copies of the
    weight are used in rotation so that no call finds its weight in the 256 MB cache.  Prints one JSON line:
    wall-clock microseconds per call (two launches: the product and the sum over the K split) and the packed bytes
    (values + scales) per second."""
    parts = [int(v) for v in spec.split(",")]
    if len(parts) not in (4, 5) or parts[2] not in (4, 8):
        print("bench.py: --packed-gemv takes K,N,BITS,ROWS[,REPS] with BITS 4 or 8", file=sys.stderr)
        return 2
    k, n, bits, rows = parts[:4]
    reps = parts[4] if len(parts) == 5 else 50
    g = np.random.Generator(np.random.PCG64(1))
    lim = 1 << (bits - 1)
    codes = g.integers(-lim, lim, (k, n), dtype=np.int8)
    scales = g.uniform(0.001, 0.01, (k, n // 32)).astype(np.float32)
    words = synth.pack_words(codes, bits)
    copies = max(1, min(8, int(600e6 // (words.nbytes + scales.nbytes))))
    weights = [M.PackedWeight(words, scales, k, n, bits) for _ in range(copies)]
    x = g.standard_normal((rows, k)).astype(np.float32)
    xd, yd = M.DeviceBuffer.from_array(x), M.DeviceBuffer(4 * rows * n)
    for w in weights:
        w.gemv_device(xd, rows, yd)
    lib.mummu_device_synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        for w in weights:
            w.gemv_device(xd, rows, yd)
    lib.mummu_device_synchronize()
    dt = (time.perf_counter() - t0) / (reps * copies)
    nbytes = weights[0].resident_bytes()
    print(json.dumps({"op": "q4s_gemv", "k": k, "n": n, "value_bits": bits, "rows": rows,
                      "us_per_call": round(dt * 1e6, 2), "packed_bytes": nbytes, "gb_per_s": round(nbytes / dt / 1e9, 1),
                      "weight_copies": copies, "calls": reps * copies}))
    for w in weights:
        w.close()
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4096)
    ap.add_argument("--warmup", type=int, default=256)
    ap.add_argument("--workload", default="olmoe_q4k_decode", choices=sorted(WORKLOADS))
    ap.add_argument("--tokens", type=int, default=1, help="tokens per step (decode batch)")
    ap.add_argument("--layers", type=int, default=16, help="distinct layer banks the steps rotate over")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--stack", action="store_true",
                    help="a step is x <- x + MoE_l(RmsNorm_l(x)) through all --layers layers (reported per layer)")
    ap.add_argument("--shared-inter", type=int, default=0,
                    help="also give every layer a shared expert of this intermediate width with a sigmoid gate "
                         "(Qwen-style block; same bank types); the CPU baseline leg is skipped")
    ap.add_argument("--no-steady", action="store_true",
                    help="leave out the event-timed replays behind `steady` (rocprofv3's kernel trace has crashed inside "
                         "hipGraphLaunch between event records; the profile commands pass this)")
    ap.add_argument("--no-deferred-combine", action="store_true",
                    help="decode steps that take the one-launch form: enqueue the sum over a token's eight weighted rows as a launch "
                         "of its own after every step, instead of leaving it to the launch of the next step (see "
                         "mummu_moe_set_deferred_combine)")
    ap.add_argument("--tile-order", action="store_true",
                    help="several tokens per step: order the decode workgroups so that tokens sharing an expert fetch its rows "
                         "once, from two tokens on (mummu_moe_set_tile_order; by default the library does so from six tokens "
                         "on, where it is also the faster order)")
    ap.add_argument("--no-tile-order", action="store_true", help="never order the decode workgroups that way")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--probe-read", action="store_true",
                    help="instead of the workload: what a read-only kernel streams on this GPU (a ceiling for the roofline's "
                         "achieved figure), one JSON line")
    ap.add_argument("--packed-gemv", default=None, metavar="K,N,BITS,ROWS[,REPS]",
                    help="instead of the workload: time the packed-GEMV op on a [K, N] weight of 4- or 8-bit values, "
                         "one JSON line")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus must be 1 "
              "(sharding the experts over several GPUs is a design note of this library, not built).", file=sys.stderr)
        return 2

    from mummu_amd import _lib, moe as M, synth

    if _lib.device_count() < 1:
        print("bench.py: no HIP device", file=sys.stderr)
        return 3

    if args.probe_read:
        return probe_read(M)
    if args.packed_gemv:
        return packed_gemv(M, _lib.load(), synth, args.packed_gemv)

    w = WORKLOADS[args.workload]
    H, I, E, k, norm = w["hidden"], w["inter"], w["experts"], w["top_k"], w["norm"]
    bank_t = BANK_TYPES[w["bank"]]
    down_t = BANK_TYPES[w.get("down", w["bank"])]
    router_t = M.F16
    n = args.tokens
    L = args.layers

    def bank_bytes(in_dim, out_dim):
        return E * out_dim * synth.row_bytes(bank_t, in_dim)

    g = np.random.Generator(np.random.PCG64(args.seed))

    def make_bank(in_dim, out_dim, seed, t=None):
        t = bank_t if t is None else t
        if t not in (M.F16, M.F32, M.BF16):
            return synth.random_bank_fast(t, [in_dim, out_dim, E], seed)
        gg = np.random.Generator(np.random.PCG64(seed))
        w32 = gg.standard_normal(E * out_dim * in_dim, dtype=np.float32) * np.float32(0.02)
        if t == M.BF16:
            return (w32.view(np.uint32) >> np.uint32(16)).astype(np.uint16).view(np.uint8)  # (truncated: statistics only)
        return (w32 if t == M.F32 else w32.astype(np.float16)).view(np.uint8)

    def make_bank_1(ne, seed, t):
        gg = np.random.Generator(np.random.PCG64(seed))
        w32 = gg.standard_normal(ne[0] * ne[1] * ne[2], dtype=np.float32) * np.float32(0.02)
        if t == M.BF16:
            return (w32.view(np.uint32) >> np.uint32(16)).astype(np.uint16).view(np.uint8)
        return (w32 if t == M.F32 else w32.astype(np.float16)).view(np.uint8)

    t_setup = time.time()
    moe = M.SparseMoe(M.SparseMoeConfig(H, I, E, k), num_layers=L, max_tokens=max(n, 8), norm_topk_prob=norm,
                      router_flavour=w.get("flavour", 0))
    deferred = not args.no_deferred_combine and not args.stack and not args.shared_inter
    moe.set_deferred_combine(deferred)
    tile_order = True if args.tile_order else (False if args.no_tile_order else None)
    moe.set_tile_order(tile_order)
    routers = []
    keep_layer0 = None
    for l in range(L):
        router = (g.standard_normal((E, H), dtype=np.float32) * np.float32(0.02)).astype(np.float16)
        gate = make_bank(H, I, args.seed * 1000 + 3 * l)
        up = make_bank(H, I, args.seed * 1000 + 3 * l + 1)
        down = make_bank(I, H, args.seed * 1000 + 3 * l + 2, down_t)
        moe.load_layer(l, router, router_t, gate, bank_t, up, bank_t, down, down_t, np.ones(H, np.float32) if args.stack else None)
        if args.shared_inter:
            IS = args.shared_inter
            sh = [synth.random_bank_fast(t_, ne, args.seed * 7000 + 3 * l + j) if t_ not in (M.F16, M.F32, M.BF16) else
                  make_bank_1(ne, args.seed * 7000 + 3 * l + j, t_)
                  for j, (t_, ne) in enumerate(((bank_t, [H, IS, 1]), (bank_t, [H, IS, 1]), (down_t, [IS, H, 1])))]
            gate_vec = (g.standard_normal(H, dtype=np.float32) * np.float32(0.05)).astype(np.float32)
            moe.load_shared_expert(l, IS, sh[0], bank_t, sh[1], bank_t, sh[2], down_t, gate_vec)
        routers.append(router)
        if l == 0:
            keep_layer0 = (router, gate, up, down)
    # a pool of distinct token batches: routing differs from step to step
    pool = 64
    xs = g.standard_normal((pool, n, H), dtype=np.float32)
    x_dev = [M.DeviceBuffer.from_array(xs[i]) for i in range(pool)]
    out_dev = M.DeviceBuffer(n * H * 4)
    setup_s = time.time() - t_setup

    expert_bytes = 2 * I * synth.row_bytes(bank_t, H) + H * synth.row_bytes(down_t, I)
    gate_up_expert_bytes = 2 * I * synth.row_bytes(bank_t, H)
    router_bytes = E * H * 2

    # distinct experts per step, from the actual routing of every (layer, token batch) pair used
    period = int(L * pool // np.gcd(L, pool))
    distinct = {}
    for s in range(min(period, L * pool)):
        l, p = s % L, s % pool
        if (l, p) in distinct:
            continue
        r = moe.route(xs[p], k, norm, layer=l)
        distinct[(l, p)] = len(np.unique(r.ids))
    mean_distinct = float(np.mean(list(distinct.values())))

    def step(s):
        if args.stack:
            moe.stack_forward_device(x_dev[s % pool], n, k, norm, out_dev)
        else:
            moe.forward_device(s % L, x_dev[s % pool], n, k, norm, out_dev)

    use_graph = not args.no_graph
    layers_per_step = L if args.stack else 1
    rotation = min(pool, 16) if args.stack else period  # steps after which the (layer, token batch) sequence repeats
    first = args.warmup  # the timed steps go on where the warm-up stopped: none of its (layer, token batch) pairs is re-read

    def capture(s_begin, count):
        moe.graph_begin()
        for s in range(s_begin, s_begin + count):
            step(s)
        return moe.graph_end()

    # The timed region is EXACTLY args.steps steps: whole replays of one graph holding `per_graph` consecutive steps,
    # plus one replay of a shorter graph for what is left over.  A graph is never longer than the timed region, so
    # a short run (--steps 20) is still a graph replay.
    per_graph = max(1, min(rotation if rotation <= 1024 else L, args.steps))
    graph = tail_graph = None
    replays, left = divmod(args.steps, per_graph)
    if use_graph:
        graph = capture(first, per_graph)
        tail_graph = capture(first + replays * per_graph, left) if left else None

    def timed_steps():
        if graph is not None:
            for _ in range(replays):
                graph.launch()
            if tail_graph is not None:
                tail_graph.launch()
        else:
            for s in range(first, first + args.steps):
                step(s)

    # one plain copy of known size on the same stream (untimed): under `rocprofv3 --pmc
    # FETCH_SIZE` / `WRITE_SIZE` its dispatch calibrates the counters the roofline's `traffic`
    # figure is scaled by
    probe_bytes = 256 << 20
    probe_src, probe_dst = M.DeviceBuffer(probe_bytes), M.DeviceBuffer(probe_bytes)
    M.probe_copy(probe_dst, probe_src, probe_bytes, moe.stream)
    M.synchronize()
    del probe_src, probe_dst

    # warm-up: args.warmup eager steps (steps 0 .. warmup-1), then, untimed, one replay of each graph so that its
    # first-launch upload is not inside the timed region.  That replay reads the same pairs as the timed one will,
    # per_graph steps earlier: with every step streaming `layer_bytes` of distinct weights, what a step needs has
    # been pushed out of the 256 MB Infinity Cache again when (per_graph - 1) * layer_bytes exceeds it (`cache_cold`).
    for s in range(args.warmup):
        step(s)
    if graph is not None:
        graph.launch()
        if tail_graph is not None:
            tail_graph.launch()
    M.synchronize()
    moe.check()
    moe.timer_start()
    t0 = time.perf_counter()
    timed_steps()
    ev_ms = moe.timer_stop()
    M.synchronize()
    wall = time.perf_counter() - t0
    moe.check()

    ms_per_step = wall * 1e3 / args.steps / layers_per_step  # per layer
    value = n * args.steps * layers_per_step / wall

    # steady state: >= 200 replays of a graph over one whole rotation, each replay timed on the device between two
    # HIP events (no host synchronisation in between): median and p10 / p90 of the per-layer time
    steady = None
    if use_graph and not args.no_steady:
        rot_graph = graph if per_graph == rotation else capture(first, min(rotation, 1024))
        rot_steps = per_graph if per_graph == rotation else min(rotation, 1024)
        reps = max(200, -(-2048 // rot_steps))
        rot_graph.launch()
        M.synchronize()
        us = np.sort(rot_graph.launch_timed(reps).astype(np.float64)) * 1e3 / (rot_steps * layers_per_step)
        moe.check()
        steady = {"steps": reps * rot_steps, "replays": reps, "steps_per_replay": rot_steps,
                  "us_per_layer_p10": round(float(np.percentile(us, 10)), 3), "us_per_layer_p50": round(float(np.percentile(us, 50)), 3),
                  "us_per_layer_p90": round(float(np.percentile(us, 90)), 3), "us_per_layer_min": round(float(us[0]), 3),
                  "us_per_layer_max": round(float(us[-1]), 3)}
        if rot_graph is not graph:
            rot_graph.close()

    layers_per_step = L if args.stack else 1
    ms_per_step = wall * 1e3 / args.steps / layers_per_step  # per layer
    value = n * args.steps * layers_per_step / wall

    # per-kernel durations: eager launches bracketed by HIP events on the library's stream
    moe.kernel_timing(True)
    probe_steps = min(args.steps, 800)
    for s in range(probe_steps):
        step(s)
    kt = moe.kernel_times()
    moe.kernel_timing(False)
    per_kernel_us = {name: (tot / cnt * 1e3 if cnt else None) for name, (tot, cnt) in kt.items()}
    layer_bytes = mean_distinct * expert_bytes + router_bytes + n * H * 8
    # the dominant kernel and the bytes one launch of it has to move
    # at one token the gate/up launch is the fused one where the device allows it: it also reads the router and the f32 row
    fused = n == 1 and moe.router_exchange_state()[0]
    kernel_bytes = {"decode_layer": mean_distinct * expert_bytes + router_bytes + n * H * 4,
                    "gate_up": mean_distinct * gate_up_expert_bytes + (router_bytes + n * H * 4 if fused else n * E * 4),
                    "down_combine": mean_distinct * (expert_bytes - gate_up_expert_bytes),
                    "down": mean_distinct * (expert_bytes - gate_up_expert_bytes),
                    "gemm_gate_up": mean_distinct * gate_up_expert_bytes}
    timed = {name: us for name, us in per_kernel_us.items() if us is not None and name in kernel_bytes}
    dom = max(timed, key=lambda name: timed[name] * kt[name][1]) if timed else None
    eager_us = timed.get(dom) if dom else None
    gu_bytes = kernel_bytes[dom] if dom else 0.0
    # The dominant kernel's duration inside the timed graph: the median event-timed replay, per step, less what the step's
    # other launches take (their eager event-bound averages times their launches per step).  The eager figure of the
    # dominant kernel itself is kept beside it: it moves by 10 % from box to box, the replays do not.
    gu_us, source = eager_us, "eager launches, HIP events bound to each dispatch"
    if dom and steady is not None:
        per_step = max(probe_steps * layers_per_step, 1)
        others = sum(tot / per_step * 1e3 for name, (tot, cnt) in kt.items() if cnt and name != dom)
        dom_launches = kt[dom][1] / per_step
        in_graph = (steady["us_per_layer_p50"] - others) / max(dom_launches, 1e-9)
        if in_graph > 0:
            gu_us, source = in_graph, ("median of the event-timed graph replays per layer, less the layer's other launches "
                                       "(eager event-bound averages)")
    achieved = gu_bytes / (gu_us * 1e-6) / 1e9 if gu_us else None
    layer_frac = (layer_bytes / (steady["us_per_layer_p50"] * 1e-6) / 1e9 / HBM_PEAK_GBS) if steady is not None else None

    layer_gbs = layer_bytes / (ms_per_step * 1e-3) / 1e9
    # batched calls: matrix-core rate of the two grouped GEMMs (2*H*I flops per assignment and projection)
    mfma = None
    if per_kernel_us.get("gemm_gate_up") and per_kernel_us.get("gemm_down"):
        peak = 2500.0 if w["bank"] in ("F16", "F32", "BF16") else 5000.0  # dense f16 TFLOP/s, int8 TOP/s
        gu_t = n * k * 2 * 2 * H * I / (per_kernel_us["gemm_gate_up"] * 1e-6) / 1e12
        dn_t = n * k * 2 * H * I / (per_kernel_us["gemm_down"] * 1e-6) / 1e12
        mfma = {"unit": "TFLOP/s" if w["bank"] in ("F16", "BF16") else "TOP/s", "peak": peak, "gemm_gate_up": round(gu_t, 1),
                "gemm_down": round(dn_t, 1), "gemm_gate_up_frac": round(gu_t / peak, 4), "gemm_down_frac": round(dn_t / peak, 4),
                "hbm_floor_us": round(layer_bytes / (HBM_PEAK_GBS * 1e3), 1)}

    out = {
        "metric": "MoE-layer tokens/s + achieved HBM GB/s (Q4_K, OLMoE shape, 1 GPU)",
        "value": round(value, 1),
        "unit": "layer-tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if w["bank"] in ("F16", "F32", "BF16") else ("i8*i16->i32" if w["bank"] == "Q8_0" else "u4*i16->i32") +
                 " (v_dot4_i32_i8), f32 scales",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: hidden {H}, {E} experts, top-{k}, inter {I}, {w['bank']} experts{' (' + w['down'] + ' down)' if 'down' in w else ''}, "
                               f"f16 router, norm_topk_prob={str(norm).lower()}, {n} token(s)/step, rotating over {L} layer banks",
                   "tokens_per_step": n, "layers": L, "stack": bool(args.stack), "shared_inter": args.shared_inter,
                   "deferred_combine": bool(deferred), "tile_order": "from 6 tokens" if tile_order is None else tile_order, "warm_next_router": os.environ.get("MUMMU_WARM_NEXT", "1") != "0", "hip_graph": graph is not None, "steps_per_graph_launch": per_graph if graph is not None else None,
                   "graph_replays_timed": (replays + (1 if left else 0)) if graph is not None else 0,
                   "first_timed_step": first,
                   "cache_cold": bool((per_graph - 1) * layer_bytes * layers_per_step > 256e6) if graph is not None else
                                 bool(min(L, args.steps) * layer_bytes > 256e6),
                   "mean_distinct_experts_per_step": round(mean_distinct, 3),
                   "launches_per_step": {k_: int(round(cnt / max(probe_steps * (L if args.stack else 1), 1))) for k_, (tot, cnt) in kt.items() if cnt}},
        "us_per_layer": round(ms_per_step * 1e3, 3),
        "event_ms_per_step": round(ev_ms / args.steps / layers_per_step, 6),
        "steady": steady,
        "layer_algorithmic_bytes": int(layer_bytes),
        "layer_hbm_gbs": round(layer_gbs, 1),
        "layer_hbm_frac": round(layer_gbs / HBM_PEAK_GBS, 4),
        "kernel_us": {k_: (round(v, 3) if v is not None else None) for k_, v in per_kernel_us.items()},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1) if achieved else None,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4) if achieved else None,
                     "traffic": profiled_traffic(args.workload, n, dom),
                     "algorithmic_bytes_per_launch": int(gu_bytes), "avg_launch_us": round(gu_us, 3) if gu_us else None,
                     "avg_launch_us_from": source, "avg_launch_us_eager": round(eager_us, 3) if eager_us else None,
                     "layer_frac": round(layer_frac, 4) if layer_frac else None},
        "mfma": mfma,
        "device": M.device_name(),
        "setup_s": round(setup_s, 1),
    }

    if not args.no_cpu_baseline and not args.shared_inter:
        out["cpu_baseline"] = cpu_baseline(keep_layer0, w, bank_t, down_t, xs, n, args.cpu_seconds)
    print(json.dumps(out))
    return 0


def cpu_baseline(layer0, w, bank_t, down_t, xs, n, budget_s):
    """The oracle's routed path (the reference's qwen4exp algorithm: per hit expert, dequantize
    row chunks and dot them in the fixed 8-lane order; OpenMP over rows where the reference
    uses rayon) on layer 0 of the same banks, same token batches, for about budget_s seconds."""
    from oracle import binding as orc
    router, gate, up, down = layer0
    H, I, E, k, norm = w["hidden"], w["inter"], w["experts"], w["top_k"], w["norm"]
    banks = orc.LayerBanks(H, I, E, gate, up, down, bank_t, bank_t, down_t)  # the oracle uses the same ggml type ids
    flavour = w.get("flavour", 0)
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    orc.moe_forward(banks, router, orc.F16, xs[0], k, norm, flavour)  # warm
    done, t0, best = 0, time.perf_counter(), None
    while time.perf_counter() - t0 < budget_s:
        t1 = time.perf_counter()
        orc.moe_forward(banks, router, orc.F16, xs[done % xs.shape[0]], k, norm, flavour)
        dt = time.perf_counter() - t1
        best = dt if best is None else min(best, dt)
        done += 1
    total = time.perf_counter() - t0
    return {"value": round(n * done / total, 2), "unit": "layer-tokens/s", "cores": threads, "kind": "port",
            "sample": f"{done} steps of the same workload on layer 0 ({n} token(s)/step), mean over {total:.1f} s; "
                      f"best step {best * 1e3:.1f} ms",
            "cpu": _cpu_model()}


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


if __name__ == "__main__":
    sys.exit(main())
