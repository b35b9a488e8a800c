#!/usr/bin/env python3
"""Benchmark of the quantized MoE expert GEMV path on one MI355X.

A "step" is one pass of the hot path over one batch: one MXFP4 MoE decode layer (router top-8
selection from given logits -> fused gate/up + SwiGLU -> down + ordered accumulation: three
launches) at the headline shape (256 experts, hidden 4096, expert intermediate 1024, top-8,
no shared expert), T tokens. Consecutive steps walk DIFFERENT layers' weights (a ring of
`--layers` full layers, as a model's decode step walks its MoE layers), so every step streams its
experts from HBM, not from the 256 MB Infinity Cache / L2. The steps are captured once in a HIP
graph (the serving form of the reference's decode walk) and timed with events on the launch stream.

Prints ONE JSON line: whole-layer achieved HBM GB/s (algorithmic bytes / time), µs per layer,
the dominant kernel's roofline, and the CPU oracle timed on this machine's host cores.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0
E, H, I, K = 256, 4096, 1024, 8          # the headline configuration (MXFP4 MoE decode layer)
EXPERT_BYTES = 3 * I * H // 2 + 3 * I * H // 32          # payload + e8m0 scales of gate, up, down
GATE_UP_BYTES = 2 * (I * H // 2 + I * H // 32)
# HBM-side bytes per launch of the two GEMV kernels at the default workload (T = 8, 256 experts) come from rocprofv3
# --pmc FETCH_SIZE / WRITE_SIZE runs scaled by the library's plain copy kernel: a counter cannot be read from inside
# this process, so the figures are read out of the committed summary of those runs (its `traffic_bytes_per_launch`
# lines, which also name the kernels they were taken from) and dropped from the line when the workload differs.
TRAFFIC_PROFILE = "profiles/moe_gemv_kernels_mxfp4_c3_t8_hbm_counters.txt"


# The sources that define the two profiled kernels: the counter summary names the digest of the build it was taken
# from, and its figures are used only while the tree's digest is the same (a kernel body can change without its name).
KERNEL_SOURCES = ("gemv_core.hpp", "gemv_kernels.hpp", "swiglu.hpp", "numerics.hpp", "router_select.hpp")


def kernel_source_digest():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        h.update((ROOT / "dgpp_amd" / "csrc" / name).read_bytes())
    return h.hexdigest()[:16]


def measured_traffic():
    """{"gate_up": bytes, "down": bytes, "gate_up_kernel": name, "down_kernel": name, "digest": ...} from the counter
    summary, or {}; {"stale": digest} when the summary was taken from other kernel sources than the tree holds."""
    out = {}
    try:
        text = (ROOT / TRAFFIC_PROFILE).read_text()
    except OSError:
        return out
    for line in text.splitlines():
        part = line.split()
        if len(part) >= 4 and part[0] == "traffic_bytes_per_launch":
            out[part[1]] = float(part[2])
            out[part[1] + "_kernel"] = " ".join(part[3:])
        if len(part) >= 2 and part[0] == "kernel_source_digest":
            out["digest"] = part[1]
    try:
        now = kernel_source_digest()
    except OSError:
        return {}
    if out.get("digest") != now:
        return {"stale": out.get("digest"), "tree": now}
    return out


DOWN_BYTES = H * I // 2 + H * I // 32


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--tokens", type=int, default=8, help="decode batch of the headline number (1..8)")
    ap.add_argument("--layers", type=int, default=16, help="ring of distinct layers' weights (cold-cache rotation)")
    ap.add_argument("--experts", type=int, default=E, help="experts per layer (256 = the headline shape)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="'layer', 'gate_up' or 'down': run only that timed graph (for profiling)")
    ap.add_argument("--no-others", action="store_true", help="skip the T=1/4/8 side measurements")
    ap.add_argument("--no-probe", action="store_true",
                    help="skip the plain-read yardstick (a cold read of the same byte count) beside the two kernel legs")
    ap.add_argument("--eager", action="store_true", help="launch the timed steps eagerly instead of as one HIP graph")
    ap.add_argument("--probe-copy", type=int, default=0, metavar="MiB",
                    help="also run the library's plain copy kernel over this many MiB three times (counter calibration)")
    ap.add_argument("--configs", default=None, help="other benchmark configurations to time beside the headline, comma "
                    "separated out of c1,c2,c2round,c4,c5,c5skew,w8a8,qwen_tail,slotbench,readprobe,router,pair,dispatch ('' for none; default: c1,c2,c4,c5, none under --tune)")
    ap.add_argument("--replays", type=int, default=0, help="timed graph replays per measurement (0 = at least 50 and at "
                    "least 1000 steps; a small number keeps a run under a profiler's counters short)")
    ap.add_argument("--tune", default="", help="bench A/B switches as key=value,... (dgpp_tune_set)")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU (the path shards by experts or by the intermediate "
              "dimension with a single all-reduce after the layer; no multi-GPU figure is produced). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    os.environ.setdefault("DGPP_AMD_BENCH", "1")   # the A/B legs steer the library's measurement switches: opt in
    import torch
    from dgpp_amd import _lib, hostgen as hg, launch as L, moe_layer as ML

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = _lib.load()   # fails loudly when the HIP library has not been built
    if not lib.dgpp_tune_enabled():
        print("bench.py: the library's measurement switches are off (DGPP_AMD_BENCH is set to something other than 1, "
              "or the library was built with -DDGPP_NO_TUNE): the A/B legs would all time the default form", file=sys.stderr)
        sys.exit(1)
    for kv in filter(None, args.tune.split(",")):
        k, v = kv.split("=")
        lib.dgpp_tune_set(int(k), int(v))
    dev = torch.device("cuda:0")
    nE, nL = args.experts, args.layers
    t_build = time.time()

    # ---- layer 0: host-generated N(0, 0.02) weights, MXFP4-quantised with the library's encoder ----------
    gu_p = torch.empty((nE, 2, I, H // 2), dtype=torch.uint8)
    gu_s = torch.empty((nE, 2, I, H // 32), dtype=torch.uint8)
    dn_p = torch.empty((nE, H, I // 2), dtype=torch.uint8)
    dn_s = torch.empty((nE, H, I // 32), dtype=torch.uint8)
    for e in range(nE):
        seed = 0xD6990000 + 3 * 16 + e * 3
        for m in range(2):
            p, s = hg.encode_mxfp4(hg.normal_f32(seed + m, (I, H), 0.02))
            gu_p[e, m], gu_s[e, m] = torch.from_numpy(p), torch.from_numpy(s)
        p, s = hg.encode_mxfp4(hg.normal_f32(seed + 2, (H, I), 0.02))
        dn_p[e], dn_s[e] = torch.from_numpy(p), torch.from_numpy(s)
    host_layer0 = (gu_p, gu_s, dn_p, dn_s)
    # ---- the ring: layer l is layer 0 with its experts rotated by 37*l (distinct addresses) ------------
    layers, keep = [], []
    cfg = L.make_config(H, I, nE, K, n_shared_experts=0, routed_scaling_factor=1.0, swiglu_limit=float("inf"),
                        router_mode=L.ROUTER_SOFTMAX_TOPK)
    max_t = max(16, args.tokens)
    d0 = [t.to(dev) for t in host_layer0]
    for l in range(nL):
        if l == 0:
            bufs = d0
        else:
            sh = (37 * l) % nE
            bufs = [torch.roll(t, shifts=sh, dims=0).contiguous() for t in d0]
        keep.append(bufs)
        views = []
        for e in range(nE):
            for m in range(3):
                v = L.MoeExpertView()
                if m < 2:
                    v.payload, v.fp4_scales = bufs[0][e, m].data_ptr(), bufs[1][e, m].data_ptr()
                else:
                    v.payload, v.fp4_scales = bufs[2][e].data_ptr(), bufs[3][e].data_ptr()
                v.scale_shift_rows = v.scale_shift_cols = 7
                v.fp4_group = 32
                views.append(v)
        layers.append(ML.MoeLayer(cfg, ML.EXPERTS_MXFP4, views, max_t))
    build_s = time.time() - t_build

    def inputs(T):
        xs = torch.from_numpy(hg.normal_bf16(0xD6990000 + 3 * 16 + T, (nL, T, H)).view(np.int16)).to(dev)
        lg = hg.bf16_to_f32(hg.normal_bf16(0xD6990100 + T, (nL, T, nE)))        # router logits N(0,1), bf16 values
        return xs, torch.from_numpy(lg).to(dev), lg

    stream = torch.cuda.Stream()

    def time_graph(enqueue, steps, warmup, stats=None):
        """Captures `steps` calls of enqueue(i) in one HIP graph and replays it back to back at least 50 times (and until
        at least 1000 steps have run), with an event on the launch stream between consecutive replays. A replay's time
        is the span between its two events; the figure returned is the MEDIAN replay divided by `steps`, in seconds per
        step, so it does not depend on how many steps one graph holds (the replays queue behind each other: a graph's
        launch set-up overlaps its predecessor's run). `stats`, when given, receives median / min / max per step in
        microseconds and the replay count. `warmup` eager steps run before the capture and one untimed replay after it."""
        replays = args.replays if args.replays > 0 else max(50, -(-1000 // max(steps, 1)))
        with torch.cuda.stream(stream):
            for i in range(max(warmup, 1)):
                enqueue(i)
            stream.synchronize()
            if args.eager:
                evs = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
                evs[0].record(stream)
                for r in range(replays):
                    for i in range(steps):
                        enqueue(i)
                    evs[r + 1].record(stream)
            else:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=stream):
                    for i in range(steps):
                        enqueue(i)
                g.replay()
                stream.synchronize()
                evs = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
                torch.cuda.synchronize()
                evs[0].record(stream)
                for r in range(replays):
                    g.replay()
                    evs[r + 1].record(stream)
            torch.cuda.synchronize()
        per = np.array([evs[r].elapsed_time(evs[r + 1]) for r in range(replays)], dtype=np.float64) * 1e-3 / steps
        if stats is not None:
            stats.update({"us_median": float(np.median(per)) * 1e6, "us_min": float(per.min()) * 1e6,
                          "us_max": float(per.max()) * 1e6, "replays": replays, "steps_per_replay": steps})
        return float(np.median(per))

    probe_buf = {}

    def plain_read_us(nbytes):
        """What ONE cold launch of the library's plain streaming-read probe costs for this many bytes (16-byte loads, a
        contiguous span per block, nothing computed or stored): successive launches walk successive windows of a 1 GiB
        buffer, so every window has left the caches when it is read again. The yardstick a weight-streaming launch of
        the same size is read against; timed like the kernel legs (median of graph replays)."""
        if "buf" not in probe_buf:
            probe_buf["buf"] = torch.zeros(1 << 30, dtype=torch.uint8, device=dev)
            probe_buf["sink"] = torch.zeros(8192, dtype=torch.int32, device=dev)
        buf, sink = probe_buf["buf"], probe_buf["sink"]
        nbytes = int(nbytes) // 256 * 256
        nwin = max(1, buf.numel() // nbytes)
        best = None
        for blocks in (1024, 2048, 4096):
            def step(i):
                if lib.dgpp_probe_read(buf.data_ptr() + (i % nwin) * nbytes, nbytes, sink.data_ptr(), 0, blocks, 1,
                                       stream.cuda_stream) != 0:
                    raise RuntimeError(lib.dgpp_last_error().decode())
            sec = time_graph(step, max(16, min(nwin, 64)), 2)
            best = sec if best is None or sec < best else best
        return best * 1e6

    def measure(T, steps, warmup, only=""):
        # a graph holds whole walks of the ring (at least four), so that a replay never meets a layer its predecessor has
        # just left and the few microseconds between two replays stay below one percent of a replay
        steps = max(4, -(-steps // nL)) * nL
        xs, lg_d, lg = inputs(T)
        outs = torch.empty((nL, T, H), dtype=torch.int16, device=dev)
        # distinct experts per layer-step (the algorithmic bytes count each distinct expert once)
        l64 = lg.astype(np.float64)
        uniq = []
        for l in range(nL):
            top = np.argsort(-l64[l], axis=1, kind="stable")[:, :K]
            uniq.append(len(np.unique(top)))
        u_mean = float(np.mean([uniq[i % nL] for i in range(steps)]))
        layer_bytes = u_mean * EXPERT_BYTES + T * (H * 2 * 2) + T * K * 8
        res = {"tokens": T, "distinct_experts_mean": u_mean, "algorithmic_bytes": layer_bytes}

        def full(i):
            l = i % nL
            layers[l].enqueue_decode_scores(xs[l], H, lg_d[l], lg_d[l], outs[l], T, stream)

        if only in ("", "layer"):
            st = {}
            sec = time_graph(full, steps, warmup, st)
            res["us_per_layer"] = sec * 1e6
            res["timing"] = st
            res["gbps"] = layer_bytes / sec / 1e9
            res["frac_of_peak"] = res["gbps"] / HBM_PEAK_GBPS
        # the dominant kernel alone: the fused gate/up + SwiGLU slot kernel on the routes the layers hold
        slots = T * (K + 1)
        acts = torch.empty((nL, slots, I), dtype=torch.int16, device=dev)
        orders = []
        with torch.cuda.stream(stream):
            for l in range(nL):
                full(l)                                       # leaves ids / weights in the layer's scratch
                o = None
                if T * K > 128:     # as the layer does: small batches need no slot order (sharers found by ballot)
                    o = torch.empty(slots, dtype=torch.int32, device=dev)
                    L.launch_moe_slot_order(layers[l].ids_ptr, o, slots, K, nE, stream)
                orders.append(o)
            stream.synchronize()
        def gate_up(i):
            l = i % nL
            L.launch_moe_slot_gate_up_swiglu_fp4(xs[l], H, layers[l].ids_ptr, orders[l],
                                                 layers[l]._views_ptr, I, H, 0, 0, None, None, None, None, acts[l], I,
                                                 slots, K, float("inf"), stream, -1, 32)

        if only in ("", "gate_up"):
            st_k = {}
            sec_k = time_graph(gate_up, steps, warmup, st_k)
            res["gate_up_timing"] = st_k
            kbytes = u_mean * GATE_UP_BYTES + T * H * 2 + T * K * I * 2
            res["gate_up_us"] = sec_k * 1e6
            res["gate_up_bytes"] = kbytes
            res["gate_up_gbps"] = kbytes / sec_k / 1e9
            if not args.no_probe:
                res["gate_up_plain_read_us"] = plain_read_us(kbytes)
                res["gate_up_frac_of_plain_read"] = res["gate_up_plain_read_us"] / res["gate_up_us"]
        def down(i):   # the layer's second GEMV kernel: token-major down projection + ordered accumulation
            l = i % nL
            L.launch_moe_slot_down_accum_fp4(acts[l], I, layers[l].ids_ptr, layers[l]._views_ptr, H, I, T, K,
                                             layers[l].weights_ptr, outs[l], None, stream, 32)

        if only in ("", "down"):
            st_d = {}
            sec_d = time_graph(down, steps, warmup, st_d)
            res["down_timing"] = st_d
            dbytes = u_mean * DOWN_BYTES + T * K * I * 2 + T * H * 2
            res["down_us"] = sec_d * 1e6
            res["down_bytes"] = dbytes
            res["down_gbps"] = dbytes / sec_d / 1e9
            if not args.no_probe:
                res["down_plain_read_us"] = plain_read_us(dbytes)
                res["down_frac_of_plain_read"] = res["down_plain_read_us"] / res["down_us"]
        return res

    for lyr in layers:     # device pointer of the layer's expert table, for the single-kernel leg
        lyr._views_ptr = lyr.views_ptr

    if args.probe_copy > 0:
        nbytes = args.probe_copy << 20
        src = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        dst = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        with torch.cuda.stream(stream):
            for _ in range(3):
                if lib.dgpp_probe_copy(dst.data_ptr(), src.data_ptr(), nbytes, stream.cuda_stream) != 0:
                    raise RuntimeError(lib.dgpp_last_error().decode())
            stream.synchronize()
        del src, dst

    T = args.tokens
    main_res = measure(T, args.steps, args.warmup, args.only)
    others = {}
    if not args.only and not args.tune and not args.no_others:
        for t in (1, 4, 8, 16):
            if t != T:
                others[f"T{t}"] = measure(t, args.steps, args.warmup)

    # ---- the other benchmark configurations (reported beside the headline, never part of `value`) -----------
    def ring_copies(tensors, nbytes, want=2 * 256 * 2**20 + 64 * 2**20):
        """Device copies of a weight set so that consecutive timed launches never find it in the caches."""
        n = max(2, -(-want // nbytes))
        return [[t.clone() for t in tensors] if i else list(tensors) for i in range(n)]

    def bench_c1():
        n = k = 4096
        payload, scales = hg.encode_fp8_blocks(hg.f32_to_bf16(hg.normal_f32(0xD6990010, (n, k), 0.02)), 128, 128)
        ring = ring_copies([torch.from_numpy(payload).to(dev), torch.from_numpy(scales).to(dev)], payload.nbytes)
        act = torch.from_numpy(hg.normal_bf16(0xD6990011, (1, k)).view(np.int16)).to(dev)
        out = torch.empty((len(ring), n), dtype=torch.int16, device=dev)
        def step(i):
            r = i % len(ring)
            L.launch_scale_gemm_bf16(act, k, ring[r][0], ring[r][1], out[r], 1, n, k, stream)
        sec = time_graph(step, args.steps, args.warmup)
        nbytes = n * k + (n // 128) * (k // 128) * 4 + k * 2 + n * 2
        return {"workload": "C1 dense FP8 block-128 GEMV 4096x4096, batch 1", "us": sec * 1e6, "algorithmic_bytes": nbytes,
                "gbps": nbytes / sec / 1e9, "frac_of_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS}

    def bench_c2():
        n, k = 17408, 5120
        payload, scales, ws2 = hg.encode_nvfp4(hg.normal_f32(0xD6990020, (n, k), 0.02))
        glob = torch.tensor([1.0 / np.float32(ws2)], dtype=torch.float32, device=dev)
        ring = ring_copies([torch.from_numpy(payload).to(dev), torch.from_numpy(scales).to(dev)],
                           payload.nbytes + scales.nbytes)
        mats = [L.Fp4Matrix(r[0].data_ptr(), r[1].data_ptr(), glob.data_ptr(), n, k, 16, 0, None) for r in ring]
        res = {}
        for m in (1, 8):
            act = torch.from_numpy(hg.normal_bf16(0xD6990021, (m, k)).view(np.int16)).to(dev)
            out = torch.empty((len(ring), m, n), dtype=torch.int16, device=dev)
            def step(i):
                r = i % len(ring)
                L.launch_fp4_gemv_bf16(act, k, mats[r], out[r], m, n, k, stream)
            sec = time_graph(step, args.steps, args.warmup)
            nbytes = n * k // 2 + n * k // 16 + 4 + m * (k * 2 + n * 2)
            res[f"batch{m}"] = {"us": sec * 1e6, "algorithmic_bytes": nbytes, "gbps": nbytes / sec / 1e9,
                                "frac_of_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS}
            if m > 4:   # the same launcher pinned to the vector core (what it ran before the row-count dispatch)
                lib.dgpp_tune_set(5, 1)
                sec = time_graph(step, args.steps, args.warmup)
                lib.dgpp_tune_set(5, 0)
                res[f"batch{m}_vector_core"] = {"us": sec * 1e6, "gbps": nbytes / sec / 1e9,
                                                "frac_of_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS}
            def step_mma(i):
                r = i % len(ring)
                L.launch_dense_mma_fp4_bf16(act, k, mats[r], out[r], m, n, k, stream)
            sec = time_graph(step_mma, args.steps, args.warmup)
            res[f"batch{m}_matrix_core"] = {"us": sec * 1e6, "gbps": nbytes / sec / 1e9,
                                            "frac_of_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS}
            ws = torch.empty(4 * m * n, dtype=torch.float32, device=dev)
            def step_split(i):
                r = i % len(ring)
                L.launch_mma_gemv_fp4_bf16(act, k, mats[r], out[r], m, n, k, 0, stream, ws, ws.numel() * 4)
            sec = time_graph(step_split, args.steps, args.warmup)
            res[f"batch{m}_matrix_core_split_k"] = {"us": sec * 1e6, "gbps": nbytes / sec / 1e9,
                                                    "frac_of_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS}
        res["workload"] = "C2 dense NVFP4 GEMV 17408x5120 (gate_up shape), batch 1 and 8 (one weight pass)"
        return res

    def bench_c2round():
        """C2's matrix at eight rows with the row count varied around what one resident round of the chip holds (1024 row
        groups of 16 rows x four K parts = 4096 wavefront slots): 16384 rows fill one round exactly, 17408 (C2) and 20480
        need a second."""
        k, m = 5120, 8
        res = {"workload": "dense NVFP4 GEMV [n x 5120], batch 8, n = 16384 / 17408 / 20480: the matrix-core forms around one "
                           "resident round (4096 wavefront tasks)"}
        act = torch.from_numpy(hg.normal_bf16(0xD6990021, (m, k)).view(np.int16)).to(dev)
        for n in (16384, 17408, 20480):
            payload, scales, ws2 = hg.encode_nvfp4(hg.normal_f32(0xD6990020, (n, k), 0.02))
            glob = torch.tensor([1.0 / np.float32(ws2)], dtype=torch.float32, device=dev)
            ring = ring_copies([torch.from_numpy(payload).to(dev), torch.from_numpy(scales).to(dev)],
                               payload.nbytes + scales.nbytes)
            mats = [L.Fp4Matrix(r[0].data_ptr(), r[1].data_ptr(), glob.data_ptr(), n, k, 16, 0, None) for r in ring]
            out = torch.empty((len(ring), m, n), dtype=torch.int16, device=dev)
            ws = torch.empty(4 * m * n, dtype=torch.float32, device=dev)
            nbytes = n * k // 2 + n * k // 16 + 4 + m * (k * 2 + n * 2)
            legs = {
                "launcher": lambda i: L.launch_fp4_gemv_bf16(act, k, mats[i % len(ring)], out[i % len(ring)], m, n, k, stream),
                "matrix_core_no_workspace": lambda i: L.launch_dense_mma_fp4_bf16(act, k, mats[i % len(ring)], out[i % len(ring)], m, n, k, stream),
                "matrix_core_split_k": lambda i: L.launch_mma_gemv_fp4_bf16(act, k, mats[i % len(ring)], out[i % len(ring)], m, n, k, 0, stream,
                                                                            ws, ws.numel() * 4),
            }
            row = {"row_groups_x_parts": (n // 16) * 4}
            for name, fn in legs.items():
                sec = time_graph(fn, args.steps, args.warmup)
                row[name] = {"us": sec * 1e6, "gbps": nbytes / sec / 1e9}
            res[f"n{n}"] = row
            del ring, mats, out, ws
        return res

    def expert_table(per_expert_views, n_exp):
        return [v for e in range(n_exp) for v in per_expert_views[e]]

    def bench_c4():
        cE, cH, cI, cK, cT = 128, 2048, 768, 8, 32
        gen = []
        for e in range(cE):   # every expert its own weights: 604 MB per layer, far beyond the caches
            mats = []
            for mi, (r, c) in enumerate(((cI, cH), (cI, cH), (cH, cI))):
                pw, sw = hg.encode_fp8_blocks(hg.f32_to_bf16(hg.normal_f32(0xD6994000 + e * 3 + mi, (r, c), 0.02)), 128, 128)
                mats.append((torch.from_numpy(pw).to(dev), torch.from_numpy(sw).to(dev)))
            gen.append(mats)
        ring = [gen, [[(a.clone(), b.clone()) for a, b in mats] for mats in gen]]
        cfg4 = L.make_config(cH, cI, cE, cK, n_shared_experts=0, routed_scaling_factor=1.0, swiglu_limit=float("inf"),
                             router_mode=L.ROUTER_SOFTMAX_TOPK)
        lay = []
        for g in ring:
            views = []
            for e in range(cE):
                for pw, sw in g[e]:
                    v = L.MoeExpertView()
                    v.payload, v.scales = pw.data_ptr(), sw.data_ptr()
                    v.scale_shift_rows = v.scale_shift_cols = 7
                    v.fp4_group = 16
                    views.append(v)
            lay.append(ML.MoeLayer(cfg4, ML.EXPERTS_FP8, views, cT))
        ids = hg.zipf_routes(0xD6990040 + cT, 1.1, cT, cK, cE)
        lg = hg.bf16_to_f32(hg.normal_bf16(0xD6990041, (cT, cK))).astype(np.float64)
        wts = np.exp(lg - lg.max(1, keepdims=True))
        wts = (wts / wts.sum(1, keepdims=True)).astype(np.float32)
        x = torch.from_numpy(hg.normal_bf16(0xD6990042, (cT, cH)).view(np.int16)).to(dev)
        ids_d, w_d = torch.from_numpy(ids).to(dev), torch.from_numpy(wts).to(dev)
        out = torch.empty((2, cT, cH), dtype=torch.int16, device=dev)
        uniq = len(np.unique(ids))
        nbytes = uniq * (3 * cI * cH + 3 * (cI // 128) * (cH // 128) * 4) + cT * cH * 4
        res = {"workload": f"C4 FP8 block-128 MoE layer, 128 experts, hidden 2048, inter 768, top-8, T=32 Zipf(1.1) "
                           f"routing ({uniq} distinct experts, busiest {int(np.bincount(ids.ravel()).max())} tokens)",
               "algorithmic_bytes": nbytes}
        for name, fn in (("decode_slots", lambda i: lay[i % 2].enqueue_decode_routed(x, cH, ids_d, w_d, out[i % 2], cT, stream)),
                         ("grouped", lambda i: lay[i % 2].enqueue_grouped_routed(x, cH, ids_d, w_d, out[i % 2], cT, stream)),
                         ("grouped_matrix_core",
                          lambda i: lay[i % 2].enqueue_prefill_routed(x, cH, ids_d, w_d, out[i % 2], cT, stream))):
            sec = time_graph(fn, max(args.steps // 4, 10), args.warmup)
            res[name] = {"us": sec * 1e6, "gbps": nbytes / sec / 1e9, "frac_of_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS}
        for l_ in lay:
            l_.close()
        return res

    def bench_c5(skew=False):
        cE, cH, cI, cK, cT, cSI, G = 256, 6144, 2048, 8, 64, 4096, 8
        keep5, gen = [], []
        for g in range(G):    # G generated experts; the 256 table entries are device COPIES of them (own addresses)
            mats = []
            for mi, (r, c) in enumerate(((cI, cH), (cI, cH), (cH, cI))):
                pw, sw, ws2 = hg.encode_nvfp4(hg.normal_f32(0xD6995000 + g * 3 + mi, (r, c), 0.02))
                mats.append((torch.from_numpy(pw).to(dev), torch.from_numpy(sw).to(dev),
                             torch.tensor([1.0 / np.float32(ws2)], dtype=torch.float32, device=dev)))
            gen.append(mats)
        views = []
        for e in range(cE):
            for pw, sw, gl in gen[e % G]:
                pc, sc_ = (pw, sw) if e < G else (pw.clone(), sw.clone())
                keep5 += [pc, sc_]
                v = L.MoeExpertView()
                v.payload, v.fp4_scales, v.fp4_global = pc.data_ptr(), sc_.data_ptr(), gl.data_ptr()
                v.scale_shift_rows = v.scale_shift_cols = 7
                v.fp4_group = 16
                views.append(v)
        cfg5 = L.make_config(cH, cI, cE, cK, n_shared_experts=0, routed_scaling_factor=1.0, swiglu_limit=float("inf"),
                             router_mode=L.ROUTER_SOFTMAX_TOPK)
        lay = ML.MoeLayer(cfg5, ML.EXPERTS_NVFP4, views, cT)
        x = torch.from_numpy(hg.normal_bf16(0xD6990050, (cT, cH)).view(np.int16)).to(dev)
        lg_h = hg.bf16_to_f32(hg.normal_bf16(0xD6990051, (cT, cE)))
        lg5 = torch.from_numpy(lg_h).to(dev)
        uniq = len(np.unique(np.argsort(-lg_h.astype(np.float64), axis=1, kind="stable")[:, :cK]))
        sh = []
        for mi, (r, c) in enumerate(((cSI, cH), (cSI, cH), (cH, cSI))):
            pw, sw = hg.encode_mxfp8(hg.normal_f32(0xD6995900 + mi, (r, c), 0.02))
            sh.append((torch.from_numpy(pw).to(dev), torch.from_numpy(sw).to(dev)))
        routed = torch.empty((cT, cH), dtype=torch.float32, device=dev)
        g_d, u_d, a_d = (torch.empty((cT, cSI), dtype=torch.int16, device=dev) for _ in range(3))
        shared_down = torch.empty((cT, cH), dtype=torch.float32, device=dev)
        rows_id = torch.arange(cT, dtype=torch.int32, device=dev)
        ones = torch.ones(cT, dtype=torch.float32, device=dev)
        out = torch.empty((cT, cH), dtype=torch.int16, device=dev)

        def routed_part(i):
            lay.enqueue_decode_scores(x, cH, lg5, lg5, None, cT, stream, out_f32=routed)

        def shared_part(i):
            L.launch_scale_gemm_grid_e8m0_bf16(x, cH, sh[0][0], sh[0][1], g_d, cT, cSI, cH, stream, 0, 0, 5)
            L.launch_scale_gemm_grid_e8m0_bf16(x, cH, sh[1][0], sh[1][1], u_d, cT, cSI, cH, stream, 0, 0, 5)
            L.launch_moe_swiglu_clamp(g_d, u_d, a_d, cT * cSI, float("inf"), stream)
            L.launch_scale_gemm_grid_e8m0_f32(a_d, cSI, sh[2][0], sh[2][1], shared_down, cT, cH, cSI, stream, 0, 0, 5)
            L.launch_moe_accum(routed, shared_down, rows_id, ones, cT, cH, stream)
            L.launch_moe_round_bf16(out, routed, cT * cH, stream)

        ids5 = torch.empty((cT, cK), dtype=torch.int32, device=dev)
        w5 = torch.empty((cT, cK), dtype=torch.float32, device=dev)
        L.launch_moe_router_select(lg5, lg5, ids5, w5, cfg5, cT, stream)

        # The routed experts in the activation-quantized NVFP4 (W4A4) form, the layer driver's leg of it: segment, quantize
        # the token rows, grouped gate and up over the row list, SwiGLU + quantize in one launch, grouped down, ordered
        # accumulation over the BF16 down rows. Different numerics from the legs beside it (NVFP4 activations).
        def w4a4_chain(ids_t, w_t):
            return lambda i: lay.enqueue_prefill_routed_w4a4(x, cH, ids_t, w_t, None, cT, stream, out_f32=routed)
        if skew:
            # The same layer under Zipf(1.1) expert popularity: few experts take most tokens, so routed segments reach
            # 16 and more rows - the shape the matrix-core grouped form is for. Routes are given (ids drawn from the
            # popularity law, weights the renormalised softmax of N(0,1) draws); routed experts only.
            ids_h = hg.zipf_routes(0xD6990058, 1.1, cT, cK, cE)
            lw = hg.bf16_to_f32(hg.normal_bf16(0xD6990059, (cT, cK))).astype(np.float64)
            wz = np.exp(lw - lw.max(1, keepdims=True))
            wz = (wz / wz.sum(1, keepdims=True)).astype(np.float32)
            ids_z, w_z = torch.from_numpy(ids_h).to(dev), torch.from_numpy(wz).to(dev)
            counts = np.bincount(ids_h.ravel(), minlength=cE)
            uz = int(np.count_nonzero(counts))
            per_expert = 3 * cI * cH // 2 + 3 * cI * cH // 16 + 12
            nb = uz * per_expert + cT * cH * 6
            res = {"workload": f"C5's routed NVFP4 experts under Zipf(1.1) routing, T=64: {uz} distinct experts, busiest "
                               f"{int(counts.max())} tokens, {int(np.count_nonzero(counts >= 16))} experts with >= 16 tokens",
                   "algorithmic_bytes": nb, "flops": 2.0 * cT * cK * 3 * cI * cH}
            legs = (("decode_slots", lambda i: lay.enqueue_decode_routed(x, cH, ids_z, w_z, None, cT, stream, out_f32=routed)),
                    ("grouped_matrix_core", lambda i: lay.enqueue_prefill_routed(x, cH, ids_z, w_z, None, cT, stream, out_f32=routed)),
                    ("grouped_matrix_core_w4a4", w4a4_chain(ids_z, w_z)))
            for name, fn in legs:
                sec = time_graph(fn, max(args.steps // 10, 5), 2)
                res[name] = {"us": sec * 1e6, "gbps": nb / sec / 1e9, "frac_of_peak": nb / sec / 1e9 / HBM_PEAK_GBPS,
                             "tflops": res["flops"] / sec / 1e12}
            lay.close()
            return res

        def routed_mc(i):
            lay.enqueue_prefill_routed(x, cH, ids5, w5, None, cT, stream, out_f32=routed)

        def shared_mc(i):
            L.launch_mma_gemv_fp8e8m0_bf16(x, cH, sh[0][0], sh[0][1], g_d, cT, cSI, cH, 0, 0, 5, stream)
            L.launch_mma_gemv_fp8e8m0_bf16(x, cH, sh[1][0], sh[1][1], u_d, cT, cSI, cH, 0, 0, 5, stream)
            L.launch_moe_swiglu_clamp(g_d, u_d, a_d, cT * cSI, float("inf"), stream)
            L.launch_mma_gemv_fp8e8m0_f32(a_d, cSI, sh[2][0], sh[2][1], shared_down, cT, cH, cSI, 0, 0, 5, stream)
            L.launch_moe_accum(routed, shared_down, rows_id, ones, cT, cH, stream)
            L.launch_moe_round_bf16(out, routed, cT * cH, stream)

        # The shared expert in the activation-quantized form: x and the SwiGLU output go through the MXFP8 row
        # quantizers and the three projections run on the block-scaled matrix-core instruction (different
        # numerics from the legs above: the activations carry MXFP8 rounding; SwiGLU-OAI with alpha 1.702, limit 7).
        xq, aq = (torch.empty((cT, d), dtype=torch.uint8, device=dev) for d in (cH, cSI))
        xq_s, aq_s = (torch.empty((cT, d // 32), dtype=torch.uint8, device=dev) for d in (cH, cSI))

        def shared_w8a8(i):
            L.launch_mxfp8_quantize_rows(x, cH, cT, cH, xq, xq_s, stream)
            L.launch_mxfp8_gemm_bf16(xq, xq_s, sh[0][0], sh[0][1], g_d, cT, cSI, cH, stream)
            L.launch_mxfp8_gemm_bf16(xq, xq_s, sh[1][0], sh[1][1], u_d, cT, cSI, cH, stream)
            L.launch_minimax_swiglu_mxfp8_rows(g_d, u_d, cSI, cT, cSI, 1.702, 7.0, aq, aq_s, stream)
            L.launch_mxfp8_gemm_f32(aq, aq_s, sh[2][0], sh[2][1], shared_down, cT, cH, cSI, stream)
            L.launch_moe_accum(routed, shared_down, rows_id, ones, cT, cH, stream)
            L.launch_moe_round_bf16(out, routed, cT * cH, stream)

        sws = torch.empty(4 * cT * max(cSI, cH), dtype=torch.float32, device=dev)   # split-K workspace: parts(k) * m * n floats

        def shared_part_ws(i):   # the same launchers given a split-K workspace
            nb_ = sws.numel() * 4
            L.launch_scale_gemm_grid_e8m0_bf16(x, cH, sh[0][0], sh[0][1], g_d, cT, cSI, cH, stream, 0, 0, 5, sws, nb_)
            L.launch_scale_gemm_grid_e8m0_bf16(x, cH, sh[1][0], sh[1][1], u_d, cT, cSI, cH, stream, 0, 0, 5, sws, nb_)
            L.launch_moe_swiglu_clamp(g_d, u_d, a_d, cT * cSI, float("inf"), stream)
            L.launch_scale_gemm_grid_e8m0_f32(a_d, cSI, sh[2][0], sh[2][1], shared_down, cT, cH, cSI, stream, 0, 0, 5, sws, nb_)
            L.launch_moe_accum(routed, shared_down, rows_id, ones, cT, cH, stream)
            L.launch_moe_round_bf16(out, routed, cT * cH, stream)

        def stitched(i):        # the shared expert through the GEMV-named launchers (they take the matrix core at 64 rows)
            routed_part(i)
            shared_part(i)

        # the whole layer as ONE call of the layer driver: the MXFP8 shared expert of its own width runs as dense
        # projections on a second stream beside the routed passes, then the chain's last step and the rounding
        cfg5s = L.make_config(cH, cI, cE, cK, n_shared_experts=1, routed_scaling_factor=1.0, swiglu_limit=float("inf"),
                              router_mode=L.ROUTER_SOFTMAX_TOPK)
        lay1 = ML.MoeLayer(cfg5s, ML.EXPERTS_NVFP4, views, cT, shared_inter=cSI, sh_payload=[t[0] for t in sh],
                           sh_scales_e8m0=[t[1] for t in sh])

        def full(i):
            lay1.enqueue_decode_scores(x, cH, lg5, lg5, out, cT, stream)

        def full_mc(i):   # the same layer through the driver's matrix-core grouped path (routes given)
            lay1.enqueue_prefill_routed(x, cH, ids5, w5, out, cT, stream)

        def full_w8a8(i):
            routed_part(i)
            shared_w8a8(i)

        n_steps = max(args.steps // 10, 5)
        per_expert = 3 * cI * cH // 2 + 3 * cI * cH // 16 + 12
        shared_bytes = 3 * cSI * cH + 3 * cSI * cH // 32
        nbytes = uniq * per_expert + shared_bytes + cT * cH * 4
        res = {"workload": f"C5 NVFP4 routed MoE (256 experts, hidden 6144, inter 2048, top-8, {uniq} distinct; decode slots) "
                           f"+ MXFP8 shared expert (inter 4096, dense projections: launch_scale_gemm_grid_e8m0_*, the matrix-core form at 64 rows) as ONE layer-driver call, T=64; routed expert weights = device copies of {G} generated experts",
               "algorithmic_bytes": nbytes}
        for name, fn, nb in (("layer", full, nbytes), ("layer_matrix_core", full_mc, nbytes),
                             ("layer_stitched_from_launchers", stitched, nbytes),
                             ("routed_only", routed_part, uniq * per_expert + cT * cH * 6),
                             ("routed_only_matrix_core", routed_mc, uniq * per_expert + cT * cH * 6),
                             ("routed_only_matrix_core_w4a4", w4a4_chain(ids5, w5), uniq * per_expert + cT * cH * 6),
                             ("shared_only_gemv_launchers", shared_part, shared_bytes + cT * cH * 4),
                             ("shared_only_gemv_launchers_split_k_workspace", shared_part_ws, shared_bytes + cT * cH * 4),
                             ("shared_only", shared_mc, shared_bytes + cT * cH * 4),
                             ("shared_only_w8a8_scaled_matrix_core", shared_w8a8, shared_bytes + cT * cH * 4),
                             ("layer_with_w8a8_shared", full_w8a8, nbytes)):
            sec = time_graph(fn, n_steps, 2)
            res[name] = {"us": sec * 1e6, "algorithmic_bytes": nb, "gbps": nb / sec / 1e9,
                         "frac_of_peak": nb / sec / 1e9 / HBM_PEAK_GBPS}
        lay.close()
        lay1.close()
        return res

    def bench_slotbench():
        """The reference's own micro-benchmark of this path (benchmarks/micro/moe_slot_bench.cu: the whole decode chain
        - router dots, selection, gate/up + SwiGLU, down, accumulation - at its per-rank production geometry: 288
        experts, top-8 sigmoid-bias routing, hidden 4096, expert slice 512, one block-FP8 shared expert; 1, 2 and 8
        rows; routed experts NVFP4 or block FP8), timed here on the MI355X beside the figures it publishes for a
        GB10 (docs/nvfp4_plan.md:299-300, docs/measurements.md:485-488). Not one of BASELINE's configurations: run with
        --configs slotbench. Cold: 16 input row sets route to different experts, two copies of the routed weights
        alternate and every step has its own copy of the shared expert."""
        bE, bH, bI, bK, G, NX = 288, 4096, 512, 8, 8, 16
        published = {"nvfp4": {1: 209.0, 2: 334.0, 8: 929.0}, "fp8": {1: 273.0, 2: 469.0, 8: 1420.0}}
        gate = torch.from_numpy(hg.normal_bf16(0xD6996000, (bE, bH), 1.0 / 64.0).view(np.int16)).to(dev)
        bias = torch.from_numpy(hg.normal_f32(0xD6996001, (bE,), 0.05)).to(dev)
        shared = []
        for c in range(NX):
            tri = []
            for mi, (r, cc) in enumerate(((bI, bH), (bI, bH), (bH, bI))):
                if c == 0:
                    pw, sw = hg.encode_fp8_blocks(hg.f32_to_bf16(hg.normal_f32(0xD6996100 + mi, (r, cc), 0.02)), 128, 128)
                    tri.append((torch.from_numpy(pw).to(dev), torch.from_numpy(sw).to(dev)))
                else:
                    tri.append((shared[0][mi][0].clone(), shared[0][mi][1].clone()))
            shared.append(tri)
        cfgb = L.make_config(bH, bI, bE, bK, n_shared_experts=1, routed_scaling_factor=2.5, swiglu_limit=float("inf"),
                             router_mode=L.ROUTER_SIGMOID_BIAS)
        res = {"workload": "the reference's moe_slot_bench geometry: 288 experts, top-8 sigmoid-bias router from the hidden rows, "
                           "hidden 4096, expert slice 512, one block-FP8 shared expert; whole decode chain (enqueue_decode), cold"}
        for fmt in ("nvfp4", "fp8"):
            gen = []
            for g in range(G):
                mats = []
                for mi, (r, cc) in enumerate(((bI, bH), (bI, bH), (bH, bI))):
                    wf = hg.normal_f32(0xD6996200 + g * 3 + mi, (r, cc), 0.02)
                    if fmt == "nvfp4":
                        pw, sw, ws2 = hg.encode_nvfp4(wf)
                        mats.append((torch.from_numpy(pw).to(dev), torch.from_numpy(sw).to(dev),
                                     torch.tensor([1.0 / np.float32(ws2)], dtype=torch.float32, device=dev)))
                    else:
                        pw, sw = hg.encode_fp8_blocks(hg.f32_to_bf16(wf), 128, 128)
                        mats.append((torch.from_numpy(pw).to(dev), torch.from_numpy(sw).to(dev), None))
                gen.append(mats)
            keep, tables = [], []
            for copy in range(2):
                views = []
                for e in range(bE):
                    for pw, sw, gl in gen[e % G]:
                        pc, sc_ = pw.clone(), sw.clone()
                        keep += [pc, sc_]
                        v = L.MoeExpertView()
                        v.payload = pc.data_ptr()
                        if fmt == "nvfp4":
                            v.fp4_scales, v.fp4_global = sc_.data_ptr(), gl.data_ptr()
                        else:
                            v.scales = sc_.data_ptr()
                        v.scale_shift_rows = v.scale_shift_cols = 7
                        v.fp4_group = 16
                        views.append(v)
                tables.append(views)
            per_expert = (3 * bI * bH // 2 + 3 * bI * bH // 16 + 12) if fmt == "nvfp4" else (3 * bI * bH + 3 * (bI // 128) * (bH // 128) * 4)
            shared_bytes = 3 * bI * bH + 3 * (bI // 128) * (bH // 128) * 4
            for rows in (1, 2, 4, 8):
                lay = [ML.MoeLayer(cfgb, ML.EXPERTS_NVFP4 if fmt == "nvfp4" else ML.EXPERTS_FP8, tables[c % 2], rows,
                                   shared_inter=bI, sh_payload=[t[0] for t in shared[c]], sh_scales=[t[1] for t in shared[c]],
                                   router_gate=gate, router_bias=bias) for c in range(NX)]
                x = torch.from_numpy(hg.normal_bf16(0xD6996300 + rows, (NX, rows, bH)).view(np.int16)).to(dev)
                out = torch.empty((NX, rows, bH), dtype=torch.int16, device=dev)

                def step(i):
                    c = i % NX
                    lay[c].enqueue_decode(x[c], bH, out[c], rows, stream)
                sec = time_graph(step, args.steps, args.warmup)
                # the reference's accounting: rows * (top_k experts + the shared one), no expert sharing
                slot_bytes = rows * (bK * per_expert + shared_bytes)
                res[f"{fmt}_rows{rows}"] = {
                    "us": sec * 1e6,
                    "reference_published_us_on_gb10": published[fmt].get(rows),
                    "slot_bytes_no_expert_sharing": slot_bytes,
                    "slot_gbps": slot_bytes / sec / 1e9,
                    "frac_of_peak": slot_bytes / sec / 1e9 / HBM_PEAK_GBPS}
                for l_ in lay:
                    l_.close()
            del keep, tables, gen
            torch.cuda.empty_cache()
        return res

    def bench_w8a8():
        """The activation-quantized MXFP8 GEMM at the C5 shared expert's projection shapes, swept over the row count
        (not one of the headline benchmark's configurations: run with --configs w8a8). Weights rotate so that no launch finds them cached."""
        res = {"workload": "MXFP8 x MXFP8 block-scaled GEMM (scaled matrix-core instruction), rotating weights"}
        for n, k in ((4096, 6144), (6144, 4096)):
            pw, sw = hg.encode_mxfp8(hg.normal_f32(0xD6996000 + n, (n, k), 0.02))
            ring = ring_copies([torch.from_numpy(pw).to(dev), torch.from_numpy(sw).to(dev)], pw.nbytes)
            for m in (1, 16, 64, 256):
                x = torch.from_numpy(hg.normal_bf16(0xD6996100 + m, (m, k)).view(np.int16)).to(dev)
                xq = torch.empty((m, k), dtype=torch.uint8, device=dev)
                xs = torch.empty((m, k // 32), dtype=torch.uint8, device=dev)
                out = torch.empty((m, n), dtype=torch.int16, device=dev)
                L.launch_mxfp8_quantize_rows(x, k, m, k, xq, xs, stream)

                def step(i):
                    r = i % len(ring)
                    L.launch_mxfp8_gemm_bf16(xq, xs, ring[r][0], ring[r][1], out, m, n, k, stream)

                def quant(i):
                    L.launch_mxfp8_quantize_rows(x, k, m, k, xq, xs, stream)

                sec = time_graph(step, args.steps, args.warmup)
                nbytes = (n + m) * k * 33 // 32 + m * n * 2
                res[f"gemm_m{m}_n{n}_k{k}"] = {"us": sec * 1e6, "algorithmic_bytes": nbytes, "gbps": nbytes / sec / 1e9,
                                              "frac_of_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                                              "tflops": 2.0 * m * n * k / sec / 1e12}
                qsec = time_graph(quant, args.steps, args.warmup)
                res[f"quantize_rows{m}_k{k}"] = {"us": qsec * 1e6}
        return res

    def bench_qwen_tail():
        """The gated shared expert's decode tail (block-FP8 weights, hidden 2048, shared inter 512) in its two launches
        against the seven-launch chain it is bitwise equal to (not one of the headline benchmark's configurations: --configs qwen_tail)."""
        H, S, K = 2048, 512, 10
        res = {"workload": f"gated shared expert decode tail, FP8 block-128, hidden {H}, inter {S}: two launches vs the unfused chain"}
        mats = [hg.encode_fp8_blocks(hg.f32_to_bf16(hg.normal_f32(0xD6997000 + i, shape, 0.03)), 128, 128)
                for i, shape in enumerate(((S, H), (S, H), (H, S)))]
        ring = ring_copies([torch.from_numpy(a).to(dev) for pair in mats for a in pair], sum(p.nbytes for p, _ in mats))
        gvec = torch.from_numpy(hg.normal_bf16(0xD6997010, (H,), 0.03).view(np.int16)).to(dev)
        for T in (1, 8):
            x = torch.from_numpy(hg.normal_bf16(0xD6997020 + T, (T, H)).view(np.int16)).to(dev)
            contrib = torch.from_numpy(hg.normal_f32(0xD6997030 + T, (T * (K + 1), H), 0.3)).to(dev)
            wts = torch.from_numpy(np.abs(hg.normal_f32(0xD6997040 + T, (T, K), 0.2)).astype(np.float32)).to(dev)
            act, g_o, u_o = (torch.empty((T, S), dtype=torch.int16, device=dev) for _ in range(3))
            sw = torch.empty((T,), dtype=torch.float32, device=dev)
            down = torch.empty((T, H), dtype=torch.float32, device=dev)
            routed = torch.empty((T, H), dtype=torch.float32, device=dev)
            out = torch.empty((T, H), dtype=torch.int16, device=dev)
            rows_id = torch.arange(T, dtype=torch.int32, device=dev)

            def fused(i):
                gp, gs, up, us, dp, ds = ring[i % len(ring)]
                L.qwen_moe_shared_tail_decode_routed_fp8(x, H, gp, gs, up, us, dp, ds, gvec, act, sw, contrib, wts, K, out, T, H, S,
                                                         stream)

            def chain(i):
                gp, gs, up, us, dp, ds = ring[i % len(ring)]
                L.launch_scale_gemm_grid_bf16(x, H, gp, gs, g_o, T, S, H, stream, 0, 7, 7)
                L.launch_scale_gemm_grid_bf16(x, H, up, us, u_o, T, S, H, stream, 0, 7, 7)
                L.launch_moe_swiglu_clamp(g_o, u_o, act, T * S, float("inf"), stream)
                L.launch_scale_gemm_grid_f32(act, S, dp, ds, down, T, H, S, stream, 0, 7, 7)
                L.qwen_moe_shared_gate_bf16(x, gvec, sw, T, H, stream)
                L.launch_moe_slot_accum_routed_f32(routed, contrib, wts, T, H, K, stream)
                L.launch_moe_accum(routed, down, rows_id, sw, T, H, stream)
                L.launch_moe_round_bf16(out, routed, T * H, stream)

            nbytes = 3 * S * H + 3 * (S // 128) * (H // 128) * 4 + T * H * 2 + T * (K + 1) * H * 4 + T * H * 2
            for name, fn in (("two_launches", fused), ("unfused_chain", chain)):
                sec = time_graph(fn, args.steps, args.warmup)
                res[f"T{T}_{name}"] = {"us": sec * 1e6, "algorithmic_bytes": nbytes, "gbps": nbytes / sec / 1e9,
                                       "frac_of_peak": nbytes / sec / 1e9 / HBM_PEAK_GBPS}
        return res

    def bench_readprobe():
        """The plain-read ceiling of this chip (not one of the headline benchmark's configurations: --configs readprobe):
        the library's streaming read kernel (16-byte loads, eight in flight per lane, nothing stored) over a 1 GiB buffer
        (every launch cold: four times the 256 MB Infinity Cache) and over a 128 MiB buffer read again and again (served
        by the Infinity Cache), by grid size, access pattern (one contiguous span per block / the grid striding together)
        and load form (plain / nontemporal). A weight-streaming kernel cannot beat the best of these rates."""
        res = {"workload": "plain streaming read, 16 bytes per lane, blocks of 256 threads"}
        sink = torch.zeros(8192, dtype=torch.int32, device=dev)
        best = {}
        for label, mib in (("cold_1GiB", 1024), ("cache_resident_128MiB", 128)):
            buf = torch.zeros(mib << 20, dtype=torch.uint8, device=dev)
            for blocks in (512, 1024, 2048, 4096, 8192):
                for span in (1, 0):
                    for nt in (0, 1):
                        def step(i):
                            if lib.dgpp_probe_read(buf.data_ptr(), buf.numel(), sink.data_ptr(), nt, blocks, span,
                                                   stream.cuda_stream) != 0:
                                raise RuntimeError(lib.dgpp_last_error().decode())
                        st = {}
                        sec = time_graph(step, 8, 2, st)
                        key = f"{label}_blocks{blocks}_{'span' if span else 'stride'}_{'nontemporal' if nt else 'plain'}"
                        res[key] = {"us": sec * 1e6, "gbps": buf.numel() / sec / 1e9, "us_min": st["us_min"], "us_max": st["us_max"]}
                        if label not in best or res[key]["gbps"] > best[label][1]:
                            best[label] = (key, res[key]["gbps"])
            del buf
        # What ONE cold launch of a given size costs (the yardstick for the small-batch GEMV launches, which read
        # 17 - 60 MB each): successive launches read successive windows of a 1 GiB buffer, so every window has left the
        # caches by the time it is read again. Time per launch includes the hand-over to the next launch of the graph, as
        # a layer's dependent launches do.
        mib = 1024
        buf = torch.zeros(mib << 20, dtype=torch.uint8, device=dev)
        win = {}
        for w_mib in (16, 32, 48, 64, 128, 256):
            nwin = mib // w_mib
            wbytes = w_mib << 20
            for blocks in (1024, 2048, 4096):
                def step(i):
                    if lib.dgpp_probe_read(buf.data_ptr() + (i % nwin) * wbytes, wbytes, sink.data_ptr(), 0, blocks, 1,
                                           stream.cuda_stream) != 0:
                        raise RuntimeError(lib.dgpp_last_error().decode())
                sec = time_graph(step, max(16, nwin), 2)
                cur = win.get(w_mib)
                if cur is None or sec * 1e6 < cur["us"]:
                    win[w_mib] = {"us": sec * 1e6, "gbps": wbytes / sec / 1e9, "blocks": blocks}
        res["cold_window_per_launch"] = {f"{k}MiB": v for k, v in win.items()}
        del buf
        res["best"] = {k: {"form": v[0], "gbps": v[1], "frac_of_peak": v[1] / HBM_PEAK_GBPS} for k, v in best.items()}
        return res

    def bench_router():
        """The router's two launches (score rows, selection) at decode batch sizes: the one-row dots kernel against the
        token-tiled one (from 16 rows on), for the C3 (256 x 4096) and C5 (256 x 6144) router shapes. The gate stays
        cache-resident here (2-3 MB), as it does between a layer's steps."""
        res = {}
        for name, (rE, rH, rK) in (("c3_256x4096", (256, 4096, 8)), ("c5_256x6144", (256, 6144, 8))):
            rcfg = L.make_config(rH, 64, rE, rK, n_shared_experts=0, routed_scaling_factor=1.0, router_mode=L.ROUTER_SOFTMAX_TOPK)
            gate = torch.from_numpy(hg.normal_bf16(0xD6990400, (rE, rH), 1.0 / np.sqrt(rH)).view(np.int16)).to(dev)
            for T in (16, 32, 64, 128):
                x = torch.from_numpy(hg.normal_bf16(0xD6990401 + T, (T, rH)).view(np.int16)).to(dev)
                ids, w = torch.empty((T, rK), dtype=torch.int32, device=dev), torch.empty((T, rK), dtype=torch.float32, device=dev)
                sc, bi = torch.empty((T, rE), dtype=torch.float32, device=dev), torch.empty((T, rE), dtype=torch.float32, device=dev)
                for tiled, tt in ((False, 0), (True, 2), (True, 4)):
                    def step(i):
                        L.launch_moe_router(x, gate, None, ids, w, sc, bi, rcfg, T, stream, None, tiled)
                    lib.dgpp_tune_set(10, tt)         # tokens per wavefront of the tiled form
                    sec = time_graph(step, args.steps, args.warmup)
                    lib.dgpp_tune_set(10, 0)
                    res[f"{name}_T{T}_{f'tiled{tt}' if tiled else 'one_row'}"] = {"us": sec * 1e6}
        res["workload"] = "router: score rows + selection, two launches, softmax top-8"
        return res

    def bench_pair():
        """Two FP8 projections of one k in one matrix-core launch against two launches (the reference's decode pair:
        launch_mma_gemv_fp8_bf16_pair), cold weights, with and without a split-K workspace."""
        res = {"workload": "two block-FP8 projections (n 1536 and 576, k 7168) of one batch: one launch against two"}
        k, n0, n1 = 7168, 1536, 576
        mats = []
        for i, n in enumerate((n0, n1)):
            p_, s_ = hg.encode_fp8_blocks(hg.f32_to_bf16(hg.normal_f32(0xD6990500 + i, (n, k), 0.02)), 128, 128)
            mats.append((torch.from_numpy(p_).to(dev), torch.from_numpy(s_).to(dev)))
        ring = ring_copies([mats[0][0], mats[0][1], mats[1][0], mats[1][1]], sum(t.numel() for m_ in mats for t in m_[:1]))
        for m in (1, 8):
            act = torch.from_numpy(hg.normal_bf16(0xD6990510 + m, (m, k)).view(np.int16)).to(dev)
            o0 = torch.empty((m, n0), dtype=torch.int16, device=dev)
            o1 = torch.empty((m, n1), dtype=torch.int16, device=dev)
            ws = torch.empty(4 * m * (n0 + n1), dtype=torch.float32, device=dev)
            for use_ws in (False, True):
                w_, wb = (ws, ws.numel() * 4) if use_ws else (None, 0)
                def one(i):
                    r = ring[i % len(ring)]
                    L.launch_mma_gemv_fp8_bf16_pair(act, r[0], r[1], o0, n0, 0, act, r[2], r[3], o1, n1, 0, k, m, k, 7, 7, stream, w_, wb)
                def two(i):
                    r = ring[i % len(ring)]
                    L.launch_mma_gemv_fp8_bf16(act, k, r[0], r[1], o0, m, n0, k, 0, 7, 7, stream, w_, wb)
                    L.launch_mma_gemv_fp8_bf16(act, k, r[2], r[3], o1, m, n1, k, 0, 7, 7, stream, w_, wb)
                tag = f"m{m}_{'split_k' if use_ws else 'unsplit'}"
                res[tag + "_one_launch"] = {"us": time_graph(one, args.steps, args.warmup) * 1e6}
                res[tag + "_two_launches"] = {"us": time_graph(two, args.steps, args.warmup) * 1e6}
        return res

    def bench_dispatch():
        """What the dense launchers' choice between the two cores rests on: one to eight rows against cold weights of
        several sizes on the vector core, on the matrix core unsplit (row tiles only, or the K parts side by side inside
        sixteen-wavefront blocks), and on the matrix core with a split-K workspace
        (us per launch; --configs dispatch)."""
        res = {"workload": "dense GEMV by row count: vector core / matrix core / matrix core with a split-K workspace, cold weights"}
        cases = [("fp8", 1536, 7168), ("fp8", 4096, 4096), ("fp8", 12288, 6144), ("nvfp4", 2048, 4096), ("nvfp4", 8192, 4096),
                 ("nvfp4", 17408, 5120), ("mxfp4", 6144, 2048), ("mxfp4", 17408, 5120)]
        for kind, n, k in cases:
            w = hg.normal_f32(0xD6990600 + n, (n, k), 0.02)
            glob = None
            if kind == "fp8":
                p_, s_ = hg.encode_fp8_blocks(hg.f32_to_bf16(w), 128, 128)
            elif kind == "nvfp4":
                p_, s_, ws2 = hg.encode_nvfp4(w)
                glob = torch.tensor([1.0 / np.float32(ws2)], dtype=torch.float32, device=dev)
            else:
                p_, s_ = hg.encode_mxfp4(w)
            ring = ring_copies([torch.from_numpy(p_).to(dev), torch.from_numpy(s_).to(dev)], p_.nbytes)
            mats = None if kind == "fp8" else [L.Fp4Matrix(r[0].data_ptr(), r[1].data_ptr(), glob.data_ptr() if glob is not None else None,
                                                            n, k, 16 if kind == "nvfp4" else 32, 0, None) for r in ring]
            for m in (1, 2, 4, 5, 6, 8):
                act = torch.from_numpy(hg.normal_bf16(0xD6990610 + m, (m, k)).view(np.int16)).to(dev)
                out = torch.empty((m, n), dtype=torch.int16, device=dev)
                ws = torch.empty(4 * m * n, dtype=torch.float32, device=dev)
                row = {}
                for name, core, w_, teams in (("vector_core", 1, None, 0), ("matrix_core", 2, None, 1),
                                              ("matrix_core_parts_side_by_side", 2, None, 2), ("matrix_core_split_k", 2, ws, 0)):
                    wb = ws.numel() * 4 if w_ is not None else 0
                    def step(i):
                        r = i % len(ring)
                        if kind == "fp8":
                            L.launch_mma_gemv_fp8_bf16(act, k, ring[r][0], ring[r][1], out, m, n, k, 0, 7, 7, stream, w_, wb)
                        elif w_ is None:
                            L.launch_fp4_gemv_bf16(act, k, mats[r], out, m, n, k, stream)
                        else:
                            L.launch_mma_gemv_fp4_bf16(act, k, mats[r], out, m, n, k, 0, stream, w_, wb)
                    lib.dgpp_tune_set(5, core)
                    lib.dgpp_tune_set(11, teams)   # K parts side by side in sixteen-wavefront blocks: 1 never, 2 always
                    row[name] = time_graph(step, 32, 3) * 1e6
                    lib.dgpp_tune_set(5, 0)
                    lib.dgpp_tune_set(11, 0)
                lib.dgpp_tune_set(5, 0)
                def chosen(i):
                    r = i % len(ring)
                    if kind == "fp8":
                        L.launch_mma_gemv_fp8_bf16(act, k, ring[r][0], ring[r][1], out, m, n, k, 0, 7, 7, stream, None, 0)
                    else:
                        L.launch_fp4_gemv_bf16(act, k, mats[r], out, m, n, k, stream)
                row["launcher_without_workspace"] = time_graph(chosen, 32, 3) * 1e6
                res[f"{kind}_{n}x{k}_m{m}"] = {"us": row["launcher_without_workspace"], **{k_: round(v, 2) for k_, v in row.items()}}
            del ring, mats
            torch.cuda.empty_cache()
        return res

    other_configs = {}
    configs = args.configs if args.configs is not None else ("" if args.tune else "c1,c2,c4,c5")
    if not args.only:
        for name in filter(None, configs.split(",")):
            t0 = time.time()
            other_configs[name] = {"c1": bench_c1, "c2": bench_c2, "c2round": bench_c2round, "c4": bench_c4, "c5": bench_c5, "c5skew": lambda: bench_c5(True), "w8a8": bench_w8a8, "qwen_tail": bench_qwen_tail, "readprobe": bench_readprobe,
                                   "slotbench": bench_slotbench, "router": bench_router, "pair": bench_pair, "dispatch": bench_dispatch}[name]()
            other_configs[name]["setup_and_run_seconds"] = time.time() - t0
            torch.cuda.empty_cache()

    # ---- CPU baseline: the oracle's layer forward (dequantise to double, fp64 dots) on a bounded sample ----
    cpu = None
    if not args.no_cpu and not args.only:
        sys.path.insert(0, str(ROOT / "tests"))
        import oracle_lib as orc
        xs, lg_d, lg = inputs(1)
        l64 = lg[0].astype(np.float64)
        ids = np.empty((1, K), np.int32)
        w = np.empty((1, K), np.float32)
        orc.oracle().orc_router_select(orc.p(l64), orc.p(l64), 1, 1, nE, K, 1.0, 1, orc.p(ids), orc.p(w))
        mats, hold = [], []
        zero8 = np.zeros(1, np.uint8)
        used = set(int(v) for v in ids.ravel())
        for e in range(nE):
            for m in range(3):
                if e in used:
                    pa = (gu_p[e, m] if m < 2 else dn_p[e]).numpy()
                    sa = (gu_s[e, m] if m < 2 else dn_s[e]).numpy()
                    hold += [pa, sa]
                    mats.append(orc.make_matrix(1, pa, sa, group=32))
                else:
                    mats.append(orc.make_matrix(1, zero8, zero8, group=32))
        xl = hg.normal_bf16(0xD6990000 + 3 * 16 + 1, (nL, 1, H))      # the bench's own T=1 inputs, one row per ring layer
        x1 = xl[0]
        cores = min(16, os.cpu_count() or 1)
        # a bounded sample, about 10 s of CPU work: the same layer pass over different token rows
        n_one, n_many = 6, 48
        t0 = time.time()
        for r in range(n_one):
            raw_r, _ = orc.moe_forward(np.ascontiguousarray(xl[r % nL]), ids, w, H, I, I, mats, None, float("inf"), threads=1)
            if r == 0:
                raw1 = raw_r
        t_one = (time.time() - t0) / n_one
        t0 = time.time()
        for r in range(n_many):
            orc.moe_forward(np.ascontiguousarray(xl[r % nL]), ids, w, H, I, I, mats, None, float("inf"), threads=cores)
        t_many = (time.time() - t0) / n_many
        bytes1 = K * EXPERT_BYTES + 2 * H * 2 + K * 8
        cpu = {"value": bytes1 / t_many / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": f"{n_many} layer passes at T=1 (8 experts, 53.5 MB each) on {cores} threads and {n_one} on one thread "
                         "through the CPU oracle: weights dequantised to double, fp64 dots, reference rounding points",
               "us_per_layer": t_many * 1e6, "single_thread_us_per_layer": t_one * 1e6,
               "single_thread_gbps": bytes1 / t_one / 1e9}
        # the same pass on the GPU must agree with what was just computed on the CPU
        out1 = torch.empty((1, H), dtype=torch.int16, device=dev)
        layers[0].enqueue_decode_scores(xs[0], H, lg_d[0], lg_d[0], out1, 1, None)
        torch.cuda.synchronize()
        got_bits = out1.cpu().numpy().view(np.uint16)
        got = hg.bf16_to_f32(got_bits).astype(np.float64)[0]
        ref = raw1[0]
        floor = 0.02 * float(np.sqrt(np.mean(ref ** 2)))
        # against the unrounded fp64 oracle: the raw figure carries the bf16 output's own rounding (up to 2^-8 = 3.9e-3),
        # the second one is the error beyond that rounding (the parity tests' measure, bound 2e-3)
        cpu["gpu_vs_cpu_max_rel"] = float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), floor)))
        cpu["gpu_vs_cpu_beyond_bf16_rounding"] = orc.north_star_rel(got_bits[0], ref)

        # ---- the reference's OWN CPU oracle (compiled from its sources into oracle/_ref), where that was built ----
        # glm_moe_ref_forward at the same layer shape: router GEMV over the hidden row, 8 routed experts and the
        # shared expert it always runs (here: expert 0's matrices once more), single-threaded, weights dequantised
        # to double per use. Timed on a few token rows; its output must equal the port's bit for bit.
        ref_lib = orc.ref()
        if ref_lib is not None and hasattr(ref_lib, "ref_moe_layer_create"):
            mat_pay = [3 * I * H // 2 // 3] * 3                      # gate, up, down payload bytes (equal sizes)
            mat_sc = [I * H // 32] * 3
            pay = np.empty((nE + 1) * sum(mat_pay), np.uint8)
            sc = np.empty((nE + 1) * sum(mat_sc), np.uint8)
            for e in range(nE + 1):
                src = e % nE                                          # the shared triple = expert 0's matrices
                po, so = e * sum(mat_pay), e * sum(mat_sc)
                for m in range(3):
                    pm = (gu_p[src, m] if m < 2 else dn_p[src]).numpy().ravel()
                    sm = (gu_s[src, m] if m < 2 else dn_s[src]).numpy().ravel()
                    pay[po + m * mat_pay[0]: po + (m + 1) * mat_pay[0]] = pm
                    sc[so + m * mat_sc[0]: so + (m + 1) * mat_sc[0]] = sm
            gate = hg.normal_bf16(0xD6990200, (nE, H), std=1.0 / 64.0)   # logits = x . gate ~ N(0, 1)
            ref_layer = ref_lib.ref_moe_layer_create(H, I, nE, K, 1, 1.0, 1, float("inf"), orc.p(gate), None, 32, orc.p(pay),
                                                     pay.size, orc.p(sc), sc.size, None, 0)
            if ref_layer:
                n_ref = 8
                ref_out = np.empty((1, H), np.uint16)
                row0 = np.ascontiguousarray(xl[0])
                t0 = time.time()
                for r in range(n_ref):
                    row = np.ascontiguousarray(xl[r % nL])
                    rc = ref_lib.ref_moe_layer_forward(ref_layer, orc.p(row), 1, orc.p(ref_out))
                    assert rc == 0, "the reference oracle threw"
                t_ref = (time.time() - t0) / n_ref
                # the port on the reference's own routing of row 0 (its router is the reference's, bit for bit: tests)
                rc = ref_lib.ref_moe_layer_forward(ref_layer, orc.p(row0), 1, orc.p(ref_out))
                rid, rw, rb = np.empty((1, K), np.int32), np.empty((1, K), np.float32), np.empty((1, nE), np.float64)
                ref_lib.ref_router(orc.p(row0), orc.p(gate), None, 1, 1, nE, H, K, 1.0, 1, orc.p(rid), orc.p(rw), orc.p(rb))
                used_r = set(int(v) for v in rid.ravel()) | {0}
                mats_r, hold_r = [], []
                for e in range(nE):
                    for m in range(3):
                        if e in used_r:
                            pa = (gu_p[e, m] if m < 2 else dn_p[e]).numpy()
                            sa = (gu_s[e, m] if m < 2 else dn_s[e]).numpy()
                            hold_r += [pa, sa]
                            mats_r.append(orc.make_matrix(1, pa, sa, group=32))
                        else:
                            mats_r.append(orc.make_matrix(1, zero8, zero8, group=32))
                _, port_bits = orc.moe_forward(row0, rid, rw, H, I, I, mats_r, mats_r[0:3], float("inf"), threads=cores)
                ref_lib.ref_moe_layer_destroy(ref_layer)
                bytes_ref = (K + 1) * EXPERT_BYTES + nE * H * 2 + 2 * H * 2
                port = dict(cpu)
                cpu = {"value": bytes_ref / t_ref / 1e9, "unit": "GB/s", "cores": 1, "kind": "reference",
                       "sample": f"{n_ref} T=1 passes of the reference's own glm_moe_ref_forward (compiled from its sources: router "
                                 f"GEMV + 8 routed MXFP4 experts + the shared expert it always runs = {bytes_ref / 1e6:.1f} MB per "
                                 "pass), one thread as the reference runs it. NOT the GPU's workload one to one: a GPU T=1 "
                                 f"pass is 8 routed experts and no router GEMV ({(K * EXPERT_BYTES) / 1e6:.1f} MB); compare the GB/s, "
                                 "not us_per_layer. `port` times exactly the GPU's T=1 workload (8 experts, given logits)",
                       "us_per_layer": t_ref * 1e6,
                       "port_equals_reference_bits": bool(np.array_equal(port_bits, ref_out)),
                       "gpu_vs_cpu_max_rel": port.pop("gpu_vs_cpu_max_rel"),
                       "gpu_vs_cpu_beyond_bf16_rounding": port.pop("gpu_vs_cpu_beyond_bf16_rounding"),
                       "port": port}
                del pay, sc

    sec = main_res.get("us_per_layer", float("nan")) * 1e-6
    line = {
        "metric": "MXFP4 MoE decode layer achieved HBM GB/s (algorithmic bytes / time) on 1 MI355X",
        "value": main_res.get("gbps"),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec * 1e3,
        "us_per_layer": main_res.get("us_per_layer"),
        "frac_of_hbm_peak": main_res.get("frac_of_peak"),
        # the reference's own bench counts rows * top_k * per-expert bytes ("no expert sharing", benchmarks/micro/moe_slot_bench.cu:238-264)
        "reference_style_slot_gbps": (T * K * EXPERT_BYTES / sec / 1e9) if sec == sec else None,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic: layer 0 host-generated N(0,0.02) weights MXFP4-quantised (E2M1 + E8M0/32, ceil-pow2 "
                "scales); the other ring layers are device copies with the experts rotated; x ~ N(0,1) bf16, "
                "router logits ~ N(0,1)",
        "config": {"workload": f"BASELINE config 3: MXFP4 MoE decode layer, {nE} experts, hidden {H}, inter {I}, "
                               f"top-{K} softmax-renormalised, no shared expert, T={T} tokens",
                   "tokens": T, "ring_layers": nL, "timing": "median over back-to-back replays (>= 50, >= 1000 layer passes) of one HIP graph of "
                   "`steps` layer passes rounded up to whole walks of the layer ring (at least four), an event on the launch stream between "
                   "replays; weights cold (ring >= 2x the 256 MB cache)",
                   "timing_stats": main_res.get("timing"),
                   "distinct_experts_mean": main_res["distinct_experts_mean"],
                   "algorithmic_bytes_per_layer": main_res["algorithmic_bytes"]},
        "roofline": None,
        "cpu_baseline": cpu,
        "headline_legs": {k: v for k, v in main_res.items() if k.startswith(("gate_up_", "down_"))},
        "other_batches": others,
        "other_configs": other_configs,
        "build_seconds": build_s,
    }
    traffic = measured_traffic()
    same_workload = T == 8 and nE == E and not args.tune
    if "gate_up_us" in main_res:
        line["roofline"] = {"kernel": "slot_gate_up_kernel<MXFP4> (fused gate/up GEMV + SwiGLU)", "bound": "hbm",
                            "achieved": main_res["gate_up_gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                            "frac": main_res["gate_up_gbps"] / HBM_PEAK_GBPS,
                            "traffic": traffic.get("gate_up") if same_workload else None,
                            "traffic_source": ((TRAFFIC_PROFILE + ": " + traffic.get("gate_up_kernel", "") + ", kernel sources " +
                                                traffic["digest"]) if "digest" in traffic else
                                               (TRAFFIC_PROFILE + " was taken from kernel sources " + str(traffic.get("stale")) +
                                                ", the tree holds " + str(traffic.get("tree")) + ": not used")
                                               if "stale" in traffic else None) if same_workload else None,
                            "bytes_per_launch": main_res["gate_up_bytes"], "us_per_launch": main_res["gate_up_us"]}
        if "gate_up_plain_read_us" in main_res:   # this chip's plain cold read of the same byte count, same timing method
            line["roofline"]["plain_read_same_bytes_us"] = main_res["gate_up_plain_read_us"]
            line["roofline"]["frac_of_plain_read"] = main_res["gate_up_frac_of_plain_read"]
        if "down_us" in main_res:
            line["roofline"]["second_kernel"] = {
                "kernel": "token_down_accum_kernel<MXFP4> (down GEMV + ordered accumulation, bf16 out)",
                "achieved": main_res["down_gbps"],
                "traffic": traffic.get("down") if same_workload else None,
                "frac": main_res["down_gbps"] / HBM_PEAK_GBPS, "bytes_per_launch": main_res["down_bytes"],
                "us_per_launch": main_res["down_us"]}
            if "down_plain_read_us" in main_res:
                line["roofline"]["second_kernel"]["plain_read_same_bytes_us"] = main_res["down_plain_read_us"]
                line["roofline"]["second_kernel"]["frac_of_plain_read"] = main_res["down_frac_of_plain_read"]
    print(json.dumps(line))


if __name__ == "__main__":
    main()
