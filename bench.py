#!/usr/bin/env python3
"""Headline benchmark of the MFQ packed-weight matmul path on one MI355X.

A step is one decode pass over the three NINT4 (4,32,6) FFN projections of BASELINE config 2 at
batch 1 (gate and up 12288x4096, down 4096x12288).  Gate and up share their input, so they are kept
as one row-concatenated weight and run as one launch (the reference's NintLinearGroup); down is the
second launch.  Steps rotate over `--copies` distinct weight sets so the 83 MB a step reads never
sits in the 256 MB Infinity Cache.
`value` = algorithmic bytes (compact MFQ payload + bf16 x + fp32 y) / wall time of the timed steps.
Inputs are resident in HBM before the timed region.  One JSON line goes to stdout; the rest to stderr.

    python bench.py [--gpus 1] [--steps 200] [--warmup 30] [--copies 8] [--no-extras]
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense fp16/bf16 MFMA


def log(*a):
    print(*a, file=sys.stderr, flush=True)


TRAFFIC_PROFILE = ROOT / "profiles" / "nint_gemv_xreg_4_32_config2_decode.md"


def profiled_traffic():
    """HBM bytes per launch of the headline kernel as measured with rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE, scaled by a
    plain copy): the line `TRAFFIC_BYTES_PER_LAUNCH = <bytes>` of the committed profile summary, or None."""
    import re
    try:
        m = re.search(r"^TRAFFIC_BYTES_PER_LAUNCH\s*=\s*([0-9.eE+]+)", TRAFFIC_PROFILE.read_text(), re.M)
    except OSError:
        return None
    return float(m.group(1)) if m else None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--copies", type=int, default=8)
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run a plain 256 MiB device copy 20 times (the reference kernel the HBM counters of a "
                         "rocprofv3 --pmc run are scaled by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no sharding, no collectives); use --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from tyloquant_amd import _lib as L
    from tyloquant_amd import runtime as R
    from tyloquant_amd import synth

    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    lib = L.lib()
    rng = np.random.default_rng(2)
    t0 = time.time()

    # ---- BASELINE config 2 weights: NINT4 (4,32,6), N(0, 0.02) ---------------------------------
    H, FF = 4096, 12288
    shapes = {"gate": (FF, H), "up": (FF, H), "down": (H, FF)}
    blobs = {}
    for i, (name, (n, k)) in enumerate(shapes.items()):
        blobs[name] = synth.nint_linear_blob(100 + i, n, k, 4, 32, 6, slab_rows=1024)[1]
    base = {"gate_up": (R.NintLinearGroup.from_blobs([blobs["gate"], blobs["up"]]).w, None),
            "down": (R.load_quant_linear("NINT4", blobs["down"]).weight, blobs["down"]),
            "gate": (R.load_quant_linear("NINT4", blobs["gate"]).weight, blobs["gate"])}
    for name in ("gate_up", "down"):
        log(f"[bench] {name} {base[name][0].out}x{base[name][0].neuron_len} NINT4-32 payload "
            f"{base[name][0].payload_bytes} B ({time.time() - t0:.1f}s)")
    launches = ("gate_up", "down")
    lshape = {"gate_up": (2 * FF, H), "down": (H, FF)}

    def clone(w):
        c = R.NintWeight(w.desc, w.data.clone(), w.shape)
        return c

    sets = [{n: (base[n][0] if c == 0 else clone(base[n][0])) for n in launches} for c in range(args.copies)]
    sets[0]["gate"] = base["gate"][0]
    x_h = torch.from_numpy(synth.activations(rng, 1, H, outlier_frac=0.001)).to(torch.bfloat16).to(dev)
    x_f = torch.from_numpy(synth.activations(rng, 1, FF)).to(torch.bfloat16).to(dev)
    y = {n: torch.empty((1, lshape[n][0]), dtype=torch.float32, device=dev) for n in launches}
    step_bytes = sum(base[n][0].payload_bytes + 2 * lshape[n][1] + 4 * lshape[n][0] for n in launches)
    n_per_step = len(launches)

    def launch(wset, stream):
        for n in launches:
            w = wset[n]
            x = x_f if n == "down" else x_h
            rc = lib.mfq_hip_nint_gemv(C.byref(w.desc), w.data.data_ptr(), x.data_ptr(), L.X_BF16, x.stride(0), 1,
                                       y[n].data_ptr(), lshape[n][0], stream)
            if rc:
                L.check(rc)

    def stream_ptr():
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    # Decode runs under HIP graphs.  One graph = one pass over all weight sets; a second, shorter graph covers the
    # steps left over when --steps is not a multiple of the number of sets, so that a timed window of exactly
    # --steps steps is graph replays only.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch(sets[0], stream_ptr())
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    per_replay = len(sets)
    full, rest = divmod(args.steps, per_replay)

    def capture(nsets):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for s_ in sets[:nsets]:
                launch(s_, stream_ptr())
        return g
    graph = capture(per_replay)
    graph_rest = capture(rest) if rest else None

    def run_steps(nsteps):
        f, r = divmod(nsteps, per_replay)
        for _ in range(f):
            graph.replay()
        if r == rest and graph_rest is not None:
            graph_rest.replay()
        else:
            for i in range(r):
                launch(sets[i], stream_ptr())

    run_steps(args.warmup)
    torch.cuda.synchronize()
    # Timed region: `windows` windows of exactly --steps steps each, every window bracketed by a device synchronisation
    # on both sides (wall clock) and by HIP events on the launch stream; the line reports the median window.
    windows = max(5, -(-200 // max(1, args.steps * n_per_step)))
    walls, gpus = [], []
    for _ in range(windows):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t_start = time.perf_counter()
        e0.record()
        run_steps(args.steps)
        e1.record()
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t_start)
        gpus.append(e0.elapsed_time(e1))
    wall = float(np.median(walls))
    gpu_ms = float(np.median(gpus))
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes * args.steps / wall / 1e9
    n_launch = n_per_step * args.steps
    avg_launch_us = gpu_ms * 1e3 / n_launch
    bytes_per_launch = step_bytes / float(n_per_step)
    achieved = bytes_per_launch / (avg_launch_us * 1e-6) / 1e9
    log(f"[bench] decode C2 M=1: {value:.1f} GB/s whole-job (median of {windows} windows of {args.steps} steps; "
        f"min {step_bytes * args.steps / max(walls) / 1e9:.0f}, max {step_bytes * args.steps / min(walls) / 1e9:.0f}), "
        f"{avg_launch_us:.2f} us/launch by HIP events -> {achieved:.1f} GB/s per launch")

    # parity guard on what was just timed (size-independent property: linearity in x)
    launch(sets[0], stream_ptr())
    torch.cuda.synchronize()
    y1 = y["gate_up"][:, :FF].clone()
    x2 = (x_h.float() * 2).to(torch.bfloat16)
    yy = R.nint_matmul(sets[-1]["gate_up"], x2, force="gemv")[:, :FF]
    lin_err = float(((yy - 2 * y1).norm() / (2 * y1).norm()).item())
    assert lin_err < 1e-5, f"GEMV is not linear in x / copies differ: {lin_err}"

    extras = {"linearity_rel_err": lin_err, "gpu_ms_median_window": gpu_ms, "windows": windows,
              "value_min_gbps": step_bytes * args.steps / max(walls) / 1e9,
              "value_max_gbps": step_bytes * args.steps / min(walls) / 1e9,
              "launch_us_min_window": min(gpus) * 1e3 / n_launch, "launch_us_max_window": max(gpus) * 1e3 / n_launch}

    # What the memory system gives a read-only launch, measured in this run: one kernel that only reads, (a) 1 GiB in
    # one launch (the streaming ceiling), (b) buffers of the two GEMV launches' sizes, rotating over 8 copies in a graph
    # exactly like the timed steps (start-up and drain of a launch of that size included).
    def read_probe_gbps(nbytes, ncopies, reps):
        bufs = [torch.empty(nbytes, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(ncopies)]
        sink = torch.zeros(16, dtype=torch.int32, device=dev)

        def go():
            for b in bufs:
                rc = lib.mfq_hip_read_probe(b.data_ptr(), nbytes, sink.data_ptr(), stream_ptr())
                if rc:
                    L.check(rc)
        s2 = torch.cuda.Stream()
        s2.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s2):
            go()
        torch.cuda.current_stream().wait_stream(s2)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            go()
        g.replay()
        torch.cuda.synchronize()
        ts = []
        for _ in range(5):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(reps):
                g.replay()
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b) / (reps * ncopies))
        del bufs
        return nbytes / (float(np.median(ts)) * 1e-3) / 1e9, float(np.median(ts)) * 1e3
    extras["hbm_read_ceiling_gbps"], _ = read_probe_gbps(1 << 30, 2, 3)
    for n in launches:
        gb, us = read_probe_gbps(int(base[n][0].desc.total_bytes), 8, 10)
        extras[f"read_only_{n}_gbps"], extras[f"read_only_{n}_us"] = gb, us
    ro_us = 0.5 * (extras["read_only_gate_up_us"] + extras["read_only_down_us"])
    extras["launch_us_vs_read_only_launch"] = avg_launch_us / ro_us
    log(f"[bench] read-only kernel: 1 GiB {extras['hbm_read_ceiling_gbps']:.0f} GB/s; gate_up-sized "
        f"{extras['read_only_gate_up_us']:.2f} us, down-sized {extras['read_only_down_us']:.2f} us per launch "
        f"(GEMV launches take {extras['launch_us_vs_read_only_launch']:.2f}x that)")
    torch.cuda.empty_cache()
    if args.calibrate:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def time_fn(fn, reps, warm=5):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps

    def graph_ms(fn, reps, warm=2):
        """ms per call of fn() when it is replayed from a HIP graph (decode runs under graphs)."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        for _ in range(warm):
            g.replay()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps

    def clone_w(w):
        import copy
        c = copy.copy(w)
        c.data = w.data.clone()
        if hasattr(w, "_ws"):
            c._ws = type(w._ws)()
        return c

    def bf16(a):
        return torch.from_numpy(a).to(torch.bfloat16).to(dev)

    cpu4_rows = None
    if not args.no_extras:
        from tyloquant_amd import formats as F
        from tyloquant_amd import runtime_vq as RV
        # hot (one weight set, cache-resident between launches)
        hot_ms = time_fn(lambda: launch(sets[0], stream_ptr()), 100)
        extras["decode_hot_gbps"] = step_bytes / (hot_ms * 1e-3) / 1e9
        # ---- config 2: batch sweep on the gate shape (GEMV up to 8 rows, MFMA path above) -------------
        wg = sets[0]["gate"]
        for M in (16, 512, 2048):
            xm = bf16(synth.activations(rng, M, H, outlier_frac=0.001))
            ms = time_fn(lambda: R.nint_matmul(wg, xm), 10, warm=3)
            extras[f"prefill_M{M}_tflops"] = 2.0 * M * FF * H / (ms * 1e-3) / 1e12
            extras[f"prefill_M{M}_ms"] = ms
            extras[f"prefill_M{M}_frac_of_f16_mfma_peak"] = extras[f"prefill_M{M}_tflops"] / MFMA_F16_PEAK_TFLOPS
        # ---- config 2: small batches on the gate+up tensor, rotating over the weight sets (graph replay) ---------
        one_us = None
        for M in (1, 2, 4, 8, 16):
            xm = bf16(synth.activations(rng, M, H, outlier_frac=0.001))
            us = graph_ms(lambda: [R.nint_matmul(s_["gate_up"], xm) for s_ in sets], 10) / len(sets) * 1e3
            one_us = one_us or us
            extras[f"small_batch_gate_up_M{M}_us"] = us
            extras[f"small_batch_gate_up_M{M}_vs_one_row"] = us / one_us
        log("[bench] config 2 gate+up 24576x4096 at 1/2/4/8/16 rows: " + ", ".join(
            f"{extras[f'small_batch_gate_up_M{M}_us']:.1f} us" for M in (1, 2, 4, 8, 16)))
        log(f"[bench] config 2 extras: {extras}")
        del sets[1:]
        torch.cuda.empty_cache()

        # ---- config 1: NINT3 (3,24,5) 4096x4096 at batch 1, rotating over 40 copies (310 MB) --------
        w1 = R.load_quant_linear("NINT3", synth.nint_linear_blob(7, 4096, 4096, 3, 24, 5, slab_rows=1024)[1]).weight
        c1 = [w1] + [clone_w(w1) for _ in range(39)]
        x1 = bf16(synth.activations(rng, 1, 4096))
        ms = graph_ms(lambda: [R.nint_matmul(w, x1, force="gemv") for w in c1], 20) / len(c1)
        b1 = w1.payload_bytes + 2 * 4096 + 4 * 4096
        extras["config1_nint3_us"] = ms * 1e3
        extras["config1_nint3_gbps"] = b1 / (ms * 1e-3) / 1e9
        log(f"[bench] config 1 NINT3 4096x4096 M=1: {ms * 1e3:.2f} us, {extras['config1_nint3_gbps']:.0f} GB/s")
        del c1

        # ---- NINT8-0 (Q8_0 blocks) 12288x4096, batch {1, 8}, 8 rotating copies (428 MB) ---------------
        w8 = R.load_quant_linear(*synth.nint8_zero_blob(8, FF, H)).weight
        c8 = [w8] + [clone_w(w8) for _ in range(7)]
        for M in (1, 8):
            x8 = bf16(synth.activations(rng, M, H))
            ms = graph_ms(lambda: [R.nint8_zero_matmul(w, x8) for w in c8], 10) / len(c8)
            extras[f"nint8_zero_M{M}_us"] = ms * 1e3
            extras[f"nint8_zero_M{M}_gbps"] = w8.payload_bytes / (ms * 1e-3) / 1e9
            log(f"[bench] NINT8-0 {FF}x{H} M={M}: {ms * 1e3:.2f} us, {extras[f'nint8_zero_M{M}_gbps']:.0f} GB/s of payload")
        del c8, w8

        # ---- config 3: NVQ3J-512 17408x5120 and its transpose, batch {1,4,8}, 8 rotating copies -----
        for name, (n3, k3) in {"up": (17408, 5120), "down": (5120, 17408)}.items():
            w3 = synth.tile_rows(RV.NvqWeight.from_blob(synth.nvq3j512_blob(11, 1024, k3)[1]), n3)
            c3 = [w3] + [clone_w(w3) for _ in range(7)]
            for M in (1, 4, 8):
                x3 = bf16(synth.activations(rng, M, k3))
                ms = graph_ms(lambda: [RV.nvq_matmul(w, x3) for w in c3], 10) / len(c3)
                b3 = w3.payload_bytes + 2 * M * k3 + 4 * M * n3
                extras[f"config3_nvq_{name}_M{M}_us"] = ms * 1e3
                extras[f"config3_nvq_{name}_M{M}_gbps"] = b3 / (ms * 1e-3) / 1e9
            log(f"[bench] config 3 NVQ3J-512 {n3}x{k3}: " + ", ".join(
                f"M={M} {extras[f'config3_nvq_{name}_M{M}_gbps']:.0f} GB/s" for M in (1, 4, 8)))
            del c3, w3
        torch.cuda.empty_cache()

        # ---- config 4: 256 mixed-bit experts + 1 shared, hidden 4096, intermediate 2048, top-8 ------
        # N(0, 0.02) weights through the expert-wise NINT quantizer (a 1024-row slab per precision, tiled over its
        # cohort), loaded and run by the C++ host runtime (libmfq_runtime.so): nint_moe_ffn_forward with a reserved
        # scratch, recorded into a HIP graph.
        rt = C.CDLL(str(ROOT / "tyloquant_amd" / "lib" / "libmfq_runtime.so"))
        rt.mfq_rt_last_error.restype = C.c_char_p
        rt.mfq_rt_load_nint_moe.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(C.c_void_p)]
        rt.mfq_rt_free_nint_moe.argtypes = [C.c_void_p]
        rt.mfq_rt_load_quant_linear.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_void_p)]
        rt.mfq_rt_free_quant_linear.argtypes = [C.c_void_p]
        rt.mfq_rt_moe_scratch_create.argtypes = [C.POINTER(C.c_void_p)]
        rt.mfq_rt_moe_scratch_free.argtypes = [C.c_void_p]
        rt.mfq_rt_moe_scratch_reserve.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        rt.mfq_rt_moe_ffn_forward_scratch.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int64,
                                                      C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                                      C.c_void_p, C.c_void_p]

        def rt_check(rc):
            if rc:
                raise RuntimeError(rt.mfq_rt_last_error().decode(errors="replace"))
        E, HID, INTER, TOPK = 256, 4096, 2048, 8
        ebits = np.random.default_rng(4).choice([2, 3, 4, 5], size=E, p=[0.1, 0.4, 0.4, 0.1])
        per_expert = np.zeros(E)
        handles = []
        # the CPU leg's sample of this config: one token, its eight routed experts (chosen here so that their rows can be
        # cut out of the cohort payloads before those are dropped)
        cpu4_logits = np.random.default_rng(44).standard_normal((1, E)).astype(np.float32)
        cpu4_ids = np.argsort(-cpu4_logits, axis=-1, kind="stable")[:, :TOPK].astype(np.int32)
        cpu4_rows = [{}, {}]      # per tensor: expert -> (packed body of its cohort, header, first row)
        for ti4, (seed, (o_, k_)) in enumerate(((40, (2 * INTER, HID)), (41, (HID, INTER)))):
            blob4, pools4 = synth.nintm_quantized_blob(seed, E, o_, k_, ebits)
            for ids4, payload4 in pools4:
                hdr = F.parse_nint(payload4)
                per_expert[ids4] += hdr.body_bytes / len(ids4)
                if not args.no_cpu:
                    body4 = None
                    for local4, e4 in enumerate(ids4):
                        if int(e4) in cpu4_ids:
                            body4 = bytes(payload4[hdr.body_off:]) if body4 is None else body4
                            cpu4_rows[ti4][int(e4)] = (body4, hdr, local4 * o_, o_)
            h4 = C.c_void_p()
            rt_check(rt.mfq_rt_load_nint_moe(blob4, len(blob4), C.byref(h4)))
            handles.append(h4)
            del blob4, pools4
        shared_bytes, shared_h = 0, []
        for seed, (o_, k_) in ((42, (2 * INTER, HID)), (43, (HID, INTER))):
            dt4, sb4 = synth.nint_linear_blob(seed, o_, k_, 4, 24, 6, slab_rows=1024)
            shared_bytes += F.parse_nint(sb4).body_bytes
            h4 = C.c_void_p()
            rt_check(rt.mfq_rt_load_quant_linear(dt4.encode(), sb4, len(sb4), C.byref(h4)))
            shared_h.append(h4)
        scratch4 = C.c_void_p()
        rt_check(rt.mfq_rt_moe_scratch_create(C.byref(scratch4)))
        rt_check(rt.mfq_rt_moe_scratch_reserve(scratch4, handles[0], handles[1], 2048, TOPK, shared_h[0], shared_h[1]))
        torch.cuda.synchronize()
        log(f"[bench] config 4 tensors quantized and loaded by the C++ runtime ({time.time() - t0:.1f}s)")
        for T, nb in ((1, 8), (64, 2), (2048, 1)):
            xs4 = [bf16(synth.activations(rng, T, HID)) for _ in range(nb)]
            lg4 = [torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).to(dev) for _ in range(nb)]
            out4 = torch.empty((T, HID), dtype=torch.float32, device=dev)

            def moe_all():
                for i in range(nb):
                    rt_check(rt.mfq_rt_moe_ffn_forward_scratch(scratch4, handles[0], handles[1], xs4[i].data_ptr(), L.X_BF16,
                                                               HID, T, lg4[i].data_ptr(), TOPK, L.TOPK_DELAYED_SOFTMAX, 0,
                                                               shared_h[0], shared_h[1], out4.data_ptr(), stream_ptr()))
            moe_all()
            torch.cuda.synchronize()
            assert bool(torch.isfinite(out4).all()), "MoE layer produced non-finite outputs"
            hit_bytes = 0.0
            for lgt in lg4:
                hit = torch.unique(torch.topk(lgt, TOPK, dim=1).indices).cpu().numpy()
                hit_bytes += per_expert[hit].sum() + shared_bytes
            ms = graph_ms(moe_all, 5 if T < 2048 else 2) / nb
            extras[f"config4_moe_T{T}_ms"] = ms
            extras[f"config4_moe_T{T}_tokens_per_s"] = T / (ms * 1e-3)
            extras[f"config4_moe_T{T}_weight_gbps"] = hit_bytes / nb / (ms * 1e-3) / 1e9
            extras[f"config4_moe_T{T}_tflops"] = (2.0 * T * TOPK * 3 * HID * INTER + 2.0 * T * 3 * HID * INTER) / (ms * 1e-3) / 1e12
            log(f"[bench] config 4 MoE T={T} (C++ host, HIP graph): {ms:.3f} ms, {T / (ms * 1e-3):.0f} tokens/s, "
                f"{extras[f'config4_moe_T{T}_weight_gbps']:.0f} GB/s of expert payload")
        extras["config4_host"] = "C++ runtime (libmfq_runtime.so), graph replay"
        rt.mfq_rt_moe_scratch_free(scratch4)
        for h4 in shared_h:
            rt.mfq_rt_free_quant_linear(h4)
        for h4 in handles:
            rt.mfq_rt_free_nint_moe(h4)
        torch.cuda.empty_cache()

        # ---- config 5: 36-layer linear stack, mixed formats by seed, batch {1,16} -------------------
        shapes5 = {"qkv": (6144, 4096), "o": (4096, 4096), "gate": (12288, 4096), "up": (12288, 4096), "down": (4096, 12288)}
        fmts = ["NEPQ1-S", "NINT3", "NVQ3J-512", "NINT5"]
        pick = np.random.default_rng(5).choice(4, size=(36, 5), p=[0.2, 0.4, 0.25, 0.15])
        proto = {}

        def proto_weight(fmt, n, k):
            key = (fmt, n, k)
            if key not in proto:
                if fmt == "NINT3":
                    proto[key] = ("nint", synth.random_nint_weight(50, n, k, 3, 24, 5))
                elif fmt == "NINT5":
                    proto[key] = ("nint", synth.random_nint_weight(51, n, k, 5, 28, 7))
                elif fmt == "NVQ3J-512":
                    proto[key] = ("nvq", synth.tile_rows(RV.NvqWeight.from_blob(synth.nvq3j512_blob(52, 512, k)[1]), n))
                else:
                    proto[key] = ("nepq", synth.tile_rows(RV.NepqWeight.from_blob(synth.nepq1_blob(53, fmt, 512, k)[1]), n))
            return proto[key]
        stack, bytes5 = [], 0
        for layer in range(36):
            for ti, (tname, (n, k)) in enumerate(shapes5.items()):
                kind, w = proto_weight(fmts[pick[layer, ti]], n, k)
                stack.append((kind, clone_w(w), n, k))
                bytes5 += w.payload_bytes
        extras["config5_payload_gb"] = bytes5 / 1e9
        mm = {"nint": R.nint_matmul, "nvq": RV.nvq_matmul, "nepq": RV.nepq_matmul}
        for M in (1, 16):
            xk = {k: bf16(synth.activations(rng, M, k)) for k in (4096, 12288)}
            ms = graph_ms(lambda: [mm[kind](w, xk[k]) for kind, w, n, k in stack], 3, warm=1)
            tot = bytes5 + sum(2 * M * k + 4 * M * n for _, _, n, k in stack)
            extras[f"config5_stack_M{M}_ms"] = ms
            extras[f"config5_stack_M{M}_gbps"] = tot / (ms * 1e-3) / 1e9
            log(f"[bench] config 5 stack (180 matmuls, {bytes5 / 1e9:.2f} GB) M={M}: {ms:.3f} ms, "
                f"{extras[f'config5_stack_M{M}_gbps']:.0f} GB/s")
        del stack, proto
        torch.cuda.empty_cache()

        # ---- OCP MX payloads (no BASELINE config): 12288 x 4096 MXFP4 / MXFP8 read in place, batch {1, 16} ----
        from tyloquant_amd.runtime_mx import MxWeight, mx_matmul
        for mx_dtype in ("MXFP4", "MXFP8"):
            blob = synth.mx_blob(60, mx_dtype, 12288, 4096)[1]
            ncopy = 12  # rotating copies: 320 / 604 MB, beyond the 256 MB the last-level cache could keep
            mxw = [MxWeight.from_blob(mx_dtype, blob) for _ in range(ncopy)]
            for M in (1, 16):
                xm = [bf16(synth.activations(rng, M, 4096)) for _ in range(ncopy)]
                ms = graph_ms(lambda: [mx_matmul(mxw[i], xm[i]) for i in range(ncopy)], 5, warm=2) / ncopy
                key = f"{mx_dtype.lower()}_12288x4096_M{M}"
                extras[f"{key}_us"] = ms * 1e3
                extras[f"{key}_gbps"] = mxw[0].payload_bytes / (ms * 1e-3) / 1e9
                log(f"[bench] {mx_dtype} 12288x4096 M={M}: {ms * 1e3:.1f} us, {extras[f'{key}_gbps']:.0f} GB/s of payload")
            del mxw
        # ---- NVQ2J (E8 vectors, 2 bits per weight; no BASELINE config): 12288 x 4096 read in place from its bit streams ----
        e8_blob = synth.nvq2j_blob(61, 12288, 4096)
        e8 = [R.load_quant_linear(*e8_blob) for _ in range(4)]
        for M in (1, 16, 64):
            xe = [bf16(synth.activations(rng, M, 4096)) for _ in range(4)]
            ms = graph_ms(lambda: [e8[i](xe[i]) for i in range(4)], 5, warm=2) / 4
            extras[f"nvq2j_12288x4096_M{M}_us"] = ms * 1e3
            extras[f"nvq2j_12288x4096_M{M}_gbps"] = e8[0].weight.payload_bytes / (ms * 1e-3) / 1e9
            log(f"[bench] NVQ2J 12288x4096 M={M}: {ms * 1e3:.1f} us, {extras[f'nvq2j_12288x4096_M{M}_gbps']:.0f} GB/s of payload")
        del e8
        torch.cuda.empty_cache()

    cpu = None
    if not args.no_cpu:
        from oracle import c_oracle
        from oracle import mfq_oracle as O

        def best_of(fn, n=3):
            best, res = 1e9, None
            for _ in range(n):
                t1 = time.perf_counter()
                res = fn()
                best = min(best, time.perf_counter() - t1)
            return best, res
        cpu_cfg = {}
        # config 1: the whole NINT3 4096 x 4096 tensor, one row
        blob1 = synth.nint_linear_blob(7, 4096, 4096, 3, 24, 5, slab_rows=1024)[1]
        h1 = F.parse_nint(blob1)
        body1 = bytes(blob1[h1.body_off:])
        xc1 = synth.activations(np.random.default_rng(101), 1, 4096).astype(np.float32)
        sec, _ = best_of(lambda: c_oracle.matmul_nt(xc1, c_oracle.nint_dequant(body1, 3, 5, 24, 4096, 4096)))
        cpu_cfg["config1"] = {"value": (h1.body_bytes + 2 * 4096 + 4 * 4096) / sec / 1e9, "unit": "GB/s", "cores": c_oracle.threads(),
                              "kind": "port", "sample": f"NINT3 (3,24,5) 4096x4096 at M=1, whole tensor: dequantize + x@W.T, best of 3 ({sec * 1e3:.0f} ms)"}
        # config 3: a 1024-row slab of the NVQ3J-512 17408 x 5120 tensor, one row
        blob3 = synth.nvq3j512_blob(11, 1024, 5120)[1]
        t3 = O.unpack_nvq(blob3)
        xc3 = synth.activations(np.random.default_rng(103), 1, 5120).astype(np.float32)
        sec, _ = best_of(lambda: c_oracle.matmul_nt(xc3, c_oracle.nvq_jsc_dequant(t3)))
        cpu_cfg["config3"] = {"value": O.nvq_payload_nbytes("d4_512", 1024, 5120) / sec / 1e9, "unit": "GB/s", "cores": c_oracle.threads(),
                              "kind": "port", "sample": "NVQ3J-512 at M=1, a 1024-row slab of the 17408x5120 tensor (unpacked fields): "
                                                        f"dequantize + x@W.T, best of 3 ({sec * 1e3:.0f} ms)"}
        # config 4: one token through its eight routed experts (the shared expert's two GEMVs left out)
        if cpu4_rows is not None and all(len(d) == cpu4_ids.size for d in cpu4_rows):
            xc4 = synth.activations(np.random.default_rng(104), 1, HID).astype(np.float32)
            sel4 = np.take_along_axis(cpu4_logits, cpu4_ids.astype(np.int64), axis=-1).astype(np.float64)
            w4 = np.exp(sel4 - sel4.max(-1, keepdims=True))
            w4 = (w4 / w4.sum(-1, keepdims=True)).astype(np.float32)

            def moe_cpu():
                dense = [{e: c_oracle.nint_dequant_rows(b, hd.bits, hd.sub_bits, hd.gs, hd.out, hd.neuron_len, r0, nr)
                          for e, (b, hd, r0, nr) in rows.items()} for rows in cpu4_rows]
                return c_oracle.moe_ffn(xc4, cpu4_ids, w4, dense[0], dense[1], E)
            sec, _ = best_of(moe_cpu)
            cpu_cfg["config4"] = {"value": 1.0 / sec, "unit": "tokens/s", "cores": c_oracle.threads(), "kind": "port",
                                  "sample": "MoE layer at T=1: the token's 8 routed experts of 256 (mixed 2/3/4/5-bit), dequantize "
                                            f"their rows + gate/up, SwiGLU, down, weighted sum; shared expert left out; best of 3 ({sec * 1e3:.0f} ms)"}
            del cpu4_rows
        # config 5: a 512-row slab of an NEPQ1-S 6144 x 4096 tensor (the other formats of the stack are configs 1 and 3)
        blob5 = synth.nepq1_blob(53, "NEPQ1-S", 512, 4096)[1]
        t5 = O.unpack_nepq(blob5)
        tab5 = np.stack([np.stack([O.unpack_ternary_table(p.tobytes()[:1024]), O.unpack_ternary_table(p.tobytes()[1024:])])
                         for p in t5.table_payloads])
        xc5 = synth.activations(np.random.default_rng(105), 1, 4096).astype(np.float32)
        sec, _ = best_of(lambda: c_oracle.matmul_nt(xc5, c_oracle.nepq1s_dequant(t5, tab5)[0]))
        cpu_cfg["config5"] = {"value": O.nepq_payload_nbytes("NEPQ1-S", 1, 512, 4096, len(t5.table_payloads)) / sec / 1e9, "unit": "GB/s",
                              "cores": c_oracle.threads(), "kind": "port",
                              "sample": f"NEPQ1-S at M=1, a 512-row slab (unpacked fields): dequantize + x@W.T, best of 3 ({sec * 1e3:.0f} ms)"}
        log(f"[bench] cpu baselines of configs 1, 3, 4, 5: {cpu_cfg}")
        blob = base["gate"][1]
        from tyloquant_amd import formats as F
        h = F.parse_nint(blob)
        body = bytes(blob[h.body_off:])
        xf = x_h.float().cpu().numpy()
        best_full, best_mm = 1e9, 1e9
        W = None
        for _ in range(3):
            t1 = time.perf_counter()
            W = c_oracle.nint_dequant(body, h.bits, h.sub_bits, h.gs, h.out, h.neuron_len)
            yc = c_oracle.matmul_nt(xf, W)
            best_full = min(best_full, time.perf_counter() - t1)
        for _ in range(5):
            t1 = time.perf_counter()
            yc = c_oracle.matmul_nt(xf, W)
            best_mm = min(best_mm, time.perf_counter() - t1)
        gbytes = (base["gate"][0].payload_bytes + 2 * H + 4 * FF) / 1e9
        ref = y1.cpu().numpy()
        cpu_rel = float(np.linalg.norm(ref - yc) / np.linalg.norm(yc))
        assert cpu_rel < 1e-3, f"GPU GEMV differs from the CPU path: {cpu_rel}"
        cpu = {"value": gbytes / best_full, "unit": "GB/s", "cores": c_oracle.threads(), "kind": "port",
               "sample": "gate 12288x4096 NINT4-32 at M=1: dequantize to fp32 + x@W.T, best of 3 "
                         f"({best_full * 1e3:.0f} ms); matmul alone on pre-dequantized W {best_mm * 1e3:.1f} ms",
               "matmul_only_value": gbytes / best_mm, "gpu_vs_cpu_rel_l2": cpu_rel, "configs": cpu_cfg}
        log(f"[bench] cpu baseline: {cpu}")

    line = {
        "metric": "decode_qgemv_hbm_gbps", "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic (N(0,0.02) weights through the NINT quantizer on a "
        "1024-row slab tiled to shape; N(0,1) bf16 activations, 0.1% channels x20)",
        "config": {"workload": "BASELINE config 2 decode: NINT4 (4,32,6) gate/up 12288x4096 + down 4096x12288 at M=1, "
                               f"gate+up as one grouped launch, {args.copies} rotating weight sets "
                               f"({args.copies * step_bytes / 1e6:.0f} MB)",
                   "step_bytes": step_bytes, "launches_per_step": n_per_step, "hip_graph": True,
                   # the library's effective tuning thresholds and CU count for this run
                   "library": lib.mfq_hip_config().decode(errors="replace")},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE, each scaled by what the counter
                     # reads for a plain 256 MiB copy: the figure the committed profile summary states
                     "traffic": profiled_traffic(),
                     "kernel": "nint_gemv_xreg_kernel<PairedUnit<4,32>,0,1>", "avg_launch_us": avg_launch_us,
                     "bytes_per_launch": bytes_per_launch},
        "cpu_baseline": cpu,
        "extras": extras,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
