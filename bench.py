#!/usr/bin/env python3
"""Benchmark of the fused data-parallel path on one MI355X.

A step is ONE pass of the hot path over one batch of synthetic input already resident in HBM: the DNN
preprocessing chain of configuration 3 (64 crops of a 1920x1080 BGR image -> bilinear resize to 224x224 ->
BGR->RGB -> (x - mean) / std -> planar float32 64x3x224x224), issued through the C++ host API
(executeOperations<TransformDPP<>>) -> C ABI -> one gfx950 kernel.

Every measurement is W warm-up steps, a synchronisation, and then exactly K timed steps back to back on one stream.  The
events (and the host clock) that bracket the K steps are taken by the case driver itself, right before its first launch
and right after its last: this script needs about 100 us of Python to marshal a call's arguments, and with the bracket
around the Python call a short run (K = 20) would charge that idle time to the kernel.  Every measurement starts after
30 ms of GPU idle (see Timer.run).  `kernel_us_5_runs_min_mean_max` of the headline shows the K steps repeated four more
times, `kernel_us_1000_launches` one batch of 1000 launches (the first launches after idle are then a small part).

Prints ONE JSON line.  `value` is output Mpix/s of the whole job; `roofline` prices the kernel's algorithmic bytes
against the 8 TB/s HBM peak using the launch duration measured with HIP events on the launch stream;
`cpu_baseline` is the same chain on the reference library's single-threaded CPU backend (oracle/_ref, when built)
or on the plain-C oracle, timed on this machine's host cores.  `others` carries the same measurements for the
remaining four configurations.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--list-compiled", action="store_true",
                    help="print to stderr the kernel symbol and signature of every chain compiled at run time")
    ap.add_argument("--only", default="", help="comma separated subset of c1,c2,c3,c4,c5,ext (c3 is always run)")
    return ap.parse_args()


class Timer:
    """K back-to-back launches through the host API, bracketed by events on the launch stream and by wall clock."""

    def __init__(self, torch, fkl, cases):
        self.torch, self.fkl, self.cases = torch, fkl, cases
        self.lib = fkl.lib()
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        fkl.check(self.lib.fklhip_event_create(C.byref(self.e0)), "event_create")
        fkl.check(self.lib.fklhip_event_create(C.byref(self.e1)), "event_create")

    def run(self, fn, steps, warmup, settle=0.03):
        torch = self.torch
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        # Every measurement starts from a GPU that has been idle for a moment.  A short batch of launches that follows the
        # end of another burst within a few milliseconds catches the GPU on its way down to its idle state and reads up to
        # 30 % slower (measured: 20 launches of configuration 3 right after 300 others, median 10.6 us per launch; after
        # 20 ms of idle 8.37 us, and never above 8.8 us); which of the two a line got used to depend on what ran before it.
        if settle > 0:
            torch.cuda.synchronize()
            time.sleep(settle)
        if warmup > 0:
            self.cases.set_reps(warmup)
            fn()
        torch.cuda.synchronize()
        # The case driver records e0 right before its first launch and e1 right after its last one, and notes the host
        # clock at that point: the timed region is the K steps through the host API, without this script's own
        # marshalling of the call's arguments (about 100 us of Python, during which the GPU would sit idle).
        self.cases.time_next(stream, self.e0, self.e1)
        self.cases.set_reps(steps)
        fn()
        torch.cuda.synchronize()
        wall_ms = (time.clock_gettime_ns(time.CLOCK_MONOTONIC) - self.cases.timed_start_ns()) * 1e-6
        ms = C.c_float()
        self.fkl.check(self.lib.fklhip_event_elapsed_ms(C.byref(ms), self.e0, self.e1), "event_elapsed")
        return wall_ms / steps, ms.value / steps   # per step: wall clock, device events


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this path runs on ONE GPU (asked for {args.gpus}); every output pixel is independent, "
              "so more GPUs would only split the batch. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import fusedkernellibrary_amd as fkl
    import fkl_cases as cases
    import workloads as wl

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    fkl.lib()   # raises if the HIP library is missing: there is no fallback
    built_in = {s for s, _ in fkl.signatures()}
    dev = torch.device("cuda:0")
    timer = Timer(torch, fkl, cases)
    only = set(filter(None, args.only.split(","))) or {"c1", "c2", "c3", "c4", "c5", "ext"}
    results = {}

    def record(name, out_px, alg_bytes, fn, steps, warmup, best_of=1):
        wall_ms, dev_ms = min((timer.run(fn, steps, warmup) for _ in range(best_of)), key=lambda t: t[1])
        ll = fkl.last_launch()
        results[name] = {
            "mpix_per_s": out_px / 1e6 / (wall_ms * 1e-3),
            "ms_per_step": wall_ms,
            "kernel_us": dev_ms * 1e3,
            "algorithmic_bytes": alg_bytes,
            "achieved_gbs": alg_bytes / (dev_ms * 1e-3) / 1e9,
            "frac_of_hbm_peak": alg_bytes / (dev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "kernel": ll["kernel"], "grid": ll["grid"], "block": ll["block"], "lds_bytes": ll["lds_bytes"],
        }
        return results[name]

    # ---- configuration 3: the headline workload -------------------------------------------------------------
    c3 = wl.config3()
    union_px = wl.config3_union_pixels(c3["rects"], 1920, 1080)
    a3 = 64 * 3 * 224 * 224 * 4 + 3 * union_px
    src3 = torch.from_numpy(c3["src"]).to(dev)
    out3 = torch.zeros((64, 3, 224, 224), dtype=torch.float32, device=dev)
    f3 = lambda: cases.crop_resize_norm_split(src3, c3["rects"], c3["dst"], c3["sub"], c3["div"], out3)
    # (timed after the other configurations, further down: the first launches of a process run on a GPU that has not
    # reached its working clocks yet, and the headline should not depend on what happened to be measured first)

    # what a launch costs when there is nothing to do: the same host path and kernel on a 64 x 1 image
    tiny_in = torch.zeros((1, 64), dtype=torch.float32, device=dev)
    tiny_out = torch.zeros_like(tiny_in)
    floor = record("launch_floor_copy_64x1", 64, 512, lambda: cases.copy_f32(tiny_in, tiny_out), args.steps, args.warmup)
    floor["note"] = "duration of one launch that moves 512 bytes, back to back on one stream: the floor under every kernel_us here"

    # ---- the other four configurations (reported under "others") ------------------------------------------------
    if "c1" in only:
        c = wl.config1()
        s = torch.from_numpy(c["src"]).to(dev)
        o = torch.zeros((5, 64, 128, 3), dtype=torch.uint8, device=dev)
        a1 = 128 * 64 * 5 * 3 + int((c["rects"][:, 2] * c["rects"][:, 3]).sum()) * 3
        record("c1", 128 * 64 * 5, a1, lambda: cases.crop_resize_par_u8(s, c["rects"], c["dst"], c["bg"], c["mul"], c["sub"], o),
               args.steps, args.warmup)
    if "c2" in only:
        c = wl.config2()
        s = torch.from_numpy(c["src"]).to(dev)
        o = torch.zeros_like(s)
        for n in c["n_ops_sweep"]:
            # (best of three batches each: the crossover below compares launches that differ by a few percent)
            record(f"c2_n{n}", 3840 * 2160, 2 * 3840 * 2160 * 4, lambda n=n: cases.add_mul_chain(s, n, c["add"], c["mul"], o),
                   args.steps, args.warmup, best_of=3)
            if n >= 50:
                # n dependent fp32 instructions per element that no contraction or packing may merge: 8.3 M elements are
                # 129 600 wave-wide elements, at the 2.45 cycles per instruction and SIMD this chip was measured to issue
                results[f"c2_n{n}"]["valu_issue_floor_us"] = 129600 * n * 2.45 / 1024 / 2.3e3
        record("copy_f32_4k", 3840 * 2160, 2 * 3840 * 2160 * 4, lambda: cases.copy_f32(s, o), args.steps, args.warmup, best_of=3)
        # Where instruction issue takes over from bandwidth (the sweep of the reference's instruction-count benchmark,
        # benchmarks/numinstructions/benchmark_numinstructions_x_operation.h:33-43): the first N of the sweep whose launch
        # takes 5 % longer than the plain copy of the same image, the straight line through the launches beyond it
        # (what a launch costs whatever its length + what one more operation costs), and the N at which that line meets
        # the copy's duration.
        copy_us = results["copy_f32_4k"]["kernel_us"]
        sweep = [(n, results[f"c2_n{n}"]["kernel_us"]) for n in c["n_ops_sweep"]]
        beyond = [(n, us) for n, us in sweep if us > 1.05 * copy_us]
        cross = {"copy_us": copy_us, "sweep_n": [n for n, _ in sweep], "sweep_us": [us for _, us in sweep],
                 "first_n_5_percent_above_copy": beyond[0][0] if beyond else None}
        if len(beyond) >= 2:
            per_op, fixed = np.polyfit(np.array([n for n, _ in beyond], np.float64), np.array([us for _, us in beyond]), 1)
            cross.update({"fit_through_n": [n for n, _ in beyond], "fixed_us": float(fixed), "per_op_us": float(per_op),
                          "line_meets_copy_at_n": float((copy_us - fixed) / per_op)})
        results["c2_crossover"] = cross
    if "c5" in only:
        c = wl.config5()
        s = torch.from_numpy(c["nv12"]).to(dev)
        o = torch.zeros((3, 1080, 1920), dtype=torch.float32, device=dev)
        record("c5", 1920 * 1080, 3840 * 2160 * 3 // 2 + 3 * 1080 * 1920 * 4,
               lambda: cases.nv12_rgb_resize_split(s, c["width"], c["height"], c["dst"], c["scale"], o), args.steps, args.warmup)
    if "c4" in only:
        # 100 images of uniform random bytes (generated on the GPU: the content does not affect the timing and the
        # seeded host generator of the parity tests needs several seconds for 622 MB)
        g = torch.Generator(device=dev)
        g.manual_seed(4)
        srcs = [torch.randint(0, 256, (1080, 1920, 3), dtype=torch.uint8, device=dev, generator=g) for _ in range(100)]
        outs = [torch.empty_like(t) for t in srcs]
        p = wl.RawMT(44)
        mul = np.stack([p.range_floats(3, 0.5, 2.0) for _ in range(100)])
        add = np.stack([p.range_floats(3, -64.0, 64.0) for _ in range(100)])
        record("c4", 100 * 1920 * 1080, 2 * 100 * 1920 * 1080 * 3, lambda: cases.batch_muladd_sat(srcs, mul, add, outs),
               max(10, args.steps // 10), max(2, args.warmup // 10))
        # this run's own check of what it timed: every plane against the same arithmetic done by torch on the GPU (one
        # multiplication, one addition, round half to even, clamp: each rounded once, as the chain's operations are)
        for i in range(100):
            m, a = torch.from_numpy(mul[i]).to(dev), torch.from_numpy(add[i]).to(dev)
            if not torch.equal(outs[i], torch.clamp(torch.round(srcs[i].to(torch.float32) * m + a), 0, 255).to(torch.uint8)):
                print(f"bench.py: configuration 4, image {i}: the output differs from mul, add, round-half-even, clamp", file=sys.stderr)
                sys.exit(3)
        results["c4"]["note"] = ("inputs: uniform random bytes made on the GPU; all 100 outputs of this run checked bit for bit against the same "
                                 "arithmetic in torch (the seeded inputs and the reference's digests: tests/test_gpu_parity.py)")

        del srcs, outs

    if "ext" in only:
        # rows beyond the five benchmark configurations: warp, conditional batch, fill
        import math
        rng = np.random.RandomState(7)
        img = torch.from_numpy(rng.randint(0, 256, (1080, 1920, 3)).astype(np.uint8)).to(dev)
        th = math.radians(7.0)
        affine = [[math.cos(th), -math.sin(th), 40.0], [math.sin(th), math.cos(th), -60.0]]
        wo = torch.zeros((1080, 1920, 3), dtype=torch.float32, device=dev)
        record("warp_affine_1080p_u8x3", 1920 * 1080, 1920 * 1080 * (3 + 12), lambda: cases.warp(img, affine, False, (1920, 1080), wo),
               args.steps, args.warmup)
        rects8 = c3["rects"][:8]
        o8 = torch.zeros((8, 3, 224, 224), dtype=torch.float32, device=dev)
        record("c3_b8_default_planes_5_of_8", 8 * 224 * 224, 8 * 3 * 224 * 224 * 4,
               lambda: cases.crop_resize_default_norm_split(src3, rects8, (224, 224), 5, (0.0, 0.0, 0.0), c3["sub"], c3["div"], o8),
               args.steps, args.warmup)

        # the read-back operations, pixel formats and launch patterns either side of the path (1080p unless noted)
        W, H = 1920, 1080
        fo = torch.zeros((H, W, 3), dtype=torch.float32, device=dev)
        record("deinterlace_blend_1080p_u8x3", W * H, W * H * (3 + 12), lambda: cases.deinterlace(img, 1, fo), args.steps, args.warmup)
        po = torch.zeros((H + 32, W + 32, 3), dtype=torch.uint8, device=dev)
        record("pad_reflect101_16px_1080p_u8x3", (W + 32) * (H + 32), W * H * 3 + (W + 32) * (H + 32) * 3,
               lambda: cases.pad(img, 4, 16, 16, po), args.steps, args.warmup)
        uyvy = torch.from_numpy(rng.randint(0, 256, (H, 2 * W)).astype(np.uint8)).to(dev)
        record("uyvy_to_rgb_full709_1080p", W * H, W * H * (2 + 12), lambda: cases.yuv_to_rgb(10, 1, 1, uyvy, W, H, fo), args.steps, args.warmup)
        nv12 = torch.zeros((H + H // 2, W), dtype=torch.uint8, device=dev)
        record("rgb_to_nv12_limited709_1080p", W * H, W * H * 3 + W * H * 3 // 2, lambda: cases.rgb_to_yuv(0, 0, 1, img, nv12), args.steps, args.warmup)
        t4 = torch.from_numpy(rng.rand(4, H, W, 3).astype(np.float32)).to(dev)
        small = torch.from_numpy(rng.randint(0, 256, (540, 960, 3)).astype(np.uint8)).to(dev)
        d4 = torch.zeros((4, H, W, 3), dtype=torch.float32, device=dev)
        record("divergent_2_pointwise_2_resize_planes_1080p", 4 * W * H, 2 * W * H * 24 + 2 * (960 * 540 * 3 + W * H * 12),
               lambda: cases.divergent_mixed(t4, 1.5, small, d4), args.steps, args.warmup)
        frames = [torch.from_numpy(rng.randint(0, 256, (720, 1280, 3)).astype(np.uint8)).to(dev) for _ in range(3)]
        px = 1280 * 720
        record("circular_tensor_update_b8_720p", 8 * px, px * 3 + 2 * px * 12 + 7 * 2 * px * 12, lambda: cases.circular_update_b8(frames),
               max(10, args.steps // 4), max(2, args.warmup // 4))
        cases.circular_update_b8(frames, release=True)
        # two images in, one out (DualSourceRead -> Add -> Cast -> Mul -> SaturateCast), and one image out as three planes
        img2 = torch.from_numpy(rng.randint(0, 256, (H, W, 3)).astype(np.uint8)).to(dev)
        mean = torch.zeros((H, W * 3), dtype=torch.uint8, device=dev)
        record("mean_of_two_1080p_u8x3", W * H, 3 * W * H * 3, lambda: cases.dual(8, img.view(H, W * 3), img2.view(H, W * 3), W, H, mean),
               args.steps, args.warmup)
        planes = [torch.zeros((H, W), dtype=torch.float32, device=dev) for _ in range(3)]
        record("u8x3_to_three_float_planes_1080p", W * H, W * H * (3 + 12),
               lambda: cases.split_write(1, img.view(H, W * 3), W, H, planes, None, (1 / 255.0, 1 / 255.0, 1 / 255.0, 0)), args.steps, args.warmup)
        del fo, po, uyvy, nv12, t4, d4, frames, img2, mean, planes
        # the same four chains at 3840 x 2160, where the launch floor is a smaller part of a launch
        W, H = 3840, 2160
        img4k = torch.from_numpy(rng.randint(0, 256, (H, W, 3)).astype(np.uint8)).to(dev)
        fo = torch.zeros((H, W, 3), dtype=torch.float32, device=dev)
        affine4k = [[math.cos(th), -math.sin(th), 80.0], [math.sin(th), math.cos(th), -120.0]]
        record("warp_affine_2160p_u8x3", W * H, W * H * (3 + 12), lambda: cases.warp(img4k, affine4k, False, (W, H), fo), args.steps, args.warmup)
        record("deinterlace_blend_2160p_u8x3", W * H, W * H * (3 + 12), lambda: cases.deinterlace(img4k, 1, fo), args.steps, args.warmup)
        uyvy = torch.from_numpy(rng.randint(0, 256, (H, 2 * W)).astype(np.uint8)).to(dev)
        record("uyvy_to_rgb_full709_2160p", W * H, W * H * (2 + 12), lambda: cases.yuv_to_rgb(10, 1, 1, uyvy, W, H, fo), args.steps, args.warmup)
        po = torch.zeros((H + 32, W + 32, 3), dtype=torch.uint8, device=dev)
        record("pad_reflect101_16px_2160p_u8x3", (W + 32) * (H + 32), W * H * 3 + (W + 32) * (H + 32) * 3,
               lambda: cases.pad(img4k, 4, 16, 16, po), args.steps, args.warmup)
        del img4k, fo, uyvy, po

    # ---- configuration 3, the headline: W warm-up steps, then exactly K timed steps ---------------------------------
    r3 = record("c3", 64 * 224 * 224, a3, f3, args.steps, args.warmup)
    got3 = out3.cpu().numpy()
    # the same K steps four more times, for the spread (not used for `value`)
    again = [timer.run(f3, args.steps, args.warmup)[1] * 1e3 for _ in range(4)] + [r3["kernel_us"]]
    r3["kernel_us_5_runs_min_mean_max"] = [min(again), sum(again) / len(again), max(again)]
    # The same K steps recorded once into a HIP graph (kernel nodes only: the launch path allocates nothing and records no
    # memset) and replayed: what the steps cost when the host issues one graph launch instead of K kernel launches.
    graph = torch.cuda.CUDAGraph()
    cases.set_reps(args.steps)
    with torch.cuda.graph(graph):
        f3()
    torch.cuda.synchronize()
    graph_runs = []
    for _ in range(5):
        graph.replay()                                   # warm-up replay
        torch.cuda.synchronize()
        time.sleep(0.03)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        t0 = time.perf_counter()
        fkl.check(timer.lib.fklhip_event_record(timer.e0, stream), "event_record")
        graph.replay()
        fkl.check(timer.lib.fklhip_event_record(timer.e1, stream), "event_record")
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / args.steps
        ms = C.c_float()
        fkl.check(timer.lib.fklhip_event_elapsed_ms(C.byref(ms), timer.e0, timer.e1), "event_elapsed")
        graph_runs.append((wall, ms.value / args.steps))
    if out3.cpu().numpy().tobytes() != got3.tobytes():
        print("bench.py: the graph replay's output differs from the eager launches'", file=sys.stderr)
        sys.exit(3)
    r3["graph_replay"] = {"ms_per_step_graph": min(w for w, _ in graph_runs), "kernel_us_graph": min(d for _, d in graph_runs) * 1e3,
                          "runs_wall_ms_per_step": [w for w, _ in graph_runs], "runs_kernel_us": [d * 1e3 for _, d in graph_runs],
                          "note": "K steps captured once into a HIP graph of K kernel nodes, one replay timed (wall clock around replay + "
                                  "synchronise, events around the replay); best of 5"}
    del graph
    # and one long batch: what a launch costs once the first launches after the idle state are a small part of the batch
    # (the second of two such batches: the first also pays for the launch queue's and the runtime's argument buffers growing)
    timer.run(f3, 1000, 300, settle=0)
    long_wall_ms, long_dev_ms = timer.run(f3, 1000, 0, settle=0)
    r3["kernel_us_1000_launches"] = long_dev_ms * 1e3
    # wall clock per step of the same batch: the one synchronisation at the end of a timed region (10 - 20 us) is then a
    # thousandth of a step instead of a twentieth
    r3["ms_per_step_1000_launches"] = long_wall_ms
    # the same 64 crops to planes of twice the rows (224 x 448): what a launch costs that does not depend on its size, and what
    # 38.5 MB more of output cost once the kernel runs (the source bytes are the same, so they count for nothing here)
    out3x2 = torch.zeros((64, 3, 448, 224), dtype=torch.float32, device=dev)
    f3x2 = lambda: cases.crop_resize_norm_split(src3, c3["rects"], (224, 448), c3["sub"], c3["div"], out3x2)
    # (both in batches of at most 50 launches: longer sequences of the larger launch read up to 20 % slower from about
    # 2 ms on, which would be charged to the marginal cost)
    short = min(args.steps, 50)
    twice = min(timer.run(f3x2, short, args.warmup)[1] * 1e3 for _ in range(3))
    once = min(again) if short == args.steps else min(timer.run(f3, short, args.warmup)[1] * 1e3 for _ in range(3))
    r3["twice_the_rows"] = {"launches_per_batch": short, "kernel_us_once": once, "kernel_us": twice, "marginal_us": twice - once, "fixed_us": 2 * once - twice,
                            "marginal_gbs": 64 * 3 * 224 * 224 * 4 / ((twice - once) * 1e-6) / 1e9,
                            "marginal_frac": 64 * 3 * 224 * 224 * 4 / ((twice - once) * 1e-6) / 1e9 / HBM_PEAK_GBS}
    del out3x2

    if args.list_compiled:
        # kernel symbol of every chain compiled at run time ("fkd_jit_" + FNV-1a of the signature), for reading profiles
        for sig in (s for s, _ in fkl.signatures() if s not in built_in):
            h = 14695981039346656037
            for b in sig.encode() + b"\0":
                h = ((h ^ b) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
            print(f"fkd_jit_{h:016x}  {sig}", file=sys.stderr)

    # ---- CPU baseline: the same chain on this machine's host cores, one thread, bounded sample --------------------
    cpu = None
    if not args.no_cpu:
        import oracle_lib as ol
        kind = "reference" if ol.have_ref() else "port"
        fn = ol.ref_crop_resize_norm_split if kind == "reference" else ol.oracle_crop_resize_norm_split
        want = fn(c3["src"], c3["rects"], c3["dst"], c3["sub"], c3["div"])   # warm-up, and the parity check of this run
        if want.tobytes() != got3.tobytes():       # the claim is bit-identical output: any difference fails the run
            denom = np.maximum(np.abs(want), np.float32(1e-30))
            rel = float(np.max(np.abs(got3 - want) / denom))
            print(f"bench.py: GPU output differs from the CPU baseline (max rel {rel:.3e})", file=sys.stderr)
            sys.exit(3)
        iters, t_total = 0, 0.0
        best = 1e9
        while t_total < 12.0 and iters < 200:
            t0 = time.perf_counter()
            fn(c3["src"], c3["rects"], c3["dst"], c3["sub"], c3["div"])
            dt = time.perf_counter() - t0
            best = min(best, dt)
            t_total += dt
            iters += 1
        cpu = {"value": 64 * 224 * 224 / 1e6 / best, "unit": "Mpix/s", "cores": 1, "kind": kind,
               "sample": f"configuration 3 at full size, best of {iters} single-threaded passes ({t_total:.1f} s of CPU work)",
               "ms_per_step": best * 1e3}

    line = {
        "metric": "fused-pipeline output Mpix/s (DNN preprocessing batch, configuration 3) on 1 MI355X",
        "value": r3["mpix_per_s"], "unit": "Mpix/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r3["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (seeded uniform random pixels and crop rectangles)",
        "config": {"workload": "configs[2]: 64 crops of uchar3 BGR 1920x1080 -> bilinear 224x224 IGNORE_AR -> BGR2RGB -> "
                               "(x-mean)/std -> TensorSplit planar float32 64x3x224x224, one fused launch per step",
                   "output_pixels_per_step": 64 * 224 * 224, "union_source_pixels": union_px,
                   "sum_of_crop_areas_bytes": int(sum(int(r[2]) * int(r[3]) for r in c3["rects"])) * 3},
        "roofline": {"bound": "hbm", "achieved": r3["achieved_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": r3["frac_of_hbm_peak"], "traffic": traffic_c3()[0], "traffic_note": traffic_c3()[1],
                     "algorithmic_bytes": a3, "kernel_us": r3["kernel_us"], "kernel": "fkd::k_" + r3["kernel"],
                     "kernel_us_5_runs_min_mean_max": r3["kernel_us_5_runs_min_mean_max"],
                     "kernel_us_1000_launches": r3["kernel_us_1000_launches"],
                     "frac_1000_launches": a3 / (r3["kernel_us_1000_launches"] * 1e-6) / 1e9 / HBM_PEAK_GBS,
                     "ms_per_step_1000_launches": r3["ms_per_step_1000_launches"],
                     "twice_the_rows": r3["twice_the_rows"], "graph_replay": r3["graph_replay"]},
        "cpu_baseline": cpu,
        "others": {k: v for k, v in results.items() if k != "c3"},
    }
    print(json.dumps(line))


# HBM bytes one launch of configuration 3 moves: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE of this script, scaled by what the
# same counters read for its plain copy chain of known size.  Measured under the profiler, not in this run (the counters
# need it attached): profiles/k_strip_config3.txt holds the commands and the readings.  The figure belongs to the kernel
# sources it was measured on: their digest is kept beside it, and a run on other sources reports no traffic figure rather
# than a stale one.
TRAFFIC_C3_BYTES = 52066000
TRAFFIC_C3_SOURCES = ("fusedkernellibrary_amd/csrc/fkd_kernels.hpp", "fusedkernellibrary_amd/csrc/fkd_launch.hpp",
                      "include/fkd/ops.hpp", "include/fkd/types.hpp", "include/fkd/launch_info.hpp")
TRAFFIC_C3_SOURCES_SHA256 = "89f542a2e77568a8a23247e74374aaaafbd2c26b093af28469f2c0811798663c"


def device_sources_sha256():
    import hashlib
    h = hashlib.sha256()
    for rel in TRAFFIC_C3_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def traffic_c3():
    """(bytes, note): the measured figure while the kernel sources are the ones it was measured on, else (None, why)."""
    now = device_sources_sha256()
    if now == TRAFFIC_C3_SOURCES_SHA256:
        return TRAFFIC_C3_BYTES, "rocprofv3 FETCH_SIZE + WRITE_SIZE, copy-calibrated (profiles/k_strip_config3.txt)"
    return None, ("the kernel sources changed since the counters were read (" + now[:16] + " now, " + TRAFFIC_C3_SOURCES_SHA256[:16] +
                  " then): re-measure as in profiles/k_strip_config3.txt")

if __name__ == "__main__":
    main()
