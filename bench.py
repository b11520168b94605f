#!/usr/bin/env python3
"""Benchmark of the GGUF quantized-matmul hot path on one MI355X.

Headline metric: Q4_K decode GEMV at Llama-3-8B FFN shapes, batch 1 -- gate/up
14336x4096 and down 4096x14336 -- in GB/s of algorithmic bytes (GGUF weight bytes + f32 activations
read + f32 outputs written) with everything resident in HBM.

One "step" is one decode pass of the hot path over a rotating pool of distinct FFN weight sets (the
pool is far larger than the 256 MB last-level cache, so every launch streams its weights from HBM):
per layer   [quantize(x) + gate and up GEMV] in one launch ; [quantize(h) + down GEMV] in one launch
(the decode GEMV quantizes its f32 activations to Q8_K in its own prologue).

The same JSON line carries
  roofline      the dominant kernel (the Q4_K gate+up GEMV launch, two thirds of the bytes):
                algorithmic bytes per launch / average launch duration, timed with HIP events over
                back-to-back launches on the kernel's stream
  cpu_baseline  the CPU oracle (scalar restatement of the ggml CPU path) timed on this host
  gemm          the batch-512 prefill GEMM over one Llama-3-8B-shaped layer (TOPS, % of the int8 MFMA peak)
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


def rel_err(y, ref, floor=1e-2):
    """max |y - ref| / max(|ref|, floor * rms(ref)): the path's tolerance metric (bar 1e-3)"""
    import numpy as np
    y, ref = np.asarray(y, np.float64), np.asarray(ref, np.float64)
    rms = float(np.sqrt(np.mean(ref * ref)))
    return float(np.max(np.abs(y - ref) / np.maximum(np.abs(ref), floor * rms + 1e-300)))


def observed_clocks():
    """current shader / memory clock as the driver reports them right now through sysfs (the level marked '*' in
    pp_dpm_sclk / pp_dpm_mclk of the first GPU that has them); None where they cannot be read.  No child process:
    a process that has initialised the GPU must not start one that re-executes itself."""
    import glob
    import re
    out = {}
    for key in ("sclk", "mclk", "fclk"):
        for path in sorted(glob.glob(f"/sys/class/drm/card*/device/pp_dpm_{key}")):
            try:
                txt = open(path).read()
            except OSError:
                continue
            m = re.search(r"(\d+)\s*Mhz\s*\*", txt, re.IGNORECASE)
            if m:
                out[key + "_mhz"] = int(m.group(1))
                break
    return out or None


HBM_PEAK_GBS = 8000.0     # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA

Q4_0, Q8_0, Q4_K, Q6_K, Q8_K = 2, 8, 12, 14, 15
TRAFFIC_SUMMARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "gate_up_traffic.json")
FFN_K, FFN_M = 4096, 14336


def alg_bytes(wbytes: int, k: int, m: int, n: int = 1) -> int:
    return wbytes + 4 * k * n + 4 * m * n


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--ramp", type=int, default=30,
                    help="untimed steps before the warmup steps: the first few milliseconds after the uploads run at a lower "
                         "clock (three warmup steps are 2 ms; the mean over the next 20 steps then reads 3 %% below the median)")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the pure-read ceiling measurement")
    ap.add_argument("--layers", type=int, default=32, help="distinct FFN weight sets in the rotating pool")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline budget (0 = skip)")
    ap.add_argument("--no-gemm", action="store_true", help="skip the batch-512 prefill GEMM section")
    ap.add_argument("--no-other", action="store_true",
                    help="skip the short timings of the other benchmark configurations (Q4_0 / Q8_0 GEMV, Q6_K head) "
                         "and of the expert-indexed and Q4_0 GEMM paths")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (known traffic, for scaling rocprofv3 HBM counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path has no multi-GPU part); use --gpus 1",
              file=sys.stderr)
        return 2

    import numpy as np
    import torch  # device memory and stream plumbing only

    from ollama_amd import qmm, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ctx = qmm.Context(0)
    info = ctx.device_info()
    # a real (non-null) stream: the library launches on it and the HIP events below are recorded on it
    stream = torch.cuda.Stream(device=dev)
    torch.cuda.set_stream(stream)
    assert stream.cuda_stream != 0
    ctx.set_stream(stream.cuda_stream)

    # ---- synthetic weights: one encoded FFN, the other pool entries are row-rotated copies
    t0 = time.time()
    base = {
        "gate": synth.weights(Q4_K, FFN_M, FFN_K, seed=1003),
        "up": synth.weights(Q4_K, FFN_M, FFN_K, seed=1013),
        "down": synth.weights(Q4_K, FFN_K, FFN_M, seed=1023),
    }
    pool = []
    for layer in range(args.layers):
        ent = {}
        for name, raw in base.items():
            m, k = (FFN_M, FFN_K) if name != "down" else (FFN_K, FFN_M)
            ent[name] = ctx.upload(Q4_K, np.roll(raw, layer * 37, axis=0) if layer else raw, k, m)
        pool.append(ent)
    wbytes = base["gate"].size
    assert wbytes == base["down"].size == 33030144
    setup_s = time.time() - t0

    g = torch.Generator(device="cpu").manual_seed(2003)
    x = torch.randn(1, FFN_K, generator=g, dtype=torch.float32).to(dev)
    h = torch.randn(1, FFN_M, generator=g, dtype=torch.float32).to(dev)
    y_gate = torch.empty(1, FFN_M, dtype=torch.float32, device=dev)
    y_up = torch.empty(1, FFN_M, dtype=torch.float32, device=dev)
    y_down = torch.empty(1, FFN_K, dtype=torch.float32, device=dev)
    def step():
        for ent in pool:
            ctx.mulmat_multi_device([ent["gate"], ent["up"]], x.data_ptr(), 1, [y_gate.data_ptr(), y_up.data_ptr()])
            ctx.mulmat_device(ent["down"], h.data_ptr(), 1, y_down.data_ptr())

    def gate_up_only():
        for ent in pool:
            ctx.mulmat_multi_device([ent["gate"], ent["up"]], x.data_ptr(), 1, [y_gate.data_ptr(), y_up.data_ptr()])

    def timed(fn, iters):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(iters):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / 1e3  # seconds

    for _ in range(args.ramp + args.warmup):
        step()
    torch.cuda.synchronize()
    t_step = timed(step, args.steps)
    clocks_under_load = observed_clocks()
    bytes_per_step = args.layers * (2 * alg_bytes(wbytes, FFN_K, FFN_M) + alg_bytes(wbytes, FFN_M, FFN_K))
    value = bytes_per_step * args.steps / t_step / 1e9
    # the same step again, every step between events of its own: median and best next to the mean above
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    torch.cuda.synchronize()
    evs[0].record(stream)
    for i in range(args.steps):
        step()
        evs[i + 1].record(stream)
    torch.cuda.synchronize()
    per_step_ms = sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(args.steps))
    median_ms, best_ms = per_step_ms[len(per_step_ms) // 2], per_step_ms[0]

    # ---- the timed launches did the work: keep the outputs of the last step (the last pool entry's weights) for the
    # check against the CPU oracle, which runs after every timed section (device-to-device copies here: no host work and
    # no idle GPU between the timed sections)
    kept = {"gate": y_gate.clone(), "up": y_up.clone(), "down": y_down.clone()}

    # dominant kernel alone, back to back (HIP events on the stream the kernels run on), at ramped clocks like the step
    for _ in range(max(1, args.ramp // 4)):
        gate_up_only()
    t_k = timed(gate_up_only, args.steps)
    launches = args.layers * args.steps
    avg_launch_s = t_k / launches
    bytes_per_launch = 2 * wbytes + 4 * FFN_K + 2 * 4 * FFN_M  # two weight matrices, x once, two outputs
    achieved = bytes_per_launch / avg_launch_s / 1e9

    traffic_bytes = None
    if os.path.exists(TRAFFIC_SUMMARY):
        with open(TRAFFIC_SUMMARY) as f:
            traffic_bytes = json.load(f).get("hbm_bytes_per_launch")
    out = {
        "metric": "Q4_K decode GEMV GB/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "untimed_ramp_steps": args.ramp,
        "ms_per_step": round(t_step / args.steps * 1e3, 4),
        "ms_per_step_median": round(median_ms, 4),
        "ms_per_step_best": round(best_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {
            "workload": "Q4_K decode GEMV, Llama-3-8B FFN shapes (gate/up 14336x4096, down 4096x14336), batch 1, "
                        "f32 activations quantized to Q8_K inside the GEMV launch",
            "pool_layers": args.layers,
            "untimed_ramp_steps": args.ramp,
            "launches_per_step": 2 * args.layers,
            "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
            "device": info["name"],
            "compute_units": info["compute_units"],
            "clock_mhz_nominal": info["clock_mhz"],
            "clocks_observed_under_load": clocks_under_load,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "gemv_thin_kernel<PolQ4K, 1, true, 1, 1, 1, false, 1> (gate+up in one launch, 28672 rows x 4096)",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            # HBM bytes per launch from two rocprofv3 --pmc runs of this script (FETCH_SIZE and WRITE_SIZE, scaled by
            # what the same counters read for a 1 GiB copy); the figures and their commands are in the tracked summary
            "traffic": traffic_bytes,
            "avg_launch_us": round(avg_launch_s * 1e6, 3),
            "bytes_per_launch": int(bytes_per_launch),
        },
    }

    # ---- the same step captured once into a HIP graph on the stream and replayed (a separate figure, never `value`): the
    # 2 x pool_layers launches of a step without the host's per-call work between them
    gstep = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gstep, stream=stream):
        step()
    for _ in range(args.warmup):
        gstep.replay()
    t_g = timed(gstep.replay, args.steps)
    same = all(bool(torch.equal(a, b)) for a, b in ((y_gate, kept["gate"]), (y_up, kept["up"]), (y_down, kept["down"])))
    out["step_replayed_from_hip_graph"] = {"ms_per_step": round(t_g / args.steps * 1e3, 4),
                                           "GB/s": round(bytes_per_step * args.steps / t_g / 1e9, 1),
                                           "bit_identical_to_eager": same}
    del gstep
    if not same:
        print("bench.py: the replayed graph of the step differs from the eager step", file=sys.stderr)
        return 1

    # ---- what a pure read of the same bytes reaches in one launch on this machine (launch included): the
    # practical ceiling next to the GEMV's figure.  Best of a few grid shapes, rotating buffers like the weights.
    sr_path = os.path.join(os.path.dirname(qmm.LIB_PATH), "libmi_streamread.so")
    if os.path.exists(sr_path) and not args.no_ceiling:
        sr = ctypes.CDLL(sr_path)
        sr.mi_stream_read.restype = ctypes.c_int
        sr.mi_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                      ctypes.c_void_p]
        nbytes = bytes_per_launch // 16 * 16
        bufs = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev) for _ in range(16)]
        scratch = torch.zeros(8192, dtype=torch.int32, device=dev)
        best = None
        for threads in (256, 1024):
            for blocks in (256, 512, 1024, 2048, 4096, 8192):
                for unroll in (1, 2, 4, 8):
                    if blocks * threads > 4096 * 1024 // 2:
                        continue
                    fn = lambda: [sr.mi_stream_read(b.data_ptr(), nbytes, blocks, threads, unroll, scratch.data_ptr(),
                                                    stream.cuda_stream) for b in bufs]
                    fn()
                    tm = timed(fn, 3) / (3 * len(bufs))
                    if os.environ.get("CEIL_VERBOSE"):
                        print(f"read {threads}x{blocks} unroll {unroll}: {tm * 1e6:.2f} us", file=sys.stderr)
                    if best is None or tm < best[0]:
                        best = (tm, blocks, unroll, threads)
        ceil_gbs = nbytes / best[0] / 1e9
        out["read_ceiling"] = {"bytes": nbytes, "us": round(best[0] * 1e6, 2), "GB/s": round(ceil_gbs, 1),
                               "frac_of_hbm_peak": round(ceil_gbs / HBM_PEAK_GBS, 4),
                               "grid": f"{best[1]} workgroups of {best[3]}, {best[2]} loads of 16 bytes in flight per lane",
                               "what": "one launch that only reads the gate+up launch's bytes, back to back over rotating buffers"}
        out["roofline"]["frac_of_read_ceiling"] = round(achieved / ceil_gbs, 4)
        del bufs

    # ---- prefill GEMM: one Llama-3-8B-shaped layer at batch 512 (the secondary metric)
    if not args.no_gemm:
        NB = 512
        layer = [("attn_q", Q4_K, 4096, 4096), ("attn_k", Q4_K, 1024, 4096), ("attn_v", Q4_K, 1024, 4096),
                 ("attn_o", Q4_K, 4096, 4096), ("ffn_gate", Q4_K, 14336, 4096), ("ffn_up", Q4_K, 14336, 4096),
                 ("ffn_down", Q6_K, 4096, 14336)]
        small = {}
        for name, t, m, k in layer:
            if (t, m, k) not in small:
                rows = min(m, 2048)
                raw = synth.weights(t, rows, k, seed=1005 + m % 89)
                small[(t, m, k)] = np.tile(raw, ((m + rows - 1) // rows, 1))[:m]
        copies = 3  # rotate three copies of the layer (414 MB) so weights are not cache-resident
        gw = [[ctx.upload(t, np.roll(small[(t, m, k)], 11 * c, axis=0), k, m) for name, t, m, k in layer]
              for c in range(copies)]
        xb = torch.randn(NB, 4096, generator=g, dtype=torch.float32).to(dev)
        hb = torch.randn(NB, 14336, generator=g, dtype=torch.float32).to(dev)
        ys = [torch.empty(NB, m, dtype=torch.float32, device=dev) for name, t, m, k in layer]
        actb_x = ctx.act_create(Q8_K, 4096, NB)
        actb_h = ctx.act_create(Q8_K, 14336, NB)

        def layer_pass():
            for c in range(copies):
                ctx.act_quantize(actb_x, xb.data_ptr(), NB, qmm.DEVICE)
                # q, k and v share x and are small: one launch over their concatenated rows
                ctx.mulmat_q8_multi_device(gw[c][0:3], actb_x, [ys[0].data_ptr(), ys[1].data_ptr(), ys[2].data_ptr()])
                ctx.mulmat_q8_device(gw[c][3], actb_x, ys[3].data_ptr())
                # gate and up share x as well: one launch of the fp16 kernel over both (the bits of two launches)
                ctx.mulmat_q8_multi_device(gw[c][4:6], actb_x, [ys[4].data_ptr(), ys[5].data_ptr()])
                # down has its input to itself: the one-call form quantizes only the planes a Q6_K product reads
                ctx.mulmat_device(gw[c][6], hb.data_ptr(), NB, ys[6].data_ptr())

        layer_pass()
        gsteps = max(17, args.steps // 4)  # x 3 rotating copies: at least 50 timed launches per matrix
        t_g = timed(layer_pass, gsteps) / (gsteps * copies)
        ops = sum(2.0 * NB * m * k for name, t, m, k in layer)
        per = {}
        ctx.act_quantize(actb_h, hb.data_ptr(), NB, qmm.DEVICE)  # for the per-matrix timing of ffn_down
        for i, (name, t, m, k) in enumerate(layer):
            if name in ("attn_v", "ffn_up", "attn_o"):
                continue
            act = actb_h if k == 14336 else actb_x
            fn = lambda i=i, act=act: [ctx.mulmat_q8_device(gw[c][i], act, ys[i].data_ptr()) for c in range(copies)]
            fn()
            tm = timed(fn, gsteps) / (gsteps * copies)
            per[name] = {"us": round(tm * 1e6, 1), "tops": round(2.0 * NB * m * k / tm / 1e12, 1)}
        fn = lambda: [ctx.mulmat_q8_multi_device(gw[c][0:3], actb_x, [ys[0].data_ptr(), ys[1].data_ptr(), ys[2].data_ptr()])
                      for c in range(copies)]
        fn()
        tm = timed(fn, gsteps) / (gsteps * copies)
        per["attn_q+k+v (one launch)"] = {"us": round(tm * 1e6, 1), "tops": round(2.0 * NB * 6144 * 4096 / tm / 1e12, 1)}
        fn = lambda: [ctx.mulmat_q8_multi_device(gw[c][4:6], actb_x, [ys[4].data_ptr(), ys[5].data_ptr()]) for c in range(copies)]
        fn()
        tm = timed(fn, gsteps) / (gsteps * copies)
        per["ffn_gate+up (one launch)"] = {"us": round(tm * 1e6, 1), "tops": round(2.0 * NB * 2 * 14336 * 4096 / tm / 1e12, 1)}
        out["gemm"] = {
            "metric": "prefill GEMM TOPS (Q4_K gate + up in one launch on fp16 MFMA, the rest on int8 MFMA; priced against the int8 peak)",
            "workload": "one Llama-3-8B-shaped layer, batch 512: q/o 4096x4096, k/v 1024x4096, gate/up 14336x4096 Q4_K; "
                        "down 4096x14336 Q6_K; activations quantized to Q8_K on GPU inside the timed region",
            "value": round(ops / t_g / 1e12, 1),
            "unit": "TOPS",
            "us_per_layer": round(t_g * 1e6, 1),
            "gop_per_layer": round(ops / 1e9, 2),
            "roofline": {"bound": "mfma", "achieved": round(ops / t_g / 1e12, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                         "frac": round(ops / t_g / 1e12 / INT8_PEAK_TOPS, 4)},
            "per_matrix": per,
        }
        # the same layer at batch 2048 (not the configuration the metric is quoted on): every matrix then has tiles
        # enough to fill the CUs, which is what the 4096-row projections lack at batch 512
        NB2 = 2048
        xb2 = torch.randn(NB2, 4096, generator=g, dtype=torch.float32).to(dev)
        hb2 = torch.randn(NB2, 14336, generator=g, dtype=torch.float32).to(dev)
        ys2 = [torch.empty(NB2, m, dtype=torch.float32, device=dev) for name, t, m, k in layer]
        actb_x2 = ctx.act_create(Q8_K, 4096, NB2)

        def layer_pass_2048():
            for c in range(copies):
                ctx.act_quantize(actb_x2, xb2.data_ptr(), NB2, qmm.DEVICE)
                ctx.mulmat_q8_multi_device(gw[c][0:3], actb_x2, [ys2[0].data_ptr(), ys2[1].data_ptr(), ys2[2].data_ptr()])
                ctx.mulmat_q8_device(gw[c][3], actb_x2, ys2[3].data_ptr())
                ctx.mulmat_q8_multi_device(gw[c][4:6], actb_x2, [ys2[4].data_ptr(), ys2[5].data_ptr()])
                ctx.mulmat_device(gw[c][6], hb2.data_ptr(), NB2, ys2[6].data_ptr())

        layer_pass_2048()
        t_g2 = timed(layer_pass_2048, gsteps) / (gsteps * copies)
        out["gemm"]["batch_2048"] = {"value": round(ops * (NB2 / NB) / t_g2 / 1e12, 1), "unit": "TOPS",
                                     "us_per_layer": round(t_g2 * 1e6, 1)}
        actb_x2.free()
        del xb2, hb2, ys2
        for row in gw:
            for wt in row:
                wt.free()
        # what the matrix cores sustain on this machine when they do nothing else (random operands, a few ms per
        # launch, two waves per SIMD on every CU): the practical ceiling of an MFMA-bound kernel
        mr_path = os.path.join(os.path.dirname(qmm.LIB_PATH), "libmi_mfmarate.so")
        if os.path.exists(mr_path) and not args.no_ceiling:
            mr = ctypes.CDLL(mr_path)
            mr.mi_mfma_rate.restype = ctypes.c_int
            mr.mi_mfma_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
            mout = torch.zeros(256, dtype=torch.float32, device=dev)
            mclk = torch.zeros(2, dtype=torch.int64, device=dev)
            blocks, iters = 2 * info["compute_units"], 8000
            ceil = {}
            for kind, name, flop in ((0, "f16_32x32x16", 32768.0), (1, "i8_32x32x32", 65536.0),
                                     (2, "f16_32x32x16_prefill_operands", 32768.0), (3, "i8_32x32x32_prefill_operands", 65536.0)):
                fn = lambda: mr.mi_mfma_rate(kind, iters, blocks, mout.data_ptr(), mclk.data_ptr(), stream.cuda_stream)
                timed(fn, 2)
                tm = timed(fn, 3) / 3
                c = mclk.cpu().tolist()
                ceil[name] = {"T(FL)OP/s": round(blocks * 4 * 4.0 * iters * flop / tm / 1e12, 1), "ms_per_launch": round(tm * 1e3, 2),
                              "shader_clock_mhz": round(c[0] / (c[1] / 100.0)) if c[1] else None}
            ceil["what"] = ("a loop of nothing but MFMAs, 4 independent accumulators per wave, 2 waves per SIMD on every CU, timed like the GEMM "
                            "launches; on random bits, and on operands distributed like the prefill kernels' (normal activations quantized to "
                            "int8; block scale x nibble as fp16, bare nibbles for int8); the clock is the one workgroup 0 ran at (its cycle "
                            "counter over the 100 MHz counter)")
            out["gemm"]["mfma_ceiling"] = ceil
            gate = per.get("ffn_gate")
            if gate:  # the fp16 kernel issues 17 MFMAs for 16 algorithmic ones
                out["gemm"]["ffn_gate_frac_of_f16_ceiling"] = round(gate["tops"] * 17 / 16 / ceil["f16_32x32x16"]["T(FL)OP/s"], 4)
                out["gemm"]["ffn_gate_frac_of_f16_ceiling_prefill_operands"] = round(
                    gate["tops"] * 17 / 16 / ceil["f16_32x32x16_prefill_operands"]["T(FL)OP/s"], 4)

    # ---- the other configurations, one short timing each: f32 activations in HBM, quantization included
    if not args.no_other:
        def plain_rows(t, rows, k):
            # rows of an unquantized weight type (F32 / F16 / BF16) as the bytes a GGUF file holds
            w = (np.random.default_rng(1100 + t).standard_normal((rows, k)) * 0.02).astype(np.float32)
            if t == qmm.F16:
                return w.astype(np.float16).view(np.uint8)
            return (w.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8) if t == qmm.BF16 else w.view(np.uint8)

        def time_mulmat(t, m, k, n, copies, path=qmm.PATH_AUTO):
            rows = min(m, 2048)
            base = plain_rows(t, rows, k) if t in qmm.PLAIN_TYPES else synth.weights(t, rows, k, seed=1100 + t)
            raw = np.tile(base, ((m + rows - 1) // rows, 1))[:m]
            ws = [ctx.upload(t, np.roll(raw, 13 * c, axis=0), k, m) for c in range(copies)]
            xs = torch.randn(n, k, generator=g, dtype=torch.float32).to(dev)
            yo = torch.empty(n, m, dtype=torch.float32, device=dev)
            fn = lambda: [ctx.mulmat_device(wt, xs.data_ptr(), n, yo.data_ptr(), path) for wt in ws]
            fn()
            reps = max(2, 200 // copies)
            tm = timed(fn, reps) / (reps * copies)
            for wt in ws:
                wt.free()
            return tm, raw.size

        other = {}
        for label, t, m, k, ns, copies in (("Q4_K q_proj 4096x4096", Q4_K, 4096, 4096, (2, 4, 8), 40),  # (one column would share the headline kernel's name in a profile)
                                           ("Q4_0 GEMV 4096x4096", Q4_0, 4096, 4096, (1,), 40),
                                           ("Q8_0 skinny 4096x4096", Q8_0, 4096, 4096, (1, 2, 4, 8), 40),
                                           ("Q6_K ffn_down 4096x14336", Q6_K, 4096, 14336, (4, 8), 10),
                                           ("Q6_K v_proj 1024x4096", Q6_K, 1024, 4096, (4, 8), 40),
                                           ("Q6_K head 128256x4096", Q6_K, 128256, 4096, (1, 8), 3)):
            for n in ns:
                tm, wb = time_mulmat(t, m, k, n, copies)
                gbs = alg_bytes(wb, k, m, n) / tm / 1e9
                other[f"{label} B={n}"] = {"us": round(tm * 1e6, 2), "GB/s": round(gbs, 1),
                                           "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
        # q, k and v of a layer through one multi call (f32 x in, quantization included)
        qkv_ms = (4096, 1024, 1024)
        qkv_sets = []
        for c in range(20):
            qkv_sets.append([ctx.upload(Q4_K, np.roll(synth.weights(Q4_K, m, 4096, seed=1150 + i), 13 * c, axis=0), 4096, m)
                             for i, m in enumerate(qkv_ms)])
        for n in (2, 4, 8):  # (one column would share the headline kernel's name in a profile)
            xs = torch.randn(n, 4096, generator=g, dtype=torch.float32).to(dev)
            yq = [torch.empty(n, m, dtype=torch.float32, device=dev) for m in qkv_ms]
            fn = lambda: [ctx.mulmat_multi_device(ws3, xs.data_ptr(), n, [y_.data_ptr() for y_ in yq]) for ws3 in qkv_sets]
            fn()
            tm = timed(fn, 10) / (10 * len(qkv_sets))
            other[f"Q4_K attn q+k+v (6144x4096) one call B={n}"] = {"us": round(tm * 1e6, 2)}
        for ws3 in qkv_sets:
            for wt in ws3:
                wt.free()
        for label, t in (("Q4_0", Q4_0), ("Q8_0", Q8_0)):
            tm, _ = time_mulmat(t, 4096, 4096, 512, 6)
            other[f"{label} GEMM 4096x4096 B=512"] = {"us": round(tm * 1e6, 1), "TOPS": round(2.0 * 512 * 4096 * 4096 / tm / 1e12, 1)}
        # every Mulmat of one decoded token of a Llama-3-8B-shaped model in the Q4_K_M mixture (attn_v and ffn_down in Q6_K in
        # half of the layers, the output head in Q6_K): q + k + v in one call, o, gate + up in one call, down, per layer, each
        # launch reading what the one before wrote (the dependency chain of a real decode; attention, norms and the
        # gating between the products are not part of the path and not run); weights distinct per layer, 4.6 GB in all
        if len(pool) >= 32:
            def tiled(t, m, k, seed, shift):
                rows = min(m, 2048)
                return np.roll(np.tile(synth.weights(t, rows, k, seed=seed), ((m + rows - 1) // rows, 1))[:m], shift, axis=0)
            att = []
            for li in range(32):
                more = li % 2 == 0  # the layers the mixture gives more bits
                att.append({"q": ctx.upload(Q4_K, tiled(Q4_K, 4096, 4096, 1301, 7 * li), 4096, 4096),
                            "k": ctx.upload(Q4_K, tiled(Q4_K, 1024, 4096, 1302, 7 * li), 4096, 1024),
                            "v": ctx.upload(Q6_K if more else Q4_K, tiled(Q6_K if more else Q4_K, 1024, 4096, 1303, 7 * li), 4096, 1024),
                            "o": ctx.upload(Q4_K, tiled(Q4_K, 4096, 4096, 1304, 7 * li), 4096, 4096),
                            "down6": ctx.upload(Q6_K, tiled(Q6_K, FFN_K, FFN_M, 1305, 7 * li), FFN_M, FFN_K) if more else None})
            head = ctx.upload(Q6_K, tiled(Q6_K, 128256, 4096, 1306, 0), 4096, 128256)
            hid = torch.randn(1, 4096, generator=g, dtype=torch.float32).to(dev)
            yq = torch.empty(1, 4096, dtype=torch.float32, device=dev)
            yk = torch.empty(1, 1024, dtype=torch.float32, device=dev)
            yv = torch.empty(1, 1024, dtype=torch.float32, device=dev)
            yo = torch.empty(1, 4096, dtype=torch.float32, device=dev)
            yg = torch.empty(1, FFN_M, dtype=torch.float32, device=dev)
            yu = torch.empty(1, FFN_M, dtype=torch.float32, device=dev)
            yl = torch.empty(1, 128256, dtype=torch.float32, device=dev)

            def token():
                for li in range(32):
                    a, f = att[li], pool[li]
                    ctx.mulmat_multi_device([a["q"], a["k"], a["v"]], hid.data_ptr(), 1, [yq.data_ptr(), yk.data_ptr(), yv.data_ptr()])
                    ctx.mulmat_device(a["o"], yq.data_ptr(), 1, yo.data_ptr())
                    ctx.mulmat_multi_device([f["gate"], f["up"]], yo.data_ptr(), 1, [yg.data_ptr(), yu.data_ptr()])
                    ctx.mulmat_device(a["down6"] or f["down"], yg.data_ptr(), 1, hid.data_ptr())
                ctx.mulmat_device(head, hid.data_ptr(), 1, yl.data_ptr())

            token()
            token()
            tm = timed(token, 5) / 5
            used = [head]
            for li in range(32):
                a, f = att[li], pool[li]
                used += [a["q"], a["k"], a["v"], a["o"], f["gate"], f["up"], a["down6"] or f["down"]]
            tok_bytes = sum(wt.gguf_bytes for wt in used)
            other["Llama-3-8B-shaped Q4_K_M token: all Mulmat calls of a decode step (32 layers + head), one after the other"] = {
                "us": round(tm * 1e6, 1), "launch_groups": 32 * 4 + 1, "weight_GB": round(tok_bytes / 1e9, 3),
                "GB/s": round(tok_bytes / tm / 1e9, 1), "frac_of_hbm_peak": round(tok_bytes / tm / 1e9 / HBM_PEAK_GBS, 4),
                "tokens/s_if_nothing_else_ran": round(1.0 / tm, 1)}
            # the same 129 calls captured once into a HIP graph on the stream and replayed: what a caller that builds its
            # decode step as a graph (Context.Compute of a fixed graph) pays; the replay's outputs are checked against the
            # eager calls' bit for bit, on replays with eager work between them
            hid0 = hid.clone()
            token()
            want_l = yl.clone()
            hid.copy_(hid0)
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=stream):
                token()
            same = True
            for _ in range(3):
                hid.copy_(hid0)
                gr.replay()
                torch.cuda.synchronize()
                same = same and bool(torch.equal(yl, want_l))
                token()
                torch.cuda.synchronize()
            if not same:
                print("bench.py: the replayed graph of the token differs from the eager calls", file=sys.stderr)
                return 1
            gr.replay()
            tg = timed(gr.replay, 5) / 5
            other["Llama-3-8B-shaped Q4_K_M token: the same calls replayed from one captured HIP graph"] = {
                "us": round(tg * 1e6, 1), "GB/s": round(tok_bytes / tg / 1e9, 1),
                "frac_of_hbm_peak": round(tok_bytes / tg / 1e9 / HBM_PEAK_GBS, 4),
                "tokens/s_if_nothing_else_ran": round(1.0 / tg, 1), "bit_identical_to_eager": True}
            del gr
            for a in att:
                for wt in a.values():
                    if wt is not None:
                        wt.free()
            head.free()
        # Q5_K (the tensors the Q4_K_S mixture raises): kept as a Q4_K tensor of rows twice as long
        for label, m, k, ns, copies in (("Q5_K v_proj 1024x4096", 1024, 4096, (1, 4), 40), ("Q5_K ffn_down 4096x14336", 4096, 14336, (1, 4), 10)):
            for n in ns:
                tm, wb = time_mulmat(qmm.Q5_K, m, k, n, copies)
                gbs = alg_bytes(wb, k, m, n) / tm / 1e9
                other[f"{label} B={n}"] = {"us": round(tm * 1e6, 2), "GB/s": round(gbs, 1),
                                           "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
        tm, _ = time_mulmat(qmm.Q5_K, 4096, 4096, 512, 6)
        other["Q5_K GEMM 4096x4096 B=512"] = {"us": round(tm * 1e6, 1), "TOPS": round(2.0 * 512 * 4096 * 4096 / tm / 1e12, 1)}
        # the unquantized weight types (F16 / BF16 / F32 files, and the tensors a K-quant file keeps unquantized)
        for label, t, m, k, ns, copies in (("F16 ffn_gate 14336x4096", qmm.F16, 14336, 4096, (1, 4, 8), 6),
                                           ("BF16 q_proj 4096x4096", qmm.BF16, 4096, 4096, (1, 8), 16),
                                           ("F32 q_proj 4096x4096", qmm.F32, 4096, 4096, (1,), 8)):
            for n in ns:
                tm, wb = time_mulmat(t, m, k, n, copies)
                gbs = alg_bytes(wb, k, m, n) / tm / 1e9
                other[f"{label} B={n}"] = {"us": round(tm * 1e6, 2), "GB/s": round(gbs, 1),
                                           "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
        for label, t in (("F16", qmm.F16), ("BF16", qmm.BF16), ("F32", qmm.F32)):
            tm, _ = time_mulmat(t, 4096, 4096, 512, 6)
            other[f"{label} GEMM 4096x4096 B=512"] = {"us": round(tm * 1e6, 1), "TFLOP/s": round(2.0 * 512 * 4096 * 4096 / tm / 1e12, 1)}
        tm, _ = time_mulmat(qmm.F16, 14336, 4096, 512, 3)
        other["F16 GEMM ffn_gate 14336x4096 B=512"] = {"us": round(tm * 1e6, 1), "TFLOP/s": round(2.0 * 512 * 14336 * 4096 / tm / 1e12, 1)}
        # expert-indexed product: 128 experts of 768x2048 (Q4_K), 8 used per token
        n_exp, n_used, em, ek = 128, 8, 768, 2048
        raw = np.tile(synth.weights(Q4_K, 2048, ek, seed=1201), (n_exp * em // 2048, 1))
        stacks = [ctx.upload(Q4_K, np.roll(raw, 13 * c, axis=0), ek, n_exp * em) for c in range(6)]
        for toks in (1, 8, 512):
            xe = torch.randn(toks, 1, ek, generator=g, dtype=torch.float32).to(dev)
            ids = torch.stack([torch.randperm(n_exp, generator=g)[:n_used] for _ in range(toks)]).to(torch.int32).to(dev)
            ye = torch.empty(toks, n_used, em, dtype=torch.float32, device=dev)
            fn = lambda: [ctx.mulmat_id_device(st, n_exp, xe.data_ptr(), 1, ids.data_ptr(), n_used, toks, ye.data_ptr())
                          for st in stacks]
            fn()
            tm = timed(fn, 10) / (10 * len(stacks))
            other[f"MulmatID Q4_K 128x(768x2048) top-8 tokens={toks}"] = {"us": round(tm * 1e6, 2)}
        # a Mixtral-8x7B-shaped down projection: 8 experts of 4096 x 14336, 2 used per token, one token (66 MB of weights read)
        raw_mix = np.tile(synth.weights(Q4_K, 2048, FFN_M, seed=1202), (8 * FFN_K // 2048, 1))
        mix_stacks = [ctx.upload(Q4_K, np.roll(raw_mix, 13 * c, axis=0), FFN_M, 8 * FFN_K) for c in range(3)]
        xmix = torch.randn(1, 1, FFN_M, generator=g, dtype=torch.float32).to(dev)
        idmix = torch.tensor([[5, 2]], dtype=torch.int32).to(dev)
        ymix = torch.empty(1, 2, FFN_K, dtype=torch.float32, device=dev)
        fn = lambda: [ctx.mulmat_id_device(st, 8, xmix.data_ptr(), 1, idmix.data_ptr(), 2, 1, ymix.data_ptr()) for st in mix_stacks]
        fn()
        tm = timed(fn, 10) / (10 * len(mix_stacks))
        other["MulmatID Q4_K 8x(4096x14336) top-2 tokens=1"] = {"us": round(tm * 1e6, 2), "GB/s": round(2 * wbytes / tm / 1e9, 1)}
        for st in mix_stacks:
            st.free()
        del raw_mix
        # the same on MXFP4 expert stacks (kept as Q8_0 planes): 32 experts of 2880 x 2880, 4 used per token
        mx_exp, mx_used, mm, mk = 32, 4, 2880, 2880
        raw_mx = np.tile(synth.weights(qmm.MXFP4, 2880, mk, seed=1203), (mx_exp, 1))
        mx_stacks = [ctx.upload(qmm.MXFP4, np.roll(raw_mx, 13 * c, axis=0), mk, mx_exp * mm) for c in range(4)]
        for toks in (1, 8, 512):
            xm = torch.randn(toks, 1, mk, generator=g, dtype=torch.float32).to(dev)
            idm = torch.stack([torch.randperm(mx_exp, generator=g)[:mx_used] for _ in range(toks)]).to(torch.int32).to(dev)
            ym = torch.empty(toks, mx_used, mm, dtype=torch.float32, device=dev)
            fn = lambda: [ctx.mulmat_id_device(st, mx_exp, xm.data_ptr(), 1, idm.data_ptr(), mx_used, toks, ym.data_ptr())
                          for st in mx_stacks]
            fn()
            tm = timed(fn, 10) / (10 * len(mx_stacks))
            other[f"MulmatID MXFP4 32x(2880x2880) top-4 tokens={toks}"] = {"us": round(tm * 1e6, 2)}
        for st in mx_stacks:
            st.free()
        # one token through a mixture-of-experts feed-forward block: gate and up experts with their gating in
        # one launch, the down experts (one activation row per used expert) in a second
        raw_d = np.tile(synth.weights(Q4_K, 2048, em, seed=1202), (n_exp * ek // 2048, 1))
        downs = [ctx.upload(Q4_K, np.roll(raw_d, 13 * c, axis=0), em, n_exp * ek) for c in range(3)]
        xe = torch.randn(1, 1, ek, generator=g, dtype=torch.float32).to(dev)
        ids = torch.randperm(n_exp, generator=g)[:n_used].reshape(1, n_used).to(torch.int32).to(dev)
        he = torch.empty(1, n_used, em, dtype=torch.float32, device=dev)
        yd = torch.empty(1, n_used, ek, dtype=torch.float32, device=dev)

        def moe_block():
            for c in range(3):
                ctx.mulmat_id_swiglu_device(stacks[2 * c], stacks[2 * c + 1], n_exp, xe.data_ptr(), 1, ids.data_ptr(), n_used, 1,
                                            he.data_ptr())
                ctx.mulmat_id_device(downs[c], n_exp, he.data_ptr(), n_used, ids.data_ptr(), n_used, 1, yd.data_ptr())

        moe_block()
        tm = timed(moe_block, 20) / (20 * 3)
        other["decode expert FFN block 128x(768x2048) top-8: gate, up and gating in one launch, down in a second"] = {"us": round(tm * 1e6, 2)}
        for st in stacks + downs:
            st.free()
        # decode feed-forward block with its producers, on the main pool: RMSNorm -> gate, up (one launch) and
        # SILU(gate) * up -> down (one launch), against the same block through the stand-alone f32 kernels
        gnorm = torch.randn(FFN_K, generator=g, dtype=torch.float32).to(dev)
        xn = torch.empty(1, FFN_K, dtype=torch.float32, device=dev)
        act = torch.empty(1, FFN_M, dtype=torch.float32, device=dev)
        vp = ctypes.c_void_p

        def block_fused():
            for ent in pool:
                ctx.mulmat_produced_device([ent["gate"], ent["up"]], qmm.PRODUCE_RMSNORM, gnorm.data_ptr(), x.data_ptr(), 1,
                                           [y_gate.data_ptr(), y_up.data_ptr()], eps=1e-5)
                ctx.mulmat_produced_device([ent["down"]], qmm.PRODUCE_SWIGLU, y_up.data_ptr(), y_gate.data_ptr(), 1,
                                           [y_down.data_ptr()])

        def block_unfused():
            L = qmm.lib()
            for ent in pool:
                qmm._check(L.mi_qmm_rms_norm(ctx._h, vp(x.data_ptr()), vp(gnorm.data_ptr()), 1e-5, FFN_K, 1, vp(xn.data_ptr()), qmm.DEVICE))
                ctx.mulmat_multi_device([ent["gate"], ent["up"]], xn.data_ptr(), 1, [y_gate.data_ptr(), y_up.data_ptr()])
                qmm._check(L.mi_qmm_swiglu(ctx._h, vp(y_gate.data_ptr()), vp(y_up.data_ptr()), FFN_M, 1, vp(act.data_ptr()), qmm.DEVICE))
                ctx.mulmat_device(ent["down"], act.data_ptr(), 1, y_down.data_ptr())

        def block_paired():
            for ent in pool:
                ctx.mulmat_swiglu_device(ent["gate"], ent["up"], x.data_ptr(), 1, act.data_ptr(), qmm.PRODUCE_RMSNORM,
                                         gnorm.data_ptr(), 1e-5)
                ctx.mulmat_device(ent["down"], act.data_ptr(), 1, y_down.data_ptr())

        for label, fn in (("RMSNorm, gate, up and their gating in one launch, down in a second", block_paired),
                          ("RMSNorm and SwiGLU inside the two product launches", block_fused),
                          ("rms_norm, gate+up, swiglu, down: four launches", block_unfused)):
            fn()
            tm = timed(fn, 5) / (5 * len(pool))
            other[f"decode FFN block, {label}"] = {"us": round(tm * 1e6, 2)}
        # the headline step at a few tokens (several sequences decoding together): gate + up in one call, down in a second
        for n in (2, 3, 4, 8):
            xb = torch.randn(n, FFN_K, generator=g, dtype=torch.float32).to(dev)
            hb = torch.randn(n, FFN_M, generator=g, dtype=torch.float32).to(dev)
            ygb = torch.empty(n, FFN_M, dtype=torch.float32, device=dev)
            yub = torch.empty(n, FFN_M, dtype=torch.float32, device=dev)
            ydb = torch.empty(n, FFN_K, dtype=torch.float32, device=dev)

            def step_n():
                for ent in pool:
                    ctx.mulmat_multi_device([ent["gate"], ent["up"]], xb.data_ptr(), n, [ygb.data_ptr(), yub.data_ptr()])
                    ctx.mulmat_device(ent["down"], hb.data_ptr(), n, ydb.data_ptr())

            step_n()
            tm = timed(step_n, 5) / (5 * len(pool))
            other[f"Q4_K decode FFN step (gate + up one call, down) B={n}"] = {"us": round(tm * 1e6, 2), "GB/s": round(3 * wbytes / tm / 1e9, 1)}
        # weight encoders (a one-off step when a quantized model is made): f32 rows on the device -> GGUF blocks
        xe = (torch.randn(FFN_M, FFN_K, generator=g, dtype=torch.float32) * 0.02).to(dev)
        for label, t in (("Q4_0", Q4_0), ("Q8_0", Q8_0), ("Q4_K", Q4_K), ("Q6_K", Q6_K)):
            oe = torch.empty(FFN_M * qmm.row_size(t, FFN_K), dtype=torch.uint8, device=dev)
            fn = lambda: ctx.quantize_weights_device(t, xe.data_ptr(), FFN_K, FFN_M, oe.data_ptr())
            fn()
            tm = timed(fn, 3) / 3
            other[f"weight encoder {label} 14336x4096 f32 -> blocks"] = {"us": round(tm * 1e6, 1), "Gweights/s": round(FFN_M * FFN_K / tm / 1e9, 1)}
        out["other_configs"] = other

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    # ---- the outputs of the timed step against the CPU oracle on a slab of rows (after every timed section)
    import oracle
    last = args.layers - 1
    slab = 64
    checks = {}
    for name, act, k, m in (("gate", x, FFN_K, FFN_M), ("up", x, FFN_K, FFN_M), ("down", h, FFN_M, FFN_K)):
        raw = np.roll(base[name], last * 37, axis=0) if last else base[name]
        want = oracle.mul_mat(Q4_K, np.ascontiguousarray(raw[:slab]), k, slab, act.cpu().numpy(), nthreads=4)
        err = rel_err(kept[name].cpu().numpy()[:, :slab], want)
        checks[name] = err
        if not err <= 1e-3:
            print(f"bench.py: y_{name} of the timed step differs from the oracle (rel err {err})", file=sys.stderr)
            return 1
    out["config"]["outputs_checked_against_oracle"] = {k_: float(f"{v_:.2e}") for k_, v_ in checks.items()}

    # ---- CPU baseline: the oracle (scalar port of the ggml CPU path) on this host's cores -------
    if args.cpu_seconds > 0:
        xh = x.cpu().numpy()

        def cpu_rate(threads, seconds):
            reps, t_cpu = 0, 0.0
            t_begin = time.time()
            while t_cpu < seconds:
                t1 = time.time()
                oracle.mul_mat(Q4_K, base["gate"], FFN_K, FFN_M, xh, nthreads=threads)
                t_cpu += time.time() - t1
                reps += 1
                if time.time() - t_begin > 3 * seconds:
                    break
            return alg_bytes(wbytes, FFN_K, FFN_M) * reps / t_cpu / 1e9, reps, t_cpu

        threads = min(16, os.cpu_count() or 1)
        cpu_gbs, reps, t_cpu = cpu_rate(threads, args.cpu_seconds * 0.7)
        one_gbs, reps1, t_cpu1 = cpu_rate(1, args.cpu_seconds * 0.3)
        out["cpu_baseline"] = {
            "value": round(cpu_gbs, 2),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": f"{reps} x Q4_K gate GEMV 14336x4096 batch 1 (quantize + dot), {t_cpu:.1f} s of CPU work",
            "one_thread": {"value": round(one_gbs, 2), "cores": 1, "sample": f"{reps1} x the same product, {t_cpu1:.1f} s"},
        }
    out["config"]["setup_s"] = round(setup_s, 1)
    print(json.dumps(out), flush=True)
    for ent in pool:
        for w in ent.values():
            w.free()
    ctx.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
