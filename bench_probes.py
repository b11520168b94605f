#!/usr/bin/env python3
"""Machine questions behind the kernels' designs, each answered by a small probe kernel (ollama_amd/csrc/probes.hip).

    python bench_probes.py [--probe all|empty|lds|lane_map|copy_stream|handoff] [--iters N]

prints one JSON line per probe.  Not part of the product and not part of bench.py's metric: these are the measurements
that the design notes quote (launch cost of an empty kernel; which lanes the LDS serves together on a 16-byte read;
what the address coalescer makes of different lane orders; what the copy stream of a staged small-batch kernel costs by
itself and which copies cost what; what a fence-free hand-off of a partial tile between workgroups costs).  For the
LDS probe the bank-conflict counter comes from running this file under `rocprofv3 --pmc SQ_LDS_BANK_CONFLICT`: the
dispatches of lds_b128_kernel appear in the order of the patterns printed here.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "ollama_amd", "libmi_probes.so")


def load():
    if not os.path.exists(LIB):
        raise SystemExit(f"{LIB} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
    L = ctypes.CDLL(LIB)
    vp, ci, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
    L.mi_probe_empty.argtypes = [ci, ci, vp]
    L.mi_probe_lds_b128.argtypes = [vp, ci, ci, vp, vp]
    L.mi_probe_lane_map.argtypes = [ci, vp, i64, ci, ci, vp, vp]
    L.mi_probe_flood_read.argtypes = [ci, vp, ci, vp, vp]
    L.mi_probe_copy_stream.argtypes = [vp, vp, vp, vp, vp, vp, i64, ci, ci, ci, vp, vp]
    L.mi_probe_handoff.argtypes = [vp, vp, vp, vp, ci, ci, ctypes.c_uint, ci, vp]
    return L


def timed(fn, iters, stream):
    stream.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    stream.synchronize()
    return (time.perf_counter() - t0) / iters


def check(rc):
    if rc != 0:
        raise RuntimeError(f"probe launch failed: {rc}")


def probe_empty(L, dev, stream, iters):
    """launch-to-launch time of a kernel that does nothing, one wave and one full grid of 1024-thread workgroups"""
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    out = {}
    for name, blocks, threads in (("one_wave", 1, 64), ("a_workgroup_of_1024_per_cu", cus, 1024), ("16_waves_per_cu_in_4_workgroups", 4 * cus, 256)):
        fn = lambda: check(L.mi_probe_empty(blocks, threads, stream.cuda_stream))
        timed(fn, 200, stream)
        out[name + "_us"] = round(min(timed(fn, iters, stream) for _ in range(5)) * 1e6, 2)
    return {"probe": "empty_kernel_launch_to_launch", **out, "launches_per_timing": iters}


def lds_patterns():
    """byte offsets of the 64 lanes' 16-byte reads; a pattern is free of conflicts iff the lanes that the LDS serves in
    one cycle fall on different 16-byte slots modulo 256 bytes (or on the same address)"""
    pats = {}
    pats["linear"] = [16 * l for l in range(64)]
    # free of conflicts iff 16 CONSECUTIVE lanes are served together: lanes 16..31 use the slots rotated by four
    pats["for_16_consecutive_lanes"] = [(512 if l >= 32 else 0) + 256 * ((l >> 4) & 1) + 16 * ((l + (4 if (l >> 4) & 1 else 0)) & 15) for l in range(64)]
    # free of conflicts iff the groups are quads {0,3,5,6} and {1,2,4,7} of each half-wave
    ga, gb = [0, 3, 5, 6], [1, 2, 4, 7]
    offs = []
    for l in range(64):
        q, j, half = (l & 31) >> 2, l & 3, l >> 5
        grp, pos = (0, ga.index(q)) if q in ga else (1, gb.index(q))
        offs.append(512 * half + 256 * grp + 16 * (4 * pos + j))
    pats["for_quads_0356_and_1247"] = offs
    pats["rows_of_128_bytes_piece_0"] = [128 * l for l in range(64)]                       # a tile as stored, unswizzled
    pats["rows_of_128_bytes_xor_row_bits"] = [128 * l + 16 * ((l >> 1) & 7) for l in range(64)]  # piece ^ ((row >> 1) & 7)
    pats["one_slot"] = [256 * l for l in range(64)]
    return pats


def probe_lds(L, dev, stream, iters):
    res = {}
    out = torch.zeros(3, dtype=torch.int64, device=dev)
    n = 12 * 1024
    for waves in (1, 4):
        for name, offs in lds_patterns().items():
            o = torch.tensor(offs, dtype=torch.int32, device=dev)
            check(L.mi_probe_lds_b128(o.data_ptr(), n, waves, out.data_ptr(), stream.cuda_stream))
            stream.synchronize()
            c = out.cpu().tolist()
            res.setdefault(name, {})[f"{waves}_wave" + ("s" if waves > 1 else "")] = round(c[0] / (c[1] * waves), 2)
    return {"probe": "ds_read_b128_lane_groups", "cycles_per_wave_read": res, "reads_per_wave": n,
            "note": "one wave alone is bound by the latency of its twelve reads in flight; with four waves a read of 1 KiB without conflicts "
                    "takes 8 cycles of the LDS (128 bytes per cycle); dispatch order under rocprofv3 = all patterns at one wave, then at four"}


def probe_lane_map(L, dev, stream, iters):
    """33 MB of 144-byte records, 16 rows per wave-step: which lane reads which 16 bytes"""
    rows, nsb = 14336, 16
    nbuf = 6  # rotate: 6 x 33 MB is more than the caches hold
    bufs = [torch.randint(0, 255, (rows * nsb * 144 + 4096,), dtype=torch.uint8, device=dev) for _ in range(nbuf)]
    out = torch.zeros(256, dtype=torch.int32, device=dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    res = {}
    for mode, name in ((0, "lane = row + 16 * piece (MFMA operand order)"), (1, "lane = 4 * row + piece (quads on 64 contiguous bytes)"),
                       (3, "lane = 8 * row + piece (eight lanes on a row's 128 contiguous bytes)"), (2, "linear 1 KiB per load (no rows)")):
        best = None
        for blocks in (cus // 2, cus, 2 * cus, 4 * cus):
            def fn():
                for b in bufs:
                    check(L.mi_probe_lane_map(mode, b.data_ptr(), rows, nsb, blocks, out.data_ptr(), stream.cuda_stream))
            timed(fn, 3, stream)
            t = min(timed(fn, max(3, iters // 20), stream) for _ in range(3)) / nbuf
            if best is None or t < best[0]:
                best = (t, blocks)
        nbytes = rows * nsb * 128
        res[name] = {"us": round(best[0] * 1e6, 2), "GB/s": round(nbytes / best[0] / 1e9), "workgroups_of_4_waves": best[1]}
    return {"probe": "lane_order_of_16_byte_loads", "bytes_read_per_launch": rows * nsb * 128, "modes": res}


def probe_flood_read(L, dev, stream, iters):
    """the gate + up launch of the deep direct-load kernel as a pure read: 1792 groups of 16 rows x 2304 bytes, all requested at once"""
    groups, nbuf = 1792, 4
    bufs = [torch.randint(0, 255, (groups * 36864,), dtype=torch.uint8, device=dev) for _ in range(nbuf)]
    out = torch.zeros(256, dtype=torch.int32, device=dev)
    res = {}
    for mode, name in ((0, "quads of lanes on 64 contiguous bytes of 16 rows (the kernel's order)"), (1, "contiguous: 1 KiB per load, 8 whole rows per wave")):
        def fn():
            for b in bufs:
                check(L.mi_probe_flood_read(mode, b.data_ptr(), groups, out.data_ptr(), stream.cuda_stream))
        timed(fn, 5, stream)
        t = min(timed(fn, max(5, iters // 10), stream) for _ in range(3)) / nbuf
        res[name] = {"us": round(t * 1e6, 2), "GB/s": round(groups * 36864 / t / 1e9)}
    return {"probe": "all_loads_in_flight_at_once", "bytes": groups * 36864, "shape": "256 workgroups of 14 waves, 18 loads of 16 bytes per lane", "modes": res}


def probe_copy_stream(L, dev, stream, iters):
    """the output head's shape: 128256 rows x 16 super-blocks, a row group of 16 per wave-step"""
    rows, nsb = 128256, 16
    mk = lambda n: torch.randint(0, 255, (n + 4096,), dtype=torch.uint8, device=dev)
    ql, qh, sc, d = mk(rows * nsb * 128), mk(rows * nsb * 64), mk(rows * nsb * 16), mk(rows * nsb * 2)
    aq, ad = mk(nsb * 2048), mk(nsb * 512)
    out = torch.zeros(256, dtype=torch.int32, device=dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    res = {}
    for mask, name in ((63, "all nine copies"), (63 - 16, "without the activations' quants"), (3 + 32, "without sub-block and super-block scales and activation quants"),
                       (3, "low and high quant bits only (91 % of the bytes)"), (1, "low quant bits only (61 %)"), (0, "none (loop and LDS reads only)")):
        fn = lambda: check(L.mi_probe_copy_stream(ql.data_ptr(), qh.data_ptr(), sc.data_ptr(), d.data_ptr(), aq.data_ptr(), ad.data_ptr(), rows, nsb,
                                                  mask, 4 * cus, out.data_ptr(), stream.cuda_stream))
        timed(fn, 3, stream)
        res[name] = round(min(timed(fn, max(3, iters // 20), stream) for _ in range(3)) * 1e6, 1)
    return {"probe": "copy_stream_of_a_staged_kernel", "rows": rows, "super_blocks_per_row": nsb, "weight_bytes": rows * nsb * 210,
            "waves": "2 per workgroup, 4 workgroups per CU", "us": res}


def probe_handoff(L, dev, stream, iters):
    """64 tiles x 4 partial planes of 128 KiB: everyone writes its plane (no hand-off) against two hops through flags"""
    tiles = 64
    part = torch.zeros(4 * tiles * 32768, dtype=torch.float32, device=dev)
    y = torch.zeros(tiles * 32768, dtype=torch.float32, device=dev)
    flag = torch.zeros(4 * tiles, dtype=torch.int32, device=dev)
    err = torch.zeros(1, dtype=torch.int32, device=dev)
    epoch = [0]
    def run(hops):
        epoch[0] += 1
        check(L.mi_probe_handoff(part.data_ptr(), flag.data_ptr(), y.data_ptr(), err.data_ptr(), tiles, hops, epoch[0], 1 << 16, stream.cuda_stream))
    res = {}
    for hops in (0, 2):
        fn = lambda: run(hops)
        timed(fn, 10, stream)
        res[f"hops_{hops}_us"] = round(min(timed(fn, max(10, iters // 5), stream) for _ in range(3)) * 1e6, 2)
    # every value must be 1 + 2 + 3 + 4 on every checked launch
    wrong = 0
    for _ in range(20):
        y.zero_()
        run(2)
        stream.synchronize()
        wrong += int((y != 10.0).sum().item())
    res["per_hop_us"] = round((res["hops_2_us"] - res["hops_0_us"]) / 2, 2)
    return {"probe": "fence_free_handoff_between_workgroups", "tiles": tiles, "tile_bytes": 131072, **res, "wrong_values_in_20_checked_launches": wrong,
            "polls_that_ran_out": int(err.item())}


PROBES = {"empty": probe_empty, "lds": probe_lds, "lane_map": probe_lane_map, "flood_read": probe_flood_read, "copy_stream": probe_copy_stream, "handoff": probe_handoff}


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--probe", default="all", choices=["all"] + list(PROBES))
    ap.add_argument("--iters", type=int, default=200, help="launches per timing of the short probes (the long ones take a twentieth)")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("bench_probes.py needs a GPU")
    L = load()
    dev = torch.device("cuda:0")
    stream = torch.cuda.Stream(dev)
    with torch.cuda.stream(stream):
        for name, fn in PROBES.items():
            if args.probe in ("all", name):
                print(json.dumps(fn(L, dev, stream, args.iters)), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
