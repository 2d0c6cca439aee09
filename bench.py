#!/usr/bin/env python3
"""Benchmark of the block-floating-point data-format path on one MI355X.

One "step" is one pass of the streaming conversion over one batch of synthetic input that is
already resident in HBM: tilize + pack of a bf16 [8,1,8192,8192] tensor (U(-8,8), seed 2) to
Bfp8_b, then unpack + untilize back to bf16.  `value` is the algorithmic bytes both kernels move
per step divided by the wall time per step.  The same run times the Bfp8_b-weight GEMM
(8192^3 and the 4096x4096-weight shapes) and the BERT-large FFN block, and the CPU oracle on a
bounded sample of the same workload on the host cores.

Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16

# HBM bytes per launch on the streaming workload, measured with two rocprofv3 --pmc runs (FETCH_SIZE,
# then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads for a plain 1 GiB
# device copy (FETCH_SIZE reads half the KiB actually fetched on this part: factor 2.0; WRITE_SIZE
# factor 1.0).  Summary: profiles/streaming_bf16_8x8192x8192_hbm_traffic.txt
MEASURED_TRAFFIC_BYTES = {
    # (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0) x 1024 per launch; the two factors come from the 1 GiB copy in the same runs
    "tilize_pack": 1644306558,      # 1,644,167,168 algorithmic
    "unpack_untilize": 1644428290,
    # GEMM kernels, same method: profiles/gemm_bfp8b_bench_shapes_hbm_traffic.txt (the forms with a workspace include
    # their first pass / their reduction; the FFN figure is the sum of its two matmuls)
    "gemm_8192": 1287420995, "gemm_8192_ws": 1954009668, "gemm_M8192": 354720605, "gemm_M8192_ws": 521480554,
    "gemm_M512": 55775136, "gemm_M256": 36911741, "gemm_M256_ws": 70524592, "gemm_M32": 21361155, "gemm_M64": 23731588, "gemm_M128": 28477299,
    "ffn": 134321260,
}


# where the `traffic` figures come from: counter summaries under profiles/, taken with the library built at this commit
TRAFFIC_SOURCE = {"streaming": "profiles/streaming_bf16_8x8192x8192_hbm_traffic.txt",
                  "gemm": "profiles/gemm_bfp8b_bench_shapes_hbm_traffic.txt",
                  "library_commit": "260d22f"}  # the counters were read on the library built from this commit


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=20)
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-CPU oracle timing")
    p.add_argument("--no-gemm", action="store_true", help="skip the GEMM / FFN section")
    p.add_argument("--eager-timing", action="store_true", help="time every launch eagerly, no HIP graph (for counter runs)")
    p.add_argument("--gemm-only", action="store_true", help="skip the streaming section's secondary lines (fp32 sources, queue forms)")
    p.add_argument("--sustained-seconds", type=float, default=2.0,
                   help="length of the sustained 8192^3 loops whose clock and power are sampled (0: skip them)")
    p.add_argument("--no-host-push", action="store_true", help="skip the host push / read-back lines (PCIe inclusive)")
    p.add_argument("--ablation", action="store_true",
                   help="instead of the benchmark: time the fused 8192^3 GEMM of the library and of every tt-buda_amd/libttbfp_ablate<bits>.so "
                        "beside it (make -C tt-buda_amd/csrc ablate ABLATE=<bits>: parts of the kernel's work left out, wrong results on purpose), "
                        "each in a sustained loop with clock and power sampled; prints one JSON line")
    p.add_argument("--data-probe", action="store_true",
                   help="instead of the benchmark: the fused 8192^3 GEMM on random, constant and all-zero operands, each in a sustained loop "
                        "with clock and power sampled (the kernel's cycle count does not depend on the data; the clock the power cap allows does); "
                        "prints one JSON line")
    p.add_argument("--power-probe", type=float, default=0.0, metavar="SECONDS",
                   help="instead of the benchmark: run each 8192^3 GEMM form (fused, with workspace, the vendor library's plain bf16 "
                        "GEMM through torch.matmul) back to back for SECONDS while rocm-smi is polled for clock and power; prints one JSON line")
    return p.parse_args()


def power_probe(seconds, torch, capi):
    """Sustained 8192^3 loops with clock and power samples: what the part settles at once it has warmed into its power limit."""
    import re
    import subprocess
    import threading

    F = capi.DataFormatCode
    n = 8192
    g = torch.Generator(device="cuda:0").manual_seed(30)
    wp = capi.tilize_pack(torch.randn(1, 1, n, n, generator=g, device="cuda:0") * 0.02, F.Bfp8_b)
    g = torch.Generator(device="cuda:0").manual_seed(31)
    x = torch.randn(n, n, generator=g, device="cuda:0").bfloat16()
    wb = (torch.randn(n, n, generator=g, device="cuda:0") * 0.02).bfloat16()
    y = torch.empty(n, n, dtype=torch.bfloat16, device="cuda:0")
    ws = torch.empty(capi.gemm_workspace_bytes(n, n, n), dtype=torch.uint8, device="cuda:0")
    forms = {"fused Bfp8_b-weight GEMM": lambda: capi.gemm_bfp8b(x, wp, n, out=y),
             "Bfp8_b-weight GEMM with a workspace (bf16 panel)": lambda: capi.gemm_bfp8b(x, wp, n, out=y, workspace=ws),
             "vendor library, plain bf16 GEMM (torch.matmul)": lambda: torch.matmul(x, wb, out=y)}
    out = {}
    for name, fn in forms.items():
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        samples, stop = [], threading.Event()

        def poll():
            while not stop.is_set():
                # socket power and the clock of each of the eight XCDs (their mean is what the matrix cores run at)
                txt = subprocess.run(["amd-smi", "metric", "-p", "-c"], capture_output=True, text=True).stdout
                xcd = [int(m) for m in re.findall(r"GFX_\d+:\s*\n\s*CLK: (\d+) MHz", txt)]
                watts = re.search(r"SOCKET_POWER: ([0-9.]+) W", txt)
                samples.append((sum(xcd) / len(xcd) if xcd else None, float(watts.group(1)) if watts else None))
                stop.wait(0.25)

        th = threading.Thread(target=poll)
        t0 = time.perf_counter()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        launches = 0
        th.start()
        while time.perf_counter() - t0 < seconds:
            for _ in range(50):
                fn()
            launches += 50
            torch.cuda.synchronize()
        e1.record()
        torch.cuda.synchronize()
        stop.set()
        th.join()
        ms = e0.elapsed_time(e1) / launches
        late = samples[len(samples) // 2:]  # the second half of the run: the part has settled
        clocks = sorted(c for c, _ in late if c)
        watts = sorted(w for _, w in late if w)
        tf = 2.0 * n ** 3 / ms / 1e9
        out[name] = {"ms": round(ms, 4), "tflops": round(tf, 1), "frac_of_2500": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "launches": launches,
                     "xcd_clock_mhz_median": round(clocks[len(clocks) // 2]) if clocks else None,
                     "socket_power_w_median": watts[len(watts) // 2] if watts else None,
                     # what the matrix cores could do at the clock the part actually ran at: 256 CUs x 4 SIMDs x 1024 flop per clock
                     "mfma_peak_at_that_clock_tflops": round(256 * 4 * 1024 * clocks[len(clocks) // 2] * 1e6 / 1e12, 1) if clocks else None}
    cap = re.search(r"Max Graphics Package Power \(W\): ([0-9.]+)", subprocess.run(["rocm-smi", "--showmaxpower"], capture_output=True, text=True).stdout)
    print(json.dumps({"power_probe_seconds": seconds, "shape": "8192 x 8192 x 8192", "max_package_power_w": float(cap.group(1)) if cap else None,
                      "max_clock_mhz": 2400, "forms": out}))


def sustained(fn, seconds, flops, torch):
    """fn() launched back to back for `seconds` while amd-smi is polled: average launch time over the whole run and the
    median XCD clock and socket power of its second half (the part has then settled into its power limit)."""
    import re
    import subprocess
    import threading

    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    samples, stop = [], threading.Event()

    def poll():
        while not stop.is_set():
            try:
                txt = subprocess.run(["amd-smi", "metric", "-p", "-c"], capture_output=True, text=True, timeout=20).stdout
            except Exception:
                return
            xcd = [int(m) for m in re.findall(r"GFX_\d+:\s*\n\s*CLK: (\d+) MHz", txt)]
            watts = re.search(r"SOCKET_POWER: ([0-9.]+) W", txt)
            samples.append((time.perf_counter(), sum(xcd) / len(xcd) if xcd else None, float(watts.group(1)) if watts else None))
            stop.wait(0.1)

    th = threading.Thread(target=poll)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    launches = 0
    th.start()
    while time.perf_counter() - t0 < seconds:
        for _ in range(50):
            fn()
        launches += 50
        torch.cuda.synchronize()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    stop.set()
    th.join()
    ms = e0.elapsed_time(e1) / launches
    late = [(c, w) for t, c, w in samples if t0 + (t1 - t0) / 2 <= t <= t1]  # sampled while the loop ran, second half
    clocks = sorted(c for c, _ in late if c)
    watts = sorted(w for _, w in late if w)
    tf = flops / ms / 1e9
    clock = clocks[len(clocks) // 2] if clocks else None
    return {"seconds": round(t1 - t0, 2), "launches": launches, "ms": round(ms, 4), "tflops": round(tf, 1),
            "frac_of_peak": round(tf / MFMA_BF16_PEAK_TFLOPS, 4), "samples": len(late),
            "clock_mhz": round(clock) if clock else None, "power_w": watts[len(watts) // 2] if watts else None,
            # what the matrix cores deliver at the clock the part ran at: 256 CUs x 4 SIMDs x 1024 flop per clock
            "mfma_peak_at_clock_tflops": round(256 * 4 * 1024 * clock * 1e6 / 1e12, 1) if clock else None,
            "frac_of_peak_at_clock": round(tf / (256 * 4 * 1024 * clock * 1e6 / 1e12), 4) if clock else None}


def ablation_probe(seconds, torch, capi):
    """What the parts of the 256 x 256 kernel cost: the same 8192^3 launch from the library and from its ablated copies."""
    import ctypes
    import glob

    F = capi.DataFormatCode
    n = 8192
    g = torch.Generator(device="cuda:0").manual_seed(30)
    wp = capi.tilize_pack(torch.randn(1, 1, n, n, generator=g, device="cuda:0") * 0.02, F.Bfp8_b)
    g = torch.Generator(device="cuda:0").manual_seed(31)
    x = torch.randn(n, n, generator=g, device="cuda:0").bfloat16()
    y = torch.empty(n, n, dtype=torch.bfloat16, device="cuda:0")
    left_out = {1: "dequantization", 2: "X loads", 4: "W fetches", 8: "MFMAs", 16: "LDS stores of the dequantized weights"}
    libs = [("the library (nothing left out)", capi.lib())]
    for path in sorted(glob.glob(os.path.join(os.path.dirname(capi.LIB_PATH), "libttbfp_ablate*.so"))):
        bits = int(os.path.basename(path)[len("libttbfp_ablate"):-3])
        L = ctypes.CDLL(path)
        L.ttbfp_gemm_bfp8b_bf16.restype, L.ttbfp_gemm_bfp8b_bf16.argtypes = capi.SYMBOLS["ttbfp_gemm_bfp8b_bf16"]
        libs.append(("without " + ", ".join(v for k, v in left_out.items() if bits & k) + " (TTBFP_ABLATE=%d)" % bits, L))
    out = {}
    for name, L in libs:
        def fn(L=L):
            st = L.ttbfp_gemm_bfp8b_bf16(n, n, n, x.data_ptr(), wp.data_ptr(), None, 0, y.data_ptr(), F.Float16_b, capi._stream())
            assert st == 0
        out[name] = sustained(fn, seconds, 2.0 * n ** 3, torch)
    print(json.dumps({"ablation_seconds": seconds, "shape": "8192 x 8192 x 8192, fused kernel on 256 x 256 tiles, bf16 result", "forms": out}))


def data_probe(seconds, torch, capi):
    """The same launch on operands that make the matrix cores switch more or fewer bits: what the power cap costs."""
    F = capi.DataFormatCode
    n = 8192
    g = torch.Generator(device="cuda:0").manual_seed(30)
    w_rand = capi.tilize_pack(torch.randn(1, 1, n, n, generator=g, device="cuda:0") * 0.02, F.Bfp8_b)
    g = torch.Generator(device="cuda:0").manual_seed(31)
    x_rand = torch.randn(n, n, generator=g, device="cuda:0").bfloat16()
    w_const = capi.tilize_pack(torch.full((1, 1, n, n), 0.0123, device="cuda:0"), F.Bfp8_b)
    w_zero = torch.zeros_like(w_rand)
    x_zero = torch.zeros(n, n, dtype=torch.bfloat16, device="cuda:0")
    y = torch.empty(n, n, dtype=torch.bfloat16, device="cuda:0")
    cases = [("W N(0,0.02), X N(0,1): the benchmark's operands", w_rand, x_rand), ("W one value (0.0123), X N(0,1)", w_const, x_rand),
             ("W all-zero tiles, X N(0,1)", w_zero, x_rand), ("W N(0,0.02), X zero", w_rand, x_zero), ("W zero, X zero", w_zero, x_zero)]
    out = {}
    for name, wp, x in cases:
        r = sustained(lambda: capi.gemm_bfp8b(x, wp, n, out=y), seconds, 2.0 * n ** 3, torch)
        if r["clock_mhz"]:
            r["cycles_per_simd"] = round(r["ms"] * 1e-3 * r["clock_mhz"] * 1e6)
        out[name] = r
    print(json.dumps({"data_probe_seconds": seconds, "shape": "8192 x 8192 x 8192, fused kernel, bf16 result", "forms": out}))


def time_kernel(fn, steps, warmup, torch):
    """(average, minimum) duration of fn() in ms by HIP events on the stream the kernels are launched on.  The average
    comes from one pair of events around `steps` back-to-back launches (an event between launches would put its own
    marker into the queue and widen the gaps), the minimum from a second pass with an event after every launch."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    avg = e0.elapsed_time(e1) / steps
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    evs[0].record()
    for i in range(steps):
        fn()
        evs[i + 1].record()
    torch.cuda.synchronize()
    return avg, min(evs[i].elapsed_time(evs[i + 1]) for i in range(steps))


def time_launches(fn, steps, warmup, torch):
    """Average device time of fn() in ms for kernels shorter than the host's launch path (a Python call through ctypes
    costs 15-25 us): `steps` launches recorded back to back into one HIP graph, the replay bracketed by two events.
    Returns None if the launches cannot be captured."""
    try:
        for _ in range(max(warmup, 1)):
            fn()  # first calls also do the kernels' one-time attribute set-up, which must stay out of the capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(steps):
                fn()
        graph.replay()
        torch.cuda.synchronize()
        per = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            per.append(e0.elapsed_time(e1) / steps)
        return sorted(per)[1]
    except Exception as exc:  # timing aid only: the eager figure stands
        print("bench.py: graph timing unavailable (%s)" % exc, file=sys.stderr)
        torch.cuda.synchronize()
        return None


def host_push_lines(torch):
    """push_input of a pinned host tensor into a Bfp8_b queue and get_output back, through the host layer, host link
    included: the figure the reference publishes for its own push path (8.7 GB/s fp32 / fp16, 8.9 GB/s bf16 on chip 0:
    pybuda/test/galaxy/utils/verify_push_bandwidth.py:10-12) on its own shapes
    (pybuda/test/galaxy/test_galaxy_inputs.py:119) and on 128 MiB.  GB/s of row-major bytes on the host side.  These
    lines are PCIe bound and are not part of `value`."""
    from tt_buda_amd import tensor as T
    from tt_buda_amd._C import DataFormat as DF
    from tt_buda_amd._C import backend_api as B
    from tt_buda_amd.backend import BackendAPI

    OK = B.BackendStatusCode.Success
    api = BackendAPI(0)
    lines = {"reference_published_gbs": {"float32": 8.7, "float16": 8.7, "bfloat16": 8.9,
                                         "source": "pybuda/test/galaxy/utils/verify_push_bandwidth.py:10-12 (other hardware)"}}
    cases = [("galaxy_shape1_32x1x128x128", (32, 1, 128, 128)), ("galaxy_shape2_256x1x1028x384", (256, 1, 1028, 384)),
             ("128MiB", None)]
    try:
        for tag, shp in cases:
            for dtype, dname in ((torch.float32, "fp32"), (torch.bfloat16, "bf16")):
                shape = shp or ((8, 1, 2048, 2048) if dtype == torch.float32 else (8, 1, 2048, 4096))
                n, rows, cols = shape[0], (shape[2] + 31) // 32 * 32, (shape[3] + 31) // 32 * 32
                name = "hostpush_%s_%s" % (tag, dname)
                q = api.create_queue(name, DF.Bfp8_b, (1, rows, cols), num_slots=n, input_count=n)
                x = torch.rand(*shape, dtype=torch.float32).to(dtype).pin_memory()
                desc = T.pytorch_tensor_to_tensor_desc(x)
                nbytes = x.numel() * x.element_size()
                push_s, get_s = [], []
                for it in range(8):
                    t0 = time.perf_counter()
                    st = B.push_input(q, desc, False, 5, -1)
                    t1 = time.perf_counter()
                    assert st == OK, B.last_error()
                    out = B.PytorchTensorDesc()
                    if dtype == torch.float32:
                        out.format = DF.Float32
                    t2 = time.perf_counter()
                    st = B.get_output(q, out, False, 5, -1, shape[2] if shape[2] != rows else 0, shape[3] if shape[3] != cols else 0)
                    t3 = time.perf_counter()
                    assert st == OK, B.last_error()
                    assert list(out.shape) == list(shape), (list(out.shape), shape)
                    assert B.free_tensor(out) == OK and B.pop_output(q, False, 5) == OK
                    if it >= 2:  # the first rounds fill the block pools
                        push_s.append(t1 - t0)
                        get_s.append(t3 - t2)
                pm, gm = sorted(push_s)[len(push_s) // 2], sorted(get_s)[len(get_s) // 2]
                lines["%s_%s" % (tag, dname)] = {"shape": list(shape), "bytes": nbytes, "queue_format": "Bfp8_b",
                                                 "push_input_ms": round(pm * 1e3, 4), "push_input_gbs": round(nbytes / pm / 1e9, 2),
                                                 "get_output_ms": round(gm * 1e3, 4), "get_output_gbs": round(nbytes / gm / 1e9, 2)}
    finally:
        api.shutdown()
    lines["note"] = ("pinned host tensor -> push_input (H2D copy + tilize/pack into the queue) and get_output (unpack/untilize + D2H copy into "
                     "pooled pinned memory); wall clock of the call, median of 6 after 2 warm-up rounds; host link included, never part of `value`")
    return lines


def roofline(bound, achieved, peak, unit, traffic=None):
    return {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": traffic}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (every box here has one); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch

    from tt_buda_amd import capi

    F = capi.DataFormatCode
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    capi.check(capi.lib().ttbfp_init(0))
    dev = "cuda:0"
    if args.power_probe > 0:
        power_probe(args.power_probe, torch, capi)
        return
    if args.ablation:
        ablation_probe(args.sustained_seconds or 2.0, torch, capi)
        return
    if args.data_probe:
        data_probe(args.sustained_seconds or 2.0, torch, capi)
        return

    # ---- streaming workload: bf16 [8,1,8192,8192], U(-8,8), seed 2 --------------------------------
    shape = (8, 1, 8192, 8192)
    g = torch.Generator(device=dev).manual_seed(2)
    x = torch.empty(shape, dtype=torch.bfloat16, device=dev)
    for w in range(shape[0]):  # slice by slice keeps the fp32 temporary small
        x[w] = (torch.rand(shape[1:], generator=g, device=dev) * 16 - 8).bfloat16()
    elems = x.numel()
    packed = torch.empty(capi.packed_size(F.Bfp8_b, shape), dtype=torch.uint8, device=dev)
    back = torch.empty_like(x)
    bytes_pack = elems * 2 + packed.numel()      # 3.0625 B/elem: bf16 in, Bfp8_b out
    bytes_unpack = packed.numel() + elems * 2    # same the other way

    def step():
        capi.tilize_pack(x, F.Bfp8_b, out=packed)
        capi.unpack_untilize(packed, F.Bfp8_b, shape, out=back)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    value = (bytes_pack + bytes_unpack) / (ms_per_step * 1e-3) / 1e9

    pack_ms, pack_min = time_kernel(lambda: capi.tilize_pack(x, F.Bfp8_b, out=packed), args.steps, args.warmup, torch)
    unpack_ms, unpack_min = time_kernel(lambda: capi.unpack_untilize(packed, F.Bfp8_b, shape, out=back), args.steps,
                                        args.warmup, torch)
    pack_gbs = bytes_pack / (pack_ms * 1e-3) / 1e9
    unpack_gbs = bytes_unpack / (unpack_ms * 1e-3) / 1e9
    kernels = {
        "tilize_pack_bf16_to_bfp8b": dict(ms=round(pack_ms, 4), min_ms=round(pack_min, 4), bytes=bytes_pack,
                                          roofline=roofline("hbm", pack_gbs, HBM_PEAK_GBS, "GB/s",
                                                            MEASURED_TRAFFIC_BYTES["tilize_pack"])),
        "unpack_untilize_bfp8b_to_bf16": dict(ms=round(unpack_ms, 4), min_ms=round(unpack_min, 4), bytes=bytes_unpack,
                                              roofline=roofline("hbm", unpack_gbs, HBM_PEAK_GBS, "GB/s",
                                                                MEASURED_TRAFFIC_BYTES["unpack_untilize"])),
    }
    dominant = "tilize_pack_bf16_to_bfp8b" if pack_ms >= unpack_ms else "unpack_untilize_bfp8b_to_bf16"
    # yardstick, and the reference the traffic counters are scaled by: a plain device-to-device copy of the same 1 GiB tensor
    spare = torch.empty_like(x)
    copy_ms, _ = time_kernel(lambda: capi.check(capi.lib().ttbfp_memcpy_d2d(spare.data_ptr(), x.data_ptr(), elems * 2, capi._stream())),
                             args.steps, args.warmup, torch)
    del spare
    kernels["reference_copy_1GiB_device_to_device"] = dict(ms=round(copy_ms, 4), bytes=elems * 4,
                                                           roofline=roofline("hbm", elems * 4 / copy_ms / 1e6, HBM_PEAK_GBS, "GB/s"))

    # The headline certifies itself: outside the timed region, the bytes the timed launches left in `packed` and the
    # floats in `back` are compared bit for bit with the CPU oracle on the first and the last 32-row band of the tensor.
    import numpy as np

    import oracle as O

    band_bytes = (shape[3] // 32) * capi.tile_bytes(F.Bfp8_b)
    for w_i, r0 in ((0, 0), (shape[0] - 1, shape[2] - 32)):
        rows = x[w_i:w_i + 1, :, r0:r0 + 32].view(torch.int16).cpu().numpy().view(np.uint16)
        want = O.tilize_pack(rows, O.Bfp8_b)
        first = (w_i * (shape[2] // 32) + r0 // 32) * band_bytes
        assert np.array_equal(packed[first:first + band_bytes].cpu().numpy(), want.reshape(-1)), "bench.py: packed bytes differ from the oracle"
        want_back = O.unpack_untilize(want, O.Bfp8_b, (1, 1, 32, shape[3]), O.Float16_b)
        got_back = back[w_i:w_i + 1, :, r0:r0 + 32].view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(got_back, want_back), "bench.py: round-trip values differ from the oracle"

    # other source/destination pairs of the same kernels (secondary lines): fp32 [4,1,8192,8192], 1 GiB like the bf16 tensor
    x32 = torch.randn(4, 1, 8192, 8192, device=dev) if not args.gemm_only else None
    for fmt, name in (((F.Bfp8_b, "bfp8b"), (F.Bfp4_b, "bfp4b"), (F.Bfp2_b, "bfp2b")) if not args.gemm_only else ()):
        pk = torch.empty(capi.packed_size(fmt, x32.shape), dtype=torch.uint8, device=dev)
        bk = torch.empty_like(x32)
        b = x32.numel() * 4 + pk.numel()
        ms, _ = time_kernel(lambda: capi.tilize_pack(x32, fmt, out=pk), args.steps, args.warmup, torch)
        kernels[f"tilize_pack_fp32_to_{name}"] = dict(ms=round(ms, 4), bytes=b,
                                                      roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        ms, _ = time_kernel(lambda: capi.unpack_untilize(pk, fmt, x32.shape, out=bk), args.steps, args.warmup, torch)
        kernels[f"unpack_untilize_{name}_to_fp32"] = dict(ms=round(ms, 4), bytes=b,
                                                          roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
    x32 = pk = bk = None

    # the same workload laid into the buffers of a queue: an 8 x 8 grid of 16 x 8 micro blocks of 2 x 4 tiles,
    # column-major micro-block order, without and with the 32-byte header + padding per tile
    for header, name in (((0, "queue_g8x8_u2x4_c"), (1, "queue_g8x8_u2x4_c_headers")) if not args.gemm_only else ()):
        lay = capi.QueueLayout(8, 8, 16, 8, 2, 4, 1, header)
        qbytes = capi.queue_buffer_bytes(F.Bfp8_b, shape, lay) * 64
        qmem = torch.empty(qbytes, dtype=torch.uint8, device=dev)
        b = elems * 2 + qbytes
        ms, _ = time_kernel(lambda: capi.tilize_pack_queue(x, F.Bfp8_b, lay, out=qmem), args.steps, args.warmup, torch)
        kernels[f"tilize_pack_bf16_to_bfp8b_{name}"] = dict(ms=round(ms, 4), bytes=b,
                                                            roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        ms, _ = time_kernel(lambda: capi.unpack_untilize_queue(qmem, F.Bfp8_b, shape, lay, out=back), args.steps, args.warmup, torch)
        kernels[f"unpack_untilize_bfp8b_{name}_to_bf16"] = dict(ms=round(ms, 4), bytes=b,
                                                                roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        del qmem

    # the general kernels (any strides and alignments, one thread per face row) and the padding / narrowing forms of the row
    # kernels, on a 256 MiB fp32 tensor: a source whose element stride is 8 bytes (every other column of a wider tensor), and
    # a ragged [.., 8190, 8168] view packed with zero padding and read back narrowed
    if not args.gemm_only:
        wide = torch.randn(1, 1, 8192, 16384, device=dev)
        strided = wide[:, :, :, ::2]
        pk = torch.empty(capi.packed_size(F.Bfp8_b, strided.shape), dtype=torch.uint8, device=dev)
        b = strided.numel() * 4 + pk.numel()
        ms, _ = time_kernel(lambda: capi.tilize_pack(strided, F.Bfp8_b, out=pk), args.steps, args.warmup, torch)
        kernels["tilize_pack_fp32_to_bfp8b_general_strided_source"] = dict(ms=round(ms, 4), bytes=b, roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        ms, _ = time_kernel(lambda: capi.unpack_untilize(pk, F.Bfp8_b, strided.shape, out=strided), args.steps, args.warmup, torch)
        kernels["unpack_untilize_bfp8b_to_fp32_general_strided_result"] = dict(ms=round(ms, 4), bytes=b, roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        ragged = wide[:, :, :8190, :8168]
        b = ragged.numel() * 4 + pk.numel()
        ms, _ = time_kernel(lambda: capi.tilize_pack_padded(ragged, F.Bfp8_b, out=pk), args.steps, args.warmup, torch)
        kernels["tilize_pack_fp32_to_bfp8b_padded_8190x8168"] = dict(ms=round(ms, 4), bytes=b, roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        ms, _ = time_kernel(lambda: capi.unpack_untilize_narrow(pk, F.Bfp8_b, ragged.shape, out=ragged), args.steps, args.warmup, torch)
        kernels["unpack_untilize_bfp8b_to_fp32_narrowed_8190x8168"] = dict(ms=round(ms, 4), bytes=b, roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        del strided, ragged, pk
        # a sliced view with unit element stride whose first element is one element off a 16-byte boundary
        # (pybuda/pybuda/tensor.py:707-717): the row kernels with 16-byte accesses that start anywhere
        view = wide[:, :, :, 1:8161]
        pk = torch.empty(capi.packed_size(F.Bfp8_b, view.shape), dtype=torch.uint8, device=dev)
        b = view.numel() * 4 + pk.numel()
        ms, _ = time_kernel(lambda: capi.tilize_pack(view, F.Bfp8_b, out=pk), args.steps, args.warmup, torch)
        kernels["tilize_pack_fp32_to_bfp8b_view_off_by_one_element_8192x8160"] = dict(ms=round(ms, 4), bytes=b, roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        ms, _ = time_kernel(lambda: capi.unpack_untilize(pk, F.Bfp8_b, view.shape, out=view), args.steps, args.warmup, torch)
        kernels["unpack_untilize_bfp8b_to_fp32_view_off_by_one_element_8192x8160"] = dict(ms=round(ms, 4), bytes=b, roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        del wide, view, pk
        xv = x[:, :, :8160, 1:8161]  # the same on the bf16 workload tensor (its own row count: its launches stay apart from the workload's in a trace)
        pkv = torch.empty(capi.packed_size(F.Bfp8_b, xv.shape), dtype=torch.uint8, device=dev)
        b = xv.numel() * 2 + pkv.numel()
        ms, _ = time_kernel(lambda: capi.tilize_pack(xv, F.Bfp8_b, out=pkv), args.steps, args.warmup, torch)
        kernels["tilize_pack_bf16_to_bfp8b_view_off_by_one_element_8x8160x8160"] = dict(ms=round(ms, 4), bytes=b, roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        backv = back[:, :, :8160, 1:8161]
        ms, _ = time_kernel(lambda: capi.unpack_untilize(pkv, F.Bfp8_b, xv.shape, out=backv), args.steps, args.warmup, torch)
        kernels["unpack_untilize_bfp8b_to_bf16_view_off_by_one_element_8x8160x8160"] = dict(ms=round(ms, 4), bytes=b, roofline=roofline("hbm", b / ms / 1e6, HBM_PEAK_GBS, "GB/s"))
        del xv, pkv, backv

    # ---- Bfp8_b-weight GEMM and the FFN block --------------------------------------------------------
    gemm = {}
    if not args.no_gemm:
        def pack_weight(K, N, seed):
            gg = torch.Generator(device=dev).manual_seed(seed)
            w = torch.randn(1, 1, K, N, generator=gg, device=dev) * 0.02
            return capi.tilize_pack(w, F.Bfp8_b)

        ROTATE = 20  # distinct packed weights of a decode-like line: 20 x 17.8 MB = 357 MB, more than L2 and the 256 MB last-level cache hold

        def gemm_case(M, N, K, seed, workspace=False, rotate=False):
            wp = pack_weight(K, N, seed)
            gg = torch.Generator(device=dev).manual_seed(seed + 1)
            a = torch.randn(M, K, generator=gg, device=dev).bfloat16()
            y = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            # with a workspace the call converts W to a bf16 panel first (many rows) or splits K over more workgroups (few
            # macro tiles); both passes are inside the timed call
            ws = torch.empty(capi.gemm_workspace_bytes(M, N, K), dtype=torch.uint8, device=dev) if workspace else None
            ms, mn = time_kernel(lambda: capi.gemm_bfp8b(a, wp, N, out=y, workspace=ws), args.steps, args.warmup, torch)
            timing, eager_ms = "events around each eager launch", None
            if ms < 0.15 and not args.eager_timing:  # shorter than a few host launch paths: the eager figure is the host's, not the kernel's
                gms = time_launches(lambda: capi.gemm_bfp8b(a, wp, N, out=y, workspace=ws), args.steps, args.warmup, torch)
                if gms is not None:
                    timing, eager_ms, ms = "%d launches back to back in one HIP graph, events around the replay" % args.steps, ms, gms
            flops = 2.0 * M * N * K
            min_bytes = 1.0625 * K * N + 2 * M * K + 2 * M * N
            out = dict(M=M, N=N, K=K)
            if rotate:
                # A weight-streaming line timed on ONE weight measures the caches: an XCD's share of 17.8 MB fits its L2 and the
                # whole weight fits the last-level cache.  Decode streams a different weight per layer, so the line's figure is
                # taken over ROTATE distinct weights, launch i on weight i mod ROTATE; the one-weight figure stays beside it.
                out["cache_resident_ms"] = round(ms, 4)
                out["cache_resident_note"] = "the same launches on one weight, which stays in L2 and the last-level cache between them"
                wps = [wp] + [pack_weight(K, N, seed + 100 + i) for i in range(ROTATE - 1)]
                turn = [0]

                def rotating():
                    capi.gemm_bfp8b(a, wps[turn[0] % ROTATE], N, out=y)
                    turn[0] += 1

                steps_r = max(args.steps, ROTATE)
                rms, mn = time_kernel(rotating, steps_r, args.warmup, torch)
                timing = "events around %d eager launches over %d distinct weights" % (steps_r, ROTATE)
                if not args.eager_timing:
                    turn[0] = 0
                    gms = time_launches(rotating, steps_r, ROTATE, torch)
                    if gms is not None:
                        timing, eager_ms, rms = "%d launches over %d distinct weights back to back in one HIP graph, events around the replay" % (steps_r, ROTATE), rms, gms
                ms = rms
                del wps
            tf = flops / (ms * 1e-3) / 1e12
            out.update(ms=round(ms, 4), min_ms=round(mn, 4), tflops=round(tf, 2), timing=timing)
            if eager_ms is not None:
                out["eager_ms"] = round(eager_ms, 4)
            key = ("gemm_8192" if M == N == K == 8192 else "gemm_M%d" % M if N == K == 4096 else "") + ("_ws" if workspace else "")
            traffic = MEASURED_TRAFFIC_BYTES.get(key)
            # which roof bounds the shape: flops per minimum byte against the ridge of the two peaks (2500 TFLOP/s over 8 TB/s =
            # 312 flop/B).  At N = K = 4096: M = 32 57, 64 113, 128 216 flop/B (HBM bound, the weight streams once), 512 656.
            out["flop_per_byte"] = round(flops / min_bytes, 1)
            if flops / min_bytes < MFMA_BF16_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9):
                out["roofline"] = roofline("hbm", min_bytes / (ms * 1e-3) / 1e9, HBM_PEAK_GBS, "GB/s", traffic)
            else:
                out["roofline"] = roofline("mfma", tf, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s", traffic)
            if M == N == K == 8192 and args.sustained_seconds > 0:
                # the same launch back to back for a couple of seconds with the XCD clock and the socket power sampled
                # meanwhile: what the part sustains once it sits at its power limit, and the share of the matrix cores'
                # peak at the clock it actually ran at
                out["sustained"] = sustained(lambda: capi.gemm_bfp8b(a, wp, N, out=y, workspace=ws), args.sustained_seconds, flops, torch)
            return out

        def vendor_case(M, N, K, seed):
            """Yardstick, not this library: the vendor library's plain bf16 GEMM (torch.matmul) on the same shape, nothing to dequantize."""
            gg = torch.Generator(device=dev).manual_seed(seed)
            va = torch.randn(M, K, generator=gg, device=dev).bfloat16()
            vb = (torch.randn(K, N, generator=gg, device=dev) * 0.02).bfloat16()
            vy = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            vms, vmn = time_kernel(lambda: torch.matmul(va, vb, out=vy), args.steps, args.warmup, torch)
            timing = "events around each eager launch"
            if vms < 0.15 and not args.eager_timing:
                gms = time_launches(lambda: torch.matmul(va, vb, out=vy), args.steps, args.warmup, torch)
                if gms is not None:
                    timing, vms = "%d launches back to back in one HIP graph, events around the replay" % args.steps, gms
            vtf = 2.0 * M * N * K / vms / 1e9
            out = dict(M=M, N=N, K=K, ms=round(vms, 4), min_ms=round(vmn, 4), tflops=round(vtf, 2), timing=timing,
                       roofline=roofline("mfma", vtf, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s"))
            if M == N == K == 8192 and args.sustained_seconds > 0:
                out["sustained"] = sustained(lambda: torch.matmul(va, vb, out=vy), args.sustained_seconds, 2.0 * M * N * K, torch)
            return out

        gemm["north_star_8192"] = gemm_case(8192, 8192, 8192, 30)
        gemm["north_star_8192_with_workspace"] = gemm_case(8192, 8192, 8192, 30, workspace=True)
        gemm["reference_vendor_plain_bf16_gemm_8192"] = vendor_case(8192, 8192, 8192, 31)
        gemm["config4_M32"] = gemm_case(32, 4096, 4096, 3, rotate=True)
        for M in (512, 8192):
            gemm[f"config4_M{M}"] = gemm_case(M, 4096, 4096, 3)
        gemm["reference_vendor_plain_bf16_gemm_M512"] = vendor_case(512, 4096, 4096, 32)
        gemm["config4_M8192_with_workspace"] = gemm_case(8192, 4096, 4096, 3, workspace=True)
        # few macro tiles: with a workspace K is split over more workgroups (M = 512 no longer qualifies: its fused form is level)
        gemm["weights4096_M256"] = gemm_case(256, 4096, 4096, 3)
        gemm["weights4096_M256_with_workspace"] = gemm_case(256, 4096, 4096, 3, workspace=True)
        for M in (64, 128):  # between the decode-like and the prefill-like case of config 4
            gemm[f"weights4096_M{M}"] = gemm_case(M, 4096, 4096, 3, rotate=True)

        # tensors are padded to multiples of 32, not of 64 (pybuda/pybuda/tensor.py:805-877): N an odd number of tiles (all but the
        # last tile column in the macro-tiled kernel, the last one in one-row-tile workgroups of the weight-streaming kernel),
        # K an odd number of tile rows (half a slab after the loop), both
        gemm["ragged_M512_N4128"] = gemm_case(512, 4128, 4096, 3)
        gemm["ragged_M512_K4128"] = gemm_case(512, 4096, 4128, 3)
        gemm["ragged_M8192_N4128_K4128"] = gemm_case(8192, 4128, 4128, 3)

        # BERT-large FFN: X [3072,1024]; W1 [1024,4096], W2 [4096,1024]
        w1, w2 = pack_weight(1024, 4096, 51), pack_weight(4096, 1024, 52)
        gg = torch.Generator(device=dev).manual_seed(5)
        xa = torch.randn(3072, 1024, generator=gg, device=dev).bfloat16()
        b1 = (torch.randn(4096, generator=gg, device=dev) * 0.02).bfloat16()
        b2 = (torch.randn(1024, generator=gg, device=dev) * 0.02).bfloat16()
        h = torch.empty(3072, 4096, dtype=torch.bfloat16, device=dev)
        y = torch.empty(3072, 1024, dtype=torch.bfloat16, device=dev)

        def ffn():
            capi.gemm_bfp8b(xa, w1, 4096, bias=b1, epilogue=capi.EPILOGUE_GELU, out=h)
            capi.gemm_bfp8b(h, w2, 1024, bias=b2, out=y)

        ms, mn = time_kernel(ffn, args.steps, args.warmup, torch)
        ms = (None if args.eager_timing else time_launches(ffn, args.steps, args.warmup, torch)) or ms
        flops = 2.0 * 3072 * 1024 * 4096 * 2
        tf = flops / (ms * 1e-3) / 1e12
        gemm["config5_bert_large_ffn"] = dict(ms=round(ms, 4), min_ms=round(mn, 4), tflops=round(tf, 2),
                                              roofline=roofline("mfma", tf, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s", MEASURED_TRAFFIC_BYTES["ffn"]))
        del w1, w2, xa, h, y
        # the vendor library's plain bf16 GEMM on the FFN's two matmuls (no bias, no GELU, nothing to dequantize)
        gemm["reference_vendor_plain_bf16_gemm_ffn1"] = vendor_case(3072, 4096, 1024, 53)
        gemm["reference_vendor_plain_bf16_gemm_ffn2"] = vendor_case(3072, 1024, 4096, 54)
        vsum = gemm["reference_vendor_plain_bf16_gemm_ffn1"]["ms"] + gemm["reference_vendor_plain_bf16_gemm_ffn2"]["ms"]
        gemm["reference_vendor_plain_bf16_gemm_ffn_sum"] = dict(ms=round(vsum, 4), tflops=round(flops / vsum / 1e9, 2),
                                                                note="sum of the two matmul lines above, each timed alone")

    host_push = None
    if not args.no_host_push:
        torch.cuda.synchronize()
        host_push = host_push_lines(torch)

    # ---- CPU baseline: the oracle on a bounded sample of the same workload ---------------------------
    cpu_baseline = None
    if not args.no_cpu_baseline:
        cores = max(1, min(16, os.cpu_count() or 1))
        sample_shape = (1, 1, 8192, 8192)  # one eighth of the workload
        xs = x[0:1].cpu().view(torch.int16).numpy().view(np.uint16)
        O.tilize_pack(xs[:, :, :64], O.Bfp8_b)  # load the library outside the timed region
        # repeat the sample until about 8 s (all cores) and 4 s (one thread) of wall time have gone by
        sample_bytes = (bytes_pack + bytes_unpack) / 8
        reps, t0 = 0, time.perf_counter()
        while True:
            ps = O.tilize_pack(xs, O.Bfp8_b, nthreads=cores)
            O.unpack_untilize(ps, O.Bfp8_b, sample_shape, O.Float16_b, nthreads=cores)
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= 8.0:
                break
        small = xs[:, :, :1024]
        reps1, t1 = 0, time.perf_counter()
        while True:
            p1 = O.tilize_pack(small, O.Bfp8_b, nthreads=1)
            O.unpack_untilize(p1, O.Bfp8_b, small.shape, O.Float16_b, nthreads=1)
            reps1 += 1
            dt1 = time.perf_counter() - t1
            if dt1 >= 4.0:
                break
        cpu_baseline = {
            "value": round(sample_bytes * reps / dt / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "bf16 [1,1,8192,8192] slice (1/8 of the workload) x %d passes in %.1f s: oracle tilize+pack to "
                      "Bfp8_b then unpack+untilize to bf16, OpenMP over tile rows" % (reps, dt),
            "single_thread_value": round(sample_bytes / 8 * reps1 / dt1 / 1e9, 3),
            "single_thread_sample": "bf16 [1,1,1024,8192] slice x %d passes in %.1f s, 1 thread" % (reps1, dt1),
        }
        if not args.no_gemm:
            # dequantize-then-fp32-matmul on the host cores (the golden evaluation) on config 4's seeded weight and activations,
            # M = 512: the dequantization timed once, the matmul warmed and then timed apart from it
            torch.set_num_threads(cores)
            w4 = torch.randn(4096, 4096, generator=torch.Generator().manual_seed(3)) * 0.02
            wq = O.tilize_pack(w4.view(1, 1, 4096, 4096).numpy(), O.Bfp8_b, nthreads=cores)
            a = torch.randn(512, 4096, generator=torch.Generator().manual_seed(4)).bfloat16().float()
            t2 = time.perf_counter()
            wd = torch.from_numpy(O.dequant_weight(wq, 4096, 4096))
            dt_dequant = time.perf_counter() - t2
            for _ in range(2):
                _ = a @ wd
            reps2, t3 = 0, time.perf_counter()
            while True:
                _ = a @ wd
                reps2 += 1
                dt2 = time.perf_counter() - t3
                if dt2 >= 3.0:
                    break
            cpu_baseline["gemm"] = {"value": round(2.0 * 512 * 4096 * 4096 * reps2 / dt2 / 1e12, 4), "unit": "TFLOP/s",
                                    "cores": cores, "kind": "port",
                                    "sample": "M=512, K=N=4096, config 4's weight (seed 3) and activations (seed 4): torch fp32 matmul on "
                                              "the oracle-dequantized weight, %d warmed passes in %.1f s" % (reps2, dt2),
                                    "dequantize_ms": round(dt_dequant * 1e3, 2),
                                    "value_with_dequantize_each_call": round(2.0 * 512 * 4096 * 4096 / (dt2 / reps2 + dt_dequant) / 1e12, 4)}

    line = {
        "metric": "Bfp8_b pack/unpack GB/s (% HBM peak); Bfp8_b-weight GEMM TFLOP/s (% MFMA peak)",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 <-> Bfp8_b (integer arithmetic on the 16-bit patterns; GEMM lines: bf16 x bf16 MFMA, fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": "streaming: bf16 [8,1,8192,8192] U(-8,8) seed 2 -> tilize+pack Bfp8_b -> "
                               "unpack+untilize bf16; one step = both kernels",
                   "algorithmic_bytes_per_step": bytes_pack + bytes_unpack},
        "roofline": dict(kernels[dominant]["roofline"], kernel=dominant),
        "traffic_source": TRAFFIC_SOURCE,
        "cpu_baseline": cpu_baseline,
        "kernels": kernels,
        "gemm": gemm,
        "host_push": host_push,
        "gemm_tflops_8192": gemm.get("north_star_8192", {}).get("tflops"),
        "gemm_frac_of_mfma_peak_8192": gemm.get("north_star_8192", {}).get("roofline", {}).get("frac"),
        "gemm_tflops_8192_with_workspace": gemm.get("north_star_8192_with_workspace", {}).get("tflops"),
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
