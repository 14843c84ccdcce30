#!/usr/bin/env python3
"""Headline benchmark: bs=1 2-bit decompress-matvec over the Llama-2-70B layer shapes.

One "step" = one pass of the decompress-matvec kernel over the four 70B-shaped
matrices (fused qkv 10240x8192, o_proj 8192x8192, fused up/gate 57344x8192,
down 8192x28672; 2-bit HYB code, 214 MB of packed weights), inputs resident in
HBM.  Successive steps walk through several distinct copies of the packed
weights (>= 600 MB in total) so that the 256 MB last-level cache cannot serve
them; the steps are recorded in one HIP graph so that host launch overhead
does not dilute the device time.

Prints ONE JSON line:  value = packed bytes streamed per second (GB/s), plus
  roofline      HBM roofline of the matvec kernel, measured in this run
  cpu_baseline  the reference's CPU path (torch decode + matmul, restated in
                oracle/torch_cpu_path.py) on a bounded sample, same host
  shapes        per-matrix kernel time / GB/s / fraction of 8 TB/s
  layer         whole BitshiftLinear.forward (RHT-in + matvec + RHT-out) per matrix
  gemm_4bit     batched decompress-GEMM (batch 8/16/32) time, stream GB/s, TFLOP/s
  decode_dense  packed -> dense fp16 weights: time, GB/s written, (read + written) / 8 TB/s
  measured_ceilings  copy / fill / sum bandwidth of this box (library kernels) beside the nominal peak
  e2e_decode    greedy decode tok/s of a random-init 7B-architecture 2-bit model
  sets          the other matvec sets: Llama-2-7B shapes at 2 / 3 / 4 bits, 70B shapes at 3 / 4 bits
                (set GB/s and per-matrix times, cold weights)
  single_layer  one 4096x4096 2-bit BitshiftLinear: kernel and whole forward, cold and cache-resident
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, each calibrated
# against a 256 MiB copy) are read from this summary, which names the kernel sources it was taken on
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "matvec_k2_llama70b_set_traffic.txt")
KERNEL_SOURCES = ("qtip_amd/csrc/qtip_hip.hip", "qtip_amd/csrc/qtip_device.h", "qtip_amd/csrc/qtip_wht.h")


def kernel_source_digest():
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload, bits):
    """(bytes per launch or None, note): the counter-measured HBM traffic of the headline kernel, only
    if the committed summary was taken on exactly the kernel sources of this tree."""
    if (workload, bits) != ("70b", 2):
        return None, "no counter profile for this workload"
    try:
        kv = dict(line.split(":", 1) for line in open(TRAFFIC_FILE) if ":" in line and not line.startswith("#"))
        kv = {k.strip(): v.strip() for k, v in kv.items()}
    except OSError:
        return None, "profiles/matvec_k2_llama70b_set_traffic.txt not present where this ran"
    if kv.get("kernel_source_digest") != kernel_source_digest():
        return None, "the committed counter profile was taken on older kernel sources; not carried over"
    return int(kv["traffic_bytes_per_launch"]), "FETCH_SIZE + WRITE_SIZE per launch, rocprofv3 --pmc, see " + \
        os.path.relpath(TRAFFIC_FILE, ROOT)


def timeline(shapes, ms_per_step, chained=False):
    """In-kernel readings of the 100 MHz constant clock kept by the timeline build (see QTIP_STAMPS in
    qtip_amd/csrc/qtip_hip.hip): after the timed graph replay the buffer holds, per shape, the last
    launch of that shape - i.e. the last step.  All figures in microseconds (10 ns resolution)."""
    import ctypes
    import numpy as np
    from qtip_amd import _lib
    L = _lib.lib()
    if not hasattr(L, "qtip_debug_stamps"):
        raise RuntimeError("--timeline needs the library built with -DQTIP_STAMPS (python -m bench_probe)")
    buf = np.zeros(64 * 256 * 16, dtype=np.uint64)
    L.qtip_debug_stamps.argtypes = [ctypes.c_void_p]
    rc = L.qtip_debug_stamps(buf.ctypes.data)
    if rc != 0:
        raise RuntimeError(f"qtip_debug_stamps failed ({rc})")
    st = buf.reshape(64, 256, 16).astype(np.int64)
    us = lambda ticks: round(float(ticks) / 100.0, 2)
    fml = lambda a: [us(a.min()), us(np.median(a)), us(a.max())]
    rows, ends, prev_end = {}, [], None
    for name, m, k in shapes:
        s = st[((m ^ k) >> 10) & 63]
        s = s[s[:, 0] > 0]
        t0 = s[:, 0].min()
        row = {"workgroups": int(len(s)),
               "previous_launch_last_end_to_first_start": us(t0 - prev_end) if prev_end is not None else None,
               "workgroup_starts_first_median_last": fml(s[:, 0] - t0),
               "wave15_start_after_wave0": fml(s[:, 5] - s[:, 0]),
               "start_to_table_words_picked": fml(s[:, 1] - s[:, 0]),
               "start_to_first_barrier_reached": fml(s[:, 2] - s[:, 0]),
               "start_to_first_barrier_passed": fml(s[:, 3] - s[:, 0]),
               "start_to_first_weights_in_registers": fml(s[:, 15] - s[:, 0]),
               "workgroup_ends_first_median_last_from_first_start": fml(s[:, 4] - t0),
               "span_first_start_to_last_end": us(s[:, 4].max() - t0)}
        if chained and (s[:, 10] > 0).all():
            # the transform / layer boundary in the prologue (wave 0): entered, past its three barriers, left
            row["prologue_transform_entered_barriers_left"] = [fml(s[:, i] - s[:, 0])[1] for i in (6, 7, 8, 9, 10)
                                                               if (s[:, i] > 0).all()]
        if chained:
            row["previous_launch_last_end_to_first_start"] = None  # other kernels run between these launches
        prev_end = s[:, 4].max()
        ends.append((t0, prev_end))
        rows[name] = row
    spans = sum(e - b for b, e in ends)
    if chained:
        return {"clock": "s_memrealtime, 100 MHz", "matvec_launches_of_the_last_layer": rows,
                "sum_of_spans_us": us(spans), "first_start_to_last_end_us": us(ends[-1][1] - ends[0][0])}
    return {"clock": "s_memrealtime, 100 MHz", "launches_of_the_last_step": rows,
            "sum_of_spans_us": us(spans), "first_start_to_last_end_us": us(ends[-1][1] - ends[0][0]),
            "ms_per_step_of_this_run": round(ms_per_step, 5)}


SHAPES_70B = [("qkv", 10240, 8192), ("o", 8192, 8192), ("up_gate", 57344, 8192), ("down", 8192, 28672)]
SHAPES_7B = [("qkv", 12288, 4096), ("o", 4096, 4096), ("up_gate", 22016, 4096), ("down", 4096, 11008)]


def _distinct(toks, new):
    """Distinct values among the `new` decoded tokens: 1 would mean a loop that decodes non-finite
    logits (argmax of NaN is token 0 every time)."""
    return int(toks.reshape(-1)[-new:].unique().numel())


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--settle-ms", type=float, default=60.0,
                    help="untimed replays of the timed graph before the timed one, until this much GPU time has "
                         "passed (the sustained clocks need tens of ms of continuous work); 0 = none")
    ap.add_argument("--bits", type=int, default=2)
    ap.add_argument("--workload", choices=["70b", "7b"], default="70b")
    ap.add_argument("--shape", default=None,
                    help="restrict the set to one of its matrices (qkv, o, up_gate, down): used for per-kernel "
                         "counter runs under rocprofv3")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip per-shape / layer / GEMM / end-to-end timings")
    ap.add_argument("--extras", default="shapes,layer,sets,single,gemm,decode,ceilings,e2e",
                    help="comma-separated subset of the extra sections to run: shapes, layer, sets, single, gemm, decode, "
                         "ceilings, e2e, e2e13b, e2e70b (counter runs under rocprofv3 pick one)")
    ap.add_argument("--print-kernel-source-digest", action="store_true",
                    help="print the digest that profiles/matvec_k2_llama70b_set_traffic.txt must name, and exit")
    ap.add_argument("--timeline", action="store_true",
                    help="run on the timeline build of the library (bench_probe/libqtip_hip_stamped.so: the product "
                         "sources compiled with -DQTIP_STAMPS, `python -m bench_probe`) and add the in-kernel clock "
                         "readings of the last timed step to the line: per launch, previous end -> first start, "
                         "start -> first barrier, first / median / last workgroup end")
    ap.add_argument("--calibrate-probe", action="store_true",
                    help="also time 64 launches of the stream-read probe on a fixed 64 MiB buffer in one graph (a kernel "
                         "of known duration: run once plain and once under rocprofv3 --kernel-trace, the difference "
                         "between the trace's mean for it and the plain figure is what the profiler adds per launch)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy kernel (reference point for rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE runs)")
    args = ap.parse_args()
    if args.print_kernel_source_digest:
        print(kernel_source_digest())
        return
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (--gpus 1); no multi-GPU figure is produced",
              file=sys.stderr)
        sys.exit(2)

    if args.timeline:
        import bench_probe
        os.environ["QTIP_HIP_LIBRARY"] = bench_probe.STAMPED_LIB_PATH
    import torch
    from qtip_amd import ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    K = args.bits
    shapes = SHAPES_70B if args.workload == "70b" else SHAPES_7B
    if args.shape is not None:
        shapes = [sh for sh in shapes if sh[0] == args.shape]
        if not shapes:
            ap.error(f"unknown --shape {args.shape}")
    set_bytes = sum(m * k * K // 8 for _, m, k in shapes)
    copies = max(2, -(-(600 << 20) // set_bytes))

    g = torch.Generator().manual_seed(0)
    tlut = torch.randn(512, 2, generator=g).half().to(dev)
    packed, xs, outs = {}, {}, {}
    for name, m, k in shapes:
        base = torch.randint(-32768, 32768, (m * k * K // 16,), dtype=torch.int16, generator=g)
        packed[name] = [base.to(dev)]
        for c in range(1, copies):
            packed[name].append(torch.roll(packed[name][0], 4099 * c))  # distinct contents, same statistics
        xs[name] = torch.randn(k, generator=g).half().to(dev)
        outs[name] = torch.empty(m, dtype=torch.float32, device=dev)

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)  # one elementwise copy kernel: 256 MiB read + 256 MiB written
        torch.cuda.synchronize()
        del src, dst

    def step(i):
        c = i % copies
        for name, m, k in shapes:
            ops.decompress_matvec(packed[name][c], xs[name], tlut, m, k, K, out=outs[name])

    def capture(fn):
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            fn()
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            fn()
        return gr

    def timed(gr, reps=1, settle_ms=0.0):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if settle_ms > 0:  # untimed replays first, see --settle-ms
            one = timed(gr)
            for _ in range(min(1000, int(settle_ms * 1e-3 / max(one, 1e-6)))):
                gr.replay()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            gr.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / reps

    # ---- headline: exactly `steps` steps in the timed region --------------
    # the warm-up steps run in the same form as the timed ones (one graph) and directly before
    # them: after the host-side pause of a graph capture the GPU needs a few milliseconds of work
    # to be back at its running clocks, and a short timed region would measure that ramp
    graph = capture(lambda: [step(i) for i in range(args.steps)])
    warm = capture(lambda: [step(i) for i in range(args.warmup)]) if args.warmup > 0 else None
    torch.cuda.synchronize()
    if warm is not None:
        warm.replay()
    # clock settling: the chip reaches its sustained clocks only after tens of milliseconds of
    # continuous work (a 3 ms timed region reads 10-15 % slower than a 40 ms one), so the timed
    # graph is replayed untimed until `settle_ms` of GPU time have passed, then timed once
    before_settling = None
    if args.settle_ms > 0:
        torch.cuda.synchronize()
        one = timed(graph)
        before_settling = one * 1e3 / args.steps
        for _ in range(min(1000, int(args.settle_ms * 1e-3 / max(one, 1e-6)))):
            graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dev_s = timed(graph)
    wall_s = time.perf_counter() - t0
    ms_per_step = dev_s * 1e3 / args.steps
    value = set_bytes / (dev_s / args.steps) / 1e9
    launches = args.steps * len(shapes)
    avg_launch_us = dev_s * 1e6 / launches
    achieved = (set_bytes / len(shapes)) / (avg_launch_us * 1e-6) / 1e9

    traffic, traffic_note = measured_traffic(args.workload, K)
    result = {
        "metric": "bs=1 2-bit decompress-matvec compressed-stream throughput, Llama-2-70B layer shapes",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u16 trellis states -> f16 weights, f32 accumulate",
        "data": "synthetic (seeded uniform bitstream, N(0,1) fp16 LUT and x)",
        "config": {
            "workload": ("Llama-2-70B" if args.workload == "70b" else "Llama-2-7B") +
                        f"-shaped matvec set, bs=1, {K}-bit HYB (L=16,Q=9,V=2): " +
                        ", ".join(f"{n} {m}x{k}" for n, m, k in shapes),
            "bytes_per_step": set_bytes,
            "weight_copies_rotated": copies,
            "timing": "one HIP graph holding all timed steps, HIP events on the launch stream",
            "clock_settle_ms": args.settle_ms,
            "ms_per_step_before_settling": round(before_settling, 5) if before_settling is not None else None,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": f"matvec_kernel<{K}>",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "avg_launch_us": round(avg_launch_us, 3),
            "bytes_per_launch": set_bytes // len(shapes),
            "traffic": traffic if args.shape is None else None,
            "traffic_note": traffic_note,
        },
        "host_wall_s_timed_region": round(wall_s, 4),
    }

    if args.timeline:
        result["timeline"] = timeline(shapes, ms_per_step)
    if args.calibrate_probe:
        import bench_probe
        psrc = torch.empty(64 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        gr = capture(lambda: [bench_probe.stream_read(psrc) for _ in range(64)])
        result["probe_calibration"] = {"kernel": "stream_read_probe_kernel", "bytes": psrc.numel(), "launches": 64,
                                       "us_per_launch": round(timed(gr, 3, args.settle_ms / 3) * 1e6 / 64, 3)}
        del gr, psrc

    # ---- per-shape kernel times and whole-layer times ---------------------
    extras = set() if args.no_extras else set(args.extras.split(","))
    if extras & {"shapes", "layer"}:
        from qtip_amd.codebook.bitshift import BitshiftLinear
        from qtip_amd.utils import matmul_had as mh
        per, layer = {}, {}
        for name, m, k in shapes:
            nbytes = m * k * K // 8
            # enough distinct copies of this one matrix to cycle through more than twice the 256 MB
            # last-level cache, so that every launch streams from HBM
            ncp = max(copies, -(-(600 << 20) // nbytes))
            pks = packed[name] + [torch.roll(packed[name][0], 4099 * c) for c in range(copies, ncp)]
            reps = ncp * max(1, 24 // ncp)
            gr = capture(lambda: [ops.decompress_matvec(pks[i % ncp], xs[name], tlut, m, k, K,
                                                       out=outs[name]) for i in range(reps)])
            us = timed(gr, 3, args.settle_ms / 3) * 1e6 / reps
            per[name] = {"m": m, "k": k, "us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                         "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
            del gr
            mod = BitshiftLinear(16, 16, 16, K, 2, 9, "quantlut_sym", tlut=tlut, has_kernel=True)
            hl, Kl = mh.get_hadK(k)
            hr, Kr = mh.get_hadK(m)
            SU = torch.sign(torch.randn(k, generator=g) + 1e-5).half().to(dev)
            SV = (torch.sign(torch.randn(m, generator=g) + 1e-5) / k**0.5).float().to(dev)
            inp = torch.randn(1, k, generator=g).half().to(dev)
            gr = capture(lambda: [mod(inp, pks[i % ncp].view(-1, 16 * K), SU, SV, hl, hr, Kl, Kr, 0, 8)
                                  for i in range(reps)])
            lus = timed(gr, 3, args.settle_ms / 3) * 1e6 / reps
            layer[name] = {"us": round(lus, 2), "GBps": round(nbytes / lus / 1e3, 1)}
            del gr, pks
        result["shapes"] = per
        result["layer"] = layer

    def cold_copies(base, nbytes):
        """Enough distinct copies of one matrix to cycle through more than twice the 256 MB last-level
        cache, so that every launch streams from HBM."""
        ncp = max(2, -(-(600 << 20) // nbytes))
        return [base] + [torch.roll(base, 4099 * c) for c in range(1, ncp)]

    if "sets" in extras:
        # the matvec sets the headline does not cover: 7B shapes at every bit width, 70B at 3 and 4 bits
        sets = {}
        for wl, shp, bits_list in (("7b", SHAPES_7B, (2, 3, 4)), ("70b", SHAPES_70B, (3, 4))):
            for kb in bits_list:
                if (wl, kb) == (args.workload, K):
                    continue
                sb = sum(m * k * kb // 8 for _, m, k in shp)
                ncp = max(2, -(-(600 << 20) // sb))
                pk, xv, ov = {}, {}, {}
                for name, m, k in shp:
                    base = torch.randint(-32768, 32768, (m * k * kb // 16,), dtype=torch.int16, generator=g).to(dev)
                    pk[name] = [base] + [torch.roll(base, 4099 * c) for c in range(1, ncp)]
                    xv[name] = torch.randn(k, generator=g).half().to(dev)
                    ov[name] = torch.empty(m, dtype=torch.float32, device=dev)
                nst = max(args.steps, 2 * ncp)
                gr = capture(lambda: [ops.decompress_matvec(pk[name][i % ncp], xv[name], tlut, m, k, kb, out=ov[name])
                                      for i in range(nst) for name, m, k in shp])
                st_s = timed(gr, 1, args.settle_ms) / nst
                del gr
                entry = {"GBps": round(sb / st_s / 1e9, 1), "frac_hbm_peak": round(sb / st_s / 1e9 / HBM_PEAK_GBS, 4),
                         "ms_per_step": round(st_s * 1e3, 5), "bytes_per_step": sb, "shapes": {}}
                for name, m, k in shp:
                    nbytes = m * k * kb // 8
                    pks = pk[name] + [torch.roll(pk[name][0], 4099 * c)
                                      for c in range(ncp, max(ncp, -(-(600 << 20) // nbytes)))]
                    reps = len(pks) * max(1, 24 // len(pks))
                    gr = capture(lambda: [ops.decompress_matvec(pks[i % len(pks)], xv[name], tlut, m, k, kb,
                                                               out=ov[name]) for i in range(reps)])
                    us = timed(gr, 3, args.settle_ms / 3) * 1e6 / reps
                    entry["shapes"][name] = {"m": m, "k": k, "us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                                             "frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
                    del gr, pks
                sets[f"{wl}_k{kb}"] = entry
                del pk, xv, ov
                torch.cuda.empty_cache()
        result["sets"] = sets

    if "single" in extras:
        # one BitshiftLinear, 4096 x 4096, 2 bits: the kernel alone and the whole forward (input transform
        # inside the matvec launch + output transform), with cold weights (copies rotated through more than
        # twice the last-level cache) and with one cache-resident copy
        from qtip_amd.codebook.bitshift import BitshiftLinear
        from qtip_amd.utils import matmul_had as mh
        m = k = 4096
        nbytes = m * k * 2 // 8
        base = torch.randint(-32768, 32768, (m * k * 2 // 16,), dtype=torch.int16, generator=g).to(dev)
        pks = cold_copies(base, nbytes)
        xv = torch.randn(k, generator=g).half().to(dev)
        ov = torch.empty(m, dtype=torch.float32, device=dev)
        mod = BitshiftLinear(16, 16, 16, 2, 2, 9, "quantlut_sym", tlut=tlut, has_kernel=True)
        SU = torch.sign(torch.randn(k, generator=g) + 1e-5).half().to(dev)
        SV = (torch.sign(torch.randn(m, generator=g) + 1e-5) / k**0.5).float().to(dev)
        inp = torch.randn(1, k, generator=g).half().to(dev)
        single = {"m": m, "k": k, "bits": 2, "packed_bytes": nbytes, "weight_copies_rotated": len(pks)}
        for label, pool in (("cold", pks), ("warm", pks[:1])):
            reps = max(len(pool), 150)
            gr = capture(lambda: [ops.decompress_matvec(pool[i % len(pool)], xv, tlut, m, k, 2, out=ov)
                                  for i in range(reps)])
            us = timed(gr, 3, args.settle_ms / 3) * 1e6 / reps
            del gr
            gr = capture(lambda: [mod(inp, pool[i % len(pool)].view(-1, 32), SU, SV, None, None, 1, 1, 0, 8)
                                  for i in range(reps)])
            lus = timed(gr, 3, args.settle_ms / 3) * 1e6 / reps
            del gr
            single[label] = {"kernel_us": round(us, 2), "kernel_GBps": round(nbytes / us / 1e3, 1),
                             "kernel_frac_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                             "forward_us": round(lus, 2), "forward_GBps": round(nbytes / lus / 1e3, 1)}
        result["single_layer_4096x4096_k2"] = single
        del pks, base

    if "gemm" in extras:
        # batched decompress-GEMM on the matrix cores: 4-bit weights, batch 8 / 16 / 32
        gemm = {}
        for m, k in ((28672, 8192), (8192, 28672)):
            nbytes = m * k * 4 // 8
            base = torch.randint(-32768, 32768, (m * k * 4 // 16,), dtype=torch.int16, generator=g).to(dev)
            pk4 = [base] + [torch.roll(base, 4099 * c) for c in range(1, 6)]
            for B in (8, 16, 32):
                X = torch.randn(B, k, generator=g).half().to(dev)
                gr = capture(lambda: [ops.decompress_gemm(pk4[i % 6], X, tlut, m, k, 4) for i in range(12)])
                us = timed(gr, 3, args.settle_ms / 3) * 1e6 / 12
                tf = 2.0 * m * k * B / us / 1e6
                gemm[f"{m}x{k}_b{B}"] = {"us": round(us, 2), "stream_GBps": round(nbytes / us / 1e3, 1),
                                         "TFLOPs": round(tf, 1), "frac_mfma_f16_peak": round(tf / 2500.0, 4)}
                del gr
            del pk4, base
        result["gemm_4bit"] = gemm

    if "ceilings" in extras:
        import bench_probe  # libqtip_probe.so: the measurement aids, a library of their own beside this script
        # what the memory system of this box delivers to simple kernels, next to the 8 TB/s nominal peak:
        # a 1 GiB device-to-device copy (read + write), a fill (write only), a BLAS dot product and the library's
        # own read probe (read only; the probe uses the matvec's persistent grid and non-temporal 16-byte loads)
        src = torch.empty(1 << 28, dtype=torch.int32, device=dev).random_(0, 100)
        dst = torch.empty_like(src)
        nb = src.numel() * 4
        fa, fb = src.view(torch.float32)[:1 << 27], src.view(torch.float32)[1 << 27:]  # two 512 MiB operands
        cases = {"copy_read_plus_write": (lambda: dst.copy_(src), 2 * nb),
                 "fill_write": (lambda: dst.fill_(1), nb),
                 "blas_dot_read": (lambda: torch.dot(fa, fb), nb),
                 "stream_read": (lambda: bench_probe.stream_read(src), nb)}
        ceil = {}
        for name, (fn, moved) in cases.items():
            gr = capture(lambda: [fn() for _ in range(4)])
            ceil[name + "_GBps"] = round(moved / (timed(gr, 3, args.settle_ms / 3) / 4) / 1e9, 1)
            del gr
        del src, dst
        # issue rates of the instructions the 2-bit decode consists of, and its loop without memory:
        # ns one wave-instruction (one wave-load) occupies a SIMD with 4 waves per SIMD, as in the matvec
        issue = {}
        iters = 2000
        for name in bench_probe.KINDS:
            gr = capture(lambda: bench_probe.issue(name, iters, tlut))
            t = timed(gr, 3, args.settle_ms / 6)
            per = iters * 4 * (1 if name.startswith("decode_loop") else bench_probe.OPS_PER_ITER)
            issue[name] = round(t * 1e9 / per, 2 if per > iters * 4 else 1)
            del gr
        ceil["issue_ns_per_wave_instruction_and_simd"] = {k: v for k, v in issue.items() if not k.startswith("decode_loop")}
        ceil["decode_loop_ns_per_wave_load_and_simd"] = {
            "loop_without_memory": issue["decode_loop"], "vector_alu_part_alone": issue["decode_loop_valu"]}
        result["measured_ceilings"] = ceil

    if "decode" in extras:
        # packed -> dense fp16 weights (the reference's decode_compressed); bound by the dense write
        dec = {}
        for m, k in ((28672, 8192), (57344, 8192)):
            for bits in (2, 4):
                pkd = torch.randint(-32768, 32768, (m * k * bits // 16,), dtype=torch.int16, generator=g).to(dev)
                ops.decode(pkd, tlut, m, k, bits)
                gr = capture(lambda: [ops.decode(pkd, tlut, m, k, bits) for _ in range(4)])
                us = timed(gr, 3, args.settle_ms / 3) * 1e6 / 4
                dec[f"{m}x{k}_k{bits}"] = {"us": round(us, 1), "written_GBps": round(m * k * 2 / us / 1e3, 1),
                                           "frac_hbm_peak": round((m * k * 2 + m * k * bits // 8) / us / 1e3 / HBM_PEAK_GBS, 4)}
                del gr, pkd
        result["decode_dense"] = dec

    if "e2e" in extras:
        # end-to-end greedy decode, random-init Llama-2-7B architecture, every linear 2-bit
        from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder, generate
        model = LlamaDecoder(LlamaConfig(K=2), max_cache_len=512, device=dev)
        prompt = torch.randint(0, 32000, (1, 128), generator=g).to(dev)
        toks, dt, tps = generate(model, prompt, 256, use_graph=True, fused=True)
        # bytes a decoded token must read: every packed matrix, the fp16 lm_head and the keys / values so far
        tok_bytes = sum(l.trellis.numel() * 2 for l in model.modules() if hasattr(l, "trellis")) + \
            model.lm_head.numel() * 2 + 2 * 32 * (128 + 128) * 4096 * 2
        result["e2e_decode"] = {"model": "Llama-2-7B architecture, random init, 2-bit HYB, fused qkv and up/gate",
                                "prompt": 128, "new_tokens": 256, "tok_per_s": round(tps, 1),
                                "ms_per_token": round(1e3 / tps, 3), "distinct_new_tokens": _distinct(toks, 256),
                                "bytes_per_token": tok_bytes,
                                "frac_hbm": round(tok_bytes * tps / 1e9 / HBM_PEAK_GBS, 4)}
        if args.timeline:
            # the four matvec launches of the last layer of the last decoded token (qkv and up/gate with the
            # layer boundary in their prologue, o with its input transform, down plain)
            result["e2e_decode"]["timeline"] = timeline(SHAPES_7B, 1e3 / tps, chained=True)
        del model
        torch.cuda.empty_cache()
        # the layout of the published checkpoints: seven separate projections per layer (grouped launches)
        model = LlamaDecoder(LlamaConfig(K=2), max_cache_len=512, device=dev, fused=False)
        toks, dt, tps = generate(model, prompt, 256, use_graph=True, fused=True)
        result["e2e_decode_separate_projections"] = {
            "model": "Llama-2-7B architecture, random init, 2-bit HYB, q/k/v/o/gate/up/down separate",
            "prompt": 128, "new_tokens": 256, "tok_per_s": round(tps, 1), "ms_per_token": round(1e3 / tps, 3),
            "distinct_new_tokens": _distinct(toks, 256)}
        del model
        torch.cuda.empty_cache()

    if "e2e70b" in extras:
        # the same loop on the Llama-2-70B architecture (80 layers, GQA 64/8 heads, 17 GB of 2-bit weights);
        # not part of the default run: building the random model takes a minute
        from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder, generate
        cfg70 = LlamaConfig(hidden=8192, heads=64, kv_heads=8, layers=80, ffn=28672, vocab=32000, K=2)
        model = LlamaDecoder(cfg70, max_cache_len=512, device=dev)
        prompt = torch.randint(0, 32000, (1, 128), generator=g).to(dev)
        toks, dt, tps = generate(model, prompt, 128, use_graph=True, fused=True)
        result["e2e_decode_70b"] = {"model": "Llama-2-70B architecture, random init, 2-bit HYB, fused qkv and up/gate",
                                    "prompt": 128, "new_tokens": 128, "tok_per_s": round(tps, 1),
                                    "ms_per_token": round(1e3 / tps, 3), "distinct_new_tokens": _distinct(toks, 128)}
        del model
        torch.cuda.empty_cache()

    if "e2e13b" in extras:
        # a hidden size that is a table order times a power of two (5120 = 40 x 128), separate projections
        from qtip_amd.llama_decode import LlamaConfig, LlamaDecoder, generate
        cfg13 = LlamaConfig(hidden=5120, heads=40, kv_heads=40, layers=40, ffn=13824, vocab=32000, K=2)
        model = LlamaDecoder(cfg13, max_cache_len=512, device=dev, fused=False)
        prompt = torch.randint(0, 32000, (1, 128), generator=g).to(dev)
        toks, dt, tps = generate(model, prompt, 128, use_graph=True, fused=True)
        result["e2e_decode_13b"] = {"model": "Llama-2-13B architecture, random init, 2-bit HYB, separate projections",
                                    "prompt": 128, "new_tokens": 128, "tok_per_s": round(tps, 1),
                                    "ms_per_token": round(1e3 / tps, 3), "distinct_new_tokens": _distinct(toks, 128)}
        del model
        torch.cuda.empty_cache()

    # ---- CPU baseline (bounded sample) -------------------------------------
    if not args.no_cpu:
        from oracle import torch_cpu_path
        cores = torch.get_num_threads()
        t_dec = t_mm = 0.0
        worst = 0.0
        reps = 2
        for name, m, k in shapes:  # one pass over the whole set = one step, best of `reps`
            pk = packed[name][0].cpu()
            x = xs[name].cpu()
            r = torch_cpu_path.time_layer(pk, x, tlut.cpu(), m, k, K, reps=reps)
            t_dec += r["decode_s"]
            t_mm += r["matmul_s"]
            gpu = outs[name].clone()
            ops.decompress_matvec(packed[name][0], xs[name], tlut, m, k, K, out=gpu)
            ref = r["out"].double()
            worst = max(worst, float((gpu.cpu().double() - ref).abs().max() / ref.abs().max()))
            del r, pk
        cpu_s = t_dec + t_mm
        result["cpu_baseline"] = {
            "value": round(set_bytes / cpu_s / 1e9, 4),
            "unit": "GB/s",
            "cores": cores,
            "kind": "port",
            "sample": f"one step (the same {len(shapes)} matrices, {set_bytes >> 20} MiB packed), best of {reps}: torch CPU "
                      f"trellis decode {t_dec:.2f} s + fp32 matvec {t_mm:.3f} s",
            "ms_per_step": round(cpu_s * 1e3, 1),
            "gpu_vs_cpu_max_rel_err": worst,
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
