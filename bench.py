#!/usr/bin/env python3
"""Benchmark of the convolutional hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload yolov3|yolov4|resnet50|mobilenetv2|resnet18|yolov3_tiny|yolov5s]

A step is one forward of one batch through NetBuilder's device-resident path (input already in HBM): every
launch of the planned graph, and for detection networks the candidate compaction on the device plus copy-back,
sort and NMS on the host, so that a step ends with the boxes (or logits) in host memory.  Prints ONE JSON line.
`value` is the whole-job rate over the K timed steps; the median of the per-step times is reported beside it.
By default the K steps are dealt round-robin to three instances of the network (--instances; each a NetBuilder with its own
stream, driven by its own host thread, two batches in flight each), which is how a server keeps the device busy across
the gaps between the launches of one forward; `one_instance_images_per_s` of the same line is the rate of one instance alone.

    python bench.py --conv-shape b,c,h,w,oc,k,stride [--tile n] [--reps 20] [--residual] [--conv-dtype f16|f32]

times one convolution shape through the kernel C ABI instead: with every implicit-GEMM tile configuration that accepts
it (microseconds and TFLOP/s per tile), or, with --tile, launches that configuration --reps times and nothing else,
which is the form to put behind `rocprofv3 --pmc ... --` when the counters of one kernel are wanted.
"""
import argparse
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from msnhnet_amd import netapi, zoo  # noqa: E402

# workload -> (dtype, batch, input size) : the benchmark configurations
WORKLOADS = {"resnet18": ("f32", 1, 224), "resnet50": ("f16", 32, 224), "mobilenetv2": ("f16", 64, 224),
             "yolov3": ("f16", 8, 608), "yolov4": ("f16", 16, 608),
             # two of the reference's other shipped detectors, at the input size of their own graph files
             "yolov3_tiny": ("f16", 8, 416), "yolov5s": ("f16", 8, 512)}
PEAK = {"f16": 2500.0, "f32": 157.3}        # dense MFMA peak, TFLOP/s


def cpu_baseline(arch, size, tmp, seed, budget_s=30.0):
    """Reference CPU forward (its own code, as shipped: AVX2+FMA, all OpenMP threads) on a bounded sample of the
    same workload: batch-1 forwards of the same graph and weights, repeated while they fit the time budget."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import refshim
    g = zoo.ARCHS[arch](batch=1, size=size)
    net = os.path.join(tmp, f"{arch}_cpu.msnhnet")
    with open(net, "w") as f:
        f.write(g.text())
    binp = os.path.join(tmp, f"{arch}_cpu.msnhbin")
    zoo.seeded_weights(g.slots, seed).tofile(binp)
    x = zoo.seeded_input(1, 3, size, size, seed + 1)[0]
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    if refshim.available():
        kind = "reference"
        r = refshim.RefNet(net, binp, scalar=False)
        run = lambda: r.run(x, capture=False)
    else:
        import msnh_oracle_net as on
        kind = "port"
        o = on.OracleNet(net, binp)
        run = lambda: o.run(x)
    t0 = time.time()
    run()                                   # first forward doubles as warm-up when it is already long
    first = time.time() - t0
    times = [first]
    while sum(times) + min(times) < budget_s and len(times) < 20:
        t0 = time.time()
        run()
        times.append(time.time() - t0)
    best = min(times[1:]) if len(times) > 1 else first
    return {"value": round(1.0 / best, 5), "unit": "images/s", "cores": cores, "kind": kind,
            "sample": f"{len(times)} batch-1 forward(s) of {arch}-{size} float32 on the host CPU, best of the timed ones "
                      f"({best:.2f} s per image incl. its NMS)"}


# HBM bytes per launch (fetch + write) of the dominant kernels, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script and kept in profiles/hbm_traffic.json, one entry per (workload, dtype, batch) with the hash of the plan it was measured
# on (launch kinds, algorithms and shapes; not the tile choices, which the per-layer search may settle differently from run to
# run).  A plan that hashes differently -- a kernel or a fusion changed since -- reports null instead of a stale figure.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
HBM_PEAK = 8000.0           # GB/s


def plan_hash(plan_text):
    """hash of a plan description without its tile numbers and arena size"""
    import hashlib
    import re
    # (which of the GEMM-type kernels and which tile runs a layer is the per-layer search's choice and may differ between two runs)
    lines = [re.sub(r"\[(igemm_splitk|igemm|pointwise)", "[gemm", re.sub(r" t\d+", "", l)) for l in plan_text.splitlines()[1:]]
    return hashlib.sha256("\n".join(lines).encode()).hexdigest()[:16]


def measured_traffic(workload, dtype, batch, plan_text, key):
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    e = table.get(f"{workload}|{dtype}|{batch}")
    if not e or e.get("plan_hash") != plan_hash(plan_text):
        return None
    return e.get(key)


def attainable(rows, peak_tflops):
    """rows: netapi.Net.profile_each_op_values().  For every convolution / connected launch the time it cannot beat is
    t_min = max(FLOPs / MFMA peak, least bytes / HBM peak); returns the sums that say how far the measured launches are from that
    bound, split by which roof binds."""
    out = {"mfma_bound": {"launches": 0, "us": 0.0, "us_min": 0.0, "tflops": 0.0}, "hbm_bound": {"launches": 0, "us": 0.0, "us_min": 0.0, "gbs": 0.0}}
    flops_m = bytes_h = 0.0
    for kind, algo, layer, tile, flops, nbytes, us, ks in rows:
        if int(kind) not in (0, 7) or int(algo) == MSNH_CONV_DEPTHWISE:
            continue
        t_m = flops / (peak_tflops * 1e12) * 1e6
        t_h = nbytes / (HBM_PEAK * 1e9) * 1e6
        c = out["mfma_bound"] if t_m >= t_h else out["hbm_bound"]
        c["launches"] += 1
        c["us"] += us
        c["us_min"] += max(t_m, t_h)
        if t_m >= t_h:
            flops_m += flops
        else:
            bytes_h += nbytes
    m, h = out["mfma_bound"], out["hbm_bound"]
    m["tflops"] = round(flops_m / m["us"] * 1e-6, 1) if m["us"] else None
    h["gbs"] = round(bytes_h / h["us"] * 1e-3, 1) if h["us"] else None
    m["frac_of_mfma_peak"] = round(m["tflops"] / peak_tflops, 4) if m["us"] else None
    h["frac_of_hbm_peak"] = round(h["gbs"] / HBM_PEAK, 4) if h["us"] else None
    total_us, total_min = m["us"] + h["us"], m["us_min"] + h["us_min"]
    for c in (m, h):
        c["us"], c["us_min"] = round(c["us"], 1), round(c["us_min"], 1)
    return round(total_min / total_us, 4) if total_us else None, out


def bandwidth_kinds(rows):
    """the bandwidth-bound launches of the plan by kind (depthwise, pools, upsample, copies, decode, ...): GB/s on least bytes"""
    names = {1: "affine", 2: "add", 3: "copy", 4: "maxpool", 5: "avgpool", 6: "upsample", 8: "input_cast", 9: "yolo_decode", 10: "pad", 11: "slice",
             12: "bilinear", 13: "softmax", 14: "col2im"}
    acc = {}
    for kind, algo, layer, tile, flops, nbytes, us, ks in rows:
        name = "depthwise" if (int(kind) == 0 and int(algo) == MSNH_CONV_DEPTHWISE) else names.get(int(kind))
        if name is None:
            continue
        a = acc.setdefault(name, [0, 0.0, 0.0])
        a[0] += 1
        a[1] += nbytes
        a[2] += us
    return {k: {"launches": v[0], "us": round(v[2], 1), "gbs": round(v[1] / v[2] * 1e-3, 1), "frac_of_hbm_peak": round(v[1] / v[2] * 1e-3 / HBM_PEAK, 4)}
            for k, v in acc.items() if v[2] > 0}


MSNH_CONV_DEPTHWISE = 3


def conv_shape_mode(a):
    """One convolution shape through msnh_hip_conv2d: every tile configuration timed with device events, or one forced
    configuration launched --reps times (nothing else runs then: the form for a counter run).  Random inputs; results
    are not checked here (the parity tests do that)."""
    import ctypes

    import torch

    from msnhnet_amd import hipabi as abi
    b, c, h, w, oc, k, stride = (int(v) for v in a.conv_shape.split(","))
    pad = k // 2
    oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    dt = abi.F16 if a.conv_dtype == "f16" else abi.F32
    tdt = torch.float16 if a.conv_dtype == "f16" else torch.float32
    L = abi.lib()
    abi.check(L.msnh_hip_init(0))
    d = abi.ConvDesc(dt, dt, b, h, w, c, c, oc, oh, ow, oc, k, stride, pad, 1, 1, abi.ACT["leaky"], 0.1, 1 if a.residual else 0, oc,
                     abi.ACT["none"], 0.1, 1.0, 1.0, abi.ALGO[a.conv_algo], 0)
    x = torch.randn(b, h, w, c, dtype=tdt, device="cuda")
    # (random values in the packed layout of the algorithm: tap-major filters, or the 16 transformed filter matrices of Winograd F(2x2,3x3))
    wt = torch.randn(int(L.msnh_hip_conv2d_packed_weight_elems(ctypes.byref(d), abi.ALGO[a.conv_algo])), dtype=tdt, device="cuda") * 0.05
    ws_bytes = int(L.msnh_hip_conv2d_workspace_bytes(ctypes.byref(d), abi.ALGO[a.conv_algo]))
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device="cuda")
    y = torch.empty(b, oh, ow, oc, dtype=tdt, device="cuda")
    res = torch.randn(b, oh, ow, oc, dtype=tdt, device="cuda") if a.residual else None
    sc = torch.ones(oc, device="cuda")
    sh = torch.zeros(oc, device="cuda")

    def ptr(t):
        return ctypes.c_void_p(t.data_ptr()) if t is not None else None

    def run():
        abi.check(L.msnh_hip_conv2d(ctypes.byref(d), ptr(x), ptr(wt), ptr(sc), ptr(sh), ptr(res), ptr(y), ptr(ws), ws_bytes, None))

    torch.cuda.synchronize()
    if a.switches:
        # the LDS-patch kernel with parts switched off (timing diagnostics library): where a launch's time goes and what clock the part
        # holds under each mix of work
        from msnhnet_amd import diag
        if a.tile not in (46, 52) or k != 3 or stride != 1 or a.conv_dtype != "f16" or a.residual:
            sys.exit("--switches: --tile 46 or 52, a 3x3 stride-1 float16 shape, no --residual")
        D = diag.lib()
        e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
        abi.check(L.msnh_hip_event_create(ctypes.byref(e0)))
        abi.check(L.msnh_hip_event_create(ctypes.byref(e1)))
        clocks = torch.zeros(2, dtype=torch.int64, device="cuda")
        torch.cuda.synchronize()

        def timed(fn):
            fn()
            fn()
            abi.check(L.msnh_hip_event_record(e0, None))
            for _ in range(a.reps):
                fn()
            abi.check(L.msnh_hip_event_record(e1, None))
            abi.check(L.msnh_hip_event_sync(e1))
            ms = ctypes.c_float()
            abi.check(L.msnh_hip_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
            return ms.value * 1e3 / a.reps

        for sw in diag.switches():
            def one():
                rc = D.msnh_hip_diag_patch8(a.tile, sw, b, c, h, w, oc, ptr(x), ptr(wt), ptr(sc), ptr(sh), ptr(y), ptr(clocks), None)
                if rc:
                    sys.exit(f"msnh_hip_diag_patch8: error {rc} (tile {a.tile}, switches {sw}): {L.msnh_hip_last_error()}")
            us = timed(one)
            line = f"tile {a.tile} switches {sw:2d} {diag.describe(sw):78s} {us:8.2f} us per launch"
            if sw & 64:
                t = clocks.cpu().numpy()
                line += f"; main loop {int(t[0])} shader ticks in {t[1] / 100:.2f} us = {t[0] / max(int(t[1]), 1) * 100:.0f} MHz"
            print(line, flush=True)
        for blocks, threads in ((256, 768), (256, 256), (2048, 256)):
            us = timed(lambda: D.msnh_hip_diag_empty_launch(blocks, threads, None))
            print(f"empty kernel {blocks} x {threads}: {us:8.2f} us per launch", flush=True)
        L.msnh_hip_event_destroy(e0)
        L.msnh_hip_event_destroy(e1)
        return
    if a.tile > 0:
        d.tile = a.tile
        if not L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), a.tile):
            sys.exit(f"tile {a.tile} does not take this shape")
        import time
        run()
        abi.check(L.msnh_hip_stream_sync(None))
        t0 = time.perf_counter()
        for _ in range(a.reps):
            run()
        abi.check(L.msnh_hip_stream_sync(None))
        us = (time.perf_counter() - t0) / a.reps * 1e6
        print(f"tile {a.tile}: {a.reps} launches of {a.conv_shape}, {us:.2f} us per launch back to back (host clock)")
        return
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    abi.check(L.msnh_hip_event_create(ctypes.byref(e0)))
    abi.check(L.msnh_hip_event_create(ctypes.byref(e1)))
    flops = 2.0 * b * oc * oh * ow * c * k * k
    # (the one-launch Winograd form has no tile configurations: it is timed as tile 0)
    for tile in ([0] if a.conv_algo == "winograd_fused" else range(1, L.msnh_hip_conv2d_tile_count() + 1)):
        d.tile = tile
        if not L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), tile):
            continue
        run()
        run()
        abi.check(L.msnh_hip_event_record(e0, None))
        for _ in range(a.reps):
            run()
        abi.check(L.msnh_hip_event_record(e1, None))
        abi.check(L.msnh_hip_event_sync(e1))
        ms = ctypes.c_float()
        abi.check(L.msnh_hip_event_elapsed_ms(e0, e1, ctypes.byref(ms)))
        us = ms.value * 1e3 / a.reps
        print(f"tile {tile:2d}: {us:8.2f} us  {flops / us * 1e-6:7.1f} TFLOP/s", flush=True)
    L.msnh_hip_event_destroy(e0)
    L.msnh_hip_event_destroy(e1)


def mbconv_shape_mode(a):
    """One inverted-residual block (1x1 expand, 3x3 depthwise, 1x1 project, relu6 twice, optional residual) through msnh_hip_mbconv,
    --reps launches back to back after one warm-up launch.  Random inputs and weights; results are not checked here (tests/test_mbconv_gpu.py
    does that)."""
    import ctypes
    import time

    import numpy as np
    import torch

    from msnhnet_amd import hipabi as abi
    b, cin, h, w, cexp, cout, stride, with_res = (int(v) for v in a.mbconv_shape.split(","))
    L = abi.lib()
    abi.check(L.msnh_hip_init(0))
    oh, ow = (h - 1) // stride + 1, (w - 1) // stride + 1
    d = abi.MbconvDesc(b, h, w, cin, cin, cexp, stride, cout, oh, ow, cout, abi.ACT["relu6"], abi.ACT["relu6"], abi.ACT["none"], abi.ACT["none"],
                       0.1, 0.1, 0.1, 0.1, 1 if with_res else 0, cout, 1.0, 1.0, 1.0, 1.0)
    if not L.msnh_hip_mbconv_supported(ctypes.byref(d)):
        sys.exit("msnh_hip_mbconv does not take this block")
    rng = np.random.default_rng(a.seed)
    we = rng.standard_normal((cexp, cin), dtype=np.float32) * np.float32(0.2)
    wd = rng.standard_normal((cexp, 9), dtype=np.float32) * np.float32(0.3)
    wp = rng.standard_normal((cout, cexp), dtype=np.float32) * np.float32(0.1)
    packed = np.zeros(L.msnh_hip_mbconv_packed_bytes(ctypes.byref(d)), np.uint8)
    hp = lambda arr: arr.ctypes.data_as(ctypes.c_void_p)
    abi.check(L.msnh_hip_mbconv_pack(ctypes.byref(d), hp(we), None, None, hp(wd), None, None, hp(wp), hp(packed)))
    x = torch.randn(b, h, w, cin, dtype=torch.float16, device="cuda")
    y = torch.empty(b, oh, ow, cout, dtype=torch.float16, device="cuda")
    r = torch.randn(b, oh, ow, cout, dtype=torch.float16, device="cuda") if with_res else None
    pd = torch.from_numpy(packed).cuda()
    dp = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    torch.cuda.synchronize()

    def run():
        abi.check(L.msnh_hip_mbconv(ctypes.byref(d), dp(x), dp(pd), None, None, dp(r), dp(y), None))

    run()
    abi.check(L.msnh_hip_stream_sync(None))
    t0 = time.perf_counter()
    for _ in range(a.reps):
        run()
    abi.check(L.msnh_hip_stream_sync(None))
    us = (time.perf_counter() - t0) / a.reps * 1e6
    flops = 2.0 * b * (h * w * cexp * cin + oh * ow * cexp * 9 + oh * ow * cout * cexp)
    nbytes = 2.0 * b * (h * w * cin + oh * ow * cout * (2 if with_res else 1))
    print(f"mbconv {a.mbconv_shape}: {a.reps} launches, {us:.2f} us per launch back to back (host clock), {flops / us * 1e-6:.1f} TFLOP/s, "
          f"{nbytes / us * 1e-3:.0f} GB/s on input + output" + (" + residual" if with_res else ""))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--conv-shape", default=None, help="b,c,h,w,oc,k,stride: time this one convolution shape instead of a workload")
    ap.add_argument("--mbconv-shape", default=None,
                    help="b,in_c,h,w,exp_c,out_c,stride,residual(0|1): launch this one inverted-residual block (msnh_hip_mbconv) --reps times and "
                         "print the time per launch (the form to put behind rocprofv3 --pmc)")
    ap.add_argument("--tile", type=int, default=0, help="--conv-shape: launch only this tile configuration, --reps times, untimed")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--switches", action="store_true",
                    help="--conv-shape with --tile 46 or 52: the LDS-patch kernel timed with parts of it switched off and with the shader clock read inside "
                         "(timing diagnostics library, include/msnh_hip_diag.h)")
    ap.add_argument("--residual", action="store_true", help="--conv-shape: with a fused residual add")
    ap.add_argument("--conv-dtype", default="f16", choices=["f16", "f32"])
    ap.add_argument("--conv-algo", default="igemm", choices=["igemm", "winograd", "winograd_fused"],
                    help="--conv-shape: the implicit GEMM (default) or the three-launch Winograd F(2x2,3x3) form (input transform, 16 GEMMs as one grouped launch "
                         "with the tile given, output transform)")
    ap.add_argument("--workload", default="yolov3", choices=sorted(WORKLOADS))
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--input", default="device", choices=["device", "host_f32", "host_u8"],
                    help="device (default, the headline figure): the batch is resident in HBM when the clock starts.  host_f32: the "
                         "reference's own calling convention, a host float image per call (runYoloGPU / runClassifyGPU), PCIe "
                         "inclusive.  host_u8: 8-bit host images, letterboxed on the device, PCIe inclusive.")
    ap.add_argument("--nms", default="auto", choices=["host", "auto", "device"],
                    help="detection workloads: sort + NMS on the host, on the device, or (library default) on the device while the "
                         "previous result had at most 2048 candidates per image -- the seeded weights give 11k, so auto means host here")
    ap.add_argument("--instances", type=int, default=3,
                    help="network instances on the GPU, each with its own stream and arena, fed round-robin by one host thread each "
                         "(netapi.NetGroup; device-resident input only).  The device runs their forwards side by side, which fills the launch gaps, "
                         "prologues and write bursts that a single stream leaves open.  1 = one instance, two batches in flight on one stream")
    ap.add_argument("--depth", type=int, default=2, help="--instances > 1: batches in flight per instance (detectors; a classifier has one)")
    ap.add_argument("--per-op", default=None, metavar="FILE",
                    help="also write the per-launch table (every launch of the plan timed on its own with device events: microseconds, "
                         "algorithmic TFLOP/s and GB/s with every tensor counted once) to FILE")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch a plain 256 MiB -> 256 MiB channel-copy kernel 5 times (a known-size reference for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (no sharding, no collectives); use --gpus 1")

    import torch          # device memory for the synthetic input only
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the hot path has no CPU fallback")
    if a.conv_shape:
        conv_shape_mode(a)
        return
    if a.mbconv_shape:
        mbconv_shape_mode(a)
        return

    dtype, batch, size = WORKLOADS[a.workload]
    tmp = tempfile.mkdtemp(prefix="msnh_bench_")
    netp, binp, g = zoo.write_model(a.workload, tmp, batch, size, seed=a.seed)
    netapi.set_device_nms({"host": 0, "auto": 1, "device": 2}[a.nms])
    group = None
    if a.instances > 1 and a.input == "device":
        group = netapi.NetGroup(netp, binp, instances=a.instances, depth=a.depth, fp16=(dtype == "f16"))
        net = group.nets[0]
    else:
        net = netapi.Net(netp, binp, fp16=(dtype == "f16"))
    detect = a.workload.startswith("yolo")

    if a.copy_probe:
        import ctypes
        from msnhnet_amd import hipabi
        src = torch.ones(1 << 27, dtype=torch.float16).cuda()          # 256 MiB
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(5):
            hipabi.check(hipabi.lib().msnh_hip_copy_channels(hipabi.F16, (1 << 27) // 256, 256, ctypes.c_void_p(src.data_ptr()), 256, 1.0,
                                                             ctypes.c_void_p(dst.data_ptr()), 256, None))
        hipabi.check(hipabi.lib().msnh_hip_stream_sync(None))
        del src, dst

    def marker():
        """With --copy-probe: one tiny absmax launch (a kernel no forward uses), a delimiter between the phases of this script in a
        kernel trace."""
        if a.copy_probe:
            import ctypes
            from msnhnet_amd import hipabi
            hipabi.check(hipabi.lib().msnh_hip_absmax(hipabi.F16, 1, 8, ctypes.c_void_p(mark.data_ptr()), 8, ctypes.c_void_p(mark.data_ptr() + 64), None))

    mark = torch.zeros(64, dtype=torch.float16).cuda()
    x = torch.from_numpy(zoo.seeded_input(batch, 3, size, size, a.seed + 1)).cuda()
    torch.cuda.synchronize()
    dev_in = x.data_ptr()

    host_x = zoo.seeded_input(batch, 3, size, size, a.seed + 1) if a.input == "host_f32" else None
    host_u8 = None
    if a.input == "host_u8":
        host_u8 = np.random.default_rng(a.seed + 2).integers(0, 256, (batch, size, size, 3), dtype=np.uint8)

    # device-resident input: the batch is written once into the network's own input buffer (msnhnet_device_input, the documented
    # serving path: a producer on the device writes there) and every step runs on it; no copy of the input inside the timed region
    if group is not None:
        group.prime(dev_in)
    elif host_u8 is None and host_x is None:
        net.enqueue(dev_in)
        _ = net.fetch_yolo() if detect else net.fetch_classify()

    def feed():
        if host_u8 is not None:
            for i in range(batch):
                net.set_input_image_u8(i, host_u8[i])
        net.enqueue(None)

    on_device = [0]

    def run_steps(k, stamps=None, host=None, use_group=True):
        """k forwards + k result fetches.  Detection keeps two batches in flight: while the host sorts and
        suppresses the boxes of batch i the device already runs batch i+1.  stamps collects the time at which each
        step's result reached the host."""
        out = None
        tick = (lambda: stamps.append(time.perf_counter())) if stamps is not None else (lambda: None)
        if group is not None and use_group and host is None:
            # every instance's thread keeps `depth` batches in flight; results come back in submission order
            for _ in range(k):
                group.submit(None)
            group.flush()
            for _ in range(k):
                out = group.fetch()
                tick()
            on_device[0] = None
        elif host is not None:
            for _ in range(k):
                out = net.run_yolo(host) if detect else net.run_classify(host)
                tick()
        elif detect:
            feed()
            for _ in range(k - 1):
                feed()
                out = net.fetch_yolo()
                tick()
                on_device[0] += net.last_nms_on_device()
            out = net.fetch_yolo()
            tick()
            on_device[0] += net.last_nms_on_device()
        else:
            for _ in range(k):
                feed()
                out = net.fetch_classify()
                tick()
        return out

    # set-up, not warm-up: the first forwards allocate the two copy-back slots (pinned host and device snapshots) and start the
    # host worker threads; they belong to building the network like the plan and the tile search
    run_steps(4, host=host_x)
    if a.warmup > 0:
        run_steps(a.warmup, host=host_x)
    net.sync()
    marker()
    torch.cuda.synchronize()
    stamps = []
    on_device[0] = 0
    import gc
    gc.collect()
    gc.disable()          # a collection in the middle of the host stage would be timed as a step of several milliseconds
    t0 = time.perf_counter()
    out = run_steps(a.steps, stamps, host=host_x)
    net.sync()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    steps_on_device = on_device[0]
    single_rate = None
    if group is not None:
        # the same run with one instance alone (two batches in flight on one stream), for comparison
        on_device[0] = 0
        k1 = min(a.steps, 100)
        if detect:
            net.set_copy_on_forward_stream(False)       # as a NetBuilder on its own runs: copy-back on a stream beside the next forward
            run_steps(4, use_group=False)
        ts = time.perf_counter()
        run_steps(k1, use_group=False)
        net.sync()
        single_rate = round(batch * k1 / (time.perf_counter() - ts), 2)
        if detect:
            net.set_copy_on_forward_stream(True)
    gc.enable()
    marker()
    ms_per_step = dt / a.steps * 1e3
    per_step = np.diff(np.array([t0] + stamps)) * 1e3
    if group is not None and len(stamps) > 2 * a.instances:
        # results of different instances arrive in bursts (they are handed out in submission order): the time between results is
        # taken over one round of the instances
        st = np.array([t0] + stamps)
        per_step = (st[a.instances:] - st[:-a.instances]) / a.instances * 1e3
    slow = [i for i, v in enumerate(per_step) if v > 5.0]
    # (pipelined detection: the first interval holds two forwards, every later one is a steady-state step)
    ms_median = float(np.median(per_step[1:])) if len(per_step) > 1 else float(per_step[0])
    steady = per_step[1:] if len(per_step) > 1 else per_step
    ms_spread = [round(float(np.percentile(steady, q)), 4) for q in (0, 10, 50, 90, 99, 100)]

    # the reference's own calling convention beside the headline: one synchronous run*GPU(std::vector<float>) per batch, the float
    # host image uploaded inside the call (PCIe inclusive; never `value`)
    host_rate = None
    if a.input == "device" and not a.copy_probe:
        hx = zoo.seeded_input(batch, 3, size, size, a.seed + 1)
        run_steps(2, host=hx)
        th = time.perf_counter()
        run_steps(5, host=hx)
        host_rate = round(batch * 5 / (time.perf_counter() - th), 2)

    # device-only time of the captured forward (no host post-processing), for orientation
    all_ms, n_all, _ = net.profile_ops(-1, 10)
    gpu_only_ms = all_ms / 10

    # roofline of the dominant kernel family: the convolution launches, timed with device events on the
    # library's stream; algorithmic FLOPs = 2*B*Cout*OH*OW*(Cin/g)*k*k per launch (direct-convolution count)
    plan_text = net.plan_detail()
    marker()
    conv_ms, launches, flops, conv_bytes = net.profile_ops_bytes(0, 10)
    marker()
    achieved = flops / (conv_ms * 1e-3) / 1e12 if conv_ms > 0 else 0.0
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK[dtype], "unit": "TFLOP/s",
                "frac": round(achieved / PEAK[dtype], 4), "traffic": measured_traffic(a.workload, dtype, batch, plan_text, "conv_hbm_bytes_per_launch"),
                "kernel": "convolution launches (implicit-GEMM MFMA + stem)", "launches_per_step": launches // 10,
                "avg_launch_us": round(conv_ms * 1e3 / max(launches, 1), 2), "flops_per_step": flops / 10,
                "least_bytes_per_launch": int(conv_bytes / max(launches, 1)),
                # the same FLOPs over the time between results of the timed region (everything included: the other launches, decode, copy-back,
                # host stage, several instances overlapping): what the job as a whole extracts from the matrix cores
                "whole_job_tflops": round(flops / 10 / (ms_per_step * 1e-3) / 1e12, 2), "whole_job_frac": round(flops / 10 / (ms_per_step * 1e-3) / 1e12 / PEAK[dtype], 4)}

    # How far the launches are from the roof that binds each of them: a launch cannot beat max(FLOPs / MFMA peak, least bytes / HBM
    # peak).  Every launch is timed on its own here (back-to-back repetitions), so the sums are a little below the in-order pass above.
    rows = net.profile_each_op_values(20)
    roofline["attainable_frac"], roofline["by_binding_roof"] = attainable(rows, PEAK[dtype])
    roofline["plan_hash"] = plan_hash(plan_text)
    bw = bandwidth_kinds(rows)

    # what the matrix cores of this part sustain with nothing in their way (pure MFMA loops, three wavefronts per SIMD as in the
    # convolution kernels), and the shader clock they hold meanwhile: `peak` above is the published figure at the maximum clock
    if dtype == "f16":
        import ctypes
        from msnhnet_amd import hipabi
        tf, mhz, sec = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        hipabi.check(hipabi.lib().msnh_hip_mfma_probe(3, 20000, ctypes.byref(tf), ctypes.byref(mhz), ctypes.byref(sec), None))
        roofline["mfma_probe"] = {"sustained": round(tf.value, 1), "unit": "TFLOP/s", "shader_mhz": round(mhz.value), "ms": round(sec.value * 1e3, 3),
                                  "frac_of_sustained": round(achieved / tf.value, 4) if tf.value > 0 else None}

    # a network with depthwise convolutions is judged against the HBM roof as well: those launches move
    # (input + output + weights) bytes each and compute next to nothing
    roofline_hbm = None
    dw_ms, dw_n, _, dw_bytes = net.profile_ops_bytes(1000 + MSNH_CONV_DEPTHWISE, 10)
    if dw_n > 0:
        gbs = dw_bytes / (dw_ms * 1e-3) / 1e9
        roofline_hbm = {"bound": "hbm", "achieved": round(gbs, 1), "peak": 8000.0, "unit": "GB/s", "frac": round(gbs / 8000.0, 4),
                        "traffic": measured_traffic(a.workload, dtype, batch, plan_text, "depthwise_hbm_bytes_per_launch"), "kernel": "convDepthwise3x3FastKernel",
                        "launches_per_step": dw_n // 10, "avg_launch_us": round(dw_ms * 1e3 / dw_n, 2), "bytes_per_step": dw_bytes / 10}

    res = {"metric": f"images/sec on 1 MI355X ({a.workload} {size} {dtype} b{batch})", "value": round(batch / (ms_per_step * 1e-3), 2),
           "unit": "images/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
           "config": {"workload": f"{a.workload}-{size} {dtype} batch {batch}, seeded He-normal weights, U[0,1) input, "
                                  f"{'input resident in the network input buffer on the device' if a.input == 'device' else a.input + ' input'} -> {'boxes' if detect else 'logits'} on host"
                                  + (f"; {a.instances} network instances fed round-robin, {group.depth} batch(es) in flight each, a step = one batch of one instance "
                                     f"(ms_per_step = time between results)" if group is not None else ""),
                      "instances": a.instances if group is not None else 1, "one_instance_images_per_s": single_rate, "batches_in_flight": (a.instances * group.depth) if group is not None else (2 if detect else 1),
                      "input": a.input, "seed": a.seed, "ms_per_step_median": round(ms_median, 4), "ms_per_step_percentiles_0_10_50_90_99_100": ms_spread, "steps_over_5ms": slow, "device_launches_per_step": n_all // 10,
                      "device_ms_per_step_eager": round(gpu_only_ms, 4), "host_f32_images_per_s": host_rate},
           "roofline": roofline}
    if roofline_hbm is not None:
        res["roofline_hbm"] = roofline_hbm
    if bw:
        res["bandwidth_launches"] = bw
    if detect:
        res["config"]["boxes_per_image"] = [int(len(b)) for b in out]
        res["config"]["nms"] = a.nms
        res["config"]["steps_with_nms_on_device"] = steps_on_device
    if a.per_op:
        with open(a.per_op, "w") as f:
            f.write(net.profile_each_op(20))
    if group is not None:
        group.close()
    if not a.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(a.workload, size, tmp, a.seed)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
