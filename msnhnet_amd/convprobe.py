"""Time one convolution shape with each (or one forced) implicit-GEMM tile configuration, through the kernel C ABI.

    python -m msnhnet_amd.convprobe --shape 8,256,38,38,512,3,1 [--tile 38] [--reps 20] [--residual] [--dtype f16]

--shape is batch,in_c,h,w,out_c,ksize,stride (pad = ksize // 2).  Without --tile every configuration that accepts the
shape is timed with device events and printed as microseconds / TFLOP/s; with --tile that configuration is launched
--reps times and nothing else runs, which is the form to put behind `rocprofv3 --pmc ... --` when the counters of one
kernel are wanted.  Random inputs; the results are not checked here (the parity tests do that).
"""
import argparse
import ctypes

import torch

from . import hipabi as abi


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--shape", required=True)
    ap.add_argument("--tile", type=int, default=0)
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--residual", action="store_true")
    ap.add_argument("--dtype", default="f16", choices=["f16", "f32"])
    a = ap.parse_args()
    b, c, h, w, oc, k, stride = (int(v) for v in a.shape.split(","))
    pad = k // 2
    oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    dt = abi.F16 if a.dtype == "f16" else abi.F32
    tdt = torch.float16 if a.dtype == "f16" else torch.float32
    L = abi.lib()
    abi.check(L.msnh_hip_init(0))
    d = abi.ConvDesc(dt, dt, b, h, w, c, c, oc, oh, ow, oc, k, stride, pad, 1, 1, abi.ACT["leaky"], 0.1, 1 if a.residual else 0, oc,
                     abi.ACT["none"], 0.1, 1.0, 1.0, abi.ALGO["igemm"], 0)
    x = torch.randn(b, h, w, c, dtype=tdt, device="cuda")
    wt = torch.randn(oc, k * k, c, dtype=tdt, device="cuda") * 0.05
    y = torch.empty(b, oh, ow, oc, dtype=tdt, device="cuda")
    res = torch.randn(b, oh, ow, oc, dtype=tdt, device="cuda") if a.residual else None
    sc = torch.ones(oc, device="cuda")
    sh = torch.zeros(oc, device="cuda")

    def ptr(t):
        return ctypes.c_void_p(t.data_ptr()) if t is not None else None

    def run():
        abi.check(L.msnh_hip_conv2d(ctypes.byref(d), ptr(x), ptr(wt), ptr(sc), ptr(sh), ptr(res), ptr(y), None, 0, None))

    torch.cuda.synchronize()
    if a.tile > 0:
        d.tile = a.tile
        if not L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), a.tile):
            raise SystemExit(f"tile {a.tile} does not take this shape")
        for _ in range(a.reps):
            run()
        abi.check(L.msnh_hip_stream_sync(None))
        print(f"tile {a.tile}: {a.reps} launches of {a.shape}")
        return
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    abi.check(L.msnh_hip_event_create(ctypes.byref(e0)))
    abi.check(L.msnh_hip_event_create(ctypes.byref(e1)))
    flops = 2.0 * b * oc * oh * ow * c * k * k
    for tile in range(1, L.msnh_hip_conv2d_tile_count() + 1):
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


if __name__ == "__main__":
    main()
