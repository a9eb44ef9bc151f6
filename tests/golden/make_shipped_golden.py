"""Writes tests/golden/shipped_golden.npz: every graph file the reference ships (models/*/*.msnhnet) run through the reference's own
CPU forward (oracle/_ref, scalar mode) on seeded weights and a seeded input.

Run in a container that holds the reference (graph files and the built oracle/_ref library):
    python tests/golden/make_shipped_golden.py
Stored per graph: the graph text as fed to both sides (the shipped file with its input size reduced where the graph allows it, so the
CPU forward takes seconds), the seeds, per-layer statistics of the reference's outputs, its final tensor and its boxes.  Weights are not
stored: both sides draw them from the seed through the host library's own description of the weights file (msnhnet_weight_layout).
Graphs the reference itself cannot run are recorded with the error text.
"""
import glob
import os
import re
import sys
import time
import zlib

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "tests"), os.path.join(ROOT, "oracle")):
    sys.path.insert(0, p)

import refshim  # noqa: E402
from make_golden import layer_stats  # noqa: E402
from msnhnet_amd import netapi, zoo  # noqa: E402

REF_MODELS = "/root/reference/models"
OUT = os.path.join(HERE, "shipped_golden.npz")
TMP = "/tmp/msnh_shipped"
os.makedirs(TMP, exist_ok=True)

# input sizes (height, width) tried in place of the shipped one, first that the reference builds and runs wins; detectors and
# segmentation graphs only -- a graph that ends in connected layers is tied to its size
REDUCED = {"yolov3": (96, 96), "yolov3_darknet": (96, 96), "yolov4": (96, 96), "yolov3_tiny": (96, 96), "yolov3_tiny_pad": (96, 96),
           "yolov5m": (128, 128), "yolov5s": (128, 128), "mobilenetv2_yolov3_lite": (128, 128), "mobilenetv2_yolov3_lite1": (128, 128),
           "mobilenetv2_yolov3_nano": (128, 128), "yoloface100k": (96, 96), "yoloface500k": (64, 96), "unet": (64, 64), "deeplabv3": (64, 64),
           "fcns": (96, 96)}


def with_size(text, hw):
    h, w = hw
    text = re.sub(r"(\n\s*width:\s*)\d+", lambda m: m.group(1) + str(w), text, count=1)
    return re.sub(r"(\n\s*height:\s*)\d+", lambda m: m.group(1) + str(h), text, count=1)


def seeded_weights_for(netp, seed):
    m = netapi.Net(netp)
    w = zoo.seeded_weights(zoo.slots_from_layout(m.weight_layout()), seed)
    dims = m.dims()
    m.close()
    return w, dims


def main():
    store, names = {}, []
    for k, path in enumerate(sorted(glob.glob(os.path.join(REF_MODELS, "*", "*.msnhnet")))):
        name = os.path.basename(path)[:-len(".msnhnet")]
        shipped = open(path, encoding="utf-8-sig").read()
        seed = 500 + 2 * k
        done = False
        for text in ([with_size(shipped, REDUCED[name])] if name in REDUCED else []) + [shipped]:
            netp = os.path.join(TMP, name + ".msnhnet")
            binp = os.path.join(TMP, name + ".msnhbin")
            with open(netp, "w") as f:
                f.write(text)
            try:
                w, (b, c, h, wd) = seeded_weights_for(netp, seed)
            except Exception as e:                                   # the host library refuses the graph (at this size)
                err = "host: " + str(e)
                continue
            w.tofile(binp)
            x = zoo.seeded_input(1, c, h, wd, seed + 1)[0]
            t0 = time.time()
            try:
                r = refshim.RefNet(netp, binp, scalar=True)
                outs = r.run(x)
            except refshim.RefError as e:
                err = "reference: " + str(e)
                continue
            dt = time.time() - t0
            store[f"{name}/graph"] = np.frombuffer(zlib.compress(text.encode(), 9), np.uint8)
            store[f"{name}/seed"] = np.array([seed, b, c, h, wd], np.int64)
            store[f"{name}/stats"] = np.stack([layer_stats(o) for o in outs])
            final = outs[-1] if outs[-1].size else outs[-2]
            store[f"{name}/final"] = final if final.size <= 4096 else final[(np.arange(4096, dtype=np.int64) * 7919) % final.size]
            store[f"{name}/final_size"] = np.array([final.size], np.int64)
            store[f"{name}/boxes"] = r.boxes()
            store[f"{name}/types"] = np.frombuffer("\n".join(r.layer_info(i)["type"] for i in range(r.num_layers())).encode(), np.uint8)
            print(f"{name:28s} {c}x{h}x{wd} weights {w.size:10d} reference forward {dt:6.2f} s boxes {len(r.boxes())}", flush=True)
            r.close()
            done = True
            break
        if not done:
            store[f"{name}/error"] = np.frombuffer(err.encode(), np.uint8)
        if f"{name}/error" in store:
            print(f"{name:28s} NOT RUN: {bytes(store[f'{name}/error']).decode()[:120]}", flush=True)
        names.append(name)
    store["names"] = np.frombuffer("\n".join(names).encode(), np.uint8)
    np.savez_compressed(OUT, **store)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
