"""TEST INFRASTRUCTURE.  Writes tests/golden/yolov4_608_candidates.npz from the reference's CPU forward (oracle/_ref, scalar mode) on
the first and the last image of the YOLOv4-608 benchmark batch (weights seed 5, input seed 6), which takes minutes per image and
so cannot run inside the GPU tests.  Per slot:

  rows        the reference's candidates before sorting, [n, 8] = x y w h objectness, best class score, class, cell (scan order)
  boxes       what YoloOutLayer returned, [m, 7], in its order
  obj_logits  the objectness logit of every cell (22743 floats), cells in scan order
  near        per candidate, bit c set when the logit of channel c (0 x .. 4 objectness, 5+j class j) lies within
              2e-2 * max|head logits| + 90 of zero, i.e. where a float16 error inside the tolerance can move the decoded value across a
              jump of the decode (the logistic's step at these magnitudes, the range where exp is finite); packed with numpy.packbits
  absmax      max|logit| per head

Run in the build container: python tests/golden/make_yolov4_candidates.py
"""
import os
import sys
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)
import netutil as nu  # noqa: E402
import refshim  # noqa: E402
from msnhnet_amd import zoo  # noqa: E402

OUT = os.path.join(ROOT, "tests", "golden", "yolov4_608_candidates.npz")
NEAR_REL, NEAR_ABS = 2e-2, 90.0


def main():
    tmp = tempfile.mkdtemp(prefix="msnh_gold_")
    netp, binp, gw = zoo.write_model("yolov4", tmp, 1, 608, seed=5)
    xs = zoo.seeded_input(16, 3, 608, 608, 6)
    r = refshim.RefNet(netp, binp, scalar=True)
    yolo = [i for i in range(r.num_layers()) if r.layer_info(i)["type"] == "yolo"]
    per = r.layer_info(yolo[0])["outC"] // 3
    store = {"per": np.array([per], np.int64), "near_rel_abs": np.array([NEAR_REL, NEAR_ABS])}
    for slot in (0, 15):
        outs = r.run(xs[slot])
        rows = nu.yolo_scan([outs[i] for i in yolo], per, 0.5)
        logits, head = nu.head_logits_by_cell([outs[i - 1] for i in yolo], per)
        absmax = np.array([np.abs(outs[i - 1]).max() for i in yolo], np.float64)
        cells = rows[:, 7].astype(np.int64)
        near = np.abs(logits[cells]) <= (NEAR_REL * absmax[head[cells]] + NEAR_ABS)[:, None]
        key = f"slot{slot}"
        store[f"{key}/rows"] = rows
        store[f"{key}/boxes"] = r.boxes()
        store[f"{key}/obj_logits"] = logits[:, 4].astype(np.float32)
        store[f"{key}/near"] = np.packbits(near, axis=1)
        store[f"{key}/absmax"] = absmax
        print("slot", slot, "candidates", len(rows), "boxes", len(store[f"{key}/boxes"]), "near bits", int(near.sum()), "wall ms", r.wall_ms(), flush=True)
    r.close()
    np.savez_compressed(OUT, **store)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
