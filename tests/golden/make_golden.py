"""Writes tests/golden/ref_golden.npz from the reference's own CPU forward (oracle/_ref, scalar mode).

Run in a container that holds the reference sources and the built oracle/_ref library:
    python tests/golden/make_golden.py
Only data is stored: graph text written by msnhnet_amd.zoo (our own emitter), seeded weights / inputs for the small
cases, and the reference's outputs -- whole tensors for the micro cases, per-layer statistics plus the final
logits / boxes for the five benchmark architectures at reduced size, and the per-layer shape tables at full size.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "tests"), os.path.join(ROOT, "oracle")):
    sys.path.insert(0, p)

import refshim  # noqa: E402
from msnhnet_amd import zoo  # noqa: E402

OUT = os.path.join(HERE, "ref_golden.npz")
TMP = "/tmp/msnh_golden"
os.makedirs(TMP, exist_ok=True)


PREPROC_CASES = [(40, 56, 32, 24, 11), (31, 20, 40, 40, 12), (24, 24, 24, 24, 13)]
LETTERBOX_CASES = [(48, 64, 40, 40, 1), (70, 50, 64, 64, 2), (30, 30, 52, 52, 3), (36, 36, 36, 36, 4)]


def layer_stats(a):
    a = np.asarray(a, np.float64)
    fin = np.isfinite(a)
    v = a[fin]
    idx = (np.arange(16) * 7919) % max(a.size, 1)
    return np.array([a.size, fin.sum(), v.sum() if v.size else 0, np.abs(v).sum() if v.size else 0, v.max() if v.size else 0,
                     v.min() if v.size else 0] + [a[i] if a.size else 0 for i in idx], np.float64)


def micro_cases():
    """(name, graph builder) -- one or two layers each, geometry chosen to hit every branch of the ops."""
    def g(c, h, w, fn):
        gw = zoo.GraphWriter(1, c, h, w)
        fn(gw)
        return gw
    cases = {
        "conv_k1": lambda: g(8, 7, 9, lambda q: q.conv(12, 1, 1, 0, bn=0, act="none")),
        "conv_k3_p1_leaky_bn": lambda: g(6, 11, 10, lambda q: q.conv(10, 3, 1, 1, bn=1, act="leaky")),
        "conv_k3_s2": lambda: g(5, 13, 12, lambda q: q.conv(7, 3, 2, 1, bn=0, act="relu")),
        "conv_k5_p2_mish": lambda: g(4, 9, 9, lambda q: q.conv(6, 5, 1, 2, bn=1, act="mish")),
        "conv_k7_s2_p3": lambda: g(3, 20, 18, lambda q: q.conv(8, 7, 2, 3, bn=0, bias=False, act="none")),
        "conv_groups2": lambda: g(8, 8, 8, lambda q: q.conv(12, 3, 1, 1, groups=2, bn=0, act="relu6")),
        "conv_depthwise_s2": lambda: g(10, 9, 11, lambda q: q.conv(10, 3, 2, 1, groups=10, bn=1, act="relu6")),
        "conv_nobias": lambda: g(4, 6, 6, lambda q: q.conv(5, 3, 1, 0, bn=0, bias=False, act="swish")),
        "bn_relu": lambda: g(6, 5, 7, lambda q: (q.conv(6, 1, 1, 0, bn=0, bias=False, act="none"), q.batchnorm("relu"))),
        "maxpool_k2s2": lambda: g(4, 8, 10, lambda q: (q.conv(4, 1, 1, 0, bn=0, act="none"), q.maxpool(2, 2, 0))),
        "maxpool_k3s2p1": lambda: g(4, 9, 11, lambda q: (q.conv(4, 1, 1, 0, bn=0, act="none"), q.maxpool(3, 2, 1))),
        "maxpool_k5s1p2": lambda: g(3, 7, 7, lambda q: (q.conv(3, 1, 1, 0, bn=0, act="none"), q.maxpool(5, 1, 2))),
        "avgpool_k3s2p1": lambda: g(3, 9, 9, lambda q: (q.conv(3, 1, 1, 0, bn=0, act="none"), q.localavgpool(3, 2, 1))),
        "avgpool_k7_fc": lambda: g(3, 7, 7, lambda q: (q.conv(16, 1, 1, 0, bn=0, act="relu"), q.localavgpool(7), q.connect(10))),
        "upsample_route": lambda: g(4, 5, 6, lambda q: (q.conv(6, 3, 1, 1, bn=1, act="leaky"), q.conv(4, 1, 1, 0, bn=1, act="leaky"),
                                                      q.upsample(2), q.conv(6, 3, 2, 1, bn=0, act="none"), q.route([-1, 0]))),
        "resblock": lambda: g(6, 6, 6, lambda q: (q.conv(8, 1, 1, 0, bn=1, act="leaky"),
                                                 q.resblock(2, lambda: (q.conv_node(4, 1, 1, 0, act="leaky"), q.conv_node(8, 3, 1, 1, act="leaky")), "relu"))),
        # (a block as the very first layer crashes the reference: its workspace is sized from top-level convs only)
        "res2block": lambda: g(4, 8, 8, lambda q: (q.conv(4, 3, 1, 1, bn=0, act="relu"),
                                                  q.res2block(lambda: (q.conv_node(6, 3, 2, 1, act="relu"), q.conv_node(6, 3, 1, 1, act="none")),
                                                              lambda: q.conv_node(6, 1, 2, 0, act="none"), "relu"))),
        "addblock_identity": lambda: g(6, 5, 5, lambda q: (q.conv(6, 1, 1, 0, bn=1, act="mish"),
                                                          q.addblock(2, [lambda: (q.conv_node(3, 1, 1, 0, act="mish"), q.conv_node(6, 3, 1, 1, act="mish")), None]))),
        # (the reference sizes its ping-pong pools from sub-layer outputs only, so the concat result must not be the
        #  largest tensor of the net: a wide conv in front keeps it from overrunning the pool)
        "concatblock_spp": lambda: g(4, 9, 9, lambda q: (q.conv(32, 1, 1, 0, bn=1, act="leaky"), q.conv(8, 1, 1, 0, bn=1, act="leaky"),
                                                        q.concatblock([lambda: q.maxpool_node(5, 1, 2), lambda: q.maxpool_node(3, 1, 1), None]))),
        # ---- layer types of the other shipped graphs --------------------------------------------------------------
        "conv_hardswish": lambda: g(6, 7, 8, lambda q: q.conv(9, 3, 1, 1, bn=1, act="hardswish")),
        "act_after_bn": lambda: g(5, 8, 8, lambda q: (q.conv(8, 3, 1, 1, bn=0, act="none"), q.batchnorm("none"), q.act("hardswish"),
                                                      q.maxpool(2, 2, 0), q.act("leaky"))),
        "padding_then_pool": lambda: g(4, 7, 9, lambda q: (q.conv(8, 3, 1, 1, bn=1, act="leaky"), q.padding(0, 1, 0, 1, 0.0), q.maxpool(2, 1, 0))),
        "padding_first": lambda: g(3, 14, 12, lambda q: (q.padding(3, 3, 3, 3, 0.0), q.conv(8, 7, 2, 0, bn=0, act="relu"), q.padding(1, 0, 2, 1, -1.5))),
        "route_add": lambda: g(4, 6, 6, lambda q: (q.conv(8, 3, 1, 1, bn=1, act="leaky"), q.conv(8, 1, 1, 0, bn=1, act="none"),
                                                   q.conv(8, 3, 1, 1, bn=1, act="none"), q.route([-1, -3], add_model=True),
                                                   q.route([-1, 1, 0], add_model=True, act="relu"))),
        "varop": lambda: g(4, 5, 7, lambda q: (q.conv(6, 3, 1, 1, bn=0, act="none"), q.conv(6, 1, 1, 0, bn=0, act="relu"), q.varop("add", [0]),
                                               q.act("relu"), q.varop("sub", [0, 1]), q.varop("subInv", [0]), q.varop("mulConst", None, 0.75),
                                               q.varop("subConstInv", None, 2.0), q.varop("addConst", None, -0.5))),
        "slice_focus": lambda: g(3, 10, 12, lambda q: (q.act("none"), q.slice(0, 1, 0, 2, 0, 2), q.route([-2]), q.slice(0, 1, 1, 2, 0, 2),
                                                       q.route([-4]), q.slice(0, 1, 0, 2, 1, 2), q.route([-6]), q.slice(0, 1, 1, 2, 1, 2),
                                                       q.route([-7, -5, -3, -1]), q.conv(8, 3, 1, 1, bn=1, act="hardswish"))),
        "slice_channels": lambda: g(3, 6, 6, lambda q: (q.conv(10, 1, 1, 0, bn=0, act="none"), q.slice(1, 3, 1, 1, 2, 3))),
        "globalavg_fc_softmax": lambda: g(3, 6, 5, lambda q: (q.conv(12, 3, 1, 1, bn=0, act="relu"), q.globalavgpool(), q.connect(7), q.softmax())),
        "softmax_map": lambda: g(3, 5, 6, lambda q: (q.conv(2, 3, 1, 1, bn=0, act="none"), q.softmax(2.0))),
        "bilinear_x2": lambda: g(3, 5, 6, lambda q: (q.conv(6, 3, 1, 1, bn=0, act="none"), q.upsample_bilinear(2.0, 2.0, 0))),
        "bilinear_align": lambda: g(3, 6, 4, lambda q: (q.conv(6, 1, 1, 0, bn=0, act="none"), q.upsample_bilinear(2.5, 1.5, 1))),
        "deconv_k2s2": lambda: g(6, 5, 7, lambda q: (q.conv(8, 3, 1, 1, bn=1, act="relu"), q.deconv(8, 2, 2, 0, act="relu"), q.batchnorm("none"),
                                                     q.conv(8, 3, 2, 1, bn=0, act="none"), q.route([-1, 0], add_model=True))),
        "deconv_k3s2p1": lambda: g(4, 6, 5, lambda q: (q.conv(8, 1, 1, 0, bn=0, act="none"), q.deconv(5, 3, 2, 1, act="leaky"))),
        "deconv_k4s2p1_nobias": lambda: g(3, 4, 6, lambda q: (q.conv(16, 3, 1, 1, bn=0, act="relu"), q.deconv(8, 4, 2, 1, bias=False, act="none"))),
        "yolo5_head": lambda: g(8, 6, 6, lambda q: (q.conv(21, 1, 1, 0, bn=0, act="none"), q.yolo([10, 13, 16, 30, 33, 23], class_num=2, yolo_type="yolov5"),
                                                   q.yoloout([1], 0.3, 0.45, yolo_type="yolov5"))),
        "yolo_head": lambda: g(8, 6, 6, lambda q: (q.conv(21, 1, 1, 0, bn=0, act="none"), q.yolo([10, 13, 16, 30, 33, 23], class_num=2),
                                                  q.yoloout([1], 0.3, 0.45))),
        # a subtraction whose minuend / subtrahend is a convolution nobody else reads (the add moves into that convolution's launch
        # where the arithmetic allows it): previous layer - layer 0, layer 0 - previous layer, layer 0 - layer 2
        "varop_sub_conv": lambda: g(4, 6, 7, lambda q: (q.conv(6, 3, 1, 1, bn=0, act="none"), q.conv(6, 1, 1, 0, bn=0, act="relu"),
                                                       q.conv(6, 3, 1, 1, bn=1, act="leaky"), q.varop("sub", [0]), q.act("relu"))),
        "varop_subinv_conv": lambda: g(4, 6, 7, lambda q: (q.conv(6, 3, 1, 1, bn=0, act="none"), q.conv(6, 1, 1, 0, bn=0, act="relu"),
                                                          q.conv(6, 3, 1, 1, bn=1, act="leaky"), q.varop("subInv", [0]), q.act("relu"))),
        "varop_sub_conv_second": lambda: g(4, 6, 7, lambda q: (q.conv(6, 3, 1, 1, bn=0, act="none"), q.conv(6, 1, 1, 0, bn=0, act="relu"),
                                                              q.conv(6, 3, 1, 1, bn=1, act="leaky"), q.conv(6, 1, 1, 0, bn=0, act="none"),
                                                              q.varop("sub", [0, 2]))),
    }
    return cases


def main():
    if not refshim.available():
        sys.exit("oracle/_ref/libmsnh_ref.so is missing: run `make -C oracle ref` where the reference sources are present")
    store = {}
    names = []
    for name, build in micro_cases().items():
        gw = build()
        netp = os.path.join(TMP, name + ".msnhnet")
        binp = os.path.join(TMP, name + ".msnhbin")
        with open(netp, "w") as f:
            f.write(gw.text())
        seed = 100 + len(names)
        w = zoo.seeded_weights(gw.slots, seed)
        w.tofile(binp)
        c, h, wd = None, None, None
        r = refshim.RefNet(netp, binp, scalar=True)
        c0 = int(gw.text().split("channels:")[1].split()[0]); h0 = int(gw.text().split("height:")[1].split()[0]); w0 = int(gw.text().split("width:")[1].split()[0])
        x = zoo.seeded_input(1, c0, h0, w0, seed + 1)[0]
        if name in ("yolo_head", "yolo5_head"):
            x = (x - 0.5) * 8          # spread the logits so some boxes pass the threshold and some do not
        outs = r.run(x)
        store[f"micro/{name}/graph"] = np.frombuffer(gw.text().encode(), np.uint8)
        store[f"micro/{name}/weights"] = w
        store[f"micro/{name}/input"] = x.astype(np.float32)
        for i, o in enumerate(outs):
            store[f"micro/{name}/out{i}"] = o
        store[f"micro/{name}/boxes"] = r.boxes()
        names.append(name)
        r.close()
    store["micro/names"] = np.frombuffer("\n".join(names).encode(), np.uint8)

    for arch, size in (("resnet18", 224), ("resnet50", 224), ("mobilenetv2", 224), ("yolov3", 96), ("yolov4", 96)):
        netp, binp, gw = zoo.write_model(arch, TMP, 1, size, seed=11)
        x = zoo.seeded_input(1, 3, size, size, 12)[0]
        r = refshim.RefNet(netp, binp, scalar=True)
        outs = r.run(x)
        store[f"net/{arch}/size"] = np.array([size])
        store[f"net/{arch}/stats"] = np.stack([layer_stats(o) for o in outs])
        store[f"net/{arch}/final"] = outs[-1] if outs[-1].size else outs[-2]
        store[f"net/{arch}/boxes"] = r.boxes()
        store[f"net/{arch}/input_sum"] = np.array([np.float64(x.astype(np.float64).sum())])
        store[f"net/{arch}/weights_sum"] = np.array([np.float64(np.fromfile(binp, np.float32).astype(np.float64).sum())])
        r.close()

    # YOLOv4 at its full benchmark size: 70 s per image on the scalar build, so the GPU tests cannot run the reference there.  First and
    # last image of the batch of 16 the full-size test feeds (weights seed 5, input seed 6): per-layer statistics, samples of the three
    # head logit tensors, and the boxes (count, class histogram, every 8th box of the sorted list).
    netp, binp, gw = zoo.write_model("yolov4", TMP, 1, 608, seed=5)
    xs = zoo.seeded_input(16, 3, 608, 608, 6)
    r = refshim.RefNet(netp, binp, scalar=True)
    heads = [i - 1 for i in range(r.num_layers()) if r.layer_info(i)["type"] == "yolo"]
    for slot in (0, 15):
        outs = r.run(xs[slot])
        key = f"full/yolov4/slot{slot}"
        store[f"{key}/stats"] = np.stack([layer_stats(o) for o in outs])
        for k, li in enumerate(heads):
            idx = (np.arange(4096, dtype=np.int64) * 104729) % outs[li].size
            store[f"{key}/head{k}_idx"] = idx
            store[f"{key}/head{k}_val"] = outs[li][idx]
            store[f"{key}/head{k}_absmax"] = np.array([np.abs(outs[li]).max()], np.float64)
        b = r.boxes()
        key7 = np.nan_to_num(b, nan=1e30, posinf=2e30, neginf=-2e30)
        b = b[np.lexsort(key7.T[::-1])] if len(b) else b
        store[f"{key}/box_count"] = np.array([len(b)], np.int64)
        store[f"{key}/class_hist"] = np.bincount(b[:, 6].astype(np.int64), minlength=80) if len(b) else np.zeros(80, np.int64)
        store[f"{key}/boxes_every8"] = b[::8]
        print("yolov4-608 slot", slot, "boxes", len(b), "wall ms", r.wall_ms(), flush=True)
    store["full/yolov4/heads"] = np.array(heads, np.int64)
    r.close()

    # full-size shape tables and the reference's own layer-detail text
    for arch, dtype, batch, size in zoo.CONFIGS:
        gw = zoo.ARCHS[arch](batch=1, size=size)
        netp = os.path.join(TMP, f"{arch}_full.msnhnet")
        with open(netp, "w") as f:
            f.write(gw.text())
        r = refshim.RefNet(netp)
        infos = r.layer_infos()
        keys = ["outH", "outW", "outC", "outputNum", "inputNum", "numWeights"]
        store[f"shape/{arch}/table"] = np.array([[i[k] for k in keys] for i in infos], np.int64)
        store[f"shape/{arch}/types"] = np.frombuffer("\n".join(i["type"] for i in infos).encode(), np.uint8)
        store[f"shape/{arch}/detail"] = np.frombuffer(r.detail().encode(), np.uint8)
        r.close()
    # pre / post-processing around the graph: CVUtil::getPaddingZeroF32C3 on seeded 8-bit images (stored as the 8-bit
    # values it scales, i.e. round(out * 255)), YoloOutLayer::bboxResize2Org[NoPad] on seeded boxes
    for idx, (h, w, nw, nh, seed) in enumerate(LETTERBOX_CASES):
        img = np.random.default_rng(seed).integers(0, 256, (h, w, 3), dtype=np.uint8)
        for shuffle in (0, 1):
            out = refshim.letterbox_u8(img, nw, nh, False, bool(shuffle))
            store[f"letterbox/{idx}/shuffle{shuffle}"] = np.rint(out * 255.0).astype(np.uint8)
        store[f"letterbox/{idx}/case"] = np.array([h, w, nw, nh, seed], np.int64)
    # the plain-resize variants (CVUtil::getImgDataF32C3, getGoogLenetF32C3, getTransformedF32C3, getCaffeModeF32C3)
    for idx, (h, w, nw, nh, seed) in enumerate(PREPROC_CASES):
        img = np.random.default_rng(seed).integers(0, 256, (h, w, 3), dtype=np.uint8)
        mean, std = np.array([0.4, 0.5, 0.6], np.float32), np.array([0.2, 0.3, 0.25], np.float32)
        for kind in refshim.PREPROC_KINDS:
            store[f"preproc/{idx}/{kind}"] = refshim.preproc_u8(img, nw, nh, kind, mean, std, bool(idx % 2))
        store[f"preproc/{idx}/case"] = np.array([h, w, nw, nh, seed], np.int64)
        store[f"preproc/{idx}/mean"] = mean
        store[f"preproc/{idx}/std"] = std
    rng = np.random.default_rng(77)
    rows = []
    for _ in range(40):
        box = rng.uniform(0, 600, 4).astype(np.float32)
        cw, ch, ow, oh = (int(v) for v in rng.integers(32, 2000, 4))
        rows.append(np.concatenate([box, [cw, ch, ow, oh], refshim.bbox_resize2org(box, cw, ch, ow, oh, False),
                                    refshim.bbox_resize2org(box, cw, ch, ow, oh, True)]).astype(np.float64))
    store["bbox/rows"] = np.array(rows)
    np.savez_compressed(OUT, **store)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(store), "arrays")


if __name__ == "__main__":
    main()
