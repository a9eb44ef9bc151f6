"""End-to-end GPU parity through the host library's C ABI (NetBuilder build / load / runClassifyGPU / runYoloGPU)
against the reference's own CPU forward (oracle/_ref, scalar mode) when it is present, else the plain-C oracle.

Tolerances (max|a-b| / max|ref| per layer output):
  float32: 1e-4 on every top-level layer output (the reference's own FMA-contracted build and its plain-C
           restatement already differ by up to 1.7e-4 on the deepest MobileNetV2 layers, so those use 5e-4;
           decoded yolo layers are compared in units of the logit error that explains them, see netutil.yolo_layer_err);
  float16: 2e-2 on the final logits / boxes; class indices and box counts are compared exactly where the margin
           of the reference result is larger than the float16 error.
"""
import numpy as np
import pytest
import torch

import msnh_oracle_net as on
import netutil as nu
import refshim
from msnhnet_amd import netapi, zoo

pytestmark = pytest.mark.gpu


def _oracle_layers(arch, size, binp, imgs, **kw):
    """Per-image per-layer outputs from the reference (scalar mode) or, without it, the plain-C oracle."""
    path = nu.batch1_graph(arch, size, **kw)
    outs, boxes = [], []
    if refshim.available():
        r = refshim.RefNet(path, binp, scalar=True)
        for x in imgs:
            outs.append(r.run(x))
            boxes.append(r.boxes())
    else:
        o = on.OracleNet(path, binp)
        for x in imgs:
            outs.append([v.ravel() for v in o.run(x)])
            boxes.append(o.boxes if o.boxes is not None else np.zeros((0, 7), np.float32))
    return outs, boxes


SMALL = [("resnet18", 64, 2), ("resnet50", 64, 2), ("mobilenetv2", 64, 3), ("yolov3", 64, 2), ("yolov4", 64, 2), ("yolov3_tiny", 96, 2),
         ("yolov5s", 64, 2)]


@pytest.mark.parametrize("arch,size,batch", SMALL)
def test_fp32_every_layer(arch, size, batch):
    if arch in ("resnet18", "resnet50", "mobilenetv2"):
        size = 224            # the 7x7 average pool needs the full-size feature map
    net, binp, g = nu.model(arch, batch, size, seed=3)
    x = zoo.seeded_input(batch, 3, size, size, seed=4)
    ref, ref_boxes = _oracle_layers(arch, size, binp, x)
    print("running", arch, size, batch, flush=True)
    m = netapi.Net(net, binp, fp16=False, dump_layers=True)
    if arch.startswith("yolo"):
        boxes = m.run_yolo(x)
    else:
        logits = m.run_classify(x)
    n_layers = m.num_layers()
    assert n_layers == len(ref[0])
    tol = 5e-4 if arch == "mobilenetv2" else 1e-4
    worst = 0.0
    for i in range(n_layers):
        if m.layer_info(i)["type"] == "yoloout":
            continue
        got = m.layer_output(i).reshape(batch, -1)
        is_yolo = m.layer_info(i)["type"] == "yolo"
        lt = tol
        for b in range(batch):
            e = (nu.yolo_layer_err(got[b], ref[b][i], ref[b][i - 1], 85, size / m.layer_info(i)['outH'], 5 if arch == "yolov5s" else 3)
                 if is_yolo else nu.rel_err(got[b], ref[b][i]))
            worst = max(worst, e)
            assert e <= lt, f"{arch} layer {i} ({m.layer_info(i)['type']}) image {b}: {e}"
    print(arch, "worst layer error", worst)
    if arch.startswith("yolo"):
        for b in range(batch):
            rb, gb = nu.sort_boxes(ref_boxes[b]), nu.sort_boxes(boxes[b])
            assert len(rb) == len(gb), f"box count {len(gb)} vs {len(rb)}"
            assert np.array_equal(rb[:, 6], gb[:, 6])
            assert nu.rel_err(gb[:, :6], rb[:, :6]) <= 1e-4
    else:
        for b in range(batch):
            assert int(np.argmax(logits[b])) == int(np.argmax(ref[b][-1]))


@pytest.mark.parametrize("arch,size,batch", SMALL)
def test_fused_graph_equals_layer_by_layer(arch, size, batch):
    """The production path (fused launches, aliased concats, captured graph) must give what the dump path gives."""
    if arch in ("resnet18", "resnet50", "mobilenetv2"):
        size = 224
    net, binp, g = nu.model(arch, batch, size, seed=3)
    x = zoo.seeded_input(batch, 3, size, size, seed=4)
    slow = netapi.Net(net, binp, fp16=False, dump_layers=True)
    fast = netapi.Net(net, binp, fp16=False, dump_layers=False)
    if arch.startswith("yolo"):
        a, b1, b2 = slow.run_yolo(x), fast.run_yolo(x), fast.run_yolo(x)      # second call replays the graph
        for i in range(batch):
            for got in (b1[i], b2[i]):
                assert len(got) == len(a[i])
                assert nu.rel_err(nu.sort_boxes(got)[:, :6], nu.sort_boxes(a[i])[:, :6]) <= 1e-5
    else:
        a, b1, b2 = slow.run_classify(x), fast.run_classify(x), fast.run_classify(x)
        assert nu.rel_err(b1, a) <= 1e-5 and np.array_equal(b1, b2)


@pytest.mark.parametrize("arch,size,batch", SMALL)
def test_fp16_final_outputs(arch, size, batch):
    if arch in ("resnet18", "resnet50", "mobilenetv2"):
        size = 224
    net, binp, g = nu.model(arch, batch, size, seed=3)
    x = zoo.seeded_input(batch, 3, size, size, seed=4)
    ref, ref_boxes = _oracle_layers(arch, size, binp, x)
    print("running fp16", arch, size, batch, flush=True)
    m = netapi.Net(net, binp, fp16=True, dump_layers=True)
    if arch.startswith("yolo"):
        netapi.set_device_nms(0)                # sort + NMS on the host: the candidate rows come to the host with the result
        try:
            boxes = m.run_yolo(x)
            rows = [m.yolo_candidates(b) for b in range(batch)]
        finally:
            netapi.set_device_nms(1)
        # final logits = inputs of the yolo layers
        yolo = [i for i in range(m.num_layers()) if m.layer_info(i)["type"] == "yolo"]
        per = m.layer_info(yolo[0])["outC"] // 3
        conf_t, nms_t = nu.thresholds(arch)
        logits = [m.layer_output(i - 1).reshape(batch, -1) for i in yolo]
        for k, i in enumerate(yolo):
            for b in range(batch):
                e = nu.rel_err(logits[k][b], ref[b][i - 1])
                assert e <= 2e-2, f"{arch} head logits before layer {i}, image {b}: {e}"
        for b in range(batch):
            # every candidate that differs from the reference's -- present on one side only, or a row beyond 2e-2 -- sits on a reference
            # logit no farther from a jump of the decode than the measured float16 error of its head; the box count differs by no more
            # than the number of such cells; and the boxes are the reference's NMS of the returned candidates
            ref_rows, only_dev, only_ref, differing, herr = nu.attribute_against_reference(
                rows[b], [l[b] for l in logits], [ref[b][i] for i in yolo], [ref[b][i - 1] for i in yolo], per, conf_t)
            attributed = len(only_dev) + len(only_ref) + len(differing)
            print(f"{arch} image {b}: candidates {len(rows[b])} reference {len(ref_rows)}, attributed cells {attributed}, boxes {len(boxes[b])} reference {len(ref_boxes[b])}", flush=True)
            assert abs(len(boxes[b]) - len(ref_boxes[b])) <= attributed
            assert nu.same_box_set(netapi.boxes_from_candidates(rows[b], nms_t, fast=False), boxes[b])
            nu.box_sets_equal_up_to_ties(netapi.boxes_from_candidates(ref_rows, nms_t, fast=True), ref_boxes[b], nms_t)
    else:
        logits = m.run_classify(x)
        for b in range(batch):
            r = ref[b][-1]
            assert nu.rel_err(logits[b], r) <= 2e-2
            top2 = np.sort(r)[-2:]
            if top2[1] - top2[0] > 4e-2 * np.abs(r).max():
                assert int(np.argmax(logits[b])) == int(np.argmax(r))


@pytest.mark.parametrize("arch,size,batch", [("resnet18", 224, 2), ("yolov3", 160, 2)])
def test_fp16_headroom_and_hot_input(arch, size, batch):
    """The float16 scales are fixed at load from one calibration image in [0,1).  An input 4x hotter than that must still be inside
    the tolerance, the range check must report how much room is left, and it must report 0 once an input has overflowed."""
    net, binp, g = nu.model(arch, batch, size, seed=3)
    x = zoo.seeded_input(batch, 3, size, size, seed=4)
    m = netapi.Net(net, binp, fp16=True, dump_layers=True)
    h1 = m.fp16_headroom(x)
    h4 = m.fp16_headroom(4.0 * x)
    print(arch, "headroom on the [0,1) input", h1, "on the 4x input", h4, flush=True)
    assert h1 >= 8.0 and h4 >= 2.0 and h4 < h1
    hot = (4.0 * x).astype(np.float32)
    ref, ref_boxes = _oracle_layers(arch, size, binp, hot)
    if arch.startswith("yolo"):
        boxes = m.run_yolo(hot)
        for i in range(m.num_layers()):
            if m.layer_info(i)["type"] != "yolo":
                continue
            got = m.layer_output(i - 1).reshape(batch, -1)
            for b in range(batch):
                assert nu.rel_err(got[b], ref[b][i - 1]) <= 2e-2
        for b in range(batch):
            assert abs(len(boxes[b]) - len(ref_boxes[b])) <= max(2, 0.02 * len(ref_boxes[b]))
    else:
        logits = m.run_classify(hot)
        for b in range(batch):
            assert nu.rel_err(logits[b], ref[b][-1]) <= 2e-2
    assert m.fp16_headroom(4096.0 * x) < 1.0
    assert netapi.Net(net, binp, fp16=False).fp16_headroom(4096.0 * x) == float("inf")


import os
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_golden.npz"))
MICRO = bytes(GOLD["micro/names"]).decode().split("\n")


@pytest.mark.parametrize("fp16", [False, True])
@pytest.mark.parametrize("name", MICRO)
def test_micro_graphs_against_reference_golden(name, fp16, tmp_path):
    """Every micro graph of the golden file (one per op / block / layer type, outputs written by the reference's own CPU
    forward) through NetBuilder on the device: every layer output in float32 to 1e-4, in float16 to 2e-2 of the layer's range;
    boxes of the yolo heads as sets."""
    text = bytes(GOLD[f"micro/{name}/graph"]).decode()
    netp = str(tmp_path / (name + ".msnhnet"))
    binp = str(tmp_path / (name + ".msnhbin"))
    with open(netp, "w") as f:
        f.write(text)
    np.asarray(GOLD[f"micro/{name}/weights"], np.float32).tofile(binp)
    x = GOLD[f"micro/{name}/input"][None]
    print("running micro", name, "fp16" if fp16 else "fp32", flush=True)
    m = netapi.Net(netp, binp, fp16=fp16, dump_layers=True)
    is_yolo = any(m.layer_info(i)["type"] == "yoloout" for i in range(m.num_layers()))
    boxes = m.run_yolo(x) if is_yolo else None
    if not is_yolo:
        m.run_classify(x)
    tol = 2e-2 if fp16 else 1e-4
    for i in range(m.num_layers()):
        ref = GOLD[f"micro/{name}/out{i}"]
        t = m.layer_info(i)["type"]
        if ref.size == 0 or t == "yoloout" or (fp16 and t == "yolo"):
            continue
        got = m.layer_output(i).ravel()
        assert got.size == ref.size, (name, i, t, got.size, ref.size)
        assert nu.rel_err(got, ref) <= tol, (name, i, t, nu.rel_err(got, ref))
    if is_yolo and not fp16:
        rb, gb = nu.sort_boxes(GOLD[f"micro/{name}/boxes"]), nu.sort_boxes(boxes[0])
        assert len(rb) == len(gb)
        assert nu.rel_err(gb[:, :6], rb[:, :6]) <= 1e-4
    # the production path (fused launches, captured graph) gives what the layer-by-layer path gave
    fast = netapi.Net(netp, binp, fp16=fp16, dump_layers=False)
    if is_yolo:
        fb = fast.run_yolo(x)
        if not fp16:
            assert len(fb[0]) == len(boxes[0])
    else:
        a, b = m.run_classify(x), fast.run_classify(x)
        assert nu.rel_err(b, a) <= (1e-5 if not fp16 else 2e-2)


@pytest.mark.parametrize("arch,size,batch", [("resnet18", 224, 1), ("yolov3", 224, 2)])
def test_fp16_winograd_network(arch, size, batch):
    """every 3x3 stride-1 convolution through Winograd F(2x2,3x3): same final outputs within the float16 tolerance"""
    net, binp, g = nu.model(arch, batch, size, seed=3)
    x = zoo.seeded_input(batch, 3, size, size, seed=4)
    ref, ref_boxes = _oracle_layers(arch, size, binp, x)
    print("running fp16 winograd", arch, size, batch, flush=True)
    netapi.set_use_winograd(True)
    try:
        m = netapi.Net(net, binp, fp16=True, dump_layers=True)
    finally:
        netapi.set_use_winograd(False)
    assert "winograd" in m.plan_detail()
    if arch.startswith("yolo"):
        boxes = m.run_yolo(x)
        for i in range(m.num_layers()):
            if m.layer_info(i)["type"] != "yolo":
                continue
            got = m.layer_output(i - 1).reshape(batch, -1)
            for b in range(batch):
                e = nu.rel_err(got[b], ref[b][i - 1])
                assert e <= 2e-2, f"{arch} head logits before layer {i}, image {b}: {e}"
        for b in range(batch):
            assert abs(len(boxes[b]) - len(ref_boxes[b])) <= max(2, 0.02 * len(ref_boxes[b]))
    else:
        logits = m.run_classify(x)
        for b in range(batch):
            assert nu.rel_err(logits[b], ref[b][-1]) <= 2e-2


def test_tune_cache(tmp_path):
    """the per-layer search result is kept beside the weights file when asked for: the next load takes the same choices
    from the file (same plan, bit-identical outputs), a file that does not fit is ignored and rewritten, and nothing is
    written unless the switch is on"""
    import shutil
    import time
    arch, size, batch = "yolov3", 96, 2
    net0, bin0, g = nu.model(arch, batch, size, seed=3)
    net, binp = str(tmp_path / "m.msnhnet"), str(tmp_path / "m.msnhbin")
    shutil.copy(net0, net)
    shutil.copy(bin0, binp)
    x = zoo.seeded_input(batch, 3, size, size, seed=4)
    cache = binp + ".f16.tune"
    netapi.Net(net, binp, fp16=True)
    assert not os.path.exists(cache) and not os.path.exists(binp + ".f32.tune")
    netapi.set_tune_cache(True)
    try:
        t0 = time.perf_counter()
        a = netapi.Net(net, binp, fp16=True)
        t1 = time.perf_counter()
        assert os.path.exists(cache)
        text = open(cache).read()
        lines = text.splitlines()
        assert lines[0].startswith("msnhtune 2 ") and lines[0].endswith(" winograd 0") and len(lines) > 10 and all(" | " in ln for ln in lines[1:])
        b = netapi.Net(net, binp, fp16=True)
        t2 = time.perf_counter()
        print(f"load with search {t1 - t0:.3f} s, from the file {t2 - t1:.3f} s", flush=True)
        assert b.plan_detail() == a.plan_detail()
        assert open(cache).read() == text
        ya, yb = a.run_yolo(x), b.run_yolo(x)
        for i in range(batch):
            assert np.array_equal(ya[i], yb[i])
        # a line that names another launch: the whole file is dropped, the search runs and writes a fresh one
        bad = lines[:]
        bad[3] = "9 " + bad[3]
        open(cache, "w").write("\n".join(bad) + "\n")
        c = netapi.Net(net, binp, fp16=True)
        fresh = open(cache).read().splitlines()
        assert [ln.split(" | ")[0] for ln in fresh] == [ln.split(" | ")[0] for ln in lines]
        yc = c.run_yolo(x)
        for i in range(batch):
            assert abs(len(yc[i]) - len(ya[i])) <= max(2, 0.02 * len(ya[i]))
        # a choice the library refuses for the launch (a tile number past the table): same
        bad = fresh[:]
        bad[2] = bad[2].split(" | ")[0] + " | 1 999"
        open(cache, "w").write("\n".join(bad) + "\n")
        netapi.Net(net, binp, fp16=True)
        assert " | 1 999" not in open(cache).read()
        # float32 plans keep their own file
        netapi.Net(net, binp, fp16=False)
        assert os.path.exists(binp + ".f32.tune")
        # a file written under the other Winograd preference is not applied: the weights on the device are packed for the algorithm
        # family chosen before the search, and a Winograd choice on tap-major weights (or the reverse) would read them wrongly
        plain = open(cache).read()
        netapi.set_use_winograd(True)
        try:
            w = netapi.Net(net, binp, fp16=True)
            wino = open(cache).read()
            assert wino.splitlines()[0].endswith(" winograd 1") and "winograd" in w.plan_detail()
            yw = w.run_yolo(x)
        finally:
            netapi.set_use_winograd(False)
        d = netapi.Net(net, binp, fp16=True)
        assert open(cache).read().splitlines()[0].endswith(" winograd 0") and "winograd" not in d.plan_detail()
        yd = d.run_yolo(x)
        for i in range(batch):
            assert abs(len(yd[i]) - len(ya[i])) <= max(2, 0.02 * len(ya[i])) and abs(len(yw[i]) - len(ya[i])) <= max(2, 0.02 * len(ya[i]))
        # the same header with a Winograd choice spliced into a plain file: refused line by line as well
        lines_d = open(cache).read().splitlines()
        k3 = next(i for i, ln in enumerate(lines_d[1:], 1) if ln.split()[8] == "3" and ln.split()[9] == "1")
        forged = lines_d[:]
        forged[k3] = forged[k3].split(" | ")[0] + " | 4 0"
        open(cache, "w").write("\n".join(forged) + "\n")
        e = netapi.Net(net, binp, fp16=True)
        assert "winograd" not in e.plan_detail() and " | 4 0" not in open(cache).read()
        del plain
    finally:
        netapi.set_tune_cache(False)


def test_first_pair_runs_as_one_launch():
    """float16 plans of the Darknet trunks run the first layer and the first stride-2 layer as one launch (the full-resolution tensor
    between them stays on the chip); float32 plans, layer-dump runs and networks that open differently keep their own launches; the
    results are those of the layer-by-layer run to float16 accuracy"""
    size, batch = 160, 2
    net, binp, g = nu.model("yolov3", batch, size, seed=3)
    x = zoo.seeded_input(batch, 3, size, size, seed=4)
    fused = netapi.Net(net, binp, fp16=True)
    assert "stem+down" in fused.plan_detail() and "conv[stem " not in fused.plan_detail()
    assert "stem+down" not in netapi.Net(net, binp, fp16=False).plan_detail()
    slow = netapi.Net(net, binp, fp16=True, dump_layers=True)
    assert "stem+down" not in slow.plan_detail() and "conv[stem " in slow.plan_detail()
    a, b = fused.run_yolo(x), slow.run_yolo(x)
    for i in range(batch):
        assert abs(len(a[i]) - len(b[i])) <= max(2, 0.02 * len(b[i]))
        assert nu.boxes_matched_fraction(a[i], b[i], 2e-2) >= 0.95
    r50, rbin, _ = nu.model("resnet50", 2, 224, seed=3)
    assert "stem+down" not in netapi.Net(r50, rbin, fp16=True).plan_detail()


def test_weight_cache(tmp_path):
    """the packed kernels and the float16 calibration are kept beside the weights file when asked for: the next load of the same
    weights into the same graph takes them from the file (same plan, bit-identical outputs, no calibration pass); other weights under
    the same name, another graph, a cut file or the other Winograd preference make the file count for nothing and it is rewritten"""
    import shutil
    arch, size, batch = "yolov3", 96, 2
    net0, bin0, g = nu.model(arch, batch, size, seed=3)
    net, binp = str(tmp_path / "m.msnhnet"), str(tmp_path / "m.msnhbin")
    shutil.copy(net0, net)
    shutil.copy(bin0, binp)
    x = zoo.seeded_input(batch, 3, size, size, seed=4)
    pack = binp + ".f16.pack"
    plain = netapi.Net(net, binp, fp16=True)
    assert not os.path.exists(pack) and plain.load_detail().endswith("pack file off")
    netapi.set_tune_cache(True)          # the same tiles on every load below, so that outputs can be compared bit for bit
    netapi.set_weight_cache(True)
    try:
        a = netapi.Net(net, binp, fp16=True)
        assert a.load_detail().endswith("pack file written") and os.path.exists(pack) and not [f for f in os.listdir(str(tmp_path)) if ".tmp" in f]
        blob = open(pack, "rb").read()
        assert blob.startswith(b"msnhpack 2 layout ") and b" winograd 0 dtype 1\n" in blob[:100] and len(blob) > os.path.getsize(binp) // 4
        b = netapi.Net(net, binp, fp16=True)
        print(a.load_detail(), b.load_detail(), sep="\n", flush=True)
        assert b.load_detail().endswith("pack file read") and open(pack, "rb").read() == blob
        assert b.plan_detail() == a.plan_detail()
        ya, yb = a.run_yolo(x), b.run_yolo(x)
        for i in range(batch):
            assert len(ya[i]) > 0 and np.array_equal(ya[i], yb[i])
        # other weights under the same name (same size): the hash in the file does not fit, the file is rewritten
        _, bin7, _ = nu.model(arch, batch, size, seed=7)
        shutil.copy(bin7, binp)
        c = netapi.Net(net, binp, fp16=True)
        assert c.load_detail().endswith("pack file written") and open(pack, "rb").read() != blob
        netapi.set_weight_cache(False)
        d = netapi.Net(net, binp, fp16=True)
        netapi.set_weight_cache(True)
        e = netapi.Net(net, binp, fp16=True)
        assert d.load_detail().endswith("pack file off") and e.load_detail().endswith("pack file read")
        yc, yd, ye = c.run_yolo(x), d.run_yolo(x), e.run_yolo(x)
        for i in range(batch):
            assert np.array_equal(yc[i], yd[i]) and np.array_equal(ye[i], yd[i])
            assert not np.array_equal(yc[i], ya[i])
        # a cut file
        blob = open(pack, "rb").read()
        open(pack, "wb").write(blob[:len(blob) // 2])
        f = netapi.Net(net, binp, fp16=True)
        assert f.load_detail().endswith("pack file written") and open(pack, "rb").read() == blob
        # one flipped bit inside a packed kernel: its checksum refuses the file
        bad = bytearray(blob)
        bad[len(bad) * 3 // 4] ^= 0x04
        open(pack, "wb").write(bytes(bad))
        f2 = netapi.Net(net, binp, fp16=True)
        assert f2.load_detail().endswith("pack file written") and open(pack, "rb").read() == blob
        # the same graph with another activation parameter (the float16 calibration depends on it): not this graph's file
        text = open(net).read()
        assert "leaky" in text
        net_slope = str(tmp_path / "m_slope.msnhnet")
        open(net_slope, "w").write(text.replace("activation: leaky", "activation: leaky,0.3"))
        f3 = netapi.Net(net_slope, binp, fp16=True)
        assert f3.load_detail().endswith("pack file written")
        f4 = netapi.Net(net, binp, fp16=True)
        assert f4.load_detail().endswith("pack file written")
        blob = open(pack, "rb").read()
        # the same weights in another graph (batch 1): not this plan's file
        g1 = zoo.ARCHS[arch](batch=1, size=size)
        net1 = str(tmp_path / "m1.msnhnet")
        open(net1, "w").write(g1.text())
        h = netapi.Net(net1, binp, fp16=True)
        assert h.load_detail().endswith("pack file written")
        y1 = h.run_yolo(x[:1])
        assert abs(len(y1[0]) - len(yd[0])) <= max(2, 0.02 * len(yd[0]))
        # float32 plans keep their own file; the Winograd preference is part of the first line
        k = netapi.Net(net, binp, fp16=False)
        assert k.load_detail().endswith("pack file written") and os.path.exists(binp + ".f32.pack")
        assert netapi.Net(net, binp, fp16=False).load_detail().endswith("pack file read")
        netapi.Net(net, binp, fp16=True)
        netapi.set_use_winograd(True)
        try:
            w = netapi.Net(net, binp, fp16=True)
            assert w.load_detail().endswith("pack file written") and b" winograd 1 " in open(pack, "rb").read()[:100]
            w2 = netapi.Net(net, binp, fp16=True)
            assert w2.load_detail().endswith("pack file read") and "winograd" in w2.plan_detail()
            yw, yw2 = w.run_yolo(x), w2.run_yolo(x)
            for i in range(batch):
                assert np.array_equal(yw[i], yw2[i])
        finally:
            netapi.set_use_winograd(False)
    finally:
        netapi.set_weight_cache(False)
        netapi.set_tune_cache(False)


@pytest.mark.parametrize("arch,size,batch", [("yolov3", 224, 3), ("yolov3_tiny", 160, 2), ("yolov5s", 128, 2), ("yolov3", 704, 1)])
def test_device_nms_equals_host_nms(arch, size, batch):
    """same network, same input: boxes from the device's NMS (the default) and from the host's sort + NMS are identical,
    eagerly and with two forwards in flight; the 704 x 704 case has a class with more than 5000 members in the image (the
    large-class kernel)"""
    net, binp, g = nu.model(arch, batch, size, seed=3)
    xs = [zoo.seeded_input(batch, 3, size, size, seed=s) for s in (4, 5, 6)]
    print("device nms", arch, size, batch, flush=True)
    m = netapi.Net(net, binp, fp16=True)
    try:
        netapi.set_device_nms(2)
        got = [m.run_yolo(x) for x in xs]
        netapi.set_device_nms(0)
        want = [m.run_yolo(x) for x in xs]
        netapi.set_device_nms(1)
        auto = [m.run_yolo(x) for x in xs]
        with pytest.raises(netapi.MsnhnetError):
            netapi.set_device_nms(3)
    finally:
        netapi.set_device_nms(1)
    got += auto
    want += want
    assert sum(len(b) for w in want for b in w) > 0
    if size == 704:
        for w in want[:3]:
            assert 5000 <= np.bincount(w[0][:, 6].astype(np.int64)).max() <= 6144
    for g_, w_ in zip(got, want):
        for b in range(batch):
            assert np.array_equal(g_[b], w_[b], equal_nan=True)


def test_auto_nms_placement():
    """the automatic mode: thousands of candidates per image go to the device for a caller that runs one forward at a time (shorter
    latency) and to the host while forwards are pipelined and the host keeps up (no device time taken from the next forward); few
    candidates always go to the device; the boxes are the same wherever they were suppressed"""
    size, batch = 352, 2
    net, binp, g = nu.model("yolov3", batch, size, seed=3)
    x = zoo.seeded_input(batch, 3, size, size, seed=4)
    xd = torch.from_numpy(x).cuda()
    netapi.set_device_nms(1)
    m = netapi.Net(net, binp, fp16=True)
    first = m.run_yolo(x)                    # (nothing known about the candidate count yet)
    n = max(len(b) for b in first)
    assert 2048 < n <= 6144, n               # the regime this test is about (boxes <= candidates)
    one = m.run_yolo(x)
    assert m.last_nms_on_device()
    m.enqueue(xd.data_ptr())
    m.enqueue(xd.data_ptr())
    a = m.fetch_yolo()
    assert m.last_nms_on_device()            # (enqueued while nothing else was in flight)
    m.enqueue(xd.data_ptr())
    b = m.fetch_yolo()
    assert not m.last_nms_on_device()        # enqueued beside another forward
    assert "YoloOut NMS     : last result on the host, mode auto" in m.time_detail()          # the choice is on record in getTimeDetail
    c = m.fetch_yolo()
    for i in range(batch):
        for other in (a, b, c):
            assert np.array_equal(one[i], other[i], equal_nan=True)
    few = np.zeros_like(x)
    m.run_yolo(few)
    m.run_yolo(few)
    assert m.last_nms_on_device()
    assert "YoloOut NMS     : last result on the device, mode auto, " in m.time_detail()


def test_yolo_rows_copied_in_part():
    """The host path copies only a prefix of the candidate row slots ahead of time, sized from the previous result, and fetches
    the remainder on demand: a network that saw few candidates and then many (and the other way round) returns what a fresh
    network returns for each input."""
    size, batch = 320, 2
    net, binp, g = nu.model("yolov3", batch, size, seed=8)
    few = np.zeros((batch, 3, size, size), np.float32)
    many = zoo.seeded_input(batch, 3, size, size, seed=9)
    try:
        netapi.set_device_nms(0)
        want_few = netapi.Net(net, binp, fp16=True).run_yolo(few)
        want_many = netapi.Net(net, binp, fp16=True).run_yolo(many)
        m = netapi.Net(net, binp, fp16=True)
        seq = [few, many, many, few, few, many]
        got = [m.run_yolo(x) for x in seq]
        # with these weights most cells are candidates whatever the input, so the prefix is also forced to be short:
        # 100 rows ahead of time, thousands on demand; 3000: some images need more, some do not
        for forced in ("100", "3000"):
            os.environ["MSNH_YOLO_ROWS_PREFIX"] = forced
            got += [m.run_yolo(x) for x in seq]
    finally:
        os.environ.pop("MSNH_YOLO_ROWS_PREFIX", None)
        netapi.set_device_nms(1)
    seq = seq * 3
    print("boxes: few", [len(b) for b in want_few], "many", [len(b) for b in want_many], flush=True)
    assert sum(len(b) for b in want_many) > 0
    for x, g_ in zip(seq, got):
        w_ = want_few if x is few else want_many
        for b in range(batch):
            assert np.array_equal(g_[b], w_[b], equal_nan=True)


def test_spp_maxpools_run_as_a_chain():
    """the 5 / 9 / 13 pools of an SPP block become three 5-wide pools, each reading the one before, and where the tile of an image
    fits LDS they are one launch (same results: the per-layer and final-output parity tests of yolov4 and yolov5s run through this
    plan; with MSNH_NO_POOL_CHAIN the separate launches give the same boxes bit for bit)"""
    for arch, size in (("yolov4", 160), ("yolov5s", 160)):
        net, binp, g = nu.model(arch, 2, size, seed=3)
        x = zoo.seeded_input(2, 3, size, size, seed=4)
        netapi.set_tune_cache(True)                 # the same tiles in both builds below
        try:
            m = netapi.Net(net, binp, fp16=True)
            pools = [ln for ln in m.plan_detail().splitlines() if " maxpool[" in ln and " s1 " in ln]
            assert len(pools) == 3 and all("[k5 s1 p2" in ln for ln in pools), pools
            assert sum("in the launch of the pool before it" in ln for ln in pools) == 2, pools
            launches = int(m.plan_detail().split(" launches")[0].split()[-1])
            fused = m.run_yolo(x)
            os.environ["MSNH_NO_POOL_CHAIN"] = "1"
            try:
                m2 = netapi.Net(net, binp, fp16=True)
            finally:
                del os.environ["MSNH_NO_POOL_CHAIN"]
            assert "in the launch of the pool before it" not in m2.plan_detail()
            assert int(m2.plan_detail().split(" launches")[0].split()[-1]) == launches + 2
            apart = m2.run_yolo(x)
            for a, b in zip(fused, apart):
                assert len(a) > 0 and np.array_equal(a, b, equal_nan=True)
        finally:
            netapi.set_tune_cache(False)


def test_inverted_residual_blocks_run_as_one_launch():
    """float16 MobileNetV2: every expand -> depthwise -> project block whose channel counts the kernel takes is one launch
    (msnh_hip_mbconv); the block's residual add rides in it.  Against the three-launch plan (MSNH_NO_MBCONV) the logits agree to
    float16 accuracy (the widened tensors are rounded to float16 at the same points with the same scales; only the float32 summation
    order of the projection differs), and the per-layer / final parity tests of mobilenetv2 run through the fused plan."""
    for batch, size in ((3, 224),):                             # (the 7x7 average pool needs the full-size feature map; tiles cut by image edges: tests/test_mbconv_gpu.py)
        net, binp, g = nu.model("mobilenetv2", batch, size, seed=3)
        x = zoo.seeded_input(batch, 3, size, size, seed=4)
        m = netapi.Net(net, binp, fp16=True)
        detail = m.plan_detail()
        fused_lines = [ln for ln in detail.splitlines() if "conv[mbconv" in ln]
        assert len(fused_lines) == 12, detail                   # 17 blocks: the first has no expand, four have 160 / 320 channels
        assert sum("+res" in ln for ln in fused_lines) == 8, fused_lines
        launches = int(detail.split(" launches")[0].split()[-1])
        fused = m.run_classify(x)
        os.environ["MSNH_NO_MBCONV"] = "1"
        try:
            m2 = netapi.Net(net, binp, fp16=True)
        finally:
            del os.environ["MSNH_NO_MBCONV"]
        assert "mbconv" not in m2.plan_detail()
        assert int(m2.plan_detail().split(" launches")[0].split()[-1]) == launches + 24
        apart = m2.run_classify(x)
        err = np.abs(fused - apart).max() / np.abs(apart).max()
        print("fused against three launches:", size, err, flush=True)
        assert err <= 2e-3
        assert np.array_equal(fused, m.run_classify(x))


def test_conv_with_its_1x1_consumer_as_one_launch():
    """float16 YOLOv3: a convolution whose tile holds all its output channels (the 3x3 convolutions with 256 filters and fewer) can compute
    the 1x1 convolution that reads its result in the same launch (msnh_hip_conv2d_tail).  Off by default (it measured level with two
    launches inside a forward); MSNH_CONV_TAIL=1 lets the load-time search decide per pair; forced on here (MSNH_FORCE_CONV_TAIL).
    The launch itself returns the bits of two launches on the same tiles (tests/test_conv_gpu.py::test_conv_tail); two networks tuned
    separately may settle on different tiles for a layer, which changes float32 summation orders, so the comparison of the whole network
    with the default plan is to float16 accuracy: head logits within 5e-3 of their largest value (two default plans tuned separately
    have been seen 2e-3 apart on this network), as many boxes to within 1 %."""
    batch, size = 2, 160
    net, binp, g = nu.model("yolov3", batch, size, seed=5)
    x = zoo.seeded_input(batch, 3, size, size, seed=6)
    m0 = netapi.Net(net, binp, fp16=True)
    assert "igemm+1x1" not in m0.plan_detail()
    launches = int(m0.plan_detail().split(" launches")[0].split()[-1])
    want = m0.run_yolo(x)
    want_heads = [m0.yolo_head_logits(h) for h in range(3)]
    os.environ["MSNH_FORCE_CONV_TAIL"] = "1"
    try:
        m = netapi.Net(net, binp, fp16=True)
    finally:
        del os.environ["MSNH_FORCE_CONV_TAIL"]
    detail = m.plan_detail()
    fused = [ln for ln in detail.splitlines() if "conv[igemm+1x1" in ln]
    assert len(fused) >= 10, detail
    assert int(detail.split(" launches")[0].split()[-1]) == launches - len(fused)
    got = m.run_yolo(x)
    for h in range(3):
        e = nu.rel_err(m.yolo_head_logits(h), want_heads[h])
        print("head", h, "one launch per pair against two:", e, flush=True)
        assert e <= 5e-3, h
    for a, b in zip(got, want):
        assert len(b) > 0 and abs(len(a) - len(b)) <= max(2, len(b) // 100)
    assert all(np.array_equal(a, b, equal_nan=True) for a, b in zip(m.run_yolo(x), got))


@pytest.mark.parametrize("fp16", [False, True])
def test_conv_writes_the_upsampled_tensor(fp16):
    """The 1x1 convolutions in front of the two nearest-neighbour upsample layers of YOLOv3's neck write the upsampled tensors themselves
    (msnh_conv_desc::out_upsample; Plan::fuse f): no upsample launch is left in the plan, and the head logits equal those of the plan that
    keeps the upsample launches (MSNH_NO_CONV_UPSAMPLE) -- to 1e-5 in float32, to 5e-3 in float16 (two separately tuned plans may sum in
    different orders)."""
    batch, size = 2, 160
    net, binp, g = nu.model("yolov3", batch, size, seed=7)
    x = zoo.seeded_input(batch, 3, size, size, seed=8)
    m = netapi.Net(net, binp, fp16=fp16)
    detail = m.plan_detail()
    assert sum("+up2" in ln for ln in detail.splitlines()) == 2, detail
    assert not any(" upsample" in ln for ln in detail.splitlines()), detail
    got = m.run_yolo(x)
    heads = [m.yolo_head_logits(h) for h in range(3)]
    os.environ["MSNH_NO_CONV_UPSAMPLE"] = "1"
    try:
        m0 = netapi.Net(net, binp, fp16=fp16)
    finally:
        del os.environ["MSNH_NO_CONV_UPSAMPLE"]
    d0 = m0.plan_detail()
    assert "+up2" not in d0 and sum(" upsample" in ln for ln in d0.splitlines()) == 2, d0
    want = m0.run_yolo(x)
    for h in range(3):
        e = nu.rel_err(heads[h], m0.yolo_head_logits(h))
        print("head", h, "fp16" if fp16 else "fp32", e, flush=True)
        assert e <= (5e-3 if fp16 else 1e-5), h
    for a, b in zip(got, want):
        assert len(b) > 0 and abs(len(a) - len(b)) <= (max(2, len(b) // 100) if fp16 else 0)


def test_image_in_boxes_out():
    """8-bit images of different shapes -> device letterbox -> forward -> boxes in original-image pixels: equals the
    float path fed with the restatement's letterbox, followed by the restatement's rescale."""
    size, batch = 96, 2
    net, binp, g = nu.model("yolov3", batch, size, seed=3)
    rng = np.random.default_rng(12)
    imgs = [rng.integers(0, 256, (120, 200, 3), dtype=np.uint8), rng.integers(0, 256, (150, 90, 3), dtype=np.uint8)]
    m = netapi.Net(net, binp)
    for i, im in enumerate(imgs):
        m.set_input_image_u8(i, im)
    m.enqueue(None)
    got = m.fetch_yolo()
    x = np.stack([on.letterbox_u8(im, size, size) for im in imgs])
    want = m.run_yolo(x)
    for i, im in enumerate(imgs):
        assert np.array_equal(got[i], want[i])
        back = netapi.boxes_to_image(got[i], size, size, im.shape[1], im.shape[0])
        for k in range(len(back)):
            assert np.array_equal(back[k, :4], on.bbox_resize2org(got[i][k, :4], size, size, im.shape[1], im.shape[0]))
    with pytest.raises(netapi.MsnhnetError):
        m.set_input_image_u8(2, imgs[0])


def test_cpu_entry_points_refuse():
    net, binp, g = nu.model("resnet18", 1, 224, seed=3)
    m = netapi.Net(net, binp)
    with pytest.raises(netapi.MsnhnetError, match="Gpu mode , can not run with cpu"):
        m.run_classify_cpu(np.zeros(3 * 224 * 224, np.float32))
    with pytest.raises(netapi.MsnhnetError, match="input image size err. Needed :150528 given :10"):
        m.run_classify(np.zeros(10, np.float32))


@pytest.mark.parametrize("arch,size,batch,instances,depth", [("yolov3", 96, 2, 2, 2), ("yolov3", 96, 2, 3, 1), ("resnet18", 224, 2, 2, 2), ("yolov3", 96, 2, 1, 2)])
def test_net_group_results_in_submission_order(arch, size, batch, instances, depth):
    """netapi.NetGroup: several instances of a network fed round-robin by one host thread each return, in submission order, exactly
    what one instance returns for each of the submitted batches (distinct inputs, so a swapped or repeated result shows), also for the
    batches an instance still holds in flight when flush() is called; an error inside a worker surfaces in fetch()"""
    net, binp, g = nu.model(arch, batch, size, seed=11)
    xs = [zoo.seeded_input(batch, 3, size, size, seed=20 + i) for i in range(7)]
    xd = [torch.from_numpy(x).cuda() for x in xs]
    one = netapi.Net(net, binp, fp16=True)
    detect = arch.startswith("yolo")
    want = [one.run_yolo(x) if detect else one.run_classify(x) for x in xs]
    grp = netapi.NetGroup(net, binp, instances=instances, depth=depth, fp16=True)
    try:
        assert grp.detect == detect and len(grp.nets) == instances
        grp.prime(xd[0].data_ptr())
        for rounds in range(2):
            for t in xd:
                grp.submit(t.data_ptr())
            grp.flush()
            for i in range(len(xd)):
                got = grp.fetch()
                if detect:
                    assert len(got) == batch
                    for a, b in zip(got, want[i]):
                        assert np.array_equal(a, b, equal_nan=True), (rounds, i)
                else:
                    assert np.array_equal(got, want[i]), (rounds, i)
        with pytest.raises(RuntimeError):
            grp.fetch()                      # nothing outstanding
        # as a serving loop runs: a window of batches outstanding, one fetched for each one submitted, and the tail fetched without
        # flush() (a result that its instance would hold back until more work comes is asked for by the fetch itself)
        window = min(instances * depth, len(xd) - 1)
        for t in xd[:window]:
            grp.submit(t.data_ptr())
        for i in range(len(xd)):
            got = grp.fetch()
            if i + window < len(xd):
                grp.submit(xd[i + window].data_ptr())
            if detect:
                for a, b in zip(got, want[i]):
                    assert np.array_equal(a, b, equal_nan=True), ("window", i)
            else:
                assert np.array_equal(got, want[i]), ("window", i)
        assert grp.outstanding() == 0
        # on what an instance's input buffer holds (one of the submitted batches)
        grp.submit(None)
        grp.flush()
        got = grp.fetch()
        if detect:
            assert any(all(np.array_equal(a, b, equal_nan=True) for a, b in zip(got, w)) for w in want)
        else:
            assert any(np.array_equal(got, w) for w in want)
    finally:
        grp.close()


def test_net_group_refuses_bad_arguments(tmp_path):
    """a group that cannot be built reports the error of the step that failed and leaves nothing running"""
    net, binp, g = nu.model("yolov3", 2, 96, seed=3)
    with pytest.raises(netapi.MsnhnetError, match="1 to 16 instances"):
        netapi.NetGroup(net, binp, instances=0, depth=2, fp16=True)
    with pytest.raises(netapi.MsnhnetError):
        netapi.NetGroup(os.path.join(str(tmp_path), "missing.msnhnet"), binp, instances=2, depth=2, fp16=True)
    with pytest.raises(netapi.MsnhnetError):
        netapi.NetGroup(net, os.path.join(str(tmp_path), "missing.msnhbin"), instances=2, depth=2, fp16=True)
    grp = netapi.NetGroup(net, binp, instances=2, depth=2, fp16=True)      # and the library still builds one afterwards
    try:
        x = torch.from_numpy(zoo.seeded_input(2, 3, 96, 96, seed=4)).cuda()
        torch.cuda.synchronize()
        grp.prime(x.data_ptr())
        grp.submit(x.data_ptr())
        assert len(grp.fetch()) == 2
    finally:
        grp.close()


@pytest.mark.parametrize("instances,fail_at", [(1, 2), (2, 4), (2, 5)])
def test_net_group_enqueue_error_keeps_the_order(instances, fail_at, monkeypatch):
    """a batch whose enqueue fails while an earlier batch of the same instance is still in flight (depth 2): the earlier batch's
    result is handed out first, the failed submission's own fetch raises, and every later fetch returns what belongs to it"""
    size, batch = 96, 2
    net, binp, g = nu.model("yolov3", batch, size, seed=11)
    xs = [zoo.seeded_input(batch, 3, size, size, seed=40 + i) for i in range(8)]
    xd = [torch.from_numpy(x).cuda() for x in xs]
    torch.cuda.synchronize()
    one = netapi.Net(net, binp, fp16=True)
    want = [one.run_yolo(x) for x in xs]
    grp = netapi.NetGroup(net, binp, instances=instances, depth=2, fp16=True)
    try:
        grp.prime(xd[0].data_ptr())
        monkeypatch.setenv("MSNH_GROUP_FAIL_ENQUEUE", str(fail_at))
        for t in xd:
            grp.submit(t.data_ptr())
        monkeypatch.delenv("MSNH_GROUP_FAIL_ENQUEUE")
        grp.flush()
        for i in range(len(xd)):
            if i == fail_at:
                with pytest.raises(RuntimeError, match="MSNH_GROUP_FAIL_ENQUEUE"):
                    grp.fetch()
                continue
            got = grp.fetch()
            for a, b in zip(got, want[i]):
                assert np.array_equal(a, b, equal_nan=True), i
        assert grp.outstanding() == 0
    finally:
        grp.close()


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_copy_on_forward_stream_same_results(mode):
    """copy-back (and device NMS) on the forward's own stream, as the instances of a group run, returns what the copy stream beside
    the next forward returns, pipelined and one at a time, for every NMS placement"""
    size, batch = 160, 2
    net, binp, g = nu.model("yolov3", batch, size, seed=5)
    xs = [zoo.seeded_input(batch, 3, size, size, seed=30 + i) for i in range(3)]
    xd = [torch.from_numpy(x).cuda() for x in xs]
    netapi.set_device_nms(mode)
    try:
        m = netapi.Net(net, binp, fp16=True)
        want = [m.run_yolo(x) for x in xs]
        m.set_copy_on_forward_stream(True)
        for rounds in range(2):
            m.enqueue(xd[0].data_ptr())
            for i in range(1, 3):
                m.enqueue(xd[i].data_ptr())
                got = m.fetch_yolo()
                assert all(np.array_equal(a, b, equal_nan=True) for a, b in zip(got, want[i - 1]))
            got = m.fetch_yolo()
            assert all(np.array_equal(a, b, equal_nan=True) for a, b in zip(got, want[2]))
        m.set_copy_on_forward_stream(False)
        got = m.run_yolo(xs[1])
        assert all(np.array_equal(a, b, equal_nan=True) for a, b in zip(got, want[1]))
        cls = netapi.Net(*nu.model("resnet18", 1, 224, seed=3)[:2], fp16=True)
        with pytest.raises(netapi.MsnhnetError):
            cls.set_copy_on_forward_stream(True)
    finally:
        netapi.set_device_nms(1)
