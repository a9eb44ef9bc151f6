"""The reference's own entry points on the device: its C facade (src/c_api/MsnhnetLib.h: initMsnhnet, buildMsnhnet,
runClassifyNoPred, runClassifyList, runYoloList, dispose, ...) driven through a success path and compared with the oracle, and a C++
caller written only against the reference's class API (tests/cpp/ref_caller.cpp), compiled against the host headers, linked with
libMsnhnet.so and run."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

import msnh_oracle_net as on
import netutil as nu
from msnhnet_amd import netapi, zoo

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(ROOT, "tests", "golden", "ref_golden.npz"))
PRE = {"none": 0, "c1": 1, "f32c3": 2, "googlenet": 3, "padding_zero": 4, "transformed": 5, "caffe": 6}      # PredDataType


def _u8p(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte))


def _fp(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def compile_caller(tmp):
    """g++ on the caller with the host headers as the only include directory (what a user of the reference's include/ would do)"""
    exe = os.path.join(str(tmp), "ref_caller")
    lib_dir = os.path.join(ROOT, "msnhnet_amd", "lib")
    cmd = ["g++", "-std=c++11", "-O1", "-I" + os.path.join(ROOT, "msnhnet_amd", "host", "include"), os.path.join(ROOT, "tests", "cpp", "ref_caller.cpp"),
           "-o", exe, "-L" + lib_dir, "-lMsnhnet", "-Wl,-rpath," + lib_dir]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    return exe


def test_reference_api_caller_compiles_and_links(tmp_path):
    exe = compile_caller(tmp_path)
    r = subprocess.run([exe], stdout=subprocess.PIPE, text=True)
    assert r.returncode == 2 and "usage" in r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("arch,size,mode,fp16", [("resnet18", 224, "classify", False), ("yolo_head", 6, "yolo", False), ("yolov3", 96, "yolo", False),
                                                 ("resnet18", 224, "classify", True)])
def test_reference_api_caller_runs(arch, size, mode, fp16, tmp_path):
    exe = compile_caller(tmp_path)
    if arch == "yolo_head":
        # one detection head with moderate logits (a micro graph of the golden file): its boxes are pinned by the reference's own
        net, binp = str(tmp_path / "y.msnhnet"), str(tmp_path / "y.msnhbin")
        with open(net, "w") as f:
            f.write(bytes(GOLD["micro/yolo_head/graph"]).decode())
        np.asarray(GOLD["micro/yolo_head/weights"], np.float32).tofile(binp)
        x = GOLD["micro/yolo_head/input"][None]
    else:
        net, binp, g = nu.model(arch, 1, size, seed=3)
        x = zoo.seeded_input(1, 3, size, size, seed=4)
    inp, outp = str(tmp_path / "in.f32"), str(tmp_path / "out.f32")
    np.ascontiguousarray(x[0], np.float32).tofile(inp)
    print("running the C++ caller", arch, mode, flush=True)
    r = subprocess.run([exe, mode, net, binp, inp, outp] + (["fp16"] if fp16 else []), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "cpu: Gpu mode , can not run with cpu" in r.stdout
    assert "time  :" in r.stdout and "weights :" in r.stdout
    got = np.fromfile(outp, np.float32)
    if arch == "yolo_head":
        assert nu.boxes_err(got.reshape(-1, 7), GOLD["micro/yolo_head/boxes"]) <= 1e-4
        return
    o = on.OracleNet(nu.batch1_graph(arch, size), binp)
    ref = o.run(x[0])
    if mode == "classify":
        want = np.asarray(ref[-1]).ravel()
        assert got.size == want.size
        assert nu.rel_err(got, want) <= (2e-2 if fp16 else 1e-4)
        if not fp16:
            assert int(np.argmax(got)) == int(np.argmax(want))
    else:
        # (saturated objectness ties: a few boxes may be replaced by their neighbours, see netutil.boxes_matched_fraction)
        got = got.reshape(-1, 7)
        assert abs(len(got) - len(o.boxes)) <= max(2, 0.02 * len(o.boxes))
        assert nu.boxes_matched_fraction(got, o.boxes, 1e-4) >= 0.95 and nu.boxes_matched_fraction(o.boxes, got, 1e-4) >= 0.95


@pytest.mark.gpu
def test_facade_classify_success_path(tmp_path):
    """initMsnhnet -> buildMsnhnet -> getInputDim -> runClassifyNoPred -> runClassifyList (every PredDataType) -> dispose"""
    L = netapi.lib()
    size = 224
    net, binp, g = nu.model("resnet18", 1, size, seed=3)
    o = on.OracleNet(nu.batch1_graph("resnet18", size), binp)
    msg = ctypes.c_char_p()
    gpu = ctypes.c_int(0)
    assert L.withGPU(ctypes.byref(gpu)) == 1 and gpu.value == 1
    assert L.initMsnhnet() == 1
    assert L.buildMsnhnet(ctypes.byref(msg), net.encode(), binp.encode(), 0, 0) == 1
    w, h, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert L.getInputDim(ctypes.byref(w), ctypes.byref(h), ctypes.byref(c)) == 1 and (w.value, h.value, c.value) == (size, size, 3)
    x = zoo.seeded_input(1, 3, size, size, seed=4)[0]
    best = ctypes.c_int(-1)
    assert L.runClassifyNoPred(ctypes.byref(msg), _fp(x), x.size, ctypes.byref(best), 1) == 1
    assert best.value == int(np.argmax(o.run(x)[-1]))
    t = ctypes.c_float(-1)
    assert L.getGpuForwardTime(ctypes.byref(t)) == 1 and t.value > 0
    # the CPU path does not exist
    assert L.runClassifyNoPred(ctypes.byref(msg), _fp(x), x.size, ctypes.byref(best), 0) == -1
    assert b"Gpu mode , can not run with cpu" in msg.value
    assert L.runClassifyNoPred(ctypes.byref(msg), _fp(x), 10, ctypes.byref(best), 1) == -1
    assert b"input image size err" in msg.value

    rng = np.random.default_rng(31)
    img = rng.integers(0, 256, (180, 260, 3), dtype=np.uint8)
    mean, std = np.array([0.4, 0.5, 0.6], np.float32), np.array([0.2, 0.3, 0.25], np.float32)
    kinds = {"f32c3": "f32c3", "googlenet": "googlenet", "transformed": "transformed", "caffe": "caffe"}
    for pre, kind in kinds.items():
        for swap in (0, 1):
            xin = on.preproc_u8(img, size, size, kind, mean, std, nu.facade_shuffle(pre, swap))
            want = int(np.argmax(o.run(xin)[-1]))
            assert L.runClassifyList(ctypes.byref(msg), _u8p(img), 260, 180, 3, ctypes.byref(best), PRE[pre], swap, 1, _fp(mean), _fp(std)) == 1, msg.value
            assert best.value == want, (pre, swap)
    for swap in (0, 1):
        xin = on.letterbox_u8(img, size, size, False, nu.facade_shuffle("padding_zero", swap))
        assert L.runClassifyList(ctypes.byref(msg), _u8p(img), 260, 180, 3, ctypes.byref(best), PRE["padding_zero"], swap, 1, None, None) == 1
        assert best.value == int(np.argmax(o.run(xin)[-1])), ("padding_zero", swap)
    # the reference's argument errors
    for args, text in (((3, PRE["none"], None, None), b"preDataType can't be none"), ((2, PRE["f32c3"], None, None), b"channel must be 1 or 3"),
                       ((1, PRE["f32c3"], None, None), b"channel 1 must preprocess with F32_C1"), ((3, PRE["c1"], None, None), b"channel 1 can't preprocess with F32_C1"),
                       ((3, PRE["transformed"], None, None), b"mean or std can't be null")):
        ch, pre, m, s = args
        assert L.runClassifyList(ctypes.byref(msg), _u8p(img), 260, 180, ch, ctypes.byref(best), pre, 0, 1, m, s) == -1
        assert text in msg.value, msg.value
    assert L.runClassifyList(ctypes.byref(msg), _u8p(img), 260, 180, 3, ctypes.byref(best), PRE["f32c3"], 0, 0, None, None) == -1
    assert b"Gpu mode , can not run with cpu" in msg.value
    assert L.dispose() == 1
    assert L.runClassifyNoPred(ctypes.byref(msg), _fp(x), x.size, ctypes.byref(best), 1) == -1


@pytest.mark.gpu
def test_facade_yolo_success_path(tmp_path):
    """buildMsnhnet -> runYoloNoPred / runYoloList -> boxes equal the oracle's on the letterboxed image"""
    L = netapi.lib()
    size = 96
    # a head that keeps a handful of boxes (the big seeded detectors return thousands, more than the facade's container holds)
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_golden.npz"))
    net = str(tmp_path / "y.msnhnet")
    binp = str(tmp_path / "y.msnhbin")
    text = bytes(gold["micro/yolo_head/graph"]).decode()
    with open(net, "w") as f:
        f.write(text)
    np.asarray(gold["micro/yolo_head/weights"], np.float32).tofile(binp)
    x = gold["micro/yolo_head/input"]
    msg = ctypes.c_char_p()
    assert L.initMsnhnet() == 1
    assert L.buildMsnhnet(ctypes.byref(msg), net.encode(), binp.encode(), 0, 0) == 1, msg.value
    boxes = netapi.BBoxContainer()
    n = ctypes.c_int(-1)
    xx = np.ascontiguousarray(x, np.float32)
    assert L.runYoloNoPred(ctypes.byref(msg), _fp(xx), xx.size, ctypes.byref(boxes), ctypes.byref(n), 1) == 1, msg.value
    ref = gold["micro/yolo_head/boxes"]
    got = np.array([[b.x, b.y, b.w, b.h, b.conf, b.bestClsConf, b.bestClsIdx] for b in boxes.boxes[:n.value]], np.float32)
    assert n.value == len(ref) and n.value > 0
    assert nu.boxes_err(got, ref) <= 1e-4
    assert L.dispose() == 1

    # a whole detector on an 8-bit image: runYoloList == the oracle on the oracle's letterbox of that image
    net, binp, g = nu.model("yolov3_tiny", 1, size, seed=3)
    o = on.OracleNet(nu.batch1_graph("yolov3_tiny", size), binp)
    rng = np.random.default_rng(32)
    img = rng.integers(0, 256, (70, 120, 3), dtype=np.uint8)
    assert L.initMsnhnet() == 1
    assert L.buildMsnhnet(ctypes.byref(msg), net.encode(), binp.encode(), 0, 0) == 1, msg.value
    for swap in (0, 1):
        o.run(on.letterbox_u8(img, size, size, False, nu.facade_shuffle("padding_zero", swap)))
        ref = o.boxes
        rc = L.runYoloList(ctypes.byref(msg), _u8p(img), 120, 70, 3, ctypes.byref(boxes), ctypes.byref(n), swap, 1)
        if len(ref) > 1024:
            assert rc == -1 and b"BBox buffer is not enough" in msg.value
            continue
        assert rc == 1, msg.value
        got = np.array([[b.x, b.y, b.w, b.h, b.conf, b.bestClsConf, b.bestClsIdx] for b in boxes.boxes[:n.value]], np.float32).reshape(-1, 7)
        assert abs(n.value - len(ref)) <= max(2, 0.02 * len(ref))
        assert nu.boxes_matched_fraction(got, ref, 1e-4) >= 0.95 and nu.boxes_matched_fraction(ref, got, 1e-4) >= 0.95
    assert L.runYoloList(ctypes.byref(msg), _u8p(img), 120, 70, 2, ctypes.byref(boxes), ctypes.byref(n), 0, 1) == -1
    assert b"channel must be 1 or 3" in msg.value
    assert L.runYoloList(ctypes.byref(msg), _u8p(img), 120, 70, 3, ctypes.byref(boxes), ctypes.byref(n), 0, 0) == -1
    assert b"Gpu mode , can not run with cpu" in msg.value
    assert L.dispose() == 1


@pytest.mark.gpu
def test_facade_against_the_reference_facade(tmp_path):
    """runClassifyList / runYoloList of this library against the reference's own facade (src/c_api/MsnhnetLib.cpp compiled into
    oracle/_ref, CPU path) on the same 8-bit image, every PredDataType, swapRGB 0 and 1: same class index, same boxes"""
    import refshim
    from test_ref_facade_cpu import _image, small_detector
    if not refshim.available():
        pytest.skip("reference build not present")
    L = netapi.lib()
    msg = ctypes.c_char_p()
    size = 224            # (the 7x7 average pool of this library needs the full-size feature map)
    net, binp, g = nu.model("resnet18", 1, size, seed=3)
    ref = refshim.RefFacade(nu.batch1_graph("resnet18", size), binp)
    img = _image(31, 50, 70)
    mean, std = np.array([0.4, 0.5, 0.6], np.float32), np.array([0.2, 0.3, 0.25], np.float32)
    assert L.initMsnhnet() == 1
    assert L.buildMsnhnet(ctypes.byref(msg), net.encode(), binp.encode(), 0, 0) == 1, msg.value
    best = ctypes.c_int(-1)
    seen = set()
    for pre in ("f32c3", "googlenet", "transformed", "caffe", "padding_zero"):
        for swap in (0, 1):
            want = ref.classify_list(img, pre, swap, mean, std)
            print("facade", pre, swap, flush=True)
            assert L.runClassifyList(ctypes.byref(msg), _u8p(img), 70, 50, 3, ctypes.byref(best), PRE[pre], swap, 1, _fp(mean), _fp(std)) == 1, msg.value
            assert best.value == want, (pre, swap)
            seen.add((pre, want))
    assert len(seen) > 5                 # swapRGB changes the prediction for this image: the polarity is really tested
    assert L.dispose() == 1
    ref.close()

    net, binp, size = small_detector(tmp_path)
    ref = refshim.RefFacade(net, binp)
    img = _image(33, 3 * size, 4 * size)
    assert L.initMsnhnet() == 1
    assert L.buildMsnhnet(ctypes.byref(msg), net.encode(), binp.encode(), 0, 0) == 1, msg.value
    boxes = netapi.BBoxContainer()
    n = ctypes.c_int(-1)
    res = []
    for swap in (0, 1):
        want = ref.yolo_list(img, swap)
        assert L.runYoloList(ctypes.byref(msg), _u8p(img), 4 * size, 3 * size, 3, ctypes.byref(boxes), ctypes.byref(n), swap, 1) == 1, msg.value
        got = np.array([[b.x, b.y, b.w, b.h, b.conf, b.bestClsConf, b.bestClsIdx] for b in boxes.boxes[:n.value]], np.float32).reshape(-1, 7)
        assert len(want) > 0 and nu.boxes_err(got, want) <= 1e-4, swap
        res.append(want)
    assert not np.array_equal(res[0], res[1])
    assert L.dispose() == 1
    ref.close()
