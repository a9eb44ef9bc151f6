"""Host-side logic without a GPU: both shared libraries load and export every symbol the headers declare, the
`.msnhnet` reader and NetBuilder's graph construction agree with the reference (golden shape tables and the
reference's own layer-detail text), the error paths a caller can provoke raise Msnhnet's messages, and the two NMS
implementations agree.  No compute entry point is called."""
import ctypes
import os
import re

import numpy as np
import pytest

import msnh_oracle_net as on
from msnhnet_amd import hipabi, netapi, zoo

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_golden.npz"))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:msnh_hip_|msnhnet_)\w+|initMsnhnet|buildMsnhnet|runClassifyNoPred|runYoloNoPred|runClassifyList|runYoloList|dispose|withGPU|withCUDNN|"
                                 r"getCpuForwardTime|getGpuForwardTime|getInputDim)\s*\(", text)))


def test_kernel_library_exports_every_declared_symbol():
    names = _declared("msnh_hip.h")
    assert len(names) >= 40
    lib = ctypes.CDLL(hipabi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert set(hipabi.SYMBOLS) == set(names) - {"msnh_hip_conv_desc"}


def test_diagnostics_library_exports_every_declared_symbol():
    from msnhnet_amd import diag
    names = _declared("msnh_hip_diag.h")
    ctypes.CDLL(hipabi.LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    lib = ctypes.CDLL(diag.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert set(diag.SYMBOLS) == set(names)


def test_host_library_exports_every_declared_symbol():
    names = [n for n in _declared("msnhnet_c.h") if n != "msnhnet_t"]
    lib = ctypes.CDLL(netapi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    assert set(netapi.SYMBOLS) == set(names)


def _write(tmp_path, text, name="g.msnhnet"):
    p = os.path.join(str(tmp_path), name)
    with open(p, "w") as f:
        f.write(text)
    return p


@pytest.mark.parametrize("arch,dtype,batch,size", zoo.CONFIGS)
def test_graph_construction_matches_reference_tables(arch, dtype, batch, size, tmp_path):
    g = zoo.ARCHS[arch](batch=1, size=size)
    m = netapi.Net(_write(tmp_path, g.text()))
    infos = m.layer_infos()
    table = GOLD[f"shape/{arch}/table"]
    types = bytes(GOLD[f"shape/{arch}/types"]).decode().split("\n")
    assert len(infos) == len(table)
    keys = ["outH", "outW", "outC", "outputNum", "inputNum", "numWeights"]
    for i, info in enumerate(infos):
        assert info["type"] == types[i], i
        assert [info[k] for k in keys] == list(table[i]), (i, info)
    assert m.layer_detail() == bytes(GOLD[f"shape/{arch}/detail"]).decode()
    assert sum(i["numWeights"] for i in infos) == sum(s.count for s in g.slots)


SHIPPED = sorted(__import__("glob").glob("/root/reference/models/*/*.msnhnet"))
# the one graph this build refuses: yolov3_spp.msnhnet uses node names ("yolov3", "yolov3out") that the reference's own parser rejects too
REFUSED = {"yolov3_spp.msnhnet": r"\[yolov3\]"}


@pytest.mark.skipif(not SHIPPED, reason="the reference's model files are not present")
@pytest.mark.parametrize("path", SHIPPED, ids=[os.path.basename(p) for p in SHIPPED])
def test_shipped_graphs_build_like_the_reference(path):
    """Every .msnhnet file the reference ships builds here, layer for layer with the shapes and weight counts the reference's own
    NetBuilder derives (when its library is present)."""
    import refshim
    name = os.path.basename(path)
    if name in REFUSED:
        with pytest.raises(netapi.MsnhnetError, match=REFUSED[name]):
            netapi.Net(path)
        return
    infos = netapi.Net(path).layer_infos()
    assert len(infos) > 0
    if not refshim.available():
        return
    r = refshim.RefNet(path)
    ref = r.layer_infos()
    r.close()
    assert len(infos) == len(ref)
    for i, (a, b) in enumerate(zip(infos, ref)):
        # (a softmax layer leaves its image shape unset in the reference: compare the element counts only)
        keys = ["outputNum", "numWeights"] if b["type"] in ("6", "softmax") else ["outH", "outW", "outC", "outputNum", "numWeights"]
        assert [a[k] for k in keys] == [b[k] for k in keys], (name, i, a, b)


def test_zoo_totals():
    want = {"resnet18": 11699112, "resnet50": 25610152, "mobilenetv2": 3538984, "yolov3": 62001757, "yolov4": 64429405}
    gf = {"resnet18": 3.63, "resnet50": 8.18, "mobilenetv2": 0.605, "yolov3": 140.7, "yolov4": 128.4}
    for arch, dtype, batch, size in zoo.CONFIGS:
        g = zoo.ARCHS[arch](batch=batch, size=size)
        assert sum(s.count for s in g.slots) == want[arch]
        assert g.conv_flops / 1e9 == pytest.approx(gf[arch], rel=0.012)


def test_batched_graph_keeps_per_image_shapes(tmp_path):
    g = zoo.yolov3(batch=8, size=608)
    m = netapi.Net(_write(tmp_path, g.text()))
    assert m.dims() == (8, 3, 608, 608)
    info = m.layer_info(0)
    assert (info["outH"], info["outW"], info["outC"], info["batch"]) == (608, 608, 32, 8)


CFG = "config:\n  batch: 1\n  width: 8\n  height: 8\n  channels: 3\n"


@pytest.mark.parametrize("text,msg", [
    ("conv:\n  filters: 4\n", r"first node must be \[config\]"),
    (CFG + "conv:\n  filters: 4\n  bogus: 1\n", r"bogus is not supported in \[conv\]"),
    (CFG + "conv:\n  filters: four\n", r"\[conv\] filters can't convert to int"),
    (CFG + "conv:\n  filters: 4\nroute:\n  layers: 5\n", "route layer error, route layers index should < size of layers"),
    (CFG + "conv:\n  filters: 20\nyolo:\n  anchors: 1,2,3,4,5,6\n  classNum: 2\n", "class num error!"),
    (CFG + "conv:\n  filters: 21\nyolo:\n  anchors: 1,2,3,4\n  classNum: 2\n", r"\[yolo\] anchor num should be 6"),
    (CFG + "conv:\n  filters: 4\nyoloout:\n  layers: 0\n", "yoloout layer error, not a yolo layer"),
    ("config:\n  batch: 1\n  width: 0\n  height: 8\n  channels: 3\nconv:\n  filters: 4\n", "net config params err, params = 0 or < 0"),
    (CFG + "conv:\n  filters: 4\n  kSize: 3\n  kSizeY: 5\n", "only square kernels"),
    (CFG + "deconv:\n  filters: 4\n  groups: 2\n", "outside the convolutional path"),
    (CFG + "conv:\n  filters: 4\nconcatblock:\n  size: 1\n  branch:\n    empty:\n", r"size is not supported in \[concatblock\]"),
    (CFG + "conv:\n  filters: 4\nresblock:\n  size: 1\n  upsample:\n    stride: 2\n", r"upsample is not supported by \[ResBlockLayer\]"),
    (CFG + "conv:\n  filters: 4\nres2block:\n  base:\n    conv:\n      filters: 6\n  branch:\n    conv:\n      filters: 8\n", "base's outputs size is not equal"),
])
def test_build_errors(text, msg, tmp_path):
    with pytest.raises(netapi.MsnhnetError, match=msg):
        netapi.Net(_write(tmp_path, text))


def test_parser_details(tmp_path):
    text = (CFG + "# a comment line\nconv:   # trailing comment\n  filters: 4\n  kSize: 3\n  padding: 1\n  activation: leaky,0.25\n"
            "resblock:\n  size: 3\n  conv:\n    filters: 4\n    kSize: 1\n    dilation: 3\n  activation: relu\n"
            "route:\n  layers: -1,-4\nmaxpool:\n  kSize: 2\n  stride: 2\n")
    m = netapi.Net(_write(tmp_path, text))
    infos = m.layer_infos()
    assert [i["type"] for i in infos] == ["conv", "resblock", "resblock", "resblock", "route", "maxpool"]
    assert infos[4]["outC"] == 8 and infos[5]["outH"] == 4            # route -1,-4 = layers 3 and 0
    assert infos[1]["numWeights"] == 4 * 4 + 4                         # 1x1 conv + bias; dilation forced to 1 for k=1
    assert infos[1]["act"] == on.ACT["relu"] and infos[0]["act"] == on.ACT["leaky"]


def test_weight_count_errors_and_cpu_refusal(tmp_path):
    m = netapi.Net(_write(tmp_path, CFG + "conv:\n  filters: 4\n  kSize: 3\n  batchNorm: 1\n"))
    need = 4 * 3 * 9 + 4 * 4
    with pytest.raises(netapi.MsnhnetError, match=f"Load weights err, need > given. Needed :{need} given :10"):
        m.load_array(np.zeros(10, np.float32))
    with pytest.raises(netapi.MsnhnetError, match=f"Load weights err, need != given. Needed :{need} given :{need + 3}"):
        m.load_array(np.zeros(need + 3, np.float32))
    with pytest.raises(netapi.MsnhnetError, match="Gpu mode , can not run with cpu"):
        m.run_classify_cpu(np.zeros(3 * 64, np.float32))
    with pytest.raises(netapi.MsnhnetError, match="weights are not loaded"):
        m.run_classify(np.zeros(3 * 64, np.float32))


def test_reference_facade_error_protocol(tmp_path):
    L = netapi.lib()
    msg = ctypes.c_char_p()
    assert L.initMsnhnet() == 1
    assert L.buildMsnhnet(ctypes.byref(msg), b"/nonexistent.msnhnet", b"/nonexistent.msnhbin", 0, 0) == -1
    assert b"open failed" in msg.value
    w = ctypes.c_int(); h = ctypes.c_int(); c = ctypes.c_int()
    cudnn = ctypes.c_int(5)
    assert L.withCUDNN(ctypes.byref(cudnn)) == 1 and cudnn.value == 0
    assert L.dispose() == 1


def _ref_nms_python(rows, thr):
    """the reference's greedy loop, written out naively"""
    rows = [list(r) for r in rows]
    classes = []
    for r in rows:
        if int(r[6]) not in classes:
            classes.append(int(r[6]))
    out = []
    for c in classes:
        cur = [r for r in rows if int(r[6]) == c]
        if len(cur) == 1:
            out.append(cur[0]); continue
        while cur:
            bi = max(range(len(cur)), key=lambda j: (cur[j][4], -j))
            best = cur.pop(bi)
            out.append(best)
            cur = [r for r in cur if not (on.iou(r[:4], best[:4]) > thr)]
    return np.array(out, np.float32).reshape(-1, 7)


@pytest.mark.parametrize("seed", range(6))
def test_nms_variants_agree(seed):
    rng = np.random.default_rng(seed)
    n = 300
    rows = np.zeros((n, 7), np.float32)
    rows[:, 0:2] = rng.uniform(0, 200, (n, 2))
    rows[:, 2:4] = rng.uniform(5, 80, (n, 2))
    rows[:, 4] = np.round(rng.uniform(0.5, 1, n), 2)          # rounded: plenty of objectness ties
    rows[:, 5] = rng.uniform(0, 1, n)
    rows[:, 6] = rng.integers(0, 7, n)
    if seed % 2:
        rows[rng.integers(0, n, 20), 2] = np.inf               # exp overflow: NaN IoU never suppresses
    rows = rows[np.argsort(-(rows[:, 4] * rows[:, 5]), kind="stable")]
    a = netapi.nms(rows, 0.45, fast=False)
    b = netapi.nms(rows, 0.45, fast=True)
    c = _ref_nms_python(rows, 0.45)
    assert np.array_equal(a, b, equal_nan=True)
    assert np.array_equal(a, c, equal_nan=True)
    assert 0 < len(a) < n


def test_boxes_to_image_matches_the_oracle():
    import msnh_oracle_net as on
    rng = np.random.default_rng(8)
    boxes = rng.uniform(0, 600, (40, 7)).astype(np.float32)
    for (nw, nh, ow, oh) in [(608, 608, 1280, 720), (608, 608, 480, 640), (416, 416, 416, 416), (320, 224, 1000, 333)]:
        for padded in (True, False):
            got = netapi.boxes_to_image(boxes, nw, nh, ow, oh, padded)
            for i in range(len(boxes)):
                want = on.bbox_resize2org(boxes[i, :4], nw, nh, ow, oh, no_pad=not padded)
                assert np.array_equal(got[i, :4], want)
                assert np.array_equal(got[i, 4:], boxes[i, 4:])
    with pytest.raises(netapi.MsnhnetError):
        netapi.boxes_to_image(boxes, 0, 608, 10, 10)


def test_pack_file_round_trip_and_rejections(tmp_path):
    """the packed-constants file beside a weights file: what was written comes back byte for byte, and a file that belongs to other
    weights, another plan or another library build, or that is cut short, is refused (tests/cpp/packfile_check.cpp, host code only)"""
    import subprocess
    exe = str(tmp_path / "packfile_check")
    lib = os.path.join(ROOT, "msnhnet_amd", "lib")
    cmd = ["g++", "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "msnhnet_amd", "host", "include"), os.path.join(ROOT, "tests", "cpp", "packfile_check.cpp"),
           "-o", exe, "-L" + lib, "-lMsnhnet", "-lmsnh_hip", "-Wl,-rpath," + lib]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    r = subprocess.run([exe, str(tmp_path)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), r.stdout


def test_task_pool(tmp_path):
    """the worker pool of the box stage (tests/cpp/taskpool_check.cpp, host code only): each index once, exceptions propagate,
    idle workers use no CPU time -- a spinning team exhausts a container's CPU allowance and stalls the thread that feeds the GPU"""
    import subprocess
    exe = str(tmp_path / "taskpool_check")
    lib = os.path.join(ROOT, "msnhnet_amd", "lib")
    cmd = ["g++", "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "msnhnet_amd", "host", "include"), os.path.join(ROOT, "tests", "cpp", "taskpool_check.cpp"),
           "-o", exe, "-L" + lib, "-lMsnhnet", "-lmsnh_hip", "-Wl,-rpath," + lib, "-lpthread"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), r.stdout


def test_host_threads_under_sanitizers(tmp_path):
    """the multi-threaded host code -- the worker pool (tests/cpp/taskpool_check.cpp) and the box stage's parallel per-(image, class)
    suppression over it (tests/cpp/nms_pool_check.cpp, which also checks it against the reference-shaped loop) -- built from the host
    library's sources with -fsanitize=thread and with -fsanitize=address,undefined and run: no report, exit status 0"""
    import glob
    import subprocess
    host = os.path.join(ROOT, "msnhnet_amd", "host")
    lib = os.path.join(ROOT, "msnhnet_amd", "lib")
    inc = ["-I" + os.path.join(host, "include"), "-I" + os.path.join(ROOT, "include")]
    srcs = sorted(glob.glob(os.path.join(host, "src", "*.cpp")))
    builds = []
    for tag, san in (("tsan", "-fsanitize=thread"), ("asan", "-fsanitize=address,undefined")):
        common = ["g++", "-std=c++17", "-O1", "-g", san, "-fno-sanitize-recover=undefined", "-fopenmp-simd"] + inc
        tp = str(tmp_path / f"taskpool_{tag}")
        nm = str(tmp_path / f"nms_pool_{tag}")
        builds.append((tp, subprocess.Popen(common + [os.path.join(ROOT, "tests", "cpp", "taskpool_check.cpp"), os.path.join(host, "src", "TaskPool.cpp"), "-o", tp, "-lpthread"],
                                            stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        builds.append((nm, subprocess.Popen(common + [os.path.join(ROOT, "tests", "cpp", "nms_pool_check.cpp")] + srcs + ["-o", nm, "-L" + lib, "-lmsnh_hip", "-Wl,-rpath," + lib, "-lpthread"],
                                            stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    for exe, p in builds:
        out, _ = p.communicate(timeout=600)
        assert p.returncode == 0, out[-3000:]
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66", ASAN_OPTIONS="detect_leaks=1 exitcode=67", UBSAN_OPTIONS="print_stacktrace=1")
    for exe, _ in builds:
        r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300, env=env)
        assert r.returncode == 0 and r.stdout.strip().endswith("ok") and "Sanitizer" not in r.stdout, (exe, r.stdout[-3000:])
