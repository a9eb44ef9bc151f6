"""Pins the oracle (oracle/msnh_oracle.c + oracle/msnh_oracle_net.py) without a GPU:

  1. against golden vectors produced by the reference's own CPU forward (tests/golden/ref_golden.npz, written by
     tests/golden/make_golden.py from oracle/_ref): whole tensors for 20 micro graphs covering every op and block
     type, per-layer statistics + final outputs for the five benchmark architectures;
  2. live against oracle/_ref when that library is present (layer by layer);
  3. against what the mathematics fixes: brute-force double-precision cross-correlation, identity kernels,
     1x1 conv == matrix product, depthwise == per-channel correlation, brute-force pooling, closed forms for
     batch-norm / activations / YOLO decode, hand-computed IoU and NMS cases.
A dropped term, a transposed operand or a wrong index in any oracle function fails at least one of these.
"""
import os
import tempfile

import numpy as np
import pytest

import msnh_oracle_net as on
import netutil as nu
import refshim
from msnhnet_amd import zoo

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_golden.npz"))
MICRO = bytes(GOLD["micro/names"]).decode().split("\n")


def _write(tmp, name, text, weights):
    netp = os.path.join(tmp, name + ".msnhnet")
    binp = os.path.join(tmp, name + ".msnhbin")
    with open(netp, "w") as f:
        f.write(text)
    np.asarray(weights, np.float32).tofile(binp)
    return netp, binp


@pytest.mark.parametrize("name", MICRO)
def test_oracle_matches_reference_golden_micro(name, tmp_path):
    text = bytes(GOLD[f"micro/{name}/graph"]).decode()
    netp, binp = _write(str(tmp_path), name, text, GOLD[f"micro/{name}/weights"])
    o = on.OracleNet(netp, binp)
    outs = o.run(GOLD[f"micro/{name}/input"])
    for i, got in enumerate(outs):
        ref = GOLD[f"micro/{name}/out{i}"]
        if ref.size == 0:
            continue
        assert nu.rel_err(got.ravel(), ref) <= 3e-6, (name, i)
    ref_boxes = GOLD[f"micro/{name}/boxes"]
    if len(ref_boxes):
        assert len(o.boxes) == len(ref_boxes)
        assert nu.rel_err(nu.sort_boxes(o.boxes), nu.sort_boxes(ref_boxes)) <= 3e-6


def _stats(a):
    a = np.asarray(a, np.float64).ravel()
    fin = np.isfinite(a)
    v = a[fin]
    idx = (np.arange(16) * 7919) % max(a.size, 1)
    return np.array([a.size, fin.sum(), v.sum() if v.size else 0, np.abs(v).sum() if v.size else 0, v.max() if v.size else 0,
                     v.min() if v.size else 0] + [a[i] if a.size else 0 for i in idx], np.float64)


@pytest.mark.parametrize("arch", ["resnet18", "resnet50", "mobilenetv2", "yolov3", "yolov4"])
def test_oracle_matches_reference_golden_nets(arch, tmp_path):
    size = int(GOLD[f"net/{arch}/size"][0])
    netp, binp, gw = zoo.write_model(arch, str(tmp_path), 1, size, seed=11)
    x = zoo.seeded_input(1, 3, size, size, 12)[0]
    # the fixture is only meaningful if the seeded data is what it was generated from
    assert abs(x.astype(np.float64).sum() - GOLD[f"net/{arch}/input_sum"][0]) < 1e-6
    assert abs(np.fromfile(binp, np.float32).astype(np.float64).sum() - GOLD[f"net/{arch}/weights_sum"][0]) < 1e-6
    o = on.OracleNet(netp, binp)
    outs = o.run(x)
    gold = GOLD[f"net/{arch}/stats"]
    assert len(outs) == len(gold)
    tol = 5e-4 if arch == "mobilenetv2" else 5e-5       # FMA contraction in the reference build vs none here
    for i, got in enumerate(outs):
        s, g = _stats(got), gold[i]
        assert s[0] == g[0] and s[1] == g[1], (arch, i, "size / finite count")
        if g[0] == 0:
            continue
        scale = max(abs(g[4]), abs(g[5]), 1e-30)
        assert abs(s[3] - g[3]) <= tol * max(g[3], 1e-30), (arch, i, "abs-sum")
        assert abs(s[4] - g[4]) <= tol * scale and abs(s[5] - g[5]) <= tol * scale, (arch, i, "max / min")
        fin = np.isfinite(g[6:])
        assert (np.isfinite(s[6:]) == fin).all()
        assert np.abs(s[6:][fin] - g[6:][fin]).max() <= 20 * tol * scale, (arch, i, "samples")
    if arch.startswith("yolo"):
        rb = GOLD[f"net/{arch}/boxes"]
        assert abs(len(o.boxes) - len(rb)) <= 1
    else:
        assert int(np.argmax(outs[-1])) == int(np.argmax(GOLD[f"net/{arch}/final"]))
        assert nu.rel_err(outs[-1].ravel(), GOLD[f"net/{arch}/final"]) <= 10 * tol


@pytest.mark.skipif(not refshim.available(), reason="oracle/_ref is not built here")
@pytest.mark.parametrize("arch,size", [("resnet18", 224), ("mobilenetv2", 224), ("yolov3", 64), ("yolov4", 64), ("yolov3_tiny", 96), ("yolov5s", 64)])
def test_oracle_matches_reference_live(arch, size, tmp_path):
    netp, binp, gw = zoo.write_model(arch, str(tmp_path), 1, size, seed=21)
    x = zoo.seeded_input(1, 3, size, size, 22)[0]
    r = refshim.RefNet(netp, binp, scalar=True)
    ro = r.run(x)
    o = on.OracleNet(netp, binp)
    oo = o.run(x)
    tol = 5e-4 if arch == "mobilenetv2" else 2e-5
    infos = r.layer_infos()
    for i, (a, b) in enumerate(zip(ro, oo)):
        if not a.size:
            continue
        if infos[i]["type"] == "yolo":      # decoded values amplify the logit error, see netutil.yolo_layer_err
            assert nu.yolo_layer_err(b.ravel(), a, ro[i - 1], 85, size / infos[i]["outH"], 5 if arch == "yolov5s" else 3) <= tol, (arch, i)
        else:
            assert nu.rel_err(b.ravel(), a) <= tol, (arch, i)
    if arch.startswith("yolo"):
        assert len(r.boxes()) == len(o.boxes)


# ---- what the mathematics fixes ------------------------------------------------------------------------------------
def _brute_conv(x, w, stride, pad, dil, groups):
    b, c, h, wd = x.shape
    oc, cg, k, _ = w.shape
    ext = dil * (k - 1) + 1
    oh, ow = (h + 2 * pad - ext) // stride + 1, (wd + 2 * pad - ext) // stride + 1
    xp = np.zeros((b, c, h + 2 * pad, wd + 2 * pad), np.float64)
    xp[:, :, pad:pad + h, pad:pad + wd] = x
    out = np.zeros((b, oc, oh, ow), np.float64)
    ocg = oc // groups
    for o in range(oc):
        g = o // ocg
        for i in range(k):
            for j in range(k):
                patch = xp[:, g * cg:(g + 1) * cg, i * dil:i * dil + (oh - 1) * stride + 1:stride, j * dil:j * dil + (ow - 1) * stride + 1:stride]
                out[:, o] += np.einsum("bchw,c->bhw", patch, w[o, :, i, j].astype(np.float64))
    return out


@pytest.mark.parametrize("c,oc,k,stride,pad,dil,groups", [(3, 4, 3, 1, 1, 1, 1), (4, 6, 3, 2, 0, 1, 2), (2, 2, 5, 1, 2, 1, 1), (4, 4, 3, 1, 2, 2, 1),
                                                          (6, 6, 3, 1, 1, 1, 6), (5, 3, 1, 1, 0, 1, 1), (3, 2, 7, 2, 3, 1, 1)])
def test_conv_is_cross_correlation(c, oc, k, stride, pad, dil, groups):
    rng = np.random.default_rng(k * 10 + c)
    x = rng.standard_normal((2, c, 9, 8)).astype(np.float32)
    w = rng.standard_normal((oc, c // groups, k, k)).astype(np.float32)
    got = on.conv(x, w, oc, k, stride, pad, dil, groups)
    ref = _brute_conv(x, w, stride, pad, dil, groups)
    assert got.shape == ref.shape
    assert nu.rel_err(got, ref) <= 2e-6


def test_conv_identity_and_shift_kernels():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((1, 3, 6, 7)).astype(np.float32)
    w = np.zeros((3, 3, 3, 3), np.float32)
    for ch in range(3):
        w[ch, ch, 1, 1] = 1                      # centre tap: identity
    assert np.array_equal(on.conv(x, w, 3, 3, 1, 1), x)
    w[:] = 0
    for ch in range(3):
        w[ch, ch, 1, 2] = 1                      # tap to the right: out[y][x] = in[y][x+1] (no kernel flip)
    y = on.conv(x, w, 3, 3, 1, 1)
    assert np.array_equal(y[..., :-1], x[..., 1:]) and (y[..., -1] == 0).all()
    w[:] = 0
    for ch in range(3):
        w[ch, ch, 2, 1] = 1                      # tap below: out[y][x] = in[y+1][x]
    y = on.conv(x, w, 3, 3, 1, 1)
    assert np.array_equal(y[:, :, :-1], x[:, :, 1:]) and (y[:, :, -1] == 0).all()


def test_conv_1x1_is_matrix_product_and_bias_bn_closed_form():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((2, 5, 4, 3)).astype(np.float32)
    w = rng.standard_normal((7, 5, 1, 1)).astype(np.float32)
    bias = rng.standard_normal(7).astype(np.float32)
    ref = np.einsum("oc,bchw->bohw", w[:, :, 0, 0].astype(np.float64), x.astype(np.float64))
    assert nu.rel_err(on.conv(x, w, 7, 1, bias=bias), ref + bias.reshape(1, -1, 1, 1)) <= 1e-6
    g, beta, mean, var = [rng.uniform(0.5, 1.5, 7).astype(np.float32) for _ in range(4)]
    bn = ((ref - mean.reshape(1, -1, 1, 1)) / np.sqrt(var.reshape(1, -1, 1, 1).astype(np.float64) + 1e-5)) * g.reshape(1, -1, 1, 1) + beta.reshape(1, -1, 1, 1)
    got = on.conv(x, w, 7, 1, bn4=np.concatenate([g, beta, mean, var]), act="leaky", act_param=0.1)
    assert nu.rel_err(got, np.where(bn > 0, bn, 0.1 * bn)) <= 2e-6


def test_activation_special_values():
    f = lambda v, a, p=0.1: float(on.activate(np.array([v], np.float32), a, p)[0])
    assert f(0, "relu6") == 0 and f(6, "relu6") == 6 and f(7.5, "relu6") == 6 and f(-1, "relu6") == 0 and f(3, "relu6") == 3
    assert f(-2, "leaky") == pytest.approx(-0.2) and f(-2, "leaky", 0.25) == pytest.approx(-0.5) and f(2, "leaky") == 2
    assert f(-3, "relu") == 0 and f(3, "relu") == 3
    assert f(0, "mish") == 0 and f(0, "swish") == 0 and f(0, "logistic") == 0.5
    assert f(25, "mish") == pytest.approx(25.0)                      # softplus threshold +20: tanh(x) == 1
    assert f(-25, "mish") == pytest.approx(-25 * np.tanh(np.exp(-25.0)), rel=1e-5)
    assert f(1, "mish") == pytest.approx(1 * np.tanh(np.log1p(np.exp(1.0))), rel=1e-6)
    assert f(2, "swish") == pytest.approx(2 / (1 + np.exp(-2.0)), rel=1e-6)
    assert f(5, "none") == 5


def test_pooling_and_upsample_brute_force():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 3, 7, 9)).astype(np.float32)
    for k, s, p in ((2, 2, 0), (3, 2, 1), (5, 1, 2), (3, 1, 1)):
        oh, ow = (7 + 2 * p - k) // s + 1, (9 + 2 * p - k) // s + 1
        mx = np.empty((2, 3, oh, ow), np.float32)
        av = np.empty((2, 3, oh, ow), np.float64)
        for i in range(oh):
            for j in range(ow):
                ys = [y for y in range(i * s - p, i * s - p + k) if 0 <= y < 7]
                xs = [v for v in range(j * s - p, j * s - p + k) if 0 <= v < 9]
                win = x[:, :, ys][:, :, :, xs]
                mx[:, :, i, j] = win.max(axis=(2, 3))
                av[:, :, i, j] = win.astype(np.float64).mean(axis=(2, 3))          # divides by the VALID count
        assert np.array_equal(on.maxpool(x, k, s, p), mx)
        assert nu.rel_err(on.avgpool(x, k, s, p), av) <= 1e-6
    up = on.upsample(x, 2)
    assert up.shape == (2, 3, 14, 18)
    for j in range(14):
        for i in range(18):
            assert np.array_equal(up[:, :, j, i], x[:, :, j // 2, i // 2])
    assert np.array_equal(on.upsample(x, 3, 0.5), 0.5 * np.repeat(np.repeat(x, 3, axis=2), 3, axis=3))


def test_connected_is_matrix_vector():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((3, 20, 1, 1)).astype(np.float32)
    w = rng.standard_normal((6, 20)).astype(np.float32)
    b = rng.standard_normal(6).astype(np.float32)
    ref = x.reshape(3, 20).astype(np.float64) @ w.T.astype(np.float64) + b
    assert nu.rel_err(on.connected(x, w, b, 6).reshape(3, 6), ref) <= 1e-6


def test_yolo_decode_closed_form():
    rng = np.random.default_rng(4)
    cls, h, w = 3, 4, 5
    per = 5 + cls
    x = rng.standard_normal((1, 3 * per, h, w)).astype(np.float32) * 2
    anchors = np.array([10, 14, 23, 27, 37, 58], np.float32)
    out = on.yolo_decode(x, cls, anchors, 8.0)
    sig = lambda v: 1 / (1 + np.exp(-v.astype(np.float64)))
    cols, rows = np.meshgrid(np.arange(w), np.arange(h))
    for a in range(3):
        p = x[0, a * per:(a + 1) * per]
        assert nu.rel_err(out[0, a * per + 0], (sig(p[0]) + cols) * 8.0) <= 1e-6
        assert nu.rel_err(out[0, a * per + 1], (sig(p[1]) + rows) * 8.0) <= 1e-6
        assert nu.rel_err(out[0, a * per + 2], anchors[2 * a] * np.exp(p[2].astype(np.float64))) <= 1e-6
        assert nu.rel_err(out[0, a * per + 3], anchors[2 * a + 1] * np.exp(p[3].astype(np.float64))) <= 1e-6
        assert nu.rel_err(out[0, a * per + 4:(a + 1) * per], sig(p[4:])) <= 1e-6
    big = np.full((1, 3 * per, 1, 1), 100.0, np.float32)            # exp overflow -> +inf, like the benchmark weights
    o = on.yolo_decode(big, cls, anchors, 32.0)
    assert np.isinf(o[0, 2, 0, 0]) and o[0, 4, 0, 0] == 1.0


def test_iou_plus_one_convention_and_nan():
    # boxes [0,10]x[0,10] and [5,15]x[0,10] with the inclusive-pixel +1: inter = 6*11, areas 11*11
    a, b = [5, 5, 10, 10], [10, 5, 10, 10]
    assert on.iou(a, b) == pytest.approx(66 / (121 + 121 - 66))
    assert on.iou(a, a) == pytest.approx(1.0)
    assert on.iou([0, 0, 2, 2], [100, 100, 2, 2]) == 0.0
    # touching boxes still overlap by one "pixel" column under the +1 convention
    assert on.iou([0, 0, 2, 2], [2, 0, 2, 2]) == pytest.approx(3 / (9 + 9 - 3))
    assert np.isnan(on.iou([5, 5, np.inf, np.inf], [5, 5, np.inf, np.inf]))


def _head(boxes, cls_num, hw):
    """builds one decoded head [3*(5+cls), hw] holding the given (anchor, pixel) -> (x,y,w,h,obj,scores...) entries"""
    per = 5 + cls_num
    t = np.zeros((3 * per, hw, 1), np.float32)
    for (a, p), v in boxes.items():
        t[a * per:(a + 1) * per, p, 0] = v
    return t


def test_yolo_out_hand_cases():
    cls = 3
    big = [50, 50, 40, 40]
    near = [52, 50, 40, 40]          # IoU with big ~ 0.9 -> suppressed when same class
    far = [150, 150, 40, 40]
    entries = {
        (0, 0): big + [0.9, 0.1, 0.8, 0.1],       # class 1, kept (highest objectness of class 1)
        (0, 1): near + [0.8, 0.1, 0.9, 0.1],      # class 1, suppressed by the first although its obj*cls key is equal
        (1, 0): near + [0.7, 0.9, 0.1, 0.1],      # class 0, alone in its class -> passes through
        (1, 2): far + [0.6, 0.2, 0.7, 0.1],       # class 1, far away -> kept
        (2, 3): big + [0.3, 0.9, 0.9, 0.9],       # objectness below the threshold -> never a candidate
        (2, 1): big + [0.5, 0.9, 0.9, 0.9],       # objectness == threshold: strict '>' drops it
    }
    out = on.yolo_out([_head(entries, cls, 4)], cls, 0.5, 0.45)
    got = sorted((round(float(b[4]), 3), int(b[6])) for b in out)
    assert got == sorted([(0.9, 1), (0.7, 0), (0.6, 1)])
    # NMS ranks by objectness, not by objectness*class score: swap which of the overlapping pair has more objectness
    entries[(0, 0)] = big + [0.8, 0.1, 0.99, 0.1]
    entries[(0, 1)] = near + [0.9, 0.1, 0.6, 0.1]
    out = on.yolo_out([_head(entries, cls, 4)], cls, 0.5, 0.45)
    assert sorted(round(float(b[4]), 3) for b in out if int(b[6]) == 1) == [0.6, 0.9]
    # threshold is strict: iou exactly at the threshold is kept
    e2 = {(0, 0): [5, 5, 10, 10, 0.9, 1, 0, 0], (0, 1): [10, 5, 10, 10, 0.8, 1, 0, 0]}
    thr = on.iou([10, 5, 10, 10], [5, 5, 10, 10])
    assert len(on.yolo_out([_head(e2, cls, 2)], cls, 0.5, thr)) == 2
    assert len(on.yolo_out([_head(e2, cls, 2)], cls, 0.5, np.nextafter(np.float32(thr), np.float32(0)))) == 1
    assert len(on.yolo_out([_head({}, cls, 2)], cls, 0.5, 0.5)) == 0


def test_parse_msnhnet_duplicate_keys_and_expansion(tmp_path):
    g = zoo.yolov3(batch=1, size=64)
    netp = os.path.join(str(tmp_path), "y.msnhnet")
    with open(netp, "w") as f:
        f.write(g.text())
    o = on.OracleNet(netp)
    assert len(o.top) == 53                      # 23 residual blocks expanded from 5 `size:` entries
    assert [k for k, _ in o.top].count("resblock") == 23


# ---- pre / post-processing around the graph ------------------------------------------------------------------------
LETTERBOX_SHAPES = [(480, 640, 608, 608), (640, 480, 416, 416), (300, 300, 608, 608), (720, 1280, 608, 608), (100, 37, 64, 64),
                    (608, 608, 608, 608), (50, 80, 224, 224), (33, 33, 32, 32)]


@pytest.mark.parametrize("h,w,nw,nh", LETTERBOX_SHAPES)
def test_letterbox_against_reference(h, w, nw, nh):
    """The restatement against CVUtil::getPaddingZeroF32C3 itself.  The reference build lets the compiler fuse
    multiply-adds in the interpolation, the restatement does not: a few pixels per million land one 8-bit step apart."""
    if not refshim.available():
        pytest.skip("reference build not present")
    rng = np.random.default_rng(h * 7 + w)
    img = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
    for half in (False, True):
        for shuffle in (False, True):
            a = on.letterbox_u8(img, nw, nh, half, shuffle)
            b = refshim.letterbox_u8(img, nw, nh, half, shuffle)
            step = 1 / 127.5 if half else 1 / 255.0
            d = np.abs(a - b)
            assert d.max() <= step * 1.001
            assert (d > 1e-7).mean() <= 1e-4


def test_letterbox_mathematics():
    rng = np.random.default_rng(11)
    # same size: a pure layout change and scale
    img = rng.integers(0, 256, (24, 24, 3), dtype=np.uint8)
    out = on.letterbox_u8(img, 24, 24)
    assert np.array_equal(out, img.transpose(2, 0, 1).astype(np.float32) / np.float32(255.0))
    assert np.array_equal(on.letterbox_u8(img, 24, 24, shuffle_rgb=True), out[::-1])
    assert np.array_equal(on.letterbox_u8(img, 24, 24, half_init=True),
                          (img.transpose(2, 0, 1).astype(np.float32) - np.float32(127.5)) / np.float32(127.5))
    # padding: a wide image gets rows of 127 above (diff/2) and below (diff - diff/2)
    wide = rng.integers(0, 256, (10, 15, 3), dtype=np.uint8)
    o = on.letterbox_u8(wide, 15, 15)
    assert np.all(o[:, :2] == np.float32(127 / 255.0)) and np.all(o[:, 12:] == np.float32(127 / 255.0))
    assert np.array_equal(o[:, 2:12], wide.transpose(2, 0, 1).astype(np.float32) / np.float32(255.0))
    tall = rng.integers(0, 256, (15, 10, 3), dtype=np.uint8)
    o = on.letterbox_u8(tall, 15, 15)
    assert np.all(o[:, :, :2] == np.float32(127 / 255.0)) and np.all(o[:, :, 12:] == np.float32(127 / 255.0))
    # halving an image whose 2x2 blocks are constant returns the block values (samples fall half-way between equal pixels)
    small = rng.integers(0, 256, (16, 16, 3), dtype=np.uint8)
    big = np.repeat(np.repeat(small, 2, axis=0), 2, axis=1)
    assert np.array_equal(on.letterbox_u8(big, 16, 16), small.transpose(2, 0, 1).astype(np.float32) / np.float32(255.0))
    # against a library bilinear resize (half-pixel centres, no corner alignment) when shrinking: truncation of two
    # float evaluations of the same real number may differ by one step, never more
    import torch
    src = rng.integers(0, 256, (90, 90, 3), dtype=np.uint8)
    ours = on.letterbox_u8(src, 40, 40) * 255.0
    t = torch.from_numpy(src.transpose(2, 0, 1).astype(np.float32))[None]
    lib = torch.nn.functional.interpolate(t, size=(40, 40), mode="bilinear", align_corners=False)[0].numpy()
    assert np.abs(ours - np.floor(lib)).max() <= 1.0
    assert (np.abs(ours - np.floor(lib)) > 0).mean() < 0.02
    # enlarging: the reference's weights sum to zero on the last row and column (second sample index clamped, first not)
    up = on.letterbox_u8(np.full((8, 8, 3), 200, np.uint8), 16, 16) * 255.0
    assert np.all(up[:, :15, :15] == 200) and np.all(up[:, 15, :] == 0) and np.all(up[:, :, 15] == 0)


PREPROC_SHAPES = [(480, 640, 224, 224), (50, 80, 64, 48), (33, 33, 32, 32), (224, 224, 224, 224), (20, 33, 96, 96)]


@pytest.mark.parametrize("h,w,nw,nh", PREPROC_SHAPES)
def test_preproc_against_reference(h, w, nw, nh):
    """The plain-resize variants against CVUtil::getImgDataF32C3 / getGoogLenetF32C3 / getTransformedF32C3 / getCaffeModeF32C3
    themselves.  As for the letterbox, the reference build fuses multiply-adds: a few pixels per million land one 8-bit step
    apart, and the GoogLeNet form differs by an ulp."""
    if not refshim.available():
        pytest.skip("reference build not present")
    rng = np.random.default_rng(h * 5 + w)
    img = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
    mean, std = (0.4, 0.5, 0.6), (0.2, 0.3, 0.25)
    step = {"f32c3": 1 / 255.0, "f32c3_half": 1 / 127.5, "googlenet": 0.458 / 255.0, "transformed": 1 / 255.0 / 0.2, "caffe": 1.0}
    for kind in on.PREPROC_KINDS:
        for shuffle in (False, True):
            a = on.preproc_u8(img, nw, nh, kind, mean, std, shuffle)
            b = refshim.preproc_u8(img, nw, nh, kind, mean, std, shuffle)
            d = np.abs(a - b)
            assert d.max() <= step[kind] * 1.001, (kind, d.max())
            assert (d > 1e-6).mean() <= 1e-3, (kind, (d > 1e-6).mean())


def test_preproc_mathematics():
    rng = np.random.default_rng(21)
    img = rng.integers(0, 256, (12, 17, 3), dtype=np.uint8)
    chw = img.transpose(2, 0, 1).astype(np.float32)
    f = np.float32
    # same size: only the normalisation, in the reference's float expressions
    assert np.array_equal(on.preproc_u8(img, 17, 12, "f32c3"), chw / f(255.0))
    assert np.array_equal(on.preproc_u8(img, 17, 12, "f32c3", shuffle_rgb=True), (chw / f(255.0))[::-1])
    assert np.array_equal(on.preproc_u8(img, 17, 12, "f32c3_half"), (chw - f(127.5)) / f(127.5))
    gs, gm = np.array([0.229, 0.224, 0.225], f), np.array([0.485, 0.456, 0.406], f)
    want = chw / f(255.0) * (gs / f(0.5))[:, None, None] + ((gm - f(0.5)) / f(0.5))[:, None, None]
    assert np.array_equal(on.preproc_u8(img, 17, 12, "googlenet"), want.astype(f))
    mean, std = np.array([0.4, 0.5, 0.6], f), np.array([0.2, 0.3, 0.25], f)
    assert np.array_equal(on.preproc_u8(img, 17, 12, "transformed", mean, std), ((chw / f(255.0)) - mean[:, None, None]) / std[:, None, None])
    assert np.array_equal(on.preproc_u8(img, 17, 12, "caffe"), chw - np.array([123.68, 116.779, 103.939], f)[:, None, None])
    # the GoogLeNet form is the ImageNet normalisation re-expressed for a net trained on (x - 0.5) / 0.5 inputs (closed form, double)
    x = chw.astype(np.float64) / 255.0
    ident = (x * gs.astype(np.float64)[:, None, None] + gm.astype(np.float64)[:, None, None] - 0.5) / 0.5
    assert np.abs(on.preproc_u8(img, 17, 12, "googlenet") - ident).max() < 1e-6
    # a square image: plain resize == letterbox (nothing to pad)
    sq = rng.integers(0, 256, (30, 30, 3), dtype=np.uint8)
    assert np.array_equal(on.preproc_u8(sq, 20, 20, "f32c3"), on.letterbox_u8(sq, 20, 20))
    # separate scale factors per axis: halving only the width of an image whose column pairs are equal returns the pair values.
    # Along the axis that keeps its size the reference's weights (i1 - s) and (s - i0) are both zero on the last row / column
    # (second sample index clamped to the first): that line comes out 0, as it does when enlarging.
    small = rng.integers(0, 256, (9, 8, 3), dtype=np.uint8)
    want = small.transpose(2, 0, 1).astype(f) / f(255.0)
    wide = np.repeat(small, 2, axis=1)
    got = on.preproc_u8(wide, 8, 9, "f32c3")
    assert np.array_equal(got[:, :8], want[:, :8]) and np.all(got[:, 8] == 0)
    tall = np.repeat(small, 2, axis=0)
    got = on.preproc_u8(tall, 8, 9, "f32c3")
    assert np.array_equal(got[:, :, :7], want[:, :, :7]) and np.all(got[:, :, 7] == 0)


def test_preproc_against_golden():
    """vectors written by the reference build (present also where the build is not)"""
    idx = 0
    while f"preproc/{idx}/case" in GOLD.files:
        h, w, nw, nh, seed = (int(v) for v in GOLD[f"preproc/{idx}/case"])
        img = np.random.default_rng(seed).integers(0, 256, (h, w, 3), dtype=np.uint8)
        mean, std = GOLD[f"preproc/{idx}/mean"], GOLD[f"preproc/{idx}/std"]
        for kind in on.PREPROC_KINDS:
            want = GOLD[f"preproc/{idx}/{kind}"]
            got = on.preproc_u8(img, nw, nh, kind, mean, std, bool(idx % 2))
            scale = {"f32c3": 255.0, "f32c3_half": 127.5, "googlenet": 255.0 / 0.44, "transformed": 255.0 * float(std.min()), "caffe": 1.0}[kind]
            d = np.abs(got - want) * scale
            assert d.max() <= 1.05 and (d > 1e-3).mean() <= 1e-3, (idx, kind, d.max())
        idx += 1
    assert idx >= 3


def test_bbox_back_to_image():
    # 1280x720 letterboxed into 608x608: scale 0.475, 133 rows of padding above; the centre maps to the centre
    b = on.bbox_resize2org([304.0, 304.0, 95.0, 47.5], 608, 608, 1280, 720)
    assert np.allclose(b, [640.0, 360.0, 200.0, 100.0], rtol=1e-6)
    b = on.bbox_resize2org([304.0, 304.0, 95.0, 47.5], 608, 608, 720, 1280)
    assert np.allclose(b, [360.0, 640.0, 200.0, 100.0], rtol=1e-6)
    b = on.bbox_resize2org([100.0, 50.0, 10.0, 20.0], 416, 416, 832, 416, no_pad=True)
    assert np.allclose(b, [200.0, 50.0, 20.0, 20.0], rtol=1e-6)
    if refshim.available():
        rng = np.random.default_rng(5)
        for _ in range(50):
            box = rng.uniform(0, 600, 4).astype(np.float32)
            cw, ch, ow, oh = (int(v) for v in rng.integers(32, 2000, 4))
            for no_pad in (False, True):
                assert np.array_equal(on.bbox_resize2org(box, cw, ch, ow, oh, no_pad), refshim.bbox_resize2org(box, cw, ch, ow, oh, no_pad))


def test_letterbox_and_bbox_against_golden():
    """the same two comparisons against vectors the reference build wrote (present also where the build is not)"""
    idx = 0
    while f"letterbox/{idx}/case" in GOLD.files:
        h, w, nw, nh, seed = (int(v) for v in GOLD[f"letterbox/{idx}/case"])
        img = np.random.default_rng(seed).integers(0, 256, (h, w, 3), dtype=np.uint8)
        for shuffle in (0, 1):
            want = GOLD[f"letterbox/{idx}/shuffle{shuffle}"].astype(np.int32)
            got = np.rint(on.letterbox_u8(img, nw, nh, False, bool(shuffle)) * 255.0).astype(np.int32)
            assert np.abs(got - want).max() <= 1 and (got != want).mean() <= 1e-3
        idx += 1
    assert idx >= 4
    for row in GOLD["bbox/rows"]:
        box = row[:4].astype(np.float32)
        cw, ch, ow, oh = (int(v) for v in row[4:8])
        assert np.array_equal(on.bbox_resize2org(box, cw, ch, ow, oh, False), row[8:12].astype(np.float32))
        assert np.array_equal(on.bbox_resize2org(box, cw, ch, ow, oh, True), row[12:16].astype(np.float32))
