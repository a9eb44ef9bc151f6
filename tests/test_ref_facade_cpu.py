"""What swapRGB means in the reference's C facade, taken from the facade itself (src/c_api/MsnhnetLib.cpp compiled into oracle/_ref):
for every PredDataType and both values of swapRGB, runClassifyList / runYoloList return what the reference's network returns on the
CVUtil input form with needShuffleRGB = netutil.facade_shuffle(...), and not what it returns with the other value.  The GPU facade
tests take their expectation from the same table and from the reference's facade directly."""
import os

import numpy as np
import pytest

import netutil as nu
import refshim

pytestmark = pytest.mark.skipif(not refshim.available(), reason="reference build not present")
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "ref_golden.npz"))


def _image(seed, h, w):
    rng = np.random.default_rng(seed)
    img = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
    img[..., 0] //= 4                               # very different first and third channel: exchanging them changes the result
    img[..., 2] = 255 - img[..., 2] // 3
    return img


def test_reference_facade_classify_polarity():
    size = 64
    net, binp, g = nu.model("resnet18", 1, size, seed=3)
    p1 = nu.batch1_graph("resnet18", size)
    f = refshim.RefFacade(p1, binp)
    r = refshim.RefNet(p1, binp)
    img = _image(31, 50, 70)
    mean, std = np.array([0.4, 0.5, 0.6], np.float32), np.array([0.2, 0.3, 0.25], np.float32)
    decided = 0
    for pre in ("f32c3", "googlenet", "transformed", "caffe", "padding_zero"):
        best = {}
        for sh in (False, True):
            x = refshim.letterbox_u8(img, size, size, False, sh) if pre == "padding_zero" else refshim.preproc_u8(img, size, size, pre, mean, std, sh)
            best[sh] = int(np.argmax(r.run(x)[-1]))
        for swap in (0, 1):
            got = f.classify_list(img, pre, swap, mean, std)
            assert got == best[nu.facade_shuffle(pre, swap)], (pre, swap, got, best)
            if best[False] != best[True]:
                assert got != best[not nu.facade_shuffle(pre, swap)]
                decided += 1
    assert decided >= 6             # the image separates the two channel orders for at least three of the five forms
    f.close()
    r.close()


def small_detector(tmp_path, size=12, seed=7):
    """a 3-channel detection head with moderate logits (a handful of boxes, far below the facade's 1024-box container):
    the golden micro graph yolo_head with 3 input channels and a 3x3 kernel, seeded weights"""
    text = bytes(GOLD["micro/yolo_head/graph"]).decode()
    text = text.replace("width: 6", f"width: {size}").replace("height: 6", f"height: {size}").replace("channels: 8", "channels: 3")
    text = text.replace("kSize: 1", "kSize: 3\n  padding: 1")
    net, binp = str(tmp_path / "small_det.msnhnet"), str(tmp_path / "small_det.msnhbin")
    with open(net, "w") as fh:
        fh.write(text)
    rng = np.random.default_rng(seed)
    w = rng.normal(0, 0.6, 21 * 3 * 9).astype(np.float32)
    b = rng.normal(0, 0.5, 21).astype(np.float32)
    np.concatenate([w, b]).tofile(binp)             # a convolution without batch norm reads its kernel, then its bias
    return net, binp, size


def test_reference_facade_yolo_polarity(tmp_path):
    net, binp, size = small_detector(tmp_path)
    f = refshim.RefFacade(net, binp)
    r = refshim.RefNet(net, binp)
    img = _image(33, 3 * size, 4 * size)
    boxes = {}
    for sh in (False, True):
        r.run(refshim.letterbox_u8(img, size, size, False, sh))
        boxes[sh] = r.boxes()
    assert 0 < len(boxes[False]) < 1024 and not np.array_equal(boxes[False], boxes[True])
    for swap in (0, 1):
        got = f.yolo_list(img, swap)
        assert np.array_equal(got, boxes[nu.facade_shuffle("padding_zero", swap)]), swap
    f.close()
    r.close()
