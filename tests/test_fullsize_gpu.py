"""The five benchmark configurations at their full sizes (batch, resolution, dtype as benchmarked).

Where the reference's own CPU forward finishes in seconds (the classifiers; YOLOv3 on the vectorised build, which has
no max-pool and so is not touched by the reference's AVX max-pool defect) image 0 of the batch is compared with it
directly.  YOLOv4-608 (70 s per image on the scalar build, SPP max-pools rule out the vectorised one) and the other
images are covered by properties that do not depend on the size: a batch of identical images gives identical results
per image, two runs are bit-identical, the captured graph equals the layer-by-layer run, and float16 stays within
its tolerance of the float32 plan of the same library (which is pinned against the reference layer by layer at small
sizes in test_net_gpu.py).
"""
import numpy as np
import pytest

import netutil as nu
import refshim
from msnhnet_amd import netapi, zoo

pytestmark = pytest.mark.gpu

FULL = [("resnet18", 224, 1, False), ("resnet50", 224, 32, True), ("mobilenetv2", 224, 64, True),
        ("yolov3", 608, 8, True), ("yolov4", 608, 16, True)]


def _head_logits(m, batch):
    outs = []
    for i in range(m.num_layers()):
        if m.layer_info(i)["type"] == "yolo":
            outs.append(m.layer_output(i - 1).reshape(batch, -1))
    return outs


@pytest.mark.parametrize("arch,size,batch,fp16", FULL)
def test_full_size_configuration(arch, size, batch, fp16):
    net, binp, g = nu.model(arch, batch, size, seed=5)
    img = zoo.seeded_input(1, 3, size, size, seed=6)
    x = np.repeat(img, batch, axis=0)                      # the same image in every slot of the batch
    detect = arch.startswith("yolo")
    print("full size", arch, size, batch, "fp16" if fp16 else "fp32", flush=True)
    fast = netapi.Net(net, binp, fp16=fp16)
    if detect:
        b1, b2 = fast.run_yolo(x), fast.run_yolo(x)
        for i in range(batch):
            assert np.array_equal(b1[i], b2[i]), "two runs differ"
            assert np.array_equal(b1[i], b1[0]), f"image {i} of a batch of identical images differs"
    else:
        l1, l2 = fast.run_classify(x), fast.run_classify(x)
        assert np.array_equal(l1, l2), "two runs differ"
        for i in range(batch):
            assert np.array_equal(l1[i], l1[0]), f"image {i} of a batch of identical images differs"
    del fast

    # layer-by-layer run of the same plan: same final results, and the final logits for the comparisons below
    slow = netapi.Net(net, binp, fp16=fp16, dump_layers=True)
    # (each build runs its own tile search, so the two float16 plans may accumulate in a different order: their
    # float16 roundings then differ by an ulp here and there, which the depth of the network amplifies)
    if detect:
        bs = slow.run_yolo(x)
        if fp16:
            assert abs(len(bs[0]) - len(b1[0])) <= max(2, 0.01 * len(b1[0]))
        else:
            assert nu.rel_err(nu.sort_boxes(bs[0])[:, :6], nu.sort_boxes(b1[0])[:, :6]) <= 1e-5
        final = [h[0] for h in _head_logits(slow, batch)]
    else:
        ls = slow.run_classify(x)
        assert nu.rel_err(ls, l1) <= (5e-3 if fp16 else 1e-5)
        final = [ls[0]]
    del slow

    if fp16:
        # the float32 plan of this library on one image
        f32 = netapi.Net(nu.batch1_graph(arch, size), binp, fp16=False, dump_layers=True)
        if detect:
            f32.run_yolo(img)
            want = [h[0] for h in _head_logits(f32, 1)]
        else:
            want = [f32.run_classify(img)[0]]
        del f32
        for got, ref in zip(final, want):
            assert nu.rel_err(got, ref) <= 2e-2

    # the reference itself, where it finishes in seconds
    if refshim.available() and arch != "yolov4":
        path = nu.batch1_graph(arch, size)
        r = refshim.RefNet(path, binp, scalar=not detect)
        outs = r.run(img[0])
        if detect:
            heads = [i - 1 for i in range(r.num_layers()) if r.layer_info(i)["type"] == "yolo"]
            for got, li in zip(final, heads):
                assert nu.rel_err(got, outs[li]) <= (2e-2 if fp16 else 1e-4)
            ref_boxes = r.boxes()
            assert abs(len(b1[0]) - len(ref_boxes)) <= max(2, 0.02 * len(ref_boxes))
        else:
            assert nu.rel_err(final[0], outs[-1]) <= (2e-2 if fp16 else 1e-4)
            if fp16 is False:
                assert int(np.argmax(final[0])) == int(np.argmax(outs[-1]))
        r.close()
