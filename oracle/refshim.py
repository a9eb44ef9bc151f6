"""TEST INFRASTRUCTURE ONLY.  ctypes binding of oracle/_ref/libmsnh_ref.so (the reference's own CPU forward, built by
oracle/Makefile from the reference sources where they lie): the checker of the parity tests and the timed CPU baseline of
bench.py.  Nothing in the product package imports it."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
REF_SO = os.path.join(_HERE, "_ref", "libmsnh_ref.so")

LAYER_TYPE = {0: "conv", 2: "connect", 3: "maxpool", 4: "localavgpool", 8: "route", 13: "batchnorm",
              15: "yolo", 16: "yoloout", 18: "upsample", 20: "empty", 27: "resblock", 28: "res2block",
              29: "concatblock", 30: "addblock"}


def available() -> bool:
    return os.path.exists(REF_SO)


_lib = None


def lib():
    global _lib
    if _lib is None:
        L = ctypes.CDLL(REF_SO)
        vp, cp, ci, ll = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_longlong
        fp = ctypes.POINTER(ctypes.c_float)
        L.ref_create.restype = vp
        L.ref_create.argtypes = [ci]
        L.ref_destroy.argtypes = [vp]
        L.ref_build.argtypes = [vp, cp, cp, ci]
        L.ref_load.argtypes = [vp, cp, cp, ci]
        L.ref_num_layers.argtypes = [vp]
        L.ref_layer_info.argtypes = [vp, ci, ctypes.POINTER(ll), cp, ci]
        L.ref_layer_detail.argtypes = [vp, cp, ll]
        L.ref_layer_detail.restype = ll
        L.ref_run.argtypes = [vp, fp, ll, ci, cp, ci]
        L.ref_last_wall_ms.argtypes = [vp]
        L.ref_last_wall_ms.restype = ctypes.c_double
        L.ref_inference_time.argtypes = [vp]
        L.ref_inference_time.restype = ctypes.c_float
        L.ref_layer_output.argtypes = [vp, ci, fp, ll]
        L.ref_layer_output.restype = ll
        L.ref_boxes.argtypes = [vp, fp, ll]
        L.ref_boxes.restype = ll
        u8p = ctypes.POINTER(ctypes.c_ubyte)
        L.ref_letterbox_u8.argtypes = [u8p, ci, ci, ci, ci, ci, ci, fp, cp, ci]
        L.ref_bbox_resize2org.argtypes = [fp, ci, ci, ci, ci, ci]
        L.ref_preproc_u8.argtypes = [u8p, ci, ci, ci, ci, ci, fp, fp, ci, fp, cp, ci]
        ip = ctypes.POINTER(ci)
        L.ref_facade_build.argtypes = [cp, cp, ci]
        L.ref_facade_classify_list.argtypes = [u8p, ci, ci, ci, ci, fp, fp, ip]
        L.ref_facade_yolo_list.argtypes = [u8p, ci, ci, ci, fp, ci, ip]
        _lib = L
    return _lib


class RefError(RuntimeError):
    pass


class RefNet:
    """One reference NetBuilder.  scalar=True runs the scalar (non-AVX) branches, the parity oracle."""

    def __init__(self, msnhnet, msnhbin=None, scalar=True):
        self.L = lib()
        self.h = self.L.ref_create(1 if scalar else 0)
        err = ctypes.create_string_buffer(1024)
        if self.L.ref_build(self.h, msnhnet.encode(), err, 1024) != 0:
            raise RefError(err.value.decode())
        if msnhbin is not None:
            if self.L.ref_load(self.h, msnhbin.encode(), err, 1024) != 0:
                raise RefError(err.value.decode())

    def close(self):
        if self.h:
            self.L.ref_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def num_layers(self):
        return self.L.ref_num_layers(self.h)

    def layer_info(self, i):
        info = (ctypes.c_longlong * 10)()
        name = ctypes.create_string_buffer(64)
        self.L.ref_layer_info(self.h, i, info, name, 64)
        keys = ["type", "outH", "outW", "outC", "outputNum", "inputNum", "numWeights", "memReUse", "batch", "act"]
        d = dict(zip(keys, [int(v) for v in info]))
        d["type"] = LAYER_TYPE.get(d["type"], str(d["type"]))
        return d

    def layer_infos(self):
        return [self.layer_info(i) for i in range(self.num_layers())]

    def detail(self):
        n = self.L.ref_layer_detail(self.h, None, 0)
        buf = ctypes.create_string_buffer(n + 1)
        self.L.ref_layer_detail(self.h, buf, n + 1)
        return buf.value.decode(errors="replace")

    def run(self, img, capture=True):
        """img: one CHW float32 image.  Returns list of per-top-level-layer outputs (flat arrays)."""
        x = np.ascontiguousarray(img, dtype=np.float32).ravel()
        err = ctypes.create_string_buffer(1024)
        rc = self.L.ref_run(self.h, x.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), x.size, 1 if capture else 0, err, 1024)
        if rc != 0:
            raise RefError(err.value.decode())
        outs = []
        for i in range(self.num_layers()):
            n = self.L.ref_layer_output(self.h, i, None, 0)
            a = np.empty(max(n, 0), np.float32)
            if n > 0:
                self.L.ref_layer_output(self.h, i, a.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), n)
            outs.append(a)
        return outs

    def boxes(self):
        n = self.L.ref_boxes(self.h, None, 0)
        a = np.empty((n, 7), np.float32)
        if n:
            self.L.ref_boxes(self.h, a.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), n)
        return a

    def wall_ms(self):
        return self.L.ref_last_wall_ms(self.h)

    def inference_time_ms(self):
        return float(self.L.ref_inference_time(self.h))


def letterbox_u8(img, net_w, net_h, half_init=False, shuffle_rgb=False):
    """img: HWC uint8, 3 channels.  CVUtil::getPaddingZeroF32C3 -> CHW float32."""
    import numpy as np
    a = np.ascontiguousarray(img, np.uint8)
    h, w, c = a.shape
    assert c == 3
    out = np.empty((3, net_h, net_w), np.float32)
    err = ctypes.create_string_buffer(1024)
    rc = lib().ref_letterbox_u8(a.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), w, h, net_w, net_h, int(half_init), int(shuffle_rgb),
                                out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), err, 1024)
    if rc != 0:
        raise RefError(err.value.decode())
    return out


PREPROC_KINDS = {"f32c3": 0, "f32c3_half": 1, "googlenet": 2, "transformed": 3, "caffe": 4}


def preproc_u8(img, net_w, net_h, kind="f32c3", mean=(0, 0, 0), std=(1, 1, 1), shuffle_rgb=False):
    """img: HWC uint8, 3 channels.  CVUtil::getImgDataF32C3 / getGoogLenetF32C3 / getTransformedF32C3 / getCaffeModeF32C3 -> CHW float32."""
    import numpy as np
    a = np.ascontiguousarray(img, np.uint8)
    h, w, c = a.shape
    assert c == 3
    out = np.empty((3, net_h, net_w), np.float32)
    m = np.ascontiguousarray(mean, np.float32)
    sd = np.ascontiguousarray(std, np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    err = ctypes.create_string_buffer(1024)
    rc = lib().ref_preproc_u8(a.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), w, h, net_w, net_h, PREPROC_KINDS[kind], m.ctypes.data_as(fp),
                              sd.ctypes.data_as(fp), int(shuffle_rgb), out.ctypes.data_as(fp), err, 1024)
    if rc != 0:
        raise RefError(err.value.decode())
    return out


def bbox_resize2org(xywh, cur_w, cur_h, org_w, org_h, no_pad=False):
    import numpy as np
    b = np.array(xywh, np.float32)
    lib().ref_bbox_resize2org(b.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), cur_w, cur_h, org_w, org_h, int(no_pad))
    return b


class RefFacade:
    """The reference's own C facade (src/c_api/MsnhnetLib.cpp, the build without OpenCV) on its CPU path: initMsnhnet + buildMsnhnet,
    then runClassifyList / runYoloList on 8-bit HWC images.  One process-wide network, as in the reference."""
    PRE = {"none": 0, "c1": 1, "f32c3": 2, "googlenet": 3, "padding_zero": 4, "transformed": 5, "caffe": 6}      # PredDataType

    def __init__(self, msnhnet, msnhbin, scalar=True):
        self.L = lib()
        if self.L.ref_facade_build(msnhnet.encode(), msnhbin.encode(), 1 if scalar else 0) != 1:
            raise RefError("the reference's buildMsnhnet failed")

    def classify_list(self, img, pre, swap_rgb, mean=None, std=None):
        a = np.ascontiguousarray(img, np.uint8)
        h, w, c = a.shape
        assert c == 3
        fp = ctypes.POINTER(ctypes.c_float)
        m = None if mean is None else np.ascontiguousarray(mean, np.float32)
        sd = None if std is None else np.ascontiguousarray(std, np.float32)
        best = ctypes.c_int(-1)
        rc = self.L.ref_facade_classify_list(a.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), w, h, self.PRE[pre], int(swap_rgb),
                                             None if m is None else m.ctypes.data_as(fp), None if sd is None else sd.ctypes.data_as(fp),
                                             ctypes.byref(best))
        if rc != 1:
            raise RefError(f"the reference's runClassifyList returned {rc}")
        return best.value

    def yolo_list(self, img, swap_rgb):
        a = np.ascontiguousarray(img, np.uint8)
        h, w, c = a.shape
        assert c == 3
        out = np.empty((1024, 7), np.float32)
        n = ctypes.c_int(0)
        rc = self.L.ref_facade_yolo_list(a.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), w, h, int(swap_rgb),
                                         out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), 1024, ctypes.byref(n))
        if rc != 1:
            raise RefError(f"the reference's runYoloList returned {rc}")
        return out[:n.value].copy()

    def close(self):
        self.L.ref_facade_dispose()
