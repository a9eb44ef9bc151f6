"""ctypes binding of the host library's C ABI (include/msnhnet_c.h): NetBuilder build / load / run.

There is no CPU fallback: loading fails loudly if the libraries are not built, and every run entry point needs
a GPU (the CPU entry points of the reference API exist and raise "Gpu mode , can not run with cpu").
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libMsnhnet.so")

SYMBOLS = [
    "initMsnhnet", "buildMsnhnet", "runClassifyNoPred", "runYoloNoPred", "runClassifyList", "runYoloList", "dispose", "withGPU", "withCUDNN", "getCpuForwardTime",
    "getGpuForwardTime", "getInputDim", "msnhnet_last_error", "msnhnet_create", "msnhnet_destroy", "msnhnet_set_use_fp16", "msnhnet_set_use_winograd", "msnhnet_set_tune_cache", "msnhnet_set_weight_cache", "msnhnet_load_detail", "msnhnet_set_device_nms", "msnhnet_set_input_image_u8", "msnhnet_set_input_image", "msnhnet_boxes_to_image",
    "msnhnet_set_keep_class_scores", "msnhnet_set_save_layer_output", "msnhnet_build", "msnhnet_load", "msnhnet_load_from_memory",
    "msnhnet_input_dims", "msnhnet_num_layers", "msnhnet_layer_info", "msnhnet_layer_detail", "msnhnet_plan_detail", "msnhnet_conv_flops", "msnhnet_weight_layout", "msnhnet_fp16_headroom", "msnhnet_last_nms_on_device", "msnhnet_set_copy_on_forward_stream",
    "msnhnet_run_classify", "msnhnet_run_classify_gpu", "msnhnet_run_yolo_gpu", "msnhnet_layer_output", "msnhnet_yolo_head_logits", "msnhnet_yolo_candidates", "msnhnet_device_input",
    "msnhnet_enqueue", "msnhnet_sync", "msnhnet_fetch_classify", "msnhnet_fetch_yolo", "msnhnet_gpu_inference_time", "msnhnet_time_detail",
    "msnhnet_profile_ops", "msnhnet_profile_ops_bytes", "msnhnet_profile_each_op", "msnhnet_profile_each_op_values", "msnhnet_yolo_max_boxes", "msnhnet_nms", "msnhnet_boxes_from_candidates",
    "msnhnet_group_create", "msnhnet_group_destroy", "msnhnet_group_info", "msnhnet_group_instance", "msnhnet_group_prime", "msnhnet_group_submit",
    "msnhnet_group_flush", "msnhnet_group_fetch_classify", "msnhnet_group_fetch_yolo",
]

LAYER_TYPE = {0: "conv", 1: "deconv", 2: "connect", 3: "maxpool", 4: "localavgpool", 5: "globalavgpool", 6: "softmax", 8: "route", 9: "varop",
              12: "act", 13: "batchnorm", 15: "yolo", 16: "yoloout", 18: "upsample", 20: "empty", 24: "slice", 27: "resblock", 28: "res2block",
              29: "concatblock", 30: "addblock", 31: "padding"}


class MsnhnetError(RuntimeError):
    pass


class BBox(ctypes.Structure):
    _fields_ = [("x", ctypes.c_float), ("y", ctypes.c_float), ("w", ctypes.c_float), ("h", ctypes.c_float), ("conf", ctypes.c_float),
                ("bestClsConf", ctypes.c_float), ("bestClsIdx", ctypes.c_uint32), ("angle", ctypes.c_float)]


class BBoxContainer(ctypes.Structure):
    _fields_ = [("boxes", BBox * 1024)]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MsnhnetError(f"{LIB_PATH} is missing: build it first (python -m msnhnet_amd.build)")
    L = ctypes.CDLL(LIB_PATH)
    vp, ci, ll, cp = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong, ctypes.c_char_p
    fp = ctypes.POINTER(ctypes.c_float)
    ip = ctypes.POINTER(ci)
    llp = ctypes.POINTER(ll)
    cpp = ctypes.POINTER(cp)
    L.buildMsnhnet.argtypes = [cpp, cp, cp, ci, ci]
    L.runClassifyNoPred.argtypes = [cpp, fp, ci, ip, ci]
    L.runYoloNoPred.argtypes = [cpp, fp, ci, ctypes.POINTER(BBoxContainer), ip, ci]
    u8p = ctypes.POINTER(ctypes.c_ubyte)
    L.runClassifyList.argtypes = [cpp, u8p, ci, ci, ci, ip, ci, ci, ci, fp, fp]
    L.runYoloList.argtypes = [cpp, u8p, ci, ci, ci, ctypes.POINTER(BBoxContainer), ip, ci, ci]
    L.withGPU.argtypes = [ip]
    L.withCUDNN.argtypes = [ip]
    L.getCpuForwardTime.argtypes = [fp]
    L.getGpuForwardTime.argtypes = [fp]
    L.getInputDim.argtypes = [ip, ip, ip]
    L.msnhnet_last_error.restype = cp
    L.msnhnet_create.argtypes = [ctypes.POINTER(vp)]
    L.msnhnet_destroy.argtypes = [vp]
    L.msnhnet_set_use_fp16.argtypes = [ci]
    L.msnhnet_set_use_winograd.argtypes = [ci]
    L.msnhnet_set_tune_cache.argtypes = [ci]
    L.msnhnet_set_weight_cache.argtypes = [ci]
    L.msnhnet_set_device_nms.argtypes = [ci]
    L.msnhnet_set_input_image_u8.argtypes = [vp, ci, ctypes.POINTER(ctypes.c_ubyte), ci, ci, ci, ci]
    L.msnhnet_set_input_image.argtypes = [vp, ci, ctypes.POINTER(ctypes.c_ubyte), ci, ci, ci, fp, fp, ci]
    L.msnhnet_boxes_to_image.argtypes = [fp, ll, ci, ci, ci, ci, ci]
    L.msnhnet_set_keep_class_scores.argtypes = [ci]
    L.msnhnet_set_save_layer_output.argtypes = [vp, ci]
    L.msnhnet_build.argtypes = [vp, cp]
    L.msnhnet_load.argtypes = [vp, cp]
    L.msnhnet_load_from_memory.argtypes = [vp, fp, ctypes.c_size_t]
    L.msnhnet_input_dims.argtypes = [vp, ip, ip, ip, ip]
    L.msnhnet_num_layers.argtypes = [vp]
    L.msnhnet_layer_info.argtypes = [vp, ci, llp, cp, ci]
    for n in ("msnhnet_layer_detail", "msnhnet_plan_detail", "msnhnet_time_detail", "msnhnet_load_detail"):
        getattr(L, n).argtypes = [vp, cp, ll]
        getattr(L, n).restype = ll
    L.msnhnet_conv_flops.argtypes = [vp]
    L.msnhnet_weight_layout.argtypes = [vp, llp, ll]
    L.msnhnet_weight_layout.restype = ll
    L.msnhnet_fp16_headroom.argtypes = [vp, fp, ll, fp]
    L.msnhnet_yolo_head_logits.argtypes = [vp, ci, fp, ll]
    L.msnhnet_yolo_head_logits.restype = ll
    L.msnhnet_yolo_candidates.argtypes = [vp, ci, fp, ll]
    L.msnhnet_yolo_candidates.restype = ll
    L.msnhnet_last_nms_on_device.argtypes = [vp, ip]
    L.msnhnet_conv_flops.restype = ctypes.c_double
    L.msnhnet_run_classify.argtypes = [vp, fp, ll, fp, ll, llp]
    L.msnhnet_run_classify_gpu.argtypes = [vp, fp, ll, fp, ll, llp]
    L.msnhnet_run_yolo_gpu.argtypes = [vp, fp, ll, ip, fp, ll, llp]
    L.msnhnet_layer_output.argtypes = [vp, ci, fp, ll]
    L.msnhnet_layer_output.restype = ll
    L.msnhnet_device_input.argtypes = [vp, ctypes.POINTER(fp)]
    L.msnhnet_enqueue.argtypes = [vp, vp]
    L.msnhnet_sync.argtypes = [vp]
    L.msnhnet_fetch_classify.argtypes = [vp, fp, ll, llp]
    L.msnhnet_fetch_yolo.argtypes = [vp, ip, fp, ll, llp]
    L.msnhnet_set_copy_on_forward_stream.argtypes = [vp, ci]
    L.msnhnet_group_create.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ci, ci, ctypes.POINTER(vp)]
    L.msnhnet_group_destroy.argtypes = [vp]
    L.msnhnet_group_info.argtypes = [vp, ip, ip, ip]
    L.msnhnet_group_instance.argtypes = [vp, ci, ctypes.POINTER(vp)]
    L.msnhnet_group_prime.argtypes = [vp, vp]
    L.msnhnet_group_submit.argtypes = [vp, vp]
    L.msnhnet_group_flush.argtypes = [vp]
    L.msnhnet_group_fetch_classify.argtypes = [vp, fp, ll, llp]
    L.msnhnet_group_fetch_yolo.argtypes = [vp, ip, fp, ll, llp]
    L.msnhnet_profile_ops.argtypes = [vp, ci, ci, fp, ip, ctypes.POINTER(ctypes.c_double)]
    L.msnhnet_profile_ops_bytes.argtypes = [vp, ci, ci, fp, ip, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    L.msnhnet_profile_each_op.argtypes = [vp, ci, cp, ll]
    L.msnhnet_profile_each_op.restype = ll
    L.msnhnet_profile_each_op_values.argtypes = [vp, ci, ctypes.POINTER(ctypes.c_double), ll]
    L.msnhnet_profile_each_op_values.restype = ll
    L.msnhnet_nms.argtypes = [fp, ll, ctypes.c_float, ci, fp, ll, llp]
    L.msnhnet_boxes_from_candidates.argtypes = [fp, ll, ctypes.c_float, ci, fp, ll, llp]
    L.msnhnet_yolo_max_boxes.argtypes = [vp]
    L.msnhnet_yolo_max_boxes.restype = ll
    L.msnhnet_gpu_inference_time.argtypes = [vp]
    L.msnhnet_gpu_inference_time.restype = ctypes.c_float
    _lib = L
    return L


def _check(rc):
    if rc != 0:
        raise MsnhnetError(lib().msnhnet_last_error().decode(errors="replace"))


def _fp(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def set_use_fp16(on):
    _check(lib().msnhnet_set_use_fp16(1 if on else 0))


def boxes_to_image(boxes, net_w, net_h, org_w, org_h, padded=True):
    """rows of 7 floats (x y w h conf clsConf cls) from network-input pixels to original-image pixels; returns a copy"""
    b = np.ascontiguousarray(boxes, np.float32).reshape(-1, 7).copy()
    _check(lib().msnhnet_boxes_to_image(_fp(b), len(b), net_w, net_h, org_w, org_h, int(padded)))
    return b


def set_device_nms(mode):
    """0 host, 1 by the previous result's candidate count (default), 2 device"""
    _check(lib().msnhnet_set_device_nms(int(mode)))


def set_tune_cache(on):
    _check(lib().msnhnet_set_tune_cache(1 if on else 0))


def set_weight_cache(on):
    _check(lib().msnhnet_set_weight_cache(1 if on else 0))


def set_use_winograd(on):
    _check(lib().msnhnet_set_use_winograd(1 if on else 0))


def nms(rows, thresh, fast=True):
    """YoloOutLayer::nms on rows of (x y w h conf bestClsConf bestClsIdx); host only."""
    rows = np.ascontiguousarray(rows, np.float32).reshape(-1, 7)
    out = np.zeros_like(rows)
    n = ctypes.c_longlong()
    _check(lib().msnhnet_nms(_fp(rows), len(rows), thresh, 1 if fast else 0, _fp(out), len(rows), ctypes.byref(n)))
    return out[:n.value]


def boxes_from_candidates(rows8, thresh, fast=True):
    """the host stage of YoloOutLayer on candidate rows [n, 8] (x y w h objectness, class score, class, cell; any order): scan order,
    sort by objectness * class score, per-class NMS; returns rows of 7 floats.  Host only."""
    rows8 = np.ascontiguousarray(rows8, np.float32).reshape(-1, 8)
    out = np.zeros((len(rows8), 7), np.float32)
    n = ctypes.c_longlong()
    _check(lib().msnhnet_boxes_from_candidates(_fp(rows8), len(rows8), thresh, 1 if fast else 0, _fp(out), len(rows8), ctypes.byref(n)))
    return out[:n.value]


class Net:
    """One NetBuilder.  `fp16` is the process-wide NetBuilder::setUseFp16 switch, applied before the build."""

    def __init__(self, msnhnet_path=None, msnhbin_path=None, fp16=False, dump_layers=False):
        self.L = lib()
        self.h = ctypes.c_void_p()
        _check(self.L.msnhnet_create(ctypes.byref(self.h)))
        set_use_fp16(fp16)
        if dump_layers:
            _check(self.L.msnhnet_set_save_layer_output(self.h, 1))
        if msnhnet_path:
            self.build(msnhnet_path)
        if msnhbin_path:
            self.load(msnhbin_path)

    @classmethod
    def borrowed(cls, handle):
        """A view of a NetBuilder that somebody else owns (an instance of a NetGroup): every query works, close() leaves it alone."""
        self = cls.__new__(cls)
        self.L = lib()
        self.h = handle
        self._borrowed = True
        return self

    def close(self):
        if self.h:
            if not getattr(self, "_borrowed", False):
                self.L.msnhnet_destroy(self.h)
            self.h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def build(self, path):
        _check(self.L.msnhnet_build(self.h, path.encode()))

    def load(self, path):
        _check(self.L.msnhnet_load(self.h, path.encode()))

    def load_array(self, w):
        w = np.ascontiguousarray(w, np.float32)
        _check(self.L.msnhnet_load_from_memory(self.h, _fp(w), w.size))

    def set_copy_on_forward_stream(self, on):
        """detectors: copy-back on the forward's own stream (what the instances of a NetGroup use) or on a stream of its own (default)"""
        _check(self.L.msnhnet_set_copy_on_forward_stream(self.h, 1 if on else 0))

    def last_nms_on_device(self):
        v = ctypes.c_int()
        _check(self.L.msnhnet_last_nms_on_device(self.h, ctypes.byref(v)))
        return bool(v.value)

    def fp16_headroom(self, x):
        """factor by which input x could grow before a float16 activation overflows (0: it did); see msnhnet_fp16_headroom"""
        x = np.ascontiguousarray(x, np.float32)
        h = ctypes.c_float()
        _check(self.L.msnhnet_fp16_headroom(self.h, _fp(x), x.size, ctypes.byref(h)))
        return h.value

    def weight_layout(self):
        """-> list of (what, count, fan_in) in .msnhbin order: 0 kernel, 1 bn scale, 2 bn shift, 3 running mean, 4 running variance, 5 bias,
        6 connected weights (msnhnet_weight_layout); needs the graph built, not the weights"""
        n = self.L.msnhnet_weight_layout(self.h, None, 0)
        if n < 0:
            _check(1)
        buf = (ctypes.c_longlong * (3 * max(n, 1)))()
        self.L.msnhnet_weight_layout(self.h, buf, n)
        return [(int(buf[3 * i]), int(buf[3 * i + 1]), int(buf[3 * i + 2])) for i in range(n)]

    def dims(self):
        v = [ctypes.c_int() for _ in range(4)]
        _check(self.L.msnhnet_input_dims(self.h, *[ctypes.byref(x) for x in v]))
        return tuple(x.value for x in v)          # batch, channels, height, width

    def num_layers(self):
        return self.L.msnhnet_num_layers(self.h)

    def layer_info(self, i):
        info = (ctypes.c_longlong * 10)()
        name = ctypes.create_string_buffer(64)
        _check(self.L.msnhnet_layer_info(self.h, i, info, name, 64))
        keys = ["type", "outH", "outW", "outC", "outputNum", "inputNum", "numWeights", "memReUse", "batch", "act"]
        d = dict(zip(keys, [int(v) for v in info]))
        d["type"] = LAYER_TYPE.get(d["type"], str(d["type"]))
        d["name"] = name.value.decode()
        return d

    def layer_infos(self):
        return [self.layer_info(i) for i in range(self.num_layers())]

    def _text(self, fn):
        n = fn(self.h, None, 0)
        if n < 0:
            _check(1)
        buf = ctypes.create_string_buffer(n + 1)
        fn(self.h, buf, n + 1)
        return buf.value.decode(errors="replace")

    def layer_detail(self):
        return self._text(self.L.msnhnet_layer_detail)

    def plan_detail(self):
        return self._text(self.L.msnhnet_plan_detail)

    def load_detail(self):
        return self._text(self.L.msnhnet_load_detail)

    def time_detail(self):
        return self._text(self.L.msnhnet_time_detail)

    def conv_flops(self):
        return float(self.L.msnhnet_conv_flops(self.h))

    def run_classify_cpu(self, img):
        x = np.ascontiguousarray(img, np.float32).ravel()
        n = ctypes.c_longlong()
        _check(self.L.msnhnet_run_classify(self.h, _fp(x), x.size, None, 0, ctypes.byref(n)))

    def run_classify(self, img):
        x = np.ascontiguousarray(img, np.float32).ravel()
        b = self.dims()[0]
        last = self.layer_info(self.num_layers() - 1)
        out = np.empty(b * last["outputNum"], np.float32)
        n = ctypes.c_longlong()
        _check(self.L.msnhnet_run_classify_gpu(self.h, _fp(x), x.size, _fp(out), out.size, ctypes.byref(n)))
        return out[:n.value].reshape(b, -1)

    def _boxes(self, fn, *head):
        b = self.dims()[0]
        counts = (ctypes.c_int * b)()
        total = ctypes.c_longlong()
        if getattr(self, "_box_buf", None) is None:
            self._box_buf = np.zeros((max(int(self.L.msnhnet_yolo_max_boxes(self.h)), 1), 7), np.float32)
        boxes = self._box_buf
        _check(fn(self.h, *head, counts, _fp(boxes), boxes.shape[0], ctypes.byref(total)))
        out, at = [], 0
        for i in range(b):
            out.append(boxes[at:at + counts[i]].copy())
            at += counts[i]
        return out

    def run_yolo(self, img):
        x = np.ascontiguousarray(img, np.float32).ravel()
        return self._boxes(self.L.msnhnet_run_yolo_gpu, _fp(x), x.size)

    def layer_output(self, i):
        n = self.L.msnhnet_layer_output(self.h, i, None, 0)
        if n < 0:
            _check(1)
        a = np.empty(n, np.float32)
        if n:
            self.L.msnhnet_layer_output(self.h, i, _fp(a), n)
        return a

    def yolo_head_logits(self, head):
        """input of detection head `head` after the last fetched result, batch-major NCHW float32 (flat)"""
        n = self.L.msnhnet_yolo_head_logits(self.h, head, None, 0)
        if n < 0:
            _check(1)
        a = np.empty(n, np.float32)
        self.L.msnhnet_yolo_head_logits(self.h, head, _fp(a), n)
        return a

    def yolo_candidates(self, image):
        """candidate rows [n, 8] of one image of the last fetched result (x y w h objectness, class score, class, cell number)"""
        n = self.L.msnhnet_yolo_candidates(self.h, image, None, 0)
        if n < 0:
            _check(1)
        a = np.empty((n, 8), np.float32)
        if n:
            self.L.msnhnet_yolo_candidates(self.h, image, _fp(a), n)
        return a

    def device_input_ptr(self):
        p = ctypes.POINTER(ctypes.c_float)()
        _check(self.L.msnhnet_device_input(self.h, ctypes.byref(p)))
        return ctypes.cast(p, ctypes.c_void_p).value

    def enqueue(self, device_ptr=None):
        _check(self.L.msnhnet_enqueue(self.h, ctypes.c_void_p(device_ptr) if device_ptr else None))

    def sync(self):
        _check(self.L.msnhnet_sync(self.h))

    def fetch_classify(self):
        b = self.dims()[0]
        last = self.layer_info(self.num_layers() - 1)
        out = np.empty(b * last["outputNum"], np.float32)
        n = ctypes.c_longlong()
        _check(self.L.msnhnet_fetch_classify(self.h, _fp(out), out.size, ctypes.byref(n)))
        return out[:n.value].reshape(b, -1)

    def fetch_yolo(self):
        return self._boxes(self.L.msnhnet_fetch_yolo)

    def set_input_image_u8(self, index, img, half_init=False, shuffle_rgb=False):
        """img: HWC uint8, 3 channels; letterboxed on the device into slot `index` of the input batch."""
        a = np.ascontiguousarray(img, np.uint8)
        h, w, c = a.shape
        if c != 3:
            raise ValueError("3-channel image expected")
        _check(self.L.msnhnet_set_input_image_u8(self.h, index, a.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), w, h,
                                                 int(half_init), int(shuffle_rgb)))

    def set_input_image(self, index, img, preproc, mean=None, std=None, shuffle_rgb=False):
        """img: HWC uint8, 3 channels; pre-processed on the device (preproc: a msnh_preproc value of include/msnh_hip.h) into slot `index`."""
        a = np.ascontiguousarray(img, np.uint8)
        h, w, c = a.shape
        if c != 3:
            raise ValueError("3-channel image expected")
        m = np.ascontiguousarray(mean, np.float32) if mean is not None else None
        sd = np.ascontiguousarray(std, np.float32) if std is not None else None
        _check(self.L.msnhnet_set_input_image(self.h, index, a.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), w, h, int(preproc),
                                              _fp(m) if m is not None else None, _fp(sd) if sd is not None else None, int(shuffle_rgb)))

    def profile_ops(self, kind, reps):
        """-> (total ms, launches, algorithmic FLOPs) of `reps` eager passes over the launches of one kind (-1 = all)."""
        ms, n, f = ctypes.c_float(), ctypes.c_int(), ctypes.c_double()
        _check(self.L.msnhnet_profile_ops(self.h, kind, reps, ctypes.byref(ms), ctypes.byref(n), ctypes.byref(f)))
        return ms.value, n.value, f.value

    def profile_ops_bytes(self, kind, reps):
        """-> (total ms, launches, algorithmic FLOPs, least bytes moved); kind as profile_ops, or 1000 + a convolution algorithm"""
        ms, n, f, b = ctypes.c_float(), ctypes.c_int(), ctypes.c_double(), ctypes.c_double()
        _check(self.L.msnhnet_profile_ops_bytes(self.h, kind, reps, ctypes.byref(ms), ctypes.byref(n), ctypes.byref(f), ctypes.byref(b)))
        return ms.value, n.value, f.value, b.value

    def profile_each_op_values(self, reps=20):
        """[launches, 8]: kind, algorithm, layer, tile, FLOPs, least bytes, microseconds, ksize * 100 + stride of every live launch"""
        a = np.zeros((4096, 8), np.float64)                 # (one call: the measurement itself is what takes time)
        n = self.L.msnhnet_profile_each_op_values(self.h, reps, a.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), len(a))
        if n < 0:
            _check(1)
        return a[:n].copy()

    def profile_each_op(self, reps=20):
        n = self.L.msnhnet_profile_each_op(self.h, reps, None, 0)
        if n < 0:
            _check(1)
        buf = ctypes.create_string_buffer(n + 1)
        self.L.msnhnet_profile_each_op(self.h, reps, buf, n + 1)
        return buf.value.decode()

    def gpu_inference_time_ms(self):
        return float(self.L.msnhnet_gpu_inference_time(self.h))


class NetGroup:
    """Several instances of one network on one GPU, fed round-robin: a throughput configuration for serving (msnhnet_group_* of
    include/msnhnet_c.h; the host threads and queues live in the library).

    Each instance is a NetBuilder of its own (own stream, activation arena and captured graph; one packed copy of the weights serves all), driven by one host
    thread that enqueues a batch and fetches the result of an earlier one, so that `instances * depth` batches are in flight.  The
    device then runs the forwards of different instances side by side: the launch gaps, prologues and write bursts of one
    forward's kernels are filled by another's, which a single stream cannot do.  Results come back in submission order.

    prime(ptr) runs the device-resident float32 NCHW batch at `ptr` once on every instance (call it before the first submit).
    submit(ptr) hands the next batch to the next instance: a device pointer (copied into the instance's input buffer on its
    stream; keep it valid until the result is fetched) or None to run on what that buffer holds.  flush() makes the instances
    deliver what they still hold in flight now (a fetch of a held-back result asks for it by itself).  fetch() returns the oldest outstanding result (boxes per image for a detector,
    logits for a classifier); an error raised inside an instance's thread surfaces in the fetch of its batch."""

    def __init__(self, msnhnet_path, msnhbin_path, instances=2, depth=2, fp16=False):
        self.L = lib()
        set_use_fp16(fp16)
        self.g = ctypes.c_void_p()
        _check(self.L.msnhnet_group_create(msnhnet_path.encode(), msnhbin_path.encode(), instances, depth, ctypes.byref(self.g)))
        n, d, det = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        _check(self.L.msnhnet_group_info(self.g, ctypes.byref(n), ctypes.byref(d), ctypes.byref(det)))
        self.depth, self.detect = d.value, bool(det.value)
        self.nets = []
        for i in range(n.value):
            h = ctypes.c_void_p()
            _check(self.L.msnhnet_group_instance(self.g, i, ctypes.byref(h)))
            self.nets.append(Net.borrowed(h))
        self._submitted = 0
        self._fetched = 0
        self._batch = self.nets[0].dims()[0]
        if self.detect:
            self._boxes = np.zeros((max(int(self.L.msnhnet_yolo_max_boxes(self.nets[0].h)), 1), 7), np.float32)
        else:
            self._outputs = self.nets[0].layer_info(self.nets[0].num_layers() - 1)["outputNum"]

    def prime(self, device_ptr):
        _check(self.L.msnhnet_group_prime(self.g, ctypes.c_void_p(device_ptr) if device_ptr else None))

    def submit(self, device_ptr=None):
        _check(self.L.msnhnet_group_submit(self.g, ctypes.c_void_p(device_ptr) if device_ptr else None))
        self._submitted += 1

    def flush(self):
        _check(self.L.msnhnet_group_flush(self.g))

    def outstanding(self):
        return self._submitted - self._fetched

    def fetch(self):
        if self._fetched >= self._submitted:
            raise RuntimeError("nothing outstanding")
        self._fetched += 1               # (a batch whose fetch reports an error is consumed as well)
        if self.detect:
            counts = (ctypes.c_int * self._batch)()
            total = ctypes.c_longlong()
            _check(self.L.msnhnet_group_fetch_yolo(self.g, counts, _fp(self._boxes), self._boxes.shape[0], ctypes.byref(total)))
            out, at = [], 0
            for i in range(self._batch):
                out.append(self._boxes[at:at + counts[i]].copy())
                at += counts[i]
            return out
        out = np.empty(self._batch * self._outputs, np.float32)
        n = ctypes.c_longlong()
        _check(self.L.msnhnet_group_fetch_classify(self.g, _fp(out), out.size, ctypes.byref(n)))
        return out[:n.value].reshape(self._batch, -1)

    def close(self):
        for n in self.nets:
            n.close()
        if self.g:
            self.L.msnhnet_group_destroy(self.g)
            self.g = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
