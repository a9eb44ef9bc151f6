"""TEST INFRASTRUCTURE ONLY -- graph-level restatement of the reference CPU forward.

Reads a `.msnhnet` graph and a `.msnhbin` blob with its own small reader and runs the graph one
image at a time (the reference forward is batch-1 only: src/net/MsnhNetBuilder.cpp:680-684; a batch
is N independent runs) on the plain-C ops of `libmsnh_oracle.so`.  Only tests, the smoke check and
the CPU-baseline leg of the benchmark may import this module.

Reference behaviour restated here:
  * document-order repeated keys, `size: n` block expansion, negative route / yoloout indices
    (src/io/MsnhParser.cpp:140-682, 2162-2165, 2618-2621);
  * weight slicing order (src/net/MsnhNetBuilder.cpp:624-663 and each layer's loadAllWeigths);
  * run loop (src/net/MsnhNetBuilder.cpp:665-817) and block semantics
    (src/layers/Msnh{ResBlock,Res2Block,AddBlock,ConcatBlock,Route,UpSample,Yolo,YoloOut}Layer.cpp).
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmsnh_oracle.so")

ACT = {"logistic": 0, "relu": 1, "relu6": 2, "leaky": 8, "swish": 16, "hardswish": 17, "mish": 18, "none": 22}
_fp = ctypes.POINTER(ctypes.c_float)
_lib = None


def lib():
    global _lib
    if _lib is None:
        L = ctypes.CDLL(_SO)
        ci, cf, ll = ctypes.c_int, ctypes.c_float, ctypes.c_longlong
        L.msnh_or_conv.argtypes = [_fp, ci, ci, ci, ci, _fp, ci, ci, ci, ci, ci, ci, _fp, _fp, cf, ci, cf, _fp, _fp]
        L.msnh_or_batchnorm.argtypes = [_fp, ci, ci, ci, _fp, cf, ci, cf, _fp]
        L.msnh_or_maxpool.argtypes = [_fp, ci, ci, ci, ci, ci, ci, ci, ci, ci, _fp]
        L.msnh_or_avgpool.argtypes = [_fp, ci, ci, ci, ci, ci, ci, ci, ci, ci, _fp]
        L.msnh_or_connected.argtypes = [_fp, ci, ci, ci, _fp, _fp, ci, cf, _fp]
        L.msnh_or_upsample.argtypes = [_fp, ci, ci, ci, ci, ci, ci, cf, _fp]
        L.msnh_or_activate_array.argtypes = [_fp, ll, ci, cf]
        L.msnh_or_activate.argtypes = [cf, ci, cf]
        L.msnh_or_activate.restype = cf
        L.msnh_or_yolo_decode.argtypes = [_fp, ci, ci, ci, ci, _fp, cf, ci]
        L.msnh_or_pad.argtypes = [_fp, ci, ci, ci, ci, ci, ci, ci, ci, cf, _fp]
        L.msnh_or_slice.argtypes = [_fp, ci, ci, ci, ci, ci, ci, ci, ci, ci, ci, _fp]
        L.msnh_or_bilinear.argtypes = [_fp, ci, ci, ci, ci, ci, ci, ci, _fp]
        L.msnh_or_softmax.argtypes = [_fp, ci, ci, cf, _fp]
        L.msnh_or_deconv.argtypes = [_fp, ci, ci, ci, ci, _fp, ci, ci, ci, ci, _fp, ci, cf, _fp]
        L.msnh_or_global_avgpool.argtypes = [_fp, ci, ci, ci, _fp]
        L.msnh_or_iou.argtypes = [_fp, _fp]
        L.msnh_or_iou.restype = cf
        L.msnh_or_yolo_out.argtypes = [ctypes.POINTER(_fp), ctypes.POINTER(ci), ci, ci, cf, cf, _fp, ll]
        L.msnh_or_letterbox_u8.argtypes = [ctypes.POINTER(ctypes.c_ubyte), ci, ci, ci, ci, ci, ci, _fp]
        L.msnh_or_preproc_u8.argtypes = [ctypes.POINTER(ctypes.c_ubyte), ci, ci, ci, ci, ci, _fp, _fp, ci, _fp]
        L.msnh_or_bbox_resize2org.argtypes = [_fp, ci, ci, ci, ci]
        L.msnh_or_bbox_resize2org_nopad.argtypes = [_fp, ci, ci, ci, ci]
        L.msnh_or_yolo_out.restype = ll
        L.msnh_or_im2col.argtypes = [_fp, ci, ci, ci, ci, ci, ci, ci, ci, ci, ci, ci, _fp]
        L.msnh_or_gemm_nn.argtypes = [ci, ci, ci, _fp, ci, _fp, ci, _fp, ci]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(_fp) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


# ---------------------------------------------------------------------------------------------
# op wrappers (NCHW float32 numpy in/out)
# ---------------------------------------------------------------------------------------------
def conv(x, w, filters, k, stride=1, pad=0, dil=1, groups=1, bn4=None, bias=None, eps=1e-5, act="none", act_param=0.1):
    x = _f32(x)
    b, c, h, wd = x.shape
    if k == 1:
        dil = 1
    oh = (h + 2 * pad - (dil * (k - 1) + 1)) // stride + 1
    ow = (wd + 2 * pad - (dil * (k - 1) + 1)) // stride + 1
    out = np.empty((b, filters, oh, ow), np.float32)
    ws = np.empty(max(1, (c // groups) * k * k * oh * ow), np.float32)
    w = _f32(w)
    bn4 = _f32(bn4) if bn4 is not None else None
    bias = _f32(bias) if bias is not None else None
    lib().msnh_or_conv(_p(x), b, c, h, wd, _p(w), filters, k, stride, pad, dil, groups, _p(bn4), _p(bias),
                       eps, ACT[act], act_param, _p(ws), _p(out))
    return out


def batchnorm(x, bn4, eps=1e-5, act="none", act_param=0.1):
    x = _f32(x)
    b, c = x.shape[:2]
    hw = int(np.prod(x.shape[2:]))
    out = np.empty_like(x)
    bn4 = _f32(bn4)
    lib().msnh_or_batchnorm(_p(x), b, c, hw, _p(bn4), eps, ACT[act], act_param, _p(out))
    return out


def _pool(fn, x, k, stride, pad):
    x = _f32(x)
    b, c, h, w = x.shape
    oh = (h + 2 * pad - k) // stride + 1
    ow = (w + 2 * pad - k) // stride + 1
    out = np.empty((b, c, oh, ow), np.float32)
    fn(_p(x), b, c, h, w, k, stride, pad, oh, ow, _p(out))
    return out


def maxpool(x, k, stride, pad):
    return _pool(lib().msnh_or_maxpool, x, k, stride, pad)


def avgpool(x, k, stride, pad):
    return _pool(lib().msnh_or_avgpool, x, k, stride, pad)


def connected(x, w, bias, outputs, act="none", act_param=0.1):
    x = _f32(x)
    b = x.shape[0]
    inputs = x.size // b
    out = np.empty((b, outputs, 1, 1), np.float32)
    w = _f32(w)
    bias = _f32(bias) if bias is not None else None
    lib().msnh_or_connected(_p(x), b, inputs, outputs, _p(w), _p(bias), ACT[act], act_param, _p(out))
    return out


def upsample(x, stride, scale=1.0):
    x = _f32(x)
    b, c, h, w = x.shape
    out = np.empty((b, c, h * stride, w * stride), np.float32)
    lib().msnh_or_upsample(_p(x), b, c, h, w, stride, stride, scale, _p(out))
    return out


def activate(x, act, act_param=0.1):
    out = _f32(x).copy()
    lib().msnh_or_activate_array(_p(out), out.size, ACT[act], act_param)
    return out


def yolo_decode(x, class_num, anchors6, ratio, version=3):
    out = _f32(x).copy()
    b, c, h, w = out.shape
    a = _f32(anchors6)
    lib().msnh_or_yolo_decode(_p(out), b, w, h, class_num, _p(a), ratio, version)
    return out


def pad(x, top, down, left, right, value=0.0):
    x = _f32(x)
    b, c, h, w = x.shape
    out = np.empty((b, c, h + top + down, w + left + right), np.float32)
    lib().msnh_or_pad(_p(x), b, c, h, w, top, down, left, right, value, _p(out))
    return out


def slice_(x, start0, step0, start1, step1, start2, step2):
    x = _f32(x)
    b, c, h, w = x.shape
    ext = lambda n, st, sp: (n - st) // sp + (1 if (n - st) % sp else 0)
    out = np.empty((b, ext(c, start0, step0), ext(h, start1, step1), ext(w, start2, step2)), np.float32)
    lib().msnh_or_slice(_p(x), b, c, h, w, start0, step0, start1, step1, start2, step2, _p(out))
    return out


def deconv(x, w, filters, k, stride, pad, bias=None, act="none", act_param=0.1):
    """w: [in_c][filters][k][k] flat"""
    x = _f32(x)
    b, c, h, wd = x.shape
    oh, ow = (h - 1) * stride - 2 * pad + k, (wd - 1) * stride - 2 * pad + k
    out = np.empty((b, filters, oh, ow), np.float32)
    w = _f32(w)
    bias = _f32(bias) if bias is not None else None
    lib().msnh_or_deconv(_p(x), b, c, h, wd, _p(w), filters, k, stride, pad, _p(bias), ACT[act], act_param, _p(out))
    return out


def softmax(x, temperature=1.0):
    x = _f32(x)
    out = np.empty_like(x)
    lib().msnh_or_softmax(_p(x), x.shape[0], x.size // x.shape[0], temperature, _p(out))
    return out


def global_avgpool(x):
    x = _f32(x)
    b, c, h, w = x.shape
    out = np.empty((b, c, 1, 1), np.float32)
    lib().msnh_or_global_avgpool(_p(x), b, c, h * w, _p(out))
    return out


def bilinear(x, out_h, out_w, align_corners=0):
    x = _f32(x)
    b, c, h, w = x.shape
    out = np.empty((b, c, out_h, out_w), np.float32)
    lib().msnh_or_bilinear(_p(x), b, c, h, w, out_h, out_w, align_corners, _p(out))
    return out


def iou(b1, b2):
    a, b = _f32(b1), _f32(b2)
    return float(lib().msnh_or_iou(_p(a), _p(b)))


def letterbox_u8(img, net_w, net_h, half_init=False, shuffle_rgb=False):
    """img: HWC uint8 with 3 channels -> CHW float32 network input (pad to square with 127, bilinear resize)."""
    a = np.ascontiguousarray(img, np.uint8)
    h, w, c = a.shape
    assert c == 3
    out = np.empty((3, net_h, net_w), np.float32)
    lib().msnh_or_letterbox_u8(a.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), w, h, net_w, net_h, int(half_init), int(shuffle_rgb), _p(out))
    return out


PREPROC_KINDS = {"f32c3": 0, "f32c3_half": 1, "googlenet": 2, "transformed": 3, "caffe": 4}


def preproc_u8(img, net_w, net_h, kind="f32c3", mean=(0, 0, 0), std=(1, 1, 1), shuffle_rgb=False):
    """img: HWC uint8 with 3 channels -> CHW float32 network input by plain bilinear resize + one of the reference's normalisations."""
    a = np.ascontiguousarray(img, np.uint8)
    h, w, c = a.shape
    assert c == 3
    out = np.empty((3, net_h, net_w), np.float32)
    m, sd = _f32(mean), _f32(std)
    lib().msnh_or_preproc_u8(a.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), w, h, net_w, net_h, PREPROC_KINDS[kind], _p(m), _p(sd), int(shuffle_rgb), _p(out))
    return out


def bbox_resize2org(xywh, cur_w, cur_h, org_w, org_h, no_pad=False):
    b = _f32(xywh).copy()
    (lib().msnh_or_bbox_resize2org_nopad if no_pad else lib().msnh_or_bbox_resize2org)(_p(b), cur_w, cur_h, org_w, org_h)
    return b


def yolo_out(heads, class_num, conf, nms):
    """heads: list of decoded [3*(5+classes), H, W] arrays of ONE image.  Returns [n,7] boxes."""
    hs = [_f32(h) for h in heads]
    n = len(hs)
    ptrs = (_fp * n)(*[_p(h) for h in hs])
    hw = (ctypes.c_int * n)(*[int(h.shape[-1] * h.shape[-2]) for h in hs])
    cap = sum(3 * v for v in hw)
    out = np.zeros((max(cap, 1), 7), np.float32)
    cnt = lib().msnh_or_yolo_out(ptrs, hw, n, class_num, conf, nms, _p(out), cap)
    return out[:cnt].copy()


# ---------------------------------------------------------------------------------------------
# `.msnhnet` reader: nested (key, value | children) lists in document order
# ---------------------------------------------------------------------------------------------
def parse_msnhnet(text):
    rows = []
    for raw in text.splitlines():
        line = raw.split("#", 1)[0].rstrip()
        if not line.strip():
            continue
        indent = len(line) - len(line.lstrip(" "))
        key, _, val = line.strip().partition(":")
        rows.append((indent, key.strip(), val.strip()))

    def build(i, indent):
        items = []
        while i < len(rows) and rows[i][0] == indent:
            _, key, val = rows[i]
            i += 1
            if val == "" and i < len(rows) and rows[i][0] > indent:
                children, i = build(i, rows[i][0])
                items.append((key, children))
            else:
                items.append((key, val if val != "" else []))
        return items, i

    items, _ = build(0, rows[0][0] if rows else 0)
    return items


def _kv(children):
    return {k: v for k, v in children if not isinstance(v, list)}


def _act(d):
    parts = d.get("activation", "none").split(",")
    name = parts[0].strip()
    if name not in ACT:
        name = "relu"          # unknown names silently become relu (src/layers/MsnhActivations.cpp:4-30)
    return name, (float(parts[1]) if len(parts) > 1 else 0.1)


class OracleNet:
    """Graph + weights; `run(img)` returns per-top-level-layer outputs of one image like the reference dump."""

    def __init__(self, msnhnet_path, msnhbin_path=None):
        with open(msnhnet_path) as f:
            self.items = parse_msnhnet(f.read())
        if not self.items or self.items[0][0] != "config":
            raise ValueError("The first params must be config")
        cfg = _kv(self.items[0][1])
        self.batch = int(cfg.get("batch", 1))
        self.c, self.h, self.w = int(cfg["channels"]), int(cfg["height"]), int(cfg["width"])
        self.top = []
        for key, ch in self.items[1:]:
            reps = 1
            if key in ("resblock", "res2block", "addblock"):
                reps = int(_kv(ch).get("size", 1))
            for _ in range(reps):
                self.top.append((key, ch))
        self.weights = np.fromfile(msnhbin_path, dtype="<f4") if msnhbin_path else None
        self.boxes = None

    # -- weights ---------------------------------------------------------------------------------
    def _take(self, n):
        v = self.weights[self._wp:self._wp + n]
        if v.size != n:
            raise ValueError("Load weights err, need > given")
        self._wp += n
        return v

    # -- simple (non-block) nodes ----------------------------------------------------------------
    def _simple(self, key, ch, x):
        d = _kv(ch) if isinstance(ch, list) else {}
        if key == "conv":
            filters = int(d.get("filters", 1)); k = int(d.get("kSize", 1)); s = int(d.get("stride", 1))
            p = int(d.get("padding", 0)); dil = int(d.get("dilation", 1)); g = int(d.get("groups", 1))
            bn = int(d.get("batchNorm", 0)); ub = int(d.get("useBias", 1)); eps = float(d.get("eps", 1e-5))
            act, ap = _act(d)
            cin = x.shape[1]
            w = self._take(filters * (cin // g) * k * k)
            bn4 = bias = None
            if bn:
                # scales, biases(=beta, only present when useBias), rollMean, rollVariance
                # (src/layers/MsnhConvolutionalLayer.cpp:1275-1288)
                scales = self._take(filters)
                beta = self._take(filters) if ub else np.zeros(filters, np.float32)
                mean = self._take(filters); var = self._take(filters)
                bn4 = np.concatenate([scales, beta, mean, var])
            elif ub:
                bias = self._take(filters)
            return conv(x, w, filters, k, s, p, dil, g, bn4, bias, eps, act, ap)
        if key == "batchnorm":
            c = x.shape[1]
            act, ap = _act(d)
            return batchnorm(x, self._take(4 * c), float(d.get("eps", 1e-5)), act, ap)
        if key == "maxpool":
            return maxpool(x, int(d.get("kSize", 1)), int(d.get("stride", 1)), int(d.get("padding", 0)))
        if key == "localavgpool":
            return avgpool(x, int(d.get("kSize", 1)), int(d.get("stride", 1)), int(d.get("padding", 0)))
        if key == "connect":
            outputs = int(d["output"])
            inputs = x.size // x.shape[0]
            w = self._take(inputs * outputs)
            bias = self._take(outputs) if int(d.get("useBias", 1)) else None
            act, ap = _act(d)
            return connected(x, w, bias, outputs, act, ap)
        if key == "empty":
            return x.copy()
        if key == "upsample":
            if d.get("type", "nearest").strip() == "bilinear":
                # output extent int(extent * scale) (src/layers/MsnhUpSampleLayer.cpp:20-24)
                sx = float(d.get("scaleX", d.get("scale", 1.0))); sy = float(d.get("scaleY", d.get("scale", 1.0)))
                return bilinear(x, int(x.shape[2] * np.float32(sy)), int(x.shape[3] * np.float32(sx)), int(d.get("alignCorners", 0)))
            return upsample(x, int(d.get("stride", d.get("strideX", 1))), float(d.get("scale", d.get("scaleX", 1.0))))
        if key == "deconv":
            filters = int(d.get("filters", 1)); k = int(d.get("kSize", 1)); st = int(d.get("stride", 1)); p = int(d.get("padding", 0))
            act, ap = _act(d)
            w = self._take(x.shape[1] * filters * k * k)
            bias = self._take(filters) if int(d.get("useBias", 1)) else None
            return deconv(x, w, filters, k, st, p, bias, act, ap)
        if key == "softmax":
            if int(d.get("groups", 1)) != 1:
                raise ValueError("softmax groups")
            return softmax(x, float(d.get("temperature", 1.0)))
        if key == "globalavgpool":
            return global_avgpool(x)
        if key == "act":
            act, ap = _act(d)
            return activate(x, act, ap)
        if key == "padding":
            return pad(x, int(d.get("top", 0)), int(d.get("down", 0)), int(d.get("left", 0)), int(d.get("right", 0)),
                       float(d.get("paddingVal", 0)))
        if key == "slice":
            return slice_(x, int(d.get("start0", 0)), int(d.get("step0", 1)), int(d.get("start1", 0)), int(d.get("step1", 1)),
                          int(d.get("start2", 0)), int(d.get("step2", 1)))
        raise ValueError(f"{key} is not supported")

    def _seq(self, nodes, x):
        for key, ch in nodes:
            if key in ("size", "activation"):
                continue
            x = self._simple(key, ch, x)
        return x

    # -- forward of one image ----------------------------------------------------------------------
    def run(self, img):
        x = _f32(img).reshape(1, self.c, self.h, self.w)
        self._wp = 0
        outs = []
        heads = {}
        for li, (key, ch) in enumerate(self.top):
            d = _kv(ch) if isinstance(ch, list) else {}
            if key == "resblock":
                body = [(k, v) for k, v in ch if k not in ("size", "activation")]
                y = self._seq(body, x) + x                      # F(x) += x  (MsnhResBlockLayer.cpp:261)
                # block activation params are not propagated by the parser (src/io/MsnhParser.cpp:413)
                x = activate(y, _act(d)[0], 0.1)
            elif key == "res2block":
                base = self._seq(dict(ch)["base"], x)
                br = self._seq(dict(ch)["branch"], x)
                x = activate(br + base, _act(d)[0], _act(d)[1])  # branch += base (MsnhRes2BlockLayer.cpp:401)
            elif key == "addblock":
                acc = None
                for k, v in ch:
                    if k != "branch":
                        continue
                    y = self._seq(v, x)
                    acc = y if acc is None else y + acc         # b[i] += b[i-1] (MsnhAddBlockLayer.cpp:308-315)
                x = activate(acc, _act(d)[0], _act(d)[1])
            elif key == "concatblock":
                ys = [self._seq(v, x) for k, v in ch if k == "branch"]
                x = np.concatenate(ys, axis=1)
            elif key == "route":
                idx = [int(t) for t in d["layers"].split(",") if t.strip() != ""]
                idx = [i if i >= 0 else li + i for i in idx]
                if int(d.get("addModel", 0)) == 1:
                    # zero-filled output, then += each listed layer in list order (src/layers/MsnhRouteLayer.cpp:77-115)
                    x = np.zeros_like(outs[idx[0]])
                    for i in idx:
                        x = (x + outs[i]).astype(np.float32)
                else:
                    x = np.concatenate([outs[i] for i in idx], axis=1)
                act, ap = _act(d)
                if act != "none":
                    x = activate(x, act, ap)
            elif key == "varop":
                # one listed layer: A = previous layer, B = it; two: A, B = the listed layers
                # (src/layers/MsnhVariableOpLayer.cpp:78-165); constant forms use A and constVal (:166-240)
                idx = [int(t) for t in d.get("layers", "").split(",") if t.strip() != ""]
                idx = [i if i >= 0 else li + i for i in idx]
                kind = d.get("type", "add").strip()
                cv = np.float32(float(d.get("constVal", 0)))
                if kind.endswith("Const") or kind.endswith("ConstInv"):
                    a = x if not idx else outs[idx[0]]
                    x = {"addConst": lambda: a + cv, "subConst": lambda: a - cv, "subConstInv": lambda: cv - a, "mulConst": lambda: a * cv,
                         "divConst": lambda: a / cv, "divConstInv": lambda: cv / a}[kind]().astype(np.float32)
                else:
                    a, b = (x, outs[idx[0]]) if len(idx) == 1 else (outs[idx[0]], outs[idx[1]])
                    x = {"add": lambda: a + b, "sub": lambda: a - b, "subInv": lambda: b - a, "mul": lambda: a * b, "div": lambda: a / b,
                         "divInv": lambda: b / a}[kind]().astype(np.float32)
            elif key == "yolo":
                anchors = [float(t) for t in d["anchors"].split(",")]
                cls = int(d.get("classNum", 1))
                if 3 * (cls + 5) != x.shape[1]:
                    raise ValueError("class num error!")
                version = 5 if d.get("yoloType", "yolov3").strip().startswith("yolov5") else 3
                x = yolo_decode(x, cls, anchors, self.h / x.shape[2], version)
                heads[li] = (x, cls)
            elif key == "yoloout":
                idx = [int(t) for t in d["layers"].split(",") if t.strip() != ""]
                idx = [i if i >= 0 else li + i for i in idx]
                cls = heads[idx[0]][1]
                self.boxes = yolo_out([heads[i][0][0] for i in idx], cls, float(d.get("confThresh", 0)),
                                      float(d.get("nmsThresh", 0)))
                x = np.zeros((1, 0, 1, 1), np.float32)
            else:
                x = self._simple(key, ch, x)
            outs.append(x)
        if self.weights is not None and self._wp != self.weights.size:
            raise ValueError("Load weights err, need != given")
        return outs
