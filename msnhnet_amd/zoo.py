"""Synthetic workload builder: `.msnhnet` graph text + seeded `.msnhbin` weights.

The five benchmark configurations are standard architectures (ResNet-18/50, MobileNetV2, YOLOv3,
YOLOv4).  Instead of shipping graph files, this module *writes* them from the architecture
definition with a tiny emitter, and at the same time records every weight tensor in the order the
`.msnhbin` loader consumes it, so that seeded weights can be generated without parsing anything.

File format facts this relies on (reference citations):
  * `.msnhnet` is one YAML mapping with repeated keys in layer order; first node `config`
    (src/io/MsnhParser.cpp:146-176, 728-768).
  * `resblock/res2block/addblock` with `size: n` are instantiated n times (src/io/MsnhParser.cpp:408-415,
    465-472, 522-529), each instance with its own weights.
  * `.msnhbin` is a headerless little-endian float32 array (src/io/MsnhParser.cpp:684-726) consumed
    layer by layer: conv = weights[Cout][Cin/g][k][k] then (scales, biases, rollMean, rollVariance) when
    batchNorm else biases when useBias (src/layers/MsnhConvolutionalLayer.cpp:1255-1290); batchnorm
    layer = scales, biases, rollMean, rollVariance (src/layers/MsnhBatchNormLayer.cpp:469-472);
    connected = weights[out][in] then biases (src/layers/MsnhConnectedLayer.cpp:508-535);
    res2block = base layers then branch layers (src/layers/MsnhRes2BlockLayer.cpp:272-298).

Weight distributions follow the benchmark configuration: conv He-normal N(0, 2/fan_in) with
fan_in = Cin/groups*k*k; BN gamma~U[0.5,1.5], beta~N(0,0.1), mean~N(0,0.1), var~U[0.5,1.5];
FC and non-BN conv bias use U(-1/sqrt(fan_in), 1/sqrt(fan_in)) for weights and bias.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import numpy as np


@dataclass
class WeightSlot:
    kind: str            # conv_w | bn_gamma | bn_beta | bn_mean | bn_var | bias | fc_w
    count: int
    fan_in: int = 0


@dataclass
class _Shape:
    c: int
    h: int
    w: int


class GraphWriter:
    """Emits `.msnhnet` text and tracks shapes / weight slots / conv FLOPs."""

    def __init__(self, batch: int, channels: int, height: int, width: int):
        self.lines: List[str] = []
        self.slots: List[WeightSlot] = []
        self.shape = _Shape(channels, height, width)
        self.batch = batch
        self.n_top = 0                      # number of top-level layers emitted so far
        self.top_shapes: List[_Shape] = []  # output shape of each top-level layer
        self.conv_flops = 0                 # 2*MACs per image, conv layers only
        self.fc_flops = 0
        self.n_conv = 0
        self._indent = 0
        self._emit("config:")
        self._emit(f"  batch: {batch}")
        self._emit(f"  width: {width}")
        self._emit(f"  height: {height}")
        self._emit(f"  channels: {channels}")

    # -- low-level ---------------------------------------------------------------------------
    def _emit(self, s: str):
        self.lines.append(" " * self._indent + s)

    def text(self) -> str:
        return "\n".join(self.lines) + "\n"

    def _top_done(self, times: int = 1):
        for _ in range(times):
            self.top_shapes.append(_Shape(self.shape.c, self.shape.h, self.shape.w))
            self.n_top += 1

    # -- weight / shape bookkeeping --------------------------------------------------------------
    def _conv_apply(self, filters, k, stride, pad, groups, bn, bias):
        s = self.shape
        cin_g = s.c // groups
        fan_in = cin_g * k * k
        self.slots.append(WeightSlot("conv_w", filters * cin_g * k * k, fan_in))
        if bn:
            self.slots += [WeightSlot("bn_gamma", filters), WeightSlot("bn_beta", filters),
                           WeightSlot("bn_mean", filters), WeightSlot("bn_var", filters)]
        elif bias:
            self.slots.append(WeightSlot("bias", filters, fan_in))
        oh = (s.h + 2 * pad - k) // stride + 1
        ow = (s.w + 2 * pad - k) // stride + 1
        self.conv_flops += 2 * filters * oh * ow * cin_g * k * k
        self.n_conv += 1
        self.shape = _Shape(filters, oh, ow)

    def _bn_apply(self):
        c = self.shape.c
        self.slots += [WeightSlot("bn_gamma", c), WeightSlot("bn_beta", c),
                       WeightSlot("bn_mean", c), WeightSlot("bn_var", c)]

    # -- node emitters (used both at top level and inside blocks) --------------------------------
    def conv_node(self, filters, k=1, stride=1, pad=0, groups=1, bn=1, bias=None, act="none"):
        """bias=None keeps the file default (useBias 1)."""
        self._emit("conv:")
        self._emit(f"  batchNorm: {bn}")
        self._emit(f"  filters: {filters}")
        self._emit(f"  kSize: {k}")
        self._emit(f"  stride: {stride}")
        if pad:
            self._emit(f"  padding: {pad}")
        if groups != 1:
            self._emit(f"  groups: {groups}")
        if bias is not None:
            self._emit(f"  useBias: {int(bias)}")
        self._emit(f"  activation: {act}")
        self._conv_apply(filters, k, stride, pad, groups, bn, True if bias is None else bias)

    def bn_node(self, act="none", eps=None):
        self._emit("batchnorm:")
        self._emit(f"  activation: {act}")
        if eps is not None:
            self._emit(f"  eps: {eps}")
        self._bn_apply()

    def maxpool_node(self, k, stride, pad):
        self._emit("maxpool:")
        self._emit(f"  kSize: {k}")
        self._emit(f"  stride: {stride}")
        self._emit(f"  padding: {pad}")
        s = self.shape
        self.shape = _Shape(s.c, (s.h + 2 * pad - k) // stride + 1, (s.w + 2 * pad - k) // stride + 1)

    # -- top-level layers ------------------------------------------------------------------------
    def conv(self, *a, **kw):
        self.conv_node(*a, **kw)
        self._top_done()

    def batchnorm(self, act="none", eps=None):
        self.bn_node(act, eps)
        self._top_done()

    def maxpool(self, k, stride, pad):
        self.maxpool_node(k, stride, pad)
        self._top_done()

    def localavgpool(self, k, stride=1, pad=0):
        self._emit("localavgpool:")
        self._emit(f"  kSize: {k}")
        self._emit(f"  stride: {stride}")
        self._emit(f"  padding: {pad}")
        s = self.shape
        self.shape = _Shape(s.c, (s.h + 2 * pad - k) // stride + 1, (s.w + 2 * pad - k) // stride + 1)
        self._top_done()

    def connect(self, output, act="none"):
        self._emit("connect:")
        self._emit(f"  output: {output}")
        self._emit(f"  activation: {act}")
        s = self.shape
        n_in = s.c * s.h * s.w
        self.slots.append(WeightSlot("fc_w", n_in * output, n_in))
        self.slots.append(WeightSlot("bias", output, n_in))
        self.fc_flops += 2 * n_in * output
        self.shape = _Shape(output, 1, 1)
        self._top_done()

    def upsample(self, stride):
        self._emit("upsample:")
        self._emit(f"  stride: {stride}")
        s = self.shape
        self.shape = _Shape(s.c, s.h * stride, s.w * stride)
        self._top_done()

    def route(self, layers: List[int], add_model: bool = False, act: Optional[str] = None):
        """`layers` as written in the file: negative = relative to this route layer."""
        self._emit("route:")
        self._emit("  layers: " + ",".join(str(v) for v in layers))
        if add_model:
            self._emit("  addModel: 1")
        if act:
            self._emit(f"  activation: {act}")
        idx = [v if v >= 0 else self.n_top + v for v in layers]
        shp = [self.top_shapes[i] for i in idx]
        self.shape = _Shape(shp[0].c if add_model else sum(s.c for s in shp), shp[0].h, shp[0].w)
        self._top_done()

    def act(self, act: str):
        self._emit("act:")
        self._emit(f"  activation: {act}")
        self._top_done()

    def padding(self, top, down, left, right, value=0.0):
        self._emit("padding:")
        for k, v in (("top", top), ("down", down), ("left", left), ("right", right)):
            self._emit(f"  {k}: {v}")
        self._emit(f"  paddingVal: {value}")
        s = self.shape
        self.shape = _Shape(s.c, s.h + top + down, s.w + left + right)
        self._top_done()

    def slice(self, start0, step0, start1, step1, start2, step2):
        self._emit("slice:")
        for k, v in (("start0", start0), ("step0", step0), ("start1", start1), ("step1", step1), ("start2", start2), ("step2", step2)):
            self._emit(f"  {k}: {v}")
        s = self.shape
        ext = lambda n, st, sp: (n - st) // sp + (1 if (n - st) % sp else 0)
        self.shape = _Shape(ext(s.c, start0, step0), ext(s.h, start1, step1), ext(s.w, start2, step2))
        self._top_done()

    def varop(self, kind: str, layers: Optional[List[int]] = None, const: float = 0.0):
        self._emit("varop:")
        if layers:
            self._emit("  layers: " + ",".join(str(v) for v in layers))
        self._emit(f"  type: {kind}")
        self._emit(f"  constVal: {const}")
        self._top_done()

    def deconv(self, filters, k, stride, pad=0, bias=True, act="none"):
        self._emit("deconv:")
        self._emit(f"  filters: {filters}")
        self._emit(f"  kSize: {k}")
        self._emit(f"  stride: {stride}")
        if pad:
            self._emit(f"  padding: {pad}")
        if not bias:
            self._emit("  useBias: 0")
        self._emit(f"  activation: {act}")
        s = self.shape
        self.slots.append(WeightSlot("conv_w", s.c * filters * k * k, s.c * k * k))
        if bias:
            self.slots.append(WeightSlot("bias", filters, s.c * k * k))
        self.conv_flops += 2 * s.c * filters * k * k * s.h * s.w
        self.shape = _Shape(filters, (s.h - 1) * stride - 2 * pad + k, (s.w - 1) * stride - 2 * pad + k)
        self._top_done()

    def softmax(self, temperature: float = 1.0):
        self._emit("softmax:")
        self._emit("  groups: 1")
        self._emit(f"  temperature: {temperature}")
        self._top_done()

    def globalavgpool(self):
        self._emit("globalavgpool:")
        self.shape = _Shape(self.shape.c, 1, 1)
        self._top_done()

    def upsample_bilinear(self, scale_x: float, scale_y: float, align_corners: int = 0):
        self._emit("upsample:")
        self._emit("  type: bilinear")
        self._emit(f"  scaleX: {scale_x}")
        self._emit(f"  scaleY: {scale_y}")
        self._emit(f"  alignCorners: {align_corners}")
        s = self.shape
        self.shape = _Shape(s.c, int(np.float32(s.h) * np.float32(scale_y)), int(np.float32(s.w) * np.float32(scale_x)))
        self._top_done()

    def yolo(self, anchors: List[int], class_num=80, yolo_type: Optional[str] = None):
        self._emit("yolo:")
        self._emit("  anchors: " + ",".join(str(v) for v in anchors))
        self._emit(f"  classNum: {class_num}")
        if yolo_type:
            self._emit(f"  yoloType: {yolo_type}")
        self._top_done()

    def yoloout(self, layers: List[int], conf: float, nms: float, yolo_type: Optional[str] = None):
        self._emit("yoloout:")
        self._emit("  layers: " + ",".join(str(v) for v in layers))
        self._emit(f"  confThresh: {conf}")
        self._emit(f"  nmsThresh: {nms}")
        self._emit("  useSoftNms: 0")
        if yolo_type:
            self._emit(f"  yoloType: {yolo_type}")
        self._top_done()

    # -- blocks.  `body` callables emit sub-nodes; with size>1 the slots are replayed per instance ---
    def _block(self, name, size, act, emit_body):
        """emit_body() is called once for the text and `size-1` more times with text muted."""
        self._emit(f"{name}:")
        self._emit(f"  size: {size}")
        self._indent += 2
        emit_body()
        self._indent -= 2
        if act is not None:
            self._emit(f"  activation: {act}")
        self._top_done()
        for _ in range(size - 1):
            saved = self.lines
            self.lines = []
            emit_body()
            self.lines = saved
            self._top_done()

    def resblock(self, size, body, act="none"):
        """out = act(x + body(x))  (src/layers/MsnhResBlockLayer.cpp:215-302)."""
        self._block("resblock", size, act, body)

    def res2block(self, base, branch, act="none", size=1):
        """out = act(base(x) + branch(x))  (src/layers/MsnhRes2BlockLayer.cpp:342-447)."""
        def emit():
            start = _Shape(self.shape.c, self.shape.h, self.shape.w)
            self._emit("base:")
            self._indent += 2
            base()
            self._indent -= 2
            end = self.shape
            self.shape = start
            self._emit("branch:")
            self._indent += 2
            branch()
            self._indent -= 2
            assert (self.shape.c, self.shape.h, self.shape.w) == (end.c, end.h, end.w)
        self._block("res2block", size, act, emit)

    def addblock(self, size, branches, act=None):
        """out = sum of branches; a `None` branch is `empty:` = identity (src/layers/MsnhAddBlockLayer.cpp:255-357)."""
        def emit():
            start = _Shape(self.shape.c, self.shape.h, self.shape.w)
            end = None
            for br in branches:
                self.shape = _Shape(start.c, start.h, start.w)
                self._emit("branch:")
                self._indent += 2
                if br is None:
                    self._emit("empty:")
                else:
                    br()
                self._indent -= 2
                if end is not None:
                    assert (self.shape.c, self.shape.h, self.shape.w) == (end.c, end.h, end.w)
                end = self.shape
        self._block("addblock", size, act, emit)

    def concatblock(self, branches):
        """Channel concat of branch outputs in order (src/layers/MsnhConcatBlockLayer.cpp:255-355).
        Only `branch:` keys are written: any other key would create a spurious empty branch
        (src/io/MsnhParser.cpp:1972-2054)."""
        self._emit("concatblock:")
        start = _Shape(self.shape.c, self.shape.h, self.shape.w)
        total = 0
        self._indent += 2
        for br in branches:
            self.shape = _Shape(start.c, start.h, start.w)
            self._emit("branch:")
            self._indent += 2
            if br is None:
                self._emit("empty:")
            else:
                br()
            self._indent -= 2
            total += self.shape.c
        self._indent -= 2
        self.shape = _Shape(total, self.shape.h, self.shape.w)
        self._top_done()


# ------------------------------------------------------------------------------------------------
# architectures
# ------------------------------------------------------------------------------------------------
def _conv_bn(g: GraphWriter, filters, k, stride, pad, act):
    """ResNet style: bias-less conv followed by a stand-alone batchnorm node."""
    g.conv_node(filters, k, stride, pad, bn=0, bias=False, act="none")
    g.bn_node(act)


def resnet18(batch=1, size=224) -> GraphWriter:
    g = GraphWriter(batch, 3, size, size)
    g.conv(64, 7, 2, 3, bn=0, bias=False, act="none")
    g.batchnorm("relu")
    g.maxpool(3, 2, 1)

    def basic(c, stride=1):
        def body():
            _conv_bn(g, c, 3, stride, 1, "relu")
            _conv_bn(g, c, 3, 1, 1, "none")
        return body

    g.resblock(1, basic(64), "relu")
    g.resblock(1, basic(64), "relu")
    for c in (128, 256, 512):
        g.res2block(basic(c, 2), lambda c=c: _conv_bn(g, c, 1, 2, 0, "none"), "relu")
        g.resblock(1, basic(c), "relu")
    g.localavgpool(7)
    g.connect(1000)
    return g


def resnet50(batch=1, size=224) -> GraphWriter:
    g = GraphWriter(batch, 3, size, size)
    g.conv(64, 7, 2, 3, bn=0, bias=False, act="none")
    g.batchnorm("relu")
    g.maxpool(3, 2, 1)

    def bottleneck(c, stride=1):
        def body():
            _conv_bn(g, c, 1, 1, 0, "relu")
            _conv_bn(g, c, 3, stride, 1, "relu")
            _conv_bn(g, 4 * c, 1, 1, 0, "none")
        return body

    for c, n, stride in ((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)):
        g.res2block(bottleneck(c, stride), lambda c=c, s=stride: _conv_bn(g, 4 * c, 1, s, 0, "none"), "relu")
        g.resblock(n - 1, bottleneck(c), "relu")
    g.localavgpool(7)
    g.connect(1000)
    return g


def mobilenetv2(batch=1, size=224) -> GraphWriter:
    g = GraphWriter(batch, 3, size, size)
    g.conv(32, 3, 2, 1, bn=1, act="relu6")

    def inverted(cin, cout, stride, expand):
        hidden = cin * expand

        def body():
            if expand != 1:
                g.conv_node(hidden, 1, 1, 0, bn=1, act="relu6")
            g.conv_node(hidden, 3, stride, 1, groups=hidden, bn=1, act="relu6")
            g.conv_node(cout, 1, 1, 0, bn=1, act="none")
        return body

    cin = 32
    for t, c, n, s in ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2),
                       (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)):
        g.addblock(1, [inverted(cin, c, s, t)])                       # first block of a stage: no residual
        if n > 1:
            g.addblock(n - 1, [inverted(c, c, 1, t), None])           # residual blocks
        cin = c
    g.conv(1280, 1, 1, 0, bn=1, act="relu6")
    g.localavgpool(7)
    g.connect(1000)
    return g


def yolov3(batch=1, size=608, conf=0.5, nms=0.6) -> GraphWriter:
    g = GraphWriter(batch, 3, size, size)
    lk = "leaky"
    g.conv(32, 3, 1, 1, act=lk)

    def res(c):
        def body():
            g.conv_node(c // 2, 1, 1, 0, act=lk)
            g.conv_node(c, 3, 1, 1, act=lk)
        return body

    for c, n in ((64, 1), (128, 2), (256, 8), (512, 8), (1024, 4)):
        g.conv(c, 3, 2, 1, act=lk)
        g.resblock(n, res(c), "none")
    # after the backbone: top-level index 28 is the last 1024 block; 23 = last 512 block, 14 = last 256 block
    idx512, idx256 = 23, 14

    def pair(c):
        def body():
            g.conv_node(c, 1, 1, 0, act=lk)
            g.conv_node(2 * c, 3, 1, 1, act=lk)
        return body

    def head(c):
        def body():
            g.conv_node(2 * c, 3, 1, 1, act=lk)
            g.conv_node(255, 1, 1, 0, bn=0, act="none")
        return body

    yolos = []
    # scale 1 (stride 32)
    g.addblock(2, [pair(512)])
    g.conv(512, 1, 1, 0, act=lk)
    g.addblock(1, [head(512)])
    g.yolo([116, 90, 156, 198, 373, 326]); yolos.append(g.n_top - 1)
    # scale 2 (stride 16)
    g.route([-3])
    g.conv(256, 1, 1, 0, act=lk)
    g.upsample(2)
    g.route([-1, idx512])
    g.addblock(2, [pair(256)])
    g.conv(256, 1, 1, 0, act=lk)
    g.addblock(1, [head(256)])
    g.yolo([30, 61, 62, 45, 59, 119]); yolos.append(g.n_top - 1)
    # scale 3 (stride 8)
    g.route([-3])
    g.conv(128, 1, 1, 0, act=lk)
    g.upsample(2)
    g.route([-1, idx256])
    g.addblock(3, [pair(128)])
    g.conv(255, 1, 1, 0, bn=0, act="none")
    g.yolo([10, 13, 16, 30, 33, 23]); yolos.append(g.n_top - 1)
    g.yoloout(yolos, conf, nms)
    return g


def yolov4(batch=1, size=608, conf=0.5, nms=0.5) -> GraphWriter:
    g = GraphWriter(batch, 3, size, size)
    mi, lk = "mish", "leaky"
    g.conv(32, 3, 1, 1, act=mi)

    def csp_stage(c, n, first=False):
        """downsample conv, two 1x1 splits, n residual units, 1x1, concat, 1x1 fuse."""
        half = c if first else c // 2
        g.conv(c, 3, 2, 1, act=mi)
        g.conv(half, 1, 1, 0, act=mi)             # split A (kept for the concat)
        g.route([-2])
        g.conv(half, 1, 1, 0, act=mi)             # split B

        def unit():
            g.conv_node(c // 2 if first else half, 1, 1, 0, act=mi)
            g.conv_node(half, 3, 1, 1, act=mi)
        g.addblock(n, [unit, None])
        g.conv(half, 1, 1, 0, act=mi)
        g.route([-1, -(n + 4)])
        g.conv(c, 1, 1, 0, act=mi)

    csp_stage(64, 1, first=True)
    csp_stage(128, 2)
    csp_stage(256, 8); idx256 = g.n_top - 1      # 32
    csp_stage(512, 8); idx512 = g.n_top - 1      # 47
    csp_stage(1024, 4)

    g.conv(512, 1, 1, 0, act=lk)
    g.conv(1024, 3, 1, 1, act=lk)
    g.conv(512, 1, 1, 0, act=lk)
    g.concatblock([lambda: g.maxpool_node(13, 1, 6), lambda: g.maxpool_node(9, 1, 4),
                   lambda: g.maxpool_node(5, 1, 2), None])
    g.conv(512, 1, 1, 0, act=lk)
    g.conv(1024, 3, 1, 1, act=lk)
    g.conv(512, 1, 1, 0, act=lk); idx_p5 = g.n_top - 1        # 65

    def pair(c):
        def body():
            g.conv_node(c, 1, 1, 0, act=lk)
            g.conv_node(2 * c, 3, 1, 1, act=lk)
        return body

    def pair_rev(c):
        def body():
            g.conv_node(2 * c, 3, 1, 1, act=lk)
            g.conv_node(c, 1, 1, 0, act=lk)
        return body

    g.conv(256, 1, 1, 0, act=lk)
    g.upsample(2)
    g.route([idx512])
    g.conv(256, 1, 1, 0, act=lk)
    g.route([-1, -3])
    g.addblock(2, [pair(256)])
    g.conv(256, 1, 1, 0, act=lk); idx_p4 = g.n_top - 1        # 73
    g.conv(128, 1, 1, 0, act=lk)
    g.upsample(2)
    g.route([idx256])
    g.conv(128, 1, 1, 0, act=lk)
    g.route([-1, -3])
    g.conv(128, 1, 1, 0, act=lk)
    g.addblock(2, [pair_rev(128)])
    g.conv(256, 3, 1, 1, act=lk)
    g.conv(255, 1, 1, 0, bn=0, act="none")
    yolos = []
    g.yolo([12, 16, 19, 36, 40, 28]); yolos.append(g.n_top - 1)
    g.route([-4])
    g.conv(256, 3, 2, 1, act=lk)
    g.route([-1, idx_p4])
    g.addblock(2, [pair(256)])
    g.conv(256, 1, 1, 0, act=lk)
    g.conv(512, 3, 1, 1, act=lk)
    g.conv(255, 1, 1, 0, bn=0, act="none")
    g.yolo([36, 75, 76, 55, 72, 146]); yolos.append(g.n_top - 1)
    g.route([-4])
    g.conv(512, 3, 2, 1, act=lk)
    g.route([-1, idx_p5])
    g.addblock(3, [pair(512)])
    g.conv(255, 1, 1, 0, bn=0, act="none")
    g.yolo([142, 110, 192, 243, 459, 401]); yolos.append(g.n_top - 1)
    g.yoloout(yolos, conf, nms, "yolov4")
    return g


def yolov3_tiny(batch=1, size=416, conf=0.2, nms=0.2) -> GraphWriter:
    """The reference's yolov3_tiny graph (models/yolov3_tiny/yolov3_tiny.msnhnet): six conv + max-pool stages, the last
    pool with stride 1 behind a one-pixel padding layer, two heads."""
    g = GraphWriter(batch, 3, size, size)
    lk = "leaky"
    for i, c in enumerate((16, 32, 64, 128, 256)):
        g.conv(c, 3, 1, 1, act=lk)
        g.maxpool(2, 2, 0)
    g.conv(512, 3, 1, 1, act=lk)                 # layer 10
    g.padding(0, 1, 0, 1, 0.0)
    g.maxpool(2, 1, 0)
    g.conv(1024, 3, 1, 1, act=lk)
    g.conv(256, 1, 1, 0, act=lk)                 # layer 14
    g.conv(512, 3, 1, 1, act=lk)
    g.conv(255, 1, 1, 0, bn=0, act="none")
    yolos = []
    g.yolo([81, 82, 135, 169, 344, 319]); yolos.append(g.n_top - 1)
    g.route([-4])
    g.conv(128, 1, 1, 0, act=lk)
    g.upsample(2)
    g.route([-1, 8])
    g.conv(256, 3, 1, 1, act=lk)
    g.conv(255, 1, 1, 0, bn=0, act="none")
    g.yolo([10, 14, 23, 27, 37, 58]); yolos.append(g.n_top - 1)
    g.yoloout(yolos, conf, nms)
    return g


def yolov5s(batch=1, size=512, conf=0.5, nms=0.5) -> GraphWriter:
    """YOLOv5s in the node vocabulary of the reference's exported graph (models/yolov5s/yolov5s.msnhnet): focus slices,
    bias-less conv + batchnorm(eps 1e-3) + stand-alone hardswish, CSP stages whose residuals are `varop: add`, SPP, three
    yolov5 heads."""
    g = GraphWriter(batch, 3, size, size)

    def cbh(c, k, s):
        g.conv(c, k, s, k // 2, bn=0, bias=False, act="none")
        g.batchnorm("none", 0.001)
        g.act("hardswish")

    def csp(c, n, shortcut=True):
        start = g.n_top - 1                       # the layer feeding the stage
        h = c // 2
        cbh(h, 1, 1)
        for _ in range(n):
            inp = g.n_top - 1
            cbh(h, 1, 1)
            cbh(h, 3, 1)
            if shortcut:
                g.varop("add", [inp])
        g.conv(h, 1, 1, 0, bn=0, bias=False, act="none")
        a = g.n_top - 1
        g.route([start])
        g.conv(h, 1, 1, 0, bn=0, bias=False, act="none")
        b = g.n_top - 1
        g.route([a, b])
        g.batchnorm("none", 0.001)
        g.act("leaky,0.1")
        cbh(c, 1, 1)

    # focus
    g.act("none")
    g.slice(0, 1, 0, 2, 0, 2); g.route([-2])
    g.slice(0, 1, 1, 2, 0, 2); g.route([-4])
    g.slice(0, 1, 0, 2, 1, 2); g.route([-6])
    g.slice(0, 1, 1, 2, 1, 2)
    g.route([-7, -5, -3, -1])
    cbh(32, 3, 1)
    cbh(64, 3, 2); csp(64, 1)
    cbh(128, 3, 2); csp(128, 3); p3 = g.n_top - 1
    cbh(256, 3, 2); csp(256, 3); p4 = g.n_top - 1
    cbh(512, 3, 2)
    # SPP
    cbh(256, 1, 1); x = g.n_top - 1
    g.maxpool(5, 1, 2); m5 = g.n_top - 1
    g.route([x]); g.maxpool(9, 1, 4); m9 = g.n_top - 1
    g.route([x]); g.maxpool(13, 1, 6); m13 = g.n_top - 1
    g.route([x, m5, m9, m13])
    cbh(512, 1, 1)
    csp(512, 1, False)
    cbh(256, 1, 1); h5 = g.n_top - 1
    g.upsample(2); g.route([-1, p4]); csp(256, 1, False)
    cbh(128, 1, 1); h4 = g.n_top - 1
    g.upsample(2); g.route([-1, p3]); csp(128, 1, False); o3 = g.n_top - 1
    cbh(128, 3, 2); g.route([-1, h4]); csp(256, 1, False); o4 = g.n_top - 1
    cbh(256, 3, 2); g.route([-1, h5]); csp(512, 1, False); o5 = g.n_top - 1
    yolos = []
    for src, anchors in ((o3, [10, 13, 16, 30, 33, 23]), (o4, [30, 61, 62, 45, 59, 119]), (o5, [116, 90, 156, 198, 373, 326])):
        g.route([src])
        g.conv(255, 1, 1, 0, bn=0, act="none")
        g.yolo(anchors, yolo_type="yolov5"); yolos.append(g.n_top - 1)
    g.yoloout(yolos, conf, nms, "yolov5")
    return g


ARCHS = {"resnet18": resnet18, "resnet50": resnet50, "mobilenetv2": mobilenetv2,
         "yolov3": yolov3, "yolov4": yolov4, "yolov3_tiny": yolov3_tiny, "yolov5s": yolov5s}

# The benchmark configurations: (architecture, compute dtype, batch, input size)
CONFIGS = [
    ("resnet18", "fp32", 1, 224),
    ("resnet50", "fp16", 32, 224),
    ("mobilenetv2", "fp16", 64, 224),
    ("yolov3", "fp16", 8, 608),
    ("yolov4", "fp16", 16, 608),
]


# ------------------------------------------------------------------------------------------------
# seeded data
# ------------------------------------------------------------------------------------------------
def seeded_weights(slots: List[WeightSlot], seed: int) -> np.ndarray:
    """Flat float32 blob in `.msnhbin` order, drawn slot by slot from one PCG64 stream."""
    rng = np.random.Generator(np.random.PCG64(seed))
    parts = []
    for s in slots:
        if s.kind == "conv_w":
            v = rng.standard_normal(s.count, dtype=np.float32) * np.float32(math.sqrt(2.0 / s.fan_in))
        elif s.kind in ("bn_gamma", "bn_var"):
            v = rng.uniform(0.5, 1.5, s.count).astype(np.float32)
        elif s.kind in ("bn_beta", "bn_mean"):
            v = rng.standard_normal(s.count, dtype=np.float32) * np.float32(0.1)
        elif s.kind in ("fc_w", "bias"):
            b = 1.0 / math.sqrt(s.fan_in)
            v = rng.uniform(-b, b, s.count).astype(np.float32)
        else:
            raise ValueError(s.kind)
        parts.append(v.astype(np.float32))
    return np.concatenate(parts) if parts else np.zeros(0, np.float32)


_LAYOUT_KINDS = {0: "conv_w", 1: "bn_gamma", 2: "bn_beta", 3: "bn_mean", 4: "bn_var", 5: "bias", 6: "fc_w"}


def slots_from_layout(layout) -> List[WeightSlot]:
    """(what, count, fan_in) triples of netapi.Net.weight_layout -> weight slots for seeded_weights: a seeded weights file for any graph
    the host library can build, not only the ones this module emits."""
    return [WeightSlot(_LAYOUT_KINDS[w], n, max(f, 1)) for w, n, f in layout]


def seeded_input(batch: int, channels: int, height: int, width: int, seed: int) -> np.ndarray:
    """NCHW float32 ~U[0,1)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.random((batch, channels, height, width), dtype=np.float32)


def write_model(arch: str, directory: str, batch: int, size: int, seed: int = 0,
                **kw) -> Tuple[str, str, GraphWriter]:
    """Writes `<arch>_b<batch>_<size>.msnhnet/.msnhbin` into `directory`; returns both paths."""
    import os
    g = ARCHS[arch](batch=batch, size=size, **kw)
    stem = os.path.join(directory, f"{arch}_b{batch}_{size}")
    with open(stem + ".msnhnet", "w") as f:
        f.write(g.text())
    seeded_weights(g.slots, seed).tofile(stem + ".msnhbin")
    return stem + ".msnhnet", stem + ".msnhbin", g
