"""GPU parity of msnh_hip_conv2d (every algorithm) against the plain-C oracle convolution.

Tolerances: float32 1e-5 of max|ref| (only the accumulation order differs); float16 2e-3 of max|ref| with the
oracle fed the same float16-rounded inputs and weights (accumulation is float32, the output is rounded once)."""
import ctypes

import numpy as np
import pytest

import msnh_oracle_net as on
from msnhnet_amd import hipabi as abi

pytestmark = pytest.mark.gpu

TOL = {abi.F32: 1e-5, abi.F16: 2e-3}


def _case(rng, b, c, h, w, oc, k, groups=1):
    x = rng.standard_normal((b, c, h, w), dtype=np.float32)
    wt = rng.standard_normal((oc, c // groups, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (c // groups * k * k)))
    return x, wt


def _ref(x, wt, stride, pad, dil, groups, scale, shift, act, act_param, residual, act2, res_mul, out_mul):
    oc, _, k, _ = wt.shape
    y = on.conv(x, wt, oc, k, stride, pad, dil, groups)
    if scale is not None:
        y = y * scale.reshape(1, -1, 1, 1)
    if shift is not None:
        y = y + shift.reshape(1, -1, 1, 1)
    y = on.activate(y.astype(np.float32), act, act_param)
    if residual is not None:
        y = on.activate((y + np.float32(res_mul) * residual).astype(np.float32), act2, 0.1)
    return (np.float32(out_mul) * y).astype(np.float32)


CASES = [
    # b, c, h, w, oc, k, stride, pad, dil, groups
    (2, 16, 13, 11, 40, 3, 1, 1, 1, 1),
    (1, 32, 19, 19, 255, 1, 1, 0, 1, 1),
    (2, 24, 17, 15, 48, 3, 2, 1, 1, 1),
    (1, 16, 20, 20, 32, 3, 1, 2, 2, 1),
    (2, 32, 9, 9, 64, 3, 1, 1, 1, 2),
    (1, 64, 14, 14, 128, 3, 1, 1, 1, 1),
    (3, 128, 7, 7, 96, 1, 1, 0, 1, 1),
    (1, 8, 5, 5, 8, 5, 1, 2, 1, 1),
    (1, 72, 10, 12, 200, 3, 1, 1, 1, 1),
]


@pytest.mark.parametrize("dtype", [abi.F32, abi.F16])
@pytest.mark.parametrize("algo", ["igemm", "direct"])
@pytest.mark.parametrize("case", CASES)
def test_conv_plain(case, algo, dtype):
    import gpuutil as gu
    b, c, h, w, oc, k, stride, pad, dil, groups = case
    rng = np.random.default_rng(hash(case) % (2 ** 31))
    x, wt = _case(rng, b, c, h, w, oc, k, groups)
    if dtype == abi.F16:
        x, wt = gu.round_f16(x), gu.round_f16(wt)
    print("case", case, algo, dtype, flush=True)
    y, used = gu.conv2d(x, wt, dtype=dtype, stride=stride, pad=pad, dil=dil, groups=groups, algo=algo)
    assert used == algo
    ref = _ref(x, wt, stride, pad, dil, groups, None, None, "none", 0.1, None, "none", 1.0, 1.0)
    assert gu.rel_err(y, ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [abi.F32, abi.F16])
@pytest.mark.parametrize("algo", ["igemm", "direct"])
@pytest.mark.parametrize("act,act2", [("leaky", "none"), ("none", "relu"), ("mish", "none"), ("relu6", "leaky"), ("swish", "none")])
def test_conv_epilogue(act, act2, algo, dtype):
    """folded batch-norm, activation, residual add + second activation, power-of-two scales, channel-slice output."""
    import gpuutil as gu
    rng = np.random.default_rng(7)
    x, wt = _case(rng, 2, 32, 12, 10, 48, 3)
    res = rng.standard_normal((2, 48, 12, 10), dtype=np.float32)
    scale = rng.uniform(0.5, 1.5, 48).astype(np.float32)
    shift = (rng.standard_normal(48) * 0.1).astype(np.float32)
    if dtype == abi.F16:
        x, wt, res = gu.round_f16(x), gu.round_f16(wt), gu.round_f16(res)
    print("epilogue", act, act2, algo, dtype, flush=True)
    y, _ = gu.conv2d(x, wt, dtype=dtype, stride=1, pad=1, scale=scale, shift=shift, act=act, residual=res, act2=act2,
                     res_mul=4.0, out_mul=0.25, algo=algo, in_ld=40, out_ld=64, res_ld=56)
    ref = _ref(x, wt, 1, 1, 1, 1, scale, shift, act, 0.1, res, act2, 4.0, 0.25)
    assert gu.rel_err(y, ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [abi.F32, abi.F16])
def test_conv_every_tile_configuration(dtype):
    """all tile configurations of the implicit GEMM give the same answer (odd sizes exercise every edge guard)"""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(21)
    x, wt = _case(rng, 2, 40, 21, 19, 136, 3)
    res = rng.standard_normal((2, 136, 21, 19), dtype=np.float32)
    if dtype == abi.F16:
        x, wt, res = gu.round_f16(x), gu.round_f16(wt), gu.round_f16(res)
    ref = _ref(x, wt, 1, 1, 1, 1, None, None, "leaky", 0.1, res, "none", 1.0, 1.0)
    n = abi.lib().msnh_hip_conv2d_tile_count()
    assert n >= 1
    ran = 0
    for tile in range(1, n + 1):
        print("tile", tile, dtype, flush=True)
        try:
            y, _ = gu.conv2d(x, wt, dtype=dtype, stride=1, pad=1, act="leaky", residual=res, algo="igemm", tile=tile)
        except abi.HipError as e:
            assert "this tile needs" in str(e)
            continue
        ran += 1
        assert gu.rel_err(y, ref) <= TOL[dtype], tile
    assert ran >= 16            # 3x3 stride 1: the LDS-patch configurations apply too


@pytest.mark.parametrize("dtype", [abi.F32, abi.F16])
@pytest.mark.parametrize("k,stride", [(3, 1), (3, 2), (1, 1)])
def test_conv_multi_wavefront_tiles(k, stride, dtype):
    """The 8- and 12-wavefront tile configurations over several channel tiles and pixel tiles: 520 output channels (three 256-row
    tiles, the last one 8 rows), pixel counts that are no multiple of 192, 128 or 96, a ragged last channel chunk, residual add."""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(100 + 10 * k + stride)
    b, c, h, w, oc = 3, 72, 25, 23, 520
    x, wt = _case(rng, b, c, h, w, oc, k)
    pad = k // 2
    oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    res = rng.standard_normal((b, oc, oh, ow), dtype=np.float32)
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    if dtype == abi.F16:
        x, wt, res = gu.round_f16(x), gu.round_f16(wt), gu.round_f16(res)
    ref = _ref(x, wt, stride, pad, 1, 1, scale, shift, "leaky", 0.1, res, "relu", 1.0, 1.0)
    ran = 0
    for tile in range(32, abi.lib().msnh_hip_conv2d_tile_count() + 1):
        print("multi-wavefront tile", tile, k, stride, dtype, flush=True)
        try:
            y, _ = gu.conv2d(x, wt, dtype=dtype, stride=stride, pad=pad, scale=scale, shift=shift, act="leaky", residual=res, act2="relu",
                             algo="igemm", tile=tile)
        except abi.HipError as e:
            assert "this tile needs" in str(e)
            continue
        ran += 1
        assert gu.rel_err(y, ref) <= TOL[dtype], tile
    assert ran >= 8


@pytest.mark.parametrize("dtype", [abi.F32, abi.F16])
@pytest.mark.parametrize("k,stride", [(3, 1), (3, 2), (1, 1)])
def test_conv_xcd_arrangements(k, stride, dtype):
    """msnh_conv_desc::xcd_blocks only changes which workgroup computes which tile: every arrangement gives the bits of the default
    one, for every tile configuration that takes the shape.  328 output channels and 3 x 23 x 21 pixels make channel-tile and
    pixel-tile counts that the 2 x 4, 4 x 2 and 8 x 1 grids of XCDs do not divide (XCDs with fewer tiles, ids past the last tile);
    the default arrangement is checked against the oracle, and so is the library's own choice (xcd_blocks = 0)."""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(300 + 10 * k + stride)
    b, c, h, w, oc = 3, 64, 23, 21, 328
    x, wt = _case(rng, b, c, h, w, oc, k)
    pad = k // 2
    oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    res = rng.standard_normal((b, oc, oh, ow), dtype=np.float32)
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    if dtype == abi.F16:
        x, wt, res = gu.round_f16(x), gu.round_f16(wt), gu.round_f16(res)
    ref = _ref(x, wt, stride, pad, 1, 1, scale, shift, "leaky", 0.1, res, "none", 1.0, 1.0)
    kw = dict(dtype=dtype, stride=stride, pad=pad, scale=scale, shift=shift, act="leaky", residual=res, algo="igemm")
    ran = 0
    for tile in range(1, abi.lib().msnh_hip_conv2d_tile_count() + 1):
        print("xcd arrangements, tile", tile, k, stride, dtype, flush=True)
        try:
            y1, _ = gu.conv2d(x, wt, tile=tile, xcd_blocks=1, **kw)
        except abi.HipError as e:
            assert "this tile" in str(e)
            continue
        ran += 1
        assert gu.rel_err(y1, ref) <= TOL[dtype], tile
        for g in (0, 2, 4, 8):
            yg, _ = gu.conv2d(x, wt, tile=tile, xcd_blocks=g, **kw)
            assert np.array_equal(yg, y1), (tile, g)
    assert ran >= 8
    with pytest.raises(abi.HipError, match="xcd_blocks"):
        gu.conv2d(x, wt, tile=1, xcd_blocks=3, **kw)


@pytest.mark.parametrize("dtype", [abi.F32, abi.F16])
@pytest.mark.parametrize("shape", [(2, 16, 19, 19, 40), (1, 64, 38, 38, 96), (3, 8, 7, 5, 16), (1, 32, 76, 76, 64), (2, 72, 13, 11, 136), (1, 200, 20, 20, 264)])
def test_conv_patch_tiles(shape, dtype):
    """3x3 stride-1 layers with the input patch resident in LDS: image borders, batch seams, ragged channel chunks; the last shape runs
    four channel chunks (both patch stages in turn, the last chunk ragged) over two channel tiles"""
    import ctypes
    import gpuutil as gu
    gu.init()
    b, c, h, w, oc = shape
    rng = np.random.default_rng(sum(shape))
    x, wt = _case(rng, b, c, h, w, oc, 3)
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    if dtype == abi.F16:
        x, wt = gu.round_f16(x), gu.round_f16(wt)
    ref = _ref(x, wt, 1, 1, 1, 1, scale, shift, "leaky", 0.1, None, "none", 1.0, 1.0)
    ran = 0
    for tile in range(14, abi.lib().msnh_hip_conv2d_tile_count() + 1):
        print("patch tile", tile, shape, dtype, flush=True)
        try:
            y, _ = gu.conv2d(x, wt, dtype=dtype, stride=1, pad=1, scale=scale, shift=shift, act="leaky", algo="igemm", tile=tile)
        except abi.HipError as e:
            assert "this tile" in str(e)
            continue
        ran += 1
        assert gu.rel_err(y, ref) <= TOL[dtype], tile
    assert ran >= 3


def test_conv_f16_in_f32_out():
    import gpuutil as gu
    rng = np.random.default_rng(11)
    x, wt = _case(rng, 2, 64, 8, 8, 255, 1)
    x, wt = gu.round_f16(x), gu.round_f16(wt)
    bias = rng.standard_normal(255).astype(np.float32)
    y, used = gu.conv2d(x, wt, dtype=abi.F16, out_dtype=abi.F32, shift=bias, out_ld=256)
    assert used == "igemm"
    ref = _ref(x, wt, 1, 0, 1, 1, None, bias, "none", 0.1, None, "none", 1.0, 1.0)
    assert gu.rel_err(y, ref) <= 1e-5


@pytest.mark.parametrize("dtype", [abi.F32, abi.F16])
@pytest.mark.parametrize("c,h,w,k,stride,pad", [(32, 14, 14, 3, 1, 1), (96, 15, 13, 3, 2, 1), (20, 9, 9, 3, 1, 1), (16, 8, 8, 5, 1, 2)])
def test_conv_depthwise(c, h, w, k, stride, pad, dtype):
    import gpuutil as gu
    rng = np.random.default_rng(c)
    x, wt = _case(rng, 2, c, h, w, c, k, groups=c)
    scale = rng.uniform(0.5, 1.5, c).astype(np.float32)
    shift = (rng.standard_normal(c) * 0.1).astype(np.float32)
    if dtype == abi.F16:
        x, wt = gu.round_f16(x), gu.round_f16(wt)
    y, used = gu.conv2d(x, wt, dtype=dtype, stride=stride, pad=pad, groups=c, scale=scale, shift=shift, act="relu6")
    assert used == "depthwise"
    ref = _ref(x, wt, stride, pad, 1, c, scale, shift, "relu6", 0.1, None, "none", 1.0, 1.0)
    assert gu.rel_err(y, ref) <= TOL[dtype]


@pytest.mark.parametrize("b,c,h,w,stride", [(2, 32, 14, 14, 1), (1, 144, 9, 21, 1), (2, 24, 7, 7, 1), (1, 960, 7, 7, 1), (3, 64, 33, 18, 2), (1, 8, 5, 70, 1),
                                            (2, 384, 14, 14, 2), (1, 32, 112, 112, 1), (2, 96, 15, 13, 2), (1, 16, 1, 1, 1), (1, 40, 3, 2, 2)])
@pytest.mark.parametrize("act", ["relu6", "leaky"])
def test_conv_depthwise_index_forms(b, c, h, w, stride, act):
    """3x3 depthwise float16: the kernel with 32-bit index arithmetic and reciprocal-multiplication divisions (the default where every
    size is below 2^31) and the general one (tile 1) agree with the reference convolution and with each other bit for bit; sizes that
    are not multiples of the strip, one-pixel images, an output stride wider than the channel count"""
    import gpuutil as gu
    rng = np.random.default_rng(c * h + w)
    x, wt = _case(rng, b, c, h, w, c, 3, groups=c)
    scale = rng.uniform(0.5, 1.5, c).astype(np.float32)
    shift = (rng.standard_normal(c) * 0.1).astype(np.float32)
    x, wt = gu.round_f16(x), gu.round_f16(wt)
    ref = _ref(x, wt, stride, 1, 1, c, scale, shift, act, 0.1, None, "none", 1.0, 1.0)
    outs = []
    for tile in (1, 0):
        y, used = gu.conv2d(x, wt, dtype=abi.F16, stride=stride, pad=1, groups=c, scale=scale, shift=shift, act=act, tile=tile, out_ld=(c + 15) // 8 * 8)
        assert used == "depthwise"
        assert gu.rel_err(y, ref) <= TOL[abi.F16], tile
        outs.append(y)
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("out_dtype", [abi.F32, abi.F16])
@pytest.mark.parametrize("h,w,oc,k,stride,pad", [(33, 31, 32, 3, 1, 1), (40, 40, 64, 7, 2, 3), (25, 27, 32, 3, 2, 1), (70, 100, 64, 3, 1, 1),
                                                 (37, 45, 64, 7, 2, 3), (30, 70, 32, 7, 1, 3), (21, 19, 128, 7, 2, 0), (224, 224, 64, 7, 2, 3),
                                                 (9, 150, 64, 7, 2, 5), (31, 33, 64, 5, 2, 2)])
def test_conv_stem(h, w, oc, k, stride, pad, out_dtype):
    """first layer: NCHW float32 in, NHWC out, cast fused"""
    import gpuutil as gu
    rng = np.random.default_rng(oc + k)
    x = rng.random((2, 3, h, w), dtype=np.float32)
    wt = rng.standard_normal((oc, 3, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (3 * k * k)))
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    y, used = gu.conv2d(x, wt, dtype=out_dtype, stride=stride, pad=pad, scale=scale, shift=shift, act="leaky")
    assert used == "stem"
    if out_dtype == abi.F16 and k == 3:
        # the matrix-core variant casts image and weights to float16 on the way in
        x, wt = gu.round_f16(x), gu.round_f16(wt)
    ref = _ref(x, wt, stride, pad, 1, 1, scale, shift, "leaky", 0.1, None, "none", 1.0, 1.0)
    assert gu.rel_err(y, ref) <= (1e-5 if out_dtype == abi.F32 else 1e-3)


@pytest.mark.parametrize("b,c,h,w,oc", [(2, 16, 12, 10, 24), (1, 32, 19, 19, 64), (3, 8, 7, 9, 8), (1, 64, 38, 38, 128)])
@pytest.mark.parametrize("with_res", [False, True])
def test_conv_winograd(b, c, h, w, oc, with_res):
    """Winograd F(2x2,3x3): same result as the direct form (odd sizes exercise the partial tiles), full epilogue."""
    import gpuutil as gu
    rng = np.random.default_rng(b * 100 + c)
    x, wt = _case(rng, b, c, h, w, oc, 3)
    res = rng.standard_normal((b, oc, h, w), dtype=np.float32) if with_res else None
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    x, wt = gu.round_f16(x), gu.round_f16(wt)
    if with_res:
        res = gu.round_f16(res)
    y, used = gu.conv2d(x, wt, dtype=abi.F16, stride=1, pad=1, scale=scale, shift=shift, act="leaky", residual=res, act2="none",
                        res_mul=2.0, out_mul=0.5, algo="winograd", out_ld=oc + 8, res_ld=oc + 8 if with_res else None)
    assert used == "winograd"
    ref = _ref(x, wt, 1, 1, 1, 1, scale, shift, "leaky", 0.1, res, "none", 2.0, 0.5)
    # the transformed weights are rounded to float16 a second time: a little above the direct kernel's tolerance
    assert gu.rel_err(y, ref) <= 3 * TOL[abi.F16]
    # every tile configuration of the transformed-domain GEMM that accepts the shape gives the same answer
    L = abi.lib()
    for tile in (2, 8, 12):
        y2, _ = gu.conv2d(x, wt, dtype=abi.F16, stride=1, pad=1, scale=scale, shift=shift, act="leaky", residual=res, act2="none",
                          res_mul=2.0, out_mul=0.5, algo="winograd", out_ld=oc + 8, res_ld=oc + 8 if with_res else None, tile=tile)
        assert gu.rel_err(y2, ref) <= 3 * TOL[abi.F16]


@pytest.mark.parametrize("b,c,h,w,oc", [(2, 16, 12, 10, 24), (1, 32, 19, 19, 64), (3, 48, 7, 9, 8), (1, 64, 38, 38, 128), (8, 256, 38, 38, 512), (2, 32, 21, 37, 136)])
@pytest.mark.parametrize("with_res", [False, True])
def test_conv_winograd_fused(b, c, h, w, oc, with_res):
    """Winograd F(2x2,3x3) in one launch (input transform into LDS with packed float16 additions, 16 accumulator sets in registers,
    output transform in the epilogue): same result as the direct form within the Winograd tolerance, odd sizes (partial tiles at the
    right and bottom edge), tile runs that cross image seams, partial channel blocks, channel slices of wider tensors, full epilogue"""
    import gpuutil as gu
    rng = np.random.default_rng(b * 100 + c + 7)
    x, wt = _case(rng, b, c, h, w, oc, 3)
    res = rng.standard_normal((b, oc, h, w), dtype=np.float32) if with_res else None
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    x, wt = gu.round_f16(x), gu.round_f16(wt)
    if with_res:
        res = gu.round_f16(res)
    kw = dict(dtype=abi.F16, stride=1, pad=1, scale=scale, shift=shift, act="leaky", residual=res, act2="leaky" if with_res else "none",
              res_mul=2.0, out_mul=0.5, algo="winograd_fused", in_ld=c + 8, out_ld=oc + 8, res_ld=oc + 16 if with_res else None)
    print("winograd fused", (b, c, h, w, oc), with_res, flush=True)
    y, used = gu.conv2d(x, wt, **kw)
    assert used == "winograd_fused"
    ref = _ref(x, wt, 1, 1, 1, 1, scale, shift, "leaky", 0.1, res, "leaky" if with_res else "none", 2.0, 0.5)
    e = gu.rel_err(y, ref)
    print("error", e, flush=True)
    # float16 transformed weights and two float16 roundings in the input transform: above the direct kernel's tolerance
    assert e <= 4 * TOL[abi.F16]
    y2, _ = gu.conv2d(x, wt, **kw)
    assert np.array_equal(y, y2)


SPLITK_CASES = [
    # b, c, h, w, oc, k, stride, pad, groups
    (1, 512, 7, 7, 512, 3, 1, 1, 1),
    (2, 256, 14, 14, 512, 3, 2, 1, 1),
    (1, 1024, 7, 7, 256, 1, 1, 0, 1),
    (1, 72, 10, 12, 200, 3, 1, 1, 1),       # ragged K chunks and a partial channel tile
    (2, 128, 9, 9, 64, 3, 1, 1, 2),
    (16, 2048, 1, 1, 1000, 1, 1, 0, 1),     # a fully connected layer
]


@pytest.mark.parametrize("dtype", [abi.F32, abi.F16])
@pytest.mark.parametrize("case", SPLITK_CASES)
def test_conv_split_k(case, dtype):
    """Split-K implicit GEMM: the K loop cut over several workgroups, partial sums added in slice order.  Same result
    as the oracle to the one-pass kernel's tolerance, with the full epilogue, for every tile configuration that takes
    the shape, and bit-identical from run to run."""
    import ctypes
    import gpuutil as gu
    b, c, h, w, oc, k, stride, pad, groups = case
    rng = np.random.default_rng(sum(case))
    x, wt = _case(rng, b, c, h, w, oc, k, groups)
    oh = (h + 2 * pad - k) // stride + 1
    ow = (w + 2 * pad - k) // stride + 1
    res = rng.standard_normal((b, oc, oh, ow), dtype=np.float32)
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    if dtype == abi.F16:
        x, wt, res = gu.round_f16(x), gu.round_f16(wt), gu.round_f16(res)
    ref = _ref(x, wt, stride, pad, 1, groups, scale, shift, "leaky", 0.1, res, "relu", 2.0, 0.5)
    kw = dict(dtype=dtype, stride=stride, pad=pad, groups=groups, scale=scale, shift=shift, act="leaky", residual=res, act2="relu",
              res_mul=2.0, out_mul=0.5, algo="igemm_splitk", out_ld=oc + 8, res_ld=oc + 8)
    L = abi.lib()
    d = abi.ConvDesc(dtype, dtype, b, h, w, c, c, oc, oh, ow, oc + 8, k, stride, pad, 1, groups, abi.ACT["leaky"], 0.1, 1, oc + 8, abi.ACT["relu"], 0.1, 2.0, 0.5,
                     abi.ALGO["igemm_splitk"], 0)
    tried = 0
    for tile in range(0, L.msnh_hip_conv2d_tile_count() + 1):
        d.tile = tile
        if not L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), tile):
            continue
        y, used = gu.conv2d(x, wt, tile=tile, **kw)
        assert used == "igemm_splitk"
        assert gu.rel_err(y, ref) <= TOL[dtype], (tile, gu.rel_err(y, ref))
        if tried % 4 == 0:
            y2, _ = gu.conv2d(x, wt, tile=tile, **kw)
            assert np.array_equal(y, y2), tile
        tried += 1
    assert tried >= 3


def test_conv_split_k_rejects():
    """Split-K needs its workspace, a K loop long enough to cut, and few enough output tiles to be worth cutting."""
    import ctypes
    L = abi.lib()
    # a 1x1 layer over 16 channels has a single tile step
    d = abi.ConvDesc(abi.F16, abi.F16, 1, 8, 8, 16, 16, 16, 8, 8, 16, 1, 1, 0, 1, 1, 22, 0.1, 0, 16, 22, 0.1, 1.0, 1.0, abi.ALGO["igemm_splitk"], 0)
    assert all(L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), t) == 0 for t in range(0, L.msnh_hip_conv2d_tile_count() + 1))
    # a launch that already fills the chip
    d = abi.ConvDesc(abi.F16, abi.F16, 8, 76, 76, 256, 256, 256, 76, 76, 256, 3, 1, 1, 1, 1, 22, 0.1, 0, 256, 22, 0.1, 1.0, 1.0, abi.ALGO["igemm_splitk"], 1)
    assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), 1) == 0
    # a good shape without its workspace
    d = abi.ConvDesc(abi.F16, abi.F16, 1, 7, 7, 512, 512, 512, 7, 7, 512, 3, 1, 1, 1, 1, 22, 0.1, 0, 512, 22, 0.1, 1.0, 1.0, abi.ALGO["igemm_splitk"], 1)
    assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), 1) == 1
    assert L.msnh_hip_conv2d_workspace_bytes(ctypes.byref(d), abi.ALGO["igemm_splitk"]) == 8 * 49 * 512 * 4
    buf = ctypes.c_void_p(256)
    assert L.msnh_hip_conv2d(ctypes.byref(d), buf, buf, None, None, None, buf, None, 0, None) != 0
    assert b"workspace" in L.msnh_hip_last_error()


@pytest.mark.parametrize("b,c,h,w,oc", [(2, 64, 19, 17, 32), (1, 16, 30, 30, 96), (3, 24, 9, 11, 144 - 16), (2, 128, 13, 13, 64), (1, 96, 7, 7, 24),
                                         (2, 32, 8, 8, 16), (1, 128, 20, 21, 128), (4, 8, 5, 5, 8), (1, 80, 12, 9, 40)])
@pytest.mark.parametrize("with_res", [False, True])
def test_conv_pointwise(b, c, h, w, oc, with_res):
    """1x1 convolution with the weights resident in LDS and pixels loaded straight into MFMA fragments: every combination of
    channel-block counts, ragged K (in_c % 16 == 8), partial last blocks (out_c % 32 != 0), pixel tails, full epilogue."""
    import gpuutil as gu
    rng = np.random.default_rng(b * 1000 + c + oc)
    x, wt = _case(rng, b, c, h, w, oc, 1)
    res = rng.standard_normal((b, oc, h, w), dtype=np.float32) if with_res else None
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    x, wt = gu.round_f16(x), gu.round_f16(wt)
    if with_res:
        res = gu.round_f16(res)
    y, used = gu.conv2d(x, wt, dtype=abi.F16, scale=scale, shift=shift, act="leaky", residual=res, act2="relu6", res_mul=2.0, out_mul=0.5,
                        algo="pointwise", in_ld=c + 8, out_ld=oc + 8, res_ld=oc + 16 if with_res else None)
    assert used == "pointwise"
    ref = _ref(x, wt, 1, 0, 1, 1, scale, shift, "leaky", 0.1, res, "relu6", 2.0, 0.5)
    assert gu.rel_err(y, ref) <= TOL[abi.F16]
    # without the affine
    y, _ = gu.conv2d(x, wt, dtype=abi.F16, act="none", algo="pointwise")
    assert gu.rel_err(y, _ref(x, wt, 1, 0, 1, 1, None, None, "none", 0.1, None, "none", 1.0, 1.0)) <= TOL[abi.F16]


def test_conv_pointwise_rejects():
    import ctypes
    L = abi.lib()
    mk = lambda **kw: abi.ConvDesc(**{**dict(dtype=abi.F16, out_dtype=abi.F16, batch=1, in_h=8, in_w=8, in_c=16, in_ld=16, out_c=16, out_h=8, out_w=8, out_ld=16,
                                             ksize=1, stride=1, pad=0, dilation=1, groups=1, act=22, act_param=0.1, has_residual=0, res_ld=16, act2=22,
                                             act2_param=0.1, res_mul=1.0, out_mul=1.0, algo=abi.ALGO["pointwise"], tile=0), **kw})
    assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(mk()), 0) == 1
    assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(mk()), 1) == 0
    for bad in (dict(in_c=136, in_ld=136), dict(out_c=136, out_ld=136), dict(in_c=12, in_ld=16), dict(dtype=abi.F32, out_dtype=abi.F32),
                dict(ksize=3, pad=1), dict(stride=2, out_h=4, out_w=4), dict(groups=2)):
        assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(mk(**bad)), 0) == 0, bad


def test_conv_winograd_rejects():
    import ctypes
    import gpuutil as gu
    gu.init()
    L = abi.lib()
    # stride 2 is not a Winograd shape
    d = abi.ConvDesc(abi.F16, abi.F16, 1, 8, 8, 16, 16, 16, 4, 4, 16, 3, 2, 1, 1, 1, 22, 0.1, 0, 16, 22, 0.1, 1.0, 1.0, abi.ALGO["winograd"], 0)
    assert L.msnh_hip_conv2d(ctypes.byref(d), 16, 16, None, None, None, 16, 256, 1 << 20, None) != 0
    assert b"Winograd" in L.msnh_hip_last_error()
    # a good shape without its workspace
    d = abi.ConvDesc(abi.F16, abi.F16, 1, 8, 8, 16, 16, 16, 8, 8, 16, 3, 1, 1, 1, 1, 22, 0.1, 0, 16, 22, 0.1, 1.0, 1.0, abi.ALGO["winograd"], 0)
    assert L.msnh_hip_conv2d_workspace_bytes(ctypes.byref(d), abi.ALGO["winograd"]) > 0
    assert L.msnh_hip_conv2d(ctypes.byref(d), 256, 256, None, None, None, 256, None, 0, None) != 0
    assert b"workspace" in L.msnh_hip_last_error()


def test_conv_rejects_bad_shapes():
    import ctypes
    import gpuutil as gu
    gu.init()
    L = abi.lib()
    d = abi.ConvDesc(abi.F16, abi.F16, 1, 8, 8, 12, 12, 16, 8, 8, 16, 3, 1, 1, 1, 1, 22, 0.1, 0, 16, 22, 0.1, 1.0, 1.0, abi.ALGO["igemm"], 0)
    assert L.msnh_hip_conv2d(ctypes.byref(d), 16, 16, None, None, None, 16, None, 0, None) != 0      # in_c % 8
    assert b"IGEMM" in L.msnh_hip_last_error()
    d = abi.ConvDesc(abi.F16, abi.F16, 1, 8, 8, 16, 16, 16, 9, 8, 16, 3, 1, 1, 1, 1, 22, 0.1, 0, 16, 22, 0.1, 1.0, 1.0, 0, 0)
    assert L.msnh_hip_conv2d(ctypes.byref(d), 16, 16, None, None, None, 16, None, 0, None) != 0      # wrong out_h


@pytest.mark.parametrize("b,h,w,c2,act", [(2, 32, 64, 64, "leaky"), (1, 37, 45, 32, "mish"), (3, 16, 16, 128, "relu"), (1, 608, 608, 64, "leaky")])
def test_conv_stem_down(b, h, w, c2, act):
    """first layer (3x3 stride 1, 32 filters, NCHW float32 in) + 3x3 stride-2 layer as one launch: equal to the two layers run one
    after the other with the intermediate rounded to float16 (odd sizes exercise ragged tiles and the zero padding of the
    intermediate at all four borders; mid_mul / out_mul are the power-of-two scales of a float16 plan)"""
    import torch

    import gpuutil as gu
    gu.init()
    L = abi.lib()
    rng = np.random.default_rng(b * 1000 + h + c2)
    x = rng.random((b, 3, h, w), dtype=np.float32)
    w1 = rng.standard_normal((32, 3, 3, 3), dtype=np.float32) * np.float32(np.sqrt(2.0 / 27))
    w2 = rng.standard_normal((c2, 32, 3, 3), dtype=np.float32) * np.float32(np.sqrt(2.0 / 288))
    s1, h1 = rng.uniform(0.5, 1.5, 32).astype(np.float32), (rng.standard_normal(32) * 0.1).astype(np.float32)
    s2, h2 = rng.uniform(0.5, 1.5, c2).astype(np.float32), (rng.standard_normal(c2) * 0.1).astype(np.float32)
    mid_mul, out_mul = 0.25, 2.0
    assert L.msnh_hip_conv_stem_down_supported(3, 32, 3, 1, 1, c2, 3, 2, 1) == 1
    assert L.msnh_hip_conv_stem_down_supported(3, 64, 3, 1, 1, c2, 3, 2, 1) == 0 and L.msnh_hip_conv_stem_down_supported(3, 32, 3, 1, 1, 96, 3, 2, 1) == 0
    p1 = np.zeros(L.msnh_hip_conv_stem_down_packed_elems(c2, 0), np.float16)
    p2 = np.zeros(L.msnh_hip_conv_stem_down_packed_elems(c2, 1), np.float16)
    abi.check(L.msnh_hip_conv_stem_down_pack(w1.ctypes.data_as(ctypes.c_void_p), c2, w2.ctypes.data_as(ctypes.c_void_p), p1.ctypes.data_as(ctypes.c_void_p),
                                             p2.ctypes.data_as(ctypes.c_void_p)))
    oh, ow = (h - 1) // 2 + 1, (w - 1) // 2 + 1
    ld = c2 + 8
    xd, p1d, p2d = gu.dev(x), gu.dev(p1), gu.dev(p2)
    s1d, h1d, s2d, h2d = gu.dev(s1), gu.dev(h1), gu.dev(s2 / np.float32(mid_mul)), gu.dev(h2)
    yd = torch.full((b, oh, ow, ld), 3.0, dtype=torch.float16).cuda()
    gu.sync()
    print("conv_stem_down", b, h, w, c2, act, flush=True)
    abi.check(L.msnh_hip_conv_stem_down(b, h, w, gu.ptr(xd), gu.ptr(p1d), gu.ptr(s1d), gu.ptr(h1d), abi.ACT[act], 0.1, mid_mul, c2, gu.ptr(p2d), gu.ptr(s2d),
                                        gu.ptr(h2d), abi.ACT[act], 0.1, out_mul, gu.ptr(yd), ld, None))
    gu.sync()
    got = gu.nchw_host(yd, c2)
    assert (yd[..., c2:].float().cpu().numpy() == 3.0).all(), "kernel wrote outside its channel slice"
    # the same in two steps: image and weights rounded to float16 as the matrix cores see them, the intermediate stored as
    # float16(mid_mul * value) and multiplied back by the second layer's scale
    mid = _ref(gu.round_f16(x), gu.round_f16(w1), 1, 1, 1, 1, s1, h1, act, 0.1, None, "none", 1.0, mid_mul)
    mid = gu.round_f16(mid)
    ref = _ref(mid, gu.round_f16(w2), 2, 1, 1, 1, s2 / np.float32(mid_mul), h2, act, 0.1, None, "none", 1.0, out_mul)
    assert got.shape == ref.shape
    assert gu.rel_err(got, ref) <= 2e-3

    # ... and with the 1x1 convolution behind it in the same launch (32 filters: the opening of Darknet-53's first residual block):
    # y carries the same bits as without, z equals the oracle's 1x1 over y as stored, and msnh_hip_conv2d's over the device's y
    assert L.msnh_hip_conv_stem_down_tail_supported(c2, 32, 1, 1, 0) == 1
    assert L.msnh_hip_conv_stem_down_tail_supported(c2, 64, 1, 1, 0) == 0 and L.msnh_hip_conv_stem_down_tail_supported(c2, 32, 3, 1, 1) == 0
    w3 = rng.standard_normal((32, c2), dtype=np.float32) * np.float32(np.sqrt(2.0 / c2))
    s3, h3 = rng.uniform(0.5, 1.5, 32).astype(np.float32), (rng.standard_normal(32) * 0.1).astype(np.float32)
    z_mul, zld = 0.5, 40
    p3 = np.zeros(L.msnh_hip_conv_stem_down_tail_packed_elems(c2), np.float16)
    abi.check(L.msnh_hip_conv_stem_down_tail_pack(c2, w3.ctypes.data_as(ctypes.c_void_p), p3.ctypes.data_as(ctypes.c_void_p)))
    p3d, s3d, h3d = gu.dev(p3), gu.dev(s3 / np.float32(out_mul)), gu.dev(h3)
    yd2 = torch.full((b, oh, ow, ld), 3.0, dtype=torch.float16).cuda()
    zd = torch.full((b, oh, ow, zld), 5.0, dtype=torch.float16).cuda()
    gu.sync()
    abi.check(L.msnh_hip_conv_stem_down_tail(b, h, w, gu.ptr(xd), gu.ptr(p1d), gu.ptr(s1d), gu.ptr(h1d), abi.ACT[act], 0.1, mid_mul, c2, gu.ptr(p2d), gu.ptr(s2d),
                                             gu.ptr(h2d), abi.ACT[act], 0.1, out_mul, gu.ptr(yd2), ld, gu.ptr(p3d), gu.ptr(s3d), gu.ptr(h3d), abi.ACT["leaky"], 0.1,
                                             z_mul, gu.ptr(zd), zld, None))
    gu.sync()
    assert torch.equal(yd2, yd)
    assert (zd[..., 32:].float().cpu().numpy() == 5.0).all(), "kernel wrote outside z's channel slice"
    z = gu.nchw_host(zd, 32)
    z_ref = _ref(got, gu.round_f16(w3).reshape(32, c2, 1, 1), 1, 0, 1, 1, s3 / np.float32(out_mul), h3, "leaky", 0.1, None, "none", 1.0, z_mul)
    assert gu.rel_err(z, z_ref) <= 2e-3
    z2, _ = gu.conv2d(got, gu.round_f16(w3).reshape(32, c2, 1, 1), dtype=abi.F16, scale=s3 / np.float32(out_mul), shift=h3, act="leaky", out_mul=z_mul, algo="igemm", tile=38)
    print("z equals a separate launch bit for bit:", bool(np.array_equal(z, z2)), flush=True)
    assert gu.rel_err(z, z2) <= 1e-3


TAIL_CASES = [
    # b, c, h, w, oc, k, stride, pad, oc2, residual
    (2, 128, 19, 19, 256, 3, 1, 1, 128, True),       # the 76x76 residual stage of Darknet-53, reduced
    (1, 64, 13, 17, 256, 3, 1, 1, 128, False),
    (2, 128, 20, 20, 256, 3, 2, 1, 128, False),      # the stride-2 convolution in front of a stage
    (1, 64, 9, 11, 200, 3, 1, 1, 72, True),          # channel counts below the tile's
    (1, 256, 14, 14, 128, 1, 1, 0, 64, True),        # 1x1 in front
    (3, 128, 16, 16, 128, 3, 1, 1, 128, True),       # the 128-channel tile
    (1, 32, 30, 30, 64, 3, 1, 1, 32, False),
]


@pytest.mark.parametrize("case", TAIL_CASES)
@pytest.mark.parametrize("write_y", [True, False])
def test_conv_tail(case, write_y):
    """msnh_hip_conv2d_tail (a convolution and the 1x1 convolution that reads its result, one launch) on every tile that carries a tail:
    y and z against the oracle's two convolutions (y rounded to float16 in between, as two launches round it), and bit for bit against
    msnh_hip_conv2d called twice."""
    import gpuutil as gu
    L = abi.lib()
    b, c, h, w, oc, k, stride, pad, oc2, with_res = case
    rng = np.random.default_rng(hash(case) % (2 ** 31))
    x, wt = _case(rng, b, c, h, w, oc, k)
    w2 = (rng.standard_normal((oc2, oc), dtype=np.float32) * np.float32(np.sqrt(2.0 / oc)))
    oh, ow = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    res = gu.round_f16(rng.standard_normal((b, oc, oh, ow), dtype=np.float32)) if with_res else None
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    scale2 = rng.uniform(0.5, 1.5, oc2).astype(np.float32)
    shift2 = (rng.standard_normal(oc2) * 0.1).astype(np.float32)
    x, wt, w2 = gu.round_f16(x), gu.round_f16(wt), gu.round_f16(w2)
    kw = dict(stride=stride, pad=pad, scale=scale, shift=shift, act="leaky", residual=res, act2="none", res_mul=2.0, out_mul=0.5)
    ran = 0
    first = L.msnh_hip_conv2d_tail_tile_first()
    for tile in [0] + list(range(first, L.msnh_hip_conv2d_tile_count() + 1)):
        got = gu.conv2d_tail(x, wt, w2, **kw, scale2=scale2, shift2=shift2, act3="leaky", z_mul=2.0, write_y=write_y, tile=tile,
                             in_ld=c + 8, out_ld=oc + 8, res_ld=oc + 16 if with_res else None, z_ld=oc2 + 8)
        if got is None:
            continue
        ran += 1
        y, z = got
        y_ref = gu.round_f16(_ref(x, wt, stride, pad, 1, 1, scale, shift, "leaky", 0.1, res, "none", 2.0, 0.5))
        z_ref = _ref(y_ref, w2.reshape(oc2, oc, 1, 1), 1, 0, 1, 1, scale2, shift2, "leaky", 0.1, None, "none", 1.0, 2.0)
        if write_y:
            assert gu.rel_err(y, y_ref) <= TOL[abi.F16], tile
        assert gu.rel_err(z, z_ref) <= 2 * TOL[abi.F16], tile     # z sees y's own rounding differences as well
        # two launches of msnh_hip_conv2d: the same bits
        y2, _ = gu.conv2d(x, wt, dtype=abi.F16, **kw, algo="igemm", tile=37 if oc > 128 else 38, in_ld=c + 8, out_ld=oc + 8, res_ld=oc + 16 if with_res else None)
        z2, _ = gu.conv2d(y2, w2.reshape(oc2, oc, 1, 1), dtype=abi.F16, scale=scale2, shift=shift2, act="leaky", out_mul=2.0, algo="igemm", tile=38)
        if write_y:
            assert np.array_equal(y, y2), tile
        assert np.array_equal(z, z2), tile
    assert ran >= 1


def test_conv_tail_rejects():
    L = abi.lib()
    mk = lambda **kw: abi.ConvDesc(**{**dict(dtype=abi.F16, out_dtype=abi.F16, batch=1, in_h=8, in_w=8, in_c=64, in_ld=64, out_c=128, out_h=8, out_w=8, out_ld=128,
                                             ksize=3, stride=1, pad=1, dilation=1, groups=1, act=22, act_param=0.1, has_residual=0, res_ld=128, act2=22,
                                             act2_param=0.1, res_mul=1.0, out_mul=1.0, algo=abi.ALGO["igemm"], tile=0), **kw})
    tk = lambda **kw: abi.ConvTailDesc(**{**dict(out_c=64, out_ld=64, act=22, act_param=0.1, out_mul=1.0, write_y=1), **kw})
    ok = lambda d, t, tile=0: L.msnh_hip_conv2d_tail_supported(ctypes.byref(d), ctypes.byref(t), tile)
    assert ok(mk(), tk()) == 1
    assert ok(mk(out_c=512, out_ld=512, res_ld=512), tk()) == 0          # more channels than a tile holds
    assert ok(mk(), tk(out_c=256, out_ld=256)) == 0                      # more tail channels than the epilogue stages
    assert ok(mk(), tk(out_c=60, out_ld=64)) == 0
    assert ok(mk(groups=2), tk()) == 0
    assert ok(mk(dtype=abi.F32, out_dtype=abi.F32), tk()) == 0
    assert ok(mk(), tk(), 37) == 0                                       # a tile without a tail
    # ... and a tile with a tail does not run a plain convolution
    assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(mk()), L.msnh_hip_conv2d_tail_tile_first()) == 0
    assert L.msnh_hip_conv2d_tail(ctypes.byref(mk()), ctypes.byref(tk()), None, None, None, None, None, None, None, None, None, None, None) != 0


@pytest.mark.parametrize("dtype", [abi.F16, abi.F32])
@pytest.mark.parametrize("case", [(2, 64, 19, 19, 40, 1, 1, 0), (1, 32, 13, 11, 64, 3, 1, 1), (3, 128, 10, 10, 128, 1, 1, 0), (1, 64, 38, 38, 256, 3, 2, 1)])
def test_conv_upsampling_epilogue(case, dtype):
    """msnh_conv_desc::out_upsample = 2: the convolution writes every result pixel to the 2 x 2 pixels it maps to under nearest-neighbour
    upsampling (the convolution in front of an UpSampleLayer writes the upsampled tensor itself), on every tile of the implicit GEMM that
    takes the shape: equal to the oracle's convolution repeated 2 x 2, and bit for bit to the same tile without it followed by the repeat."""
    import gpuutil as gu
    L = abi.lib()
    b, c, h, w, oc, k, stride, pad = case
    rng = np.random.default_rng(hash(case) % (2 ** 31))
    x, wt = _case(rng, b, c, h, w, oc, k)
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    if dtype == abi.F16:
        x, wt = gu.round_f16(x), gu.round_f16(wt)
    ref = _ref(x, wt, stride, pad, 1, 1, scale, shift, "leaky", 0.1, None, "none", 1.0, 0.5)
    ref_up = ref.repeat(2, axis=2).repeat(2, axis=3)
    ran = 0
    for tile in range(0, L.msnh_hip_conv2d_tile_count() + 1):
        kw = dict(dtype=dtype, stride=stride, pad=pad, scale=scale, shift=shift, act="leaky", out_mul=0.5, algo="igemm", tile=tile, in_ld=c + 8, out_ld=oc + 8)
        try:
            y, _ = gu.conv2d(x, wt, **kw, upsample=2)
        except abi.HipError as e:
            assert "this tile needs" in str(e) or "upsampling epilogue" in str(e), str(e)
            continue
        ran += 1
        assert y.shape == ref_up.shape
        assert gu.rel_err(y, ref_up) <= TOL[dtype], tile
        plain, _ = gu.conv2d(x, wt, **kw)
        assert np.array_equal(y, plain.repeat(2, axis=2).repeat(2, axis=3)), tile
    assert ran >= 10
    # not for the other algorithms, not with a residual
    d = abi.ConvDesc(dtype, dtype, b, h, w, c, c, oc, (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1, oc, k, stride, pad, 1, 1, 22, 0.1, 0, oc, 22, 0.1,
                     1.0, 1.0, abi.ALGO["direct"], 0, 2)
    assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), 0) == 0
    d.algo = abi.ALGO["igemm"]
    assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), 0) == 1
    d.has_residual = 1
    assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), 0) == 0
