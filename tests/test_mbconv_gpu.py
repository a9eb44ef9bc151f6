"""GPU parity of msnh_hip_mbconv (1x1 expand, 3x3 depthwise, 1x1 project of an inverted-residual block as one launch) against the
three layers composed from the plain-C oracle convolution, with the two widened tensors rounded to float16 where the launch rounds them.

Tolerance: 1e-3 of max|ref| (measured 2-4e-4) -- half the single-layer float16 bar: a widened value that sits on a float16 rounding
boundary may round the other way on the device (float32 summation order), and the projection sums up to 576 of them."""
import ctypes

import numpy as np
import pytest

import msnh_oracle_net as on
from msnhnet_amd import hipabi as abi

pytestmark = pytest.mark.gpu


def _reference(x, we, wd, wp, s1, h1, s2, h2, s3, h3, stride, acts, mul1, mul2, out_mul, res, res_mul):
    import gpuutil as gu
    cexp, cout = we.shape[0], wp.shape[0]
    e = on.conv(x, we.reshape(cexp, -1, 1, 1), cexp, 1) * s1.reshape(1, -1, 1, 1) + h1.reshape(1, -1, 1, 1)
    e = gu.round_f16(np.float32(mul1) * on.activate(e.astype(np.float32), acts[0], 0.1))
    d = on.conv(e, wd.reshape(cexp, 1, 3, 3), cexp, 3, stride, 1, 1, cexp) * s2.reshape(1, -1, 1, 1) + h2.reshape(1, -1, 1, 1)
    d = gu.round_f16(np.float32(mul2) * on.activate(d.astype(np.float32), acts[1], 0.1))
    y = on.conv(d, wp.reshape(cout, cexp, 1, 1), cout, 1) * s3.reshape(1, -1, 1, 1) + h3.reshape(1, -1, 1, 1)
    y = on.activate(y.astype(np.float32), acts[2], 0.1)
    if res is not None:
        y = on.activate((y + np.float32(res_mul) * res).astype(np.float32), acts[3], 0.1)
    return (np.float32(out_mul) * y).astype(np.float32)


def run_mbconv(x, we, wd, wp, s1, h1, s2, h2, s3, h3, stride, acts, mul1, mul2, out_mul, res, res_mul, in_ld=None, out_ld=None, res_ld=None):
    import torch
    import gpuutil as gu
    gu.init()
    L = abi.lib()
    b, cin, h, w = x.shape
    cexp, cout = we.shape[0], wp.shape[0]
    oh, ow = (h - 1) // stride + 1, (w - 1) // stride + 1
    in_ld, out_ld, res_ld = in_ld or cin, out_ld or cout, res_ld or cout
    d = abi.MbconvDesc(b, h, w, cin, in_ld, cexp, stride, cout, oh, ow, out_ld, abi.ACT[acts[0]], abi.ACT[acts[1]], abi.ACT[acts[2]], abi.ACT[acts[3]],
                       0.1, 0.1, 0.1, 0.1, 1 if res is not None else 0, res_ld, mul1, mul2, out_mul, res_mul)
    assert L.msnh_hip_mbconv_supported(ctypes.byref(d)) == 1
    nbytes = L.msnh_hip_mbconv_packed_bytes(ctypes.byref(d))
    packed = np.zeros(nbytes, np.uint8)
    f = lambda a: np.ascontiguousarray(a, np.float32).ctypes.data_as(ctypes.c_void_p)
    keep = [np.ascontiguousarray(a, np.float32) for a in (we, s1, h1, wd, s2, h2, wp)]
    abi.check(L.msnh_hip_mbconv_pack(ctypes.byref(d), *[a.ctypes.data_as(ctypes.c_void_p) for a in keep], packed.ctypes.data_as(ctypes.c_void_p)))
    xd = gu.nhwc_dev(x, abi.F16, in_ld)
    pd = torch.from_numpy(packed).cuda()
    s3d, h3d = gu.dev(s3), gu.dev(h3)
    rd = gu.nhwc_dev(res, abi.F16, res_ld) if res is not None else None
    yd = torch.full((b, oh, ow, out_ld), 5.0, dtype=torch.float16).cuda()
    abi.check(L.msnh_hip_mbconv(ctypes.byref(d), gu.ptr(xd), gu.ptr(pd), gu.ptr(s3d), gu.ptr(h3d), gu.ptr(rd), gu.ptr(yd), None))
    gu.sync()
    if out_ld > cout:
        assert (yd[..., cout:] == 5.0).all().item(), "wrote past out_c"
    return gu.nchw_host(yd, cout)


CASES = [
    # b, cin, h, w, cexp, cout, stride, residual
    (2, 16, 28, 28, 96, 24, 2, False),      # MobileNetV2's first widening block (112x112 there)
    (2, 24, 28, 28, 144, 24, 1, True),      # K of 24 padded to 32, 144 = two chunks and a quarter
    (2, 24, 21, 28, 144, 32, 2, False),
    (3, 32, 14, 14, 192, 32, 1, True),
    (2, 32, 28, 28, 192, 64, 2, False),
    (4, 64, 14, 14, 384, 64, 1, True),
    (2, 64, 14, 14, 384, 96, 1, False),
    (2, 96, 14, 14, 576, 96, 1, True),
    (2, 96, 14, 14, 576, 96, 2, False),     # 160 output channels in the network: beyond the kernel; 96 here
    (1, 8, 10, 13, 40, 8, 1, True),         # image edges inside tiles, a partial chunk, a single channel vector
    (1, 40, 9, 5, 72, 48, 2, False),
]


@pytest.mark.parametrize("case", CASES)
def test_mbconv_block(case):
    import gpuutil as gu
    b, cin, h, w, cexp, cout, stride, with_res = case
    rng = np.random.default_rng(sum(case) + 11)
    x = gu.round_f16(rng.standard_normal((b, cin, h, w), dtype=np.float32))
    we = gu.round_f16(rng.standard_normal((cexp, cin), dtype=np.float32) * np.float32(np.sqrt(2.0 / cin)))
    wd = gu.round_f16(rng.standard_normal((cexp, 9), dtype=np.float32) * np.float32(np.sqrt(2.0 / 9)))
    wp = gu.round_f16(rng.standard_normal((cout, cexp), dtype=np.float32) * np.float32(np.sqrt(1.0 / cexp)))
    aff = lambda n: (rng.uniform(0.5, 1.5, n).astype(np.float32), (rng.standard_normal(n) * 0.2).astype(np.float32))
    (s1, h1), (s2, h2), (s3, h3) = aff(cexp), aff(cexp), aff(cout)
    mul1, mul2, out_mul, res_mul = 0.5, 0.25, 2.0, 0.5
    # the consumers undo the producers' power-of-two scales, as the planner folds them
    s2 = (s2 / np.float32(mul1)).astype(np.float32)
    s3 = (s3 / np.float32(mul2)).astype(np.float32)
    oh, ow = (h - 1) // stride + 1, (w - 1) // stride + 1
    res = gu.round_f16(rng.standard_normal((b, cout, oh, ow), dtype=np.float32)) if with_res else None
    acts = ("relu6", "relu6", "none", "none")
    print("mbconv", case, flush=True)
    args = (x, we, wd, wp, s1, h1, s2, h2, s3, h3, stride, acts, mul1, mul2, out_mul, res, res_mul)
    y = run_mbconv(*args, in_ld=cin + 8, out_ld=cout + 8, res_ld=cout + 16)
    ref = _reference(*args)
    e = gu.rel_err(y, ref)
    print("error", e, flush=True)
    assert e <= 1e-3
    assert np.array_equal(y, run_mbconv(*args, in_ld=cin + 8, out_ld=cout + 8, res_ld=cout + 16))


def test_mbconv_activations_and_limits():
    """other activations in each place (an activation whose value at zero is not zero must not leak into the depthwise padding), and
    the shapes the entry point refuses"""
    import gpuutil as gu
    gu.init()
    L = abi.lib()
    rng = np.random.default_rng(5)
    b, cin, h, w, cexp, cout = 2, 16, 9, 12, 80, 16
    x = gu.round_f16(rng.standard_normal((b, cin, h, w), dtype=np.float32))
    we = gu.round_f16(rng.standard_normal((cexp, cin), dtype=np.float32) * 0.3)
    wd = gu.round_f16(rng.standard_normal((cexp, 9), dtype=np.float32) * 0.4)
    wp = gu.round_f16(rng.standard_normal((cout, cexp), dtype=np.float32) * 0.1)
    one, zero = np.ones(cexp, np.float32), np.zeros(cexp, np.float32)
    s3, h3 = np.ones(cout, np.float32), (rng.standard_normal(cout) * 0.1).astype(np.float32)
    res = gu.round_f16(rng.standard_normal((b, cout, h, w), dtype=np.float32))
    for acts in (("logistic", "leaky", "none", "relu"), ("swish", "mish", "leaky", "none"), ("hardswish", "relu", "none", "leaky")):
        print("mbconv acts", acts, flush=True)
        args = (x, we, wd, wp, one, zero + 0.3, one, zero - 0.1, s3, h3, 1, acts, 1.0, 1.0, 1.0, res, 1.0)
        e = gu.rel_err(run_mbconv(*args), _reference(*args))
        print("error", e, flush=True)
        assert e <= 1e-3
    bad = [dict(in_c=104), dict(out_c=104), dict(in_c=12), dict(stride=3), dict(out_h=5), dict(in_ld=20)]
    for change in bad:
        d = abi.MbconvDesc(1, 14, 14, 32, 32, 192, 1, 32, 14, 14, 32, abi.ACT["relu6"], abi.ACT["relu6"], abi.ACT["none"], abi.ACT["none"],
                           0.1, 0.1, 0.1, 0.1, 0, 32, 1.0, 1.0, 1.0, 1.0)
        assert L.msnh_hip_mbconv_supported(ctypes.byref(d)) == 1
        for k, v in change.items():
            setattr(d, k, v)
        assert L.msnh_hip_mbconv_supported(ctypes.byref(d)) == 0, change
        assert L.msnh_hip_mbconv_packed_bytes(ctypes.byref(d)) == 0
        assert L.msnh_hip_mbconv(ctypes.byref(d), None, None, None, None, None, None, None) != 0
