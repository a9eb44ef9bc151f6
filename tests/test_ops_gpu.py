"""GPU parity of the bandwidth-bound entry points of the C ABI against the plain-C oracle."""
import ctypes

import numpy as np
import pytest
import torch

import msnh_oracle_net as on
from msnhnet_amd import hipabi as abi

pytestmark = pytest.mark.gpu

DTYPES = [abi.F32, abi.F16]
TOL = {abi.F32: 1e-6, abi.F16: 1.5e-3}


def _x(rng, shape, dtype):
    import gpuutil as gu
    x = rng.standard_normal(shape, dtype=np.float32) * 3
    return gu.round_f16(x) if dtype == abi.F16 else x


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("c,ld", [(16, 16), (24, 40), (13, 13), (255, 256)])
@pytest.mark.parametrize("act", ["relu", "leaky", "mish", "none"])
def test_affine_act(c, ld, act, dtype):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(c)
    x = _x(rng, (2, c, 7, 5), dtype)
    bn4 = np.concatenate([rng.uniform(.5, 1.5, c), rng.standard_normal(c) * .1, rng.standard_normal(c) * .1, rng.uniform(.5, 1.5, c)]).astype(np.float32)
    ref = on.batchnorm(x, bn4, 1e-5, act)
    sq = np.sqrt(bn4[3 * c:] + np.float32(1e-5)).astype(np.float32)
    scale = (bn4[:c] / sq).astype(np.float32)
    shift = (-bn4[:c] * bn4[2 * c:3 * c] / sq + bn4[c:2 * c]).astype(np.float32)
    xd = gu.nhwc_dev(x, dtype, ld)
    yd = torch.full((2, 7, 5, ld), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()
    sd, hd = gu.dev(scale), gu.dev(shift)
    gu.sync()
    abi.check(abi.lib().msnh_hip_affine_act(dtype, dtype, 2 * 7 * 5, c, gu.ptr(xd), ld, gu.ptr(sd), gu.ptr(hd), abi.ACT[act], 0.1, 1.0, gu.ptr(yd), ld, None))
    gu.sync()
    assert gu.rel_err(gu.nchw_host(yd, c), ref) <= max(TOL[dtype], 2e-6)
    assert (yd[..., c:].float().cpu().numpy() == 3.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("c", [32, 20])
def test_add_act_and_copy(c, dtype):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(c)
    a, b = _x(rng, (2, c, 6, 6), dtype), _x(rng, (2, c, 6, 6), dtype)
    ad, bd = gu.nhwc_dev(a, dtype, c + 8), gu.nhwc_dev(b, dtype, c)
    yd = torch.full((2, 6, 6, c + 16), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_add_act(dtype, 72, c, gu.ptr(ad), c + 8, 2.0, gu.ptr(bd), c, 0.5, abi.ACT["relu"], 0.1, 0.25, gu.ptr(yd), c + 16, None))
    gu.sync()
    ref = 0.25 * on.activate((2.0 * a + 0.5 * b).astype(np.float32), "relu")
    assert gu.rel_err(gu.nchw_host(yd, c), ref) <= TOL[dtype]
    # channel-slice copy into the middle of a wider tensor
    zd = torch.full((2, 6, 6, 2 * c + 8), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()
    gu.sync()
    off = 8
    abi.check(abi.lib().msnh_hip_copy_channels(dtype, 72, c, gu.ptr(ad), c + 8, 1.0, ctypes.c_void_p(zd.data_ptr() + off * zd.element_size()), 2 * c + 8, None))
    gu.sync()
    z = zd.float().cpu().numpy()
    assert np.array_equal(z[..., off:off + c].transpose(0, 3, 1, 2), a)
    assert (z[..., :off] == 3.0).all() and (z[..., off + c:] == 3.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("c,h,w,k,s,p", [(64, 28, 28, 3, 2, 1), (32, 19, 19, 5, 1, 2), (32, 19, 19, 9, 1, 4), (16, 19, 19, 13, 1, 6), (12, 10, 9, 2, 2, 0)])
def test_maxpool(c, h, w, k, s, p, dtype):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(k)
    x = _x(rng, (2, c, h, w), dtype)
    ref = on.maxpool(x, k, s, p)
    oh, ow = ref.shape[2:]
    xd = gu.nhwc_dev(x, dtype)
    yd = torch.zeros((2, oh, ow, c), dtype=gu.TORCH_DT[dtype]).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_maxpool(dtype, 2, h, w, c, gu.ptr(xd), c, k, s, p, oh, ow, gu.ptr(yd), c, None))
    gu.sync()
    assert np.array_equal(gu.nchw_host(yd, c), ref)          # max is exact


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h,w", [(19, 19), (7, 5), (2, 2)])
def test_maxpool_windows_compose(h, w, dtype):
    """stride 1, -FLT_MAX padding: the 9 and 13 windows equal a 5 window over the 5 and the 9 result bit for bit (what the
    plan relies on when it runs the pools of an SPP block as a chain)"""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(h * 31 + w)
    c = 24
    x = _x(rng, (2, c, h, w), dtype)
    xd = gu.nhwc_dev(x, dtype)
    out = {}
    for name, src, k in (("5", xd, 5), ("9", xd, 9), ("13", xd, 13)):
        out[name] = torch.zeros((2, h, w, c), dtype=gu.TORCH_DT[dtype]).cuda()
        abi.check(abi.lib().msnh_hip_maxpool(dtype, 2, h, w, c, gu.ptr(src), c, k, 1, k // 2, h, w, gu.ptr(out[name]), c, None))
    for name, src in (("5o5", out["5"]), ("5o9", out["9"])):
        out[name] = torch.zeros((2, h, w, c), dtype=gu.TORCH_DT[dtype]).cuda()
        gu.sync()
        abi.check(abi.lib().msnh_hip_maxpool(dtype, 2, h, w, c, gu.ptr(src), c, 5, 1, 2, h, w, gu.ptr(out[name]), c, None))
    gu.sync()
    assert np.array_equal(gu.nchw_host(out["13"], c), on.maxpool(x, 13, 1, 6))
    assert torch.equal(out["5o5"], out["9"]) and torch.equal(out["5o9"], out["13"])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h,w,c,k,steps", [(19, 19, 512, 5, 3), (13, 13, 72, 5, 3), (7, 5, 24, 5, 2), (16, 16, 256, 3, 3), (2, 2, 8, 5, 3)])
def test_maxpool_chain(h, w, c, k, steps, dtype):
    """the pools of an SPP block in one launch (msnh_hip_maxpool_chain): every pool's result equals the oracle's max-pool with the
    composed window (k, 2k-1, 3k-2) and the separate launches bit for bit, also into channel slices of a wider tensor (the concat
    the block writes), with NaN, infinities and a window that holds nothing usable in the input"""
    import ctypes
    import gpuutil as gu
    gu.init()
    L = abi.lib()
    assert L.msnh_hip_maxpool_chain_supported(dtype, h, w, c, k, steps) == 1
    rng = np.random.default_rng(h * 131 + c)
    batch = 3
    x = _x(rng, (batch, c, h, w), dtype)
    x[0, 0, 0, 0] = np.nan
    x[1, 1, :, :] = -np.inf                      # a channel without any value that compares greater than -FLT_MAX
    x[2, 2, h // 2, w // 2] = np.inf
    xd = gu.nhwc_dev(x, dtype)
    ld = (steps + 1) * c + 8
    cat = torch.full((batch, h, w, ld), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()          # [pool_steps .. pool_1, (x), 8 spare channels]
    es = 2 if dtype == abi.F16 else 4
    ys = (ctypes.c_void_p * steps)(*[cat.data_ptr() + (steps - 1 - i) * c * es for i in range(steps)])
    lds = (ctypes.c_int * steps)(*([ld] * steps))
    gu.sync()
    abi.check(L.msnh_hip_maxpool_chain(dtype, batch, h, w, c, k, steps, gu.ptr(xd), c, ys, lds, None))
    gu.sync()
    got = cat.cpu()
    assert (got[..., steps * c:] == 3.0).all(), "wrote outside its slices"
    src = xd
    for i in range(steps):
        sep = torch.zeros((batch, h, w, c), dtype=gu.TORCH_DT[dtype]).cuda()
        abi.check(L.msnh_hip_maxpool(dtype, batch, h, w, c, gu.ptr(src), c, k, 1, k // 2, h, w, gu.ptr(sep), c, None))
        gu.sync()
        mine = got[..., (steps - 1 - i) * c:(steps - i) * c]
        assert torch.equal(mine.contiguous().view(torch.int16 if dtype == abi.F16 else torch.int32),
                           sep.cpu().view(torch.int16 if dtype == abi.F16 else torch.int32)), f"pool {i} differs from the separate launch"
        kk = (i + 1) * (k - 1) + 1
        finite = np.isfinite(x).all(axis=(2, 3))          # (the oracle comparison on the channels without special values)
        want = on.maxpool(x, kk, 1, kk // 2)
        have = mine.float().numpy().transpose(0, 3, 1, 2)
        assert np.array_equal(have[finite], want[finite])
        src = sep
    # geometries it does not take are refused
    assert L.msnh_hip_maxpool_chain_supported(dtype, 76, 76, 256, 5, 3) == 0
    assert L.msnh_hip_maxpool_chain_supported(dtype, h, w, c, 7, 3) == 0


@pytest.mark.parametrize("dtype,out_dtype", [(abi.F32, abi.F32), (abi.F16, abi.F16), (abi.F16, abi.F32)])
@pytest.mark.parametrize("c,h,w,k,s,p", [(512, 7, 7, 7, 1, 0), (24, 9, 9, 3, 2, 1)])
def test_avgpool(c, h, w, k, s, p, dtype, out_dtype):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(k)
    x = _x(rng, (3, c, h, w), dtype)
    ref = on.avgpool(x, k, s, p)
    oh, ow = ref.shape[2:]
    xd = gu.nhwc_dev(x, dtype)
    yd = torch.zeros((3, oh, ow, c), dtype=gu.TORCH_DT[out_dtype]).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_avgpool(dtype, out_dtype, 3, h, w, c, gu.ptr(xd), c, k, s, p, oh, ow, 1.0, gu.ptr(yd), c, None))
    gu.sync()
    assert gu.rel_err(gu.nchw_host(yd, c), ref) <= (1e-6 if out_dtype == abi.F32 else 1e-3)


@pytest.mark.parametrize("dtype,out_dtype", [(abi.F32, abi.F32), (abi.F16, abi.F16), (abi.F16, abi.F32)])
@pytest.mark.parametrize("c,h,w", [(1280, 7, 7), (20, 5, 7), (7, 3, 3), (2048, 1, 1), (264, 19, 17)])
def test_avgpool_whole_image(c, h, w, dtype, out_dtype):
    """one window over the whole image (classifier heads, globalavgpool): the mean of every channel"""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(c + h)
    x = _x(rng, (3, c, h, w), dtype)
    ref = x.astype(np.float64).mean(axis=(2, 3), keepdims=True)
    xd = gu.nhwc_dev(x, dtype)
    yd = torch.zeros((3, 1, 1, c), dtype=gu.TORCH_DT[out_dtype]).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_avgpool(dtype, out_dtype, 3, h, w, c, gu.ptr(xd), c, max(h, w), 1, 0, 1, 1, 1.0, gu.ptr(yd), c, None))
    gu.sync()
    assert gu.rel_err(gu.nchw_host(yd, c), ref) <= (1e-6 if out_dtype == abi.F32 else 1e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_upsample(dtype):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(1)
    x = _x(rng, (2, 24, 5, 7), dtype)
    ref = on.upsample(x, 2)
    xd = gu.nhwc_dev(x, dtype)
    yd = torch.full((2, 10, 14, 40), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_upsample_nearest(dtype, 2, 5, 7, 24, gu.ptr(xd), 24, 2, 1.0, gu.ptr(yd), 40, None))
    gu.sync()
    assert np.array_equal(gu.nchw_host(yd, 24), ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("c", [24, 5])
def test_pad(dtype, c):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(3)
    x = _x(rng, (2, c, 5, 7), dtype)
    ref = on.pad(x, 1, 2, 0, 3, -1.5)
    ld = (c + 7) // 8 * 8
    xd = gu.nhwc_dev(x, dtype, ld)
    yd = torch.full((2, 8, 10, ld + 8), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_pad(dtype, 2, 5, 7, c, gu.ptr(xd), ld, 1, 0, 8, 10, 1.0, -1.5, gu.ptr(yd), ld + 8, None))
    gu.sync()
    assert np.array_equal(gu.nchw_host(yd, c), ref)
    assert (yd[..., c:].float().cpu().numpy() == 3.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_slice(dtype):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(4)
    x = _x(rng, (2, 10, 9, 11), dtype)
    for args in ((0, 1, 0, 2, 1, 2), (1, 3, 1, 1, 2, 3), (9, 1, 8, 5, 0, 11)):
        ref = on.slice_(x, *args)
        oc, oh, ow = ref.shape[1:]
        xd = gu.nhwc_dev(x, dtype, 16)
        yd = torch.full((2, oh, ow, 16), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()
        gu.sync()
        abi.check(abi.lib().msnh_hip_slice(dtype, 2, 9, 11, gu.ptr(xd), 16, *args, oc, oh, ow, 1.0, gu.ptr(yd), 16, None))
        gu.sync()
        assert np.array_equal(gu.nchw_host(yd, oc), ref)
        assert (yd[..., oc:].float().cpu().numpy() == 3.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("oh,ow,align", [(10, 14, 0), (12, 9, 1), (3, 4, 0), (5, 7, 1)])
def test_upsample_bilinear(dtype, oh, ow, align):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(5)
    x = _x(rng, (2, 24, 5, 7), dtype)
    ref = on.bilinear(x, oh, ow, align)
    xd = gu.nhwc_dev(x, dtype)
    yd = torch.full((2, oh, ow, 32), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_upsample_bilinear(dtype, 2, 5, 7, 24, gu.ptr(xd), 24, oh, ow, align, 1.0, gu.ptr(yd), 32, None))
    gu.sync()
    # same float32 expression; the compiler may contract its multiply-adds
    assert gu.rel_err(gu.nchw_host(yd, 24), ref) <= (2e-6 if dtype == abi.F32 else 1e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("c,h,w,temp", [(1000, 1, 1, 1.0), (2, 9, 11, 2.0), (21, 4, 4, 0.5)])
def test_softmax(dtype, c, h, w, temp):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(6)
    x = _x(rng, (3, c, h, w), dtype) * 4
    if dtype == abi.F16:
        x = gu.round_f16(x)
    ref = on.softmax(x, temp)
    ld = (c + 7) // 8 * 8
    xd = gu.nhwc_dev(x, dtype, ld)
    yd = torch.zeros((3, h, w, ld), dtype=gu.TORCH_DT[dtype]).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_softmax(dtype, 3, h * w, c, gu.ptr(xd), ld, 1.0, temp, gu.ptr(yd), ld, 1.0, None))
    gu.sync()
    got = gu.nchw_host(yd, c)
    assert gu.rel_err(got, ref) <= (1e-5 if dtype == abi.F32 else 2e-3)
    assert np.allclose(got.reshape(3, -1).sum(1), 1.0, atol=1e-5 if dtype == abi.F32 else 5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("c,oc,h,w,k,s,p,bias", [(16, 8, 5, 7, 2, 2, 0, True), (8, 5, 6, 5, 3, 2, 1, True), (16, 8, 4, 6, 4, 2, 1, False), (8, 16, 3, 3, 3, 1, 1, True)])
def test_deconv(dtype, c, oc, h, w, k, s, p, bias):
    """Transposed convolution = 1x1 convolution to k*k*oc channels + msnh_hip_deconv_col2im, against the oracle's GEMM + col2im."""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(k * 10 + s)
    x = _x(rng, (2, c, h, w), dtype)
    wt = (rng.standard_normal((c, oc, k, k)) * 0.2).astype(np.float32)
    b = (rng.standard_normal(oc) * 0.1).astype(np.float32) if bias else None
    if dtype == abi.F16:
        x, wt = gu.round_f16(x), gu.round_f16(wt)
    ref = on.deconv(x, wt.ravel(), oc, k, s, p, b, "leaky", 0.1)
    oh, ow = ref.shape[2:]
    # first half: [k*k*oc][c] weights as a 1x1 convolution
    w1 = np.ascontiguousarray(wt.transpose(2, 3, 1, 0).reshape(k * k * oc, c, 1, 1))
    cols, _ = gu.conv2d(x, w1, dtype=dtype, algo="auto")                    # NCHW float32 [2][k*k*oc][h][w]
    cd = gu.nhwc_dev(cols, dtype)
    yd = torch.full((2, oh, ow, oc + 8), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()
    bd = gu.dev(b) if bias else None
    gu.sync()
    abi.check(abi.lib().msnh_hip_deconv_col2im(dtype, 2, h, w, oc, k, s, p, gu.ptr(cd), k * k * oc, 1.0, gu.ptr(bd) if bias else None, abi.ACT["leaky"], 0.1,
                                               oh, ow, 1.0, gu.ptr(yd), oc + 8, None))
    gu.sync()
    assert gu.rel_err(gu.nchw_host(yd, oc), ref) <= (1e-5 if dtype == abi.F32 else 4e-3)
    assert (yd[..., oc:].float().cpu().numpy() == 3.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_connected(dtype):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(2)
    x = _x(rng, (3, 512, 1, 1), dtype)
    w = rng.uniform(-0.05, 0.05, (1000, 512)).astype(np.float32)
    if dtype == abi.F16:
        w = gu.round_f16(w)
    bias = rng.uniform(-0.05, 0.05, 1000).astype(np.float32)
    ref = on.connected(x, w, bias, 1000).reshape(3, 1000)
    xd, wd, bd = gu.dev(x.reshape(3, 512), dtype), gu.dev(w, dtype), gu.dev(bias)
    yd = torch.zeros((3, 1000), dtype=torch.float32).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_connected(dtype, 3, 512, 1000, gu.ptr(xd), 1.0, gu.ptr(wd), gu.ptr(bd), abi.ACT["none"], 0.1, gu.ptr(yd), None))
    gu.sync()
    assert gu.rel_err(yd.cpu().numpy(), ref) <= 2e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch,inputs,outputs,act", [(32, 2048, 1000, "none"), (64, 1280, 1000, "relu"), (9, 64, 24, "leaky")])
def test_connected_batched(dtype, batch, inputs, outputs, act):
    """with a real batch the fully connected layer runs as the 1x1 case of the MFMA implicit GEMM"""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(batch)
    x = _x(rng, (batch, inputs, 1, 1), dtype)
    w = rng.uniform(-0.05, 0.05, (outputs, inputs)).astype(np.float32)
    if dtype == abi.F16:
        w = gu.round_f16(w)
    bias = rng.uniform(-0.05, 0.05, outputs).astype(np.float32)
    ref = on.connected(x, w, bias, outputs, act=act).reshape(batch, outputs)
    xd, wd, bd = gu.dev(x.reshape(batch, inputs), dtype), gu.dev(w, dtype), gu.dev(bias)
    yd = torch.zeros((batch, outputs), dtype=torch.float32).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_connected(dtype, batch, inputs, outputs, gu.ptr(xd), 1.0, gu.ptr(wd), gu.ptr(bd), abi.ACT[act], 0.1, gu.ptr(yd), None))
    gu.sync()
    assert gu.rel_err(yd.cpu().numpy(), ref) <= 5e-6


@pytest.mark.parametrize("dtype", DTYPES)
def test_layout_roundtrip(dtype):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(3)
    x = _x(rng, (2, 37, 9, 11), dtype)
    xd = gu.dev(x)
    yd = torch.full((2, 9, 11, 40), 3.0, dtype=gu.TORCH_DT[dtype]).cuda()
    zd = torch.zeros((2, 37, 9, 11), dtype=torch.float32).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_nchw_to_nhwc(dtype, 2, 37, 9, 11, gu.ptr(xd), 1.0, gu.ptr(yd), 40, None))
    abi.check(abi.lib().msnh_hip_nhwc_to_nchw(dtype, 2, 37, 9, 11, gu.ptr(yd), 40, 1.0, gu.ptr(zd), None))
    gu.sync()
    assert np.array_equal(gu.nchw_host(yd, 37), x)
    assert np.array_equal(zd.cpu().numpy(), x)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("version", [3, 5])
def test_yolo_decode(dtype, version):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(4)
    cls, h, w = 80, 7, 9
    per = 5 + cls
    x = (rng.standard_normal((2, 3 * per, h, w)) * 4).astype(np.float32)
    x[0, 2, 0, 0] = 100.0          # exp overflow -> inf, as with the benchmark weights
    x[1, 4, 3, 3] = -200.0
    if dtype == abi.F16:
        x = gu.round_f16(x)
    anchors = np.array([10, 13, 16, 30, 33, 23], np.float32)
    ratio = 32.0
    ref = on.yolo_decode(x, cls, anchors, ratio, version)              # [2][3*per][h][w]
    ref_shuf = ref.reshape(2, 3, per, h * w).transpose(0, 1, 3, 2)    # [2][3][hw][per]
    xd = gu.nhwc_dev(x, dtype, 256)
    dd = torch.zeros((2, 3, h * w, per), dtype=torch.float32).cuda()
    cap = 3 * h * w
    ci = torch.full((2, cap), -1, dtype=torch.int32).cuda()
    cc = torch.zeros(2, dtype=torch.int32).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_yolo_decode(dtype, 2, h, w, cls, gu.ptr(xd), 256, 1.0, anchors.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                             ratio, version, gu.ptr(dd), 3 * h * w * per, 0.5, gu.ptr(ci), cap, 1000, gu.ptr(cc), None))
    gu.sync()
    out = dd.cpu().numpy()
    assert gu.rel_err(out, ref_shuf) <= 2e-6
    for b in range(2):
        want = sorted(1000 + a * h * w + p for a in range(3) for p in range(h * w) if ref_shuf[b, a, p, 4] > 0.5)
        n = int(cc[b])
        assert sorted(ci[b, :n].cpu().numpy().tolist()) == want
    # candidate-only decode: the same list, the candidates' rows bit for bit, every other row untouched
    dd2 = torch.full((2, 3, h * w, per), -7.0, dtype=torch.float32).cuda()
    ci3 = torch.full((2, cap), -1, dtype=torch.int32).cuda()
    cc3 = torch.zeros(2, dtype=torch.int32).cuda()
    rows3 = torch.zeros((2, cap, 8), dtype=torch.float32).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_yolo_decode_candidates(dtype, 2, h, w, cls, gu.ptr(xd), 256, 1.0, anchors.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                                        ratio, version, gu.ptr(dd2), 3 * h * w * per, 0.5, gu.ptr(ci3), cap, 1000, gu.ptr(cc3), gu.ptr(rows3), None))
    gu.sync()
    out2 = dd2.cpu().numpy().reshape(2, 3 * h * w, per)
    full = out.reshape(2, 3 * h * w, per)
    for b in range(2):
        n = int(cc3[b])
        got = sorted(ci3[b, :n].cpu().numpy().tolist())
        assert got == sorted(ci[b, :int(cc[b])].cpu().numpy().tolist())
        rows_in = np.zeros(3 * h * w, bool)
        rows_in[np.array(got, np.int64) - 1000] = True
        assert np.array_equal(out2[b][rows_in], full[b][rows_in])
        assert (out2[b][~rows_in] == -7.0).all()
        # ... and its compact rows are what the gather kernel derives from the decoded rows
        r3 = rows3[b, :n].cpu().numpy()
        cells = ci3[b, :n].cpu().numpy() - 1000
        assert np.array_equal(r3[:, :5], full[b][cells][:, :5])
        assert np.array_equal(r3[:, 5], full[b][cells][:, 5:].max(1)) and np.array_equal(r3[:, 6], full[b][cells][:, 5:].argmax(1).astype(np.float32))
        assert np.array_equal(r3[:, 7], (cells + 1000).astype(np.float32))
    # ... and without a decoded buffer the same compact rows are all it writes
    ci4 = torch.full((2, cap), -1, dtype=torch.int32).cuda()
    cc4 = torch.zeros(2, dtype=torch.int32).cuda()
    rows4 = torch.zeros((2, cap, 8), dtype=torch.float32).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_yolo_decode_candidates(dtype, 2, h, w, cls, gu.ptr(xd), 256, 1.0, anchors.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                                        ratio, version, None, 3 * h * w * per, 0.5, gu.ptr(ci4), cap, 1000, gu.ptr(cc4), gu.ptr(rows4), None))
    gu.sync()
    for b in range(2):
        n = int(cc4[b])
        assert n == int(cc3[b])
        a4 = rows4[b, :n].cpu().numpy(); a3 = rows3[b, :n].cpu().numpy()
        assert np.array_equal(a4[np.argsort(a4[:, 7])], a3[np.argsort(a3[:, 7])], equal_nan=True)
    # candidate compaction: box, objectness, first-maximum class
    ci2 = (ci - 1000).clamp(min=0).contiguous()
    rows = torch.zeros((2, cap, 8), dtype=torch.float32).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_yolo_gather(2, cls, gu.ptr(dd), 3 * h * w * per, gu.ptr(ci2), cap, gu.ptr(cc), gu.ptr(rows), None))
    gu.sync()
    rows = rows.cpu().numpy()
    flat = ref_shuf.reshape(2, 3 * h * w, per)
    for b in range(2):
        for k in range(int(cc[b])):
            cell = int(rows[b, k, 7])
            r = flat[b, cell]
            assert gu.rel_err(rows[b, k, :5], r[:5]) <= 2e-6
            assert int(rows[b, k, 6]) == int(np.argmax(r[5:]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("version", [3, 5])
@pytest.mark.parametrize("keep_decoded,cls", [(False, 20), (True, 20), (True, 130)])
def test_yolo_decode_candidates_all_heads(dtype, version, keep_decoded, cls):
    """one call over all heads of a network gives the candidate list (as a set), the compact rows and -- when asked for -- the
    decoded rows that one msnh_hip_yolo_decode_candidates call per head gives, bit for bit; checked for three heads of different
    sizes (one of them with more cells than a workgroup scans, one with none above the threshold) and a list shorter than the
    number of candidates"""
    import gpuutil as gu
    gu.init()
    L = abi.lib()
    rng = np.random.default_rng(14)
    per = 5 + cls
    ld = (3 * per + 7) // 8 * 8
    shapes = [(3, 4), (6, 8), (13, 11)]
    anchors = [np.array([116, 90, 156, 198, 373, 326], np.float32), np.array([30, 61, 62, 45, 59, 119], np.float32), np.array([10, 13, 16, 30, 33, 23], np.float32)]
    ratios = [32.0, 16.0, 8.0]
    batch = 3
    xs = []
    for i, (h, w) in enumerate(shapes):
        x = (rng.standard_normal((batch, 3 * per, h, w)) * 3).astype(np.float32)
        if i == 1:
            x[:, 4::per] = -9.0                  # this head has no candidate at all
        if dtype == abi.F16:
            x = gu.round_f16(x)
        xs.append(gu.nhwc_dev(x, dtype, ld))
    cells = sum(3 * h * w for h, w in shapes)
    fp = ctypes.POINTER(ctypes.c_float)
    for cap in (cells, 40):
        def buffers():
            return (torch.full((batch, cap), -1, dtype=torch.int32).cuda(), torch.zeros(batch, dtype=torch.int32).cuda(),
                    torch.zeros((batch, cap, 8), dtype=torch.float32).cuda(), torch.full((batch, cells, per), -7.0, dtype=torch.float32).cuda())
        ci1, cc1, rows1, dec1 = buffers()
        ci2, cc2, rows2, dec2 = buffers()
        gu.sync()
        base = 0
        for i, (h, w) in enumerate(shapes):
            abi.check(L.msnh_hip_yolo_decode_candidates(dtype, batch, h, w, cls, gu.ptr(xs[i]), ld, 0.5, anchors[i].ctypes.data_as(fp), ratios[i], version,
                                                        ctypes.c_void_p(dec1.data_ptr() + base * per * 4) if keep_decoded else None, cells * per, 0.6, gu.ptr(ci1), cap, base,
                                                        gu.ptr(cc1), gu.ptr(rows1), None))
            base += 3 * h * w
        heads = (abi.YoloHead * 3)()
        base = 0
        for i, (h, w) in enumerate(shapes):
            heads[i].x = xs[i].data_ptr(); heads[i].x_ld = ld; heads[i].x_mul = 0.5; heads[i].h = h; heads[i].w = w
            for k in range(6):
                heads[i].anchors[k] = float(anchors[i][k])
            heads[i].ratio = ratios[i]; heads[i].cand_base = base
            base += 3 * h * w
        abi.check(L.msnh_hip_yolo_decode_candidates_heads(dtype, batch, cls, 3, heads, version, gu.ptr(dec2) if keep_decoded else None, cells * per, 0.6,
                                                          gu.ptr(ci2), cap, gu.ptr(cc2), gu.ptr(rows2), None))
        gu.sync()
        assert np.array_equal(cc1.cpu().numpy(), cc2.cpu().numpy())
        assert int(cc1.max()) > 40 and int(cc1.min()) > 0
        if cap == cells:
            for b in range(batch):
                n = int(cc1[b])
                assert sorted(ci1[b, :n].cpu().numpy().tolist()) == sorted(ci2[b, :n].cpu().numpy().tolist())
                a1 = rows1[b, :n].cpu().numpy(); a2 = rows2[b, :n].cpu().numpy()
                assert np.array_equal(a1[np.argsort(a1[:, 7])], a2[np.argsort(a2[:, 7])], equal_nan=True)
                assert np.array_equal(ci2[b, :n].cpu().numpy().astype(np.float32), a2[:, 7])
            assert np.array_equal(dec1.cpu().numpy(), dec2.cpu().numpy(), equal_nan=True)
            assert keep_decoded == bool((dec2.cpu().numpy() != -7.0).any())
        else:
            # a list that is too short holds some `cap` of the candidates (which ones depends on timing in both paths): every
            # entry must be a real candidate with its own row
            full_idx, full_rows = want_full
            for b in range(batch):
                got = ci2[b].cpu().numpy()
                assert len(set(got.tolist())) == cap and set(got.tolist()) <= set(full_idx[b].tolist())
                r = rows2[b].cpu().numpy()
                lookup = {int(c): full_rows[b][k] for k, c in enumerate(full_idx[b])}
                for k in range(cap):
                    assert np.array_equal(r[k], lookup[int(got[k])], equal_nan=True)
        if cap == cells:
            want_full = ([ci2[b, :int(cc2[b])].cpu().numpy() for b in range(batch)], [rows2[b, :int(cc2[b])].cpu().numpy() for b in range(batch)])
    bad = (abi.YoloHead * 2)()
    for i in range(2):
        bad[i].x = xs[i].data_ptr(); bad[i].x_ld = ld; bad[i].x_mul = 1.0; bad[i].h, bad[i].w = shapes[i]; bad[i].ratio = 8.0; bad[i].cand_base = 5 * i
    ci2, cc2, rows2, dec2 = buffers()
    assert L.msnh_hip_yolo_decode_candidates_heads(dtype, batch, cls, 2, bad, version, None, cells * per, 0.6, gu.ptr(ci2), cap, gu.ptr(cc2), gu.ptr(rows2), None) != 0
    assert L.msnh_hip_yolo_decode_candidates_heads(dtype, batch, cls, 5, bad, version, None, cells * per, 0.6, gu.ptr(ci2), cap, gu.ptr(cc2), gu.ptr(rows2), None) != 0


def _ordered_records(kept, total, image):
    rec = kept[:total]
    rec = rec[rec[:, 11] == image]
    order = sorted(range(len(rec)), key=lambda i: (-rec[i, 8], rec[i, 9], rec[i, 10]))
    return rec[order]


def test_yolo_nms():
    """device NMS records, put in the documented order, are the reference procedure's boxes bit for bit: objectness and
    class scores on a coarse grid (many exact ties in both sort keys), heavy overlap, boxes of infinite extent (NaN IoU
    never suppresses), an empty image, a sparse image, and an image with 1200 / 6100 members in one class (the large-class
    kernel, which needs the workspace); an image with more members than that, an image with a NaN score -- and without a
    workspace every image with more than 1024 members in a class -- are flagged instead"""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(21)
    cls, h, w = 6, 48, 48
    per, hw = 5 + cls, 48 * 48
    cells = 3 * hw                     # 6912
    conf_t, nms_t = 0.5, 0.45
    heads = []
    for b in range(7):
        d = np.zeros((3 * per, h, w), np.float32)
        v = d.reshape(3, per, hw)
        v[:, 0] = rng.uniform(0, 400, (3, hw)); v[:, 1] = rng.uniform(0, 400, (3, hw))
        v[:, 2] = rng.uniform(10, 70, (3, hw)); v[:, 3] = rng.uniform(10, 70, (3, hw))
        v[:, 4] = rng.integers(0, 17, (3, hw)) / 16.0
        v[:, 5:] = rng.integers(0, 9, (3, cls, hw)) / 8.0
        if b == 0:
            v[1, 2, 5:9] = np.inf
        if b in (1, 5, 6):             # one class holds 1200 / 6100 / 6912 candidates, the other classes a few
            keep = {1: 1200, 5: 6100, 6: cells}[b]
            v[:, 5] = 2.0
            obj = np.zeros(cells, np.float32)
            obj[rng.permutation(cells)[:keep]] = rng.integers(9, 17, keep) / 16.0
            v[:, 4] = obj.reshape(3, hw)
            v[0, 5, :7] = 0.0; v[0, 6, :7] = 3.0
        if b == 2:
            v[:, 4] = 0.0              # no candidate at all
        if b == 4:
            v[:, 4] = np.where(rng.uniform(size=(3, hw)) < 0.01, 0.8, 0.1)    # a sparse image, like real detections
        heads.append(d)
    rows = np.zeros((7, cells, 8), np.float32)
    cnt = np.zeros(7, np.int32)
    for b, d in enumerate(heads):
        flat = d.reshape(3, per, hw).transpose(0, 2, 1).reshape(cells, per)
        cand = np.nonzero(flat[:, 4] > conf_t)[0]
        rng.shuffle(cand)
        cnt[b] = len(cand)
        r = rows[b, :len(cand)]
        r[:, :5] = flat[cand, :5]
        r[:, 5] = flat[cand, 5:].max(1); r[:, 6] = flat[cand, 5:].argmax(1); r[:, 7] = cand
    rows[3, 7, 5] = np.nan             # image 3: a NaN class score
    rd, cd = gu.dev(rows), gu.dev(cnt)
    nbytes = abi.lib().msnh_hip_yolo_nms_workspace_bytes(7, cls, cells)
    # the larger workspace (pair tests of the large classes as a bit matrix over the whole device), whole and with a pool that only
    # takes the 1200-member class, so that the 6100-member one stays with its own workgroup
    pbytes = abi.lib().msnh_hip_yolo_nms_pair_workspace_bytes(7, cls, cells)
    pool = min(7 * cells * 98 * 8, 64 << 20)
    assert pbytes > nbytes + pool
    ws = torch.full((pbytes // 4 + 4,), 0x55555555, dtype=torch.int32).cuda()
    print("yolo_nms", cnt.tolist(), flush=True)
    for ws_bytes, flags in ((nbytes, [0, 0, 0, 2, 0, 0, 1]), (0, [0, 1, 0, 2, 0, 1, 1]), (pbytes, [0, 0, 0, 2, 0, 0, 1]),
                            (pbytes - pool + (5 << 18), [0, 0, 0, 2, 0, 0, 1])):
        with_ws = ws_bytes > 0
        ws.fill_(0x55555555)
        keptd = torch.zeros((7 * cells, 12), dtype=torch.float32).cuda()
        kcd = torch.zeros(8, dtype=torch.int32).cuda()
        gu.sync()
        print("yolo_nms workspace", ws_bytes, flush=True)
        abi.check(abi.lib().msnh_hip_yolo_nms(7, cls, gu.ptr(rd), cells, gu.ptr(cd), nms_t, gu.ptr(keptd), 7 * cells, gu.ptr(kcd),
                                              gu.ptr(ws) if with_ws else None, ws_bytes, None))
        gu.sync()
        kc = kcd.cpu().numpy()
        kept = keptd.cpu().numpy()
        assert kc[1:].tolist() == flags, kc
        total = int(kc[0])
        for b in range(7):
            if flags[b]:
                continue
            want = on.yolo_out([heads[b]], cls, conf_t, nms_t)
            got = _ordered_records(kept, total, b)
            assert len(want) == len(got), (b, len(want), len(got))
            assert np.array_equal(got[:, :7], want, equal_nan=True), b
            assert (b == 2) == (len(got) == 0)
    assert len(on.yolo_out([heads[0]], cls, conf_t, nms_t)) > 100
    with pytest.raises(abi.HipError):
        abi.check(abi.lib().msnh_hip_yolo_nms(5, cls, gu.ptr(rd), cells, gu.ptr(cd), nms_t, None, 7 * cells, gu.ptr(kcd), None, 0, None))


@pytest.mark.parametrize("dtype", DTYPES)
def test_absmax(dtype):
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(5)
    x = _x(rng, (2, 24, 9, 9), dtype)
    x[1, 3, 2, 2] = np.inf if dtype == abi.F32 else 65504.0 * 4      # non-finite entries are ignored
    xd = gu.nhwc_dev(x, dtype, 32, fill=1e4)                          # the padding channels must not be read
    r = torch.zeros(1, dtype=torch.float32).cuda()
    gu.sync()
    abi.check(abi.lib().msnh_hip_absmax(dtype, 2 * 81, 24, gu.ptr(xd), 32, gu.ptr(r), None))
    gu.sync()
    xf = xd[..., :24].float().cpu().numpy()
    assert float(r) == float(np.abs(xf[np.isfinite(xf)]).max())


@pytest.mark.parametrize("h,w,nw,nh", [(480, 640, 608, 608), (640, 480, 416, 416), (300, 300, 608, 608), (100, 37, 64, 64),
                                       (608, 608, 608, 608), (50, 80, 224, 224), (33, 33, 32, 32), (720, 1280, 608, 608)])
def test_letterbox_u8(h, w, nw, nh):
    """device letterbox == the restatement of CVUtil::getPaddingZeroF32C3, bit for bit (no fused multiply-add in either)"""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(h + 3 * w)
    img = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
    src = torch.from_numpy(img).cuda()
    for half in (0, 1):
        for shuffle in (0, 1):
            dst = torch.full((3, nh, nw), -5.0, dtype=torch.float32).cuda()
            gu.sync()
            abi.check(abi.lib().msnh_hip_letterbox_u8(gu.ptr(src), w, h, nw, nh, half, shuffle, gu.ptr(dst), None))
            gu.sync()
            assert np.array_equal(dst.cpu().numpy(), on.letterbox_u8(img, nw, nh, bool(half), bool(shuffle)))
    assert abi.lib().msnh_hip_letterbox_u8(gu.ptr(src), w, h, 0, nh, 0, 0, gu.ptr(dst), None) != 0
    assert b"letterbox" in abi.lib().msnh_hip_last_error()


@pytest.mark.parametrize("h,w,nw,nh", [(480, 640, 224, 224), (50, 80, 64, 48), (33, 33, 32, 32), (224, 224, 224, 224), (20, 33, 96, 96)])
def test_image_u8_to_input(h, w, nw, nh):
    """device resize + normalisation == the restatement of the reference's CVUtil variants, bit for bit (no fused multiply-add in either)"""
    import gpuutil as gu
    gu.init()
    rng = np.random.default_rng(h + 5 * w)
    img = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
    src = torch.from_numpy(img).cuda()
    mean, std = np.array([0.4, 0.5, 0.6], np.float32), np.array([0.2, 0.3, 0.25], np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    kinds = {"f32c3": 0, "f32c3_half": 1, "googlenet": 2, "transformed": 3, "caffe": 4}
    for kind, code in kinds.items():
        for shuffle in (0, 1):
            dst = torch.full((3, nh, nw), -5.0, dtype=torch.float32).cuda()
            gu.sync()
            abi.check(abi.lib().msnh_hip_image_u8_to_input(gu.ptr(src), w, h, nw, nh, code, mean.ctypes.data_as(fp), std.ctypes.data_as(fp), shuffle, gu.ptr(dst), None))
            gu.sync()
            assert np.array_equal(dst.cpu().numpy(), on.preproc_u8(img, nw, nh, kind, mean, std, bool(shuffle))), (kind, shuffle)
    for code, half in ((5, False), (6, True)):
        dst = torch.full((3, nh, nw), -5.0, dtype=torch.float32).cuda()
        gu.sync()
        abi.check(abi.lib().msnh_hip_image_u8_to_input(gu.ptr(src), w, h, nw, nh, code, None, None, 0, gu.ptr(dst), None))
        gu.sync()
        assert np.array_equal(dst.cpu().numpy(), on.letterbox_u8(img, nw, nh, half, False))
    assert abi.lib().msnh_hip_image_u8_to_input(gu.ptr(src), w, h, nw, nh, 3, None, None, 0, gu.ptr(dst), None) != 0
    assert b"mean or std" in abi.lib().msnh_hip_last_error()
    assert abi.lib().msnh_hip_image_u8_to_input(gu.ptr(src), w, h, nw, nh, 9, None, None, 0, gu.ptr(dst), None) != 0


def test_mfma_probe():
    """the matrix-core ceiling probe reports a rate below the data-sheet peak and above half of it, a plausible shader clock, and
    refuses nonsense arguments"""
    import gpuutil as gu
    gu.init()
    L = abi.lib()
    tf, mhz, sec = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
    abi.check(L.msnh_hip_mfma_probe(3, 4000, ctypes.byref(tf), ctypes.byref(mhz), ctypes.byref(sec), None))
    print(f"mfma probe: {tf.value:.0f} TFLOP/s at {mhz.value:.0f} MHz in {sec.value * 1e3:.3f} ms", flush=True)
    assert 1000.0 < tf.value < 2600.0
    assert 800.0 < mhz.value < 2600.0
    assert 0.0 < sec.value < 0.1
    # the rate follows from the clock: 256 CUs x 4 SIMDs x 1024 FLOP per clock, within what a short run's ramp allows
    assert 0.6 < tf.value / (mhz.value * 1e6 * 256 * 4 * 1024 / 1e12) < 1.05
    assert L.msnh_hip_mfma_probe(0, 100, ctypes.byref(tf), ctypes.byref(mhz), ctypes.byref(sec), None) != 0
    assert L.msnh_hip_mfma_probe(3, 0, ctypes.byref(tf), ctypes.byref(mhz), ctypes.byref(sec), None) != 0
    assert L.msnh_hip_mfma_probe(3, 100, None, ctypes.byref(mhz), ctypes.byref(sec), None) != 0


@pytest.mark.parametrize("tile", [46, 52])
def test_timing_diagnostics_patch_kernel(tile):
    """the timing diagnostics library: with every switch off, and with only the clock read-out on, its instantiation of the LDS-patch
    kernel returns bit for bit what the kernel library returns for the same tile; the clock read-out gives a plausible shader
    clock; every listed switch combination launches and finishes; combinations that are not instantiated and bad shapes are refused"""
    import gpuutil as gu
    import torch
    from msnhnet_amd import diag
    gu.init()
    L, D = abi.lib(), diag.lib()
    b, c, h, w, oc = 2, 128, 38, 38, 128
    rng = np.random.default_rng(tile)
    x = gu.round_f16(rng.standard_normal((b, c, h, w), dtype=np.float32))
    wt = gu.round_f16(rng.standard_normal((oc, c, 3, 3), dtype=np.float32) * np.float32(0.05))
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    shift = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    d = abi.ConvDesc(abi.F16, abi.F16, b, h, w, c, c, oc, h, w, oc, 3, 1, 1, 1, 1, abi.ACT["leaky"], 0.1, 0, oc, abi.ACT["none"], 0.1, 1.0, 1.0,
                     abi.ALGO["igemm"], tile)
    assert L.msnh_hip_conv2d_tile_supported(ctypes.byref(d), tile)
    want, used = gu.conv2d(x, wt, dtype=abi.F16, stride=1, pad=1, scale=scale, shift=shift, act="leaky", algo="igemm", tile=tile)
    assert used == "igemm"
    xd = torch.from_numpy(np.ascontiguousarray(x.transpose(0, 2, 3, 1))).cuda().half()
    packed = np.zeros(L.msnh_hip_conv2d_packed_weight_elems(ctypes.byref(d), abi.ALGO["igemm"]), np.float16)
    abi.check(L.msnh_hip_conv2d_pack_weights(ctypes.byref(d), abi.ALGO["igemm"], np.ascontiguousarray(wt, np.float32).ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                             packed.ctypes.data_as(ctypes.c_void_p)))
    assert packed.size == oc * 9 * c
    wd = torch.from_numpy(packed).cuda()
    sc, sh = torch.from_numpy(scale).cuda(), torch.from_numpy(shift).cuda()
    clocks = torch.zeros(2, dtype=torch.int64, device="cuda")
    torch.cuda.synchronize()

    def run(sw, y):
        return D.msnh_hip_diag_patch8(tile, sw, b, c, h, w, oc, gu.ptr(xd), gu.ptr(wd), gu.ptr(sc), gu.ptr(sh), gu.ptr(y), gu.ptr(clocks), None)

    for sw in (0, 64):
        y = torch.full((b, h, w, oc), 3.0, dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()                            # (the fill runs on torch's stream, the kernel on the library's)
        assert run(sw, y) == 0
        abi.check(L.msnh_hip_stream_sync(None))
        got = y.float().cpu().numpy().transpose(0, 3, 1, 2)
        assert np.array_equal(got, want), sw
    t = clocks.cpu().numpy()
    assert t[0] > 0 and t[1] > 0
    assert 500.0 < t[0] / t[1] * 100.0 < 2600.0             # shader ticks per 100 MHz tick
    y = torch.empty((b, h, w, oc), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    listed = diag.switches()
    assert 0 in listed and 64 in listed
    for sw in listed:
        assert run(sw, y) == 0, sw
    abi.check(L.msnh_hip_stream_sync(None))
    assert run(6, y) != 0                                   # not instantiated
    assert D.msnh_hip_diag_patch8(45, 0, b, c, h, w, oc, gu.ptr(xd), gu.ptr(wd), gu.ptr(sc), gu.ptr(sh), gu.ptr(y), gu.ptr(clocks), None) != 0
    assert D.msnh_hip_diag_patch8(tile, 0, b, 96, h, w, oc, gu.ptr(xd), gu.ptr(wd), gu.ptr(sc), gu.ptr(sh), gu.ptr(y), gu.ptr(clocks), None) != 0
    assert D.msnh_hip_diag_patch8(tile, 64, b, c, h, w, oc, gu.ptr(xd), gu.ptr(wd), gu.ptr(sc), gu.ptr(sh), gu.ptr(y), None, None) != 0
    assert D.msnh_hip_diag_empty_launch(256, 256, None) == 0
    assert D.msnh_hip_diag_empty_launch(0, 256, None) != 0
    abi.check(L.msnh_hip_stream_sync(None))
