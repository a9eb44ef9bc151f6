"""Helpers for GPU tests: torch only provides device memory; every kernel call goes through the C ABI."""
import ctypes

import numpy as np
import torch

from msnhnet_amd import hipabi as abi

TORCH_DT = {abi.F32: torch.float32, abi.F16: torch.float16}
_inited = False


def init():
    global _inited
    if not _inited:
        abi.check(abi.lib().msnh_hip_init(0))
        _inited = True


def sync():
    torch.cuda.synchronize()
    abi.check(abi.lib().msnh_hip_stream_sync(None))


def nhwc_dev(x_nchw, dtype, ld=None, fill=7.0):
    """NCHW numpy -> device NHWC tensor [B,H,W,ld] (channels >= C hold `fill` so stray reads show up)."""
    b, c, h, w = x_nchw.shape
    ld = ld or c
    t = torch.full((b, h, w, ld), fill, dtype=TORCH_DT[dtype])
    t[..., :c] = torch.from_numpy(np.ascontiguousarray(x_nchw.transpose(0, 2, 3, 1))).to(TORCH_DT[dtype])
    return t.cuda()


def nchw_host(t, c):
    """device NHWC tensor -> NCHW float32 numpy of the first c channels."""
    return t[..., :c].float().cpu().numpy().transpose(0, 3, 1, 2).copy()


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(TORCH_DT[dtype])
    return t.cuda()


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def round_f16(a):
    return np.asarray(a, np.float32).astype(np.float16).astype(np.float32)


def rel_err(a, b):
    """max|a-b| / max|b| over finite entries; non-finite entries must match in class."""
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    assert a.shape == b.shape, (a.shape, b.shape)
    fa, fb = np.isfinite(a), np.isfinite(b)
    assert (fa == fb).all(), "finite/non-finite mismatch"
    if (~fb).any():
        assert (np.isnan(a[~fb]) == np.isnan(b[~fb])).all() and (np.sign(a[~fb & ~np.isnan(a)]) == np.sign(b[~fb & ~np.isnan(b)])).all()
    if not fb.any():
        return 0.0
    return float(np.abs(a[fb] - b[fb]).max() / max(np.abs(b[fb]).max(), 1e-30))


def conv2d_tail(x, w_oihw, w2_oi, *, stride=1, pad=0, scale=None, shift=None, act="none", act_param=0.1, residual=None, act2="none", res_mul=1.0, out_mul=1.0,
                scale2=None, shift2=None, act3="none", act3_param=0.1, z_mul=1.0, write_y=True, tile=0, in_ld=None, out_ld=None, res_ld=None, z_ld=None):
    """msnh_hip_conv2d_tail, float16: x NCHW float32 numpy, w_oihw the first convolution's filters, w2_oi [out_c2][out_c] the 1x1 filters.
    Returns (y, z) as NCHW float32 numpy; y is None when write_y is False (the buffer is then checked to be untouched)."""
    init()
    L = abi.lib()
    b, c, h, wd = x.shape
    oc, _, k, _ = w_oihw.shape
    oc2 = w2_oi.shape[0]
    oh = (h + 2 * pad - k) // stride + 1
    ow = (wd + 2 * pad - k) // stride + 1
    d = abi.ConvDesc(abi.F16, abi.F16, b, h, wd, c, in_ld or c, oc, oh, ow, out_ld or oc, k, stride, pad, 1, 1, abi.ACT[act], act_param,
                     1 if residual is not None else 0, res_ld or oc, abi.ACT[act2], 0.1, res_mul, out_mul, abi.ALGO["igemm"], tile)
    t = abi.ConvTailDesc(oc2, z_ld or oc2, abi.ACT[act3], act3_param, z_mul, 1 if write_y else 0)
    if not L.msnh_hip_conv2d_tail_supported(ctypes.byref(d), ctypes.byref(t), tile):
        return None
    fp = ctypes.POINTER(ctypes.c_float)

    def pack(desc, w4):
        n = L.msnh_hip_conv2d_packed_weight_elems(ctypes.byref(desc), abi.ALGO["igemm"])
        packed = np.zeros(n, np.float16)
        wf = np.ascontiguousarray(w4, np.float32)
        abi.check(L.msnh_hip_conv2d_pack_weights(ctypes.byref(desc), abi.ALGO["igemm"], wf.ctypes.data_as(fp), packed.ctypes.data_as(ctypes.c_void_p)))
        return dev(packed)

    wdev = pack(d, w_oihw)
    d2 = abi.ConvDesc(abi.F16, abi.F16, b, oh, ow, oc, out_ld or oc, oc2, oh, ow, z_ld or oc2, 1, 1, 0, 1, 1, abi.ACT[act3], act3_param, 0, oc2, abi.ACT["none"], 0.1,
                      1.0, z_mul, abi.ALGO["igemm"], 0)
    w2dev = pack(d2, w2_oi.reshape(oc2, oc, 1, 1))
    xdev = nhwc_dev(x, abi.F16, in_ld)
    ydev = torch.full((b, oh, ow, out_ld or oc), 3.0, dtype=torch.float16).cuda()
    zdev = torch.full((b, oh, ow, z_ld or oc2), 5.0, dtype=torch.float16).cuda()
    mk = lambda v: dev(np.asarray(v, np.float32)) if v is not None else None
    sdev, hdev, s2dev, h2dev = mk(scale), mk(shift), mk(scale2), mk(shift2)
    rdev = nhwc_dev(residual, abi.F16, res_ld) if residual is not None else None
    sync()
    abi.check(L.msnh_hip_conv2d_tail(ctypes.byref(d), ctypes.byref(t), ptr(xdev), ptr(wdev), ptr(sdev), ptr(hdev), ptr(rdev), ptr(ydev), ptr(w2dev), ptr(s2dev),
                                     ptr(h2dev), ptr(zdev), None))
    sync()
    if (out_ld or oc) > oc:
        assert (ydev[..., oc:].float().cpu().numpy() == 3.0).all(), "kernel wrote outside y's channel slice"
    if (z_ld or oc2) > oc2:
        assert (zdev[..., oc2:].float().cpu().numpy() == 5.0).all(), "kernel wrote outside z's channel slice"
    if not write_y:
        assert (ydev.float().cpu().numpy() == 3.0).all(), "y was written although write_y is 0"
    return (nchw_host(ydev, oc) if write_y else None), nchw_host(zdev, oc2)


def conv2d(x, w_oihw, *, dtype, out_dtype=None, stride=1, pad=0, dil=1, groups=1, scale=None, shift=None, act="none",
           act_param=0.1, residual=None, act2="none", act2_param=0.1, res_mul=1.0, out_mul=1.0, algo="auto",
           in_ld=None, out_ld=None, res_ld=None, tile=0, upsample=1, xcd_blocks=0):
    """x: NCHW float32 numpy (for every algo; the stem algo is fed NCHW as is). Returns NCHW float32 numpy.
    upsample=2: msnh_conv_desc::out_upsample, the result is the 2x nearest-neighbour upsampled tensor."""
    init()
    L = abi.lib()
    out_dtype = dtype if out_dtype is None else out_dtype
    b, c, h, wd = x.shape
    oc, _, k, _ = w_oihw.shape
    ext = dil * (k - 1) + 1
    oh = (h + 2 * pad - ext) // stride + 1
    ow = (wd + 2 * pad - ext) // stride + 1
    d = abi.ConvDesc(dtype, out_dtype, b, h, wd, c, in_ld or c, oc, oh, ow, out_ld or oc, k, stride, pad, dil, groups,
                     abi.ACT[act], act_param, 1 if residual is not None else 0, res_ld or oc, abi.ACT[act2], act2_param,
                     res_mul, out_mul, abi.ALGO[algo], tile, 2 if upsample == 2 else 0, xcd_blocks)
    resolved = L.msnh_hip_conv2d_select_algo(ctypes.byref(d))
    n = L.msnh_hip_conv2d_packed_weight_elems(ctypes.byref(d), resolved)
    host_dt = np.float32 if (dtype == abi.F32 or resolved == abi.ALGO["stem"]) else np.float16
    if resolved == abi.ALGO["stem"] and dtype == abi.F16:
        n //= 2
    packed = np.zeros(n, host_dt)
    wf = np.ascontiguousarray(w_oihw, np.float32)
    abi.check(L.msnh_hip_conv2d_pack_weights(ctypes.byref(d), resolved, wf.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                             packed.ctypes.data_as(ctypes.c_void_p)))
    wdev = dev(packed)
    if resolved == abi.ALGO["stem"]:
        xdev = dev(np.ascontiguousarray(x, np.float32))
    else:
        xdev = nhwc_dev(x, dtype, in_ld)
    ydev = torch.full((b, oh * upsample, ow * upsample, out_ld or oc), 3.0, dtype=TORCH_DT[out_dtype]).cuda()
    sdev = dev(np.asarray(scale, np.float32)) if scale is not None else None
    hdev = dev(np.asarray(shift, np.float32)) if shift is not None else None
    rdev = nhwc_dev(residual, dtype, res_ld) if residual is not None else None
    wsb = L.msnh_hip_conv2d_workspace_bytes(ctypes.byref(d), resolved)
    ws = torch.empty(max(int(wsb), 16), dtype=torch.uint8).cuda()
    sync()
    abi.check(L.msnh_hip_conv2d(ctypes.byref(d), ptr(xdev), ptr(wdev), ptr(sdev), ptr(hdev), ptr(rdev), ptr(ydev), ptr(ws), wsb, None))
    sync()
    out = nchw_host(ydev, oc)
    if (out_ld or oc) > oc:
        pad_region = ydev[..., oc:].float().cpu().numpy()
        assert (pad_region == 3.0).all(), "kernel wrote outside its channel slice"
    return out, abi.ALGO_NAME[resolved]
