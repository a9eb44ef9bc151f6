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


def conv2d(x, w_oihw, *, dtype, out_dtype=None, stride=1, pad=0, dil=1, groups=1, scale=None, shift=None, act="none",
           act_param=0.1, residual=None, act2="none", act2_param=0.1, res_mul=1.0, out_mul=1.0, algo="auto",
           in_ld=None, out_ld=None, res_ld=None, tile=0):
    """x: NCHW float32 numpy (for every algo; the stem algo is fed NCHW as is). Returns NCHW float32 numpy."""
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
                     res_mul, out_mul, abi.ALGO[algo], tile)
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
    ydev = torch.full((b, oh, ow, out_ld or oc), 3.0, dtype=TORCH_DT[out_dtype]).cuda()
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
