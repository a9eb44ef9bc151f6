"""ctypes binding of the kernel library's C ABI (include/msnh_hip.h).

Loading fails loudly when `libmsnh_hip.so` has not been built; nothing here falls back to a CPU path.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmsnh_hip.so")

F32, F16 = 0, 1
ACT = {"logistic": 0, "relu": 1, "relu6": 2, "leaky": 8, "swish": 16, "hardswish": 17, "mish": 18, "none": 22}
ALGO = {"auto": 0, "direct": 1, "igemm": 2, "depthwise": 3, "winograd": 4, "stem": 5, "igemm_splitk": 6, "pointwise": 7, "stem_down": 8, "winograd_fused": 9, "mbconv": 10, "igemm_tail": 11}
ALGO_NAME = {v: k for k, v in ALGO.items()}


class ConvDesc(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int), ("out_dtype", ctypes.c_int),
                ("batch", ctypes.c_int), ("in_h", ctypes.c_int), ("in_w", ctypes.c_int), ("in_c", ctypes.c_int), ("in_ld", ctypes.c_int),
                ("out_c", ctypes.c_int), ("out_h", ctypes.c_int), ("out_w", ctypes.c_int), ("out_ld", ctypes.c_int),
                ("ksize", ctypes.c_int), ("stride", ctypes.c_int), ("pad", ctypes.c_int), ("dilation", ctypes.c_int), ("groups", ctypes.c_int),
                ("act", ctypes.c_int), ("act_param", ctypes.c_float),
                ("has_residual", ctypes.c_int), ("res_ld", ctypes.c_int), ("act2", ctypes.c_int), ("act2_param", ctypes.c_float),
                ("res_mul", ctypes.c_float), ("out_mul", ctypes.c_float), ("algo", ctypes.c_int), ("tile", ctypes.c_int), ("out_upsample", ctypes.c_int), ("xcd_blocks", ctypes.c_int)]


class ConvTailDesc(ctypes.Structure):
    """msnh_conv_tail_desc of include/msnh_hip.h"""
    _fields_ = [("out_c", ctypes.c_int), ("out_ld", ctypes.c_int), ("act", ctypes.c_int), ("act_param", ctypes.c_float), ("out_mul", ctypes.c_float),
                ("write_y", ctypes.c_int)]


class MbconvDesc(ctypes.Structure):
    """msnh_mbconv_desc of include/msnh_hip.h"""
    _fields_ = [("batch", ctypes.c_int), ("in_h", ctypes.c_int), ("in_w", ctypes.c_int), ("in_c", ctypes.c_int), ("in_ld", ctypes.c_int),
                ("exp_c", ctypes.c_int), ("stride", ctypes.c_int),
                ("out_c", ctypes.c_int), ("out_h", ctypes.c_int), ("out_w", ctypes.c_int), ("out_ld", ctypes.c_int),
                ("act1", ctypes.c_int), ("act2", ctypes.c_int), ("act3", ctypes.c_int), ("act4", ctypes.c_int),
                ("act1_param", ctypes.c_float), ("act2_param", ctypes.c_float), ("act3_param", ctypes.c_float), ("act4_param", ctypes.c_float),
                ("has_residual", ctypes.c_int), ("res_ld", ctypes.c_int),
                ("mul1", ctypes.c_float), ("mul2", ctypes.c_float), ("out_mul", ctypes.c_float), ("res_mul", ctypes.c_float)]


class HipError(RuntimeError):
    pass


_lib = None

# every symbol include/msnh_hip.h declares
SYMBOLS = [
    "msnh_hip_last_error", "msnh_hip_init", "msnh_hip_device_count", "msnh_hip_device_name", "msnh_hip_malloc", "msnh_hip_free",
    "msnh_hip_host_alloc", "msnh_hip_host_free", "msnh_hip_memcpy_h2d", "msnh_hip_memcpy_d2h", "msnh_hip_memcpy_d2d",
    "msnh_hip_fill_zero", "msnh_hip_stream_create", "msnh_hip_stream_destroy", "msnh_hip_stream_sync", "msnh_hip_event_create",
    "msnh_hip_event_destroy", "msnh_hip_event_record", "msnh_hip_stream_wait_event", "msnh_hip_event_sync", "msnh_hip_event_elapsed_ms", "msnh_hip_graph_begin",
    "msnh_hip_graph_end", "msnh_hip_graph_launch", "msnh_hip_graph_destroy", "msnh_hip_conv_stem_down_supported", "msnh_hip_conv_stem_down_packed_elems", "msnh_hip_conv_stem_down_pack", "msnh_hip_conv_stem_down", "msnh_hip_conv_stem_down_tail_supported", "msnh_hip_conv_stem_down_tail_packed_elems", "msnh_hip_conv_stem_down_tail_pack", "msnh_hip_conv_stem_down_tail", "msnh_hip_mbconv_supported", "msnh_hip_mbconv_packed_bytes", "msnh_hip_mbconv_pack", "msnh_hip_mbconv", "msnh_hip_conv2d_tile_count", "msnh_hip_conv2d_pack_layout_version", "msnh_hip_conv2d_tile_supported", "msnh_hip_conv2d_select_algo",
    "msnh_hip_conv2d_packed_weight_elems", "msnh_hip_conv2d_pack_weights", "msnh_hip_conv2d_workspace_bytes", "msnh_hip_conv2d",
    "msnh_hip_conv2d_tail_tile_first", "msnh_hip_conv2d_tail_supported", "msnh_hip_conv2d_tail", "msnh_hip_letterbox_u8", "msnh_hip_image_u8_to_input",
    "msnh_hip_affine_act", "msnh_hip_add_act", "msnh_hip_copy_channels", "msnh_hip_maxpool", "msnh_hip_maxpool_chain", "msnh_hip_maxpool_chain_supported", "msnh_hip_avgpool",
    "msnh_hip_upsample_nearest", "msnh_hip_pad", "msnh_hip_slice", "msnh_hip_upsample_bilinear", "msnh_hip_softmax", "msnh_hip_deconv_col2im", "msnh_hip_connected", "msnh_hip_nchw_to_nhwc", "msnh_hip_nhwc_to_nchw", "msnh_hip_yolo_decode", "msnh_hip_yolo_decode_candidates", "msnh_hip_yolo_decode_candidates_heads",
    "msnh_hip_yolo_gather", "msnh_hip_yolo_nms", "msnh_hip_yolo_nms_workspace_bytes", "msnh_hip_yolo_nms_pair_workspace_bytes", "msnh_hip_yolo_nms_static", "msnh_hip_yolo_nms_static_max_bytes", "msnh_hip_absmax", "msnh_hip_count_nonfinite", "msnh_hip_mfma_probe",
]


class YoloHead(ctypes.Structure):
    """msnh_yolo_head of include/msnh_hip.h"""
    _fields_ = [("x", ctypes.c_void_p), ("x_ld", ctypes.c_int), ("x_mul", ctypes.c_float), ("h", ctypes.c_int), ("w", ctypes.c_int),
                ("anchors", ctypes.c_float * 6), ("ratio", ctypes.c_float), ("cand_base", ctypes.c_int)]


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipError(f"{LIB_PATH} is missing: build it first (python -m msnhnet_amd.build)")
    L = ctypes.CDLL(LIB_PATH)
    vp, ci, cf, ll, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong, ctypes.c_size_t
    fp = ctypes.POINTER(ctypes.c_float)
    cdp = ctypes.POINTER(ConvDesc)
    L.msnh_hip_last_error.restype = ctypes.c_char_p
    L.msnh_hip_init.argtypes = [ci]
    L.msnh_hip_device_count.argtypes = [ctypes.POINTER(ci)]
    L.msnh_hip_device_name.argtypes = [ctypes.c_char_p, ci, ctypes.POINTER(ci), ctypes.POINTER(sz)]
    L.msnh_hip_malloc.argtypes = [ctypes.POINTER(vp), sz]
    L.msnh_hip_free.argtypes = [vp]
    L.msnh_hip_host_alloc.argtypes = [ctypes.POINTER(vp), sz]
    L.msnh_hip_host_free.argtypes = [vp]
    for n in ("h2d", "d2h", "d2d"):
        getattr(L, "msnh_hip_memcpy_" + n).argtypes = [vp, vp, sz, vp]
    L.msnh_hip_fill_zero.argtypes = [vp, sz, vp]
    L.msnh_hip_stream_create.argtypes = [ctypes.POINTER(vp)]
    L.msnh_hip_stream_destroy.argtypes = [vp]
    L.msnh_hip_stream_sync.argtypes = [vp]
    L.msnh_hip_event_create.argtypes = [ctypes.POINTER(vp)]
    L.msnh_hip_event_destroy.argtypes = [vp]
    L.msnh_hip_event_record.argtypes = [vp, vp]
    L.msnh_hip_stream_wait_event.argtypes = [vp, vp]
    L.msnh_hip_event_sync.argtypes = [vp]
    L.msnh_hip_event_elapsed_ms.argtypes = [vp, vp, fp]
    L.msnh_hip_graph_begin.argtypes = [vp]
    L.msnh_hip_graph_end.argtypes = [vp, ctypes.POINTER(vp)]
    L.msnh_hip_graph_launch.argtypes = [vp, vp]
    L.msnh_hip_graph_destroy.argtypes = [vp]
    L.msnh_hip_conv2d_tile_supported.argtypes = [cdp, ci]
    L.msnh_hip_conv2d_select_algo.argtypes = [cdp]
    L.msnh_hip_conv2d_packed_weight_elems.argtypes = [cdp, ci]
    L.msnh_hip_conv2d_packed_weight_elems.restype = sz
    L.msnh_hip_conv2d_pack_weights.argtypes = [cdp, ci, fp, vp]
    L.msnh_hip_letterbox_u8.argtypes = [vp, ci, ci, ci, ci, ci, ci, vp, vp]
    L.msnh_hip_image_u8_to_input.argtypes = [vp, ci, ci, ci, ci, ci, fp, fp, ci, vp, vp]
    L.msnh_hip_conv2d_workspace_bytes.argtypes = [cdp, ci]
    L.msnh_hip_conv2d_workspace_bytes.restype = sz
    L.msnh_hip_conv2d.argtypes = [cdp, vp, vp, vp, vp, vp, vp, vp, sz, vp]
    L.msnh_hip_conv2d_tail_supported.argtypes = [cdp, ctypes.POINTER(ConvTailDesc), ci]
    L.msnh_hip_conv2d_tail.argtypes = [cdp, ctypes.POINTER(ConvTailDesc), vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    L.msnh_hip_affine_act.argtypes = [ci, ci, ll, ci, vp, ci, vp, vp, ci, cf, cf, vp, ci, vp]
    L.msnh_hip_add_act.argtypes = [ci, ll, ci, vp, ci, cf, vp, ci, cf, ci, cf, cf, vp, ci, vp]
    L.msnh_hip_copy_channels.argtypes = [ci, ll, ci, vp, ci, cf, vp, ci, vp]
    L.msnh_hip_maxpool.argtypes = [ci, ci, ci, ci, ci, vp, ci, ci, ci, ci, ci, ci, vp, ci, vp]
    L.msnh_hip_maxpool_chain_supported.argtypes = [ci, ci, ci, ci, ci, ci]
    L.msnh_hip_maxpool_chain.argtypes = [ci, ci, ci, ci, ci, ci, ci, vp, ci, ctypes.POINTER(vp), ctypes.POINTER(ci), vp]
    L.msnh_hip_avgpool.argtypes = [ci, ci, ci, ci, ci, ci, vp, ci, ci, ci, ci, ci, ci, cf, vp, ci, vp]
    L.msnh_hip_upsample_nearest.argtypes = [ci, ci, ci, ci, ci, vp, ci, ci, cf, vp, ci, vp]
    L.msnh_hip_pad.argtypes = [ci, ci, ci, ci, ci, vp, ci, ci, ci, ci, ci, cf, cf, vp, ci, vp]
    L.msnh_hip_slice.argtypes = [ci, ci, ci, ci, vp, ci, ci, ci, ci, ci, ci, ci, ci, ci, ci, cf, vp, ci, vp]
    L.msnh_hip_upsample_bilinear.argtypes = [ci, ci, ci, ci, ci, vp, ci, ci, ci, ci, cf, vp, ci, vp]
    L.msnh_hip_softmax.argtypes = [ci, ci, ci, ci, vp, ci, cf, cf, vp, ci, cf, vp]
    L.msnh_hip_deconv_col2im.argtypes = [ci, ci, ci, ci, ci, ci, ci, ci, vp, ci, cf, vp, ci, cf, ci, ci, cf, vp, ci, vp]
    L.msnh_hip_connected.argtypes = [ci, ci, ci, ci, vp, cf, vp, vp, ci, cf, vp, vp]
    L.msnh_hip_nchw_to_nhwc.argtypes = [ci, ci, ci, ci, ci, vp, cf, vp, ci, vp]
    L.msnh_hip_nhwc_to_nchw.argtypes = [ci, ci, ci, ci, ci, vp, ci, cf, vp, vp]
    L.msnh_hip_yolo_decode.argtypes = [ci, ci, ci, ci, ci, vp, ci, cf, fp, cf, ci, vp, ll, cf, vp, ci, ci, vp, vp]
    L.msnh_hip_yolo_decode_candidates.argtypes = [ci, ci, ci, ci, ci, vp, ci, cf, fp, cf, ci, vp, ll, cf, vp, ci, ci, vp, vp, vp]
    L.msnh_hip_yolo_decode_candidates_heads.argtypes = [ci, ci, ci, ci, ctypes.POINTER(YoloHead), ci, vp, ll, cf, vp, ci, vp, vp, vp]
    L.msnh_hip_mfma_probe.argtypes = [ci, ci, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double), vp]
    L.msnh_hip_yolo_gather.argtypes = [ci, ci, vp, ll, vp, ci, vp, vp, vp]
    L.msnh_hip_yolo_nms.argtypes = [ci, ci, vp, ci, vp, cf, vp, ci, vp, vp, sz, vp]
    L.msnh_hip_yolo_nms_workspace_bytes.argtypes = [ci, ci, ci]
    L.msnh_hip_yolo_nms_workspace_bytes.restype = sz
    L.msnh_hip_yolo_nms_pair_workspace_bytes.argtypes = [ci, ci, ci]
    L.msnh_hip_yolo_nms_pair_workspace_bytes.restype = sz
    L.msnh_hip_yolo_nms_static.argtypes = [ci, ci, vp, ci, vp, cf, vp, ci, vp, vp]
    L.msnh_hip_yolo_nms_static_max_bytes.argtypes = []
    L.msnh_hip_yolo_nms_static_max_bytes.restype = sz
    L.msnh_hip_absmax.argtypes = [ci, ll, ci, vp, ci, vp, vp]
    L.msnh_hip_conv_stem_down_packed_elems.argtypes = [ci, ci]
    L.msnh_hip_conv_stem_down_packed_elems.restype = sz
    L.msnh_hip_conv_stem_down_pack.argtypes = [vp, ci, vp, vp, vp]
    L.msnh_hip_conv_stem_down.argtypes = [ci, ci, ci, vp, vp, vp, vp, ci, cf, cf, ci, vp, vp, vp, ci, cf, cf, vp, ci, vp]
    L.msnh_hip_conv_stem_down_tail_supported.argtypes = [ci, ci, ci, ci, ci]
    L.msnh_hip_conv_stem_down_tail_packed_elems.argtypes = [ci]
    L.msnh_hip_conv_stem_down_tail_packed_elems.restype = sz
    L.msnh_hip_conv_stem_down_tail_pack.argtypes = [ci, vp, vp]
    L.msnh_hip_conv_stem_down_tail.argtypes = [ci, ci, ci, vp, vp, vp, vp, ci, cf, cf, ci, vp, vp, vp, ci, cf, cf, vp, ci, vp, vp, vp, ci, cf, cf, vp, ci, vp]
    L.msnh_hip_count_nonfinite.argtypes = [ci, ll, ci, vp, ci, vp, vp]
    L.msnh_hip_mbconv_supported.argtypes = [vp]
    L.msnh_hip_mbconv_packed_bytes.argtypes = [vp]
    L.msnh_hip_mbconv_packed_bytes.restype = sz
    L.msnh_hip_mbconv_pack.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp]
    L.msnh_hip_mbconv.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp]
    _lib = L
    return L


def check(rc):
    if rc != 0:
        raise HipError(lib().msnh_hip_last_error().decode(errors="replace"))
