"""ctypes binding of include/ogle_hip.h.

Arguments are device pointers (integers, e.g. torch.Tensor.data_ptr()) and plain
sizes; PyTorch only supplies device memory and the stream.  Every wrapper raises
OgleError when the library reports a non-zero status.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libogle_hip.so")

OK, ERR_INVALID_ARG, ERR_UNSUPPORTED, ERR_LAUNCH, ERR_NOT_FOUND, ERR_NO_DEVICE = 0, -1, -2, -3, -4, -5
F32, F16 = 0, 1
ACT_NONE, ACT_CLIP, ACT_RELU = 0, 1, 2
VARIANT_NHWC4, VARIANT_PW, VARIANT_ANY4 = 0, 1, 2
FILTER_OHWI, FILTER_HWC = 0, 1
POOL_MAX, POOL_AVG, POOL_GLOBAL_AVG = 0, 1, 2
CONCAT_MAX_INPUTS = 16

# every symbol include/ogle_hip.h declares
SYMBOLS = [
    "ogle_hip_abi_version", "ogle_hip_last_error", "ogle_hip_status_string",
    "ogle_hip_registry_lookup", "ogle_hip_registry_size", "ogle_hip_registry_name",
    "ogle_hip_sync", "ogle_hip_packed_filter_elems", "ogle_hip_pack_filter",
    "ogle_hip_convert", "ogle_hip_conv2d", "ogle_hip_dwconv2d", "ogle_hip_pwconv_gemm",
    "ogle_hip_pool2d", "ogle_hip_concat", "ogle_hip_ssd_decode", "ogle_hip_ssd_detect",
    "ogle_hip_expf", "ogle_hip_transpose", "ogle_hip_conv_workspace_bytes",
    "ogle_hip_conv2d_batch", "ogle_hip_ssd_topk_nms", "ogle_hip_unary", "ogle_hip_add",
    "ogle_hip_batchnorm", "ogle_hip_gemm", "ogle_hip_gemm_workspace_bytes",
    "ogle_hip_conv2d_noalloc", "ogle_hip_launch_count",
    "ogle_hip_conv2d_batch_begin", "ogle_hip_conv2d_batch_finish",
    "ogle_hip_kernel_timing_begin", "ogle_hip_kernel_timing_end",
    "ogle_hip_conv_takes_image_stride",
]
CONV_NOALLOC_SCRATCH_BYTES = 16 << 20
UNARY_RELU, UNARY_CLIP = 0, 1


class OgleError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("ogle_hip status %d: %s" % (status, message))
        self.status = status


class ConvArgs(ctypes.Structure):
    _fields_ = [
        ("input_dev", ctypes.c_void_p), ("filter_dev", ctypes.c_void_p),
        ("bias_dev", ctypes.c_void_p), ("output_dev", ctypes.c_void_p),
        ("n", ctypes.c_int32), ("in_h", ctypes.c_int32), ("in_w", ctypes.c_int32),
        ("in_c", ctypes.c_int32),
        ("out_h", ctypes.c_int32), ("out_w", ctypes.c_int32), ("out_c", ctypes.c_int32),
        ("kernel_size", ctypes.c_int32), ("stride", ctypes.c_int32),
        ("padding", ctypes.c_int32), ("dilation", ctypes.c_int32), ("group", ctypes.c_int32),
        ("act", ctypes.c_int32), ("min_value", ctypes.c_float), ("max_value", ctypes.c_float),
        ("act_variant", ctypes.c_int32), ("dtype", ctypes.c_int32),
        ("workspace_dev", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("output2_dev", ctypes.c_void_p), ("out_c_split", ctypes.c_int32),
        ("out_image_stride", ctypes.c_int64),
    ]


class PoolArgs(ctypes.Structure):
    _fields_ = [
        ("input_dev", ctypes.c_void_p), ("output_dev", ctypes.c_void_p),
        ("n", ctypes.c_int32), ("in_h", ctypes.c_int32), ("in_w", ctypes.c_int32),
        ("c", ctypes.c_int32), ("out_h", ctypes.c_int32), ("out_w", ctypes.c_int32),
        ("kernel_size", ctypes.c_int32), ("stride", ctypes.c_int32),
        ("padding", ctypes.c_int32), ("pool_type", ctypes.c_int32), ("dtype", ctypes.c_int32),
    ]


class ConcatArgs(ctypes.Structure):
    _fields_ = [
        ("inputs_dev", ctypes.c_void_p * CONCAT_MAX_INPUTS),
        ("axis_len", ctypes.c_int64 * CONCAT_MAX_INPUTS),
        ("output_dev", ctypes.c_void_p), ("n_inputs", ctypes.c_int32),
        ("outer", ctypes.c_int64), ("inner", ctypes.c_int64), ("dtype", ctypes.c_int32),
    ]


class TransposeArgs(ctypes.Structure):
    _fields_ = [
        ("input_dev", ctypes.c_void_p), ("output_dev", ctypes.c_void_p),
        ("in_shape", ctypes.c_int32 * 4), ("perm", ctypes.c_int32 * 4), ("dtype", ctypes.c_int32),
    ]


class DecodeArgs(ctypes.Structure):
    _fields_ = [
        ("prediction_dev", ctypes.c_void_p), ("anchors_dev", ctypes.c_void_p),
        ("boxes_dev", ctypes.c_void_p), ("batch", ctypes.c_int32), ("priors", ctypes.c_int32),
        ("anchors_batch_stride", ctypes.c_int64), ("variances", ctypes.c_float * 4),
    ]


class DetectArgs(ctypes.Structure):
    _fields_ = [
        ("logits_dev", ctypes.c_void_p), ("prediction_dev", ctypes.c_void_p),
        ("anchors_dev", ctypes.c_void_p), ("boxes_dev", ctypes.c_void_p),
        ("batch", ctypes.c_int32), ("priors", ctypes.c_int32), ("classes", ctypes.c_int32),
        ("anchors_batch_stride", ctypes.c_int64), ("variances", ctypes.c_float * 4),
        ("score_threshold", ctypes.c_float), ("image_width", ctypes.c_float),
        ("image_height", ctypes.c_float),
        ("kept_count_dev", ctypes.c_void_p), ("kept_prior_dev", ctypes.c_void_p),
        ("kept_class_dev", ctypes.c_void_p), ("kept_score_dev", ctypes.c_void_p),
        ("kept_box_dev", ctypes.c_void_p), ("kept_rect_dev", ctypes.c_void_p),
    ]


class UnaryArgs(ctypes.Structure):
    _fields_ = [("input_dev", ctypes.c_void_p), ("output_dev", ctypes.c_void_p),
                ("count", ctypes.c_int64), ("op", ctypes.c_int32), ("min_value", ctypes.c_float),
                ("max_value", ctypes.c_float), ("dtype", ctypes.c_int32)]


class BinaryArgs(ctypes.Structure):
    _fields_ = [("a_dev", ctypes.c_void_p), ("b_dev", ctypes.c_void_p), ("output_dev", ctypes.c_void_p),
                ("count", ctypes.c_int64), ("dtype", ctypes.c_int32)]


class BatchNormArgs(ctypes.Structure):
    _fields_ = [("input_dev", ctypes.c_void_p), ("gamma_dev", ctypes.c_void_p),
                ("beta_dev", ctypes.c_void_p), ("mean_dev", ctypes.c_void_p),
                ("var_dev", ctypes.c_void_p), ("output_dev", ctypes.c_void_p),
                ("outer", ctypes.c_int64), ("channels", ctypes.c_int32), ("epsilon", ctypes.c_float),
                ("dtype", ctypes.c_int32)]


class GemmArgs(ctypes.Structure):
    _fields_ = [("a_dev", ctypes.c_void_p), ("b_dev", ctypes.c_void_p), ("c_dev", ctypes.c_void_p),
                ("y_dev", ctypes.c_void_p), ("m", ctypes.c_int32), ("n", ctypes.c_int32),
                ("k", ctypes.c_int32), ("trans_b", ctypes.c_int32), ("c_rank", ctypes.c_int32),
                ("alpha", ctypes.c_float), ("beta", ctypes.c_float),
                ("workspace_dev", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t)]


class NmsArgs(ctypes.Structure):
    _fields_ = [
        ("kept_count_dev", ctypes.c_void_p), ("kept_prior_dev", ctypes.c_void_p),
        ("kept_class_dev", ctypes.c_void_p), ("kept_score_dev", ctypes.c_void_p),
        ("kept_box_dev", ctypes.c_void_p), ("kept_rect_dev", ctypes.c_void_p),
        ("batch", ctypes.c_int32), ("stride", ctypes.c_int32), ("topk", ctypes.c_int32),
        ("nms_threshold", ctypes.c_float),
        ("final_count_dev", ctypes.c_void_p), ("final_prior_dev", ctypes.c_void_p),
        ("final_class_dev", ctypes.c_void_p), ("final_score_dev", ctypes.c_void_p),
        ("final_box_dev", ctypes.c_void_p), ("final_rect_dev", ctypes.c_void_p),
    ]


_lib = None


def lib():
    """The loaded kernel library.  Fails loudly if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OgleError(ERR_NO_DEVICE, "%s is missing: build it with "
                            "`make -C ogle_amd/csrc` (there is no CPU fallback)" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        l.ogle_hip_last_error.restype = ctypes.c_char_p
        l.ogle_hip_status_string.restype = ctypes.c_char_p
        l.ogle_hip_status_string.argtypes = [ctypes.c_int32]
        l.ogle_hip_registry_name.restype = ctypes.c_char_p
        l.ogle_hip_registry_name.argtypes = [ctypes.c_int32]
        l.ogle_hip_registry_lookup.argtypes = [ctypes.c_char_p, ctypes.c_char_p,
                                               ctypes.POINTER(ctypes.c_int32)]
        l.ogle_hip_sync.argtypes = [ctypes.c_void_p]
        l.ogle_hip_launch_count.restype = ctypes.c_int64
        l.ogle_hip_kernel_timing_end.restype = ctypes.c_int64
        l.ogle_hip_kernel_timing_end.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_int64]
        l.ogle_hip_packed_filter_elems.restype = ctypes.c_int64
        l.ogle_hip_packed_filter_elems.argtypes = [ctypes.c_int32] * 5
        l.ogle_hip_pack_filter.argtypes = [ctypes.c_void_p, ctypes.c_void_p] + \
            [ctypes.c_int32] * 6 + [ctypes.c_void_p]
        l.ogle_hip_convert.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p,
                                       ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p]
        for name, typ in (("ogle_hip_conv2d", ConvArgs), ("ogle_hip_dwconv2d", ConvArgs),
                          ("ogle_hip_conv2d_noalloc", ConvArgs),
                          ("ogle_hip_pwconv_gemm", ConvArgs), ("ogle_hip_pool2d", PoolArgs),
                          ("ogle_hip_concat", ConcatArgs), ("ogle_hip_ssd_decode", DecodeArgs),
                          ("ogle_hip_ssd_detect", DetectArgs),
                          ("ogle_hip_ssd_topk_nms", NmsArgs), ("ogle_hip_unary", UnaryArgs),
                          ("ogle_hip_add", BinaryArgs), ("ogle_hip_batchnorm", BatchNormArgs),
                          ("ogle_hip_gemm", GemmArgs),
                          ("ogle_hip_transpose", TransposeArgs)):
            getattr(l, name).argtypes = [ctypes.POINTER(typ), ctypes.c_void_p]
        l.ogle_hip_conv2d_batch.argtypes = [ctypes.POINTER(ConvArgs), ctypes.c_int32, ctypes.c_void_p]
        l.ogle_hip_conv2d_batch_begin.argtypes = [ctypes.POINTER(ConvArgs), ctypes.c_int32,
                                                  ctypes.POINTER(ctypes.c_int32), ctypes.c_void_p]
        l.ogle_hip_conv2d_batch_finish.argtypes = [ctypes.POINTER(ConvArgs), ctypes.c_int32, ctypes.c_void_p]
        l.ogle_hip_conv_workspace_bytes.argtypes = [ctypes.POINTER(ConvArgs)]
        l.ogle_hip_conv_workspace_bytes.restype = ctypes.c_size_t
        l.ogle_hip_conv_takes_image_stride.argtypes = [ctypes.POINTER(ConvArgs)]
        l.ogle_hip_gemm_workspace_bytes.argtypes = [ctypes.POINTER(GemmArgs)]
        l.ogle_hip_gemm_workspace_bytes.restype = ctypes.c_size_t
        l.ogle_hip_expf.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64,
                                    ctypes.c_void_p]
        _lib = l
    return _lib


def last_error():
    return lib().ogle_hip_last_error().decode()


def check(status):
    if status != OK:
        raise OgleError(status, last_error())


def registry_names():
    l = lib()
    return [l.ogle_hip_registry_name(i).decode() for i in range(l.ogle_hip_registry_size())]


def registry_lookup(name, options=""):
    h = ctypes.c_int32(0)
    check(lib().ogle_hip_registry_lookup(name.encode(), options.encode(), ctypes.byref(h)))
    return h.value


def sync(stream=0):
    check(lib().ogle_hip_sync(stream))


def out_size(n, k, stride, pad, dilation=1):
    return (n - (k * dilation - dilation + 1) + 2 * pad) // stride + 1


def conv_args(x_ptr, w_ptr, b_ptr, y_ptr, n, h, w, c, o, k, stride=1, pad=0, dilation=1, group=1,
              act=ACT_NONE, minv=0.0, maxv=0.0, variant=VARIANT_NHWC4, dtype=F32):
    return ConvArgs(x_ptr, w_ptr, b_ptr, y_ptr, n, h, w, c,
                    out_size(h, k, stride, pad, dilation), out_size(w, k, stride, pad, dilation), o,
                    k, stride, pad, dilation, group, act, minv, maxv, variant, dtype, None, 0, None, 0, 0)
