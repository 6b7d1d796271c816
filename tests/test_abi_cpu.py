"""CPU-only checks of the C ABI: the library loads, exports every symbol the header
declares, and rejects bad arguments with error codes instead of aborting (the
reference aborts through CHECK / LOG(FATAL); the failures exercised here are the
ones its kernels check: conv2d.cc:71-86,189, pool.cc:36-50, concat.cc:116-121,
decoder.cc:82-85).  No kernel is launched."""
import ctypes
import os
import re

import pytest

from ogle_amd import hip as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "ogle_hip.h")).read()
    declared = set(re.findall(r"\b(ogle_hip_[a-z0-9_]+)\s*\(", header))
    assert declared == set(H.SYMBOLS)
    lib = H.lib()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.ogle_hip_abi_version() == 101


def test_registry_covers_the_reference_shader_table():
    names = H.registry_names()
    for stem in ["conv2d", "conv2d_any4", "conv2d_dw", "conv2d_dw_any4", "conv2d_pw",
                 "conv2d_pw_any4", "conv2d_grp", "pool", "pool_any4", "concat_multi", "decoder"]:
        assert stem in names
    h0 = H.registry_lookup("conv2d_pw", "")
    h1 = H.registry_lookup("conv2d_pw", "#define USE_BIAS\n#define USE_CLIP\n")
    assert h0 != h1 and (h0 >> 8) == (h1 >> 8)
    with pytest.raises(H.OgleError) as e:
        H.registry_lookup("no_such_shader")
    assert e.value.status == H.ERR_NOT_FOUND and "no_such_shader" in str(e.value)


def _conv(**kw):
    base = dict(x_ptr=0x1000, w_ptr=0x2000, b_ptr=None, y_ptr=0x3000, n=1, h=8, w=8, c=8, o=8, k=3,
                stride=1, pad=1)
    base.update(kw)
    return H.conv_args(**base)


def test_conv_argument_errors():
    lib = H.lib()
    a = _conv()
    a.out_h = 7                     # does not follow from the input size
    assert lib.ogle_hip_conv2d(ctypes.byref(a), None) == H.ERR_INVALID_ARG
    assert "output" in H.last_error()
    a = _conv(group=3)              # channels not divisible by group
    assert lib.ogle_hip_conv2d(ctypes.byref(a), None) == H.ERR_INVALID_ARG
    a = _conv(x_ptr=None)
    assert lib.ogle_hip_conv2d(ctypes.byref(a), None) == H.ERR_INVALID_ARG
    a = _conv(k=3, pad=1)           # pointwise entry needs 1x1 s1 p0
    assert lib.ogle_hip_pwconv_gemm(ctypes.byref(a), None) == H.ERR_INVALID_ARG
    a = _conv(group=4)              # depthwise entry needs group == C
    assert lib.ogle_hip_dwconv2d(ctypes.byref(a), None) == H.ERR_INVALID_ARG
    a = _conv(dtype=7)
    assert lib.ogle_hip_conv2d(ctypes.byref(a), None) == H.ERR_INVALID_ARG
    assert lib.ogle_hip_conv2d(None, None) == H.ERR_INVALID_ARG


def test_pool_concat_decode_argument_errors():
    lib = H.lib()
    p = H.PoolArgs(0x1000, 0x2000, 1, 8, 8, 4, 5, 4, 2, 2, 0, H.POOL_MAX, H.F32)  # out_h wrong
    assert lib.ogle_hip_pool2d(ctypes.byref(p), None) == H.ERR_INVALID_ARG
    p = H.PoolArgs(0x1000, 0x2000, 1, 8, 6, 4, 1, 1, 8, 1, 0, H.POOL_GLOBAL_AVG, H.F32)  # H != W
    assert lib.ogle_hip_pool2d(ctypes.byref(p), None) == H.ERR_INVALID_ARG
    c = H.ConcatArgs()
    c.n_inputs = 17
    assert lib.ogle_hip_concat(ctypes.byref(c), None) == H.ERR_INVALID_ARG
    c.n_inputs = 0
    assert lib.ogle_hip_concat(ctypes.byref(c), None) == H.ERR_INVALID_ARG
    d = H.DecodeArgs(0x1000, 0x2000, 0x3000, 2, 100, 17, (ctypes.c_float * 4)(.1, .1, .2, .2))
    assert lib.ogle_hip_ssd_decode(ctypes.byref(d), None) == H.ERR_INVALID_ARG
    assert lib.ogle_hip_packed_filter_elems(H.FILTER_HWC, 8, 2, 3, 3) == -1
    assert lib.ogle_hip_packed_filter_elems(H.FILTER_OHWI, 8, 2, 3, 3) == 144
    assert H.lib().ogle_hip_status_string(H.ERR_UNSUPPORTED) == b"unsupported"
