"""ctypes binding of libwinoconv_hip.so (the C ABI declared in include/winoconv.h).

The library is built in-tree by `build()` (hipcc, gfx950) and loaded by `load()`.
There is no fallback: if the shared object is missing or a call fails, an exception
is raised.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libwinoconv_hip.so")
CSRC = os.path.join(_HERE, "csrc")

WC_F32, WC_F16, WC_BF16 = 0, 1, 2
WC_OK, WC_ERR_BAD_ARG, WC_ERR_UNSUPPORTED, WC_ERR_WORKSPACE, WC_ERR_HIP = 0, -1, -2, -3, -4
WC_MAX_PIECES = 64
WC_STATIC_SCRATCH_BYTES = 64 * 1024 * 1024

c_int_p = ctypes.POINTER(ctypes.c_int)


class Piece(ctypes.Structure):
    _fields_ = [("tap0", ctypes.c_int * 3), ("r", ctypes.c_int * 3), ("t_offset", ctypes.c_int)]


class Plan(ctypes.Structure):
    _fields_ = [("n_pieces", ctypes.c_int), ("t_total", ctypes.c_int), ("tap_step", ctypes.c_int),
                ("m", ctypes.c_int * 3), ("piece", Piece * WC_MAX_PIECES)]


class ConvDesc(ctypes.Structure):
    _fields_ = [("ndim", ctypes.c_int), ("N", ctypes.c_int), ("C", ctypes.c_int), ("K", ctypes.c_int),
                ("in_", ctypes.c_int * 3), ("kernel", ctypes.c_int * 3), ("pad", ctypes.c_int * 3),
                ("stride", ctypes.c_int), ("m", ctypes.c_int), ("dtype", ctypes.c_int),
                ("chunk_images", ctypes.c_int), ("whole_kernel", ctypes.c_int), ("stacked", ctypes.c_int),
                ("unfused", ctypes.c_int), ("x_layout", ctypes.c_int), ("y_layout", ctypes.c_int),
                ("direct", ctypes.c_int)]


# name -> (restype, argtypes); every symbol include/winoconv.h declares
_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
_desc_p, _plan_p = ctypes.POINTER(ConvDesc), ctypes.POINTER(Plan)
_i64_5 = ctypes.POINTER(ctypes.c_int64)
SIGNATURES = {
    "wc_version": (ctypes.c_char_p, []),
    "wc_last_error": (ctypes.c_char_p, []),
    "wc_test_gemm_override": (_i, [_i, _i]),
    "wc_plan_dwm": (_i, [_i, _i, _i, c_int_p] + [c_int_p] * 8),
    "wc_plan_conv": (_i, [_desc_p, _plan_p]),
    "wc_conv_auto": (_i, [_desc_p]),
    "wc_conv_out_dims": (_i, [_desc_p, c_int_p, c_int_p]),
    "wc_padded_channels": (_i, [_i]),
    "wc_padded_channels8": (_i, [_i]),
    "wc_wino_split2d": (_i, [_vp, _vp] + [_i] * 10 + [_vp]),
    "wc_wino_split3d": (_i, [_vp, _vp] + [_i] * 13 + [_vp]),
    "wc_wino_concat2d": (_i, [_vp, _vp] + [_i] * 6 + [_vp]),
    "wc_wino_concat3d": (_i, [_vp, _vp] + [_i] * 7 + [_vp]),
    "wc_layout_copy": (_i, [_vp, _vp, _i, _i, ctypes.c_longlong, _i, _i, _vp]),
    "wc_filter_transform": (_i, [_desc_p, _plan_p, _vp, _i64_5, _vp, _vp]),
    "wc_input_transform": (_i, [_desc_p, _plan_p, _vp, _i, _vp, _vp]),
    "wc_batched_gemm": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "wc_output_transform": (_i, [_desc_p, _plan_p, _vp, _vp, _i, _vp, _vp]),
    "wc_conv_workspace_bytes": (_i, [_desc_p, ctypes.POINTER(_sz)]),
    "wc_conv_u_elems": (_i, [_desc_p, ctypes.POINTER(_sz)]),
    "wc_conv_forward": (_i, [_desc_p, _vp, _vp, _i64_5, _vp, _vp, _vp, _vp, _sz, _vp]),
    "wc_conv_forward_static": (_i, [_desc_p, _vp, _vp, _i64_5, _vp, _vp, _vp, _vp]),
    "wc_conv_backward_input_workspace_bytes": (_i, [_desc_p, ctypes.POINTER(_sz)]),
    "wc_conv_backward_input": (_i, [_desc_p, _vp, _vp, _i64_5, _vp, _vp, _sz, _vp]),
    "wc_conv_forward_timed": (_i, [_desc_p, _vp, _vp, _i64_5, _vp, _vp, _vp, _vp, _sz, _vp, ctypes.POINTER(ctypes.c_float)]),
    "wc_conv_backward_weight_workspace_bytes": (_i, [_desc_p, ctypes.POINTER(_sz)]),
    "wc_conv_backward_weight": (_i, [_desc_p, _vp, _vp, _vp, _i64_5, _vp, _sz, _vp]),
}

_lib = None


def _ext_make_args():
    """Paths the Makefile's `ext` target needs (torch, Python and pybind11 headers, the module suffix)."""
    import sysconfig
    import pybind11
    import torch
    return ["TORCH_DIR=%s" % os.path.dirname(torch.__file__), "PY_INC=%s" % sysconfig.get_paths()["include"],
            "PYBIND_INC=%s" % pybind11.get_include(), "EXT_SUFFIX=%s" % sysconfig.get_config_var("EXT_SUFFIX")]


def ext_path():
    import sysconfig
    return os.path.join(_HERE, "MakePytorchBackend" + sysconfig.get_config_var("EXT_SUFFIX"))


def build(jobs=8, verbose=False):
    """Compile every HIP source for gfx950 into libwinoconv_hip.so (hipcc) and the host layer, the
    pybind11 module MakePytorchBackend (g++), always from scratch."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.run(["make", "-C", CSRC, "clean"] + _ext_make_args(), check=True, stdout=out)
    subprocess.run(["make", "-C", CSRC, "-j%d" % jobs], check=True, stdout=out)
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("build finished without producing %s" % LIB_PATH)
    subprocess.run(["make", "-C", CSRC, "ext"] + _ext_make_args(), check=True, stdout=out)
    if not os.path.exists(ext_path()):
        raise RuntimeError("build finished without producing %s" % ext_path())
    return LIB_PATH


def load():
    """Load the shared library (built beforehand) and attach the C signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "%s is missing: build it with pytorch_winoconv_amd.build() (needs hipcc); "
            "there is no fallback implementation" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if a declared symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class WinoconvError(RuntimeError):
    pass


def check(rc):
    """Turn a wc_status into a Python exception (the reference calls exit(-1) instead:
    src/winograd_conv.cpp:80-84,116-126)."""
    if rc == WC_OK:
        return
    msg = load().wc_last_error().decode()
    if rc == WC_ERR_BAD_ARG:
        raise ValueError(msg)
    if rc == WC_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise WinoconvError("winoconv error %d: %s" % (rc, msg))
