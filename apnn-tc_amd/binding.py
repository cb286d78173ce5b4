"""ctypes binding of include/apnn_tc.h.  Loading fails loudly when the library has not been built."""
import ctypes
import os
import subprocess

__all__ = [
    "LIB_PATH", "lib", "build", "Epilogue", "GemmDesc", "ConvDesc", "Plan", "ApnnError", "check",
    "KERNEL_VALU_TILE", "KERNEL_VALU_DIRECT", "KERNEL_MFMA_FP4", "KERNEL_MFMA_I8", "KERNEL_PATCH_FP4",
    "EPI_INT32", "EPI_LOWBITS", "EPI_BN", "POOL_NONE", "POOL_AVG2X2", "POOL_MAX2X2",
    "PATH_AUTO", "PATH_VALU", "PATH_MFMA", "PATH_MFMA_I8", "PATH_MFMA_PATCH", "PATH_MFMA_XS", "KERNEL_MFMA_FP4_XS", "WEIGHT_UNSIGNED", "WEIGHT_SYMMETRIC",
    "OK", "EINVAL", "ENULL", "EALIGN", "EUNSUPPORTED", "DECLARED_SYMBOLS",
]

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "lib", "libapnn_tc.so")

EPI_INT32, EPI_LOWBITS, EPI_BN = 0, 1, 2
POOL_NONE, POOL_AVG2X2, POOL_MAX2X2 = 0, 1, 2
PATH_AUTO, PATH_VALU, PATH_MFMA, PATH_MFMA_I8, PATH_MFMA_PATCH, PATH_MFMA_XS = 0, 1, 2, 3, 4, 5
WEIGHT_UNSIGNED, WEIGHT_SYMMETRIC = 0, 1
OK, EINVAL, ENULL, EALIGN, EUNSUPPORTED = 0, -1, -2, -3, -4

_vp = ctypes.c_void_p
_ci = ctypes.c_int


class Epilogue(ctypes.Structure):
    _fields_ = [("mode", _ci), ("out_bits", _ci), ("pool", _ci),
                ("thresholds", _vp), ("flip", _vp), ("residual", _vp), ("save_acc", _vp),
                ("residual_planes", _vp), ("residual_bits", _ci), ("residual_scale", _ci)]


class GemmDesc(ctypes.Structure):
    _fields_ = [("W", _vp), ("X", _vp), ("D", _vp), ("M", _ci), ("N", _ci), ("K", _ci),
                ("wb", _ci), ("xb", _ci), ("weight_mode", _ci), ("epi", Epilogue), ("path", _ci)]


class ConvDesc(ctypes.Structure):
    _fields_ = [("W", _vp), ("X", _vp), ("O", _vp), ("batch", _ci), ("H", _ci), ("Wd", _ci),
                ("cin_pad", _ci), ("COUT", _ci), ("R", _ci), ("S", _ci), ("stride", _ci), ("pad", _ci),
                ("halo", _ci), ("wb", _ci), ("xb", _ci), ("weight_mode", _ci), ("epi", Epilogue),
                ("path", _ci)]


class Plan(ctypes.Structure):
    _fields_ = [("path", _ci), ("kernel", _ci), ("tile", _ci), ("tile_rows", _ci), ("tile_cols", _ci),
                ("split_k", _ci), ("workgroups", ctypes.c_longlong), ("patch_pixels", _ci), ("fp4_exact", _ci)]


KERNEL_VALU_TILE, KERNEL_VALU_DIRECT, KERNEL_MFMA_FP4, KERNEL_MFMA_I8, KERNEL_PATCH_FP4, KERNEL_MFMA_FP4_XS = 0, 1, 2, 3, 4, 5

_GEMM_SIG = [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _ci, _vp]
_CONV_SIG = [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp]

_GEMM_NAMES = ["apmm_w1a2", "apmm_w1a3", "apmm_w1a4", "apmm_w2a2", "apmm_w1a8", "apmm_w2a8", "apmm_w4a4", "apmm_w1a1",
               "apmm_w1a2_decompose", "apmm_w1a3_decompose", "apmm_w1a4_decompose", "apmm_w2a2_decompose"]
_CONV_NAMES = ["apconv_w1a2", "apconv_w1a3", "apconv_w1a4", "apconv_w2a2", "apconv_w1a5", "apconv_w2a6",
               "apconv_w1a8", "apconv_w2a8", "APConv_w2a8_pack", "APConv_w2a8_pack_pool",
               "APConv_w1a2_pack", "APConv_w1a3_pack", "APConv_w1a4_pack", "APConv_w2a2_pack",
               "APConv_w1a2_pack_pool", "APConv_w2a2_pack_pool"]
DECLARED_SYMBOLS = _GEMM_NAMES + _CONV_NAMES + ["apnn_gemm", "apnn_conv", "apnn_pack_bits", "apnn_pack_bits_fc_hidden", "apnn_conv_i8_bn",
                                                "apnn_pool_pack", "apnn_unpack_sum", "apnn_fc_i8",
                                                "apnn_conv_i8_bn_pack", "apnn_pool_planes", "apnn_quantize_pack", "apnn_fold_bn", "apnn_conv_pair",
                                                "apnn_gemm_plan", "apnn_conv_plan", "apnn_quantize_pack_u8", "apnn_binarize_pack",
                                                "apnn_residual_prepare",
                                                "apnn_device_error", "apnn_device_cus", "apnn_version"]


class ApnnError(RuntimeError):
    pass


def check(rc, what=""):
    if rc != 0:
        kind = {EINVAL: "APNN_EINVAL", ENULL: "APNN_ENULL", EALIGN: "APNN_EALIGN",
                EUNSUPPORTED: "APNN_EUNSUPPORTED"}.get(rc, "hipError_t %d" % rc)
        raise ApnnError("%s failed: %s" % (what or "apnn call", kind))


def build(force=True):
    """Compile libapnn_tc.so for gfx950 with hipcc (cross-compiles without a GPU)."""
    cmd = ["make", "-C", os.path.join(PKG_DIR, "csrc"), "-j8"]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    return LIB_PATH


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        # When PyTorch supplies the device buffers, its bundled HIP runtime has to be the one this
        # library binds to (same SONAME): two runtimes in one process do not share allocations.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        if not os.path.exists(LIB_PATH):
            raise ApnnError("%s is missing: run `make -C apnn-tc_amd/csrc` (or __graft_entry__.build())" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for n in _GEMM_NAMES:
            getattr(L, n).argtypes = _GEMM_SIG
            getattr(L, n).restype = _ci
        for n in _CONV_NAMES:
            getattr(L, n).argtypes = _CONV_SIG
            getattr(L, n).restype = _ci
        L.apnn_gemm.argtypes = [ctypes.POINTER(GemmDesc), _vp]
        L.apnn_gemm.restype = _ci
        L.apnn_conv.argtypes = [ctypes.POINTER(ConvDesc), _vp]
        L.apnn_conv.restype = _ci
        L.apnn_gemm_plan.argtypes = [ctypes.POINTER(GemmDesc), ctypes.POINTER(Plan)]
        L.apnn_gemm_plan.restype = _ci
        L.apnn_conv_plan.argtypes = [ctypes.POINTER(ConvDesc), ctypes.POINTER(Plan)]
        L.apnn_conv_plan.restype = _ci
        L.apnn_conv_pair.argtypes = [ctypes.POINTER(ConvDesc), ctypes.POINTER(ConvDesc), _vp]
        L.apnn_conv_pair.restype = _ci
        L.apnn_pack_bits.argtypes = [_vp, _vp, _ci, _ci, _ci, _ci, _vp]
        L.apnn_pack_bits.restype = _ci
        L.apnn_pack_bits_fc_hidden.argtypes = [_vp, _vp, _ci, _ci, _ci, _ci, _vp]
        L.apnn_pack_bits_fc_hidden.restype = _ci
        L.apnn_conv_i8_bn.argtypes = [_vp] * 5 + [_ci] * 11 + [_vp]
        L.apnn_conv_i8_bn.restype = _ci
        L.apnn_conv_i8_bn_pack.argtypes = [_vp] * 4 + [_ci] * 11 + [_vp]
        L.apnn_conv_i8_bn_pack.restype = _ci
        L.apnn_pool_planes.argtypes = [_vp, _vp] + [_ci] * 8 + [_vp]
        L.apnn_pool_planes.restype = _ci
        L.apnn_pool_pack.argtypes = [_vp, _vp] + [_ci] * 9 + [_vp]
        L.apnn_pool_pack.restype = _ci
        L.apnn_unpack_sum.argtypes = [_vp, _vp, ctypes.c_longlong] + [_ci] * 5 + [_vp]
        L.apnn_unpack_sum.restype = _ci
        L.apnn_fc_i8.argtypes = [_vp] * 6 + [_ci] * 3 + [_vp]
        L.apnn_fc_i8.restype = _ci
        L.apnn_quantize_pack.argtypes = [_vp, _vp, _ci, _ci, _ci, _ci, ctypes.c_float, ctypes.c_float, _vp]
        L.apnn_quantize_pack.restype = _ci
        L.apnn_quantize_pack_u8.argtypes = [_vp, _vp, _ci, _ci, _ci, _ci, _vp]
        L.apnn_quantize_pack_u8.restype = _ci
        L.apnn_binarize_pack.argtypes = [_vp, _vp, _ci, _ci, _ci, _vp]
        L.apnn_binarize_pack.restype = _ci
        L.apnn_residual_prepare.argtypes = [_vp, _vp] + [_ci] * 7 + [_vp]
        L.apnn_residual_prepare.restype = _ci
        L.apnn_fold_bn.argtypes = [_vp] * 4 + [ctypes.c_float] * 3 + [_ci, _ci, _vp, _vp]
        L.apnn_fold_bn.restype = _ci
        L.apnn_device_error.argtypes = [ctypes.POINTER(_ci), _vp]
        L.apnn_device_error.restype = _ci
        L.apnn_device_cus.argtypes = []
        L.apnn_device_cus.restype = _ci
        L.apnn_version.argtypes = []
        L.apnn_version.restype = ctypes.c_char_p
        _lib = L
    return _lib
