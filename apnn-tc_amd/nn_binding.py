"""ctypes binding of include/apnn_nn.h (libapnn_nn.so): whole networks built from the layer API."""
import ctypes
import os

from . import binding

__all__ = ["NN_LIB_PATH", "nn_lib", "LayerDesc", "NET_ALEXNET", "NET_RESNET18", "NET_VGG",
           "LAYER_INCONV_I8", "LAYER_CONV", "LAYER_FC", "LAYER_OUT_I8", "LAYER_IMAGE_QUANT", "NET_RESNET18_REFERENCE", "NN_DECLARED_SYMBOLS"]

NN_LIB_PATH = os.path.join(binding.PKG_DIR, "lib", "libapnn_nn.so")
NET_ALEXNET, NET_RESNET18, NET_VGG, NET_RESNET18_REFERENCE = 0, 1, 2, 3
LAYER_INCONV_I8, LAYER_CONV, LAYER_FC, LAYER_OUT_I8, LAYER_IMAGE_QUANT = 0, 1, 2, 3, 4
NN_DECLARED_SYMBOLS = ["apnn_net_create", "apnn_net_destroy", "apnn_net_forward", "apnn_net_forward_graph",
                       "apnn_net_layer_count", "apnn_net_layer", "apnn_net_bench", "apnn_nn_download"]

_ci, _vp = ctypes.c_int, ctypes.c_void_p


class LayerDesc(ctypes.Structure):
    _fields_ = ([("name", ctypes.c_char * 16)] +
                [(n, _ci) for n in ("kind", "batch", "in_h", "in_w", "in_c", "in_cpad", "out_h", "out_w", "out_c",
                                    "out_cpad", "R", "S", "stride", "pad", "pool_win", "pool_stride", "pool_pad",
                                    "a_bits", "w_bits", "out_bits", "shortcut_layer", "shortcut_scale",
                                    "global_pool_shift", "residual_layer", "residual_channels", "residual_pitch",
                                    "residual_pool", "save_residual")] +
                [(n, _vp) for n in ("input", "weights", "thresholds", "scale", "bias", "output", "residual_out")])


_lib = None


def nn_lib():
    global _lib
    if _lib is None:
        binding.lib()  # loads torch's HIP runtime first, then libapnn_tc.so
        if not os.path.exists(NN_LIB_PATH):
            raise binding.ApnnError("%s is missing: run `make -C apnn-tc_amd/csrc`" % NN_LIB_PATH)
        L = ctypes.CDLL(NN_LIB_PATH)
        L.apnn_net_create.argtypes = [_ci, _ci, ctypes.c_ulonglong, _ci]
        L.apnn_net_create.restype = _vp
        L.apnn_net_destroy.argtypes = [_vp]
        L.apnn_net_destroy.restype = None
        L.apnn_net_forward.argtypes = [_vp, _vp, _vp, _vp]
        L.apnn_net_forward.restype = _ci
        L.apnn_net_forward_graph.argtypes = [_vp, _vp, _vp, _vp]
        L.apnn_net_forward_graph.restype = _ci
        L.apnn_net_layer_count.argtypes = [_vp]
        L.apnn_net_layer_count.restype = _ci
        L.apnn_net_layer.argtypes = [_vp, _ci, ctypes.POINTER(LayerDesc)]
        L.apnn_net_layer.restype = _ci
        L.apnn_net_bench.argtypes = [_vp, _vp, _vp, _ci, _ci, _ci, _vp, ctypes.POINTER(ctypes.c_float),
                                     ctypes.POINTER(ctypes.c_double)]
        L.apnn_net_bench.restype = _ci
        L.apnn_nn_download.argtypes = [_vp, _vp, ctypes.c_ulonglong]
        L.apnn_nn_download.restype = _ci
        _lib = L
    return _lib
