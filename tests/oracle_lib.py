"""ctypes view of oracle/liboracle.so plus numpy helpers shared by the tests.

The oracle is the checker.  The product library never goes through this module.
"""
import ctypes
import json
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")

u32p = ctypes.POINTER(ctypes.c_uint32)
i32p = ctypes.POINTER(ctypes.c_int32)
u8p = ctypes.POINTER(ctypes.c_uint8)
i8p = ctypes.POINTER(ctypes.c_int8)


class ConvGeom(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in
                ("batch", "H", "W", "cwords", "cout", "R", "S", "stride", "pad", "halo", "wb", "xb", "sym_w")]


def _build():
    so = os.path.join(ORACLE_DIR, "liboracle.so")
    src = os.path.join(ORACLE_DIR, "apnn_oracle.c")
    if not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "-B"], stdout=subprocess.DEVNULL)
    return so


_lib = None


def lib():
    global _lib
    if _lib is None:
        L = ctypes.CDLL(_build())
        ci = ctypes.c_int
        L.oracle_gemm_literal.argtypes = [u32p, u32p, i32p, ci, ci, ci, ci, ci]
        L.oracle_gemm.argtypes = [u32p, u32p, i32p, ci, ci, ci, ci, ci, ci, ci]
        L.oracle_gemm_rows.argtypes = [u32p, u32p, i32p, ci, ci, ci, ci, ci, ci, ci, ci, ci]
        L.oracle_conv3x3_literal.argtypes = [u32p, u32p, i32p, ci, ci, ci, ci, ci, ci]
        L.oracle_conv.argtypes = [u32p, u32p, i32p, ctypes.POINTER(ConvGeom), ci]
        L.oracle_conv_out_h.argtypes = [ctypes.POINTER(ConvGeom)]
        L.oracle_conv_out_w.argtypes = [ctypes.POINTER(ConvGeom)]
        L.oracle_lowbits_pack.argtypes = [i32p, u32p, ci, ci, ci]
        L.oracle_avgpool2x2.argtypes = [i32p, i32p, ci, ci, ci, ci]
        L.oracle_maxpool2x2.argtypes = [i32p, i32p, ci, ci, ci, ci]
        L.oracle_bn_quantize.argtypes = [i32p, i32p, i32p, u8p, i32p, ci, ci, ci]
        L.oracle_pack_bits.argtypes = [u32p, u32p, ci, ci, ci, ci]
        L.oracle_quantize_val.argtypes = [ctypes.POINTER(ctypes.c_float), u32p, ctypes.c_longlong, ci, ctypes.c_float,
                                          ctypes.c_float]
        L.oracle_unpack_bits.argtypes = [u32p, u32p, ci, ci, ci, ci]
        L.oracle_conv_i8.argtypes = [i8p, i8p, i32p] + [ci] * 9
        L.oracle_fnv1a64.argtypes = [ctypes.c_void_p, ctypes.c_uint64]
        L.oracle_fnv1a64.restype = ctypes.c_uint64
        for f in ("oracle_gemm_literal", "oracle_gemm", "oracle_gemm_rows", "oracle_conv3x3_literal",
                  "oracle_conv", "oracle_lowbits_pack", "oracle_avgpool2x2", "oracle_maxpool2x2",
                  "oracle_bn_quantize", "oracle_pack_bits", "oracle_unpack_bits", "oracle_conv_i8", "oracle_quantize_val"):
            getattr(L, f).restype = None
        _lib = L
    return _lib


def _p(a, t):
    return a.ctypes.data_as(t) if a is not None else None


def c32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


# ---- thin numpy wrappers -------------------------------------------------------------------

def gemm_literal(W, X, M, N, K, wb, xb):
    D = np.empty((M, N), np.int32)
    lib().oracle_gemm_literal(_p(c32(W), u32p), _p(c32(X), u32p), _p(D, i32p), M, N, K, wb, xb)
    return D


def gemm(W, X, M, N, K, wb, xb, sym_w=0, nthreads=1):
    D = np.empty((M, N), np.int32)
    lib().oracle_gemm(_p(c32(W), u32p), _p(c32(X), u32p), _p(D, i32p), M, N, K, wb, xb, sym_w, nthreads)
    return D


def gemm_rows(W, X, M, N, K, wb, xb, m0, m1, sym_w=0, nthreads=1):
    D = np.zeros((M, N), np.int32)
    lib().oracle_gemm_rows(_p(c32(W), u32p), _p(c32(X), u32p), _p(D, i32p), M, N, K, wb, xb, sym_w, m0, m1, nthreads)
    return D[m0:m1]


def conv3x3_literal(Wt, X, H, Wd, CIN, COUT, wb, xb):
    O = np.empty((H, Wd, COUT), np.int32)
    lib().oracle_conv3x3_literal(_p(c32(Wt), u32p), _p(c32(X), u32p), _p(O, i32p), H, Wd, CIN, COUT, wb, xb)
    return O


def conv(Wt, X, *, batch, H, W, cwords, cout, R, S, stride, pad, halo, wb, xb, sym_w=0, nthreads=1):
    g = ConvGeom(batch, H, W, cwords, cout, R, S, stride, pad, halo, wb, xb, sym_w)
    Ho, Wo = lib().oracle_conv_out_h(g), lib().oracle_conv_out_w(g)
    O = np.empty((batch, Ho, Wo, cout), np.int32)
    lib().oracle_conv(_p(c32(Wt), u32p), _p(c32(X), u32p), _p(O, i32p), ctypes.byref(g), nthreads)
    return O


def lowbits_pack(acc, rows, cols, out_bit):
    acc = np.ascontiguousarray(acc, np.int32).reshape(rows, cols)
    out = np.empty((out_bit, rows, cols // 32), np.uint32)
    lib().oracle_lowbits_pack(_p(acc, i32p), _p(out, u32p), rows, cols, out_bit)
    return out


def avgpool2x2(x):
    x = np.ascontiguousarray(x, np.int32)
    B, H, W, C = x.shape
    out = np.empty((B, H // 2, W // 2, C), np.int32)
    lib().oracle_avgpool2x2(_p(x, i32p), _p(out, i32p), B, H, W, C)
    return out


def maxpool2x2(x):
    x = np.ascontiguousarray(x, np.int32)
    B, H, W, C = x.shape
    out = np.empty((B, H // 2, W // 2, C), np.int32)
    lib().oracle_maxpool2x2(_p(x, i32p), _p(out, i32p), B, H, W, C)
    return out


def bn_quantize(acc, resid, thr, flip, abits):
    acc = np.ascontiguousarray(acc, np.int32)
    rows, C = acc.reshape(-1, acc.shape[-1]).shape
    q = np.empty((rows, C), np.int32)
    resid_c = None if resid is None else np.ascontiguousarray(resid, np.int32)
    thr = np.ascontiguousarray(thr, np.int32)
    flip_c = None if flip is None else np.ascontiguousarray(flip, np.uint8)
    lib().oracle_bn_quantize(_p(acc, i32p), _p(resid_c, i32p), _p(thr, i32p), _p(flip_c, u8p), _p(q, i32p), rows, C, abits)
    return q.reshape(acc.shape)


def pack_bits(values, rows, C, cpad, bits):
    values = c32(values).reshape(rows, C)
    planes = np.empty((bits, rows, cpad // 32), np.uint32)
    lib().oracle_pack_bits(_p(values, u32p), _p(planes, u32p), rows, C, cpad, bits)
    return planes


def quantize_val(x, bits, min_v=-10.0, max_v=10.0):
    x = np.ascontiguousarray(x, np.float32)
    q = np.empty(x.shape, np.uint32)
    lib().oracle_quantize_val(x.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), _p(q, u32p), x.size, bits, min_v, max_v)
    return q


def unpack_bits(planes, rows, C, cpad, bits):
    planes = c32(planes)
    values = np.empty((rows, C), np.uint32)
    lib().oracle_unpack_bits(_p(planes, u32p), _p(values, u32p), rows, C, cpad, bits)
    return values


def conv_i8(Wt, X, stride, pad):
    X = np.ascontiguousarray(X, np.int8)
    Wt = np.ascontiguousarray(Wt, np.int8)
    B, H, W, C = X.shape
    cout, R, S, _ = Wt.shape
    Ho, Wo = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - S) // stride + 1
    O = np.empty((B, Ho, Wo, cout), np.int32)
    lib().oracle_conv_i8(_p(Wt, i8p), _p(X, i8p), _p(O, i32p), B, H, W, C, cout, R, S, stride, pad)
    return O


def fnv1a64(a):
    a = np.ascontiguousarray(a)
    return int(lib().oracle_fnv1a64(a.ctypes.data, a.nbytes))


# ---- independent numpy helpers (do not share code with the oracle) ---------------------------

def unpack_planes_lsb(planes):
    """[p][rows][words] uint32 bit-planes (bit k of word = element 32*word + k) -> [rows][32*words]
    int64 values sum_p 2^p * bit."""
    planes = np.asarray(planes, np.uint32)
    p, rows, words = planes.shape
    shifts = np.arange(32, dtype=np.uint32)
    bits = (planes[..., None] >> shifts) & 1                     # [p][rows][words][32]
    bits = bits.reshape(p, rows, words * 32).astype(np.int64)
    weights = (1 << np.arange(p, dtype=np.int64)).reshape(p, 1, 1)
    return (bits * weights).sum(0)


def gemm_column_sums(W, X, chunk=1024):
    """sum_m D[m][n] of the unsigned GEMM D = wvalue . xvalue^T, without forming D:
    (sum_m wvalue[m][:]) . xvalue[n][:].  Row chunks bound the memory; float64 products are exact here
    (every partial sum is far below 2^53)."""
    W, X = np.asarray(W, np.uint32), np.asarray(X, np.uint32)
    shifts = np.arange(32, dtype=np.uint32)

    def bits_of(plane_rows):                                        # [rows][words] -> [rows][32*words] uint8
        return ((plane_rows[..., None] >> shifts) & 1).astype(np.uint8).reshape(plane_rows.shape[0], -1)

    wsum = np.zeros(W.shape[2] * 32, np.int64)
    for p in range(W.shape[0]):
        for r0 in range(0, W.shape[1], chunk):
            wsum += bits_of(W[p, r0:r0 + chunk]).sum(0, dtype=np.int64) << p
    wsum_f = wsum.astype(np.float64)
    out = np.zeros(X.shape[1], np.float64)
    for p in range(X.shape[0]):
        for r0 in range(0, X.shape[1], chunk):
            out[r0:r0 + chunk] += (bits_of(X[p, r0:r0 + chunk]).astype(np.float64) @ wsum_f) * float(1 << p)
    return out.astype(np.int64)


def random_planes(rng, planes, rows, words):
    return rng.integers(0, 2 ** 32, size=(planes, rows, words), dtype=np.uint64).astype(np.uint32)


def golden_stream():
    return np.fromfile(os.path.join(GOLDEN_DIR, "glibc_rand_srand1.bin"), dtype="<u4")


def known_answers():
    with open(os.path.join(GOLDEN_DIR, "known_answers.json")) as f:
        return json.load(f)
