"""Host-only checks of the C ABI: the library loads, exports every symbol the header declares,
and rejects out-of-contract arguments with an error code instead of aborting.  No compute calls."""
import ctypes
import os
import re

import pytest

import pkg

A = pkg.load()
ROOT = pkg.ROOT


def test_library_exports_every_declared_symbol():
    L = A.lib()
    header = open(os.path.join(ROOT, "include", "apnn_tc.h")).read()
    declared = set(re.findall(r"^(?:int|const char \*)\s*\*?(\w+)\(", header, flags=re.M))
    assert declared == set(A.DECLARED_SYMBOLS), declared ^ set(A.DECLARED_SYMBOLS)
    for name in declared:
        assert hasattr(L, name), name
    assert b"gfx950" in L.apnn_version()


def test_struct_sizes_match_header_layout():
    # 3 ints (+pad) + 4 pointers; keeps the ctypes mirror honest about field order
    assert ctypes.sizeof(A.Epilogue) == 16 + 5 * 8 + 8
    assert A.GemmDesc.epi.offset == 3 * 8 + 6 * 4
    assert A.ConvDesc.epi.offset == 3 * 8 + 13 * 4 + 4


def test_named_entry_points_reject_bad_arguments():
    L = A.lib()
    good = 0x1000  # never dereferenced: every call below must fail validation first
    assert L.apmm_w1a2(None, good, good, 64, 128, 128, 1, 2, None) == A.ENULL
    assert L.apmm_w1a2(good, good + 4, good, 64, 128, 128, 1, 2, None) == A.EALIGN
    assert L.apmm_w1a2(good, good, good, 64, 128, 100, 1, 2, None) == A.EINVAL      # K % 128
    assert L.apmm_w1a2(good, good, good, 0, 128, 128, 1, 2, None) == A.EINVAL
    assert L.apmm_w1a2(good, good, good, 64, 128, 128, 2, 2, None) == A.EINVAL      # wrong bit widths
    assert L.apmm_w1a2_decompose(good, good, good, 64, 100, 128, 1, 2, None) == A.EINVAL  # N % 32
    assert L.apconv_w1a2(good, good, good, 16, 16, 96, 128, None) == A.EINVAL       # CIN % 128
    assert L.APConv_w1a2_pack(good, good, good, 16, 16, 128, 100, None) == A.EINVAL  # COUT % 32
    assert L.APConv_w1a2_pack_pool(good, good, good, 15, 16, 128, 128, None) == A.EINVAL  # odd height
    assert L.apnn_pack_bits(None, good, 4, 64, 128, 2, None) == A.ENULL
    assert L.apnn_pack_bits(good, good, 4, 200, 128, 2, None) == A.EINVAL


def test_descriptor_entry_points_reject_bad_arguments():
    L = A.lib()
    good = 0x1000
    assert L.apnn_gemm(None, None) == A.ENULL
    d = A.GemmDesc(W=good, X=good, D=good, M=64, N=128, K=128, wb=1, xb=2)
    d.epi.mode = 7
    assert L.apnn_gemm(ctypes.byref(d), None) == A.EINVAL
    d.epi.mode = A.EPI_BN
    d.epi.out_bits = 2
    assert L.apnn_gemm(ctypes.byref(d), None) == A.ENULL                            # thresholds missing
    d.epi.mode = A.EPI_INT32
    d.epi.pool = A.POOL_AVG2X2
    assert L.apnn_gemm(ctypes.byref(d), None) == A.EINVAL                           # pooling is conv-only
    c = A.ConvDesc(W=good, X=good, O=good, batch=1, H=8, Wd=8, cin_pad=48, COUT=64, R=3, S=3,
                   stride=1, pad=1, wb=1, xb=2)
    assert L.apnn_conv(ctypes.byref(c), None) == A.EINVAL                           # cin_pad % 32
    c.cin_pad = 64
    c.R = 11
    c.pad = 0
    assert L.apnn_conv(ctypes.byref(c), None) == A.EINVAL                           # filter larger than image


def test_nn_library_exports_every_declared_symbol():
    L = A.nn_lib()
    header = open(os.path.join(ROOT, "include", "apnn_nn.h")).read()
    declared = set(re.findall(r"^(?:int|void|apnn_net \*)\s*\*?(apnn_\w+)\(", header, flags=re.M))
    assert declared == set(A.NN_DECLARED_SYMBOLS), declared ^ set(A.NN_DECLARED_SYMBOLS)
    for name in declared:
        assert hasattr(L, name), name
    assert L.apnn_net_layer_count(None) == 0
    assert L.apnn_net_forward(None, None, None, None) == A.ENULL
    assert L.apnn_net_layer(None, 0, None) == A.ENULL


def test_edge_layer_entry_points_reject_bad_arguments():
    L = A.lib()
    good = 0x1000
    assert L.apnn_conv_i8_bn(None, good, good, good, None, 1, 8, 8, 3, 64, 7, 7, 2, 3, 2, 0, None) == A.ENULL
    assert L.apnn_conv_i8_bn(good, good, None, good, None, 1, 8, 8, 3, 64, 7, 7, 2, 3, 2, 0, None) == A.ENULL
    assert L.apnn_conv_i8_bn(good, good, good, good, None, 1, 8, 8, 3, 64, 7, 7, 2, 3, 9, 0, None) == A.EINVAL
    assert L.apnn_pool_pack(good, good, 1, 8, 8, 64, 100, 2, 3, 2, 1, None) == A.EINVAL      # cpad % 32
    assert L.apnn_pool_pack(good, good, 1, 8, 8, 64, 64, 2, 3, 2, 3, None) == A.EINVAL       # pad >= window
    assert L.apnn_unpack_sum(good, None, 4, 1, 64, 64, 2, 0, None) == A.ENULL
    assert L.apnn_fc_i8(good, good, good, good, good, None, 0, 10, 64, None) == A.EINVAL


def test_combinations_that_are_not_built_are_reported():
    """Rejected before any device call, so this runs without a GPU."""
    L = A.lib()
    good = 0x1000
    c = A.ConvDesc(W=good, X=good, O=good, batch=1, H=8, Wd=8, cin_pad=128, COUT=64, R=3, S=3, stride=1, pad=1,
                   wb=1, xb=2, path=A.PATH_MFMA_I8)
    assert L.apnn_conv(ctypes.byref(c), None) == A.EUNSUPPORTED          # int8 core: GEMM entry points only
    g = A.GemmDesc(W=good, X=good, D=good, M=64, N=128, K=128, wb=1, xb=2, path=A.PATH_MFMA | (1 << 8))
    assert L.apnn_gemm(ctypes.byref(g), None) == A.EUNSUPPORTED          # FP4 GEMM has no 256x256 tile
    g.wb, g.xb, g.path = 3, 5, A.PATH_MFMA
    assert L.apnn_gemm(ctypes.byref(g), None) == A.EUNSUPPORTED          # matrix-core kernels: w1a2 / w1a3 / w1a4 / w2a2
    g.path = A.PATH_MFMA_PATCH
    assert L.apnn_gemm(ctypes.byref(g), None) == A.EUNSUPPORTED          # convolution only
    g.wb, g.xb, g.path = 9, 2, A.PATH_AUTO
    assert L.apnn_gemm(ctypes.byref(g), None) == A.EINVAL                # at most 8 planes per operand
    g.wb, g.xb, g.path = 1, 2, A.PATH_VALU | (9 << 8)
    assert L.apnn_gemm(ctypes.byref(g), None) == A.EINVAL                # no such tile


def test_fold_bn_matches_double_precision_brute_force():
    """apnn_fold_bn is host-only: thresholds + flip reproduce clamp(floor(y / step)) of the double-precision
    batch-norm for every accumulator value in a range (rising, falling and constant channels)."""
    import numpy as np
    import oracle_lib as O
    L = A.lib()
    rng = np.random.default_rng(77)
    C = 24
    for bits, step, in_scale in [(1, 0.5, 1.0), (2, 0.7, 0.25), (3, 0.31, 2.0), (4, 0.2, -1.0)]:
        gamma = (rng.uniform(0.3, 2.0, C) * rng.choice([-1.0, 1.0], C)).astype(np.float32)
        gamma[3] = 0.0
        beta = rng.uniform(-1, 1, C).astype(np.float32)
        mean = rng.uniform(-20, 20, C).astype(np.float32)
        var = rng.uniform(4, 900, C).astype(np.float32)
        eps = np.float32(1e-5)
        nt = 2 ** bits - 1
        thr = np.zeros((C, nt), np.int32)
        flip = np.zeros(C, np.uint8)
        p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
        rc = L.apnn_fold_bn(p(gamma), p(beta), p(mean), p(var), eps, in_scale, step, C, bits, p(thr), p(flip))
        assert rc == 0
        assert np.all(np.diff(thr.astype(np.int64), axis=1) >= 0)
        v = np.arange(-700, 700, dtype=np.int32)
        acc = np.repeat(v[:, None], C, axis=1)
        slope = gamma.astype(np.float64) / np.sqrt(var.astype(np.float64) + np.float64(eps))
        y = slope[None, :] * (acc.astype(np.float64) * np.float64(np.float32(in_scale)) - mean.astype(np.float64)[None, :]) \
            + beta.astype(np.float64)[None, :]
        expect = np.clip(np.floor(y / np.float64(np.float32(step))), 0, nt).astype(np.int32)
        # y >= k*step  <=>  floor(y/step) >= k  holds in exact arithmetic; skip values within rounding of a level
        q = O.bn_quantize(acc, None, thr, flip, bits)
        frac = y / np.float64(np.float32(step))
        safe = np.abs(frac - np.rint(frac)) > 1e-9
        assert np.array_equal(q[safe], expect[safe])
        assert flip[3] == 0 and set(np.unique(q[:, 3])) <= {int(expect[0, 3])}
    bad = np.zeros(4, np.float32)
    assert L.apnn_fold_bn(None, p(bad), p(bad), p(bad), eps, 1.0, 1.0, 4, 2, p(thr), p(flip)) == A.ENULL
    assert L.apnn_fold_bn(p(bad), p(bad), p(bad), p(bad), eps, 1.0, 0.0, 4, 2, p(thr), p(flip)) == A.EINVAL
