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
    assert L.apnn_pack_bits_fc_hidden(None, good, 4, 64, 128, 2, None) == A.ENULL
    assert L.apnn_pack_bits_fc_hidden(good, good, 4, 200, 128, 2, None) == A.EINVAL


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
                   wb=1, xb=2, path=A.PATH_MFMA_I8 | ((0 + 1) << 8))
    assert L.apnn_conv(ctypes.byref(c), None) == A.EUNSUPPORTED          # int8 convolution has no 256x256 tile
    c.wb, c.xb, c.path = 1, 8, A.PATH_MFMA_I8
    assert L.apnn_conv(ctypes.byref(c), None) == A.EUNSUPPORTED          # wide precisions: FP4 core only
    g = A.GemmDesc(W=good, X=good, D=good, M=64, N=128, K=128, wb=1, xb=2, path=A.PATH_MFMA | (1 << 8))
    assert L.apnn_gemm(ctypes.byref(g), None) == A.EUNSUPPORTED          # FP4 GEMM has no 256x256 tile
    g.wb, g.xb, g.path = 3, 5, A.PATH_MFMA
    assert L.apnn_gemm(ctypes.byref(g), None) == A.EUNSUPPORTED          # no matrix-core kernel for w3a5
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


def _plan_gemm(**kw):
    g = A.GemmDesc(W=0x1000, X=0x1000, D=0x1000, **kw)
    plan = A.Plan()
    rc = A.lib().apnn_gemm_plan(ctypes.byref(g), ctypes.byref(plan))
    return rc, plan


def _plan_conv(**kw):
    c = A.ConvDesc(W=0x1000, X=0x1000, O=0x1000, **kw)
    plan = A.Plan()
    rc = A.lib().apnn_conv_plan(ctypes.byref(c), ctypes.byref(plan))
    return rc, plan


def test_fp4_accumulation_guard():
    """The FP4 matrix-core kernels accumulate in fp32, exact while K*(2^w-1)*(2^a-1) < 2^24.  Beyond that
    bound the library's own choice moves to the int8 core (int32 accumulate) and a pinned FP4 path is
    refused -- decided on the host, before any launch."""
    L = A.lib()
    for wb, xb in [(1, 2), (1, 3), (1, 4), (2, 2)]:
        span = (2 ** wb - 1) * (2 ** xb - 1)
        k_ok = ((2 ** 24 - 1) // span) // 128 * 128              # largest exact K
        k_bad = k_ok + 128
        assert k_ok * span < 2 ** 24 <= k_bad * span
        rc, plan = _plan_gemm(M=512, N=512, K=k_ok, wb=wb, xb=xb, path=A.PATH_AUTO)
        assert rc == 0 and plan.kernel == A.KERNEL_MFMA_FP4 and plan.fp4_exact == 1
        rc, plan = _plan_gemm(M=512, N=512, K=k_bad, wb=wb, xb=xb, path=A.PATH_AUTO)
        assert rc == 0 and plan.kernel == A.KERNEL_MFMA_I8 and plan.fp4_exact == 0
        rc, _ = _plan_gemm(M=512, N=512, K=k_bad, wb=wb, xb=xb, path=A.PATH_MFMA)
        assert rc == A.EUNSUPPORTED
        g = A.GemmDesc(W=0x1000, X=0x1000, D=0x1000, M=512, N=512, K=k_bad, wb=wb, xb=xb, path=A.PATH_MFMA)
        assert L.apnn_gemm(ctypes.byref(g), None) == A.EUNSUPPORTED
        rc, plan = _plan_gemm(M=512, N=512, K=k_bad, wb=wb, xb=xb, path=A.PATH_VALU)
        assert rc == 0 and plan.kernel == A.KERNEL_VALU_TILE
    # convolution: a 1x1 filter over 2^20 stored channels, w1a4: 2^20 * 15 < 2^24 holds, 9 taps do not
    geo = dict(batch=64, H=8, Wd=8, COUT=512, stride=1, halo=0, wb=1, xb=4)
    rc, plan = _plan_conv(cin_pad=2 ** 20, R=1, S=1, pad=0, path=A.PATH_AUTO, **geo)
    assert rc == 0 and plan.kernel == A.KERNEL_MFMA_FP4
    rc, plan = _plan_conv(cin_pad=2 ** 18, R=3, S=3, pad=1, path=A.PATH_AUTO, **geo)
    assert rc == 0 and plan.kernel == A.KERNEL_MFMA_I8 and plan.fp4_exact == 0
    for pinned in (A.PATH_MFMA, A.PATH_MFMA_PATCH):
        rc, _ = _plan_conv(cin_pad=2 ** 18, R=3, S=3, pad=1, path=pinned, **geo)
        assert rc == A.EUNSUPPORTED
    # wide precisions have no int8 kernel: beyond the bound the VALU path serves them
    rc, plan = _plan_gemm(M=512, N=512, K=2 ** 17, wb=1, xb=8, path=A.PATH_AUTO)
    assert rc == 0 and plan.kernel == A.KERNEL_VALU_TILE and plan.fp4_exact == 0
    rc, plan = _plan_gemm(M=512, N=512, K=2 ** 15, wb=1, xb=8, path=A.PATH_AUTO)
    assert rc == 0 and plan.kernel == A.KERNEL_MFMA_FP4


def test_int32_accumulator_range_guard():
    """Results are int32: a request whose largest possible magnitude -- K x weight range x activation
    range, doubled for symmetric weights, plus the largest scaled shortcut code -- reaches 2^31 would wrap
    and is refused with APNN_EINVAL on every path, by the plan call and by the launching call alike."""
    L = A.lib()
    for wb, xb in [(8, 8), (4, 4), (2, 8), (1, 8)]:
        span = (2 ** wb - 1) * (2 ** xb - 1)
        k_ok = ((2 ** 31 - 1) // span) // 128 * 128
        k_bad = k_ok + 128
        assert k_ok * span < 2 ** 31 <= k_bad * span
        for path in (A.PATH_AUTO, A.PATH_VALU):
            rc, _ = _plan_gemm(M=64, N=64, K=k_ok, wb=wb, xb=xb, path=path)
            assert rc == 0, (wb, xb, path)
            rc, _ = _plan_gemm(M=64, N=64, K=k_bad, wb=wb, xb=xb, path=path)
            assert rc == A.EINVAL, (wb, xb, path)
        g = A.GemmDesc(W=0x1000, X=0x1000, D=0x1000, M=64, N=64, K=k_bad, wb=wb, xb=xb)
        assert L.apnn_gemm(ctypes.byref(g), None) == A.EINVAL
        # symmetric weights double the range
        k_sym = ((2 ** 31 - 1) // (2 * span)) // 128 * 128
        rc, _ = _plan_gemm(M=64, N=64, K=k_sym, wb=wb, xb=xb, weight_mode=A.WEIGHT_SYMMETRIC)
        assert rc == 0
        rc, _ = _plan_gemm(M=64, N=64, K=k_sym + 128, wb=wb, xb=xb, weight_mode=A.WEIGHT_SYMMETRIC)
        assert rc == A.EINVAL
    # the w8a8 K = 131072 request (largest magnitude 8.5e9) that used to be accepted
    rc, _ = _plan_gemm(M=64, N=64, K=131072, wb=8, xb=8)
    assert rc == A.EINVAL
    # a scaled shortcut code counts: w1a2, K = 1024 leaves room for 2^31 - 1 - 3072
    epi = A.Epilogue(mode=A.EPI_BN, out_bits=2, thresholds=0x1000, residual_planes=0x1000, residual_bits=2)
    epi.residual_scale = (2 ** 31 - 1 - 3072) // 3
    rc, _ = _plan_gemm(M=64, N=64, K=1024, wb=1, xb=2, epi=epi)
    assert rc == 0
    epi.residual_scale += 1
    rc, _ = _plan_gemm(M=64, N=64, K=1024, wb=1, xb=2, epi=epi)
    assert rc == A.EINVAL
    # convolution: 9 taps x 2^17 stored channels x 255 x 255 is far beyond; 9 x 128 x 255 x 255 is not
    geo = dict(batch=1, H=8, Wd=8, COUT=64, R=3, S=3, stride=1, pad=1, halo=0, wb=8, xb=8)
    rc, _ = _plan_conv(cin_pad=128, **geo)
    assert rc == 0
    rc, _ = _plan_conv(cin_pad=2 ** 17, **geo)
    assert rc == A.EINVAL
    c = A.ConvDesc(W=0x1000, X=0x1000, O=0x1000, cin_pad=2 ** 17, **geo)
    assert L.apnn_conv(ctypes.byref(c), None) == A.EINVAL


def test_matrix_core_kernels_refuse_operands_beyond_32_bit_offsets():
    """The matrix-core kernels of the FP4 / int8 family address operand rows with 32-bit byte offsets
    through buffer descriptors: a request whose operand plane reaches 4 GiB, or whose filter is beyond the
    kernels' 24-bit index arithmetic, is refused when the family is pinned and served by the VALU kernels
    (64-bit addressing) when the library chooses."""
    # GEMM: one X plane of N x K / 8 bytes = 4 GiB
    big = dict(M=256, N=1 << 17, K=1 << 18, wb=1, xb=2)
    rc, plan = _plan_gemm(path=A.PATH_AUTO, **big)
    assert rc == 0 and plan.kernel == A.KERNEL_VALU_TILE
    for pinned in (A.PATH_MFMA, A.PATH_MFMA_I8):
        rc, _ = _plan_gemm(path=pinned, **big)
        assert rc == A.EUNSUPPORTED
    rc, plan = _plan_gemm(path=A.PATH_AUTO, M=256, N=1 << 16, K=1 << 18, wb=1, xb=2)   # 2 GiB per plane
    assert rc == 0 and plan.kernel in (A.KERNEL_MFMA_FP4, A.KERNEL_MFMA_I8)
    # convolution: a 41 x 41 filter (taps * S >= 65536) is outside the multiply-shift tap decode
    geo = dict(batch=4, H=64, Wd=64, cin_pad=128, COUT=256, stride=1, halo=0, wb=1, xb=2)
    rc, plan = _plan_conv(R=41, S=41, pad=20, path=A.PATH_AUTO, **geo)
    assert rc == 0 and plan.kernel == A.KERNEL_VALU_TILE
    rc, _ = _plan_conv(R=41, S=41, pad=20, path=A.PATH_MFMA, **geo)
    assert rc == A.EUNSUPPORTED
    rc, plan = _plan_conv(R=11, S=11, pad=5, path=A.PATH_AUTO, **geo)
    assert rc == 0 and plan.kernel == A.KERNEL_MFMA_FP4


def test_plan_reports_the_dispatchers_choices():
    """Without a device the dispatcher assumes 256 compute units: the choices for the benchmark shapes."""
    rc, plan = _plan_gemm(M=64, N=1024, K=1024, wb=1, xb=2, path=A.PATH_AUTO)
    assert rc == 0 and plan.kernel == A.KERNEL_VALU_DIRECT and plan.path == A.PATH_VALU
    rc, plan = _plan_gemm(M=8192, N=8192, K=8192, wb=1, xb=2, path=A.PATH_AUTO)
    assert rc == 0 and plan.kernel == A.KERNEL_MFMA_FP4 and (plan.tile_rows, plan.tile_cols) == (256, 128)
    assert plan.workgroups == 32 * 64
    rc, plan = _plan_conv(batch=1, H=16, Wd=16, cin_pad=1024, COUT=1024, R=3, S=3, stride=1, pad=1, halo=1, wb=1, xb=2,
                          path=A.PATH_AUTO)
    assert rc == 0 and plan.kernel == A.KERNEL_MFMA_FP4 and plan.split_k == 4
    rc, plan = _plan_conv(batch=64, H=56, Wd=56, cin_pad=64, COUT=64, R=3, S=3, stride=1, pad=1, halo=0, wb=1, xb=2,
                          path=A.PATH_AUTO)
    assert rc == 0 and plan.kernel == A.KERNEL_PATCH_FP4 and plan.patch_pixels > 0
    # per-precision tile rules on the 16x16 batch-16 sweep (tile shape and split-K factor as measured fastest)
    def conv16(C, wb, xb):
        rc, pl = _plan_conv(batch=16, H=16, Wd=16, cin_pad=C, COUT=C, R=3, S=3, stride=1, pad=1, halo=1, wb=wb, xb=xb,
                            path=A.PATH_AUTO)
        assert rc == 0 and pl.kernel == A.KERNEL_MFMA_FP4
        return (pl.tile_rows, pl.tile_cols, pl.split_k)
    assert conv16(1024, 1, 2) == (128, 128, 2)      # one 128x128 tile per compute unit: two wave groups
    assert conv16(896, 1, 2) == (32, 64, 4)         # 7/8 of the units would get a tile: 32x64 split-K is ahead
    assert conv16(896, 2, 2) == (128, 128, 2)       # two weight planes: the two-wave-group tile from 3/4
    assert conv16(640, 2, 2) == (32, 64, 4)
    assert conv16(512, 1, 4) == (32, 128, 4)        # four activation planes, all work-groups resident at once
    assert conv16(512, 1, 2) == (32, 64, 4)
    assert conv16(128, 1, 4) == (32, 32, 4)         # 512 blocks of 32x32 with five planes in all
    assert conv16(128, 1, 2) == (32, 64, 4)
    # the kernel that expands operands while staging is reachable by pinning only
    rc, plan = _plan_gemm(M=8192, N=8192, K=8192, wb=1, xb=4, path=A.PATH_AUTO)
    assert rc == 0 and plan.kernel == A.KERNEL_MFMA_FP4 and plan.path == A.PATH_MFMA
    rc, plan = _plan_gemm(M=8192, N=8192, K=8192, wb=1, xb=4, path=A.PATH_MFMA_XS)
    assert rc == 0 and plan.kernel == A.KERNEL_MFMA_FP4_XS
    assert A.lib().apnn_gemm_plan(None, ctypes.byref(A.Plan())) == A.ENULL
    g = A.GemmDesc(W=0x1000, X=0x1000, D=0x1000, M=64, N=64, K=128, wb=1, xb=2)
    assert A.lib().apnn_gemm_plan(ctypes.byref(g), None) == A.ENULL


def test_patch_capacity_bounds_every_tile():
    """The patch-resident convolution kernel stages, per work-group, the contiguous range of padded-frame
    pixels that its tile of consecutive output rows reads; the host sizes that range from a closed-form
    bound.  Brute force over every tile start of many geometries: the bound is never below the true span
    (a tile whose span exceeded it would be dropped by the kernel)."""
    tiles = [(128, 128), (256, 64), (64, 128), (128, 64), (64, 64)]
    geoms = [  # batch H W R S stride pad pool
        (3, 16, 16, 3, 3, 1, 1, 0), (2, 56, 56, 3, 3, 1, 1, 0), (5, 7, 7, 3, 3, 1, 1, 0), (4, 14, 14, 3, 3, 2, 1, 0),
        (3, 28, 28, 1, 1, 2, 0, 0), (2, 13, 11, 5, 5, 1, 2, 0), (2, 12, 20, 3, 3, 1, 1, 1), (3, 8, 8, 5, 3, 1, 1, 2),
        (9, 5, 6, 3, 3, 1, 1, 0), (2, 30, 9, 3, 1, 1, 0, 0), (7, 6, 6, 3, 3, 1, 1, 1), (2, 24, 24, 5, 5, 2, 2, 1),
        (70, 3, 3, 3, 3, 1, 1, 0), (1, 40, 6, 1, 5, 1, 2, 0), (6, 10, 10, 3, 3, 1, 0, 1),
    ]
    checked = 0
    for (batch, H, W, R, S, stride, pad, pool) in geoms:
        PHs, PWs = H + 2 * pad, W + 2 * pad
        Ho, Wo = (PHs - R) // stride + 1, (PWs - S) // stride + 1
        if pool and (Ho % 2 or Wo % 2):
            continue
        # padded-frame base of every output row, in the kernel's row order
        bases = []
        if not pool:
            for b in range(batch):
                for oy in range(Ho):
                    for ox in range(Wo):
                        bases.append((b * PHs + oy * stride) * PWs + ox * stride)
        else:
            for b in range(batch):
                for py in range(Ho // 2):
                    for px in range(Wo // 2):
                        for sub in range(4):
                            oy, ox = 2 * py + (sub >> 1), 2 * px + (sub & 1)
                            bases.append((b * PHs + oy * stride) * PWs + ox * stride)
        for t, (tr, tc) in enumerate(tiles):
            epi = A.Epilogue()
            if pool:
                epi.mode, epi.out_bits, epi.pool = A.EPI_LOWBITS, 2, pool
            rc, plan = _plan_conv(batch=batch, H=H, Wd=W, cin_pad=64, COUT=64, R=R, S=S, stride=stride, pad=pad, halo=0,
                                  wb=1, xb=2, epi=epi, path=A.PATH_MFMA_PATCH | ((t + 1) << 8))
            if rc == A.EUNSUPPORTED:      # patch or filter block does not fit in LDS
                continue
            assert rc == 0 and (plan.tile_rows, plan.tile_cols) == (tr, tc)
            worst = 0
            for a0 in range(0, len(bases), tr):
                seg = bases[a0:a0 + tr]
                worst = max(worst, max(seg) - min(seg) + (R - 1) * PWs + S)
            assert worst <= plan.patch_pixels <= 1024, (batch, H, W, R, S, stride, pad, pool, t, worst, plan.patch_pixels)
            checked += 1
    assert checked >= 40
