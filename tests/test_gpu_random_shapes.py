"""GPU parity on seeded random shapes: convolution geometry (filter R x S, stride, padding as a stored
halo or predicated, batch, stored channels, output channels), GEMM sizes, precision, weight mode,
epilogue (int32, BN-threshold or low-bit quantize, average / max pooling) and kernel path x pinned tile
are all drawn per case; the library's result through the C ABI must equal the CPU oracle's bit for bit.
A pinned path or tile that does not exist for a drawn shape answers APNN_EUNSUPPORTED / APNN_EINVAL and
the case is dropped; APNN_PATH_AUTO must take every case."""
import numpy as np
import pytest

import oracle_lib as O

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available(), "GPU tests need a device"
    return gpu_util


CONV_CHOICES = ([(1, t) for t in range(4)] + [(2, t) for t in (1, 2, 3, 4, 5, 7, 8, 9)] + [(3, t) for t in (1, 2, 3, 4, 7)] +
                [(4, t) for t in range(5)] + [(5, t) for t in (1, 2, 3, 7)] + [(p, None) for p in (0, 0, 0, 1, 2, 3, 4, 5)])
GEMM_CHOICES = ([(1, t) for t in range(5)] + [(2, t) for t in (1, 2, 3, 4, 5, 6, 9)] + [(3, t) for t in (1, 2, 6)] +
                [(5, t) for t in (1, 2, 3, 6)] + [(p, None) for p in (0, 0, 0, 0, 1, 2, 3, 5)])
CONV_COMBOS = [(1, 2), (1, 3), (1, 4), (2, 2)]
GEMM_COMBOS = CONV_COMBOS + [(1, 8), (2, 8), (4, 4), (1, 1), (3, 5), (2, 1)]


def _quantized(G, rng, acc2d, channels, mode, ob, keep):
    """Epilogue descriptor and the oracle's codes for accumulators acc2d [rows][channels] (pooling is
    applied by the caller through `pooled`)."""
    if mode == 1:
        span = max(1, int(np.abs(acc2d).max()))
        thr = np.sort(rng.integers(-span, span + 1, size=(channels, 2 ** ob - 1)), axis=1).astype(np.int32)
        flip = rng.integers(0, 2, size=channels).astype(np.uint8)
        d_thr, d_flip = G.to_dev(thr), G.to_dev(flip)
        keep += [d_thr, d_flip]
        return dict(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr, flip=d_flip), lambda a: O.bn_quantize(a, None, thr, flip, ob)
    return dict(mode=G.A.EPI_LOWBITS, out_bits=ob), lambda a: a & ((1 << ob) - 1)


@pytest.mark.parametrize("block", range(8))
def test_conv_random_shapes(G, block):
    ran = 0
    for i in range(60):
        rng = np.random.default_rng(710000 + 1000 * block + i)
        wb, xb = CONV_COMBOS[rng.integers(0, 4)]
        large = i % 6 == 5
        batch = int(rng.integers(1, 12 if large else 6))
        H, Wd = (int(rng.integers(4, 40)), int(rng.integers(4, 40))) if large else (int(rng.integers(1, 21)), int(rng.integers(1, 21)))
        cin_pad = int(rng.choice([64, 128, 256, 512] if large else [32, 64, 96, 128, 128, 160, 256, 384]))
        R = int(rng.choice([1, 2, 3, 3, 3, 5, 7]))
        S = R if rng.random() < 0.7 else int(rng.choice([1, 2, 3, 5]))
        stride = int(rng.choice([1, 1, 2, 3]))
        pad = int(rng.integers(0, max(R, S) // 2 + 1))
        halo = int(rng.random() < 0.3) if pad > 0 else 0
        mode = int(rng.choice([0, 0, 1, 2]))   # int32, int32, BN thresholds, low bits
        cout = int(rng.integers(1, 13 if large else 7)) * 32 if mode else int(rng.integers(1, 400 if large else 200))
        sym = int(rng.random() < 0.5)
        pool = int(rng.choice([0, 0, 1, 2])) if mode else 0
        ob = int(rng.integers(1, 5)) if mode else 0
        path, tile = CONV_CHOICES[rng.integers(0, len(CONV_CHOICES))]
        if H + 2 * pad < R or Wd + 2 * pad < S:
            continue
        Ho, Wo = (H + 2 * pad - R) // stride + 1, (Wd + 2 * pad - S) // stride + 1
        if pool and (Ho % 2 or Wo % 2):
            pool = 0
        case = dict(block=block, i=i, wb=wb, xb=xb, batch=batch, H=H, W=Wd, cin_pad=cin_pad, cout=cout, R=R, S=S,
                    stride=stride, pad=pad, halo=halo, sym=sym, mode=mode, pool=pool, ob=ob, path=path, tile=tile)
        Hs, Ws = (H + 2 * pad, Wd + 2 * pad) if halo else (H, Wd)
        X = O.random_planes(rng, xb, batch * Hs * Ws, cin_pad // 32)
        Wt = O.random_planes(rng, wb, cout * R * S, cin_pad // 32)
        kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=R, S=S, stride=stride, pad=pad, halo=halo, wb=wb, xb=xb)
        acc = O.conv(Wt, X, cwords=cin_pad // 32, sym_w=sym, nthreads=8, **kw)
        keep = []
        if mode == 0:
            epi, expect = None, acc.reshape(-1)
        else:
            args, quant = _quantized(G, rng, acc.reshape(-1, cout), cout, mode, ob, keep)
            epi = G.epilogue(pool=pool, **args)
            rows = batch * Ho * Wo if pool == 0 else batch * (Ho // 2) * (Wo // 2)
            if pool == 0:
                q = quant(acc.reshape(-1, cout))
            elif pool == 1:
                q = quant(O.avgpool2x2(acc).reshape(-1, cout))
            else:
                q = O.maxpool2x2(quant(acc.reshape(-1, cout)).reshape(acc.shape)).reshape(-1, cout)
            expect = O.lowbits_pack(q.astype(np.int32), rows, cout, ob).reshape(-1).view(np.int32)
        try:
            got = G.run_conv(Wt, X, cin_pad=cin_pad, sym=sym, epi=epi, path=path, tile=tile, **kw)
        except G.A.ApnnError:
            assert path != 0, "APNN_PATH_AUTO declined %r" % (case,)
            continue
        ran += 1
        assert got.shape == expect.shape and np.array_equal(got, expect), case
    assert ran >= 25


@pytest.mark.parametrize("block", range(6))
def test_gemm_random_shapes(G, block):
    ran = 0
    for i in range(80):
        rng = np.random.default_rng(810000 + 1000 * block + i)
        wb, xb = GEMM_COMBOS[rng.integers(0, len(GEMM_COMBOS))]
        M, N = int(rng.integers(1, 400)), int(rng.integers(1, 400))
        K = int(rng.integers(1, 10)) * 1024 if rng.random() < 0.2 else int(rng.integers(1, 40)) * 128
        mode = int(rng.choice([0, 0, 1, 2]))
        sym = int(rng.random() < 0.5)
        ob = int(rng.integers(1, 5)) if mode else 0
        if mode:
            N = (N + 31) // 32 * 32
        path, tile = GEMM_CHOICES[rng.integers(0, len(GEMM_CHOICES))]
        case = dict(block=block, i=i, wb=wb, xb=xb, M=M, N=N, K=K, mode=mode, sym=sym, ob=ob, path=path, tile=tile)
        W = O.random_planes(rng, wb, M, K // 32)
        X = O.random_planes(rng, xb, N, K // 32)
        acc = O.gemm(W, X, M, N, K, wb, xb, sym_w=sym, nthreads=8)
        keep = []
        if mode == 0:
            epi, expect = None, acc.reshape(-1)
        else:
            args, quant = _quantized(G, rng, acc, N, mode, ob, keep)
            epi = G.epilogue(**args)
            expect = O.lowbits_pack(quant(acc).astype(np.int32), M, N, ob).reshape(-1).view(np.int32)
        try:
            got = G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, epi=epi, path=path, tile=tile)
        except G.A.ApnnError:
            assert path != 0, "APNN_PATH_AUTO declined %r" % (case,)
            continue
        ran += 1
        assert got.shape == expect.shape and np.array_equal(got, expect), case
    assert ran >= 30


def _np_maxpool_codes(codes, win, stride, pad):
    B, H, W, C = codes.shape
    Ho, Wo = (H + 2 * pad - win) // stride + 1, (W + 2 * pad - win) // stride + 1
    padded = np.full((B, H + 2 * pad, W + 2 * pad, C), -1, codes.dtype)
    padded[:, pad:pad + H, pad:pad + W] = codes
    out = np.full((B, Ho, Wo, C), -1, codes.dtype)
    for r in range(win):
        for s in range(win):
            out = np.maximum(out, padded[:, r:r + stride * Ho:stride, s:s + stride * Wo:stride])
    return out


@pytest.mark.parametrize("block", range(4))
def test_first_layer_and_plane_pool_random_shapes(G, block):
    """int8 first layer (thresholds and bit-plane packing fused) on drawn image sizes, channel counts,
    filters, strides and paddings, then the max-pool on its bit-planes with a drawn window."""
    L = G.A.lib()
    ran = 0
    for i in range(40):
        rng = np.random.default_rng(910000 + 1000 * block + i)
        B = int(rng.integers(1, 5))
        H, Wd = int(rng.integers(8, 80)), int(rng.integers(8, 140))
        if rng.random() < 0.5:
            Wd = (Wd + 3) // 4 * 4            # rows of a multiple of four bytes take the byte-row kernel
        C = int(rng.integers(1, 5))
        cout = int(rng.choice([32, 64, 64, 96, 128]))
        R = int(rng.choice([3, 5, 7, 7, 11]))
        stride = int(rng.integers(1, 5))
        pad = int(rng.integers(0, R // 2 + 1))
        bits = int(rng.integers(1, 5))
        zero_point = int(rng.choice([0, 128]))
        if H + 2 * pad < R or Wd + 2 * pad < R:
            continue
        case = dict(block=block, i=i, B=B, H=H, W=Wd, C=C, cout=cout, R=R, stride=stride, pad=pad, bits=bits, zp=zero_point)
        if zero_point:
            Xraw = rng.integers(0, 256, size=(B, H, Wd, C)).astype(np.uint8)
            Xs = (Xraw.astype(np.int16) - zero_point).astype(np.int8)
        else:
            Xs = rng.integers(-128, 128, size=(B, H, Wd, C)).astype(np.int8)
            Xraw = Xs
        Wt = rng.integers(-128, 128, size=(cout, R, R, C)).astype(np.int8)
        acc = O.conv_i8(Wt, Xs, stride, pad)
        Ho, Wo = acc.shape[1], acc.shape[2]
        rows = B * Ho * Wo
        span = max(1, int(np.abs(acc).max()))
        thr = np.sort(rng.integers(-span, span + 1, size=(cout, 2 ** bits - 1)), axis=1).astype(np.int32)
        codes = O.bn_quantize(acc.reshape(-1, cout), None, thr, None, bits).reshape(acc.shape)
        dX, dW, dT = torch.from_numpy(Xraw).cuda(), G.to_dev(Wt), G.to_dev(thr)
        d_planes = G.dev_empty_i32(bits * rows * cout // 32, fill=-7)
        G.A.check(L.apnn_conv_i8_bn_pack(G.ptr(dX), G.ptr(dW), G.ptr(dT), G.ptr(d_planes), B, H, Wd, C, cout, R, R,
                                         stride, pad, bits, zero_point, None), "conv_i8_bn_pack %r" % (case,))
        ran += 1
        expect = O.pack_bits(codes.reshape(rows, cout).astype(np.uint32), rows, cout, cout, bits)
        assert np.array_equal(G.to_host(d_planes, np.uint32).reshape(expect.shape), expect), case
        win, st, pd = [(3, 2, 1), (2, 2, 0), (3, 1, 1), (2, 1, 0), (3, 3, 0)][rng.integers(0, 5)]
        if Ho + 2 * pd < win or Wo + 2 * pd < win:
            continue
        pooled = _np_maxpool_codes(codes, win, st, pd)
        prow = pooled.shape[0] * pooled.shape[1] * pooled.shape[2]
        d_out = G.dev_empty_i32(bits * prow * cout // 32, fill=-7)
        G.A.check(L.apnn_pool_planes(G.ptr(d_planes), G.ptr(d_out), B, Ho, Wo, cout, bits, win, st, pd, None), "pool_planes")
        pexp = O.pack_bits(pooled.reshape(prow, cout).astype(np.uint32), prow, cout, cout, bits)
        assert np.array_equal(G.to_host(d_out, np.uint32).reshape(pexp.shape), pexp), (case, win, st, pd)
    assert ran >= 20
