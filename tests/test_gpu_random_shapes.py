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


CONV_CHOICES = ([(1, t) for t in range(4)] + [(2, t) for t in (1, 2, 3, 4, 5, 7, 8)] + [(3, t) for t in (1, 2, 3, 4, 7)] +
                [(4, t) for t in range(5)] + [(5, t) for t in (1, 2, 3, 7)] + [(p, None) for p in (0, 0, 0, 1, 2, 3, 4, 5)])
GEMM_CHOICES = ([(1, t) for t in range(5)] + [(2, t) for t in (1, 2, 3, 4, 5, 6)] + [(3, t) for t in (1, 2, 6)] +
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
