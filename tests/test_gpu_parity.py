"""GPU parity: libapnn_tc.so (through its C ABI) against the CPU oracle and the committed golden
fixtures.  Integer work, so every comparison is bit-exact."""
import ctypes
import os

import numpy as np
import pytest

import oracle_lib as O

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

COMBOS = [(1, 2), (1, 3), (1, 4), (2, 2)]          # (weight bits, activation bits)
NAMES = {(1, 2): "w1a2", (1, 3): "w1a3", (1, 4): "w1a4", (2, 2): "w2a2"}


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available(), "GPU tests need a device"
    return gpu_util


def _golden():
    return np.load(os.path.join(O.GOLDEN_DIR, "golden_outputs.npz"), allow_pickle=False)


# ---- GEMM ------------------------------------------------------------------------------------

@pytest.mark.parametrize("wb,xb", COMBOS)
def test_gemm_named_entry_golden(G, wb, xb):
    """Reference-derived known answers through the reference's own entry-point names."""
    name = NAMES[(wb, xb)]
    M, N, K = 64, 128, 128
    s = O.golden_stream()
    nw, nx = wb * M * K // 32, xb * N * K // 32
    dW, dX = G.to_dev(s[:nw]), G.to_dev(s[nw:nw + nx])
    out = G.dev_empty_i32(M * N, fill=-7)
    fn = getattr(G.A.lib(), "apmm_" + name)
    G.A.check(fn(G.ptr(dW), G.ptr(dX), G.ptr(out), M, N, K, wb, xb, None), name)
    got = G.to_host(out).reshape(M, N)
    assert np.array_equal(got, _golden()["gemm_" + name])
    # decompose: low xb bits, MSB-first
    outp = G.dev_empty_i32(xb * M * N // 32, fill=-7)
    fn = getattr(G.A.lib(), "apmm_" + name + "_decompose")
    G.A.check(fn(G.ptr(dW), G.ptr(dX), G.ptr(outp), M, N, K, wb, xb, None), name)
    gotp = G.to_host(outp, np.uint32).reshape(xb, M, N // 32)
    assert np.array_equal(gotp, O.lowbits_pack(_golden()["gemm_" + name], M, N, xb))


# 0 = APNN_PATH_AUTO (the library's own choice: what the named entry points, the networks and the
# benchmark run), APNN_PATH_VALU, APNN_PATH_MFMA (FP4 operands), APNN_PATH_MFMA_I8
# 5 = APNN_PATH_MFMA_XS (FP4 operands expanded by the staging threads)
PATHS = [0, 1, 2, 3, 5]
CONV_PATHS = [0, 1, 2, 3, 4]   # 4 = APNN_PATH_MFMA_PATCH (input patch resident in LDS)
CONV_PATHS_128 = CONV_PATHS + [5]   # shapes whose stored channel count is a multiple of 128
# (path, pinned tile) pairs that are built: VALU tiles 0..3; FP4 GEMM all but 256x256 / 128x256;
# int8 GEMM 128x128, 64x64, 256x128; FP4 convolution all but 256x256 / 256x128 (8 = 32x128 split-K); int8 convolution
# 128x128, 64x64, 128x64, 32x32 split-K, 128x256
GEMM_TILES = ([(1, t) for t in range(4)] + [(2, t) for t in (1, 2, 3, 4, 5, 6, 9)] + [(3, t) for t in (1, 2, 6)] +
              [(5, t) for t in (1, 2, 3, 6)])
CONV_TILES = ([(1, t) for t in range(4)] + [(2, t) for t in (1, 2, 3, 4, 5, 7, 8, 9)] + [(3, t) for t in (1, 2, 3, 4, 7)] +
              [(4, t) for t in range(5)] + [(5, t) for t in (1, 2, 3, 7)])
GEMM_TILES_PACKED = [pt for pt in GEMM_TILES if pt != (1, 3)]     # the VALU 16x16 tile has no packed epilogue
CONV_TILES_PACKED = [pt for pt in CONV_TILES if pt != (1, 3)]


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("wb,xb", COMBOS)
@pytest.mark.parametrize("nk", [128, 256, 384, 512, 640, 768, 896, 1024])
def test_gemm_sweep_m64(G, wb, xb, nk, path):
    """The benchmark sweep of the reference: M=64, N=K=128..1024 (LIB/78_bmmaTensorCoreGemm.cu:473-477)."""
    rng = np.random.default_rng(1000 + nk + 7 * wb + xb)
    M, N, K = 64, nk, nk
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    got = G.run_gemm(W, X, M, N, K, wb, xb, path=path).reshape(M, N)
    assert np.array_equal(got, O.gemm(W, X, M, N, K, wb, xb, nthreads=8))


@pytest.mark.parametrize("sym", [0, 1])
@pytest.mark.parametrize("path,tile", GEMM_TILES)
@pytest.mark.parametrize("wb,xb", COMBOS)
def test_gemm_every_tile_ragged(G, wb, xb, tile, path, sym):
    """Row / column counts that are not multiples of any tile, every tile shape pinned, both weight modes."""
    rng = np.random.default_rng(50 + tile + 10 * wb + xb)
    M, N, K = (70, 97, 384) if path == 1 else (300, 289, 640)
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, path=path, tile=tile).reshape(M, N)
    assert np.array_equal(got, O.gemm(W, X, M, N, K, wb, xb, sym_w=sym))


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("M,N,K", [(1, 1, 128), (1, 32, 128), (3, 5, 256), (64, 32, 128), (129, 64, 2048)])
def test_gemm_edge_shapes(G, M, N, K, path):
    rng = np.random.default_rng(M * 1000 + N)
    W = O.random_planes(rng, 1, M, K // 32)
    X = O.random_planes(rng, 2, N, K // 32)
    got = G.run_gemm(W, X, M, N, K, 1, 2, path=path).reshape(M, N)
    assert np.array_equal(got, O.gemm(W, X, M, N, K, 1, 2))


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("wb,xb", COMBOS)
def test_gemm_symmetric_weights(G, wb, xb, path):
    rng = np.random.default_rng(77 + wb + xb)
    M, N, K = 64, 256, 512
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=1, path=path).reshape(M, N)
    expect = (2 * O.unpack_planes_lsb(W) - (2 ** wb - 1)) @ O.unpack_planes_lsb(X).T
    assert np.array_equal(got, expect)
    assert np.array_equal(got, O.gemm(W, X, M, N, K, wb, xb, sym_w=1))


@pytest.mark.parametrize("path,tile", GEMM_TILES_PACKED)
def test_gemm_bn_epilogue_with_residual(G, tile, path):
    rng = np.random.default_rng(91 + tile)
    M, N, K, wb, xb, ob = 48, 160, 256, 1, 2, 2
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    acc = O.gemm(W, X, M, N, K, wb, xb, sym_w=1)
    resid = rng.integers(-40, 40, size=(M, N)).astype(np.int32)
    thr = np.sort(rng.integers(-120, 120, size=(N, 2 ** ob - 1)), axis=1).astype(np.int32)
    flip = rng.integers(0, 2, size=N).astype(np.uint8)
    d_thr, d_flip, d_res = G.to_dev(thr), G.to_dev(flip), G.to_dev(resid)
    d_save = G.dev_empty_i32(M * N, fill=-7)
    epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr, flip=d_flip, resid=d_res, save=d_save)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=1, epi=epi, path=path, tile=tile).view(np.uint32).reshape(ob, M, N // 32)
    q = O.bn_quantize(acc, resid, thr, flip, ob)
    assert np.array_equal(got, O.lowbits_pack(q, M, N, ob))
    assert np.array_equal(G.to_host(d_save).reshape(M, N), acc + resid)


@pytest.mark.parametrize("path,tile", [(2, 4), (2, 5), (2, 6), (3, 6)])
@pytest.mark.parametrize("wb,xb,sym", [(1, 2, 0), (1, 2, 1), (1, 4, 1), (2, 2, 0)])
def test_gemm_split_k_tiles(G, wb, xb, sym, tile, path):
    """Tiles 4, 5: the four waves split the reduction (partial sums combined in LDS); 6, 7: the
    rectangular 256x128 tile."""
    rng = np.random.default_rng(60 + tile + 10 * wb + xb)
    M, N, K = (77, 130, 1664) if tile < 6 else (300, 289, 1664)     # K/32 = 52 words: not a multiple of the chunk
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, path=path, tile=tile).reshape(M, N)
    assert np.array_equal(got, O.gemm(W, X, M, N, K, wb, xb, sym_w=sym))


# ---- convolution -----------------------------------------------------------------------------

@pytest.mark.parametrize("wb,xb", COMBOS)
def test_conv_named_entry_golden(G, wb, xb):
    name = NAMES[(wb, xb)]
    H = Wd = 16
    CIN = COUT = 128
    s = O.golden_stream()
    nx, nw = xb * (H + 2) * (Wd + 2) * CIN // 32, wb * COUT * 9 * CIN // 32
    dX, dW = G.to_dev(s[:nx]), G.to_dev(s[nx:nx + nw])
    out = G.dev_empty_i32(H * Wd * COUT, fill=-7)
    L = G.A.lib()
    G.A.check(getattr(L, "apconv_" + name)(G.ptr(dW), G.ptr(dX), G.ptr(out), H, Wd, CIN, COUT, None), name)
    gold = _golden()
    assert np.array_equal(G.to_host(out).reshape(H, Wd, COUT), gold["conv_" + name])
    outp = G.dev_empty_i32(xb * H * Wd * COUT // 32, fill=-7)
    G.A.check(getattr(L, "APConv_" + name + "_pack")(G.ptr(dW), G.ptr(dX), G.ptr(outp), H, Wd, CIN, COUT, None), name)
    assert np.array_equal(G.to_host(outp, np.uint32).reshape(xb, H * Wd, COUT // 32), gold["conv_pack_" + name])
    if name in ("w1a2", "w2a2"):
        outq = G.dev_empty_i32(xb * (H // 2) * (Wd // 2) * COUT // 32, fill=-7)
        G.A.check(getattr(L, "APConv_" + name + "_pack_pool")(G.ptr(dW), G.ptr(dX), G.ptr(outq), H, Wd, CIN, COUT, None), name)
        pooled = O.avgpool2x2(gold["conv_" + name][None])[0]
        expect = O.lowbits_pack(pooled, (H // 2) * (Wd // 2), COUT, xb)
        assert np.array_equal(G.to_host(outq, np.uint32).reshape(expect.shape), expect)


@pytest.mark.parametrize("path", CONV_PATHS_128)
@pytest.mark.parametrize("wb,xb", COMBOS)
@pytest.mark.parametrize("C,batch", [(128, 1), (256, 1), (512, 1), (128, 16)])
def test_conv3x3_16x16_sweep(G, wb, xb, C, batch, path):
    """Benchmark family of the reference: 3x3 / stride 1 / pad 1 on a 16x16 map, halo stored."""
    rng = np.random.default_rng(300 + C + batch + wb * 3 + xb)
    H = Wd = 16
    X = O.random_planes(rng, xb, batch * (H + 2) * (Wd + 2), C // 32)
    Wt = O.random_planes(rng, wb, C * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=C, R=3, S=3, stride=1, pad=1, halo=1, wb=wb, xb=xb)
    got = G.run_conv(Wt, X, cin_pad=C, path=path, **kw).reshape(batch, H, Wd, C)
    assert np.array_equal(got, O.conv(Wt, X, cwords=C // 32, nthreads=8, **kw))


@pytest.mark.parametrize("wb,xb", COMBOS)
@pytest.mark.parametrize("batch", [1, 16])
@pytest.mark.parametrize("C", [128, 256, 384, 512, 640, 768, 896, 1024])
def test_conv3x3_16x16_benchmark_shapes_auto(G, wb, xb, C, batch):
    """Every shape of the 16x16 benchmark family on the library's own kernel choice: int32 output, then
    the fused BN-threshold requantize to a bits with thresholds drawn as sorted uniform integers in
    [0, 9*Cin*(2^a-1)(2^w-1)/2] per channel, packed for the next layer."""
    rng = np.random.default_rng(3300 + C + batch + wb * 3 + xb)
    H = Wd = 16
    X = O.random_planes(rng, xb, batch * (H + 2) * (Wd + 2), C // 32)
    Wt = O.random_planes(rng, wb, C * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=C, R=3, S=3, stride=1, pad=1, halo=1, wb=wb, xb=xb)
    acc = O.conv(Wt, X, cwords=C // 32, nthreads=16, **kw)
    got = G.run_conv(Wt, X, cin_pad=C, path=0, **kw).reshape(acc.shape)
    assert np.array_equal(got, acc)
    hi = 9 * C * (2 ** xb - 1) * (2 ** wb - 1) // 2
    thr = np.sort(rng.integers(0, hi + 1, size=(C, 2 ** xb - 1)), axis=1).astype(np.int32)
    d_thr = G.to_dev(thr)
    rows = batch * H * Wd
    epi = G.epilogue(mode=G.A.EPI_BN, out_bits=xb, thr=d_thr)
    gotq = G.run_conv(Wt, X, cin_pad=C, epi=epi, path=0, **kw).view(np.uint32).reshape(xb, rows, C // 32)
    q = O.bn_quantize(acc.reshape(rows, C), None, thr, None, xb)
    assert 0 < q.mean() < 2 ** xb - 1
    assert np.array_equal(gotq, O.lowbits_pack(q, rows, C, xb))


GEOMS = [  # batch H W cin_pad cout R stride pad halo
    (2, 14, 14, 128, 96, 3, 1, 1, 0),     # predicated halo, cout not a tile multiple
    (3, 28, 28, 64, 128, 3, 2, 1, 0),     # ResNet stride-2 3x3 on 64 stored channels (64-bit loads)
    (2, 28, 28, 64, 128, 1, 2, 0, 0),     # ResNet 1x1 stride-2 downsample
    (1, 7, 7, 256, 64, 3, 1, 1, 0),       # 7x7 map
    (2, 13, 11, 32, 40, 5, 1, 2, 0),      # 5x5 filter, 32 stored channels (32-bit loads)
    (8, 1, 1, 512, 256, 1, 1, 0, 0),      # fully connected layer as 1x1 conv, batch = rows
    (1, 9, 9, 128, 32, 3, 1, 1, 1),       # halo stored, odd size
]


@pytest.mark.parametrize("path", CONV_PATHS)
@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("wb,xb,sym", [(1, 2, 0), (1, 2, 1), (2, 2, 1), (1, 4, 0), (1, 3, 1)])
def test_conv_general_geometry(G, geom, wb, xb, sym, path):
    batch, H, Wd, cin_pad, cout, R, stride, pad, halo = geom
    rng = np.random.default_rng(hash((geom, wb, xb, sym)) % (2 ** 31))
    Hs, Ws = (H + 2 * pad, Wd + 2 * pad) if halo else (H, Wd)
    X = O.random_planes(rng, xb, batch * Hs * Ws, cin_pad // 32)
    Wt = O.random_planes(rng, wb, cout * R * R, cin_pad // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=R, S=R, stride=stride, pad=pad, halo=halo, wb=wb, xb=xb)
    expect = O.conv(Wt, X, cwords=cin_pad // 32, sym_w=sym, nthreads=8, **kw)
    got = G.run_conv(Wt, X, cin_pad=cin_pad, sym=sym, path=path, **kw).reshape(expect.shape)
    assert np.array_equal(got, expect)
    if cin_pad % 128 == 0 and path == 2:      # the expand-while-staging kernel needs 128-bit loads
        got = G.run_conv(Wt, X, cin_pad=cin_pad, sym=sym, path=5, **kw).reshape(expect.shape)
        assert np.array_equal(got, expect)


@pytest.mark.parametrize("path,tile", CONV_TILES)
def test_conv_every_tile(G, tile, path):
    rng = np.random.default_rng(400 + tile)
    batch, H, Wd, C, cout = 2, 10, 6, 128, 72
    X = O.random_planes(rng, 2, batch * H * Wd, C // 32)
    Wt = O.random_planes(rng, 1, cout * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=3, S=3, stride=1, pad=1, halo=0, wb=1, xb=2)
    expect = O.conv(Wt, X, cwords=C // 32, sym_w=1, **kw)
    got = G.run_conv(Wt, X, cin_pad=C, sym=1, path=path, tile=tile, **kw).reshape(expect.shape)
    assert np.array_equal(got, expect)


@pytest.mark.parametrize("pool", [0, 1, 2])
@pytest.mark.parametrize("path,tile", CONV_TILES_PACKED)
def test_conv_bn_epilogue(G, pool, tile, path):
    """BN-threshold requantize to a bits (+ residual / saved accumulator when not pooling,
    + avg / max pooling), packed for the next layer."""
    rng = np.random.default_rng(500 + 10 * pool + tile)
    batch, H, Wd, C, cout, wb, xb, ob = 2, 8, 12, 128, 96, 1, 2, 2
    X = O.random_planes(rng, xb, batch * H * Wd, C // 32)
    Wt = O.random_planes(rng, wb, cout * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=3, S=3, stride=1, pad=1, halo=0, wb=wb, xb=xb)
    acc = O.conv(Wt, X, cwords=C // 32, sym_w=1, **kw)
    thr = np.sort(rng.integers(-300, 300, size=(cout, 2 ** ob - 1)), axis=1).astype(np.int32)
    flip = rng.integers(0, 2, size=cout).astype(np.uint8)
    d_thr, d_flip = G.to_dev(thr), G.to_dev(flip)
    if pool == 0:
        resid = rng.integers(-100, 100, size=acc.shape).astype(np.int32)
        d_res, d_save = G.to_dev(resid), G.dev_empty_i32(acc.size, fill=-7)
        epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr, flip=d_flip, resid=d_res, save=d_save)
        q = O.bn_quantize(acc.reshape(-1, cout), resid.reshape(-1, cout), thr, flip, ob)
        rows = batch * H * Wd
    else:
        epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, pool=pool, thr=d_thr, flip=d_flip)
        if pool == 1:
            q = O.bn_quantize(O.avgpool2x2(acc).reshape(-1, cout), None, thr, flip, ob)
        else:
            q = O.maxpool2x2(O.bn_quantize(acc.reshape(-1, cout), None, thr, flip, ob).reshape(acc.shape)).reshape(-1, cout)
        rows = batch * (H // 2) * (Wd // 2)
    got = G.run_conv(Wt, X, cin_pad=C, sym=1, epi=epi, path=path, tile=tile, **kw).view(np.uint32).reshape(ob, rows, cout // 32)
    assert np.array_equal(got, O.lowbits_pack(q, rows, cout, ob))
    if pool == 0:
        assert np.array_equal(G.to_host(d_save).reshape(acc.shape), acc + resid)


def test_packed_output_feeds_next_layer(G):
    """A layer's packed output is a valid activation operand of the next layer: unpacking it with the
    packer's bit order (MSB-first) reproduces the codes, and a GEMM on it matches the oracle."""
    rng = np.random.default_rng(600)
    batch, C, cout, nxt = 16, 256, 128, 64
    X = O.random_planes(rng, 2, batch, C // 32)
    Wt = O.random_planes(rng, 1, cout, C // 32)
    kw = dict(batch=batch, H=1, W=1, cout=cout, R=1, S=1, stride=1, pad=0, halo=0, wb=1, xb=2)
    acc = O.conv(Wt, X, cwords=C // 32, sym_w=1, **kw).reshape(batch, cout)
    thr = np.sort(rng.integers(-60, 60, size=(cout, 3)), axis=1).astype(np.int32)
    d_thr = G.to_dev(thr)
    epi = G.epilogue(mode=G.A.EPI_BN, out_bits=2, thr=d_thr)
    packed = G.run_conv(Wt, X, cin_pad=C, sym=1, epi=epi, **kw).view(np.uint32).reshape(2, batch, cout // 32)
    q = O.bn_quantize(acc, None, thr, None, 2)
    assert np.array_equal(O.unpack_bits(packed, batch, cout, cout, 2), q.astype(np.uint32))
    W2 = O.random_planes(rng, 1, nxt, cout // 32)
    kw2 = dict(batch=batch, H=1, W=1, cout=nxt, R=1, S=1, stride=1, pad=0, halo=0, wb=1, xb=2)
    got = G.run_conv(W2, packed, cin_pad=cout, **kw2).reshape(batch, nxt)
    assert np.array_equal(got, O.conv(W2, packed, cwords=cout // 32, **kw2).reshape(batch, nxt))


def test_pack_bits(G):
    rng = np.random.default_rng(700)
    for rows, C, cpad, bits in [(5, 3, 128, 2), (33, 70, 128, 3), (64, 192, 256, 2), (7, 64, 64, 8), (2, 100, 128, 1)]:
        v = rng.integers(0, 2 ** bits, size=(rows, C)).astype(np.uint32)
        dv = G.to_dev(v)
        out = G.dev_empty_i32(bits * rows * cpad // 32, fill=-7)
        G.A.check(G.A.lib().apnn_pack_bits(G.ptr(dv), G.ptr(out), rows, C, cpad, bits, None), "pack_bits")
        got = G.to_host(out, np.uint32).reshape(bits, rows, cpad // 32)
        assert np.array_equal(got, O.pack_bits(v, rows, C, cpad, bits))


def test_pack_bits_fc_hidden(G):
    # the reference's loop stores all planes at the same words: the last one written (bit bits-1) stays
    rng = np.random.default_rng(701)
    for rows, C, cpad, bits in [(5, 3, 128, 2), (33, 70, 128, 3), (64, 192, 256, 2), (2, 100, 128, 1)]:
        v = rng.integers(0, 2 ** bits, size=(rows, C)).astype(np.uint32)
        dv = G.to_dev(v)
        out = G.dev_empty_i32(rows * cpad // 32, fill=-7)
        G.A.check(G.A.lib().apnn_pack_bits_fc_hidden(G.ptr(dv), G.ptr(out), rows, C, cpad, bits, None), "pack_fc_hidden")
        got = G.to_host(out, np.uint32).reshape(1, rows, cpad // 32)
        assert np.array_equal(got, O.pack_bits(v >> (bits - 1), rows, C, cpad, 1))
        assert np.array_equal(got[0], O.pack_bits(v, rows, C, cpad, bits)[bits - 1])


# ---- full-size shapes: size-independent properties + sampled rows ------------------------------

@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("wb,xb", COMBOS)
def test_gemm_2048_sampled_and_closed_form(G, wb, xb, path):
    rng = np.random.default_rng(800 + wb + xb)
    M = N = K = 2048
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    got = G.run_gemm(W, X, M, N, K, wb, xb, path=path).reshape(M, N)
    rows = np.sort(rng.choice(M, 16, replace=False))
    for m in rows:
        assert np.array_equal(got[m], O.gemm_rows(W, X, M, N, K, wb, xb, int(m), int(m) + 1, nthreads=8)[0])
    # column sums are linear in W:  sum_m D[m][n] = (sum_m wvalue[m]) . xvalue[n]
    wsum = O.unpack_planes_lsb(W).sum(0)
    assert np.array_equal(got.astype(np.int64).sum(0), O.unpack_planes_lsb(X) @ wsum)
    ones_w = np.full_like(W, 0xFFFFFFFF)
    ones_x = np.full_like(X, 0xFFFFFFFF)
    assert np.all(G.run_gemm(ones_w, ones_x, M, N, K, wb, xb, path=path) == K * (2 ** wb - 1) * (2 ** xb - 1))


@pytest.mark.parametrize("wb,xb", COMBOS)
@pytest.mark.parametrize("n", [4096, 8192])
def test_gemm_large_auto_sampled_linearity_closed_form(G, wb, xb, n):
    """M = N = K = 4096 / 8192 on the library's own kernel choice.  The oracle is too slow for 7e10 /
    5e11 outputs' worth of work, so: rows sampled at random against the oracle, every column sum against
    the linear form (each output element takes part), and the all-ones closed form K(2^w-1)(2^a-1)."""
    rng = np.random.default_rng(8800 + n + wb * 5 + xb)
    M = N = K = n
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    got = G.run_gemm(W, X, M, N, K, wb, xb, path=0).reshape(M, N)
    rows = sorted(set([0, M - 1] + [int(v) for v in rng.choice(M, 22, replace=False)]))
    for m in rows:
        assert np.array_equal(got[m], O.gemm_rows(W, X, M, N, K, wb, xb, m, m + 1, nthreads=16)[0]), m
    assert np.array_equal(got.sum(0, dtype=np.int64), O.gemm_column_sums(W, X))
    del got
    W[:] = 0xFFFFFFFF
    X[:] = 0xFFFFFFFF
    assert np.all(G.run_gemm(W, X, M, N, K, wb, xb, path=0) == K * (2 ** wb - 1) * (2 ** xb - 1))


# ---- layers on either side of the low-bit path ---------------------------------------------------

def _np_maxpool_codes(codes, win, stride, pad):
    B, H, W, C = codes.shape
    Ho, Wo = (H + 2 * pad - win) // stride + 1, (W + 2 * pad - win) // stride + 1
    padded = np.zeros((B, H + 2 * pad, W + 2 * pad, C), codes.dtype)     # codes are >= 0: zero padding == ignoring
    padded[:, pad:pad + H, pad:pad + W] = codes
    out = np.zeros((B, Ho, Wo, C), codes.dtype)
    for r in range(win):
        for s in range(win):
            out = np.maximum(out, padded[:, r:r + stride * (Ho - 1) + 1:stride, s:s + stride * (Wo - 1) + 1:stride])
    return out


@pytest.mark.parametrize("R,stride,pad,H,cout", [(7, 2, 3, 32, 64), (11, 4, 5, 35, 64), (3, 1, 1, 9, 40)])
def test_conv_i8_bn_and_pool_pack(G, R, stride, pad, H, cout):
    rng = np.random.default_rng(900 + R)
    B, C, bits = 2, 3, 2
    X = rng.integers(-128, 128, size=(B, H, H, C)).astype(np.int8)
    Wt = rng.integers(-128, 128, size=(cout, R, R, C)).astype(np.int8)
    acc = O.conv_i8(Wt, X, stride, pad)
    Ho = acc.shape[1]
    thr = np.sort(rng.integers(-60000, 60000, size=(cout, 3)), axis=1).astype(np.int32)
    dX, dW, dT = G.to_dev(X), G.to_dev(Wt), G.to_dev(thr)
    d_codes = G.guarded_empty(B * Ho * Ho * cout, torch.uint8)
    d_acc = G.dev_empty_i32(B * Ho * Ho * cout, fill=-7)
    L = G.A.lib()
    G.A.check(L.apnn_conv_i8_bn(G.ptr(dX), G.ptr(dW), G.ptr(dT), G.ptr(d_codes), G.ptr(d_acc), B, H, H, C, cout, R, R,
                                stride, pad, bits, 0, None), "conv_i8_bn")
    assert np.array_equal(G.to_host(d_acc).reshape(acc.shape), acc)
    codes = O.bn_quantize(acc.reshape(-1, cout), None, thr, None, bits).reshape(acc.shape).astype(np.uint8)
    torch.cuda.synchronize()
    assert np.array_equal(d_codes.cpu().numpy().reshape(acc.shape), codes)
    for win, st, pd in [(3, 2, 1), (2, 2, 0), (1, 1, 0)]:
        pooled = _np_maxpool_codes(codes, win, st, pd)
        rows = pooled.shape[0] * pooled.shape[1] * pooled.shape[2]
        cpad = 128
        d_planes = G.dev_empty_i32(bits * rows * cpad // 32, fill=-7)
        G.A.check(L.apnn_pool_pack(G.ptr(d_codes), G.ptr(d_planes), B, Ho, Ho, cout, cpad, bits, win, st, pd, None),
                  "pool_pack")
        expect = O.pack_bits(pooled.reshape(rows, cout).astype(np.uint32), rows, cout, cpad, bits)
        assert np.array_equal(G.to_host(d_planes, np.uint32).reshape(expect.shape), expect)


def test_unpack_sum_and_fc_i8(G):
    rng = np.random.default_rng(950)
    B, HW, C, cpad, bits, N = 4, 49, 200, 256, 2, 37
    codes = rng.integers(0, 4, size=(B * HW, C)).astype(np.uint32)
    planes = O.pack_bits(codes, B * HW, C, cpad, bits)
    d_planes = G.to_dev(planes)
    L = G.A.lib()
    d_un = G.guarded_empty(B * HW * C, torch.int8)
    G.A.check(L.apnn_unpack_sum(G.ptr(d_planes), G.ptr(d_un), B * HW, 1, C, cpad, bits, 0, None), "unpack")
    torch.cuda.synchronize()
    assert np.array_equal(d_un.cpu().numpy().reshape(B * HW, C), codes.astype(np.int8))
    d_pool = G.guarded_empty(B * C, torch.int8)
    G.A.check(L.apnn_unpack_sum(G.ptr(d_planes), G.ptr(d_pool), B, HW, C, cpad, bits, 1, None), "pool")
    torch.cuda.synchronize()
    pooled = np.minimum(127, codes.reshape(B, HW, C).sum(1) >> 1).astype(np.int8)
    assert np.array_equal(d_pool.cpu().numpy().reshape(B, C), pooled)
    Wt = rng.integers(-128, 128, size=(N, C)).astype(np.int8)
    scale = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.uniform(-1, 1, N).astype(np.float32)
    d_out = G.guarded_empty(B * N, torch.float32)
    d_acc = G.dev_empty_i32(B * N, fill=-7)
    dW, dS, dB = G.to_dev(Wt), torch.from_numpy(scale).cuda(), torch.from_numpy(bias).cuda()
    G.A.check(L.apnn_fc_i8(G.ptr(d_pool), G.ptr(dW), G.ptr(dS), G.ptr(dB), G.ptr(d_out), G.ptr(d_acc), B, N, C, None), "fc")
    acc = pooled.astype(np.int64) @ Wt.astype(np.int64).T
    assert np.array_equal(G.to_host(d_acc).reshape(B, N), acc)
    torch.cuda.synchronize()
    # float affine of an exact int32: one fp32 multiply-add, tolerance 1e-6 relative
    expect = acc.astype(np.float32) * scale[None, :] + bias[None, :]
    assert np.allclose(d_out.cpu().numpy().reshape(B, N), expect, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("Bn,N,K", [(64, 1000, 512), (64, 1000, 4096), (37, 1003, 516), (32, 130, 64), (8, 1000, 512),
                                    (40, 50, 128), (33, 999, 510)])
def test_fc_i8_batches(G, Bn, N, K):
    """int8 classifier at the batch sizes of the networks: the 8 x 8-tile kernel (batch >= 32, whole dwords),
    ragged feature / batch / K counts, and the shapes that stay on the smaller kernels."""
    rng = np.random.default_rng(960 + Bn + N + K)
    X = rng.integers(-128, 128, size=(Bn, K)).astype(np.int8)
    Wt = rng.integers(-128, 128, size=(N, K)).astype(np.int8)
    scale = rng.uniform(0.001, 0.01, N).astype(np.float32)
    bias = rng.uniform(-1, 1, N).astype(np.float32)
    d_out = G.guarded_empty(Bn * N, torch.float32)
    d_acc = G.dev_empty_i32(Bn * N, fill=-7)
    dX, dW, dS, dB = G.to_dev(X), G.to_dev(Wt), torch.from_numpy(scale).cuda(), torch.from_numpy(bias).cuda()
    G.A.check(G.A.lib().apnn_fc_i8(G.ptr(dX), G.ptr(dW), G.ptr(dS), G.ptr(dB), G.ptr(d_out), G.ptr(d_acc), Bn, N, K, None), "fc")
    acc = X.astype(np.int64) @ Wt.astype(np.int64).T
    assert np.array_equal(G.to_host(d_acc).reshape(Bn, N), acc)
    torch.cuda.synchronize()
    expect = acc.astype(np.float32) * scale[None, :] + bias[None, :]
    assert np.allclose(d_out.cpu().numpy().reshape(Bn, N), expect, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("B,HW,C,cpad,bits,shift", [(3, 150, 96, 96, 3, 2), (2, 64, 40, 64, 1, 0), (5, 9, 64, 64, 4, 0),
                                                    (2, 7, 33, 64, 2, 0)])
def test_unpack_sum_group_sizes(G, B, HW, C, cpad, bits, shift):
    """Global pooling of packed codes: groups longer than a wave (several passes), a whole wave, short
    groups (lane-split kernel), all code widths; sums saturate at 127."""
    rng = np.random.default_rng(960 + HW)
    codes = rng.integers(0, 1 << bits, size=(B * HW, C)).astype(np.uint32)
    d_planes = G.to_dev(O.pack_bits(codes, B * HW, C, cpad, bits))
    d_pool = G.guarded_empty(B * C, torch.int8)
    G.A.check(G.A.lib().apnn_unpack_sum(G.ptr(d_planes), G.ptr(d_pool), B, HW, C, cpad, bits, shift, None), "pool")
    torch.cuda.synchronize()
    pooled = np.minimum(127, codes.reshape(B, HW, C).sum(1) >> shift).astype(np.int8)
    assert np.array_equal(d_pool.cpu().numpy().reshape(B, C), pooled)


@pytest.mark.parametrize("path,tile", CONV_TILES_PACKED + [(0, None)])
def test_conv_packed_residual(G, path, tile):
    """Identity shortcut: the block input's packed codes are added, scaled, before the thresholds."""
    rng = np.random.default_rng(970 + path + 7 * (tile or 0))
    batch, H, Wd, C, wb, xb, ob = 2, 14, 14, 128, 1, 2, 2
    X = O.random_planes(rng, xb, batch * H * Wd, C // 32)
    Wt = O.random_planes(rng, wb, C * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=C, R=3, S=3, stride=1, pad=1, halo=0, wb=wb, xb=xb)
    acc = O.conv(Wt, X, cwords=C // 32, sym_w=1, **kw).reshape(-1, C)
    short = rng.integers(0, 4, size=acc.shape).astype(np.uint32)
    short_planes = O.pack_bits(short, acc.shape[0], C, C, 2)
    thr = np.sort(rng.integers(-100, 100, size=(C, 3)), axis=1).astype(np.int32)
    d_thr, d_sp = G.to_dev(thr), G.to_dev(short_planes)
    epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr, resid_planes=d_sp, resid_bits=2, resid_scale=24)
    got = G.run_conv(Wt, X, cin_pad=C, sym=1, epi=epi, path=path, tile=tile, **kw).view(np.uint32).reshape(ob, -1, C // 32)
    q = O.bn_quantize(acc + 24 * short.astype(np.int32), None, thr, None, ob)
    assert np.array_equal(got, O.lowbits_pack(q, acc.shape[0], C, ob))


@pytest.mark.parametrize("scale", [1, 3, 8, 7, 11, 21, -5, -12, 37, 1 << 14])
@pytest.mark.parametrize("path,tile", [(0, None), (2, 1), (2, 2), (2, 3), (2, 4), (2, 5), (2, 8), (2, 9), (3, 2), (4, 0), (4, 3),
                                       (5, 1)])
def test_conv_packed_shortcut_scales(G, path, tile, scale):
    """Shortcut codes of two bits and of one bit times an integer scale, added before the thresholds.  The FP4
    kernels add the term on the matrix cores when the scale is a sum of two terms +-{1, 3} * 2^j (every
    scale here but 37, which takes the per-value path like the other cores), symmetric and unsigned
    weights, every kind of tile (waves tile the output, split K, two wave groups, patch-resident,
    expanded while staging)."""
    rng = np.random.default_rng(1980 + path + 7 * (tile or 0) + (scale & 1023))
    batch, H, Wd, C, wb, xb, ob = 2, 10, 12, 128, 1, 2, 2
    X = O.random_planes(rng, xb, batch * H * Wd, C // 32)
    Wt = O.random_planes(rng, wb, C * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=C, R=3, S=3, stride=1, pad=1, halo=0, wb=wb, xb=xb)
    for sym in (1, 0):
        acc = O.conv(Wt, X, cwords=C // 32, sym_w=sym, **kw).reshape(-1, C)
        for rbits in (2, 1):
            short = rng.integers(0, 2 ** rbits, size=acc.shape).astype(np.uint32)
            short_planes = O.pack_bits(short, acc.shape[0], C, C, rbits)
            v = acc + scale * short.astype(np.int32)
            lo, hi = int(v.min()), int(v.max())
            thr = np.sort(rng.integers(lo, hi + 1, size=(C, 3)), axis=1).astype(np.int32)
            d_thr, d_sp = G.to_dev(thr), G.to_dev(short_planes)
            epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr, resid_planes=d_sp, resid_bits=rbits, resid_scale=scale)
            got = G.run_conv(Wt, X, cin_pad=C, sym=sym, epi=epi, path=path, tile=tile, **kw)
            q = O.bn_quantize(v, None, thr, None, ob)
            assert np.array_equal(got.view(np.uint32).reshape(ob, -1, C // 32), O.lowbits_pack(q, acc.shape[0], C, ob)), (sym, rbits)


@pytest.mark.parametrize("rbits", [3, 5, 8])
@pytest.mark.parametrize("path,tile", [(0, None), (1, None), (1, 0), (2, 1), (2, 2), (2, 4), (2, 5), (2, 8), (3, 2), (4, 0),
                                       (5, 1)])
def test_conv_packed_residual_wide_codes(G, path, tile, rbits):
    """Shortcut codes wider than two bits: their words are not staged before the K loop but read by the
    output stage itself, one plane at a time."""
    rng = np.random.default_rng(980 + path + 7 * (tile or 0) + rbits)
    batch, H, Wd, C, wb, xb, ob = 2, 10, 12, 128, 1, 2, 2
    X = O.random_planes(rng, xb, batch * H * Wd, C // 32)
    Wt = O.random_planes(rng, wb, C * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=C, R=3, S=3, stride=1, pad=1, halo=0, wb=wb, xb=xb)
    acc = O.conv(Wt, X, cwords=C // 32, sym_w=1, **kw).reshape(-1, C)
    short = rng.integers(0, 2 ** rbits, size=acc.shape).astype(np.uint32)
    short_planes = O.pack_bits(short, acc.shape[0], C, C, rbits)
    thr = np.sort(rng.integers(-150, 150, size=(C, 3)), axis=1).astype(np.int32)
    d_thr, d_sp = G.to_dev(thr), G.to_dev(short_planes)
    epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr, resid_planes=d_sp, resid_bits=rbits, resid_scale=3)
    got = G.run_conv(Wt, X, cin_pad=C, sym=1, epi=epi, path=path, tile=tile, **kw).view(np.uint32).reshape(ob, -1, C // 32)
    q = O.bn_quantize(acc + 3 * short.astype(np.int32), None, thr, None, ob)
    assert np.array_equal(got, O.lowbits_pack(q, acc.shape[0], C, ob))


@pytest.mark.parametrize("R,stride,pad,H,Wd,cout,C", [
    (7, 2, 3, 40, 43, 64, 3), (11, 4, 5, 67, 70, 64, 3), (3, 1, 1, 9, 12, 96, 4), (5, 2, 2, 33, 36, 32, 1),
    # row length a multiple of 4 bytes: the kernel that consumes image rows as bytes
    (7, 2, 3, 40, 44, 64, 3), (7, 2, 3, 75, 132, 128, 3), (11, 4, 5, 67, 72, 64, 3), (3, 2, 0, 20, 70, 32, 2),
    (7, 4, 3, 39, 64, 64, 3),
    # a patch of more dwords than a lane keeps in flight (stride 13: 3 x 409 dwords): staged in place
    (3, 13, 1, 40, 140, 32, 4)])
def test_conv_i8_bn_pack_and_pool_planes(G, R, stride, pad, H, Wd, cout, C):
    """First layer with packed output, then max-pool on the bit-planes."""
    rng = np.random.default_rng(990 + R + Wd)
    B, bits = 2, 2
    Xu = rng.integers(0, 256, size=(B, H, Wd, C)).astype(np.uint8)
    Wt = rng.integers(-128, 128, size=(cout, R, R, C)).astype(np.int8)
    acc = O.conv_i8(Wt, (Xu.astype(np.int16) - 128).astype(np.int8), stride, pad)
    Ho, Wo = acc.shape[1], acc.shape[2]
    thr = np.sort(rng.integers(-60000, 60000, size=(cout, 3)), axis=1).astype(np.int32)
    codes = O.bn_quantize(acc.reshape(-1, cout), None, thr, None, bits).reshape(acc.shape)
    L = G.A.lib()
    dX, dW, dT = torch.from_numpy(Xu).cuda(), G.to_dev(Wt), G.to_dev(thr)
    rows = B * Ho * Wo
    d_planes = G.dev_empty_i32(bits * rows * cout // 32, fill=-7)
    G.A.check(L.apnn_conv_i8_bn_pack(G.ptr(dX), G.ptr(dW), G.ptr(dT), G.ptr(d_planes), B, H, Wd, C, cout, R, R,
                                     stride, pad, bits, 128, None), "conv_i8_bn_pack")
    expect = O.pack_bits(codes.reshape(rows, cout).astype(np.uint32), rows, cout, cout, bits)
    assert np.array_equal(G.to_host(d_planes, np.uint32).reshape(expect.shape), expect)
    # the uint8-code / int32 outputs of the same kernel
    d_codes = G.guarded_empty(rows * cout, torch.uint8)
    d_acc = G.dev_empty_i32(rows * cout, fill=-7)
    G.A.check(L.apnn_conv_i8_bn(G.ptr(dX), G.ptr(dW), G.ptr(dT), G.ptr(d_codes), G.ptr(d_acc), B, H, Wd, C, cout, R, R,
                                stride, pad, bits, 128, None), "conv_i8_bn")
    assert np.array_equal(G.to_host(d_acc).reshape(acc.shape), acc)
    torch.cuda.synchronize()
    assert np.array_equal(d_codes.cpu().numpy().reshape(acc.shape), codes.astype(np.uint8))
    for win, st, pd in [(3, 2, 1), (2, 2, 0), (3, 1, 1)]:
        pooled = _np_maxpool_codes(codes, win, st, pd)
        prow = pooled.shape[0] * pooled.shape[1] * pooled.shape[2]
        d_out = G.dev_empty_i32(bits * prow * cout // 32, fill=-7)
        G.A.check(L.apnn_pool_planes(G.ptr(d_planes), G.ptr(d_out), B, Ho, Wo, cout, bits, win, st, pd, None), "pool_planes")
        pexp = O.pack_bits(pooled.reshape(prow, cout).astype(np.uint32), prow, cout, cout, bits)
        assert np.array_equal(G.to_host(d_out, np.uint32).reshape(pexp.shape), pexp)


@pytest.mark.parametrize("bits,zero_point", [(1, 128), (1, 0), (2, 0)])
def test_conv_i8_bn_pack_signed_input_and_one_bit(G, bits, zero_point):
    rng = np.random.default_rng(1200 + bits + zero_point)
    B, H, Wd, C, cout, R, stride, pad = 3, 30, 52, 3, 64, 7, 2, 3
    if zero_point:
        Xraw = rng.integers(0, 256, size=(B, H, Wd, C)).astype(np.uint8)
        Xs = (Xraw.astype(np.int16) - zero_point).astype(np.int8)
    else:
        Xs = rng.integers(-128, 128, size=(B, H, Wd, C)).astype(np.int8)
        Xraw = Xs
    Wt = rng.integers(-128, 128, size=(cout, R, R, C)).astype(np.int8)
    acc = O.conv_i8(Wt, Xs, stride, pad)
    rows = acc.shape[0] * acc.shape[1] * acc.shape[2]
    thr = np.sort(rng.integers(-60000, 60000, size=(cout, 2 ** bits - 1)), axis=1).astype(np.int32)
    codes = O.bn_quantize(acc.reshape(-1, cout), None, thr, None, bits)
    dX, dW, dT = torch.from_numpy(Xraw).cuda(), G.to_dev(Wt), G.to_dev(thr)
    d_planes = G.dev_empty_i32(bits * rows * cout // 32, fill=-7)
    G.A.check(G.A.lib().apnn_conv_i8_bn_pack(G.ptr(dX), G.ptr(dW), G.ptr(dT), G.ptr(d_planes), B, H, Wd, C, cout, R, R,
                                             stride, pad, bits, zero_point, None), "conv_i8_bn_pack")
    expect = O.pack_bits(codes.astype(np.uint32), rows, cout, cout, bits)
    assert np.array_equal(G.to_host(d_planes, np.uint32).reshape(expect.shape), expect)


def test_pool_planes_wide_codes(G):
    rng = np.random.default_rng(995)
    B, H, W, C, bits = 2, 9, 11, 96, 5
    codes = rng.integers(0, 2 ** bits, size=(B, H, W, C)).astype(np.int32)
    planes = O.pack_bits(codes.reshape(-1, C).astype(np.uint32), B * H * W, C, C, bits)
    d_in = G.to_dev(planes)
    pooled = _np_maxpool_codes(codes, 3, 2, 1)
    prow = pooled.shape[0] * pooled.shape[1] * pooled.shape[2]
    d_out = G.dev_empty_i32(bits * prow * C // 32, fill=-7)
    G.A.check(G.A.lib().apnn_pool_planes(G.ptr(d_in), G.ptr(d_out), B, H, W, C, bits, 3, 2, 1, None), "pool_planes")
    pexp = O.pack_bits(pooled.reshape(prow, C).astype(np.uint32), prow, C, C, bits)
    assert np.array_equal(G.to_host(d_out, np.uint32).reshape(pexp.shape), pexp)


# ---- quantizing epilogues without int32 side inputs (the register-resident output stage of the
# ---- matrix-core kernels), every code width it serves ------------------------------------------------
@pytest.mark.parametrize("mode", ["bn", "lowbits"])
@pytest.mark.parametrize("pool", [0, 1, 2])
@pytest.mark.parametrize("xb,ob", [(2, 1), (2, 2), (2, 3), (3, 3), (4, 4), (4, 1), (3, 2), (2, 4)])
@pytest.mark.parametrize("path,tile", [(2, 1), (2, 2), (2, 3), (2, 7), (2, 4), (2, 5), (2, 8), (1, None), (4, 0), (4, 1),
                                       (4, 4), (5, 1), (5, 3), (5, 7)])
def test_conv_quantize_pack_all_widths(G, path, tile, xb, ob, pool, mode):
    rng = np.random.default_rng(4000 + 100 * xb + 10 * ob + pool + (tile or 0))
    batch, H, Wd, C, cout, wb = 2, 6, 10, (128 if path == 5 or tile == 8 else 64), 96, 1
    X = O.random_planes(rng, xb, batch * H * Wd, C // 32)
    Wt = O.random_planes(rng, wb, cout * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=3, S=3, stride=1, pad=1, halo=0, wb=wb, xb=xb)
    sym = int(mode == "bn")
    acc = O.conv(Wt, X, cwords=C // 32, sym_w=sym, **kw)
    rows = batch * H * Wd if pool == 0 else batch * (H // 2) * (Wd // 2)
    if mode == "bn":
        span = int(np.abs(acc).max())
        thr = np.sort(rng.integers(-span, span, size=(cout, 2 ** ob - 1)), axis=1).astype(np.int32)
        thr[1] = thr[1, 0]                      # a channel whose thresholds coincide
        flip = rng.integers(0, 2, size=cout).astype(np.uint8)
        d_thr, d_flip = G.to_dev(thr), G.to_dev(flip)
        epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, pool=pool, thr=d_thr, flip=d_flip)
        if pool == 0:
            q = O.bn_quantize(acc.reshape(-1, cout), None, thr, flip, ob)
        elif pool == 1:
            q = O.bn_quantize(O.avgpool2x2(acc).reshape(-1, cout), None, thr, flip, ob)
        else:
            q = O.maxpool2x2(O.bn_quantize(acc.reshape(-1, cout), None, thr, flip, ob).reshape(acc.shape)).reshape(-1, cout)
    else:
        epi = G.epilogue(mode=G.A.EPI_LOWBITS, out_bits=ob, pool=pool)
        mask = (1 << ob) - 1
        if pool == 0:
            q = acc.reshape(-1, cout) & mask
        elif pool == 1:
            q = O.avgpool2x2(acc).reshape(-1, cout) & mask
        else:
            q = O.maxpool2x2(acc & mask).reshape(-1, cout)
    got = G.run_conv(Wt, X, cin_pad=C, sym=sym, epi=epi, path=path, tile=tile, **kw).view(np.uint32).reshape(ob, rows, cout // 32)
    assert np.array_equal(got, O.lowbits_pack(q.astype(np.int32), rows, cout, ob))


@pytest.mark.parametrize("sym", [0, 1])
@pytest.mark.parametrize("wb,xb,ob", [(1, 2, 2), (1, 2, 1), (1, 3, 3), (1, 4, 4), (2, 2, 2), (1, 2, 4)])
@pytest.mark.parametrize("path,tile", [(2, 1), (2, 2), (2, 3), (2, 6), (2, 5), (3, 2), (1, None), (5, 1), (5, 2), (5, 6)])
def test_gemm_quantize_pack_all_widths(G, path, tile, wb, xb, ob, sym):
    rng = np.random.default_rng(4100 + 100 * xb + 10 * ob + sym + (tile or 0))
    M, N, K = 80, 192, 384
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    acc = O.gemm(W, X, M, N, K, wb, xb, sym_w=sym)
    lo, hi = int(acc.min()), int(acc.max())
    thr = np.sort(rng.integers(lo, hi + 1, size=(N, 2 ** ob - 1)), axis=1).astype(np.int32)
    flip = rng.integers(0, 2, size=N).astype(np.uint8)
    thr[flip == 1] = -thr[flip == 1, ::-1]
    d_thr, d_flip = G.to_dev(thr), G.to_dev(flip)
    epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr, flip=d_flip)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, epi=epi, path=path, tile=tile).view(np.uint32).reshape(ob, M, N // 32)
    q = O.bn_quantize(acc, None, thr, flip, ob)
    assert 0 < q.mean() < 2 ** ob - 1
    assert np.array_equal(got, O.lowbits_pack(q, M, N, ob))


# ---- further precisions of the reference tree (any-precision kernel) -------------------------------
@pytest.mark.parametrize("wb,xb", [(1, 8), (2, 8), (4, 4), (1, 1)])
def test_gemm_named_entry_more_precisions(G, wb, xb):
    rng = np.random.default_rng(5000 + 10 * wb + xb)
    M, N, K = 64, 96, 256
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    dW, dX, out = G.to_dev(W), G.to_dev(X), G.dev_empty_i32(M * N, fill=-7)
    fn = getattr(G.A.lib(), "apmm_w%da%d" % (wb, xb))
    G.A.check(fn(G.ptr(dW), G.ptr(dX), G.ptr(out), M, N, K, wb, xb, None), "apmm")
    got = G.to_host(out).reshape(M, N)
    assert np.array_equal(got, O.unpack_planes_lsb(W) @ O.unpack_planes_lsb(X).T)
    assert np.array_equal(got, O.gemm(W, X, M, N, K, wb, xb))
    # wrong bit widths for the name are rejected
    assert fn(G.ptr(dW), G.ptr(dX), G.ptr(out), M, N, K, wb + 1, xb, None) == G.A.EINVAL


@pytest.mark.parametrize("wb,xb", [(4, 4), (1, 8), (2, 8)])
@pytest.mark.parametrize("tile", [None, 1, 2, 4])
@pytest.mark.parametrize("sym", [0, 1])
def test_wide_precisions_on_the_matrix_cores(G, wb, xb, tile, sym):
    """w4a4 / w1a8 / w2a8 as FP4 digit pairs (2 x 2, 1 x 4, 1 x 4 MFMAs per block and k-step, weighted by
    the block scale): GEMM and convolution, int32 and quantized packed output, every tile that is built."""
    rng = np.random.default_rng(5300 + 100 * wb + 10 * xb + (tile or 0) + sym)
    M, N, K = 150, 200, 1152
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    acc = O.gemm(W, X, M, N, K, wb, xb, sym_w=sym, nthreads=8)
    if not sym:
        assert np.array_equal(acc, O.unpack_planes_lsb(W) @ O.unpack_planes_lsb(X).T)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, path=2, tile=tile).reshape(M, N)
    assert np.array_equal(got, acc)
    batch, H, Wd, C, cout = 2, 9, 10, 128, 96
    Xc = O.random_planes(rng, xb, batch * H * Wd, C // 32)
    Wc = O.random_planes(rng, wb, cout * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=3, S=3, stride=1, pad=1, halo=0, wb=wb, xb=xb)
    cacc = O.conv(Wc, Xc, cwords=C // 32, sym_w=sym, nthreads=8, **kw)
    assert np.array_equal(G.run_conv(Wc, Xc, cin_pad=C, sym=sym, path=2, tile=tile, **kw).reshape(cacc.shape), cacc)
    for ob in (2, 4, 8):
        span = int(np.abs(cacc).max())
        thr = np.sort(rng.integers(-span if sym else 0, span, size=(cout, 2 ** ob - 1)), axis=1).astype(np.int32)
        d_thr = G.to_dev(thr)
        epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr)
        rows = batch * H * Wd
        gotq = G.run_conv(Wc, Xc, cin_pad=C, sym=sym, epi=epi, path=2, tile=tile, **kw).view(np.uint32).reshape(ob, rows, cout // 32)
        assert np.array_equal(gotq, O.lowbits_pack(O.bn_quantize(cacc.reshape(rows, cout), None, thr, None, ob), rows, cout, ob))
    if tile is None:     # 64 stored channels: 64-bit loads, where only the 64x64 tile is built
        Xn = O.random_planes(rng, xb, batch * H * Wd, 2)
        Wn = O.random_planes(rng, wb, cout * 9, 2)
        nacc = O.conv(Wn, Xn, cwords=2, sym_w=sym, **kw)
        assert np.array_equal(G.run_conv(Wn, Xn, cin_pad=64, sym=sym, path=2, **kw).reshape(nacc.shape), nacc)


@pytest.mark.parametrize("tile", [None, 1, 2, 4])
@pytest.mark.parametrize("sym", [0, 1])
def test_remaining_reference_precisions_on_the_matrix_cores(G, tile, sym):
    """The reference tree's remaining precisions on the FP4 digit kernels: convolution w1a5 (three digits,
    APNN-TC-lib/bmmaTensorCoreGemm/src/61_bmmaTensorCoreGemm.cu:58) and w2a6 (63_bmmaTensorCoreGemm.cu:58),
    GEMM w1a1 (84_bmmaTensorCoreGemm.cu:80), int32 and quantized packed output, every tile that is built."""
    rng = np.random.default_rng(6100 + 10 * (tile or 0) + sym)
    M, N, K = 150, 200, 1152
    W = O.random_planes(rng, 1, M, K // 32)
    X = O.random_planes(rng, 1, N, K // 32)
    acc = O.gemm(W, X, M, N, K, 1, 1, sym_w=sym, nthreads=8)
    assert np.array_equal(G.run_gemm(W, X, M, N, K, 1, 1, sym=sym, path=2, tile=tile).reshape(M, N), acc)
    plan = G.A.Plan()
    d = G.A.GemmDesc(W=0x1000, X=0x1000, D=0x1000, M=1024, N=1024, K=1024, wb=1, xb=1)
    assert G.A.lib().apnn_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 0 and plan.kernel == G.A.KERNEL_MFMA_FP4
    batch, H, Wd, C, cout = 2, 9, 10, 128, 96
    for wb, xb in [(1, 5), (2, 6)]:
        Xc = O.random_planes(rng, xb, batch * H * Wd, C // 32)
        Wc = O.random_planes(rng, wb, cout * 9, C // 32)
        kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=3, S=3, stride=1, pad=1, halo=0, wb=wb, xb=xb)
        cacc = O.conv(Wc, Xc, cwords=C // 32, sym_w=sym, nthreads=8, **kw)
        got = G.run_conv(Wc, Xc, cin_pad=C, sym=sym, path=2, tile=tile, **kw)
        assert np.array_equal(got.reshape(cacc.shape), cacc), (wb, xb)
        rows = batch * H * Wd
        for ob in (2, xb):
            span = int(np.abs(cacc).max())
            thr = np.sort(rng.integers(-span if sym else 0, span, size=(cout, 2 ** ob - 1)), axis=1).astype(np.int32)
            d_thr = G.to_dev(thr)
            epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr)
            gotq = G.run_conv(Wc, Xc, cin_pad=C, sym=sym, epi=epi, path=2, tile=tile, **kw)
            want = O.lowbits_pack(O.bn_quantize(cacc.reshape(rows, cout), None, thr, None, ob), rows, cout, ob)
            assert np.array_equal(gotq.view(np.uint32).reshape(ob, rows, cout // 32), want), (wb, xb, ob)
        c = G.A.ConvDesc(W=0x1000, X=0x1000, O=0x1000, batch=16, H=16, Wd=16, cin_pad=256, COUT=256, R=3, S=3, stride=1,
                         pad=1, halo=1, wb=wb, xb=xb)
        assert G.A.lib().apnn_conv_plan(ctypes.byref(c), ctypes.byref(plan)) == 0 and plan.kernel == G.A.KERNEL_MFMA_FP4


def test_fp4_guard_falls_back_to_int32_accumulation(G):
    """K * 15 >= 2^24 for w1a4: all-ones operands make every output K * 15, which fp32 cannot hold.  The
    library's own choice must still be exact (int8 core); the FP4 path refuses."""
    M = N = 288
    K = 1179648
    W = np.full((1, M, K // 32), 0xFFFFFFFF, np.uint32)
    X = np.full((4, N, K // 32), 0xFFFFFFFF, np.uint32)
    assert K * 15 >= 2 ** 24
    plan = G.A.Plan()
    d = G.A.GemmDesc(W=0x1000, X=0x1000, D=0x1000, M=M, N=N, K=K, wb=1, xb=4)
    assert G.A.lib().apnn_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 0 and plan.kernel == G.A.KERNEL_MFMA_I8
    assert np.all(G.run_gemm(W, X, M, N, K, 1, 4, path=0) == K * 15)
    with pytest.raises(G.A.ApnnError, match="EUNSUPPORTED"):
        G.run_gemm(W, X, M, N, K, 1, 4, path=2)
    # random weights against one all-ones activation row: popcounts of the weight rows times 15
    Wr = O.random_planes(np.random.default_rng(5), 1, M, K // 32)
    got = G.run_gemm(Wr, X, M, N, K, 1, 4, path=0).reshape(M, N)
    pop = np.array([int(np.unpackbits(Wr[0, m].view(np.uint8)).sum()) for m in range(M)])
    assert np.array_equal(got, np.repeat((15 * pop)[:, None], N, axis=1))


def test_device_error_word_stays_clear(G):
    """apnn_device_error: after patch-resident convolutions on every tile shape (the only kernel that can
    report: a patch larger than the capacity the host computed) the current device's error word reads 0,
    and the results are the oracle's."""
    rng = np.random.default_rng(77)
    batch, H, Wd, C, cout = 3, 12, 10, 64, 128
    X = O.random_planes(rng, 2, batch * H * Wd, C // 32)
    Wt = O.random_planes(rng, 1, cout * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=3, S=3, stride=1, pad=1, halo=0, wb=1, xb=2)
    ref = O.conv(Wt, X, cwords=C // 32, sym_w=1, **kw)
    code = ctypes.c_int(-1)
    assert G.A.lib().apnn_device_error(ctypes.byref(code), None) == 0   # whatever earlier tests left
    for tile in range(5):
        got = G.run_conv(Wt, X, cin_pad=C, sym=1, path=G.A.PATH_MFMA_PATCH, tile=tile, **kw)
        assert np.array_equal(got.reshape(ref.shape), ref), tile
    code = ctypes.c_int(-1)
    assert G.A.lib().apnn_device_error(ctypes.byref(code), None) == 0 and code.value == 0
    assert G.A.lib().apnn_device_error(None, None) == G.A.ENULL


@pytest.mark.parametrize("wb,xb", [(1, 2), (1, 3), (1, 4), (2, 2)])
def test_fp4_exact_just_below_the_accumulation_limit(G, wb, xb):
    """The FP4 matrix-core kernels accumulate in fp32 (raw / 4, exact while raw < 2^24).  At the largest
    128-multiple K the host still admits (K * (2^w-1) * (2^a-1) just below 2^24) every way of summing on
    that core has to be exact: a tile whose waves tile the output, a split-K tile (four partial fp32 sums
    meet in LDS), the expand-while-staging kernel, with unsigned and symmetric weights -- on all-ones
    operands (every output equals the closed form K * span, the largest value the guard admits) and on
    random operands against the oracle.  The fp32 threshold compare of the quantizing epilogue is pinned
    at the same magnitude with thresholds at K*span - 1, K*span, K*span + 1 and beyond 2^24."""
    span = (2 ** wb - 1) * (2 ** xb - 1)
    K = ((2 ** 24 - 1) // span) // 128 * 128
    assert K * span < 2 ** 24 <= (K + 128) * span
    M = N = 64
    wmax = 2 ** wb - 1
    ones_w = np.full((wb, M, K // 32), 0xFFFFFFFF, np.uint32)
    ones_x = np.full((xb, N, K // 32), 0xFFFFFFFF, np.uint32)
    rng = np.random.default_rng(2400 + 10 * wb + xb)
    rand_w = O.random_planes(rng, wb, M, K // 32)
    rand_x = O.random_planes(rng, xb, N, K // 32)
    refs = {sym: O.gemm(rand_w, rand_x, M, N, K, wb, xb, sym_w=sym, nthreads=8) for sym in (0, 1)}
    # path, pinned tile: 64x64 (waves tile the output), 32x32 split-K, expand-while-staging 64x64
    variants = [(G.A.PATH_MFMA, 2), (G.A.PATH_MFMA, 4), (G.A.PATH_MFMA_XS, 2)]
    for path, tile in variants:
        plan = G.A.Plan()
        d = G.A.GemmDesc(W=0x1000, X=0x1000, D=0x1000, M=M, N=N, K=K, wb=wb, xb=xb, path=path | ((tile + 1) << 8))
        assert G.A.lib().apnn_gemm_plan(ctypes.byref(d), ctypes.byref(plan)) == 0 and plan.fp4_exact == 1
        for sym in (0, 1):
            got = G.run_gemm(ones_w, ones_x, M, N, K, wb, xb, sym=sym, path=path, tile=tile)
            # all-ones weights are +wmax in both conventions: 2*K*span - wmax*K*(2^a-1) == K*span
            assert np.all(got == K * span), (path, tile, sym, int(got.min()), int(got.max()))
            got = G.run_gemm(rand_w, rand_x, M, N, K, wb, xb, sym=sym, path=path, tile=tile).reshape(M, N)
            assert np.array_equal(got, refs[sym]), (path, tile, sym)
    # quantizing epilogue, flip unset: thresholds around the one value every output takes
    v = K * span
    rows = {0: [v + 1, v + 2, 2 ** 24 + 5], 1: [v, v + 1, 2 ** 24 + 5], 2: [v - 1, v, 2 ** 24 + 5],
            3: [-2 ** 24 - 5, v - 2, v]}
    nt = 2 ** xb - 1
    thr = np.zeros((N, nt), np.int64)
    want_code = np.zeros(N, np.int64)
    for c in range(N):
        t3 = rows[c % 4]
        # codes wider than two bits: pad with thresholds no value reaches
        thr[c] = t3 + [2 ** 24 + 6 + k for k in range(nt - 3)]
        want_code[c] = c % 4
    thr = thr.astype(np.int32)
    d_thr = G.to_dev(thr)
    q = O.bn_quantize(np.full((M, N), v, np.int32), None, thr, None, xb)
    assert np.array_equal(q, np.repeat(want_code[None, :], M, axis=0))
    want = O.lowbits_pack(q, M, N, xb)
    for path, tile in variants[:2]:
        for sym in (0, 1):
            epi = G.epilogue(mode=G.A.EPI_BN, out_bits=xb, thr=d_thr)
            got = G.run_gemm(ones_w, ones_x, M, N, K, wb, xb, sym=sym, epi=epi, path=path, tile=tile)
            assert np.array_equal(got.view(np.uint32).reshape(xb, M, N // 32), want), (path, tile, sym)


@pytest.mark.parametrize("name,wb,xb,pack", [("apconv_w1a5", 1, 5, False), ("apconv_w2a6", 2, 6, False),
                                             ("apconv_w1a8", 1, 8, False), ("apconv_w2a8", 2, 8, False),
                                             ("APConv_w2a8_pack", 2, 8, True)])
def test_conv_named_entry_more_precisions(G, name, wb, xb, pack):
    rng = np.random.default_rng(5100 + 10 * wb + xb)
    H, Wd, C, cout = 6, 8, 128, 64
    X = O.random_planes(rng, xb, (H + 2) * (Wd + 2), C // 32)
    Xv = X.reshape(xb, H + 2, Wd + 2, C // 32)
    Xv[:, 0], Xv[:, -1], Xv[:, :, 0], Xv[:, :, -1] = 0, 0, 0, 0
    Wt = O.random_planes(rng, wb, cout * 9, C // 32)
    kw = dict(batch=1, H=H, W=Wd, cout=cout, R=3, S=3, stride=1, pad=1, halo=1, wb=wb, xb=xb)
    acc = O.conv(Wt, X, cwords=C // 32, **kw)
    dW, dX = G.to_dev(Wt), G.to_dev(X)
    words = xb * H * Wd * cout // 32 if pack else H * Wd * cout
    out = G.dev_empty_i32(words, fill=-7)
    G.A.check(getattr(G.A.lib(), name)(G.ptr(dW), G.ptr(dX), G.ptr(out), H, Wd, C, cout, None), name)
    if pack:
        expect = O.lowbits_pack(acc.reshape(-1, cout), H * Wd, cout, xb)
        assert np.array_equal(G.to_host(out, np.uint32).reshape(expect.shape), expect)
        # 2x2 average pool (C integer division) before the low bits: APConv_w2a8_pack_pool
        outq = G.dev_empty_i32(xb * (H // 2) * (Wd // 2) * cout // 32, fill=-7)
        G.A.check(getattr(G.A.lib(), name + "_pool")(G.ptr(dW), G.ptr(dX), G.ptr(outq), H, Wd, C, cout, None), name)
        pooled = O.avgpool2x2(acc)[0]
        expq = O.lowbits_pack(pooled, (H // 2) * (Wd // 2), cout, xb)
        assert np.array_equal(G.to_host(outq, np.uint32).reshape(expq.shape), expq)
    else:
        assert np.array_equal(G.to_host(out).reshape(acc.shape), acc)


@pytest.mark.parametrize("wb,xb,ob", [(3, 5, 4), (8, 8, 2), (1, 7, 3), (5, 1, 1)])
@pytest.mark.parametrize("sym", [0, 1])
def test_any_precision_descriptor_paths(G, wb, xb, ob, sym):
    """apnn_gemm / apnn_conv at bit widths without a dedicated kernel: AUTO and the VALU path serve
    them (bit-exact, all epilogues), the matrix-core paths report APNN_EUNSUPPORTED."""
    rng = np.random.default_rng(5200 + 100 * wb + 10 * xb + sym)
    M, N, K = 40, 64, 128
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    acc = O.gemm(W, X, M, N, K, wb, xb, sym_w=sym)
    for path in (0, 1):
        assert np.array_equal(G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, path=path).reshape(M, N), acc)
    with pytest.raises(G.A.ApnnError, match="EUNSUPPORTED"):
        G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, path=2)
    thr = np.sort(rng.integers(int(acc.min()), int(acc.max()) + 1, size=(N, 2 ** ob - 1)), axis=1).astype(np.int32)
    d_thr = G.to_dev(thr)
    epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, epi=epi).view(np.uint32).reshape(ob, M, N // 32)
    assert np.array_equal(got, O.lowbits_pack(O.bn_quantize(acc, None, thr, None, ob), M, N, ob))
    # convolution, stride 2, 32 stored channels
    batch, H, Wd, C, cout = 2, 9, 7, 32, 40
    Xc = O.random_planes(rng, xb, batch * H * Wd, C // 32)
    Wc = O.random_planes(rng, wb, cout * 9, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=3, S=3, stride=2, pad=1, halo=0, wb=wb, xb=xb)
    expect = O.conv(Wc, Xc, cwords=C // 32, sym_w=sym, **kw)
    assert np.array_equal(G.run_conv(Wc, Xc, cin_pad=C, sym=sym, **kw).reshape(expect.shape), expect)
    with pytest.raises(G.A.ApnnError, match="EUNSUPPORTED"):
        G.run_conv(Wc, Xc, cin_pad=C, sym=sym, path=4, **kw)


@pytest.mark.parametrize("rows,C,cpad", [(37, 3, 32), (50, 70, 128), (8, 256, 256)])
def test_quantize_pack_u8_and_binarize(G, rows, C, cpad):
    """uint8 samples -> top bits as codes -> planes; float rows -> one plane of (x >= 0) (In128Layer)."""
    rng = np.random.default_rng(6100 + rows)
    v = rng.integers(0, 256, size=(rows, C), dtype=np.uint8)
    dV = torch.from_numpy(v).cuda()
    for bits in (1, 2, 3, 8):
        planes = G.dev_empty_i32(bits * rows * cpad // 32, fill=-7)
        G.A.check(G.A.lib().apnn_quantize_pack_u8(G.ptr(dV), G.ptr(planes), rows, C, cpad, bits, None), "quantize_pack_u8")
        expect = O.pack_bits((v >> (8 - bits)).astype(np.uint32), rows, C, cpad, bits)
        assert np.array_equal(G.to_host(planes, np.uint32).reshape(expect.shape), expect)
    x = rng.normal(size=(rows, C)).astype(np.float32)
    x[0, :3] = [0.0, -0.0, np.float32(-1e-30)]
    dX = torch.from_numpy(x).cuda()
    planes = G.dev_empty_i32(rows * cpad // 32, fill=-7)
    G.A.check(G.A.lib().apnn_binarize_pack(G.ptr(dX), G.ptr(planes), rows, C, cpad, None), "binarize_pack")
    expect = O.pack_bits((x >= 0).astype(np.uint32), rows, C, cpad, 1)
    assert np.array_equal(G.to_host(planes, np.uint32).reshape(expect.shape), expect)


@pytest.mark.parametrize("pool", [0, 1])
@pytest.mark.parametrize("B,Ho,Wo,pitch,channels,cout", [(2, 7, 5, 64, 64, 64), (3, 4, 6, 128, 64, 128), (1, 3, 3, 40, 33, 70),
                                                     (2, 14, 14, 128, 128, 256)])
def test_residual_prepare(G, B, Ho, Wo, pitch, channels, cout, pool):
    rng = np.random.default_rng(6200 + Ho + cout + pool)
    f = 2 if pool else 1
    src = rng.integers(-50000, 50000, size=(B, Ho * f, Wo * f, pitch)).astype(np.int32)
    d_in = G.to_dev(src)
    d_out = G.dev_empty_i32(B * Ho * Wo * cout, fill=-7)
    G.A.check(G.A.lib().apnn_residual_prepare(G.ptr(d_in), G.ptr(d_out), B, Ho, Wo, pitch, channels, cout, pool, None),
              "residual_prepare")
    m = src.reshape(B, Ho, 2, Wo, 2, pitch).max(axis=(2, 4)) if pool else src
    expect = np.zeros((B, Ho, Wo, cout), np.int32)
    expect[..., :channels] = m[..., :channels]
    assert np.array_equal(G.to_host(d_out).reshape(expect.shape), expect)


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("rows,C,cpad", [(37, 3, 32), (50, 70, 128), (8, 256, 256)])
def test_quantize_pack(G, bits, rows, C, cpad):
    """Float image / feature map -> affine codes -> bit-planes in one kernel (Quantize_val + Bit_compression)."""
    rng = np.random.default_rng(6000 + bits + rows)
    x = rng.uniform(-12, 12, size=(rows, C)).astype(np.float32)
    x[0, :] = np.linspace(-10, 10, C, dtype=np.float32)            # includes both end points
    x[1, :] = (-10.0 + 20.0 * (np.arange(C) % (2 ** bits) + 0.5) / 2 ** bits).astype(np.float32)   # ties
    dX = torch.from_numpy(x).cuda()
    planes = G.dev_empty_i32(bits * rows * cpad // 32, fill=-7)
    G.A.check(G.A.lib().apnn_quantize_pack(G.ptr(dX), G.ptr(planes), rows, C, cpad, bits, -10.0, 10.0, None), "quantize_pack")
    codes = O.quantize_val(x, bits)
    expect = O.pack_bits(codes, rows, C, cpad, bits)
    assert np.array_equal(G.to_host(planes, np.uint32).reshape(expect.shape), expect)


@pytest.mark.parametrize("sym", [0, 1])
@pytest.mark.parametrize("wb,xb", COMBOS)
@pytest.mark.parametrize("M,N,K", [(64, 1024, 1024), (50, 36, 128), (1, 4, 2048), (64, 128, 1536), (7, 260, 640), (8, 64, 9216),
                                   (61, 1060, 512), (30, 2052, 768)])
def test_gemm_register_only_kernel(G, M, N, K, wb, xb, sym):
    """The latency-oriented GEMM kernel (eight or four lanes split K for four outputs), pinned as VALU tile 4."""
    rng = np.random.default_rng(7000 + M + N + K + 10 * wb + xb + sym)
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, path=1, tile=4).reshape(M, N)
    assert np.array_equal(got, O.gemm(W, X, M, N, K, wb, xb, sym_w=sym))


def test_gemm_register_only_kernel_limits(G):
    rng = np.random.default_rng(7100)
    W = O.random_planes(rng, 1, 8, 4)
    X = O.random_planes(rng, 2, 6, 4)
    with pytest.raises(G.A.ApnnError, match="EUNSUPPORTED"):     # N % 4 != 0
        G.run_gemm(W, X, 8, 6, 128, 1, 2, path=1, tile=4)
    assert np.array_equal(G.run_gemm(W, X, 8, 6, 128, 1, 2).reshape(8, 6), O.gemm(W, X, 8, 6, 128, 1, 2))
    X = O.random_planes(rng, 2, 32, 4)
    resid = G.to_dev(np.zeros((8, 32), np.int32))
    d_thr = G.to_dev(np.zeros((32, 3), np.int32))
    with pytest.raises(G.A.ApnnError, match="EUNSUPPORTED"):     # no residual input in this kernel
        G.run_gemm(W, X, 8, 32, 128, 1, 2, epi=G.epilogue(mode=G.A.EPI_BN, out_bits=2, thr=d_thr, resid=resid),
                   path=1, tile=4)


@pytest.mark.parametrize("sym", [0, 1])
@pytest.mark.parametrize("wb,xb,ob", [(1, 2, 2), (1, 4, 4), (2, 2, 1), (1, 3, 3)])
@pytest.mark.parametrize("M,N,K", [(64, 1024, 1024), (9, 96, 4096), (5, 32, 384), (61, 1056, 512), (33, 2080, 896)])
def test_gemm_register_only_kernel_packed(G, M, N, K, wb, xb, ob, sym):
    rng = np.random.default_rng(7200 + M + N + 10 * wb + xb + sym)
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    acc = O.gemm(W, X, M, N, K, wb, xb, sym_w=sym)
    thr = np.sort(rng.integers(int(acc.min()), int(acc.max()) + 1, size=(N, 2 ** ob - 1)), axis=1).astype(np.int32)
    flip = rng.integers(0, 2, size=N).astype(np.uint8)
    thr[flip == 1] = -thr[flip == 1, ::-1]
    d_thr, d_flip = G.to_dev(thr), G.to_dev(flip)
    epi = G.epilogue(mode=G.A.EPI_BN, out_bits=ob, thr=d_thr, flip=d_flip)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, epi=epi, path=1, tile=4).view(np.uint32).reshape(ob, M, N // 32)
    assert np.array_equal(got, O.lowbits_pack(O.bn_quantize(acc, None, thr, flip, ob), M, N, ob))
    epi = G.epilogue(mode=G.A.EPI_LOWBITS, out_bits=ob)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=sym, epi=epi, path=1, tile=4).view(np.uint32).reshape(ob, M, N // 32)
    assert np.array_equal(got, O.lowbits_pack(acc & (2 ** ob - 1), M, N, ob))


@pytest.mark.parametrize("path,tile", [(1, 4), (0, None), (2, None)])
@pytest.mark.parametrize("wb,xb", COMBOS)
@pytest.mark.parametrize("batch,H,Wd,C,cout", [(8, 6, 6, 256, 512), (3, 7, 7, 128, 96), (16, 1, 1, 1024, 256)])
def test_fully_connected_layer_as_convolution(G, batch, H, Wd, C, cout, wb, xb, path, tile):
    """Filter spans the feature map: AUTO / the pinned register-only kernel treat it as a GEMM over whole
    images; int32 and quantized packed output against the oracle convolution."""
    rng = np.random.default_rng(7300 + batch + C + 10 * wb + xb)
    X = O.random_planes(rng, xb, batch * H * Wd, C // 32)
    Wt = O.random_planes(rng, wb, cout * H * Wd, C // 32)
    kw = dict(batch=batch, H=H, W=Wd, cout=cout, R=H, S=Wd, stride=1, pad=0, halo=0, wb=wb, xb=xb)
    acc = O.conv(Wt, X, cwords=C // 32, sym_w=1, **kw).reshape(batch, cout)
    got = G.run_conv(Wt, X, cin_pad=C, sym=1, path=path, tile=tile, **kw).reshape(batch, cout)
    assert np.array_equal(got, acc)
    thr = np.sort(rng.integers(int(acc.min()), int(acc.max()) + 1, size=(cout, 3)), axis=1).astype(np.int32)
    d_thr = G.to_dev(thr)
    epi = G.epilogue(mode=G.A.EPI_BN, out_bits=2, thr=d_thr)
    got = G.run_conv(Wt, X, cin_pad=C, sym=1, epi=epi, path=path, tile=tile, **kw).view(np.uint32).reshape(2, batch, cout // 32)
    assert np.array_equal(got, O.lowbits_pack(O.bn_quantize(acc, None, thr, None, 2), batch, cout, 2))


@pytest.mark.parametrize("batch,H,C,cout", [(8, 28, 128, 256), (64, 14, 256, 512), (2, 56, 64, 128), (1, 8, 128, 64)])
@pytest.mark.parametrize("wb,xb", [(1, 2), (2, 2), (1, 4)])
def test_conv_pair_residual_block_entry(G, batch, H, C, cout, wb, xb):
    """3x3 stride-2 convolution and 1x1 stride-2 downsample of the same input in one call: each output
    equals the convolution launched on its own (and the oracle)."""
    rng = np.random.default_rng(8000 + batch + H + 10 * wb + xb)
    X = O.random_planes(rng, xb, batch * H * H, C // 32)
    W3 = O.random_planes(rng, wb, cout * 9, C // 32)
    W1 = O.random_planes(rng, wb, cout, C // 32)
    k3 = dict(batch=batch, H=H, W=H, cout=cout, R=3, S=3, stride=2, pad=1, halo=0, wb=wb, xb=xb)
    k1 = dict(batch=batch, H=H, W=H, cout=cout, R=1, S=1, stride=2, pad=0, halo=0, wb=wb, xb=xb)
    acc3 = O.conv(W3, X, cwords=C // 32, sym_w=1, nthreads=8, **k3).reshape(-1, cout)
    acc1 = O.conv(W1, X, cwords=C // 32, sym_w=1, nthreads=8, **k1).reshape(-1, cout)
    rows = acc3.shape[0]
    assert acc1.shape[0] == rows
    nt = 2 ** xb - 1
    thr3 = np.sort(rng.integers(int(acc3.min()), int(acc3.max()) + 1, size=(cout, nt)), axis=1).astype(np.int32)
    thr1 = np.sort(rng.integers(int(acc1.min()), int(acc1.max()) + 1, size=(cout, nt)), axis=1).astype(np.int32)
    dX, dW3, dW1, dT3, dT1 = G.to_dev(X), G.to_dev(W3), G.to_dev(W1), G.to_dev(thr3), G.to_dev(thr1)
    words = xb * rows * cout // 32
    o3, o1 = G.dev_empty_i32(words, fill=-7), G.dev_empty_i32(words, fill=-7)
    A = G.A
    def desc(Wd_, out, R, pad, thr):
        return A.ConvDesc(W=Wd_.data_ptr(), X=dX.data_ptr(), O=out.data_ptr(), batch=batch, H=H, Wd=H, cin_pad=C,
                          COUT=cout, R=R, S=R, stride=2, pad=pad, halo=0, wb=wb, xb=xb, weight_mode=A.WEIGHT_SYMMETRIC,
                          epi=G.epilogue(mode=A.EPI_BN, out_bits=xb, thr=thr), path=A.PATH_AUTO)
    da, db = desc(dW3, o3, 3, 1, dT3), desc(dW1, o1, 1, 0, dT1)
    A.check(A.lib().apnn_conv_pair(ctypes.byref(da), ctypes.byref(db), None), "apnn_conv_pair")
    e3 = O.lowbits_pack(O.bn_quantize(acc3, None, thr3, None, xb), rows, cout, xb)
    e1 = O.lowbits_pack(O.bn_quantize(acc1, None, thr1, None, xb), rows, cout, xb)
    assert np.array_equal(G.to_host(o3, np.uint32).reshape(e3.shape), e3)
    assert np.array_equal(G.to_host(o1, np.uint32).reshape(e1.shape), e1)
    # descriptors that do not describe the same input / output grid are rejected
    bad = desc(dW1, o1, 1, 0, dT1)
    bad.stride = 1
    assert A.lib().apnn_conv_pair(ctypes.byref(da), ctypes.byref(bad), None) == A.EINVAL


@pytest.mark.parametrize("M,N,path,tile", [
    (1500, 3022, 2, 1),    # 12 x 24 tiles of 128x128: one full band of eight tile rows and a band of four
    (1100, 4000, 2, 1),    # 9 x 32: a band of eight and a band of one
    (1100, 4000, 3, 1),    # the same grid on the int8 core
    (2048, 2048, 2, 9),    # 16 x 16 on the two-wave-group tile
    (520, 4090, 2, 2),     # 9 x 64 tiles of 64x64
    (3000, 1400, 2, 3),    # 24 x 22 tiles of 128x64
    (2530, 4096, 2, 6)])   # 10 x 32 tiles of 256x128: a band of eight and a band of two
def test_gemm_grids_walked_in_xcd_order(G, M, N, path, tile):
    """Grids of at least 256 tiles whose size is a multiple of eight are walked in per-XCD ranges, in
    bands of eight tile rows (the work-group index is regrouped inside the kernel): every tile, ragged
    edges included, is computed exactly once -- the whole output equals the oracle's, and nothing is
    written outside it (guard bytes)."""
    K, wb, xb = 256, 1, 2
    rng = np.random.default_rng(8200 + M + N + tile)
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    ref = O.gemm(W, X, M, N, K, wb, xb, sym_w=1, nthreads=8)
    got = G.run_gemm(W, X, M, N, K, wb, xb, sym=1, path=path, tile=tile).reshape(M, N)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("batch,H,C,cout,stride", [(4, 14, 256, 128, 1), (3, 20, 128, 256, 2), (16, 14, 64, 64, 1)])
def test_conv_pair_two_filter_sizes(G, batch, H, C, cout, stride):
    """apnn_conv_pair with two filters that both span several taps and differ in width (5x5 pad 2 and 3x3
    pad 1 produce the same output grid): the second problem decodes its taps with its own filter width."""
    rng = np.random.default_rng(8100 + batch + H)
    wb, xb = 1, 2
    X = O.random_planes(rng, xb, batch * H * H, C // 32)
    W5 = O.random_planes(rng, wb, cout * 25, C // 32)
    W3 = O.random_planes(rng, wb, cout * 9, C // 32)
    k5 = dict(batch=batch, H=H, W=H, cout=cout, R=5, S=5, stride=stride, pad=2, halo=0, wb=wb, xb=xb)
    k3 = dict(batch=batch, H=H, W=H, cout=cout, R=3, S=3, stride=stride, pad=1, halo=0, wb=wb, xb=xb)
    acc5 = O.conv(W5, X, cwords=C // 32, sym_w=1, nthreads=8, **k5).reshape(-1, cout)
    acc3 = O.conv(W3, X, cwords=C // 32, sym_w=1, nthreads=8, **k3).reshape(-1, cout)
    rows = acc5.shape[0]
    assert acc3.shape[0] == rows
    thr5 = np.sort(rng.integers(int(acc5.min()), int(acc5.max()) + 1, size=(cout, 3)), axis=1).astype(np.int32)
    thr3 = np.sort(rng.integers(int(acc3.min()), int(acc3.max()) + 1, size=(cout, 3)), axis=1).astype(np.int32)
    dX, dW5, dW3, dT5, dT3 = G.to_dev(X), G.to_dev(W5), G.to_dev(W3), G.to_dev(thr5), G.to_dev(thr3)
    words = xb * rows * cout // 32
    A = G.A
    def desc(Wd_, out, R, pad, thr):
        return A.ConvDesc(W=Wd_.data_ptr(), X=dX.data_ptr(), O=out.data_ptr(), batch=batch, H=H, Wd=H, cin_pad=C,
                          COUT=cout, R=R, S=R, stride=stride, pad=pad, halo=0, wb=wb, xb=xb,
                          weight_mode=A.WEIGHT_SYMMETRIC, epi=G.epilogue(mode=A.EPI_BN, out_bits=xb, thr=thr),
                          path=A.PATH_AUTO)
    e5 = O.lowbits_pack(O.bn_quantize(acc5, None, thr5, None, xb), rows, cout, xb)
    e3 = O.lowbits_pack(O.bn_quantize(acc3, None, thr3, None, xb), rows, cout, xb)
    for first_is_5 in (True, False):
        o5, o3 = G.dev_empty_i32(words, fill=-7), G.dev_empty_i32(words, fill=-7)
        d5, d3 = desc(dW5, o5, 5, 2, dT5), desc(dW3, o3, 3, 1, dT3)
        da, db = (d5, d3) if first_is_5 else (d3, d5)
        A.check(A.lib().apnn_conv_pair(ctypes.byref(da), ctypes.byref(db), None), "apnn_conv_pair")
        assert np.array_equal(G.to_host(o5, np.uint32).reshape(e5.shape), e5), first_is_5
        assert np.array_equal(G.to_host(o3, np.uint32).reshape(e3.shape), e3), first_is_5
