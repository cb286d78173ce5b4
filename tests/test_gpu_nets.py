"""End-to-end networks: every layer's GPU output is compared, bit-exactly, with the CPU oracle applied
to that layer's actual GPU input (so layer-by-layer agreement implies end-to-end agreement)."""
import ctypes

import numpy as np
import pytest

import oracle_lib as O

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def G():
    import gpu_util
    assert torch.cuda.is_available()
    return gpu_util


def _download(L, ptr, count, dtype):
    host = np.empty(count, dtype)
    rc = L.apnn_nn_download(host.ctypes.data, ptr, host.nbytes)
    assert rc == 0
    return host


def _maxpool_codes(codes, win, stride, pad):
    B, H, W, C = codes.shape
    Ho, Wo = (H + 2 * pad - win) // stride + 1, (W + 2 * pad - win) // stride + 1
    padded = np.zeros((B, H + 2 * pad, W + 2 * pad, C), codes.dtype)
    padded[:, pad:pad + H, pad:pad + W] = codes
    out = np.zeros((B, Ho, Wo, C), codes.dtype)
    for r in range(win):
        for s in range(win):
            out = np.maximum(out, padded[:, r:r + stride * (Ho - 1) + 1:stride, s:s + stride * (Wo - 1) + 1:stride])
    return out


def _check_network(G, kind, batch, path, graph):
    A = G.A
    L = A.nn_lib()
    net = L.apnn_net_create(kind, batch, 1234, path)
    assert net, "network construction failed"
    try:
        rng = np.random.default_rng(77)
        images = rng.integers(0, 256, size=(batch, 224, 224, 3), dtype=np.uint8)
        d_img = torch.from_numpy(images).cuda()
        d_logits = torch.full((batch, 1000), -1.0, dtype=torch.float32, device="cuda")
        fwd = L.apnn_net_forward_graph if graph else L.apnn_net_forward
        for _ in range(2 if graph else 1):      # a graph is replayed at least once after its capture
            A.check(fwd(net, d_img.data_ptr(), d_logits.data_ptr(), None), "forward")
            torch.cuda.synchronize()
        n = L.apnn_net_layer_count(net)
        descs = []
        for i in range(n):
            d = A.LayerDesc()
            assert L.apnn_net_layer(net, i, ctypes.byref(d)) == 0
            descs.append(d)
        for i, d in enumerate(descs):
            nt = (1 << d.out_bits) - 1 if d.kind != A.LAYER_OUT_I8 else 0
            name = d.name.decode()
            if d.kind == A.LAYER_IMAGE_QUANT:
                rows = batch * d.in_h * d.in_w
                codes = (images.reshape(rows, d.in_c) >> (8 - d.out_bits)).astype(np.uint32)
                expect = O.pack_bits(codes, rows, d.in_c, d.out_cpad, d.out_bits)
                got = _download(L, d.output, expect.size, np.uint32).reshape(expect.shape)
                assert np.array_equal(got, expect), name
            elif d.kind == A.LAYER_INCONV_I8:
                Wt = _download(L, d.weights, d.out_c * d.R * d.S * d.in_c, np.int8).reshape(d.out_c, d.R, d.S, d.in_c)
                thr = _download(L, d.thresholds, d.out_c * nt, np.int32).reshape(d.out_c, nt)
                x = (images.astype(np.int16) - 128).astype(np.int8)
                acc = O.conv_i8(Wt, x, d.stride, d.pad)
                codes = O.bn_quantize(acc.reshape(-1, d.out_c), None, thr, None, d.out_bits).reshape(acc.shape)
                if d.pool_win:
                    codes = _maxpool_codes(codes, d.pool_win, d.pool_stride, d.pool_pad)
                rows = batch * d.out_h * d.out_w
                assert codes.shape == (batch, d.out_h, d.out_w, d.out_c), name
                expect = O.pack_bits(codes.reshape(rows, d.out_c).astype(np.uint32), rows, d.out_c, d.out_cpad, d.out_bits)
                got = _download(L, d.output, expect.size, np.uint32).reshape(expect.shape)
                assert np.array_equal(got, expect), name
            elif d.kind in (A.LAYER_CONV, A.LAYER_FC):
                cw = d.in_cpad // 32
                X = _download(L, d.input, d.a_bits * batch * d.in_h * d.in_w * cw, np.uint32)
                Wt = _download(L, d.weights, d.w_bits * d.out_c * d.R * d.S * cw, np.uint32)
                thr = _download(L, d.thresholds, d.out_c * nt, np.int32).reshape(d.out_c, nt)
                acc = O.conv(Wt, X, batch=batch, H=d.in_h, W=d.in_w, cwords=cw, cout=d.out_c, R=d.R, S=d.S,
                             stride=d.stride, pad=d.pad, halo=0, wb=d.w_bits, xb=d.a_bits, sym_w=1, nthreads=16)
                if d.shortcut_layer >= 0:
                    sd = descs[d.shortcut_layer]
                    srows = batch * sd.out_h * sd.out_w
                    sp = _download(L, sd.output, sd.out_bits * srows * (sd.out_cpad // 32), np.uint32)
                    sc = O.unpack_bits(sp, srows, sd.out_c, sd.out_cpad, sd.out_bits).astype(np.int32)
                    acc = acc + d.shortcut_scale * sc.reshape(acc.shape)
                if d.residual_layer >= 0:
                    # int32 sums saved by an earlier layer: max-pooled 2x2 where this layer's map is half the
                    # size, added to the first residual_channels channels (APNN-TC-nn/src/kernel.cuh:779-831)
                    sd = descs[d.residual_layer]
                    assert sd.save_residual and sd.out_c == d.residual_pitch, name
                    f = 2 if d.residual_pool else 1
                    Hc, Wc = acc.shape[1], acc.shape[2]
                    assert (sd.out_h, sd.out_w) == (f * Hc, f * Wc), name
                    src = _download(L, sd.residual_out, batch * sd.out_h * sd.out_w * sd.out_c, np.int32)
                    src = src.reshape(batch, sd.out_h, sd.out_w, sd.out_c)
                    if d.residual_pool:
                        src = src.reshape(batch, Hc, 2, Wc, 2, sd.out_c).max(axis=(2, 4))
                    acc = acc.copy()
                    acc[..., :d.residual_channels] += src[..., :d.residual_channels]
                if d.save_residual:
                    saved = _download(L, d.residual_out, acc.size, np.int32).reshape(acc.shape)
                    assert np.array_equal(saved, acc), name + " (saved residual)"
                codes = O.bn_quantize(acc.reshape(-1, d.out_c), None, thr, None, d.out_bits).reshape(acc.shape)
                if d.pool_win:
                    codes = O.maxpool2x2(codes)
                rows = batch * d.out_h * d.out_w
                assert codes.shape == (batch, d.out_h, d.out_w, d.out_c), name
                expect = O.pack_bits(codes.reshape(rows, d.out_c).astype(np.uint32), rows, d.out_c, d.out_cpad, d.out_bits)
                got = _download(L, d.output, expect.size, np.uint32).reshape(expect.shape)
                assert np.array_equal(got, expect), name
            else:
                rows = batch * d.in_h
                planes = _download(L, d.input, d.a_bits * rows * (d.in_cpad // 32), np.uint32)
                codes = O.unpack_bits(planes, rows, d.in_c, d.in_cpad, d.a_bits).astype(np.int64)
                if d.global_pool_shift >= 0:
                    act = np.minimum(127, codes.reshape(batch, d.in_h, d.in_c).sum(1) >> d.global_pool_shift)
                else:
                    act = codes.reshape(batch, d.in_c)
                Wt = _download(L, d.weights, d.out_c * d.in_c, np.int8).astype(np.int64).reshape(d.out_c, d.in_c)
                scale = _download(L, d.scale, d.out_c, np.float32)
                bias = _download(L, d.bias, d.out_c, np.float32)
                acc = act @ Wt.T
                expect = acc.astype(np.float32) * scale[None, :] + bias[None, :]
                got = d_logits.cpu().numpy()
                # one fp32 multiply-add of an exact int32 sum
                assert np.allclose(got, expect, rtol=1e-6, atol=1e-6), name
        return n
    finally:
        L.apnn_net_destroy(net)


@pytest.mark.parametrize("graph", [False, True])
@pytest.mark.parametrize("batch", [8, 64])
def test_resnet18_benchmark_batches(G, batch, graph):
    """Batch 8 and 64 (the benchmark's configurations): the library's kernel choice depends on the batch
    (tile shapes, split-K, the patch-resident kernel), so the small-batch test does not cover them."""
    assert _check_network(G, G.A.NET_RESNET18, batch, 0, graph=graph) == 21


@pytest.mark.parametrize("kind,layers", [("alexnet", 8), ("vgg", 13)])
def test_alexnet_and_vgg_batch8(G, kind, layers):
    net = G.A.NET_ALEXNET if kind == "alexnet" else G.A.NET_VGG
    assert _check_network(G, net, 8, 0, graph=False) == layers
    assert _check_network(G, net, 8, 0, graph=True) == layers


@pytest.mark.parametrize("batch,path,graph", [(2, 0, False), (2, 1, False), (2, 2, False), (8, 0, True)])
def test_reference_style_resnet18(G, batch, path, graph):
    """The reference's own ResNet18 demo, built from its constructor argument lists
    (APNN-TC-nn/src/resnet18.cu:40-142): save_residual / inject_residual / residual_channels /
    residual_pool / ahead_fc all take part, and every layer -- the saved int32 maps included -- is
    compared with the oracle."""
    n = _check_network(G, G.A.NET_RESNET18_REFERENCE, batch, path, graph=graph)
    assert n == 1 + 1 + 16 + 1 + 1      # image quantizer, stem, 16 block convolutions, FC, output


@pytest.mark.parametrize("path", [0, 1, 2])
def test_resnet18_layer_by_layer(G, path):
    n = _check_network(G, G.A.NET_RESNET18, 2, path, graph=False)
    assert n == 1 + 16 + 3 + 1      # stem, 16 block convs, 3 downsample convs, classifier


@pytest.mark.parametrize("path", [0, 2])
def test_alexnet_layer_by_layer(G, path):
    n = _check_network(G, G.A.NET_ALEXNET, 2, path, graph=False)
    assert n == 8


def test_resnet18_graph_replay(G):
    _check_network(G, G.A.NET_RESNET18, 2, 0, graph=True)


@pytest.mark.parametrize("path", [0, 2])
def test_vgg_layer_by_layer(G, path):
    n = _check_network(G, G.A.NET_VGG, 2, path, graph=False)
    assert n == 10 + 2 + 1          # ten convolutions, two hidden FCs, classifier
