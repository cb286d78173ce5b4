"""Pins the CPU oracle: reference-derived known answers, closed forms, and library routines
that share no code with it.  Runs without a GPU."""
import numpy as np
import pytest

import oracle_lib as O


def _golden():
    import os
    return np.load(os.path.join(O.GOLDEN_DIR, "golden_outputs.npz"), allow_pickle=False)


def test_fnv1a64_is_the_published_function():
    """Published FNV-1a-64 test vectors: the empty string is the offset basis, "a" and "foobar"."""
    assert O.fnv1a64(np.zeros(0, np.uint8)) == 0xcbf29ce484222325
    assert O.fnv1a64(np.frombuffer(b"a", np.uint8)) == 0xaf63dc4c8601ec8c
    assert O.fnv1a64(np.frombuffer(b"foobar", np.uint8)) == 0x85944171f73967e8


def _gemm_inputs_from_stream(M, N, K, wb, xb):
    s = O.golden_stream()
    nw, nx = wb * M * K // 32, xb * N * K // 32
    W = s[:nw].reshape(wb, M, K // 32)
    X = s[nw:nw + nx].reshape(xb, N, K // 32)
    return W, X


def _conv_inputs_from_stream(H, Wd, CIN, COUT, wb, xb):
    s = O.golden_stream()
    nx, nw = xb * (H + 2) * (Wd + 2) * CIN // 32, wb * COUT * 9 * CIN // 32
    X = s[:nx].reshape(xb, (H + 2) * (Wd + 2), CIN // 32)
    Wt = s[nx:nx + nw].reshape(wb, COUT, 9 * CIN // 32)
    return Wt, X


@pytest.mark.parametrize("name", ["w1a2", "w1a3", "w1a4", "w2a2"])
def test_gemm_known_answers(name):
    ka = O.known_answers()["gemm"]
    c = ka["cases"][name]
    M, N, K = ka["shape"]["M"], ka["shape"]["N"], ka["shape"]["K"]
    W, X = _gemm_inputs_from_stream(M, N, K, c["wb"], c["xb"])
    for D in (O.gemm_literal(W, X, M, N, K, c["wb"], c["xb"]), O.gemm(W, X, M, N, K, c["wb"], c["xb"])):
        flat = D.ravel()
        assert (int(flat[0]), int(flat[1]), int(flat[-1])) == (c["c0"], c["c1"], c["clast"])
        assert int(flat.astype(np.int64).sum()) == c["sum"]
        assert "%016x" % O.fnv1a64(D.astype("<i4")) == c["fnv"]
    assert "%016x" % O.fnv1a64(_golden()["gemm_" + name].astype("<i4")) == c["fnv"]


@pytest.mark.parametrize("name", ["w1a2", "w1a3", "w1a4", "w2a2"])
def test_conv_known_answers(name):
    ka = O.known_answers()["conv"]
    c = ka["cases"][name]
    sh = ka["shape"]
    H, Wd, CIN, COUT = sh["H"], sh["W"], sh["CIN"], sh["COUT"]
    Wt, X = _conv_inputs_from_stream(H, Wd, CIN, COUT, c["wb"], c["xb"])
    lit = O.conv3x3_literal(Wt, X, H, Wd, CIN, COUT, c["wb"], c["xb"])
    gen = O.conv(Wt, X, batch=1, H=H, W=Wd, cwords=CIN // 32, cout=COUT, R=3, S=3, stride=1, pad=1,
                 halo=1, wb=c["wb"], xb=c["xb"])[0]
    for D in (lit, gen):
        flat = D.ravel()
        assert (int(flat[0]), int(flat[1])) == (c["c0"], c["c1"])
        assert int(flat.astype(np.int64).sum()) == c["sum"]
        assert "%016x" % O.fnv1a64(D.astype("<i4")) == c["fnv"]
    packed = O.lowbits_pack(lit, H * Wd, COUT, c["xb"])
    assert "%08x" % int(packed.ravel()[0]) == c["pack0"]
    assert "%016x" % O.fnv1a64(packed.astype("<u4")) == c["pack_fnv"]
    gold = _golden()
    assert "%016x" % O.fnv1a64(gold["conv_" + name].astype("<i4")) == c["fnv"]
    assert "%016x" % O.fnv1a64(gold["conv_pack_" + name].astype("<u4")) == c["pack_fnv"]


def test_plane_product_kat():
    """others/bit_and_utility.py of the reference: W rows against all-ones X -> popcount(W row),
    combined with 2^(i+j)."""
    kat = O.known_answers()["plane_product_kat"]
    W = np.array([[int(t, 16) for t in row.split()] for row in kat["W"]], np.uint32)
    X = np.array([[int(t, 16) for t in row.split()] for row in kat["X"]], np.uint32)
    # each hex row is one 128-bit row of one plane; treat them as 4 planes of a 1-row operand
    D = O.gemm_literal(W.reshape(4, 1, 4), X.reshape(4, 1, 4), 1, 1, 128, 4, 4)
    pop = [sum(bin(int(w)).count("1") for w in row) for row in W]
    expect = sum(pop[i] * 2 ** (i + j) for i in range(4) for j in range(4))
    assert int(D[0, 0]) == expect


@pytest.mark.parametrize("wb,xb", [(1, 2), (1, 3), (1, 4), (2, 2), (1, 1), (4, 4), (2, 8)])
def test_gemm_vs_integer_matmul(wb, xb):
    rng = np.random.default_rng(100 + 10 * wb + xb)
    M, N, K = 24, 40, 160
    W = O.random_planes(rng, wb, M, K // 32)
    X = O.random_planes(rng, xb, N, K // 32)
    expect = O.unpack_planes_lsb(W) @ O.unpack_planes_lsb(X).T
    assert np.array_equal(O.gemm_literal(W, X, M, N, K, wb, xb), expect)
    assert np.array_equal(O.gemm(W, X, M, N, K, wb, xb), expect)
    assert np.array_equal(O.gemm(W, X, M, N, K, wb, xb, nthreads=4), expect)
    # symmetric weights: wt = 2u - (2^wb - 1)
    wsigned = 2 * O.unpack_planes_lsb(W) - (2 ** wb - 1)
    expect_s = wsigned @ O.unpack_planes_lsb(X).T
    got_s = O.gemm(W, X, M, N, K, wb, xb, sym_w=1)
    assert np.array_equal(got_s, expect_s)
    # D(w) = -D(~w)
    assert np.array_equal(O.gemm(~W, X, M, N, K, wb, xb, sym_w=1), -got_s)


def test_gemm_closed_forms():
    M, N, K = 8, 32, 256
    for wb, xb in [(1, 2), (2, 2), (1, 4)]:
        ones_w = np.full((wb, M, K // 32), 0xFFFFFFFF, np.uint32)
        ones_x = np.full((xb, N, K // 32), 0xFFFFFFFF, np.uint32)
        D = O.gemm(ones_w, ones_x, M, N, K, wb, xb)
        assert np.all(D == K * (2 ** wb - 1) * (2 ** xb - 1))
        rng = np.random.default_rng(7)
        W = O.random_planes(rng, wb, M, K // 32)
        D = O.gemm(W, ones_x, M, N, K, wb, xb)
        rowval = O.unpack_planes_lsb(W).sum(1)
        assert np.array_equal(D, np.repeat((rowval * (2 ** xb - 1))[:, None], N, 1))
    # one-hot rows pick out single elements
    W = np.zeros((1, M, K // 32), np.uint32)
    for m in range(M):
        k = 31 * m + 5
        W[0, m, k // 32] = np.uint32(1) << np.uint32(k % 32)
    X = O.random_planes(np.random.default_rng(8), 2, N, K // 32)
    xv = O.unpack_planes_lsb(X)
    D = O.gemm(W, X, M, N, K, 1, 2)
    for m in range(M):
        assert np.array_equal(D[m], xv[:, 31 * m + 5])


def _np_conv(xv, wv, stride, pad):
    """xv [B][H][W][C] int64 (already zero padded if pad handled by caller), wv [cout][R][S][C]."""
    B, H, W, C = xv.shape
    cout, R, S, _ = wv.shape
    if pad:
        xv = np.pad(xv, ((0, 0), (pad, pad), (pad, pad), (0, 0)))
    Ho, Wo = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - S) // stride + 1
    out = np.zeros((B, Ho, Wo, cout), np.int64)
    for r in range(R):
        for s in range(S):
            patch = xv[:, r:r + stride * (Ho - 1) + 1:stride, s:s + stride * (Wo - 1) + 1:stride, :]
            out += np.einsum("bhwc,oc->bhwo", patch, wv[:, r, s, :])
    return out


@pytest.mark.parametrize("wb,xb,R,stride,pad,halo", [
    (1, 2, 3, 1, 1, 1), (1, 2, 3, 1, 1, 0), (2, 2, 3, 2, 1, 0), (1, 4, 1, 2, 0, 0),
    (1, 3, 5, 1, 2, 0), (1, 2, 1, 1, 0, 0)])
def test_conv_vs_numpy(wb, xb, R, stride, pad, halo):
    rng = np.random.default_rng(200 + wb * 10 + xb + R)
    B, H, Wd, cw, cout = 2, 9, 7, 2, 12
    Hs, Ws = (H + 2 * pad, Wd + 2 * pad) if halo else (H, Wd)
    X = O.random_planes(rng, xb, B * Hs * Ws, cw)
    Wt = O.random_planes(rng, wb, cout * R * R, cw)
    got = O.conv(Wt, X, batch=B, H=H, W=Wd, cwords=cw, cout=cout, R=R, S=R, stride=stride, pad=pad,
                 halo=halo, wb=wb, xb=xb)
    xv = O.unpack_planes_lsb(X).reshape(B, Hs, Ws, cw * 32)
    wv = O.unpack_planes_lsb(Wt).reshape(cout, R, R, cw * 32)
    expect = _np_conv(xv, wv, stride, 0 if halo else pad)
    assert np.array_equal(got, expect)
    got_s = O.conv(Wt, X, batch=B, H=H, W=Wd, cwords=cw, cout=cout, R=R, S=R, stride=stride, pad=pad,
                   halo=halo, wb=wb, xb=xb, sym_w=1, nthreads=3)
    expect_s = _np_conv(xv, 2 * wv - (2 ** wb - 1), stride, 0 if halo else pad)
    assert np.array_equal(got_s, expect_s)


def test_conv_1x1_is_gemm():
    rng = np.random.default_rng(31)
    B, H, Wd, cw, cout = 1, 4, 8, 4, 64
    X = O.random_planes(rng, 2, B * H * Wd, cw)
    Wt = O.random_planes(rng, 1, cout, cw)
    c = O.conv(Wt, X, batch=B, H=H, W=Wd, cwords=cw, cout=cout, R=1, S=1, stride=1, pad=0, halo=0, wb=1, xb=2)
    g = O.gemm(Wt, X, cout, H * Wd, cw * 32, 1, 2)       # D[co][pix]
    assert np.array_equal(c.reshape(H * Wd, cout), g.T)


def test_lowbits_pack_msb_first():
    acc = np.zeros((2, 64), np.int32)
    acc[0, 0] = 1          # bit0 -> plane 0, column 0 -> bit 31
    acc[0, 33] = 2         # bit1 -> plane 1, column 33 -> word 1 bit 30
    acc[1, 31] = 3
    p = O.lowbits_pack(acc, 2, 64, 2)
    assert p[0, 0, 0] == 0x80000000 and p[1, 0, 1] == 0x40000000
    assert p[0, 1, 0] == 1 and p[1, 1, 0] == 1
    rng = np.random.default_rng(5)
    acc = rng.integers(0, 1 << 20, size=(8, 96)).astype(np.int32)
    p = O.lowbits_pack(acc, 8, 96, 3)
    for b in range(3):
        bits = (acc >> b) & 1
        words = bits.reshape(8, 3, 32)
        expect = (words.astype(np.uint64) << (31 - np.arange(32, dtype=np.uint64))).sum(-1).astype(np.uint32)
        assert np.array_equal(p[b], expect)


def test_pools():
    rng = np.random.default_rng(9)
    x = rng.integers(0, 5000, size=(2, 6, 8, 5)).astype(np.int32)
    blocks = x.reshape(2, 3, 2, 4, 2, 5)
    assert np.array_equal(O.avgpool2x2(x), blocks.sum((2, 4)) // 4)
    assert np.array_equal(O.maxpool2x2(x), blocks.max((2, 4)))


def test_bn_quantize():
    rng = np.random.default_rng(11)
    rows, C = 50, 17
    acc = rng.integers(-300, 300, size=(rows, C)).astype(np.int32)
    resid = rng.integers(-50, 50, size=(rows, C)).astype(np.int32)
    # a = 1 must be the reference's  bit = !(res < bn[c])
    bn = rng.integers(-100, 100, size=(C, 1)).astype(np.int32)
    q = O.bn_quantize(acc, None, bn, None, 1)
    assert np.array_equal(q, (~(acc < bn[:, 0][None, :])).astype(np.int32))
    # multi-bit: equals float BN + uniform quantizer when thresholds are derived from the same BN
    a = 2
    gamma = rng.uniform(0.5, 2.0, C) * rng.choice([-1.0, 1.0], C)
    beta = rng.uniform(-1, 1, C)
    mu = rng.uniform(-20, 20, C)
    sigma = rng.uniform(5, 50, C)
    step = 0.7
    v = (acc.astype(np.int64) + resid)
    y = gamma * (v - mu) / sigma + beta
    expect = np.clip(np.floor(y / step), 0, 2 ** a - 1).astype(np.int32)
    # y/step >= k  <=>  s*v >= s*(mu + (k*step - beta)*sigma/gamma), s = sign(gamma)
    ks = np.arange(1, 2 ** a)
    t_real = (mu[:, None] + (ks[None, :] * step - beta[:, None]) * sigma[:, None] / gamma[:, None])
    s = np.sign(gamma)[:, None]
    thr = np.ceil(s * t_real).astype(np.int32)
    flip = (gamma < 0).astype(np.uint8)
    thr.sort(axis=1)
    q = O.bn_quantize(acc, resid, thr, flip, a)
    assert np.array_equal(q, expect)
    assert q.min() >= 0 and q.max() <= 3
    big = np.full((C, 3), 2 ** 31 - 1, np.int32)
    assert np.all(O.bn_quantize(acc, None, big, None, 2) == 0)
    assert np.all(O.bn_quantize(acc, None, -big - 1, None, 2) == 3)


def test_pack_bits_roundtrip_and_layout():
    rng = np.random.default_rng(13)
    rows, C, cpad, bits = 7, 70, 128, 3
    v = rng.integers(0, 2 ** bits, size=(rows, C)).astype(np.uint32)
    p = O.pack_bits(v, rows, C, cpad, bits)
    assert p.shape == (bits, rows, 4)
    assert np.array_equal(O.unpack_bits(p, rows, C, cpad, bits), v)
    assert np.all(p[:, :, 3] == 0)                    # pad channels zero
    assert np.all((p[:, :, 2] & np.uint32((1 << 26) - 1)) == 0)
    one = np.zeros((1, 33), np.uint32)
    one[0, 0], one[0, 32] = 1, 2
    p = O.pack_bits(one, 1, 33, 128, 2)
    assert p[0, 0, 0] == 0x80000000 and p[1, 0, 1] == 0x80000000 and p[0, 0, 1] == 0


def test_conv_i8_vs_numpy():
    rng = np.random.default_rng(17)
    X = rng.integers(-128, 128, size=(2, 11, 9, 3)).astype(np.int8)
    Wt = rng.integers(-128, 128, size=(6, 7, 7, 3)).astype(np.int8)
    got = O.conv_i8(Wt, X, 2, 3)
    expect = _np_conv(X.astype(np.int64), Wt.astype(np.int64), 2, 3)
    assert np.array_equal(got, expect)


def test_quantize_val_closed_forms_and_numpy_float32():
    """Quantize_val (NN/kernel.cuh:29-44): end points, exact levels, ties, monotonicity, and an independent
    float32 evaluation of the same expression."""
    for bits in (1, 2, 4, 8):
        top = 2 ** bits - 1
        x = np.array([-1e9, -10.0, 10.0, 1e9, 0.0], np.float32)
        q = O.quantize_val(x, bits)
        assert list(q) == [0, 0, top, top, min(top, 2 ** (bits - 1))]     # clip, clamp, mid level
        # x = -10 + 20*k/2^bits is exactly level k; half way between two levels rounds to the even one
        k = np.arange(0, 2 ** bits + 1)
        xs = (-10.0 + 20.0 * k / 2 ** bits).astype(np.float32)
        assert np.array_equal(O.quantize_val(xs, bits), np.minimum(k, top))
        if bits <= 4:
            ties = (-10.0 + 20.0 * (k[:-1] + 0.5) / 2 ** bits).astype(np.float32)   # exactly representable
            expect = np.minimum(np.where(k[:-1] % 2 == 0, k[:-1], k[:-1] + 1), top)
            assert np.array_equal(O.quantize_val(ties, bits), expect)
        rng = np.random.default_rng(40 + bits)
        r = np.sort(rng.uniform(-12, 12, 5000).astype(np.float32))
        qr = O.quantize_val(r, bits)
        assert np.all(np.diff(qr.astype(np.int64)) >= 0)
        f = np.float32
        c = np.clip(r, f(-10), f(10))
        ref = np.rint(((c - f(-10)) * f(2 ** bits) * f(1.0)) / f(20.0))
        assert np.array_equal(qr, np.minimum(ref, top).astype(np.uint32))
    # other ranges
    x = np.linspace(-1, 3, 1001).astype(np.float32)
    q = O.quantize_val(x, 3, 0.0, 2.0)
    assert q[0] == 0 and q[-1] == 7 and np.all(np.diff(q.astype(np.int64)) >= 0)
