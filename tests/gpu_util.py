"""Device-side plumbing for the GPU parity tests: torch only allocates device memory and supplies
streams; every compute call goes through the C ABI of libapnn_tc.so."""
import ctypes

import numpy as np
import torch

import pkg

A = pkg.load()


def to_dev(arr):
    arr = np.ascontiguousarray(arr)
    if arr.dtype == np.uint32:
        arr = arr.view(np.int32)
    return torch.from_numpy(arr).cuda()


def dev_empty_i32(n, fill=None):
    return guarded_empty(n, torch.int32, fill)


GUARD_BYTES = 256         # either side of every output: keeps the 16-byte alignment the entry points ask for
GUARD_BYTE = 0x5A
_live_guards = []         # (whole buffer, payload bytes, what) of the outputs the running test allocated


def guarded_empty(n, dtype=torch.int32, fill=None, what="output"):
    """A device tensor of n elements with guard bytes before and after it.  check_guards() (run by
    to_host() and after every GPU test) asserts that no guard byte changed, so a store next to an
    output buffer fails the test that made it."""
    nbytes = int(n) * torch.empty(0, dtype=dtype).element_size()
    whole = torch.empty(nbytes + 2 * GUARD_BYTES, dtype=torch.uint8, device="cuda")
    whole.fill_(GUARD_BYTE)
    view = whole[GUARD_BYTES:GUARD_BYTES + nbytes].view(dtype)
    if fill is not None:
        view.fill_(fill)
    _live_guards.append((whole, nbytes, what))
    return view


def check_guards(clear=False):
    if not _live_guards:
        return
    torch.cuda.synchronize()
    for whole, nbytes, what in _live_guards:
        lo = whole[:GUARD_BYTES].cpu().numpy()
        hi = whole[GUARD_BYTES + nbytes:].cpu().numpy()
        assert (lo == GUARD_BYTE).all(), "store below the %s buffer (%d bytes): guard byte -%d changed" % (
            what, nbytes, GUARD_BYTES - int(np.flatnonzero(lo != GUARD_BYTE)[-1]))
        assert (hi == GUARD_BYTE).all(), "store past the %s buffer (%d bytes): guard byte +%d changed" % (
            what, nbytes, int(np.flatnonzero(hi != GUARD_BYTE)[0]))
    if clear:
        _live_guards.clear()


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def to_host(t, dtype=np.int32):
    check_guards()
    a = t.cpu().numpy()
    return a.view(dtype) if dtype != a.dtype else a


def epilogue(mode=0, out_bits=0, pool=0, thr=None, flip=None, resid=None, save=None, resid_planes=None,
             resid_bits=0, resid_scale=0):
    e = A.Epilogue()
    e.mode, e.out_bits, e.pool = mode, out_bits, pool
    e.thresholds = thr.data_ptr() if thr is not None else None
    e.flip = flip.data_ptr() if flip is not None else None
    e.residual = resid.data_ptr() if resid is not None else None
    e.save_acc = save.data_ptr() if save is not None else None
    e.residual_planes = resid_planes.data_ptr() if resid_planes is not None else None
    e.residual_bits, e.residual_scale = resid_bits, resid_scale
    return e


def run_gemm(W, X, M, N, K, wb, xb, *, sym=0, epi=None, path=0, tile=None, out_words=None):
    """W, X: numpy uint32 planes.  Returns the raw int32 output buffer as numpy."""
    dW, dX = to_dev(W), to_dev(X)
    epi = epi or epilogue()
    if out_words is None:
        out_words = M * N if epi.mode == 0 else epi.out_bits * M * (N // 32)
    out = dev_empty_i32(out_words, fill=-7)
    d = A.GemmDesc(W=dW.data_ptr(), X=dX.data_ptr(), D=out.data_ptr(), M=M, N=N, K=K, wb=wb, xb=xb,
                   weight_mode=sym, epi=epi, path=path if tile is None else (path | ((tile + 1) << 8)))
    rc = A.lib().apnn_gemm(ctypes.byref(d), None)
    A.check(rc, "apnn_gemm")
    return to_host(out)


def run_conv(Wt, X, *, batch, H, W, cin_pad, cout, R, S, stride, pad, halo, wb, xb, sym=0, epi=None,
             path=0, tile=None):
    dW, dX = to_dev(Wt), to_dev(X)
    epi = epi or epilogue()
    Ho, Wo = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - S) // stride + 1
    rows = batch * Ho * Wo
    if epi.mode == 0:
        out_words = rows * cout
    else:
        out_words = epi.out_bits * (rows // 4 if epi.pool else rows) * (cout // 32)
    out = dev_empty_i32(out_words, fill=-7)
    d = A.ConvDesc(W=dW.data_ptr(), X=dX.data_ptr(), O=out.data_ptr(), batch=batch, H=H, Wd=W,
                   cin_pad=cin_pad, COUT=cout, R=R, S=S, stride=stride, pad=pad, halo=halo, wb=wb, xb=xb,
                   weight_mode=sym, epi=epi, path=path if tile is None else (path | ((tile + 1) << 8)))
    rc = A.lib().apnn_conv(ctypes.byref(d), None)
    A.check(rc, "apnn_conv")
    return to_host(out)
