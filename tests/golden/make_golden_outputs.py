"""Writes golden_outputs.npz: full int32 outputs (and packed low-bit planes for conv) of the
known-answer cases in known_answers.json, computed by the CPU oracle on the glibc rand() stream.
They are only written after the oracle's result matched every recorded reference checksum
(first/last elements, sum, first packed word), so GPU tests can compare against complete arrays.

Run:  python tests/golden/make_golden_outputs.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as O  # noqa: E402


def main():
    ka = O.known_answers()
    s = O.golden_stream()
    out = {}
    g = ka["gemm"]
    M, N, K = g["shape"]["M"], g["shape"]["N"], g["shape"]["K"]
    for name, c in g["cases"].items():
        nw, nx = c["wb"] * M * K // 32, c["xb"] * N * K // 32
        W, X = s[:nw].reshape(c["wb"], M, K // 32), s[nw:nw + nx].reshape(c["xb"], N, K // 32)
        D = O.gemm_literal(W, X, M, N, K, c["wb"], c["xb"])
        f = D.ravel()
        assert (int(f[0]), int(f[1]), int(f[-1]), int(f.astype(np.int64).sum())) == (c["c0"], c["c1"], c["clast"], c["sum"])
        out["gemm_" + name] = D
    cv = ka["conv"]
    H, Wd, CIN, COUT = (cv["shape"][k] for k in ("H", "W", "CIN", "COUT"))
    for name, c in cv["cases"].items():
        nx, nw = c["xb"] * (H + 2) * (Wd + 2) * CIN // 32, c["wb"] * COUT * 9 * CIN // 32
        X, Wt = s[:nx], s[nx:nx + nw]
        D = O.conv3x3_literal(Wt, X, H, Wd, CIN, COUT, c["wb"], c["xb"])
        f = D.ravel()
        assert (int(f[0]), int(f[1]), int(f.astype(np.int64).sum())) == (c["c0"], c["c1"], c["sum"])
        P = O.lowbits_pack(D, H * Wd, COUT, c["xb"])
        assert "%08x" % int(P.ravel()[0]) == c["pack0"]
        out["conv_" + name] = D
        out["conv_pack_" + name] = P
    path = os.path.join(HERE, "golden_outputs.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
