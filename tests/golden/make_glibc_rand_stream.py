"""Writes glibc_rand_srand1.bin: the first 12288 values of glibc rand() after srand(1), as
little-endian uint32.

The reference's benchmark mains fill their operands with rand() in a fixed order
(APNN-TC-lib/bmmaTensorCoreGemm/src/71_bmmaTensorCoreGemm.cu:305-327 for GEMM: W planes then X
planes; .../67_bmmaTensorCoreGemm.cuh:327-353 for conv: X planes incl. halo, then W planes).
glibc's generator must not be assumed on the machine that runs the tests, so the stream is stored
as data.  known_answers.json holds the checksums that the reference's own compute_ref /
compute_ref_pack produce on these inputs.

Run:  python tests/golden/make_glibc_rand_stream.py     (needs glibc)
"""
import ctypes
import os
import struct

N_WORDS = 12288

def main():
    libc = ctypes.CDLL("libc.so.6")
    libc.srand(1)
    libc.rand.restype = ctypes.c_int
    words = [libc.rand() & 0xFFFFFFFF for _ in range(N_WORDS)]
    assert words[0] == 0x6B8B4567, hex(words[0])
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "glibc_rand_srand1.bin")
    with open(out, "wb") as f:
        f.write(struct.pack("<%dI" % N_WORDS, *words))
    print("wrote", out, len(words), "words")

if __name__ == "__main__":
    main()
