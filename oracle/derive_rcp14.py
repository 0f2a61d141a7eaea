"""Derives the segment table of orc_rcp14 (oracle/fc_oracle.c) from the vrcp14ps instruction.

Needs an AVX-512 host and the compiled shim (make -C oracle ref): the instruction is run through
ref_rcp14 on every mantissa of [1, 2), the structure stated in fc_oracle.c is verified on the way
(output constant over runs of 128 mantissas, 7 low bits zero, powers of two exact), and for each of
the 64 segments the unique integers a, b with significand(d) == (a*256 - b*d) >> 9 for all 1024
offsets d are found.  Prints the table words a << 10 | b in the form they have in fc_oracle.c.

    python oracle/derive_rcp14.py
"""
import ctypes as C
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from oracle import pyoracle as po  # noqa: E402


def main():
    ref = po.ref()
    assert ref is not None, "compiled shim unavailable (make -C oracle ref on an AVX-512 host)"
    x = (np.arange(1 << 23, dtype=np.uint32) | np.uint32(0x3F800000)).view(np.float32)
    y = np.empty_like(x)
    ref.ref_rcp14(C.c_void_p(x.ctypes.data), C.c_void_p(y.ctypes.data), x.size)
    r = y.view(np.uint32).reshape(-1, 128)
    assert r[0, 0] == 0x3F800000, "1.0 must map to 1.0"
    assert (r[:, 1:] == r[:, [1]]).all() and (r[1:, 0] == r[1:, 1]).all(), "output depends on more than 16 mantissa bits"
    t = r[:, 1].astype(np.int64)
    assert (t >> 23 == 126).all() and (t & 0x7F == 0).all()
    sig = (0x800000 | (t & 0x7FFFFF)) >> 7          # 17-bit significands, 65536 of them
    d = np.arange(1024)
    words = []
    for seg in sig.reshape(64, 1024):
        slope = (seg[0] - seg[-1]) / 1023.0
        found = None
        for b in range(int(np.floor(slope * 512)) - 2, int(np.ceil(slope * 512)) + 3):
            lo = (seg * 512 + b * d).max()
            hi = ((seg + 1) * 512 + b * d).min()
            if lo < hi:
                assert found is None and hi - lo == 1 and lo % 256 == 0, "segment model is not unique"
                found = (int(lo) >> 8, b)
        assert found is not None, "segment does not follow (a*256 - b*d) >> 9"
        words.append(found[0] << 10 | found[1])
    print(",\n".join("    " + ", ".join(f"0x{w:08x}u" for w in words[i:i + 8]) for i in range(0, 64, 8)))


if __name__ == "__main__":
    main()
