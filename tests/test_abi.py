"""The C-ABI library loads and exports every symbol include/msq.h declares; host-only entry points (geometry, launch
shape, argument validation) behave as documented. No kernel is launched here."""
import ctypes as C
import os
import re

import pytest

from macseek_amd import _lib
from macseek_amd import quant as q

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "msq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(msq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 10
    L = C.CDLL(_lib.SO)
    for n in names:
        assert hasattr(L, n), "libmsq.so does not export " + n
    assert sorted(_lib.SIGNATURES) == names, "python binding and header disagree"


def test_geometry_matches_gguf_block_sizes():
    expect = {q.QType.F32: (1, 4), q.QType.F16: (1, 2), q.QType.BF16: (1, 2), q.QType.Q8_0: (32, 34),
              q.QType.Q5_K: (256, 176), q.QType.Q6_K: (256, 210), q.QType.IQ2_XXS: (256, 66), q.QType.IQ1_S: (256, 50),
              q.QType.IQ4_NL: (32, 18)}
    for t, (be, bb) in expect.items():
        assert q.block_elems(t) == be and q.block_bytes(t) == bb and q.type_name(t) == t.name
    assert q.row_bytes(q.QType.IQ1_S, 7168) == 1400 and q.row_bytes(q.QType.Q6_K, 7168) == 5880
    assert q.block_elems(39) == 0 and q.type_name(39) == "?"  # MXFP4 is not on this path


def test_matvec_supported_and_cfg():
    for t in q.QType:
        assert q.matvec_supported(t)
    assert not q.matvec_supported(39)
    c = q.matvec_cfg(q.QType.IQ1_S, 4096, 7168)
    assert c.ks == 4 and c.nr >= 1 and c.rsg >= 1  # 224 32-column units -> 4 waves across K
    c2 = q.matvec_cfg(q.QType.IQ1_S, 64, 7168)
    assert c2.ks == c.ks  # the K split (summation order) depends on cols only, never on rows
    with pytest.raises(q.QuantError) as ei:
        q.matvec_cfg(q.QType.Q6_K, 16, 100)
    assert "matvec_cfg unsupported (type Q6_K rows 16 cols 100)" in str(ei.value)


def test_matvec_rejects_misuse_without_touching_the_gpu():
    L = _lib.load()
    B = _lib.MsqBuffer
    big = B(0x1000, 0, 1 << 30)
    null = B(0, 0, 0)

    def mv(t, rows, cols, W=big, x=big, y=big, groups=1):
        return L.msq_matvec(None, t, C.byref(W), rows, cols, C.byref(x), C.byref(y), 0, groups, None)

    assert mv(39, 16, 256) == -1 and b"matvec unsupported (type ? rows 16 cols 256)" in L.msq_last_error()
    assert mv(q.QType.IQ1_S, 16, 300) == -1      # cols % 256
    assert mv(q.QType.Q8_0, 16, 48) == -1        # cols % 32
    assert mv(q.QType.BF16, 16, 128) == -1       # dense types use a virtual 256 block
    assert mv(q.QType.Q6_K, 10, 256, groups=3) == -1   # rows % groups
    assert mv(q.QType.Q6_K, 10, 256, groups=0) == -1
    assert mv(q.QType.Q6_K, 16, 256, W=null) == -2
    assert mv(q.QType.Q6_K, 16, 256, y=B(0x1000, 0, 8)) == -2  # y too small
    assert L.msq_dequant(None, q.QType.IQ1_S, C.byref(big), 100, C.byref(big)) == -1  # not a block multiple
    assert L.msq_dequant(None, q.QType.IQ1_S, C.byref(big), 0, C.byref(big)) == 0     # empty input: nothing to do
