"""The C-ABI library loads without a GPU and exports every symbol the public header declares.
Only host-side helpers are called here; nothing touches a device."""
import ctypes
import os
import re

import pytest

import cntk_amd
import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    inc = os.path.join(ROOT, "include")
    for f in sorted(os.listdir(inc)):
        if f.endswith(".h"):
            text = open(os.path.join(inc, f)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            names |= set(re.findall(r"\b(cntkq_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    L = cntk_amd.lib()
    names = declared_symbols()
    assert len(names) >= 17
    for n in names:
        assert getattr(L, n) is not None, n


def test_layout_helpers_match_oracle():
    L = cntk_amd.lib()
    for nbits in (1, 2, 4, 8, 16, 32):
        for rows in (0, 1, 5, 31, 32, 33, 147, 429, 512, 2048, 4608, 9304, 100000):
            assert L.cntkq_qwords_per_col(rows, nbits) == oracle.qwords_per_col(rows, nbits)
            assert L.cntkq_qcol_bytes(nbits, rows) == oracle.qcol_bytes(nbits, rows)
            assert L.cntkq_qmatrix_bytes(rows, 7, nbits) == 7 * oracle.qcol_bytes(nbits, rows)
    # headline shape: 264-byte columns, 2,456,256 bytes in all
    assert L.cntkq_qcol_bytes(1, 2048) == 264 and L.cntkq_qmatrix_bytes(2048, 9304, 1) == 2456256
    for bad in (0, 3, 5, 64):
        assert L.cntkq_qcol_bytes(bad, 10) == 0 and L.cntkq_qwords_per_col(10, bad) == 0


def test_stripe_range_matches_oracle():
    for cols, k in [(9304, 8), (10, 4), (3, 8), (0, 2), (135, 7), (2048, 3)]:
        for r in range(k):
            assert cntk_amd.stripe_range(cols, r, k) == oracle.stripe_range(cols, r, k)
    with pytest.raises(cntk_amd.QuantizerLogicError):
        cntk_amd.stripe_range(10, 4, 4)


def test_bad_arguments_are_reported_not_crashed():
    L = cntk_amd.lib()
    h = ctypes.c_void_p()
    # a negative device is the reference's CPU quantizer; this library has none and says so
    assert L.cntkq_create(-1, 0, ctypes.byref(h)) == 3
    assert b"CPU" in L.cntkq_last_error()
    assert L.cntkq_wait_quantize_done(None) == 1
    assert L.cntkq_quantize_async(None, None, None, 1, 1, None, 0, 0, 1, None, 0) == 1
    with pytest.raises(cntk_amd.QuantizerLogicError):
        cntk_amd.QuantizedMatrix(8, 8, 3, cntk_amd.CPUDEVICE)


def test_public_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 (no C++ types or keywords), warnings included."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc on this machine")
    src = tmp_path / "use_header.c"
    src.write_text('#include "cntk_amd_quantizer.h"\n'
                   "int main(void) { cntkq_quantize_item a; cntkq_stripe_reduce_item_f64 b; (void) a; (void) b;\n"
                   "    return cntkq_qcol_bytes(1, 2048) == 264 ? 0 : 1; }\n")
    res = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src),
                          "-o", str(tmp_path / "use_header.o")], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
