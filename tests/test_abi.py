"""The C-ABI library loads and exports every symbol the header declares (no GPU needed)."""
import re
from pathlib import Path

from loken_amd import lib

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    """Every function of the C ABI header, and the `extern "C"` part of the C++ host header."""
    text = (ROOT / "include" / "loken_gfx950.h").read_text()
    host = (ROOT / "include" / "loken_host.hpp").read_text()
    text += host[host.index('extern "C" {'):]
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(?:int|size_t|void\s*\*?)\s*(\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    l = lib.load()
    names = declared_symbols()
    assert "lk_mmvq" in names and "lk_quantize_q8_1" in names
    missing = [n for n in names if not hasattr(l, n)]
    assert not missing, missing


def test_python_signature_table_covers_the_header():
    assert sorted(lib.SIGNATURES) == declared_symbols()


def test_argument_errors_are_status_codes_not_aborts():
    l = lib.load()
    # unknown weight type and bad sizes are rejected before anything touches a device
    assert l.lk_mmvq(99, 16, 16, 16, 0, 256, 4, 1, 8, 4, None, 0, None) == lib.LK_ERR_TYPE
    assert l.lk_mmvq(lib.TYPE_Q4_K, 16, 16, 16, 0, 250, 4, 1, 8, 4, None, 0, None) == lib.LK_ERR_ARG
    assert l.lk_mmvq(lib.TYPE_Q4_K, 16, 16, 16, 0, 256, 4, 9, 8, 4, None, 0, None) == lib.LK_ERR_ARG
    assert l.lk_mmvq(lib.TYPE_Q4_K, None, 16, 16, 0, 256, 4, 1, 8, 4, None, 0, None) == lib.LK_ERR_ARG
    assert l.lk_quantize_q8_1(16, 0, 16, 100, 96, 1, None) == lib.LK_ERR_ARG
    assert l.lk_quantize_q8_1(16, 7, 16, 64, 64, 1, None) == lib.LK_ERR_TYPE
    assert l.lk_quantize_q8_1(16, 0, 16, 64, 64, 0, None) == lib.LK_OK  # no rows: nothing to do
