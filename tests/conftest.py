import json
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = Path(__file__).resolve().parent / "golden"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture
def knobs(monkeypatch):
    """Sets or clears the library's environment overrides (LK_MMQ_I8, LK_TUNE_*) for one test: the
    library keeps what it read, so every change is followed by lk_tune_refresh, and so is the
    restoring of the environment when the test ends."""
    from loken_amd import lib

    class Knobs:
        def set(self, name, value="1"):
            monkeypatch.setenv(name, value)
            lib.load().lk_tune_refresh()

        def clear(self, name):
            monkeypatch.delenv(name, raising=False)
            lib.load().lk_tune_refresh()

    yield Knobs()
    monkeypatch.undo()
    lib.load().lk_tune_refresh()


def _bits_to_f32(hex_words: str) -> np.ndarray:
    """8-hex-digit IEEE bit patterns, most significant digit first."""
    n = len(hex_words) // 8
    return np.array([int(hex_words[8 * i:8 * i + 8], 16) for i in range(n)], dtype=np.uint32).view(np.float32)


@pytest.fixture(scope="session")
def ggml_vectors():
    """ggml's own quantize/dequantize records: {"input": f32[1024], "q4_K": {"quant": u8[], "dequant": f32[1024], ...}}."""
    rec = {}
    cur = None
    for line in (GOLDEN / "ggml_vectors.txt").read_text().splitlines():
        parts = line.split()
        if parts[0] == "N":
            rec["n"] = int(parts[1])
        elif parts[0] == "INPUT":
            rec["input"] = _bits_to_f32(parts[2])
        elif parts[0] == "TYPE":
            cur = parts[1]
            rec[cur] = {"block_elems": int(parts[2]), "block_bytes": int(parts[3])}
        elif parts[0] == "QUANT":
            rec[cur]["quant"] = np.frombuffer(bytes.fromhex(parts[2]), dtype=np.uint8).copy()
            assert rec[cur]["quant"].size == int(parts[1])
        elif parts[0] == "DEQUANT":
            rec[cur]["dequant"] = _bits_to_f32(parts[2])
            assert rec[cur]["dequant"].size == int(parts[1])
    return rec


@pytest.fixture(scope="session")
def ggml_encode():
    """ggml-written blocks of an 8x512 matrix and the first 2 rows as ggml decodes them."""
    j = json.loads((GOLDEN / "ggml_encode_subset.json").read_text())
    out = {"rows": j["rows"], "cols": j["cols"], "read": j["read"],
           "x": np.frombuffer(bytes.fromhex(j["x"]), dtype="<f4").copy(), "formats": {}}
    for name, f in j["formats"].items():
        out["formats"][name] = {
            "blocks": np.frombuffer(bytes.fromhex(f["blocks"]), dtype=np.uint8).copy(),
            "expected": np.frombuffer(bytes.fromhex(f["expected"]), dtype="<f4").copy(),
        }
    return out
