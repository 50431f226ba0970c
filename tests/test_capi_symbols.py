"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports every symbol that
include/marmot_hip.h declares, block geometry answers match the reference's block sizes, and entry points
reject bad arguments without touching a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header: str):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(marmot_hip_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from marmot_amd import capi

    return capi.load_library()


def test_library_exports_every_declared_symbol(lib):
    from marmot_amd import capi

    names = declared_functions("marmot_hip.h")
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/marmot_hip.h but not exported"
        assert n in capi.SIGNATURES, f"{n} has no ctypes signature in marmot_amd/capi.py"
    assert sorted(capi.SIGNATURES) == names


def test_block_geometry(lib):
    # include/marmot/quant_block.h:24,52,97,117,126 of the reference
    assert [lib.marmot_hip_block_bytes(k) for k in (1, 5, 9, 11, 12)] == [18, 34, 144, 210, 292]
    assert [lib.marmot_hip_block_values(k) for k in (1, 5, 9, 11, 12)] == [32, 32, 256, 256, 256]
    assert lib.marmot_hip_row_bytes(9, 4096) == 16 * 144
    assert lib.marmot_hip_row_bytes(9, 4097) == 17 * 144
    assert lib.marmot_hip_row_bytes(5, 2048) == 2176
    assert lib.marmot_hip_row_bytes(11, 14336) == 56 * 210
    assert lib.marmot_hip_row_bytes(99, 256) == 0
    # benchmark shapes: 14336 x 4096 Q4_K = 33,030,144 B; Q6_K = 48,168,960 B; Q8_0 5632 x 2048 = 12,255,232 B
    assert 14336 * lib.marmot_hip_row_bytes(9, 4096) == 33030144
    assert 4096 * lib.marmot_hip_row_bytes(9, 14336) == 33030144
    assert 14336 * lib.marmot_hip_row_bytes(11, 4096) == 48168960
    assert 5632 * lib.marmot_hip_row_bytes(5, 2048) == 12255232


def test_null_device_is_rejected_without_gpu(lib):
    assert lib.marmot_hip_matmul_quantized(None, 9, None, None, 0, 1, 256, 1, None, 0, None, 0, 0) == -3
    assert b"not initialised" in lib.marmot_hip_last_error()
    assert lib.marmot_hip_dequantize(None, 9, None, 1, 256, None) == -1
    assert lib.marmot_hip_synchronize(None) == -1
    assert lib.marmot_hip_alloc(None, 16, None) == -1
    assert lib.marmot_hip_version().startswith(b"marmot_hip")


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from marmot_amd import capi

    monkeypatch.setenv("MARMOT_HIP_LIBRARY", str(tmp_path / "nope.so"))
    monkeypatch.setattr(capi, "_lib", None)
    with pytest.raises(FileNotFoundError):
        capi.load_library()
