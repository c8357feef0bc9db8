"""CPU-side checks of the C ABI: the in-tree library loads without a GPU, exports every function that
include/mllm_hip_qlinear.h declares, and its size helpers (host-only code) agree with the documented layouts."""
import ctypes as C
import os
import re

import pytest

from mllm_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_is_built_in_tree():
    assert os.path.exists(_lib.LIB_PATH), "run `python -m mllm_amd.build` (or __graft_entry__.build())"


def test_every_declared_symbol_is_exported():
    L = C.CDLL(_lib.LIB_PATH)
    names = _lib.exported_symbols()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing


def test_header_is_plain_c():
    txt = open(os.path.join(ROOT, "include", "mllm_hip_qlinear.h")).read()
    assert 'extern "C"' in txt and "torch" not in txt.lower().replace("no c++ or torch types", "")
    for line in txt.splitlines():
        assert "std::" not in line and "at::" not in line


def test_size_helpers_without_gpu():
    L = _lib.lib()
    # Q4_0: 16 bytes of codes per block + fp16 scales in rows padded to 8 entries; both regions 256-byte aligned
    N, K = 6144, 2048
    nb = K // 32
    want = -(-N * nb * 16 // 256) * 256 + -(-N * (-(-nb // 8) * 8) * 2 // 256) * 256
    assert L.mllm_hip_q_packed_bytes(0, N, K) == want
    assert L.mllm_hip_q_packed_bytes(1, N, K) == want + -(-N * nb * 16 // 256) * 256
    assert L.mllm_hip_q_packed_bytes(0, N, K + 1) == 0 and L.mllm_hip_q_packed_bytes(2, N, K) == 0
    assert L.mllm_hip_w8a8_workspace_bytes(2048, 2048) >= 2048 * 2048 + 2048 * 4
    assert L.mllm_hip_moe_workspace_bytes(512, 2048, 768, 128, 8) >= 512 * 8 * 2048 * 4
    assert L.mllm_hip_linear_q_workspace_bytes(100, 64) > 100 * 64


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmllm_hip_qlinear.so")
    with pytest.raises(_lib.HipQLinearError):
        _lib.lib()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "mllm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", ".hpp")):
                txt = open(os.path.join(dirpath, f), errors="ignore").read()
                assert not re.search(r"^\s*(from|import)\s+oracle", txt, re.M), f
                assert "liboracle" not in txt and "qlinear_oracle" not in txt, f
