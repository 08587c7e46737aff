"""The C-ABI libraries load and export every entry point that include/*.h declares (no GPU needed: nothing is launched)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header):
    txt = open(os.path.join(ROOT, "include", header)).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b((?:kc|kq4|nh)_\w+)\s*\(", txt)))


@pytest.fixture(scope="module")
def libs():
    from nanoseedlm_amd import backend
    if not os.path.exists(backend.HIP_SO) or not os.path.exists(backend.KT_SO) or not os.path.exists(backend.HOST_SO):
        backend.build()
    return backend


def test_exports_every_declared_symbol(libs):
    L = libs.hip()
    names = declared("kernels_hip.h") + declared("nslm_rt.h")
    assert len(names) > 40
    for n in names:
        assert hasattr(L, n), f"libnslm_hip.so does not export {n}"


def test_struct_layouts_match_the_reference_abi(libs):
    # engine/kernels_cuda.h:19-24 WSlice is 48 bytes; MmTile 16; RouterArgs 20; CachePool's fields at the reference's offsets
    assert C.sizeof(libs.WSlice) == 48 and C.sizeof(libs.MmTile) == 16 and C.sizeof(libs.RouterArgs) == 20
    assert libs.CachePool.unit_bytes.offset == 72 and libs.CachePool.tab.offset == 96 and libs.CachePool.off.offset == 104
    assert C.sizeof(libs.CachePool) == 168
    assert libs.Qwen4Cfg.n_exp.offset == 84 and libs.Qwen4Cfg.top_k.offset == 88


def test_kt_backend_exports(libs):
    K = libs.kt()
    txt = open(os.path.join(ROOT, "tests", "kt", "kernel_backend.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    for n in set(re.findall(r"\b(kt_\w+)\s*\(", txt)):
        assert hasattr(K, n), n
    assert K.kt_name() == b"HIP gfx950" and K.kt_mm_tile() == 128
    assert not hasattr(K, "nslm_moe_open")                             # the test binding holds no product code ...
    K = libs.host()
    assert not hasattr(K, "kt_mv")                                     # ... and the host library no test binding
    for h in ("moe_layer.h", "decode_model.h"):                        # the layer and whole-model hosts
        txt = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "nanoseedlm_amd", "csrc", h)).read(), flags=re.S)
        names = set(re.findall(r"\b(nslm_\w+)\s*\(", txt))
        assert len(names) > 8
        for n in names:
            assert hasattr(K, n), n
    txt = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "model_folder.h")).read(), flags=re.S)
    names = set(re.findall(r"\b((?:nsf|nslm_moe)_\w+)\s*\(", txt))                # the model-folder reader and its loaders
    assert len(names) >= 11
    for n in names:
        assert hasattr(K, n), n


def test_missing_library_fails_loudly(libs, monkeypatch):
    monkeypatch.setattr(libs, "_hip", None)
    monkeypatch.setattr(libs, "HIP_SO", "/nonexistent/libnslm_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        libs.hip()
