"""CPU-side checks of the C ABI: the library loads and exports every symbol the header declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dl4s_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dl4s_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    syms = _declared_symbols()
    for must in ["dl4s_hip_create", "dl4s_hip_sdpa_fwd_f32", "dl4s_hip_sdpa_decode_f32", "dl4s_hip_kv_append_f32",
                 "dl4s_hip_gemm_f32", "dl4s_hip_broadcast_f32", "dl4s_hip_permute_axes_f32", "dl4s_hip_layernorm_f32"]:
        assert must in syms
    assert len(syms) >= 35


def test_library_exports_every_declared_symbol():
    from dl4s_amd import lib
    so = ctypes.CDLL(lib.LIB_PATH)
    missing = [s for s in _declared_symbols() if not hasattr(so, s)]
    assert not missing, missing


def test_last_error_is_a_string_without_a_gpu():
    from dl4s_amd import lib
    l = lib.load()
    assert isinstance(l.dl4s_hip_last_error(), bytes)


def test_null_context_is_rejected_not_crashed():
    from dl4s_amd import lib
    l = lib.load()
    rc = l.dl4s_hip_sync(None)
    assert rc == -1 and b"ctx is NULL" in l.dl4s_hip_last_error()
    rc = l.dl4s_hip_create(0, None)
    assert rc == -1


def test_host_library_exports_every_symbol_its_header_declares():
    from dl4s_amd import host_lib, lib
    text = open(os.path.join(ROOT, "include", "dl4s_host.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(dl4s_host_[a-z0-9_]+)\s*\(", text)))
    assert "dl4s_host_transformer_greedy" in declared and "dl4s_host_mha" in declared
    ctypes.CDLL(lib.LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    so = ctypes.CDLL(host_lib.HOST_LIB_PATH)
    missing = [s for s in declared if not hasattr(so, s)]
    assert not missing, missing
    # a NULL context is an error return, never a crash
    assert so.dl4s_host_positional_encoding(None, 1, ctypes.c_int64(4), ctypes.c_int64(4), None) == -1
