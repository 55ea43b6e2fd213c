"""The C-ABI library loads and exports every symbol include/sg_abi.h declares
(no device work: runs without a GPU)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    names = set()
    for fn in os.listdir(os.path.join(ROOT, "include")):
        if fn.endswith("_abi.h"):
            src = open(os.path.join(ROOT, "include", fn)).read()
            src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
            names |= set(re.findall(r"\b(sg\w*)\s*\(", src))
    return names


def test_library_exports_every_declared_symbol():
    from grokking_optimizers import _cabi
    assert os.path.exists(_cabi.LIB_PATH), "libsg_hip.so not built: run __graft_entry__.build()"
    lib = ctypes.CDLL(_cabi.LIB_PATH)
    declared = _declared()
    assert {"sg2_batched_step", "sg2_workspace_bytes", "sg_last_error"} <= declared
    for name in sorted(declared):
        assert hasattr(lib, name), name


def test_host_side_validation_without_gpu():
    from grokking_optimizers import _cabi
    assert _cabi.workspace_bytes([0, 0]) >= 0
    n = _cabi.workspace_bytes([1000, 5000])
    assert n > 8 * 6000 * 4
    lib = _cabi.lib()
    assert lib.sg2_set_chunk_len(100) != 0 and b"multiple of 64" in lib.sg_last_error()
    assert lib.sg2_set_chunk_len(256) == 0 and lib.sg2_get_chunk_len() == 256
    assert lib.sg2_set_chunk_len(0) == 0 and lib.sg2_get_chunk_len() == 0
    assert _cabi.chunk_len_for([1000, 5000]) == 1024 and _cabi.chunk_len_for([4 << 20] * 8) == 4096
    assert lib.sg2_set_scan_window(100) != 0 and lib.sg2_set_scan_window(128) == 0 and lib.sg2_get_scan_window() == 128
    assert lib.sg2_set_scan_window(-1) == 0 and lib.sg2_get_scan_window() == 64
