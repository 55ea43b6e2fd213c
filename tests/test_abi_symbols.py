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
    assert _cabi.chunk_len_for([1000, 5000]) == 512 and _cabi.chunk_len_for([4 << 20] * 8) == 4096 and _cabi.chunk_len_for([1 << 20] * 3) == 1024
    assert lib.sg2_set_scan_window(100) != 0 and lib.sg2_set_scan_window(128) == 0 and lib.sg2_get_scan_window() == 128
    assert lib.sg2_set_scan_window(-1) == 0 and lib.sg2_get_scan_window() == 64


def test_refused_dims_name_the_reference_limit():
    """Dimensions the library refuses are refused with the reference's own limit in the message
    (csrc/supergrok2_mamba_peer_kernels.cu:1796-1801 and what its kernels take for granted); everything inside those
    limits is accepted.  No GPU work: the size query only validates."""
    import ctypes as C
    from grokking_optimizers import _cabi
    import workloads as wl
    numels = (C.c_int64 * 2)(100, 200)

    def query(**kw):
        d = _cabi.make_dims(dict(wl.DEFAULT_DIMS, **kw))
        return _cabi.lib().sg2_workspace_bytes(C.byref(d), 2, numels), _cabi.last_error()
    for kw, text in ((dict(d_state=15), "d_state must be even"), (dict(d_state=34), "MAX_D_STATE"), (dict(d_model=18), "MAX_D_MODEL"),
                     (dict(gru_hidden=9), "MAX_GRU_HIDDEN"), (dict(d_inner=36), "MAX_D_INNER"), (dict(d_inner=14), "multiple of 4"),
                     (dict(d_model=7), "d_model must be even"), (dict(num_experts=200), "pk_dim^2"), (dict(num_heads=0), "positive")):
        n, msg = query(**kw)
        assert n == 0 and text in msg, (kw, msg)
    for kw in (dict(), dict(expert_hidden=4), dict(d_model=4, d_state=8, d_inner=8), dict(d_model=16, d_state=32, d_inner=32),
               dict(d_model=12, d_state=24, d_inner=24, gru_hidden=8, num_heads=3, pk_dim=6, expert_hidden=5, num_experts=36),
               dict(num_heads=2, pk_dim=70, expert_hidden=2, num_experts=4900)):
        n, msg = query(**kw)
        assert n > 0, (kw, msg)
