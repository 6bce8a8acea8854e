"""The C-ABI library loads and exports every symbol the public header declares
(no compute calls: runs without a GPU)."""
import ctypes

from megalodon_amd import _lib


def test_library_loads_and_reports_version():
    lib = _lib.load()
    assert lib.mega_version() >= 100
    assert lib.mega_last_error() == b"" or isinstance(lib.mega_last_error(), bytes)


def test_every_declared_symbol_is_exported():
    lib = _lib.load()
    names = _lib.declared_symbols()
    assert "mega_ema_weight_fwd" in names and "mega_version" in names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/megalodon_hip.h but not exported: {missing}"


def test_invalid_argument_is_reported_not_raised_in_c():
    lib = _lib.load()
    fn = lib.mega_ema_weight_fwd
    fn.restype = ctypes.c_int
    null = ctypes.c_void_p(0)
    code = fn(null, null, null, ctypes.c_int64(1), ctypes.c_int64(16), ctypes.c_int64(8), null, null)
    assert code == 1
    assert b"null" in lib.mega_last_error()


def test_attention_rejects_an_unknown_causal_code():
    """`causal` is 0 (no mask), 1 (mask, whole rows of w written) or 2 (mask, w only as far as
    the backward reads it); anything else is an argument error before any launch."""
    lib = _lib.load()
    fn = lib.mega_attention_fwd
    fn.restype = ctypes.c_int
    null = ctypes.c_void_p(0)
    i64 = ctypes.c_int64
    code = fn(null, null, null, ctypes.c_int(1), i64(1), i64(8), i64(8), i64(1), i64(64), i64(64),
              ctypes.c_double(1.0), ctypes.c_int(3), null, null, null, null)
    assert code == 1
    assert b"causal" in lib.mega_last_error()
