"""ctypes binding of ``libmegalodon_hip.so`` (the C ABI in include/megalodon_hip.h).

There is no CPU fallback: if the shared library is missing or an entry point
returns an error, a ``RuntimeError`` is raised (the reference raises
``RuntimeError`` through TORCH_CHECK the same way).
"""
from __future__ import annotations

import ctypes
import re
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
LIB_PATH = PKG_DIR / "lib" / "libmegalodon_hip.so"
HEADER_PATH = PKG_DIR.parent / "include" / "megalodon_hip.h"

MEGA_F32, MEGA_BF16, MEGA_F16, MEGA_F64 = 0, 1, 2, 3

_lib = None

_c_i64 = ctypes.c_int64
_c_ptr = ctypes.c_void_p


def declared_symbols() -> list[str]:
    """Names of every function the public header declares."""
    text = HEADER_PATH.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mega_[a-z0-9_]+)\s*\(", text)))


def load() -> ctypes.CDLL:
    """Load the library once; raise loudly when it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} not found: build it with `python -m megalodon_amd._build` "
                "(there is no CPU fallback for the HIP ops)")
        lib = ctypes.CDLL(str(LIB_PATH))
        lib.mega_last_error.restype = ctypes.c_char_p
        lib.mega_version.restype = ctypes.c_int
        _lib = lib
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().mega_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (code {code}): {msg}")


def ptr(t) -> ctypes.c_void_p:
    """Device pointer of a torch tensor (None -> NULL)."""
    return _c_ptr(0 if t is None else t.data_ptr())


def i64(v: int) -> ctypes.c_int64:
    return _c_i64(int(v))


def u64(v: int) -> ctypes.c_uint64:
    return ctypes.c_uint64(int(v))


def f64(v: float) -> ctypes.c_double:
    return ctypes.c_double(float(v))


def i32(v: int) -> ctypes.c_int:
    return ctypes.c_int(int(v))


def dtype_code(dtype, wide_ok: bool = False) -> int:
    """Element type code of the C interface.  float64 is taken by the operators that have a
    double-precision flavour (`wide_ok`); everywhere else it is refused, not narrowed."""
    import torch
    if wide_ok and dtype == torch.float64:
        return MEGA_F64
    try:
        return {torch.float32: MEGA_F32, torch.bfloat16: MEGA_BF16, torch.float16: MEGA_F16}[dtype]
    except KeyError:
        raise RuntimeError(f"unsupported dtype {dtype} (float32, bfloat16, float16 are supported)")


def stream_ptr(device=None) -> ctypes.c_void_p:
    import torch
    return _c_ptr(torch.cuda.current_stream(device).cuda_stream)


# Optional per-entry-point device timing: when a dict is installed with
# ``set_event_log``, every call of an entry point named in it is bracketed by
# events recorded on the current stream (the stream the kernels are enqueued
# on); the (start, end) pairs are appended to the list under that name.
_event_log = None


def set_event_log(log) -> None:
    global _event_log
    _event_log = log


def call(name: str, *args) -> None:
    fn = getattr(load(), name)
    fn.restype = ctypes.c_int
    log = _event_log
    if log is not None and name in log:
        import torch
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        code = fn(*args)
        e1.record()
        log[name].append((e0, e1))
        check(code, name)
        return
    check(fn(*args), name)
