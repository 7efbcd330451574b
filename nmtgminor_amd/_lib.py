"""ctypes binding of libnmtg_hip.so (the C ABI declared in include/nmtg_hip.h).

The library is loaded on first use. There is no fallback: if the shared object is missing or a
call returns an error status, a RuntimeError is raised. PyTorch is used only for device memory
(`tensor.data_ptr()`) and the current HIP stream.
"""
import ctypes
import os
import re
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnmtg_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "nmtg_hip.h")

F32, F16, BF16 = 0, 1, 2
_DTYPE_CODES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}

ACT_NONE, ACT_RELU, ACT_GELU, ACT_SILU, ACT_AGELU = 0, 1, 2, 3, 4
ACT_CODES = {"none": ACT_NONE, "relu": ACT_RELU, "gelu": ACT_GELU, "silu": ACT_SILU, "agelu": ACT_AGELU}

_lock = threading.Lock()
_lib = None


class NativeLibraryMissing(RuntimeError):
    pass


def header_functions():
    """Names of every function include/nmtg_hip.h declares (used by the export test)."""
    with open(HEADER_PATH) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nmtg_[a-z0-9_]+)\s*\(", text)))


def load():
    """Return the loaded ctypes library, loading it on first call."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise NativeLibraryMissing(
                f"{LIB_PATH} is not built. Build it with `make -C nmtgminor_amd/csrc` "
                "(hipcc, --offload-arch=gfx950); there is no non-HIP path.")
        lib = ctypes.CDLL(LIB_PATH)
        lib.nmtg_last_error.restype = ctypes.c_char_p
        lib.nmtg_version.restype = ctypes.c_int
        for name in header_functions():
            fn = getattr(lib, name)  # AttributeError here = header / library mismatch
            if name.endswith(("_parts", "_bytes", "_blocks")) or name == "nmtg_trace_end":
                fn.restype = ctypes.c_int64
        _lib = lib
    return _lib


def dtype_code(t):
    try:
        return _DTYPE_CODES[t.dtype if isinstance(t, torch.Tensor) else t]
    except KeyError:
        raise RuntimeError(f"unsupported dtype {t.dtype if isinstance(t, torch.Tensor) else t}") from None


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    if t is None:
        return ctypes.c_void_p(0)
    return ctypes.c_void_p(t.data_ptr())


def stream_of(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def i64(v):
    return ctypes.c_int64(int(v))


def f32(v):
    return ctypes.c_float(float(v))


def i32(v):
    return ctypes.c_int(int(v))


def check(rc, what):
    if rc != 0:
        msg = load().nmtg_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what}: {msg} (status {rc})")


def require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("expected a tensor in device memory (HIP); this op has no CPU path")


def call(name, *args):
    """Call entry point `name` with already-wrapped ctypes arguments and raise on error."""
    fn = getattr(load(), name)
    check(fn(*args), name)


def trace_begin():
    check(load().nmtg_trace_begin(), "nmtg_trace_begin")


def trace_end():
    """-> {kernel name: (launches, total milliseconds)} since trace_begin()."""
    buf = ctypes.create_string_buffer(1 << 16)
    load().nmtg_trace_end(buf, ctypes.c_int64(len(buf)))
    out = {}
    for line in buf.value.decode().splitlines():
        name, count, ms = line.split()
        out[name] = (int(count), float(ms))
    return out
