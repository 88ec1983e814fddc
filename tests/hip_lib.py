"""ctypes view of libwarpctct_hip.so for the tests: loads the in-tree library
and parses include/warp_ctct_hip.h for the list of declared entry points."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# (WARPCTCT_HIP_LIB: another build of the same library, e.g. one whose host code
# is compiled with sanitizers: tests/run_host_sanitizers.sh)
LIB_PATH = os.environ.get("WARPCTCT_HIP_LIB") or os.path.join(
    ROOT, "warp-ctct_amd", "warp_ctct", "libwarpctct_hip.so")
HEADER = os.path.join(ROOT, "include", "warp_ctct_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(warpctct_\w+)\s*\(", text)))


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libwarpctct_hip.so is not built: run `make -C warp-ctct_amd`")
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.warpctct_error_string.restype = ctypes.c_char_p
        _lib.warpctct_version.restype = ctypes.c_char_p
        _lib.warpctct_workspace_bytes.restype = ctypes.c_size_t
    return _lib


def ptr(t):
    """Device (or host) address of a torch tensor / None as c_void_p."""
    if t is None:
        return ctypes.c_void_p(0)
    return ctypes.c_void_p(t.data_ptr())


def stream_ptr():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def check(rc):
    if rc != 0:
        raise RuntimeError(lib().warpctct_error_string(rc).decode())
