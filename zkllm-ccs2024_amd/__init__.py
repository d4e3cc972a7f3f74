"""MI355X (gfx950) zkLLM prover core.

The product is two native libraries built in-tree:
  libzkllm_hip.so     hand-written HIP kernels behind the C ABI of include/zkllm_hip.h
  libzkllm_prover.so  the reference's C++ class API (FrTensor, zkFC, tLookup, Commitment, ...)
                      on top of that ABI, plus C entry points for ctypes callers
This module only locates and loads them.  There is no CPU fallback: loading fails loudly when a
library has not been built, and every entry point fails when no GPU is present.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
HIP_LIB = os.path.join(_HERE, "libzkllm_hip.so")
PROVER_LIB = os.path.join(_HERE, "libzkllm_prover.so")

_libs = {}


def _load(path):
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with __graft_entry__.build() "
                           "(make -C zkllm-ccs2024_amd/csrc && make -C zkllm-ccs2024_amd/host)")
    if path not in _libs:
        _libs[path] = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    return _libs[path]


def load_hip():
    """ctypes handle of the C-ABI kernel library."""
    lib = _load(HIP_LIB)
    lib.zk_last_error.restype = ctypes.c_char_p
    return lib


def load_prover():
    """ctypes handle of the class-layer library (loads the kernel library first)."""
    load_hip()
    lib = _load(PROVER_LIB)
    lib.zkp_last_error.restype = ctypes.c_char_p
    return lib
