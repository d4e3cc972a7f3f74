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


def _want_hw_queues():
    """The library keeps up to seven streams busy (the caller's, four for openings, two for sumcheck jobs).  HIP maps
    streams onto GPU_MAX_HW_QUEUES hardware queues (4 unless set) and streams that share a queue run one after the
    other, so ask for at least sixteen (measured when this was added: the decoder layer took 7 % less time with 8 queues than with 4 and another 1 % less with 16).  The HIP runtime reads the variable when it is loaded: this must run before that.
    ZKLLM_HW_QUEUES=0 leaves the variable alone, ZKLLM_HW_QUEUES=N sets it to N."""
    want = os.environ.get("ZKLLM_HW_QUEUES", "")
    if want == "0":
        return
    try:
        cur = int(os.environ.get("GPU_MAX_HW_QUEUES", "0"))
    except ValueError:
        cur = 0
    n = int(want) if want.isdigit() else max(cur, 16)
    os.environ["GPU_MAX_HW_QUEUES"] = str(min(n, 32))


def load_hip():
    """ctypes handle of the C-ABI kernel library."""
    _want_hw_queues()
    lib = _load(HIP_LIB)
    lib.zk_last_error.restype = ctypes.c_char_p
    return lib


def load_prover():
    """ctypes handle of the class-layer library (loads the kernel library first)."""
    load_hip()
    lib = _load(PROVER_LIB)
    lib.zkp_last_error.restype = ctypes.c_char_p
    return lib
