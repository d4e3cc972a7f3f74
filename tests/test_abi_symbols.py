"""The C-ABI library loads without a GPU and exports every function include/*.h declares."""
import ctypes
import glob
import os
import re

from gpuhelp import pkg
from zkhelp import ROOT


def declared_functions():
    names = []
    for h in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        names += re.findall(r"\b(zk_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_every_declared_symbol_is_exported():
    lib = pkg.load_hip()
    names = declared_functions()
    assert len(names) > 40
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/ but not exported: {missing}"


def test_init_fails_loudly_without_gpu_or_succeeds_with_one():
    lib = pkg.load_hip()
    rc = lib.zk_init(ctypes.c_int(0))
    if rc != 0:
        assert b"no HIP device" in lib.zk_last_error() or len(lib.zk_last_error()) > 0
