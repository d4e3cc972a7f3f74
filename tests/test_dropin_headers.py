"""The reference's six driver sources compile, unmodified, against the forwarding headers of the class layer.
Only runs where the reference tree is present (it is read as compiler input, never copied)."""
import os
import subprocess

import pytest

from zkhelp import ROOT

REF = "/root/reference"
DRIVERS = ["ppgen", "commit-param", "rmsnorm", "self-attn", "ffn", "skip-connection"]


@pytest.mark.skipif(not os.path.exists(os.path.join(REF, "ffn.cu")), reason="reference tree not present")
@pytest.mark.parametrize("name", DRIVERS)
def test_reference_driver_compiles_against_compat_headers(name, tmp_path):
    src = open(os.path.join(REF, name + ".cu")).read()
    inc = os.path.join(ROOT, "zkllm-ccs2024_amd", "host", "compat")
    # the source is fed on stdin so that its quoted includes resolve to the forwarding headers, not to the reference's own
    r = subprocess.run(["g++", "-std=c++17", "-x", "c++", "-fsyntax-only", "-w", "-I" + inc, "-"], input=src, text=True, capture_output=True, cwd=tmp_path)
    assert r.returncode == 0, r.stderr[:2000]


def test_every_reference_header_name_has_a_forwarding_header(tmp_path):
    """A source that includes each class header by the reference's file name and touches one member of each compiles."""
    names = ["bls12-381", "fr-tensor", "g1-tensor", "ioutils", "commitment", "polynomial", "proof", "zkfc", "tlookup",
             "rescaling", "zksoftmax", "zkrelu"]
    src = "".join(f'#include "{n}.cuh"\n' for n in names)
    src += "void use(const FrTensor& X) { zkReLU r(16); FrTensor y = r(X); r.prove(X, y); Rescaling s(16); FrTensor z = s(X); }\n"
    inc = os.path.join(ROOT, "zkllm-ccs2024_amd", "host", "compat")
    r = subprocess.run(["g++", "-std=c++17", "-x", "c++", "-fsyntax-only", "-w", "-I" + inc, "-"], input=src, text=True, capture_output=True, cwd=tmp_path)
    assert r.returncode == 0, r.stderr[:2000]
