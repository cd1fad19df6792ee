"""The C-ABI library loads and exports every symbol the public header declares.
No compute is attempted here (runs without a GPU)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import wgml_amd as W
from wgml_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "wgml_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"WGML_API\s+[\w\s\*]+?\b(wgml_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    syms = header_symbols()
    assert len(syms) >= 55
    raw = C.CDLL(os.fspath(_lib.LIB_PATH))
    missing = [s for s in syms if not hasattr(raw, s)]
    assert not missing, missing
    # and nothing is exported that the header does not declare
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", os.fspath(_lib.LIB_PATH)], capture_output=True,
                         text=True, check=True).stdout
    exported = {ln.split()[-1] for ln in out.splitlines() if " T " in ln and "wgml_" in ln}
    assert exported == set(syms), exported ^ set(syms)


def test_binding_covers_the_header():
    declared = set(header_symbols())
    bound = set(_lib.PROTOTYPES)
    assert declared == bound, declared ^ bound


def test_version_and_host_helpers():
    assert b"gfx950" in _lib.lib.wgml_version()
    assert _lib.lib.wgml_quant_block_elems(W.Q8_0) == 32
    assert _lib.lib.wgml_quant_block_elems(W.Q4_K) == 256
    assert _lib.lib.wgml_quant_block_elems(W.Q6_K) == 256
    assert _lib.lib.wgml_quant_block_elems(W.Q4_0) == 32 and _lib.lib.wgml_quant_block_elems(W.Q5_K) == 256
    assert _lib.lib.wgml_quant_block_elems(10) == 0  # Q2_K: a format the reference cannot read either
    assert W.quant_bytes(W.Q4_K, 100) == 0          # not a whole block
    assert W.quant_bytes(W.F32, 10) == 40


def test_errors_are_reported_not_crashed():
    # null arguments come back as WGML_E_INVALID with a message
    rc = _lib.lib.wgml_ctx_synchronize(None)
    assert rc == _lib.E_INVALID and b"null" in _lib.lib.wgml_last_error()
    rc = _lib.lib.wgml_buf_create(None, 16, C.byref(C.c_void_p()))
    assert rc == _lib.E_INVALID
    with pytest.raises(W.WgmlError) as ei:
        W.rng_tokens(1, 4, 0)
    assert ei.value.code == _lib.E_INVALID


def test_no_device_is_an_error_not_a_fallback():
    # (asks the library itself whether there is a device: another runtime's view of the machine
    # need not agree with it)
    try:
        W.GpuInstance(0)
    except W.WgmlError as e:
        assert e.code == _lib.E_NO_DEVICE
    else:
        pytest.skip("a GPU is present")
