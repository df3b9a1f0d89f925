"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

import pytest

from conftest import ROOT
from spgt_amd import _lib

HEADER = os.path.join(ROOT, "include", "spgt_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(spgt_[a-z0-9_]+)\s*\(", text)))


def test_library_is_built():
    assert os.path.exists(_lib.LIB_PATH), "run `python -m spgt_amd.build` first"


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_functions()
    assert len(names) >= 8
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in spgt_hip.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature in spgt_amd/_lib.py"
    for name in _lib.SIGNATURES:
        assert name in names, f"{name} is bound in _lib.py but not declared in spgt_hip.h"


def test_version_and_error_string():
    lib = _lib.load()
    assert lib.spgt_version() >= 100
    assert isinstance(_lib.last_error(), str)


def test_workspace_queries_reject_bad_shapes():
    lib = _lib.load()
    assert lib.spgt_galerkin_attention_cccr_workspace_bytes(1, 4, 33, 100) == 0
    assert lib.spgt_galerkin_attention_cccr_workspace_bytes(8, 4, 32, 44521) > 0
    assert lib.spgt_galerkin_attention_fused_workspace_bytes(8, 44521, 4, 0) > 0
    assert lib.spgt_galerkin_attention_fused_workspace_bytes(8, 44521, 4, 1) == 0
    assert lib.spgt_batched_skinny_gemm_workspace_bytes(32, 32, 44521, 32) > 0
    assert lib.spgt_batched_skinny_gemm_workspace_bytes(0, 32, 10, 1) == 0


def test_argument_errors_are_reported_without_a_gpu():
    lib = _lib.load()
    rc = lib.spgt_galerkin_attention_cccr_forward(None, None, None, None, None, 0, 1, 4, 32, 10, None)
    assert rc == -1 and "null" in _lib.last_error()
    with pytest.raises(_lib.SpgtError):
        _lib.check(rc)


def test_ops_refuse_cpu_tensors():
    import torch
    from spgt_amd.extension.bind.galerkin_attention import batched_skinny_gemm, multihead_galerkin_attention_cccr_cuda
    q = torch.zeros(1, 4, 32, 8)
    with pytest.raises(_lib.SpgtError):
        multihead_galerkin_attention_cccr_cuda(q, q, q)
    with pytest.raises(_lib.SpgtError):
        batched_skinny_gemm(torch.zeros(2, 3, 4), torch.zeros(2, 4, 5))
