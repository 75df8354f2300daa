"""CPU-only checks of the drop-in boundary: the C-ABI library loads and exports every symbol the
header declares, and the Python layer refuses to compute anywhere but on the GPU."""

import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "nrl_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nrl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from rl_amd import _lib

    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 10
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/nrl_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared
    assert lib.nrl_version() == _lib.ABI_VERSION


def test_struct_layouts_match_header_field_order():
    from rl_amd import _lib

    text = open(os.path.join(ROOT, "include", "nrl_hip.h")).read()
    body = re.search(r"typedef struct nrl_grpo_cfg \{(.*?)\} nrl_grpo_cfg;", text, re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if decl:
            names += [n.strip() for n in decl.split(None, 1)[1].split(",")]
    assert names == [n for n, _ in _lib.NrlGrpoCfg._fields_]


def test_cpu_tensors_fail_loudly():
    import rl_amd.ops  # noqa: F401

    with pytest.raises(RuntimeError, match="GPU only"):
        torch.ops.rl_amd.logprob_fwd(torch.randn(1, 2, 8), torch.zeros(1, 2, dtype=torch.long), 2, 0, 8, 1.0, 1, False)


def test_missing_library_raises(monkeypatch):
    from rl_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/librl_amd_hip.so")
    with pytest.raises(RuntimeError, match="no other compute path"):
        _lib.load()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "rl_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, re.M), os.path.join(dirpath, f)
                assert "_work/" not in text, os.path.join(dirpath, f)
