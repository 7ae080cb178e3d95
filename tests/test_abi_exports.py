"""The C-ABI libraries load without a GPU and export every symbol the headers declare (no compute)."""
import os
import re

import pytest

import gpu_lib

ROOT = gpu_lib.ROOT


def declared(header, prefixes="llmk|gpt2"):
    src = open(os.path.join(ROOT, "include", header)).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b((?:%s)_[a-z0-9_]+)\s*\(" % prefixes, src)))


def declared_data():
    return sorted(declared("llmk_data.h", "dataloader|evalloader|lr_scheduler|tokenizer|get_learning|safe|outlier_detector|init|update|logger") )


@pytest.fixture(scope="module")
def pkg():
    p = gpu_lib.package()
    for prec in ("bf16", "fp32"):
        if not os.path.exists(p.lib_path(prec)):
            spec_dir = os.path.join(ROOT, "llm.c_amd")
            import subprocess, sys
            subprocess.run([sys.executable, os.path.join(spec_dir, "build.py"), prec], check=True)
    return p


@pytest.mark.parametrize("precision", ["bf16", "fp32"])
def test_every_declared_symbol_is_exported(pkg, precision):
    L = pkg.load(precision)
    names = declared("llmk.h") + declared("llmk_gpt2.h") + declared_data()
    assert len(names) > 50
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    assert L.llmk_precision().decode() == precision
    assert L.llmk_sizeof_floatx() == (2 if precision == "bf16" else 4)


def test_python_binding_tables_match_headers(pkg):
    assert sorted(pkg.KERNEL_ABI) == declared("llmk.h")
    assert sorted(pkg.DRIVER_ABI) == declared("llmk_gpt2.h")
    assert sorted(pkg.DATA_ABI) == declared_data() and len(pkg.DATA_ABI) > 40


def test_missing_library_raises(pkg, monkeypatch):
    monkeypatch.setattr(pkg, "LIBDIR", "/nonexistent")
    monkeypatch.setattr(pkg, "_loaded", {})
    with pytest.raises(pkg.LibraryMissing):
        pkg.load("bf16")
