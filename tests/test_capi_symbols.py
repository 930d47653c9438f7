"""CPU-side checks of the boundary: the C ABI library loads, exports every symbol include/sbhip.h
declares (and the binding table knows each of them), and the pybind11 module exposes the reference's
backend interface.  No compute calls: none of this needs a GPU."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sbhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sb_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from streambrain_amd import _capi
    lib = _capi.lib()
    names = declared_symbols()
    assert len(names) >= 45
    for name in names:
        assert hasattr(lib, name), f"{name} declared in sbhip.h but not exported"
    assert sorted(_capi.exported_symbols()) == names, "binding table and header disagree"
    assert lib.sb_abi_version() == 1


def test_uninitialised_calls_fail_with_status_not_exit():
    from streambrain_amd import _capi
    if _capi._initialised:
        pytest.skip("library already initialised in this process")
    lib = _capi.lib()
    assert lib.sb_sync() == -3  # SB_ERR_STATE
    assert b"sb_init" in lib.sb_last_error()


def test_pybind_module_has_reference_interface():
    import sys
    sys.path.insert(0, os.path.join(ROOT, "streambrain_amd"))
    import _bcpnn_backend_hip_internals as m
    assert callable(m.initialize)
    for cls in (m.PyNetwork_float32, m.PyNetwork_float64):
        # backend_full_cuda_internals.cu:764-780 (the reference's bound methods)
        for meth in ("add_dense_layer", "add_plastic_layer", "initiate_training", "train_layer",
                     "training_done", "evaluate"):
            assert hasattr(cls, meth)
        for meth in ("set_layer_state", "get_layer_state", "train_epoch", "evaluate_counts", "predict"):
            assert hasattr(cls, meth)


def test_oracle_is_not_reachable_from_the_product():
    pkg = os.path.join(ROOT, "streambrain_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"
    for f in ("BCPNN/__init__.py", "include/sbhip.h"):
        assert "oracle" not in open(os.path.join(ROOT, f)).read().lower()
