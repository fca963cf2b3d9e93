"""The C-ABI library loads and exports every symbol include/kge_mi355.h declares (no GPU needed)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "kge_mi355.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kge_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("kge_residual_fwd", "kge_score_fwd", "kge_inspect", "kge_score_bwd", "kge_build_index"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from cuke_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m cuke_amd.build"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in declared_symbols() if not hasattr(handle, n)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_binding_table_matches_header():
    from cuke_amd import _lib
    assert sorted(_lib.EXPORTS) == declared_symbols()


def test_strerror_and_version_without_gpu():
    from cuke_amd import _lib
    L = _lib.lib()
    assert L.kge_abi_version() == _lib.ABI_VERSION == 2
    assert L.kge_strerror(0) == b"ok"
    assert b"workspace" in L.kge_strerror(-4)


def test_host_side_rejects_cpu_tensors():
    import pytest
    import torch
    from cuke_amd.kge import KGEModel, KgeError
    with pytest.raises(KgeError):
        KGEModel("TransE", torch.zeros(4, 8), torch.zeros(2, 8))
    with pytest.raises(ValueError):
        KGEModel("NoSuchModel", torch.zeros(4, 8), torch.zeros(2, 8))
