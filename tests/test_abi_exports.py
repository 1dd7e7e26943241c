"""The C-ABI shared library loads and exports exactly the entry points that include/candle_qhip.h
declares (no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "candle_qhip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)          # comments
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)           # preprocessor lines
    names = re.findall(r"\b(cq_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


@pytest.fixture(scope="module")
def lib():
    from candle_amd import qhip
    if not os.path.exists(qhip.LIB_PATH):
        from candle_amd import build as qbuild
        qbuild.build(verbose=False)
    return ctypes.CDLL(qhip.LIB_PATH)


def test_header_declares_something():
    names = declared_functions()
    assert "cq_qmatmul" in names and "cq_weight_create" in names and len(names) >= 25


def test_library_exports_every_declared_symbol(lib):
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_binding_lists_every_declared_symbol():
    from candle_amd import qhip
    assert sorted(qhip.EXPORTS) == declared_functions()


def test_library_exports_nothing_undeclared(lib):
    """Every exported cq_* symbol with C linkage is declared (internal launchers are C++-mangled)."""
    import subprocess
    from candle_amd import qhip
    out = subprocess.run(["nm", "-D", "--defined-only", qhip.LIB_PATH], capture_output=True, text=True).stdout
    exported = sorted({ln.split()[-1] for ln in out.splitlines() if re.match(r".* T cq_[a-z0-9_]+$", ln)})
    assert exported == declared_functions()


def test_metadata_calls_need_no_gpu(lib):
    """Pure host-side queries (GgmlDType::block_size / type_size, k_quants VecDotType)."""
    lib.cq_block_size.restype = ctypes.c_int
    lib.cq_type_size.restype = ctypes.c_int
    lib.cq_vec_dot_type.restype = ctypes.c_int
    Q4_0, Q8_0, Q4K, Q6K, Q8K = 2, 8, 12, 14, 15
    assert (lib.cq_block_size(Q4_0), lib.cq_type_size(Q4_0)) == (32, 18)
    assert (lib.cq_block_size(Q8_0), lib.cq_type_size(Q8_0)) == (32, 34)
    assert (lib.cq_block_size(Q4K), lib.cq_type_size(Q4K)) == (256, 144)
    assert (lib.cq_block_size(Q6K), lib.cq_type_size(Q6K)) == (256, 210)
    assert (lib.cq_block_size(Q8K), lib.cq_type_size(Q8K)) == (256, 292)
    assert lib.cq_vec_dot_type(Q4_0) == Q8_0 and lib.cq_vec_dot_type(Q8_0) == Q8_0
    assert lib.cq_vec_dot_type(Q4K) == Q8K and lib.cq_vec_dot_type(Q6K) == Q8K
