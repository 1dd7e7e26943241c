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


def c_declarations():
    """[(return type, name, [(type, name), ...])] of every function the header declares."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    out = []
    for ret, name, args in re.findall(r"([A-Za-z_][\w ]*?[\s\*]+)(cq_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        params = []
        for a in " ".join(args.split()).split(","):
            a = a.strip()
            if a == "void" or not a:
                continue
            m = re.match(r"(.*?)(\w+)$", a)
            params.append((m.group(1).strip(), m.group(2)))
        out.append((" ".join(ret.split()), name, params))
    return out


_RUST_TYPES = {
    "int": "c_int", "int64_t": "i64", "size_t": "usize", "float": "f32", "void": "()",
    "const char *": "*const c_char", "const void *": "*const c_void", "void *": "*mut c_void",
    "const float *": "*const f32", "float *": "*mut f32", "float *const *": "*const *mut f32",
    "const int32_t *": "*const i32", "int32_t *": "*mut i32", "int64_t *": "*mut i64", "uint16_t *": "*mut u16",
    "uint64_t *": "*mut u64", "double *": "*mut f64",
    "cq_weight *": "*mut CqWeight", "const cq_weight *": "*const CqWeight", "cq_weight **": "*mut *mut CqWeight",
    "const cq_weight *const *": "*const *const CqWeight",
}


def rust_signature(decl):
    """The `pub fn` line a Rust sys-crate declares for one C declaration."""
    ret, name, params = decl
    args = ", ".join(f"{n}: {_RUST_TYPES[t]}" for t, n in params)
    tail = "" if ret == "void" else f" -> {_RUST_TYPES[ret]}"
    return f"pub fn {name}({args}){tail};"


def test_integration_doc_binds_every_declared_symbol():
    """The integration guide's `extern "C"` block (the sys-crate a maintainer adds) lists every entry point of
    the header with the header's argument names and the matching Rust types."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = re.search(r'extern "C" \{(.*?)\n\}', text, flags=re.S).group(1)
    got = {re.match(r"pub fn (cq_\w+)", " ".join(f.split())).group(1): " ".join(f.split()).replace("( ", "(")
           for f in re.findall(r"pub fn cq_[^;]*;", block, flags=re.S)}
    want = {d[1]: rust_signature(d) for d in c_declarations()}
    assert sorted(got) == sorted(want)
    for name in want:
        assert got[name] == want[name], (got[name], want[name])


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
    Q5_0, Q3K = 6, 11
    assert (lib.cq_block_size(3), lib.cq_type_size(3), lib.cq_vec_dot_type(3)) == (32, 20, 9)      # Q4_1 x Q8_1, k_quants.rs:51-57, :260
    assert (lib.cq_block_size(7), lib.cq_type_size(7), lib.cq_vec_dot_type(7)) == (32, 24, 9)      # Q5_1 x Q8_1, k_quants.rs:69-76, :457
    assert (lib.cq_block_size(Q5_0), lib.cq_type_size(Q5_0), lib.cq_vec_dot_type(Q5_0)) == (32, 22, Q8_0)    # k_quants.rs:61-67, :356
    assert (lib.cq_block_size(Q3K), lib.cq_type_size(Q3K), lib.cq_vec_dot_type(Q3K)) == (256, 110, Q8K)     # k_quants.rs:107-114, :877
    assert (lib.cq_block_size(10), lib.cq_type_size(10), lib.cq_vec_dot_type(10)) == (256, 84, Q8K)         # Q2K, k_quants.rs:96-103, :701
    assert (lib.cq_block_size(1), lib.cq_type_size(1), lib.cq_vec_dot_type(1)) == (0, 0, -1)                # F16: not handled
    assert (lib.cq_block_size(Q4_0), lib.cq_type_size(Q4_0)) == (32, 18)
    assert (lib.cq_block_size(Q8_0), lib.cq_type_size(Q8_0)) == (32, 34)
    assert (lib.cq_block_size(Q4K), lib.cq_type_size(Q4K)) == (256, 144)
    assert (lib.cq_block_size(Q6K), lib.cq_type_size(Q6K)) == (256, 210)
    assert (lib.cq_block_size(Q8K), lib.cq_type_size(Q8K)) == (256, 292)
    assert lib.cq_vec_dot_type(Q4_0) == Q8_0 and lib.cq_vec_dot_type(Q8_0) == Q8_0
    assert lib.cq_vec_dot_type(Q4K) == Q8K and lib.cq_vec_dot_type(Q6K) == Q8K
