"""The C-ABI library loads and exports every symbol include/cybq.h declares
(no compute calls: these run without a GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "cybq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cybq_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_operator_surface():
    names = _declared()
    for must in ("cybq_init", "cybq_destroy", "cybq_weight_upload", "cybq_weight_free", "cybq_matmul",
                 "cybq_dequant", "cybq_quantize", "cybq_strerror", "cybq_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from cyb_amd.backend import library_path
    path = library_path()
    if not os.path.exists(path):
        pytest.fail(f"{path} missing: run python -c 'import __graft_entry__ as g; g.build()'")
    lib = ctypes.CDLL(path)
    for name in _declared():
        assert hasattr(lib, name), name


def test_status_strings_and_version():
    from cyb_amd.backend import load_library
    lib = load_library()
    assert lib.cybq_version().decode().count(".") == 2
    assert lib.cybq_strerror(0) == b"ok"
    for code in range(-7, 0):
        assert lib.cybq_strerror(code) not in (b"ok", b"unknown status")
    assert lib.cybq_strerror(-99) == b"unknown status"


def test_null_arguments_are_rejected_without_a_device():
    from cyb_amd.backend import load_library
    lib = load_library()
    assert lib.cybq_init(0, None) == -1
    assert lib.cybq_matmul(None, None, None, 1, 1, None, 0, None) == -1
    assert lib.cybq_dequant(None, None, None, None) == -1
    assert lib.cybq_weight_info(None, None, None, None, None) == -1
    assert lib.cybq_last_error(None) == b""


def test_algorithmic_byte_counts():
    from cyb_amd import formats
    assert formats.weight_bytes(4, 4096, 4096) == 9_437_184
    assert formats.weight_bytes(4, 1024, 4096) == 2_359_296
    assert formats.weight_bytes(4, 14336, 4096) == 33_030_144
    assert formats.matmul_bytes(4, 14336, 4096, 1, 2, 4) == 33_095_680
    assert formats.matmul_bytes(4, 4096, 14336, 1, 2, 4) == 33_075_200
    assert formats.matmul_bytes(8, 2048, 2048, 1, 4, 4) == 4_472_832


# ---- the Rust binding (rust/cybq-sys, source only) mirrors the header 1:1 ----------------------

def _c_prototypes():
    """name -> list of parameter names, from include/cybq.h."""
    text = open(os.path.join(ROOT, "include", "cybq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = {}
    for m in re.finditer(r"\b(?:int|void|const char\*)\s+(cybq_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = [a.strip() for a in m.group(2).replace("\n", " ").split(",")]
        if args == ["void"] or args == [""]:
            args = []
        protos[m.group(1)] = [re.findall(r"[A-Za-z_][A-Za-z0-9_]*", a)[-1] for a in args]
    return protos


def _rust_prototypes():
    text = open(os.path.join(ROOT, "rust", "cybq-sys", "src", "lib.rs")).read()
    block = text[text.index('extern "C" {'):]
    protos = {}
    for m in re.finditer(r"pub fn (cybq_[a-z0-9_]+)\s*\(([^;]*?)\)\s*(?:->\s*[^;]+)?;", block, flags=re.S):
        args = [a.strip() for a in m.group(2).replace("\n", " ").split(",") if a.strip()]
        protos[m.group(1)] = [a.split(":")[0].strip() for a in args]
    return text, protos


def test_rust_binding_declares_exactly_the_header():
    c, (rust_text, r) = _c_prototypes(), _rust_prototypes()
    assert sorted(c) == sorted(_declared())                       # the prototype parser saw every entry point
    assert sorted(r) == sorted(c), set(r) ^ set(c)
    for name in c:
        assert r[name] == c[name], (name, r[name], c[name])      # same arity, same argument names, same order
    # enum values
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "cybq.h")).read(), flags=re.S)
    consts = dict(re.findall(r"\b(CYBQ_[A-Z0-9_]+)\s*=\s*(-?\d+)", header))
    assert len(consts) >= 20
    for k, v in consts.items():
        m = re.search(rf"pub const {k}: c_int = (-?\d+);", rust_text)
        assert m and m.group(1) == v, k


def test_diagnostics_stay_out_of_the_public_header():
    assert not any(n.startswith("cybq_debug") for n in _declared())
    dbg = open(os.path.join(ROOT, "cyb_amd", "csrc", "cybq_debug.h")).read()
    from cyb_amd.backend import load_library
    lib = load_library()
    for name in set(re.findall(r"\b(cybq_debug_[a-z0-9_]+)\s*\(", dbg)):
        assert hasattr(lib, name), name
