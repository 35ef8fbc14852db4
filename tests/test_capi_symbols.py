"""CPU-side checks of the C-ABI library: it loads, and it exports every function include/ckks_hip.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ckks_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:ckks|pcmm)_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_path():
    names = declared_functions()
    for must in ["ckks_ctx_create", "ckks_ntt_fwd", "ckks_ntt_inv", "ckks_modup_qj_to_t", "ckks_moddown_pql_to_ql",
                 "ckks_external_product_t", "ckks_hybrid_keyswitch", "pcmm_ppmm", "pcmm_rlwe_decompose"]:
        assert must in names


def test_library_exports_every_declared_symbol():
    from ckks_llm_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -c 'import __graft_entry__ as g; g.build()'"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, missing
    # the Python binding declares the same set (plus the arithmetic-mode test hook)
    L = _lib.load_library()
    assert L.ckks_version().decode().startswith("ckks_llm_amd")


def test_no_oracle_in_product():
    """The shipped package and library never reference the oracle."""
    pkg = os.path.join(ROOT, "ckks_llm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")) or f == "Makefile":
                src = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle_py" not in src and "ckks_oracle.h" not in src.replace("names as in ckks_oracle.h", ""), f
