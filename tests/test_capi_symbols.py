"""The C-ABI library loads and exports every symbol include/hemm.h declares (no GPU needed)."""
import ctypes
import os
import re

from __graft_entry__ import ROOT, load_package


def declared_symbols():
    names = []
    for fn in sorted(os.listdir(os.path.join(ROOT, "include"))):
        text = open(os.path.join(ROOT, "include", fn)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b((?:hemm|hellm)_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_header_symbols():
    pkg = load_package()
    L = ctypes.CDLL(pkg.LIB_PATH)
    syms = declared_symbols()
    assert "hemm_ntt" in syms and "hemm_context_create" in syms
    missing = [s for s in syms if not hasattr(L, s)]
    assert missing == []


def test_primes_helper_matches_oracle_generator():
    pkg = load_package()
    from oracle import oracle as O
    assert pkg.primes_below(60, 16, 24) == O.primes_below(60, 16, 24)
    assert pkg.primes_below(42, 10, 5) == O.primes_below(42, 10, 5)


def test_term_records_match_the_library_layout():
    """The ctypes records the Python side fills have the size the library was compiled with."""
    pkg = load_package()
    L = ctypes.CDLL(pkg.LIB_PATH)
    rot, lin = ctypes.c_uint32(0), ctypes.c_uint32(0)
    L.hemm_abi_sizes.restype = None
    L.hemm_abi_sizes(ctypes.byref(rot), ctypes.byref(lin))
    assert rot.value == ctypes.sizeof(pkg.RotTerm) == 56
    assert lin.value == ctypes.sizeof(pkg.LinTerm) == 32
