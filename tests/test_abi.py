"""CPU-side checks of the C ABI: the library loads, exports every function include/pimhip.h declares, and the
integer-only shape logic (no GPU involved) agrees with the oracle's line-by-line restatement."""
import ctypes
import itertools
import os
import re

import pytest

from oracle import oracle
from pimaicompiler_amd import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


HEADERS = ("pimhip.h", "pimhip_probe.h")   # the drop-in interface; the measurement aids


def declared_functions(headers=HEADERS):
    names = set()
    for h in headers:
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(pimhip_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_the_drop_in_header_carries_no_measurement_aids():
    assert not [n for n in declared_functions(("pimhip.h",)) if "probe" in n or "debug" in n or "trace" in n]
    assert declared_functions(("pimhip_probe.h",)) == ["pimhip_probe_stream_read", "pimhip_probe_xcc_map"]


def test_header_declares_what_the_binding_binds():
    assert declared_functions() == sorted(L.SIGNATURES)


def test_library_loads_and_exports_every_declared_symbol():
    lib = L.load()
    for name in declared_functions():
        assert hasattr(lib, name), name


def test_header_is_plain_c_and_links_against_the_library(tmp_path):
    """include/pimhip.h is what a cgo / JNI / ctypes binding reads: it has to compile as C99 with nothing but the standard
    headers, and a C program that names every declared function has to link against libpimhip.so."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    src = tmp_path / "uses_every_entry_point.c"
    names = declared_functions()
    src.write_text('#include "pimhip.h"\n#include "pimhip_probe.h"\n#include <stdio.h>\nint main(void)\n{\n    const void* table[] = {\n' +
                   "".join(f"        (const void*)&{n},\n" for n in names) +
                   '    };\n    printf("%d\\n", (int)(sizeof(table) / sizeof(table[0])));\n    return 0;\n}\n')
    exe = tmp_path / "uses_every_entry_point"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                    L.LIB_PATH, "-Wl,-rpath," + os.path.dirname(L.LIB_PATH), "-Wl,--allow-shlib-undefined"], check=True, capture_output=True)


def test_last_error_is_a_string():
    lib = L.load()
    assert isinstance(lib.pimhip_last_error(), bytes)


def test_enums_match_header():
    text = open(os.path.join(ROOT, "include", "pimhip.h")).read()
    for name, value in [("PIMHIP_OK", 0), ("PIMHIP_ERR_INVALID_ARGUMENT", 1), ("PIMHIP_ERR_UNSUPPORTED", 2),
                        ("PIMHIP_ERR_HIP", 3), ("PIMHIP_ERR_NOT_INITIALIZED", 4), ("PIMHIP_ERR_TIMEOUT", 5),
                        ("PIMHIP_ACT_RELU", 1), ("PIMHIP_I_X_W", 0), ("PIMHIP_W_X_I", 1), ("PIMHIP_GEMM_VV", 1),
                        ("PIMHIP_GEMM_MV", 2), ("PIMHIP_GEMM_VM", 3), ("PIMHIP_GEMM_MM", 4)]:
        assert re.search(rf"\b{name}\s*=\s*{value}\b", text), name
        assert getattr(L, name, getattr(L, name.replace("PIMHIP_", ""), value)) == value


def _product_broadcast(s1, s2):
    lib = L.load()
    a = (ctypes.c_int64 * 4)(*list(s1) + [0] * (4 - len(s1)))
    b = (ctypes.c_int64 * 4)(*list(s2) + [0] * (4 - len(s2)))
    ra, rb = ctypes.c_int(len(s1)), ctypes.c_int(len(s2))
    rc = lib.pimhip_gemm_broadcast(a, ctypes.byref(ra), b, ctypes.byref(rb))
    return rc, list(a[:ra.value]), list(b[:rb.value])


def _all_shapes(max_rank=4, dims=(1, 2, 3)):
    for r in range(1, max_rank + 1):
        yield from itertools.product(dims, repeat=r)


def test_gemm_broadcast_matches_oracle_on_every_small_shape_pair():
    """Exhaustive over ranks 1-4 with dims in {1,2,3}: 120 x 120 pairs."""
    n_ok = n_unsupported = 0
    for s1 in _all_shapes():
        for s2 in _all_shapes():
            orc, o1, o2 = oracle.gemm_broadcast(s1, s2)
            prc, p1, p2 = _product_broadcast(s1, s2)
            if orc == 2:
                # The reference indexes out of range here; the product only has to refuse or stay in bounds.
                assert prc in (L.PIMHIP_OK, L.PIMHIP_ERR_UNSUPPORTED, L.PIMHIP_ERR_INVALID_ARGUMENT)
                continue
            if orc == 1:
                assert prc == L.PIMHIP_ERR_INVALID_ARGUMENT, (s1, s2)
                continue
            if len(o1) == 4 and len(o2) == 4:
                assert prc == L.PIMHIP_OK, (s1, s2, o1, o2)
                n_ok += 1
            else:
                assert prc == L.PIMHIP_ERR_UNSUPPORTED, (s1, s2, o1, o2)
                n_unsupported += 1
            assert (p1, p2) == (o1, o2), (s1, s2)
    assert n_ok > 10000 and n_unsupported > 0


def test_get_gemm_type_matches_oracle():
    lib = L.load()
    for a in itertools.product((1, 2, 5), repeat=4):
        for b in itertools.product((1, 2, 5), repeat=4):
            out = ctypes.c_int(-1)
            assert lib.pimhip_get_gemm_type((ctypes.c_int64 * 4)(*a), (ctypes.c_int64 * 4)(*b), ctypes.byref(out)) == 0
            assert out.value == oracle.get_gemm_type(a, b), (a, b)


def test_gemm_broadcast_rejects_bad_ranks():
    lib = L.load()
    a = (ctypes.c_int64 * 4)(1, 1, 1, 1)
    for r1, r2 in [(0, 2), (5, 2), (2, 0), (2, 5)]:
        ra, rb = ctypes.c_int(r1), ctypes.c_int(r2)
        assert lib.pimhip_gemm_broadcast(a, ctypes.byref(ra), a, ctypes.byref(rb)) == L.PIMHIP_ERR_INVALID_ARGUMENT
        assert b"rank" in lib.pimhip_last_error()


@pytest.mark.parametrize("mat1,mat2,kind", [
    # the shapes the optimiser passes leave for the hot path (swap_addmm_inputs: W[out,in] x x^T[in,1])
    ((4096, 1024), (1024, 1), L.GEMM_MV),
    ((1, 1024), (1024, 4096), L.GEMM_VM),
    ((1, 1, 1, 1024), (1024, 4096), L.GEMM_VM),       # custom_op_ut.cpp:27-28
    ((4096, 1024), (1, 1, 1024, 1), L.GEMM_MV),       # custom_op_ut.cpp:49-50
    ((1, 1024), (1024, 1), L.GEMM_VV),
    ((13, 768), (768, 3072), L.GEMM_MM),
    ((2, 1, 13, 64), (2, 1, 64, 13), L.GEMM_MM),
])
def test_dispatch_classes_of_known_call_sites(mat1, mat2, kind):
    rc, a, b = _product_broadcast(mat1, mat2)
    assert rc == L.PIMHIP_OK
    out = ctypes.c_int(-1)
    L.load().pimhip_get_gemm_type((ctypes.c_int64 * 4)(*a), (ctypes.c_int64 * 4)(*b), ctypes.byref(out))
    assert out.value == kind


# ---- the product's shape logic against sources that do not restate it --------------------------------------------
def _abi_broadcast(s1, s2):
    rc, o1, o2 = _product_broadcast(s1, s2)
    if rc == L.PIMHIP_OK:
        return "ok", o1, o2
    if rc == L.PIMHIP_ERR_UNSUPPORTED:
        return "short", o1, o2
    return "abort", None, None


def _abi_type(o1, o2):
    from shape_cases import TYPE_NAMES
    out = ctypes.c_int(-1)
    assert L.load().pimhip_get_gemm_type((ctypes.c_int64 * 4)(*o1), (ctypes.c_int64 * 4)(*o2), ctypes.byref(out)) == 0
    return TYPE_NAMES[out.value]


def test_product_shape_logic_matches_the_hand_traced_table():
    from shape_cases import check_hand_traced
    check_hand_traced(_abi_broadcast, _abi_type, undefined_may_refuse=True)


def test_product_shape_logic_agrees_with_the_meaning_of_the_product():
    from shape_cases import check_matmul_semantics
    n_checked, n_as_product, exceptions = check_matmul_semantics(_abi_broadcast, _abi_type)
    assert n_checked > 600 and n_as_product > 550
