"""The C++ operator layer against the reference's own headers (build container only: skipped where the reference tree
is absent, e.g. on the GPU box).

oracle/Makefile's `linkcheck` target compiles a program that includes the reference's aten_ops.h where it lies, takes
the address of atenLinear / atenLstm1 / atenLstm2 / customAtenAddmm / customAtenMatmul through that header's
declarations and links it with pimaicompiler_amd/cpp/aten_ops_pimhip.cpp: a signature that drifts from the reference's
declaration is an undefined symbol.  The control build asks for a signature the reference does not declare and has to
fail at link time."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = "/root/reference"
REF_ATEN_H = os.path.join(REFERENCE, "runtime/include/executor/op_executor/aten_ops.h")
REF_UTILS_H = os.path.join(REFERENCE, "runtime/include/executor/utils/utils.h")

needs_reference = pytest.mark.skipif(not os.path.exists(REF_ATEN_H), reason="reference tree not present")


def _make(*args):
    return subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "linkcheck", *args], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True)


@needs_reference
def test_operator_layer_links_against_the_references_own_header():
    res = _make()
    assert res.returncode == 0, res.stdout
    exe = os.path.join(ROOT, "oracle", "_ref", "aten_ops_link_check")
    out = subprocess.run([exe], stdout=subprocess.PIPE, text=True)
    assert out.returncode == 0 and out.stdout.startswith("5 hot-path operators"), out.stdout


@needs_reference
def test_link_check_fails_on_a_signature_the_reference_does_not_declare(tmp_path):
    res = _make("LINKCHECK_DEFS=-DLINK_CHECK_DRIFT", f"LINKCHECK_OUT={tmp_path}/drift")
    assert res.returncode != 0
    assert "undefined reference" in res.stdout and "atenLinear(at::Tensor const&, at::Tensor const&, at::Tensor const&)" in res.stdout


def _enum_body(text, name):
    body = re.search(r"enum\s+(?:class\s+)?" + name + r"\s*\{(.*?)\}", text, flags=re.S).group(1)
    body = re.sub(r"//[^\n]*|/\*.*?\*/", "", body, flags=re.S)
    return [e.strip() for e in body.split(",") if e.strip()]


@needs_reference
def test_gemm_type_numbering_is_the_references():
    """GEMM_TYPE is a plain enum whose integers cross the boundary: same enumerators, same order, same values."""
    ref = _enum_body(open(REF_UTILS_H).read(), "GEMM_TYPE")
    assert ref == ["UNKNOW", "VV", "MV", "VM", "MM"]
    shim_text = open(os.path.join(ROOT, "pimaicompiler_amd/cpp/aten_ops_pimhip.h")).read()
    assert re.search(r"enum\s+GEMM_TYPE\s*\{", shim_text), "a plain enum as in the reference, not an enum class"
    assert _enum_body(shim_text, "GEMM_TYPE") == ref
    abi = _enum_body(open(os.path.join(ROOT, "include/pimhip.h")).read(), "PimHipGemmType")
    values = {e.split("=")[0].strip(): int(e.split("=")[1]) for e in abi}
    assert values == {"PIMHIP_GEMM_UNKNOWN": 0, "PIMHIP_GEMM_VV": 1, "PIMHIP_GEMM_MV": 2, "PIMHIP_GEMM_VM": 3, "PIMHIP_GEMM_MM": 4}
    from pimaicompiler_amd import _lib as L
    from pimaicompiler_amd import ops
    assert [int(getattr(ops.GemmType, n)) for n in ref] == [0, 1, 2, 3, 4]
    assert (L.GEMM_VV, L.GEMM_MV, L.GEMM_VM, L.GEMM_MM) == (1, 2, 3, 4)


@needs_reference
def test_hot_path_declarations_of_the_reference_header_are_the_ones_the_shim_header_repeats():
    """Text check of the five declarations, whitespace and parameter names aside (the link check is the binding one)."""
    def norm(sig):
        sig = re.sub(r"\s+", " ", sig)
        sig = re.sub(r"\s*([&*,()])\s*", r"\1", sig)
        return sig
    def decl(text, name):
        m = re.search(r"[^;{}]*\b" + name + r"\s*\([^;]*?\)\s*;", text, flags=re.S)
        return m.group(0).strip()
    def types_only(sig):
        # drop parameter names: keep what precedes the last identifier of each parameter
        head, params = sig.split("(", 1)
        params = params.rsplit(")", 1)[0]
        out = []
        for prm in re.split(r",(?![^<]*>)", params):
            prm = prm.split("=")[0].strip()
            out.append(re.sub(r"\b\w+$", "", prm).strip())
        return norm(head.split()[-1] if False else head) + "(" + ",".join(norm(o) for o in out) + ")"
    ref = open(REF_ATEN_H).read()
    shim = open(os.path.join(ROOT, "pimaicompiler_amd/cpp/aten_ops_pimhip.h")).read()
    for name in ("atenLinear", "atenLstm1", "atenLstm2", "customAtenAddmm", "customAtenMatmul"):
        assert types_only(decl(ref, name)) == types_only(decl(shim, name)), name


@needs_reference
def test_custom_ops_launchers_compile_where_the_references_do():
    """cpp/custom_ops_pimhip.h against the reference's custom_ops.h: one source holding the calls the reference's own code
    makes of the six launchers (custom_op_ut.cpp:42, :64; aten_ops_executor.cpp:159, :735) and their explicit instantiations
    is compiled once against each header (oracle/Makefile sigcheck); the control asks for an argument list neither declares."""
    ok = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "sigcheck"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert ok.returncode == 0 and "6 launchers compile against both headers" in ok.stdout, ok.stdout
    bad = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "sigcheck", "SIGCHECK_DEFS=-DSIGCHECK_DRIFT"], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True)
    assert bad.returncode != 0 and "6 launchers compile" not in bad.stdout
