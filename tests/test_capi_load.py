"""CPU checks of the C-ABI library: it loads without a GPU, exports every symbol the header declares,
and rejects bad arguments before touching a device."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tfcc_rocm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tfcc_rocm_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree(pkg):
    assert sorted(pkg.SYMBOLS) == declared_symbols()


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.lib()
    for name in declared_symbols():
        assert getattr(lib, name) is not None
    assert lib.tfcc_rocm_version().startswith(b"tfcc_rocm")


def test_bad_arguments_are_rejected_without_a_device(pkg):
    lib = pkg.lib()
    assert lib.tfcc_rocm_gemm_u8s8s32(None, None, None) == 1
    assert b"null descriptor" in lib.tfcc_rocm_last_error_string()
    d = pkg.QGemmDesc()
    assert lib.tfcc_rocm_gemm_u8s8s32(None, C.byref(d), None) == 1
    assert lib.tfcc_rocm_sgemm_strided_batched(None, None, 0, None, 0, None, None, 0, 1, 1, 1, 1) == 1
    assert lib.tfcc_rocm_requantize(None, None, 0, None, 0, 0, None, None, None, None) == 1
    assert lib.tfcc_rocm_reduce_sum_rows(None, None, 0, 1, 1, 1, None) == 1
    assert lib.tfcc_rocm_fill_async(None, C.c_void_p(16), 0, 3, 4) == 1
    assert b"element size" in lib.tfcc_rocm_last_error_string()


def test_matmul_plan_rules(pkg):
    # tfcc/core/operations/tfcc_blas.cpp:26-42 and tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:127-145
    import oracle_lib as O
    cases = [((3,), (3, 4), None), ((2, 3, 4), (5, 6, 4, 7), None), ((3, 4), (5, 6), None), ((2, 3, 4), (1, 4, 5), None),
             ((3, 4), (4, 5), (4,)), ((6, 3, 4), (4, 5), None), ((3, 4), (6, 4, 5), (5,)), ((2, 3, 5, 7), (2, 3, 7, 4), None)]
    for sa, sb, sbias in cases:
        st, want = O.matmul_plan(sa, sb, sbias)
        if st != 0:
            with pytest.raises(pkg.InvalidArgumentError):
                pkg.matmul_plan(sa, sb, sbias)
        else:
            got = pkg.matmul_plan(sa, sb, sbias)
            assert (got["m"], got["n"], got["k"], got["batch"], got["shape"]) == (want["m"], want["n"], want["k"], want["batch"], want["shape"])
            assert (got["stride_a"], got["stride_b"], got["stride_c"]) == (want["strideA"], want["strideB"], want["strideC"])
