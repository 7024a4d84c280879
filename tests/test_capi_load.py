"""CPU checks of the C-ABI library: it loads without a GPU, exports every symbol the header declares,
and rejects bad arguments before touching a device."""
import ctypes as C
import os
import re

import numpy as np
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
    cases = [((3,), (3, 4), None), ((2, 3, 4), (5, 6, 4, 7), None), ((3, 4), (5, 6), None), ((2, 3, 4), (3, 4, 5), None),
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
    # beyond the reference (which raises "shape invalid" for unequal leading dimensions): extent 1 is broadcast
    assert O.matmul_plan((16, 12, 128, 64), (1, 12, 64, 64))[0] == 2
    got = pkg.matmul_plan((16, 12, 128, 64), (1, 12, 64, 64))
    assert got["shape"] == (16, 12, 128, 64) and got["batch"] == 192
    assert got["grid"] == dict(outer=16, inner=12, strides=(12 * 128 * 64, 0, 12 * 128 * 64), inner_strides=(128 * 64, 64 * 64, 128 * 64))
    got = pkg.matmul_plan((2, 3, 1, 7, 8), (2, 3, 4, 8, 6))  # adjacent dimensions with compatible strides merge
    assert got["shape"] == (2, 3, 4, 7, 6)
    assert got["grid"] == dict(outer=6, inner=4, strides=(56, 4 * 48, 4 * 42), inner_strides=(0, 48, 42))
    assert pkg.matmul_plan((5, 1, 3, 4), (1, 1, 4, 2))["grid"] == dict(outer=5, inner=1, strides=(12, 0, 6), inner_strides=(0, 0, 0))
    with pytest.raises(NotImplementedError):
        pkg.matmul_plan((4, 1, 5, 7, 8), (1, 3, 5, 8, 6))
    with pytest.raises(pkg.InvalidArgumentError):
        pkg.matmul_plan((2, 3, 4), (3, 4, 5))


def test_broadcast_shape_rule(pkg):
    """The shape rule of tfcc/core/operations/tfcc_math.cpp:38-86 against numpy's, and its merged forms: equal rank,
    each dimension equal or 1 on one side, neighbouring dimensions never of the same kind, products preserved."""
    rng = np.random.default_rng(0)
    for _ in range(300):
        rank = int(rng.integers(1, 6))
        full = [int(rng.integers(1, 5)) for _ in range(rank)]
        s1 = [d if rng.random() < 0.6 else 1 for d in full][int(rng.integers(0, rank)):]
        s2 = [d if rng.random() < 0.6 else 1 for d in full][int(rng.integers(0, rank)):]
        shape, c1, c2 = pkg.broadcast_shapes(s1, s2)
        assert shape == tuple(np.broadcast_shapes(tuple(s1), tuple(s2)))
        assert len(c1) == len(c2) >= 1
        assert int(np.prod(c1)) == int(np.prod(s1)) and int(np.prod(c2)) == int(np.prod(s2))
        kinds = [0 if x == y else (1 if x == 1 else 2) for x, y in zip(c1, c2)]
        assert all(x == y or x == 1 or y == 1 for x, y in zip(c1, c2))
        assert all(k1 != k2 for k1, k2 in zip(kinds, kinds[1:]))
        # the merged shapes broadcast to the same values as the originals
        a = rng.normal(size=s1)
        b = rng.normal(size=s2)
        assert np.array_equal((a.reshape(c1) + b.reshape(c2)).reshape(shape), a + b)
    assert pkg.broadcast_shapes((16, 12, 128, 128), (16, 1, 1, 128)) == ((16, 12, 128, 128), (16, 1536, 128), (16, 1, 128))
    assert pkg.broadcast_shapes((7, 33), (33,)) == ((7, 33), (7, 33), (1, 33))
    assert pkg.broadcast_shapes((1,), (1,)) == ((1,), (1,), (1,))
    for bad in (((2, 3), (2, 2)), ((), (3,))):
        with pytest.raises(pkg.InvalidArgumentError):
            pkg.broadcast_shapes(*bad)
