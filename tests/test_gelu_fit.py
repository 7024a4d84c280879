"""The polynomial inside gelu_erf_f32 (wechat-tfcc_amd/csrc/common.hpp): the committed coefficients against
float64 erfc on a grid, the whole function emulated in float32 against the exact GELU, and - where scipy is
importable - against what tests/golden/fit_gelu_erfc.py derives anew.  The reference calls the C library's erff
(tfcc/mkl/kernel/tfcc_mklactivationkernel.hpp:213-220); the kernels deviate from its last bits and are held to a
tolerance instead, which this test pins on the CPU."""
import math
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def committed_coefficients():
    src = open(os.path.join(ROOT, "wechat-tfcc_amd", "csrc", "common.hpp")).read()
    body = src[src.index("__device__ static inline float gelu_erf_f32(float v) {"):]
    body = body[:body.index("float e = __builtin_amdgcn_exp2f")]
    lead = re.search(r"float p = ([-+0-9.e]+)f;", body).group(1)
    rest = re.findall(r"p = fmaf\(p, t, ([-+0-9.e]+)f\);", body)
    assert len(rest) == 8
    highest_first = [float(lead)] + [float(x) for x in rest]
    return np.asarray(highest_first[::-1], np.float32)  # lowest power first


def test_committed_coefficients_fit_erfc():
    c = committed_coefficients().astype(np.float64)
    t = np.linspace(0.0, 5.0, 200001)
    approx = np.exp2(t * np.polyval(c[::-1], t))
    exact = np.asarray([math.erfc(x) for x in t])
    assert np.abs(approx - exact).max() <= 6e-9


def test_gelu_in_float32_against_the_exact_function():
    c = committed_coefficients()
    v = np.concatenate([np.linspace(-12, 12, 400001), np.asarray([0.0, -0.0, 1e-30, -1e-30, 7.0711, -7.0711, 30.0, -30.0])]).astype(np.float32)
    f = np.float32
    q = v * f(0.70710678118654752)
    t = np.abs(q)
    p = np.full_like(t, c[8])
    for k in range(7, -1, -1):
        p = (p.astype(np.float64) * t + c[k]).astype(np.float32)  # fmaf: one rounding
    e = np.exp2(np.where(t > 5, f(0), p * t).astype(np.float64)).astype(np.float32)
    e = np.where(t > 5, f(0), e)
    w = np.where(q < 0, e, f(2) - e)
    got = ((v * f(0.5)) * w).astype(np.float64)
    exact = np.asarray([0.5 * x * math.erfc(-x / math.sqrt(2.0)) for x in v.astype(np.float64)])
    assert (np.abs(got - exact) / (1e-7 + 1e-6 * np.abs(exact))).max() <= 0.5


def test_fit_script_reproduces_the_committed_coefficients():
    pytest.importorskip("scipy")
    import importlib.util
    spec = importlib.util.spec_from_file_location("fit_gelu_erfc", os.path.join(ROOT, "tests", "golden", "fit_gelu_erfc.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    c32, worst = mod.fit()
    assert worst <= 6e-9
    # the fit is deterministic up to the linear algebra library's rounding: coefficients agree to float precision
    # where they matter (an error dP in P changes erfc by erfc(t) ln 2 t dP)
    want = committed_coefficients()
    t = np.linspace(0, 5, 20001)
    diff = np.abs(np.polyval(c32.astype(np.float64)[::-1], t) - np.polyval(want.astype(np.float64)[::-1], t))
    exact = np.asarray([math.erfc(x) for x in t])
    assert (diff * exact * math.log(2) * t).max() <= 2e-9
