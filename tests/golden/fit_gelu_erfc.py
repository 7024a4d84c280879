"""Coefficients of gelu_erf_f32 (wechat-tfcc_amd/csrc/common.hpp): P(t) ~ log2(erfc(t)) / t on [0, 5], degree 8.

erfc(t) = 2^(t P(t)); an error dP in P changes erfc by erfc(t) ln2 t dP, so the fit minimises that weighted
error (Lawson's reweighted least squares on Chebyshev nodes).  Prints the coefficients rounded to float, lowest
power first, and the largest error of erfc they leave.  Needs numpy and scipy; not used at build or run time: tests/test_gelu_fit.py runs fit() and compares what it
returns with the constants committed in the kernel source."""
import numpy as np
from scipy.special import erfc, erfcx

T, DEGREE = 5.0, 8


def target(t):
    out = np.full_like(t, -2 / np.sqrt(np.pi) / np.log(2))
    big = t >= 1e-8
    out[big] = (np.log(erfcx(t[big])) - t[big] ** 2) / np.log(2) / t[big]
    return out


def fit():
    """The coefficients as float32, lowest power first, and the largest error of erfc they leave on [0, 5]."""
    n = 4000
    t = 0.5 * T * (1 - np.cos(np.pi * (np.arange(n) + 0.5) / n))
    y = target(t)
    sensitivity = erfc(t) * np.log(2) * t + 1e-30
    lawson = np.ones(n)
    vander = np.polynomial.chebyshev.chebvander(2 * t / T - 1, DEGREE)
    for _ in range(60):
        w = np.sqrt(lawson) * sensitivity
        c, *_ = np.linalg.lstsq(vander * w[:, None], y * w, rcond=None)
        err = np.abs((vander @ c - y) * sensitivity)
        lawson *= err / err.max() + 1e-3
        lawson /= lawson.sum()
    mono = np.polynomial.chebyshev.Chebyshev(c, domain=[0, T]).convert(kind=np.polynomial.Polynomial).coef
    c32 = mono.astype(np.float32)
    tt = np.linspace(0, T, 200001)
    approx = np.exp2(tt * np.polyval(c32.astype(np.float64)[::-1], tt))
    return c32, float(np.abs(approx - erfc(tt)).max())


def main():
    c32, worst = fit()
    print(", ".join("%.9ef" % x for x in c32))
    print("largest error of erfc with these coefficients: %.2e" % worst)


if __name__ == "__main__":
    main()
