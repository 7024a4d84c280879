"""A seeded sweep of quantized products across every route of the launch code (256 x 256, 128 x 128 and 64 x 128
tiles of the direct-to-LDS kernels, the register-staged kernel for ragged K or N, batched operands, at most eight
rows) with float ranges drawn like the reference's generator draws them
(tfcc/test/python/testcase/quantization/mklquantizationmatmul.py:35-43) and with power-of-two output scales: the
int32 accumulators and the fused uint8 output against the oracle, bit for bit."""
import numpy as np
import pytest

import oracle_lib as O
from golden.make_golden import gen_ranges

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(2468)
    out = []
    for t in range(36):
        kind = t % 6
        sa = sb = None
        if kind == 0 and t < 24:   # at least 192 tiles of 256 x 256, K a multiple of 256
            m, n, k = int(rng.integers(3000, 4200)), 16 * int(rng.integers(250, 270)), 256 * int(rng.integers(1, 3))
        elif kind == 0:            # the same with a K that is not
            m, n, k = 256 * 12, 256 * 16, 16 * int(rng.integers(5, 30))
        elif kind == 1:            # aligned mid-size: 128 x 128 and 64 x 128 tiles
            m, n, k = int(rng.integers(64, 2100)), 16 * int(rng.integers(4, 130)), 16 * int(rng.integers(1, 70))
        elif kind == 2:            # ragged: the register-staged kernel
            m, n, k = int(rng.integers(1, 400)), int(rng.integers(1, 600)), int(rng.integers(1, 900))
        elif kind == 3:            # batched A against one B, and batch against batch
            bt, m, n, k = int(rng.integers(2, 5)), int(rng.integers(1, 200)), int(rng.integers(1, 300)), int(rng.integers(1, 300))
            sa, sb = (bt, m, k), ((k, n) if t % 12 == 3 else (bt, k, n))
        elif kind == 4:            # at most eight rows
            m, n, k = int(rng.integers(1, 9)), 16 * int(rng.integers(8, 700)), 16 * int(rng.integers(8, 600))
        else:                      # long K
            m, n, k = int(rng.integers(16, 300)), 16 * int(rng.integers(2, 40)), 16 * int(rng.integers(200, 800))
        if sa is None:
            sa, sb = (m, k), (k, n)
        out.append((t, sa, sb))
    return out


@pytest.mark.parametrize("seed,shape_a,shape_b", _cases())
def test_qgemm_seeded_sweep(pkg, T, seed, shape_a, shape_b):
    print("qgemm sweep", seed, shape_a, shape_b, flush=True)
    rng = np.random.default_rng(9000 + seed)
    a = rng.integers(0, 256, shape_a, dtype=np.uint8)
    b = rng.integers(-128, 128, shape_b, dtype=np.int8)
    k = shape_a[-1]
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    ranges = gen_ranges(seed) if seed % 3 else (-128.0, 127.0, -128.0, 127.0)
    oa, ob = O.qmatmul_offsets(*ranges)
    want_c = O.qgemm(a, b, oa, ob, rs, cs)
    mn_c, mx_c = O.qmatmul_range(*ranges)
    # output range from the span of the dequantized accumulators: any scale with both ends cut off a little, or a
    # power-of-two scale (the benchmark's own range, K * 64 accumulator units per level, when the inputs have its ranges)
    real = O.dequantize(want_c, mn_c, mx_c).astype(np.float64)
    lo, hi = float(real.min()), float(real.max())
    span = max(hi - lo, 1e-3)
    if seed % 2:
        mn_o, mx_o = float(np.float32(lo + 0.04 * span)), float(np.float32(hi - 0.03 * span))
    elif seed % 3 == 0:
        mn_o, mx_o = -128.0 * k * 64.0, 127.0 * k * 64.0
    else:
        level = 2.0 ** int(np.ceil(np.log2(span / 255.0)))
        mn_o = level * np.floor(lo / level)
        mn_o, mx_o = float(np.float32(mn_o)), float(np.float32(mn_o + 255.0 * level))
    want_q = O.requantize_s32_u8(want_c, mn_c, mx_c, mn_o, mx_o)
    r = [T.f1(v) for v in ranges]
    c, got_mn, got_mx = pkg.quantization_matmul(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2], r[3])
    assert np.array_equal(T.n(c), want_c)
    assert (float(T.n(got_mn)[0]), float(T.n(got_mx)[0])) == (mn_c, mx_c)
    for want_acc in (True, False):
        q, c2, _, _ = pkg.quantization_matmul_requantize(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2], r[3],
                                                         T.f1(mn_o), T.f1(mx_o), want_acc=want_acc)
        assert np.array_equal(T.n(q), want_q), want_acc
        assert c2 is None or np.array_equal(T.n(c2), want_c)
    q3, _, _, _ = pkg.quantization_matmul_requantize(T.t(a), T.t(rs), r[0], r[1], T.t(b), T.t(cs), r[2], r[3],
                                                     T.f1(mn_o), T.f1(mx_o), want_acc=False, colsum_exact=True)
    assert np.array_equal(T.n(q3), want_q)
