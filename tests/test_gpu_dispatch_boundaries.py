"""Shapes that sit on either side of the thresholds where the launch code switches kernel or tile
configuration (tile counts, K lengths, alignment), each checked like any other shape: int32 results
bit-exact against the oracle's closed form, fp32 within a relative Frobenius error of 1e-5."""
import numpy as np
import pytest

import oracle_lib as O
from conftest import rel_fro

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5


@pytest.mark.parametrize("m,n,k", [
    # 64x64 tiles: 320 / 321 / 640 / 641 of them, K on both sides of 256 and 512
    (64 * 20, 64 * 16, 512), (64 * 20 + 1, 64 * 16, 512), (64 * 20, 64 * 16 + 4, 508), (64 * 20, 64 * 32, 256),
    (64 * 20, 64 * 32 + 4, 256), (64 * 20, 64 * 32, 252), (640, 640, 516),
    # 32x96 tiles preferred or not (1024x768 gives 256 of them; 1024x772 needs a ninth tile column)
    (1024, 768, 512), (1024, 772, 512), (992, 768, 640), (96, 96, 2048),
    # 128x128 tiles from 512 tiles on
    (2048, 4096, 64), (2048, 3968, 64),
    # alignment: k or n not a multiple of 4 takes the scalar-load kernel
    (130, 258, 515), (129, 255, 512),
    # K a multiple of 32: the kernels that copy slabs straight into LDS.  One slab, two (= the ring depth), three;
    # every tile shape (32x32, 32x64, 32x96, 64x64) with 1, 2 and 4 K groups; ragged M and N edges
    (64, 64, 32), (64, 64, 64), (33, 36, 96), (96, 96, 256), (512, 512, 512), (128, 3072, 768), (100, 3000, 288),
    (1000, 760, 736), (1024, 3072, 128), (1021, 3068, 160), (640, 1280, 256), (2048, 2048, 32),
])
def test_sgemm_around_configuration_thresholds(pkg, T, m, n, k):
    print("sgemm", m, n, k, flush=True)
    rng = np.random.default_rng(m * 3 + n * 5 + k)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 1, (k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64) + bias
    got = T.n(pkg.blas_matmul(T.t(a), T.t(b), T.t(bias)))
    assert got.shape == want.shape and rel_fro(got, want) <= FP32_TOL
    # every element, not only the norm: a tile edge that went wrong shows up as a few far-off values
    assert np.abs(got - want).max() <= 1e-4 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("m,n,k", [
    # direct-to-LDS kernel: 256x256 tiles from 192 tiles on, 128x128 below; K not a multiple of the 128-byte slab
    (256 * 12, 256 * 16, 144), (256 * 12 - 1, 256 * 16, 144), (256 * 11, 256 * 16, 272), (512, 384, 4000),
    # 64x128 tiles below 128 tiles of 128x128 (1024 x 768 has 48), 128x128 from there on; ragged edges
    (1024, 768, 3072), (1000, 752, 272), (64, 128, 128), (2048, 1024, 256), (2048 - 128, 1024, 256),
    # K or N not a multiple of 16: the register-staged kernel
    (300, 272, 1000), (300, 260, 1024),
    # skinny kernel from N * K = 2^20 on (M <= 8), general kernel below
    (8, 1024, 1024), (8, 1024, 1008), (9, 1024, 1024), (1, 2048, 512),
])
def test_qgemm_around_configuration_thresholds(pkg, T, m, n, k):
    print("qgemm", m, n, k, flush=True)
    rng = np.random.default_rng(m + n * 7 + k * 11)
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (k, n), dtype=np.int8)
    rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
    for oa, ob in ((-128, 0), (-77, 31)):
        want = (a.astype(np.int64) + oa) @ (b.astype(np.int64) + ob)
        want = (want & 0xffffffff).astype(np.uint32).view(np.int32)
        got = T.n(pkg.quantization_matmul_offsets(T.t(a), T.t(rs), T.t(b), T.t(cs), oa, ob))
        assert np.array_equal(got, want), (oa, ob)
    # fused requantize equals the oracle's requantize of the oracle's accumulators
    want = O.qgemm(a, b, -128, 0, rs, cs)
    mn_c, mx_c = O.qmatmul_range(-128.0, 127.0, -128.0, 127.0)
    lim = float(max(1, k) * 2048)
    q, _, _, _ = pkg.quantization_matmul_requantize(T.t(a), T.t(rs), T.f1(-128.0), T.f1(127.0), T.t(b), T.t(cs),
                                                    T.f1(-128.0), T.f1(127.0), T.f1(-lim), T.f1(lim), want_acc=False)
    assert np.array_equal(T.n(q), O.requantize_s32_u8(want, mn_c, mx_c, -lim, lim))
