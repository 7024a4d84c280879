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
    # up to eight rows of A: the streaming kernel.  32 columns per wavefront below N = 10240, 64 from there on;
    # K below, at and past one 64-row chunk per wavefront (16 * 64 = 1024), ragged chunk tails, ragged N edges
    (1, 1, 1), (1, 64, 64), (2, 65, 63), (3, 31, 1000), (4, 4096, 1024), (5, 100, 1025), (8, 3072, 768),
    (8, 33, 2049), (7, 8192, 96), (8, 8200, 130), (1, 11008, 512), (6, 8191, 70), (5, 10240, 96), (3, 10239, 130),
    # nine rows: back on the tiled kernels
    (9, 3072, 768),
])
def test_sgemm_with_few_rows(pkg, T, m, n, k):
    import torch
    print("sgemv", m, n, k, flush=True)
    rng = np.random.default_rng(m * 3 + n * 5 + k)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 1, (k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    res = rng.normal(0, 1, (m, n)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    ta, tb, tbias, tres = T.t(a), T.t(b), T.t(bias), T.t(res)
    plain = T.n(pkg.blas_matmul(ta, tb))
    assert rel_fro(plain, want) <= FP32_TOL
    assert np.abs(plain - want).max() <= 1e-4 * max(1.0, np.abs(want).max())
    with_bias = T.n(pkg.blas_matmul(ta, tb, tbias))
    assert np.array_equal(with_bias, plain + bias)  # the bias is added to the finished sum
    # bias + residual + GELU in the same launch: the same bits as the separate kernels give
    out = torch.empty((m, n), dtype=torch.float32, device=ta.device)
    pkg.check(pkg.lib().tfcc_rocm_sgemm_fused(None, ta.data_ptr(), 0, tb.data_ptr(), 0, tbias.data_ptr(),
                                              tres.data_ptr(), 0, out.data_ptr(), 0, m, n, k, 1, 1))
    separate = T.n(pkg.gelu_accurate(pkg.add(pkg.blas_matmul(ta, tb, tbias), tres)))
    assert np.array_equal(T.n(out), separate)
    # three products that share A in one launch: each as on its own
    bs = [tb, T.t(b[:, ::-1].copy()), T.t((b * 0.5).astype(np.float32))]
    grouped = pkg.sgemm_grouped(ta, bs, [tbias, tbias, tbias])
    for g, bb in zip(grouped, bs):
        assert np.array_equal(T.n(g), T.n(pkg.blas_matmul(ta, bb, tbias)))
    # a strided A and C (rows further apart than their length) through the general entry point
    lda, ldc = k + 3, n + 5
    a_wide = np.zeros((m, lda), np.float32)
    a_wide[:, :k] = a
    c_wide = torch.full((m, ldc), 7.0, dtype=torch.float32, device=ta.device)
    pkg.sgemm_general(T.t(a_wide), tb, c_wide, m, n, k, lda, n, ldc)
    got = T.n(c_wide)
    assert np.all(got[:, n:] == 7.0)
    if m <= 8:
        assert np.array_equal(got[:, :n], plain)  # the streaming kernel does not care about alignment
    else:
        assert rel_fro(got[:, :n], want) <= FP32_TOL  # unaligned rows: another tiled kernel, another order of sums


@pytest.mark.parametrize("m,n,k", [
    # few tiles and a long K (four and two K groups in the kernels for B as stored), many tiles (one group),
    # K not a multiple of 32 (the register-staged kernels' own rule), ragged edges, nine rows
    (128, 96, 1024), (96, 96, 2048), (640, 640, 512), (512, 512, 512), (1024, 768, 768), (2048, 4096, 64),
    (100, 52, 36), (300, 260, 1000), (64 * 20, 64 * 16, 508), (9, 3072, 768), (33, 36, 96),
])
def test_sgemm_with_b_given_transposed_equals_transpose_then_multiply(pkg, T, m, n, k):
    """B handed over as [n, k] (trans_b) is summed with the K groups the kernels for [k, n] would use: the same bits
    as transposing B first, whatever the shape."""
    import torch
    print("sgemm trans_b", m, n, k, flush=True)
    rng = np.random.default_rng(m + n * 3 + k * 7)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    bt = rng.normal(0, 1, (n, k)).astype(np.float32)
    ta, tbt = T.t(a), T.t(bt)
    c = torch.empty((m, n), dtype=torch.float32, device=ta.device)
    pkg.sgemm_general(ta, tbt, c, m, n, k, k, k, n, trans_b=True)
    plain = T.n(pkg.blas_matmul(ta, T.t(np.ascontiguousarray(bt.T))))
    assert np.array_equal(T.n(c), plain)
    assert rel_fro(plain, a.astype(np.float64) @ bt.T.astype(np.float64)) <= FP32_TOL


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


@pytest.mark.parametrize("m,n,k", [
    # the products the dispatcher gives 32 x 96 tiles with four K groups: the hand-scheduled kernel with one
    # wavefront per K group.  Whole tiles; a ragged last row band; a ragged last column block; a K whose 32-k slabs do
    # not divide by four (one group gets a slab more than the others); a long narrow product; the shortest K it takes
    (1024, 768, 768), (1000, 768, 3072), (1024, 748, 1024), (1024, 768, 1056), (8192, 96, 2048), (1024, 768, 1024),
])
def test_sgemm_on_32x96_tiles_with_four_k_groups(pkg, T, m, n, k):
    """The same bits as the register-staged kernel (reached through a transposed B, which is summed with the same
    K groups), the fused bias + residual + GELU equal to the separate kernels, float64 within the fp32 tolerance."""
    import torch
    print("sgemm 32x96 / 4 K groups", m, n, k, flush=True)
    rng = np.random.default_rng(m * 5 + n * 3 + k)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 1, (k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    res = rng.normal(0, 1, (m, n)).astype(np.float32)
    ta, tb, tbias, tres = T.t(a), T.t(b), T.t(bias), T.t(res)
    plain = T.n(pkg.blas_matmul(ta, tb))
    assert rel_fro(plain, a.astype(np.float64) @ b.astype(np.float64)) <= FP32_TOL
    c = torch.empty((m, n), dtype=torch.float32, device=ta.device)
    pkg.sgemm_general(ta, T.t(np.ascontiguousarray(b.T)), c, m, n, k, k, k, n, trans_b=True)
    assert np.array_equal(T.n(c), plain)
    out = torch.empty((m, n), dtype=torch.float32, device=ta.device)
    pkg.check(pkg.lib().tfcc_rocm_sgemm_fused(None, ta.data_ptr(), 0, tb.data_ptr(), 0, tbias.data_ptr(),
                                              tres.data_ptr(), 0, out.data_ptr(), 0, m, n, k, 1, 1))
    separate = T.n(pkg.gelu_accurate(pkg.add(pkg.blas_matmul(ta, tb, tbias), tres)))
    assert np.array_equal(T.n(out), separate)
    # three products that share A in one launch (more than two tiles per CU: the rings of three 8-k slabs)
    bs = [tb, T.t(b[:, ::-1].copy()), T.t((b * 0.5).astype(np.float32))]
    grouped = pkg.sgemm_grouped(ta, bs, [tbias, tbias, tbias])
    for g, bb in zip(grouped, bs):
        assert np.array_equal(T.n(g), T.n(pkg.blas_matmul(ta, bb, tbias)))


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k,batch", [
    # products summed in one pass over K whose 128 x 96 tiles fill the CUs: four hand-scheduled wavefronts of 32 x 96 on
    # a shared ring.  Whole tiles; ragged last row band and column block; 192 tiles (three quarters of the CUs); the
    # shortest K it takes; an odd number of 32-k slabs (the unrolled loop leaves one over); two batch entries with
    # their own operands (the kernel variant that reads the batch strides before its first copies)
    (1024, 3072, 768, 1), (1000, 3000, 768, 1), (1536, 1536, 1536, 1), (1024, 3072, 512, 1), (1024, 3072, 544, 1),
    (512, 3072, 768, 2),
])
def test_sgemm_on_128x96_workgroups(pkg, T, m, n, k, batch):
    """The same bits as the register-staged kernel (reached through a transposed B: also one pass over K), the fused
    bias + residual + GELU equal to the separate kernels, float64 within the fp32 tolerance."""
    import torch
    print("sgemm 128x96 workgroups", m, n, k, batch, flush=True)
    rng = np.random.default_rng(m * 7 + n * 3 + k + batch)
    a = rng.normal(0, 1, (batch, m, k)).astype(np.float32)
    b = rng.normal(0, 1, (batch, k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    res = rng.normal(0, 1, (batch, m, n)).astype(np.float32)
    ta, tb, tbias, tres = T.t(a), T.t(b), T.t(bias), T.t(res)
    plain = T.n(pkg.blas_matmul(ta, tb))
    assert rel_fro(plain, a.astype(np.float64) @ b.astype(np.float64)) <= FP32_TOL
    c = torch.empty((batch, m, n), dtype=torch.float32, device=ta.device)
    bt = T.t(np.ascontiguousarray(np.swapaxes(b, 1, 2)))
    pkg.sgemm_general(ta, bt, c, m, n, k, k, k, n, trans_b=True, batch_outer=batch, strides=(m * k, n * k, m * n))
    assert np.array_equal(T.n(c), plain)
    out = torch.empty((batch, m, n), dtype=torch.float32, device=ta.device)
    pkg.check(pkg.lib().tfcc_rocm_sgemm_fused(None, ta.data_ptr(), m * k, tb.data_ptr(), k * n, tbias.data_ptr(),
                                              tres.data_ptr(), m * n, out.data_ptr(), m * n, m, n, k, batch, 1))
    separate = T.n(pkg.gelu_accurate(pkg.add(pkg.blas_matmul(ta, tb, tbias), tres)))
    assert np.array_equal(T.n(out), separate)


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [
    # the same hand-scheduled kernel with other numbers of 32-column blocks per wavefront: 32 x 64 tiles and four K
    # groups (the first BASELINE config; ragged), 32 x 32 tiles and four K groups (whole and ragged), 128 x 128 tiles
    # for products of 512 tiles and more (whole; ragged rows and columns; a single 32-k slab)
    (128, 3072, 768), (100, 3000, 800), (512, 512, 512), (500, 500, 544), (2048, 4096, 256), (2050, 4100, 320),
    (4096, 2048, 32),
    # two K groups: two pairs of wavefronts on 64 x 64 tiles (whole; ragged, an odd number of 32-k slabs), two
    # wavefronts on 32 x 32 tiles
    (1024, 1024, 1024), (1000, 1000, 992), (400, 400, 256), (1111, 996, 320),
    # 128 x 128 workgroups below 512 tiles, where they fill the CUs and 128 x 96 tiles do not
    (2048, 2048, 512), (1920, 2040, 544),
    # 64 x 64 tiles with four K groups: four pairs of wavefronts
    (960, 1024, 2048), (1270, 636, 544),
])
def test_sgemm_wavefront_kernel_with_one_two_and_four_column_blocks(pkg, T, m, n, k):
    """The same bits as the register-staged kernel (reached through a transposed B, summed with the same K groups), the
    fused bias + residual + GELU equal to the separate kernels, float64 within the fp32 tolerance."""
    import torch
    print("sgemm wavefront kernel, other block counts", m, n, k, flush=True)
    rng = np.random.default_rng(m * 11 + n * 3 + k)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 1, (k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    res = rng.normal(0, 1, (m, n)).astype(np.float32)
    ta, tb, tbias, tres = T.t(a), T.t(b), T.t(bias), T.t(res)
    plain = T.n(pkg.blas_matmul(ta, tb))
    assert rel_fro(plain, a.astype(np.float64) @ b.astype(np.float64)) <= FP32_TOL
    c = torch.empty((m, n), dtype=torch.float32, device=ta.device)
    pkg.sgemm_general(ta, T.t(np.ascontiguousarray(b.T)), c, m, n, k, k, k, n, trans_b=True)
    assert np.array_equal(T.n(c), plain)
    out = torch.empty((m, n), dtype=torch.float32, device=ta.device)
    pkg.check(pkg.lib().tfcc_rocm_sgemm_fused(None, ta.data_ptr(), 0, tb.data_ptr(), 0, tbias.data_ptr(),
                                              tres.data_ptr(), 0, out.data_ptr(), 0, m, n, k, 1, 1))
    separate = T.n(pkg.gelu_accurate(pkg.add(pkg.blas_matmul(ta, tb, tbias), tres)))
    assert np.array_equal(T.n(out), separate)


@pytest.mark.gpu
@pytest.mark.parametrize("batch,m,n,k", [
    # many small products: 128 x 128 tiles only where they would be mostly result (512 of them and three quarters full)
    (768, 64, 64, 64), (512, 64, 128, 64), (600, 100, 100, 96), (512, 112, 112, 32), (520, 128, 128, 64), (130, 250, 250, 64),
])
def test_batched_small_products_pick_tiles_that_they_fill(pkg, T, batch, m, n, k):
    print("batched sgemm", batch, m, n, k, flush=True)
    rng = np.random.default_rng(batch + m * 3 + n * 5 + k)
    a = rng.normal(0, 1, (batch, m, k)).astype(np.float32)
    b = rng.normal(0, 1, (batch, k, n)).astype(np.float32)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64))
    got = T.n(pkg.blas_matmul(T.t(a), T.t(b)))
    assert got.shape == want.shape and rel_fro(got, want) <= FP32_TOL
    assert np.abs(got - want).max() <= 1e-4 * max(1.0, np.abs(want).max())
    # the same bits as each product on its own: with K this short every kernel sums an element in one group over
    # ascending k, whatever its tiles
    for i in (0, batch // 2, batch - 1):
        alone = T.n(pkg.blas_matmul(T.t(a[i]), T.t(b[i])))
        assert np.array_equal(alone, got[i])
