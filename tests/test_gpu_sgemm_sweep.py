"""A seeded sweep of fp32 product shapes across every route of the launch code: the fused entry point against float64,
the product alone against the same product with B handed over transposed (the register-staged kernel, summed with the
same K groups: the same bits), and strided operands, two-level batches and a shared B through the general entry point
(padding of C must stay untouched)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5


def _shapes():
    rng = np.random.default_rng(12345)
    out = []
    for t in range(40):
        kind = t % 5
        if kind == 0:    # around the 128-row workgroups
            m, n, k = int(rng.integers(600, 3200)), int(rng.integers(700, 3300)), 32 * int(rng.integers(16, 48))
        elif kind == 1:  # around the K groups
            m, n, k = int(rng.integers(200, 1400)), int(rng.integers(90, 1000)), 32 * int(rng.integers(16, 130))
        elif kind == 2:  # small and ragged, any k
            m, n, k = int(rng.integers(1, 300)), int(rng.integers(1, 400)), int(rng.integers(1, 700))
        elif kind == 3:  # batched
            m, n, k = int(rng.integers(16, 600)), 4 * int(rng.integers(8, 400)), 32 * int(rng.integers(1, 24))
        else:            # aligned mid-size
            m, n, k = 32 * int(rng.integers(4, 70)), 32 * int(rng.integers(4, 100)), 32 * int(rng.integers(2, 64))
        batch = int(rng.integers(2, 6)) if kind == 3 else 1
        out.append((m, n, k, batch, bool(rng.integers(0, 2)), bool(rng.integers(0, 2)), int(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("m,n,k,batch,bias,residual,act", _shapes())
def test_fused_sgemm_over_random_shapes(pkg, dev, m, n, k, batch, bias, residual, act):
    import torch
    print("sgemm sweep", m, n, k, batch, bias, residual, act, flush=True)
    gen = torch.Generator(device=dev).manual_seed(m * 7 + n * 3 + k + batch)
    a = torch.randn(batch, m, k, device=dev, generator=gen)
    b = torch.randn(batch, k, n, device=dev, generator=gen)
    bi = torch.randn(n, device=dev, generator=gen) if bias else None
    r = torch.randn(batch, m, n, device=dev, generator=gen) if residual else None
    out = torch.empty(batch, m, n, device=dev)
    pkg.check(pkg.lib().tfcc_rocm_sgemm_fused(None, a.data_ptr(), m * k, b.data_ptr(), k * n,
                                              bi.data_ptr() if bias else None, r.data_ptr() if residual else None,
                                              m * n, out.data_ptr(), m * n, m, n, k, batch, act))
    ref = a.double() @ b.double()
    if bias:
        ref = ref + bi.double()
    if residual:
        ref = ref + r.double()
    if act:
        ref = 0.5 * ref * (1 + torch.erf(ref / 2 ** 0.5))
    assert ((out.double() - ref).norm() / ref.norm()).item() <= FP32_TOL
    if not residual and not act:
        c = torch.empty(batch, m, n, device=dev)
        bt = b.transpose(1, 2).contiguous()
        pkg.sgemm_general(a, bt, c, m, n, k, k, k, n, trans_b=True, batch_outer=batch,
                          strides=(m * k, n * k, m * n), bias=bi)
        assert torch.equal(c, out)


def _strided_shapes():
    rng = np.random.default_rng(777)
    out = []
    for t in range(24):
        kind = t % 4
        if kind == 0:    # 128-row workgroups, batched
            m, n, k = int(rng.integers(200, 700)), 4 * int(rng.integers(200, 800)), 32 * int(rng.integers(16, 40))
            bo, bi = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        elif kind == 1:  # K groups
            m, n, k = int(rng.integers(30, 600)), 4 * int(rng.integers(8, 300)), 32 * int(rng.integers(16, 100))
            bo, bi = 1, int(rng.integers(1, 3))
        elif kind == 2:  # 128 x 128 tiles
            m, n, k = int(rng.integers(1500, 3000)), 4 * int(rng.integers(500, 900)), 32 * int(rng.integers(1, 12))
            bo, bi = int(rng.integers(1, 3)), 1
        else:            # anything aligned to four
            m, n, k = int(rng.integers(1, 500)), 4 * int(rng.integers(1, 200)), 4 * int(rng.integers(1, 300))
            bo, bi = int(rng.integers(1, 3)), int(rng.integers(1, 3))
        pad = lambda: 4 * int(rng.integers(0, 3)) * int(rng.integers(0, 2))
        out.append((m, n, k, bo, bi, pad(), pad(), pad(), bool(rng.integers(0, 2))))
    return out


@pytest.mark.parametrize("m,n,k,outer,inner,pad_a,pad_b,pad_c,share_b", _strided_shapes())
def test_general_sgemm_with_padded_rows_and_two_level_batches(pkg, dev, m, n, k, outer, inner, pad_a, pad_b, pad_c,
                                                             share_b):
    import torch
    print("sgemm strided sweep", m, n, k, outer, inner, pad_a, pad_b, pad_c, share_b, flush=True)
    lda, ldb, ldc = k + pad_a, n + pad_b, n + pad_c
    gen = torch.Generator(device=dev).manual_seed(m * 5 + n * 3 + k + outer + inner)
    a = torch.randn(outer, inner, m, lda, device=dev, generator=gen)
    b = torch.randn(1 if share_b else outer, 1 if share_b else inner, k, ldb, device=dev, generator=gen)
    c = torch.full((outer, inner, m, ldc), float("nan"), device=dev)
    strides = (inner * m * lda, 0 if share_b else inner * k * ldb, inner * m * ldc)
    inner_strides = (m * lda, 0 if share_b else k * ldb, m * ldc)
    pkg.sgemm_general(a, b, c, m, n, k, lda, ldb, ldc, batch_outer=outer, batch_inner=inner, strides=strides,
                      inner_strides=inner_strides)
    ref = a[..., :k].double() @ b[..., :n].double()
    assert ((c[..., :n].double() - ref).norm() / ref.norm()).item() <= FP32_TOL
    if pad_c:
        assert bool(torch.isnan(c[..., n:]).all().item())
