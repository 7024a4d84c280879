"""layer_norm(a @ b + bias + residual) in one launch (tfcc_rocm_sgemm_layer_norm) against the product and the layer
norm as separate launches (bit for bit) and against a float64 model (BASELINE's fp32 tolerance)."""
import numpy as np
import pytest

from conftest import rel_fro

pytestmark = pytest.mark.gpu

FP32_TOL = 1e-5  # relative Frobenius error of fp32 results against float64, as for the products themselves


def layer_norm64(x, gamma, beta, eps):
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    return (x - mean) / np.sqrt(var + eps) * gamma + beta


# the two residual products of a BERT-base layer at batch 8 x 128, a ragged row count, a row of 960 columns (lanes
# with three and with four values of a row), a narrow one, and one without bias and residual
@pytest.mark.parametrize("m,n,k,with_bias,with_residual", [
    (1024, 768, 768, True, True), (1024, 768, 3072, True, True), (1000, 768, 3072, True, True),
    (800, 960, 4096, True, True), (8192, 96, 2048, True, True), (1024, 768, 768, False, False)])
def test_product_and_layer_norm_in_one_launch(pkg, T, m, n, k, with_bias, with_residual):
    import torch
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.05, (k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, n).astype(np.float32) if with_bias else None
    res = rng.normal(0, 1, (m, n)).astype(np.float32) if with_residual else None
    gamma = rng.normal(1, 0.1, n).astype(np.float32)
    beta = rng.normal(0, 0.1, n).astype(np.float32)
    eps = 1e-5
    ta, tb, tg, tbeta = T.t(a), T.t(b), T.t(gamma), T.t(beta)
    tbias = None if bias is None else T.t(bias)
    tres = None if res is None else T.t(res)
    assert pkg.sgemm_layer_norm_supported(ta, tb)
    counters = torch.zeros(int(pkg.lib().tfcc_rocm_sgemm_layer_norm_counters(m)), dtype=torch.int32, device=ta.device)
    out, sums = pkg.sgemm_layer_norm(ta, tb, tbias, tres, tg, tbeta, eps, counters=counters)
    # the separate launches
    sep_sums = torch.empty((m, n), dtype=torch.float32, device=ta.device)
    pkg.check(pkg.lib().tfcc_rocm_sgemm_fused(None, ta.data_ptr(), 0, tb.data_ptr(), 0,
                                              None if tbias is None else tbias.data_ptr(),
                                              None if tres is None else tres.data_ptr(), 0, sep_sums.data_ptr(), 0,
                                              m, n, k, 1, 0))
    sep = pkg.layer_norm(sep_sums, tg, tbeta, eps)
    assert np.array_equal(T.n(sums), T.n(sep_sums))
    assert np.array_equal(T.n(out), T.n(sep))
    assert int(counters.abs().sum().item()) == 0  # left as found
    # float64
    x = a.astype(np.float64) @ b.astype(np.float64)
    if bias is not None:
        x = x + bias
    if res is not None:
        x = x + res
    want = layer_norm64(x, gamma.astype(np.float64), beta.astype(np.float64), eps)
    assert rel_fro(T.n(out), want) <= FP32_TOL
    # again on the same counters and a result buffer full of something else: the same bits
    out2, _ = pkg.sgemm_layer_norm(ta, tb, tbias, tres, tg, tbeta, eps, counters=counters)
    assert np.array_equal(T.n(out2), T.n(out))
    assert int(counters.abs().sum().item()) == 0


def test_shapes_without_a_one_launch_form_are_refused(pkg, T):
    rng = np.random.default_rng(5)
    # 1024 x 3072 x 768 runs on 64 x 64 tiles with one K group; a row of 2048 columns is too long; K not a multiple of 32
    for m, n, k in ((1024, 3072, 768), (64, 2048, 4096), (1024, 768, 770)):
        a = T.t(rng.normal(0, 1, (m, k)).astype(np.float32))
        b = T.t(rng.normal(0, 1, (k, n)).astype(np.float32))
        g = T.t(np.ones(n, np.float32))
        assert not pkg.sgemm_layer_norm_supported(a, b)
        with pytest.raises(pkg.TfccRocmError, match="no one-launch form"):
            pkg.sgemm_layer_norm(a, b, None, None, g, g, 1e-5)
