"""softmax(q k^T / divisor) v in one launch against (a) the three separate kernels, bit for bit, and
(b) a float64 restatement of the node sequence of tfcc_runtime/operations/math/matmul.cpp:27-41,
softmax.cpp and tfcc/core/operations/tfcc_operator.cpp:78-95 within 1e-5 relative Frobenius error."""
import numpy as np
import pytest

from conftest import rel_fro

pytestmark = pytest.mark.gpu


@pytest.fixture
def gpu(T):
    return T


def reference64(q, k, v, divisor):
    s = np.einsum("bhsd,bhtd->bhst", q.astype(np.float64), k.astype(np.float64))
    if divisor is not None:
        s = s / divisor
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    p = e / e.sum(axis=-1, keepdims=True)
    return np.einsum("bhst,bhtd->bhsd", p, v.astype(np.float64))


def separate_kernels(pkg, torch, q, k, v, B, H, S, T, D, divisor, layout, mask=None):
    """The same result from two products and one softmax, each in a launch of its own."""
    dev = q.device
    scores = torch.empty((B, H, S, T), dtype=torch.float32, device=dev)
    if layout == "bshd":
        sq, iq, ldq = (S * H * D, H * D), D, H * D
        sk, ldk = T * H * D, H * D
    else:
        sq, iq, ldq = (H * S * D,), S * D, D
        sk, ldk = H * T * D, D
    ik = D if layout == "bshd" else T * D
    pkg.sgemm_general(q, k, scores, S, T, D, ldq, ldk, T, trans_b=True, batch_outer=B, batch_inner=H,
                      strides=(sq[0], sk, H * S * T), inner_strides=(iq, ik, S * T))
    probs = torch.empty_like(scores)
    if mask is not None:
        # Div, Add and Softmax as the nodes of a graph run them: one kernel each
        if divisor is not None:
            scores = pkg.transform2(scores, divisor, 0.0)
        scores = pkg.math_binary("add", scores, mask)
        pkg.check(pkg.lib().tfcc_rocm_softmax_f32(pkg._stream(), scores.data_ptr(), B * H * S, T, probs.data_ptr()))
    elif divisor is None:
        pkg.check(pkg.lib().tfcc_rocm_softmax_f32(pkg._stream(), scores.data_ptr(), B * H * S, T, probs.data_ptr()))
    else:
        pkg.check(pkg.lib().tfcc_rocm_softmax_div_f32(pkg._stream(), scores.data_ptr(), B * H * S, T, divisor,
                                                      probs.data_ptr()))
    out = torch.empty((B, S, H, D) if layout == "bshd" else (B, H, S, D), dtype=torch.float32, device=dev)
    if layout == "bshd":
        so, io, ldo = S * H * D, D, H * D
    else:
        so, io, ldo = H * S * D, S * D, D
    pkg.sgemm_general(probs, v, out, S, D, T, T, ldk, ldo, batch_outer=B, batch_inner=H,
                      strides=(H * S * T, sk, so), inner_strides=(S * T, ik, io))
    return out


CASES = [
    # B, H, S, T, D, divisor, layout
    (2, 12, 128, 128, 64, 8.0, "bshd"),     # the encoder layer's attention core
    (1, 3, 100, 77, 36, 6.0, "bshd"),       # ragged everywhere, head width not a multiple of 8
    (2, 2, 200, 128, 64, None, "bhsd"),     # several row blocks, no divisor, dense per-head matrices
    (1, 2, 1, 1, 4, 2.0, "bhsd"),           # the smallest: one query, one key, two heads
    (1, 1, 9, 3, 8, 2.0, "bhsd"),           # a single head of more than eight rows
    (3, 5, 64, 5, 4, 0.5, "bshd"),
    (1, 4, 65, 64, 32, 5.656854, "bhsd"),   # one row past a block; only the first column half is live
    (1, 2, 31, 97, 60, 7.75, "bshd"),
    # more blocks of 64 query rows than the GPU has CUs: blocks of 32 rows, three workgroups per CU
    (16, 12, 128, 128, 64, 8.0, "bshd"),    # the attention shape of the benchmark
    (6, 12, 200, 100, 64, 8.0, "bshd"),     # a ragged last block of 8 rows, ragged keys
    (5, 13, 261, 77, 36, None, "bhsd"),     # a last block of 5 rows, head width not a multiple of 8
]


@pytest.mark.parametrize("B,H,S,Tk,D,divisor,layout", CASES)
def test_attention_equals_separate_kernels(pkg, gpu, B, H, S, Tk, D, divisor, layout):
    import torch
    rng = np.random.default_rng(B * 1000 + S * 7 + Tk * 3 + D)
    if layout == "bshd":
        shape_q, shape_kv = (B, S, H, D), (B, Tk, H, D)
        to_bhxd = lambda x: x.transpose(0, 2, 1, 3)
    else:
        shape_q, shape_kv = (B, H, S, D), (B, H, Tk, D)
        to_bhxd = lambda x: x
    q = rng.standard_normal(shape_q).astype(np.float32)
    k = rng.standard_normal(shape_kv).astype(np.float32)
    v = rng.standard_normal(shape_kv).astype(np.float32)
    tq, tk, tv = gpu.t(q), gpu.t(k), gpu.t(v)
    out = torch.full(shape_q, float("nan"), dtype=torch.float32, device=tq.device)
    if layout == "bshd":
        ld = (H * D,) * 4
        strides = (S * H * D, Tk * H * D, Tk * H * D, S * H * D)
        inner = (D, D, D, D)
    else:
        ld = (D,) * 4
        strides = (H * S * D, H * Tk * D, H * Tk * D, H * S * D)
        inner = (S * D, Tk * D, Tk * D, S * D)
    desc = pkg.attention_desc(tq, tk, tv, out, S, Tk, D, ld, batch_outer=B, batch_inner=H, strides=strides,
                              inner_strides=inner, divisor=divisor)
    assert pkg.attention_supported(desc)
    pkg.attention(desc)
    got = gpu.n(out)
    assert np.isfinite(got).all()
    want = gpu.n(separate_kernels(pkg, torch, tq, tk, tv, B, H, S, Tk, D, divisor, layout))
    assert np.array_equal(got, want), "fused and separate kernels differ by %g" % np.abs(got - want).max()
    ref = reference64(to_bhxd(q), to_bhxd(k), to_bhxd(v), divisor)
    assert rel_fro(to_bhxd(got), ref) <= 1e-5


@pytest.mark.parametrize("B,H,S,Tk,D,divisor,per_head", [
    (2, 12, 128, 128, 64, 8.0, False),   # the encoder layer's attention core with a [B, 1, 1, T] mask
    (3, 2, 70, 100, 36, 6.0, False), (2, 3, 33, 65, 16, None, False), (2, 4, 40, 24, 32, 5.0, True),
    (1, 2, 5, 7, 8, 3.0, False),
    (9, 8, 250, 128, 64, 8.0, False), (4, 17, 250, 90, 40, 6.5, True),   # blocks of 32 query rows
])
def test_attention_with_mask_equals_separate_kernels(pkg, gpu, B, H, S, Tk, D, divisor, per_head):
    """A mask [B, 1, 1, T] (or [B, H, 1, T]) added between the division and the softmax, as BERT graphs do:
    large negative entries for padded keys, whose probabilities must come out as exact zeros."""
    import torch
    rng = np.random.default_rng(B * 100 + S + Tk)
    q = rng.standard_normal((B, S, H, D)).astype(np.float32)
    k = rng.standard_normal((B, Tk, H, D)).astype(np.float32)
    v = rng.standard_normal((B, Tk, H, D)).astype(np.float32)
    mask = np.where(rng.random((B, H if per_head else 1, 1, Tk)) < 0.3, -10000.0, 0.0).astype(np.float32)
    mask[..., 0] = 0.0  # at least one live key per row
    mask += rng.normal(0, 0.1, mask.shape).astype(np.float32)
    tq, tk, tv, tm = gpu.t(q), gpu.t(k), gpu.t(v), gpu.t(mask)
    out = torch.full((B, S, H, D), float("nan"), dtype=torch.float32, device=tq.device)
    desc = pkg.attention_desc(tq, tk, tv, out, S, Tk, D, (H * D,) * 4, batch_outer=B, batch_inner=H,
                              strides=(S * H * D, Tk * H * D, Tk * H * D, S * H * D), inner_strides=(D,) * 4,
                              divisor=divisor, mask=tm,
                              mask_strides=((H if per_head else 1) * Tk, Tk if per_head else 0))
    assert pkg.attention_supported(desc)
    pkg.attention(desc)
    got = gpu.n(out)
    want = gpu.n(separate_kernels(pkg, torch, tq, tk, tv, B, H, S, Tk, D, divisor, "bshd", mask=tm))
    assert np.isfinite(got).all() and np.array_equal(got, want)
    s64 = np.einsum("bshd,bthd->bhst", q.astype(np.float64), k.astype(np.float64))
    s64 = (s64 / divisor if divisor is not None else s64) + mask
    e = np.exp(s64 - s64.max(-1, keepdims=True))
    ref = np.einsum("bhst,bthd->bshd", e / e.sum(-1, keepdims=True), v.astype(np.float64))
    assert rel_fro(got, ref) <= 1e-5


LONG_CASES = [
    # B, H, S, T, D, divisor, layout: key sequences beyond one block of 128
    (1, 12, 384, 384, 64, 8.0, "bshd"),     # the sequence length of the question-answering model the reference documents
    (2, 3, 70, 129, 64, 8.0, "bshd"),       # one key into the second block
    (1, 2, 100, 512, 36, 6.0, "bhsd"),      # four whole blocks, head width not a multiple of 8
    (2, 2, 9, 300, 8, None, "bhsd"),        # ragged last block, no divisor
    (1, 1, 200, 1000, 64, 8.0, "bshd"),     # eight blocks
    (5, 10, 256, 200, 64, 8.0, "bshd"),     # 400 blocks of 32 query rows are more than the GPU has CUs: blocks of 64 (the cases above run as blocks of 32)
]


@pytest.mark.parametrize("B,H,S,Tk,D,divisor,layout", LONG_CASES)
@pytest.mark.parametrize("masked", [False, True])
def test_attention_over_blocks_of_keys(pkg, gpu, B, H, S, Tk, D, divisor, layout, masked):
    """Beyond 128 keys the kernel walks the keys in blocks with a running row maximum and sum: the same real
    function as the separate kernels, summed in another order, so the check is the fp32 contract (relative Frobenius
    error <= 1e-5 against float64), and closeness - not equality - to the separate kernels."""
    import torch
    print("attention over key blocks", B, H, S, Tk, D, divisor, layout, masked, flush=True)
    rng = np.random.default_rng(B * 1000 + S + Tk + D)
    shape_q = (B, S, H, D) if layout == "bshd" else (B, H, S, D)
    shape_k = (B, Tk, H, D) if layout == "bshd" else (B, H, Tk, D)
    q, k, v = (rng.normal(size=sh).astype(np.float32) for sh in (shape_q, shape_k, shape_k))
    # scores large enough that the running maximum moves from block to block
    q *= 3.0
    mask = None
    if masked:
        mask = np.where(rng.random((B, 1, 1, Tk)) < 0.3, -10000.0, 0.0).astype(np.float32)
        mask[..., Tk // 2] = 0.0
    tq, tk, tv = gpu.t(q), gpu.t(k), gpu.t(v)
    out = torch.empty(shape_q, dtype=torch.float32, device=tq.device)
    if layout == "bshd":
        kw = dict(batch_outer=B, batch_inner=H, strides=(S * H * D, Tk * H * D, Tk * H * D, S * H * D), inner_strides=(D,) * 4)
        lds = (H * D,) * 4
    else:
        kw = dict(batch_outer=B, batch_inner=H, strides=(H * S * D, H * Tk * D, H * Tk * D, H * S * D),
                  inner_strides=(S * D, Tk * D, Tk * D, S * D))
        lds = (D,) * 4
    tm = None
    if masked:
        tm = gpu.t(mask)
        kw.update(mask=tm, mask_strides=(Tk, 0))
    desc = pkg.attention_desc(tq, tk, tv, out, S, Tk, D, lds, divisor=divisor, **kw)
    assert pkg.attention_supported(desc)
    pkg.attention(desc)
    got = gpu.n(out).astype(np.float64)
    to_bhsd = (lambda x: x.transpose(0, 2, 1, 3)) if layout == "bshd" else (lambda x: x)
    s = np.einsum("bhsd,bhtd->bhst", to_bhsd(q).astype(np.float64), to_bhsd(k).astype(np.float64))
    if divisor is not None:
        s = s / divisor
    if masked:
        s = s + mask.astype(np.float64)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    ref = np.einsum("bhst,bhtd->bhsd", e / e.sum(-1, keepdims=True), to_bhsd(v).astype(np.float64))
    assert rel_fro(to_bhsd(got), ref) <= 1e-5
    assert np.all(np.isfinite(got))
    if not masked:
        sep = gpu.n(separate_kernels(pkg, torch, tq, tk, tv, B, H, S, Tk, D, divisor, layout)).astype(np.float64)
        assert rel_fro(got, sep) <= 2e-6


def test_attention_limits_are_reported(pkg, gpu):
    import torch
    x = torch.zeros(256 * 256, dtype=torch.float32, device=gpu.t(np.zeros(1, np.float32)).device)
    ok = pkg.attention_desc(x, x, x, x, 16, 128, 64, (64,) * 4)
    assert pkg.attention_supported(ok)
    assert pkg.attention_supported(pkg.attention_desc(x, x, x, x, 16, 129, 64, (64,) * 4))  # blocks of 128 keys
    for s, t, d, ld in [(16, 16, 68, 68), (16, 16, 6, 8), (16, 16, 8, 10)]:
        bad = pkg.attention_desc(x, x, x, x, s, t, d, (ld,) * 4)
        assert not pkg.attention_supported(bad)
        with pytest.raises(pkg.TfccRocmError):
            pkg.attention(bad)
    with pytest.raises(pkg.TfccRocmError):
        pkg.attention(pkg.attention_desc(x, x, x, x, 0, 16, 8, (8,) * 4))
    # a lone head of at most eight query rows: the separate product takes the streaming kernel, whose sums are
    # ordered differently, so the fused kernel declines rather than differ in the last bit
    assert not pkg.attention_supported(pkg.attention_desc(x, x, x, x, 8, 16, 8, (8,) * 4))
    assert pkg.attention_supported(pkg.attention_desc(x, x, x, x, 9, 16, 8, (8,) * 4))
    assert pkg.attention_supported(pkg.attention_desc(x, x, x, x, 8, 16, 8, (8,) * 4, batch_outer=2,
                                                      strides=(1024,) * 4))
