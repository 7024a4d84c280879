"""ctypes binding of libtfcc_rocm.so (the C ABI of include/tfcc_rocm.h) for the Python test and
benchmark harness.  PyTorch is used only as the owner of device memory and of the HIP stream; every
computation goes through the C ABI into the hand-written gfx950 kernels.  There is no fallback: a
missing library or a failing call raises.

The functions mirror the reference's operator interface for this path:
  blas_matmul            tfcc::blas::matmul                   (tfcc/core/operations/tfcc_blas.cpp:26-96)
  quantization_matmul    tfcc::mkl::quantization::matmul      (tfcc/mkl/operations/tfcc_mklquantization.h:39-42)
  reduce_sum             tfcc::mkl::quantization::reduce_sum  (tfcc/mkl/operations/tfcc_mklquantization.h:50-51)
  quantize / requantize / dequantize   tfcc::quantization::*  (tfcc/core/operations/tfcc_quantization.cpp:26-98)
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtfcc_rocm.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

S8, U8, S16, U16, S32, U32, S64, U64, F32, F64 = range(10)


class TfccRocmError(RuntimeError):
    pass


class InvalidArgumentError(ValueError):
    """tfcc::InvalidArgumentError"""


class QGemmDesc(C.Structure):
    _fields_ = [
        ("a", C.c_void_p), ("b", C.c_void_p), ("rowsum_a", C.c_void_p), ("colsum_b", C.c_void_p),
        ("stride_a", C.c_uint64), ("stride_b", C.c_uint64), ("stride_rowsum_a", C.c_uint64),
        ("stride_colsum_b", C.c_uint64), ("stride_c", C.c_uint64),
        ("m", C.c_uint), ("n", C.c_uint), ("k", C.c_uint), ("batch", C.c_uint),
        ("offset_a", C.c_int32), ("offset_b", C.c_int32),
        ("min_a", C.c_void_p), ("max_a", C.c_void_p), ("min_b", C.c_void_p), ("max_b", C.c_void_p),
        ("min_c", C.c_void_p), ("max_c", C.c_void_p),
        ("packed_b", C.c_void_p), ("colsum_b_is_exact", C.c_int),
    ]


class SgemmDesc(C.Structure):
    """tfcc_rocm_sgemm_desc"""
    _fields_ = [
        ("a", C.c_void_p), ("b", C.c_void_p), ("bias", C.c_void_p), ("residual", C.c_void_p), ("c", C.c_void_p),
        ("m", C.c_uint), ("n", C.c_uint), ("k", C.c_uint),
        ("lda", C.c_uint), ("ldb", C.c_uint), ("ldc", C.c_uint),
        ("trans_b", C.c_int),
        ("batch_outer", C.c_uint), ("batch_inner", C.c_uint),
        ("stride_a", C.c_uint64), ("stride_b", C.c_uint64), ("stride_c", C.c_uint64),
        ("inner_stride_a", C.c_uint64), ("inner_stride_b", C.c_uint64), ("inner_stride_c", C.c_uint64),
        ("stride_residual", C.c_uint64),
        ("activation", C.c_int),
    ]


class AttentionDesc(C.Structure):
    """tfcc_rocm_attention_desc"""
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("out", C.c_void_p),
        ("s", C.c_uint), ("t", C.c_uint), ("d", C.c_uint),
        ("ldq", C.c_uint), ("ldk", C.c_uint), ("ldv", C.c_uint), ("ldo", C.c_uint),
        ("batch_outer", C.c_uint), ("batch_inner", C.c_uint),
        ("stride_q", C.c_uint64), ("stride_k", C.c_uint64), ("stride_v", C.c_uint64), ("stride_out", C.c_uint64),
        ("inner_stride_q", C.c_uint64), ("inner_stride_k", C.c_uint64), ("inner_stride_v", C.c_uint64),
        ("inner_stride_out", C.c_uint64),
        ("divisor", C.c_float), ("has_divisor", C.c_int),
        ("mask", C.c_void_p), ("stride_mask", C.c_uint64), ("inner_stride_mask", C.c_uint64),
    ]


# name -> (restype, argtypes): every symbol include/tfcc_rocm.h declares
_VP, _U64, _U, _I, _F, _D, _I64 = C.c_void_p, C.c_uint64, C.c_uint, C.c_int, C.c_float, C.c_double, C.c_int64
SYMBOLS = {
    "tfcc_rocm_last_error_string": (C.c_char_p, []),
    "tfcc_rocm_version": (C.c_char_p, []),
    "tfcc_rocm_device_count": (_I, [C.POINTER(C.c_int)]),
    "tfcc_rocm_set_device": (_I, [_I]),
    "tfcc_rocm_mem_info": (_I, [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "tfcc_rocm_device_name": (_I, [C.c_char_p, C.c_size_t]),
    "tfcc_rocm_malloc": (_I, [C.POINTER(C.c_void_p), C.c_size_t]),
    "tfcc_rocm_free": (_I, [_VP]),
    "tfcc_rocm_stream_create": (_I, [C.POINTER(C.c_void_p)]),
    "tfcc_rocm_stream_destroy": (_I, [_VP]),
    "tfcc_rocm_stream_release": (_I, [_VP]),
    "tfcc_rocm_stream_synchronize": (_I, [_VP]),
    "tfcc_rocm_memcpy_h2d": (_I, [_VP, _VP, _VP, C.c_size_t]),
    "tfcc_rocm_memcpy_d2h": (_I, [_VP, _VP, _VP, C.c_size_t]),
    "tfcc_rocm_memcpy_d2d_async": (_I, [_VP, _VP, _VP, C.c_size_t]),
    "tfcc_rocm_fill_async": (_I, [_VP, _VP, _U64, _I, C.c_size_t]),
    "tfcc_rocm_sgemm_strided_batched": (_I, [_VP, _VP, _U64, _VP, _U64, _VP, _VP, _U64, _U, _U, _U, _U]),
    "tfcc_rocm_gemm_u8s8s32": (_I, [_VP, C.POINTER(QGemmDesc), _VP]),
    "tfcc_rocm_gemm_u8s8s32_requant_u8": (_I, [_VP, C.POINTER(QGemmDesc), _VP, _VP, _D, _D, _D, _I64, _VP, _VP]),
    "tfcc_rocm_gemv_packed_size": (C.c_size_t, [_U, _U]),
    "tfcc_rocm_gemv_pack_b": (_I, [_VP, _VP, _U, _U, _VP]),
    "tfcc_rocm_gemv_u8s8s32_packed": (_I, [_VP, _VP, _VP, _VP, _VP, C.c_int32, C.c_int32, _U, _U, _U, _VP, _F, _VP, _VP]),
    "tfcc_rocm_gemv_u8s8s32": (_I, [_VP, _VP, _VP, _VP, _VP, C.c_int32, C.c_int32, _U, _U, _U, _VP, _F, _VP, _VP]),
    "tfcc_rocm_gemv_u8s8s32_noalloc": (_I, [_VP, _VP, _VP, _VP, _VP, C.c_int32, C.c_int32, _U, _U, _U, _VP, _F, _VP, _VP]),
    "tfcc_rocm_gemv_u8s8s32_flags": (_I, [_VP, _VP, _VP, _VP, _VP, C.c_int32, C.c_int32, _U, _U, _U, _VP, _F, _VP, _VP, _U]),
    "tfcc_rocm_reduce_sum_rows": (_I, [_VP, _VP, _I, _U, _U, _U, _VP]),
    "tfcc_rocm_reduce_sum_cols": (_I, [_VP, _VP, _I, _U, _U, _U, _VP]),
    "tfcc_rocm_requantize": (_I, [_VP, _VP, _I, _VP, _I, _U64, _VP, _VP, _VP, _VP]),
    "tfcc_rocm_dequantize": (_I, [_VP, _VP, _I, _U64, _VP, _VP, _VP]),
    "tfcc_rocm_quantize": (_I, [_VP, _VP, _U64, _VP, _VP, _VP, _I]),
    "tfcc_rocm_quantize_minmax": (_I, [_VP, _VP, _U64, _VP, _I, _VP, _VP]),
    "tfcc_rocm_softmax_f32": (_I, [_VP, _VP, _U64, _U, _VP]),
    "tfcc_rocm_layer_norm_f32": (_I, [_VP, _VP, _VP, _VP, _F, _U64, _U, _VP]),
    "tfcc_rocm_gelu_accurate_f32": (_I, [_VP, _VP, _U64, _VP]),
    "tfcc_rocm_transform_f32": (_I, [_VP, _VP, _U64, _F, _F, _VP]),
    "tfcc_rocm_add_f32": (_I, [_VP, _VP, _VP, _U64, _U64, _VP]),
    "tfcc_rocm_event_create": (_I, [C.POINTER(_VP)]),
    "tfcc_rocm_event_destroy": (_I, [_VP]),
    "tfcc_rocm_event_record": (_I, [_VP, _VP]),
    "tfcc_rocm_event_elapsed_ms": (_I, [_VP, _VP, C.POINTER(C.c_float)]),
    "tfcc_rocm_stream_begin_capture": (_I, [_VP]),
    "tfcc_rocm_stream_end_capture": (_I, [_VP, C.POINTER(_VP)]),
    "tfcc_rocm_graph_launch": (_I, [_VP, _VP]),
    "tfcc_rocm_graph_destroy": (_I, [_VP]),
    "tfcc_rocm_sgemm_fused": (_I, [_VP, _VP, _U64, _VP, _U64, _VP, _VP, _U64, _VP, _U64, _U, _U, _U, _U, _I]),
    "tfcc_rocm_sgemm_general": (_I, [_VP, _VP]),
    "tfcc_rocm_sgemm_grouped": (_I, [_VP, _VP, C.POINTER(_VP), C.POINTER(_VP), C.POINTER(_VP), _U, _U, _U, _U]),
    "tfcc_rocm_unary_f32": (_I, [_VP, _I, _VP, _U64, _VP]),
    "tfcc_rocm_softmax_div_f32": (_I, [_VP, _VP, _U64, _U, _F, _VP]),
    "tfcc_rocm_attention_f32_supported": (_I, [C.POINTER(AttentionDesc)]),
    "tfcc_rocm_attention_f32": (_I, [_VP, C.POINTER(AttentionDesc)]),
    "tfcc_rocm_transform2_f32": (_I, [_VP, _VP, _U64, _F, _F, _VP]),
    "tfcc_rocm_binary_f32": (_I, [_VP, _I, _VP, _VP, _U64, _U64, _VP]),
    "tfcc_rocm_transpose_f32": (_I, [_VP, _VP, C.POINTER(C.c_uint), C.POINTER(C.c_uint), _I, _VP]),
    "tfcc_rocm_binary_broadcast_f32": (_I, [_VP, _I, _VP, _VP, _I, C.POINTER(C.c_uint), C.POINTER(_U64),
                                           C.POINTER(_U64), _VP]),
    "tfcc_rocm_lstm_cell_f32": (_I, [_VP, _U, _U, _VP, _VP, _VP, _VP, _F, _VP, _VP]),
    "tfcc_rocm_reduce_f32": (_I, [_VP, _I, _VP, _U64, _U, _VP]),
    "tfcc_rocm_clip_f32": (_I, [_VP, _VP, _U64, _F, _F, _VP]),
    "tfcc_rocm_leaky_relu_f32": (_I, [_VP, _VP, _U64, _F, _VP]),
    "tfcc_rocm_copy2d": (_I, [_VP, _VP, _U64, _VP, _U64, _U64, _U64]),
    "tfcc_rocm_gather_rows": (_I, [_VP, _VP, _U, _U64, _VP, _I, _U64, _VP]),
    "tfcc_rocm_cast": (_I, [_VP, _VP, _I, _VP, _I, _U64]),
    "tfcc_rocm_where": (_I, [_VP, _VP, _VP, _U64, _VP, _U64, _U, _U64, _VP]),
    "tfcc_rocm_triangle": (_I, [_VP, _VP, _U64, _U64, C.c_int64, _I, _U, _VP]),
    "tfcc_rocm_compare_value": (_I, [_VP, _I, _VP, _I, _U64, _VP, _VP]),
    "tfcc_rocm_compare": (_I, [_VP, _I, _VP, _VP, _I, _I, C.POINTER(C.c_uint), C.POINTER(_U64), C.POINTER(_U64), _VP]),
    "tfcc_rocm_topk_f32": (_I, [_VP, _VP, _U64, _U, _U, _VP, _VP]),
    "tfcc_rocm_argmax_f32": (_I, [_VP, _VP, _U64, _U, _U64, _VP]),
    "tfcc_rocm_lstm_step_f32": (_I, [_VP, _U, _U, _VP, _VP, _VP, _VP, _F, _VP, _VP, _VP]),
    "tfcc_rocm_gru_cell_gates_f32": (_I, [_VP, _U, _U, _U, _VP, _VP, _VP, _VP, _VP]),
    "tfcc_rocm_gru_cell_candidate_f32": (_I, [_VP, _U, _U, _VP, _VP, _VP, _VP, _VP, _VP]),
    "tfcc_rocm_pytorch_gru_cell_f32": (_I, [_VP, _U, _U, _VP, _VP, _VP, _VP, _VP, _VP, _VP]),
}

_lib = None


def lib():
    """The loaded library.  Raises if it has not been built (see csrc/Makefile)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TfccRocmError("%s is missing: build it with `make -C %s`" % (LIB_PATH, CSRC_DIR))
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            f = getattr(handle, name)  # AttributeError if the symbol is not exported
            f.restype = res
            f.argtypes = args
        _lib = handle
    return _lib


def check(status):
    if status != 0:
        raise TfccRocmError("tfcc_rocm error %d: %s" % (status, lib().tfcc_rocm_last_error_string().decode()))


# ---------------------------------------------------------------------------------------------
# torch-tensor convenience layer
# ---------------------------------------------------------------------------------------------

def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _type_code(dtype):
    import torch
    return {torch.int8: S8, torch.uint8: U8, torch.int16: S16, torch.int32: S32, torch.int64: S64, torch.float32: F32,
            torch.float64: F64}[dtype]


def matmul_plan(shape_a, shape_b, shape_bias=None):
    """Validation and stride rules of tfcc::blas::matmul / MKLBlasInterface::matmul
    (tfcc/core/operations/tfcc_blas.cpp:26-96, tfcc/mkl/interfaces/tfcc_mklblasinterface.cpp:127-151)."""
    ra, rb = len(shape_a), len(shape_b)
    if ra < 2 or rb < 2:
        raise InvalidArgumentError("matmul require tensors with two or more dimensions")
    if ra != rb and ra != 2 and rb != 2:
        raise InvalidArgumentError("shape invalid")
    if shape_a[-1] != shape_b[-2]:
        raise InvalidArgumentError("shape invalid")
    if shape_bias is not None and (len(shape_bias) != 1 or shape_bias[0] != shape_b[-1]):
        raise InvalidArgumentError("shape invalid")
    m, n, k = shape_a[-2], shape_b[-1], shape_a[-1]
    lead = tuple(shape_a[:-2]) if ra > rb else tuple(shape_b[:-2])
    grid = None
    if ra == rb and tuple(shape_a[:-2]) != tuple(shape_b[:-2]):
        # beyond the reference (which raises here): a leading dimension of 1 on one side is broadcast
        lead = []
        for ea, eb in zip(shape_a[:-2], shape_b[:-2]):
            if ea != eb and ea != 1 and eb != 1:
                raise InvalidArgumentError("shape invalid")
            lead.append(eb if ea == 1 else ea)
        lead = tuple(lead)
        dims, sa, sb, sc = [], [], [], []
        da, db, dc = m * k, k * n, m * n
        for ea, eb, e in reversed(list(zip(shape_a[:-2], shape_b[:-2], lead))):
            if e > 1:
                dims.insert(0, e); sa.insert(0, 0 if ea == 1 else da); sb.insert(0, 0 if eb == 1 else db); sc.insert(0, dc)
            da, db, dc = da * ea, db * eb, dc * e
        i = 0
        while i + 1 < len(dims):
            if all(s[i] == s[i + 1] * dims[i + 1] for s in (sa, sb, sc)):
                dims[i + 1] *= dims[i]
                for lst in (dims, sa, sb, sc):
                    del lst[i]
                i = max(i - 1, 0)
            else:
                i += 1
        if len(dims) > 2:
            raise NotImplementedError("matmul: broadcast over more than two groups of batch dimensions")
        while len(dims) < 2:
            dims.append(1); sa.append(0); sb.append(0); sc.append(0)
        grid = dict(outer=dims[0], inner=dims[1], strides=(sa[0], sb[0], sc[0]), inner_strides=(sa[1], sb[1], sc[1]))
    batch = 1
    for d in lead:
        batch *= d
    stride_a, stride_b = m * k, n * k
    if ra != rb:
        if ra == 2:
            stride_a = 0
        if rb == 2:
            stride_b = 0
    return dict(m=m, n=n, k=k, batch=batch, shape=lead + (m, n), stride_a=stride_a, stride_b=stride_b,
                stride_c=m * n, grid=grid)


def blas_matmul(a, b, bias=None):
    """tfcc::blas::matmul(a, b[, bias]) on fp32 device tensors."""
    import torch
    for t in (a, b) + (() if bias is None else (bias,)):
        if t.dtype != torch.float32:
            raise NotImplementedError("matmul is implemented for float32 only, like the reference's MKL device")
    p = matmul_plan(tuple(a.shape), tuple(b.shape), None if bias is None else tuple(bias.shape))
    out = torch.empty(p["shape"], dtype=torch.float32, device=a.device)
    if a.numel() == 0 or b.numel() == 0:
        return out  # uninitialised, as the reference returns it
    a, b = a.contiguous(), b.contiguous()
    bias = None if bias is None else bias.contiguous()
    if p["grid"] is not None:
        g = p["grid"]
        return sgemm_general(a, b, out, p["m"], p["n"], p["k"], p["k"], p["n"], p["n"], batch_outer=g["outer"],
                             batch_inner=g["inner"], strides=g["strides"], inner_strides=g["inner_strides"], bias=bias)
    check(lib().tfcc_rocm_sgemm_strided_batched(_stream(), _ptr(a), p["stride_a"], _ptr(b), p["stride_b"],
                                                 _ptr(bias), _ptr(out), p["stride_c"], p["m"], p["n"], p["k"],
                                                 p["batch"]))
    return out


def sgemm_general(a, b, c, m, n, k, lda, ldb, ldc, trans_b=False, batch_outer=1, batch_inner=1,
                  strides=(0, 0, 0), inner_strides=(0, 0, 0), bias=None, activation=0):
    """tfcc_rocm_sgemm_general on torch tensors used as raw buffers (all strides in elements)."""
    d = SgemmDesc()
    d.a, d.b, d.c, d.bias, d.residual = _ptr(a), _ptr(b), _ptr(c), _ptr(bias), None
    d.m, d.n, d.k, d.lda, d.ldb, d.ldc = m, n, k, lda, ldb, ldc
    d.trans_b = 1 if trans_b else 0
    d.batch_outer, d.batch_inner = batch_outer, batch_inner
    d.stride_a, d.stride_b, d.stride_c = strides
    d.inner_stride_a, d.inner_stride_b, d.inner_stride_c = inner_strides
    d.activation = activation
    check(lib().tfcc_rocm_sgemm_general(_stream(), C.byref(d)))
    return c


def attention_desc(q, k, v, out, s, t, d, ld, batch_outer=1, batch_inner=1, strides=(0, 0, 0, 0),
                   inner_strides=(0, 0, 0, 0), divisor=None, mask=None, mask_strides=(0, 0)):
    """A tfcc_rocm_attention_desc over torch tensors used as raw buffers; ld = (ldq, ldk, ldv, ldo)."""
    a = AttentionDesc()
    a.q, a.k, a.v, a.out = _ptr(q), _ptr(k), _ptr(v), _ptr(out)
    a.s, a.t, a.d = s, t, d
    a.ldq, a.ldk, a.ldv, a.ldo = ld
    a.batch_outer, a.batch_inner = batch_outer, batch_inner
    a.stride_q, a.stride_k, a.stride_v, a.stride_out = strides
    a.inner_stride_q, a.inner_stride_k, a.inner_stride_v, a.inner_stride_out = inner_strides
    a.divisor = 1.0 if divisor is None else divisor
    a.has_divisor = 0 if divisor is None else 1
    a.mask = None if mask is None else _ptr(mask)
    a.stride_mask, a.inner_stride_mask = mask_strides
    return a


def attention_supported(desc):
    return bool(lib().tfcc_rocm_attention_f32_supported(C.byref(desc)))


def attention(desc):
    """tfcc_rocm_attention_f32: out = softmax(q k^T [/ divisor]) v per batch entry."""
    check(lib().tfcc_rocm_attention_f32(_stream(), C.byref(desc)))


def sgemm_grouped(a, bs, biases):
    """[a @ b + bias for b, bias in zip(bs, biases)] in one launch (a: [m, k]; every b: [k, n])."""
    import torch
    a = a.contiguous()
    m, k = a.shape
    n = bs[0].shape[1]
    groups = len(bs)
    outs = [torch.empty((m, n), dtype=torch.float32, device=a.device) for _ in bs]
    arr = lambda ts: (_VP * groups)(*[_ptr(t) for t in ts])
    check(lib().tfcc_rocm_sgemm_grouped(_stream(), _ptr(a), arr(bs), arr(biases) if biases is not None else None,
                                        arr(outs), groups, m, n, k))
    return outs


def reduce_sum(a, row):
    """tfcc::mkl::quantization::reduce_sum: int32 sums over the last (row=True) or the
    second-to-last (row=False) dimension."""
    import torch
    if a.numel() == 0 or a.dim() < 2:
        raise InvalidArgumentError("invalid input tensor a")
    a = a.contiguous()
    r, c = a.shape[-2], a.shape[-1]
    batch = a.numel() // (r * c)
    out = torch.empty(tuple(a.shape[:-2]) + ((r,) if row else (c,)), dtype=torch.int32, device=a.device)
    f = lib().tfcc_rocm_reduce_sum_rows if row else lib().tfcc_rocm_reduce_sum_cols
    check(f(_stream(), _ptr(a), _type_code(a.dtype), batch, r, c, _ptr(out)))
    return out


def _qdesc(a, reduce_a, b, reduce_b):
    if a.numel() == 0 or a.dim() < 2:
        raise InvalidArgumentError("invalid input tensor a")
    if reduce_a.numel() == 0:
        raise InvalidArgumentError("invalid tensor reduceSumA")
    if b.numel() == 0 or b.dim() < 2:
        raise InvalidArgumentError("invalid input tensor b")
    if reduce_b.numel() == 0:
        raise InvalidArgumentError("invalid tensor reduceSumB")
    if a.shape[-1] != b.shape[-2]:
        raise InvalidArgumentError("tensor a and b don't match")
    if a.dim() != b.dim() and a.dim() != 2 and b.dim() != 2:
        raise InvalidArgumentError("tensor a and b don't match")
    if a.shape[-2] != reduce_a.shape[-1]:
        raise InvalidArgumentError("tensor a and reduceSumA don't match")
    if b.shape[-1] != reduce_b.shape[-1]:
        raise InvalidArgumentError("tensor b and reduceSumB don't match")
    if a.dim() == b.dim() and tuple(a.shape[:-2]) != tuple(b.shape[:-2]):
        raise InvalidArgumentError("tensor a and b don't match")
    m, k, n = a.shape[-2], a.shape[-1], b.shape[-1]
    shape = tuple(a.shape[:-2] if a.dim() > b.dim() else b.shape[:-2]) + (m, n)
    batch = 1
    for d in shape[:-2]:
        batch *= d
    d = QGemmDesc()
    d.a, d.b, d.rowsum_a, d.colsum_b = _ptr(a), _ptr(b), _ptr(reduce_a), _ptr(reduce_b)
    d.stride_rowsum_a = 0 if reduce_a.dim() == 1 else m
    d.stride_colsum_b = 0 if reduce_b.dim() == 1 else n
    d.stride_a = 0 if a.dim() == 2 else m * k
    d.stride_b = 0 if b.dim() == 2 else k * n
    if b.dim() == 2:  # single B: the batch folds into M (tfcc_mklquantization.cpp:140-145)
        m, d.stride_rowsum_a, d.stride_a, batch = m * batch, d.stride_rowsum_a * batch, d.stride_a * batch, 1
    d.stride_c = m * n
    d.m, d.n, d.k, d.batch = m, n, k, batch
    return d, shape


def _check_scalar(t, name):
    if t.numel() != 1 or t.dim() != 1:
        raise InvalidArgumentError("invalid tensor " + name)


def quantization_matmul(a, reduce_a, min_a, max_a, b, reduce_b, min_b, max_b):
    """tfcc::mkl::quantization::matmul: returns (int32 C, minC, maxC); ranges are 1-element device tensors."""
    import torch
    a, b, reduce_a, reduce_b = a.contiguous(), b.contiguous(), reduce_a.contiguous(), reduce_b.contiguous()
    for t, nm in ((min_a, "minA"), (max_a, "maxA"), (min_b, "minB"), (max_b, "maxB")):
        _check_scalar(t, nm)
    d, shape = _qdesc(a, reduce_a, b, reduce_b)
    c = torch.empty(shape, dtype=torch.int32, device=a.device)
    min_c = torch.empty(1, dtype=torch.float32, device=a.device)
    max_c = torch.empty(1, dtype=torch.float32, device=a.device)
    d.min_a, d.max_a, d.min_b, d.max_b = _ptr(min_a), _ptr(max_a), _ptr(min_b), _ptr(max_b)
    d.min_c, d.max_c = _ptr(min_c), _ptr(max_c)
    check(lib().tfcc_rocm_gemm_u8s8s32(_stream(), C.byref(d), _ptr(c)))
    return c, min_c, max_c


def quantization_matmul_offsets(a, reduce_a, b, reduce_b, offset_a, offset_b):
    """The same product with immediate integer offsets (kernel-level form)."""
    import torch
    a, b, reduce_a, reduce_b = a.contiguous(), b.contiguous(), reduce_a.contiguous(), reduce_b.contiguous()
    d, shape = _qdesc(a, reduce_a, b, reduce_b)
    d.offset_a, d.offset_b = offset_a, offset_b
    c = torch.empty(shape, dtype=torch.int32, device=a.device)
    check(lib().tfcc_rocm_gemm_u8s8s32(_stream(), C.byref(d), _ptr(c)))
    return c


def quantization_matmul_requantize(a, reduce_a, min_a, max_a, b, reduce_b, min_b, max_b, min_out, max_out,
                                   want_acc=False, colsum_exact=False):
    """matmul followed by requantize<uint8_t> in one kernel.  Returns (uint8 Q, int32 C or None, minC, maxC).
    colsum_exact: the caller's promise that reduce_b holds the true column sums of b."""
    import torch
    a, b, reduce_a, reduce_b = a.contiguous(), b.contiguous(), reduce_a.contiguous(), reduce_b.contiguous()
    for t, nm in ((min_a, "minA"), (max_a, "maxA"), (min_b, "minB"), (max_b, "maxB"), (min_out, "minOutput"),
                  (max_out, "maxOutput")):
        _check_scalar(t, nm)
    d, shape = _qdesc(a, reduce_a, b, reduce_b)
    q = torch.empty(shape, dtype=torch.uint8, device=a.device)
    c = torch.empty(shape, dtype=torch.int32, device=a.device) if want_acc else None
    min_c = torch.empty(1, dtype=torch.float32, device=a.device)
    max_c = torch.empty(1, dtype=torch.float32, device=a.device)
    d.min_a, d.max_a, d.min_b, d.max_b = _ptr(min_a), _ptr(max_a), _ptr(min_b), _ptr(max_b)
    d.min_c, d.max_c = _ptr(min_c), _ptr(max_c)
    d.colsum_b_is_exact = 1 if colsum_exact else 0
    check(lib().tfcc_rocm_gemm_u8s8s32_requant_u8(_stream(), C.byref(d), _ptr(c), _ptr(q), 0.0, 0.0, 0.0, 0,
                                                   _ptr(min_out), _ptr(max_out)))
    return q, c, min_c, max_c


GEMV_COLSUM_B_IS_EXACT = 1


def gemv_dequant(a, b, reduce_a, reduce_b, offset_a, offset_b, scale_a, scale_b, want_acc=True, out=None, acc=None,
                 no_alloc=False, colsum_exact=False):
    """Skinny (M <= 8) product with optional fused per-channel dequantize.  Returns (f32 or None, int32 or None).
    no_alloc: through the entry point that allocates nothing (the caller then passes `out` / `acc` too).
    colsum_exact: the caller vouches that reduce_b holds the true column sums of b."""
    import torch
    a, b = a.contiguous(), b.contiguous()
    m, k, n = a.shape[0], a.shape[1], b.shape[1]
    if acc is None and want_acc:
        acc = torch.empty((m, n), dtype=torch.int32, device=a.device)
    if out is None and scale_b is not None:
        out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    if colsum_exact:
        assert not no_alloc
        check(lib().tfcc_rocm_gemv_u8s8s32_flags(_stream(), _ptr(a), _ptr(b), _ptr(reduce_a), _ptr(reduce_b), offset_a,
                                                 offset_b, m, n, k, _ptr(acc), float(scale_a), _ptr(scale_b), _ptr(out),
                                                 GEMV_COLSUM_B_IS_EXACT))
        return out, acc
    fn = lib().tfcc_rocm_gemv_u8s8s32_noalloc if no_alloc else lib().tfcc_rocm_gemv_u8s8s32
    check(fn(_stream(), _ptr(a), _ptr(b), _ptr(reduce_a), _ptr(reduce_b), offset_a, offset_b, m, n, k, _ptr(acc),
             float(scale_a), _ptr(scale_b), _ptr(out)))
    return out, acc


def gemv_pack(b):
    """Packs an int8 [K, N] weight matrix once for gemv_dequant_packed; returns the packed buffer."""
    import torch
    b = b.contiguous()
    k, n = b.shape
    packed = torch.empty(lib().tfcc_rocm_gemv_packed_size(n, k), dtype=torch.uint8, device=b.device)
    check(lib().tfcc_rocm_gemv_pack_b(_stream(), _ptr(b), n, k, _ptr(packed)))
    return packed


def gemv_dequant_packed(a, packed, n, reduce_a, reduce_b, offset_a, offset_b, scale_a, scale_b, want_acc=True):
    """gemv_dequant on weights packed by gemv_pack (n: the column count of the original matrix)."""
    import torch
    a = a.contiguous()
    m, k = a.shape
    acc = torch.empty((m, n), dtype=torch.int32, device=a.device) if want_acc else None
    out = torch.empty((m, n), dtype=torch.float32, device=a.device) if scale_b is not None else None
    check(lib().tfcc_rocm_gemv_u8s8s32_packed(_stream(), _ptr(a), _ptr(packed), _ptr(reduce_a), _ptr(reduce_b), offset_a,
                                               offset_b, m, n, k, _ptr(acc), float(scale_a), _ptr(scale_b), _ptr(out)))
    return out, acc


def requantize(a, min_in, max_in, min_out, max_out, out_dtype):
    """tfcc::quantization::requantize<T>(a, minInput, maxInput, minOutput, maxOutput)"""
    import torch
    if a.numel() == 0:
        raise InvalidArgumentError("invalid tensor")
    for t, nm in ((min_in, "minInput"), (max_in, "maxInput"), (min_out, "minOutput"), (max_out, "maxOutput")):
        if t.numel() != 1 or t.dim() != 1:
            raise InvalidArgumentError("invalid " + nm)
    a = a.contiguous()
    out = torch.empty(a.shape, dtype=out_dtype, device=a.device)
    check(lib().tfcc_rocm_requantize(_stream(), _ptr(a), _type_code(a.dtype), _ptr(out), _type_code(out_dtype),
                                      a.numel(), _ptr(min_in), _ptr(max_in), _ptr(min_out), _ptr(max_out)))
    return out


def dequantize(a, min_v, max_v):
    """tfcc::quantization::dequantize(a, minValue, maxValue)"""
    import torch
    if a.numel() == 0:
        raise InvalidArgumentError("invalid tensor")
    for t, nm in ((min_v, "minValue"), (max_v, "maxValue")):
        if t.numel() != 1 or t.dim() != 1:
            raise InvalidArgumentError("invalid " + nm)
    a = a.contiguous()
    out = torch.empty(a.shape, dtype=torch.float32, device=a.device)
    check(lib().tfcc_rocm_dequantize(_stream(), _ptr(a), _type_code(a.dtype), a.numel(), _ptr(min_v), _ptr(max_v),
                                      _ptr(out)))
    return out


def quantize(a, out_dtype, min_v=None, max_v=None):
    """tfcc::quantization::quantize<T>(a) -> (q, min, max), or quantize<T>(a, min, max) -> q"""
    import torch
    if a.numel() == 0:
        raise InvalidArgumentError("invalid tensor")
    a = a.contiguous()
    out = torch.empty(a.shape, dtype=out_dtype, device=a.device)
    if min_v is None:
        mn = torch.empty(1, dtype=torch.float32, device=a.device)
        mx = torch.empty(1, dtype=torch.float32, device=a.device)
        check(lib().tfcc_rocm_quantize_minmax(_stream(), _ptr(a), a.numel(), _ptr(out), _type_code(out_dtype),
                                               _ptr(mn), _ptr(mx)))
        return out, mn, mx
    for t, nm in ((min_v, "minValue"), (max_v, "maxValue")):
        if t.numel() != 1 or t.dim() != 1:
            raise InvalidArgumentError("invalid " + nm)
    check(lib().tfcc_rocm_quantize(_stream(), _ptr(a), a.numel(), _ptr(min_v), _ptr(max_v), _ptr(out),
                                    _type_code(out_dtype)))
    return out


def softmax(a):
    import torch
    a = a.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_softmax_f32(_stream(), _ptr(a), a.numel() // a.shape[-1], a.shape[-1], _ptr(out)))
    return out


def layer_norm(a, gamma, beta, eps):
    import torch
    a = a.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_layer_norm_f32(_stream(), _ptr(a), _ptr(gamma.contiguous()), _ptr(beta.contiguous()),
                                          eps, a.numel() // a.shape[-1], a.shape[-1], _ptr(out)))
    return out


UNARY = {"sigmoid": 0, "tanh": 1, "relu": 2, "softplus": 3, "log": 4, "rsqrt": 5, "erf": 6, "abs": 7, "sign": 8,
         "neg": 9, "reciprocal": 10, "sqrt": 11}


def unary(name, a):
    """tfcc_rocm_unary_f32: one of UNARY applied element-wise."""
    import torch
    a = a.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_unary_f32(_stream(), UNARY[name], _ptr(a), a.numel(), _ptr(out)))
    return out


def lstm_cell(state_c, input_value, state_h_value, bias, forget):
    """CellInterface::processLSTMCell (tfcc/mkl/interfaces/tfcc_mklcellinterface.cpp:33-63): (h, cs)."""
    import torch
    if state_c.dim() != 2:
        raise InvalidArgumentError("invalid stateC")
    batch, units = state_c.shape
    if tuple(input_value.shape) != (batch, units * 4):
        raise InvalidArgumentError("invalid inputValue")
    if tuple(state_h_value.shape) != (batch, units * 4):
        raise InvalidArgumentError("invalid stateHValue")
    if tuple(bias.shape) != (units * 4,):
        raise InvalidArgumentError("invalid bias")
    state_c, input_value, state_h_value, bias = (t.contiguous() for t in (state_c, input_value, state_h_value, bias))
    h, cs = torch.empty_like(state_c), torch.empty_like(state_c)
    check(lib().tfcc_rocm_lstm_cell_f32(_stream(), batch, units, _ptr(state_c), _ptr(input_value),
                                        _ptr(state_h_value), _ptr(bias), float(forget), _ptr(h), _ptr(cs)))
    return h, cs


def gru_cell_gates(state, inputs, value, bias):
    """CellInterface::processGRUCellGates (tfcc/mkl/interfaces/tfcc_mklcellinterface.cpp:65-92)."""
    import torch
    if state.dim() != 2:
        raise InvalidArgumentError("invalid state")
    batch, units = state.shape
    if inputs.dim() != 2 or inputs.shape[0] != batch:
        raise InvalidArgumentError("invalid inputs")
    if tuple(value.shape) != (batch, units * 2):
        raise InvalidArgumentError("invalid value")
    if tuple(bias.shape) != (units * 2,):
        raise InvalidArgumentError("invalid bias")
    state, inputs, value, bias = (t.contiguous() for t in (state, inputs, value, bias))
    out = torch.empty((batch, inputs.shape[1] + units), dtype=state.dtype, device=state.device)
    check(lib().tfcc_rocm_gru_cell_gates_f32(_stream(), batch, units, inputs.shape[1], _ptr(state), _ptr(inputs),
                                             _ptr(value), _ptr(bias), _ptr(out)))
    return out


def gru_cell_candidate(state, value, bias, c_value, c_bias):
    """CellInterface::processGRUCellCandidate (tfcc/mkl/interfaces/tfcc_mklcellinterface.cpp:94-125)."""
    import torch
    if state.dim() != 2:
        raise InvalidArgumentError("invalid state")
    batch, units = state.shape
    if tuple(value.shape) != (batch, units * 2):
        raise InvalidArgumentError("invalid value")
    if tuple(bias.shape) != (units * 2,):
        raise InvalidArgumentError("invalid bias")
    if tuple(c_value.shape) != (batch, units):
        raise InvalidArgumentError("invalid cValue")
    if tuple(c_bias.shape) != (units,):
        raise InvalidArgumentError("invalid cBias")
    state, value, bias, c_value, c_bias = (t.contiguous() for t in (state, value, bias, c_value, c_bias))
    out = torch.empty_like(state)
    check(lib().tfcc_rocm_gru_cell_candidate_f32(_stream(), batch, units, _ptr(state), _ptr(value), _ptr(bias),
                                                 _ptr(c_value), _ptr(c_bias), _ptr(out)))
    return out


def pytorch_gru_cell(state, input_value, state_value, gate_bias, candidate_i_bias, candidate_h_bias):
    """CellInterface::processPyTorchGRUCell (tfcc/mkl/interfaces/tfcc_mklcellinterface.cpp:127-165)."""
    import torch
    if state.dim() != 2:
        raise InvalidArgumentError("invalid state")
    batch, units = state.shape
    if tuple(input_value.shape) != (batch, units * 3):
        raise InvalidArgumentError("invalid inputValue")
    if tuple(state_value.shape) != (batch, units * 3):
        raise InvalidArgumentError("invalid stateValue")
    if tuple(gate_bias.shape) != (units * 2,):
        raise InvalidArgumentError("invalid gateBias")
    if tuple(candidate_i_bias.shape) != (units,):
        raise InvalidArgumentError("invalid candidateIBias")
    if tuple(candidate_h_bias.shape) != (units,):
        raise InvalidArgumentError("invalid candidateHBias")
    ts = [t.contiguous() for t in (state, input_value, state_value, gate_bias, candidate_i_bias, candidate_h_bias)]
    out = torch.empty_like(ts[0])
    check(lib().tfcc_rocm_pytorch_gru_cell_f32(_stream(), batch, units, *[_ptr(t) for t in ts], _ptr(out)))
    return out


def gelu_accurate(a):
    import torch
    a = a.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_gelu_accurate_f32(_stream(), _ptr(a), a.numel(), _ptr(out)))
    return out


def transform(a, alpha, beta):
    import torch
    a = a.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_transform_f32(_stream(), _ptr(a), a.numel(), alpha, beta, _ptr(out)))
    return out


def add(a, b):
    """a + b where b's shape equals the trailing dims of a's."""
    import torch
    a, b = a.contiguous(), b.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_add_f32(_stream(), _ptr(a), _ptr(b), a.numel(), b.numel(), _ptr(out)))
    return out


def transform2(a, alpha, beta):
    """a / alpha + beta"""
    import torch
    a = a.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_transform2_f32(_stream(), _ptr(a), a.numel(), alpha, beta, _ptr(out)))
    return out


BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "pow": 4, "max": 5, "min": 6}


def binary(op, a, b):
    """a (op) b where b's shape equals the trailing dims of a's; op in BINARY_OPS."""
    import torch
    a, b = a.contiguous(), b.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_binary_f32(_stream(), BINARY_OPS[op], _ptr(a), _ptr(b), a.numel(), b.numel(), _ptr(out)))
    return out


def gather(params, indices):
    """tfcc::nn::gather (tfcc/core/operations/tfcc_nn.cpp:345-385): rows of params by index, zeros for an index
    outside [0, rows)."""
    import torch
    if params.numel() == 0:
        raise InvalidArgumentError("invalid tensor")
    params, indices = params.contiguous(), indices.contiguous()
    out = torch.empty(tuple(indices.shape) + tuple(params.shape[1:]), dtype=params.dtype, device=params.device)
    if indices.numel() == 0:
        return out
    chunk = params.numel() // params.shape[0] * params.element_size()
    check(lib().tfcc_rocm_gather_rows(_stream(), _ptr(params), params.shape[0], chunk, _ptr(indices),
                                      _type_code(indices.dtype), indices.numel(), _ptr(out)))
    return out


def cast(a, dtype):
    """tfcc::data::cast: element-wise static_cast."""
    import torch
    a = a.contiguous()
    out = torch.empty(a.shape, dtype=dtype, device=a.device)
    if a.numel():
        check(lib().tfcc_rocm_cast(_stream(), _ptr(a), _type_code(a.dtype), _ptr(out), _type_code(dtype), a.numel()))
    return out


def _split_at(shape, axis):
    s1 = 1
    for d in shape[:axis]:
        s1 *= d
    s3 = 1
    for d in shape[axis + 1:]:
        s3 *= d
    return s1, shape[axis], s3


def slice_axis(a, axis, start, end):
    """tfcc::base::slice (tfcc/core/operations/tfcc_base.cpp:28-41; end is clipped to the dimension as
    tfcc/mkl/interfaces/tfcc_mklbasicinterface.cpp:490 clips it)."""
    import torch
    if axis >= a.dim():
        raise InvalidArgumentError("invalid axis")
    if start >= end:
        raise InvalidArgumentError("start large than end")
    if start >= a.shape[axis]:
        raise InvalidArgumentError("invalid start")
    a = a.contiguous()
    end = min(end, a.shape[axis])
    s1, s2, s3 = _split_at(tuple(a.shape), axis)
    shape = list(a.shape)
    shape[axis] = end - start
    out = torch.empty(shape, dtype=a.dtype, device=a.device)
    e = a.element_size()
    if out.numel():
        check(lib().tfcc_rocm_copy2d(_stream(), a.data_ptr() + start * s3 * e, s2 * s3 * e, _ptr(out),
                                     (end - start) * s3 * e, s1, (end - start) * s3 * e))
    return out


def concat(values, axis):
    """tfcc::base::concat (tfcc/core/operations/tfcc_base.cpp:86-106)."""
    import torch
    if len(values) == 0:
        raise InvalidArgumentError("values.size could not be zero")
    for v in values:
        if axis >= v.dim():
            raise InvalidArgumentError("invalid axis")
        if v.dim() != values[0].dim() or any(i != axis and v.shape[i] != values[0].shape[i] for i in range(v.dim())):
            raise InvalidArgumentError("invalid shape")
    values = [v.contiguous() for v in values]
    shape = list(values[0].shape)
    shape[axis] = sum(v.shape[axis] for v in values)
    out = torch.empty(shape, dtype=values[0].dtype, device=values[0].device)
    s1, total, s3 = _split_at(tuple(shape), axis)
    e = out.element_size()
    offset = 0
    for v in values:
        width = v.shape[axis] * s3 * e
        if width and s1:
            check(lib().tfcc_rocm_copy2d(_stream(), _ptr(v), width, out.data_ptr() + offset, total * s3 * e, s1, width))
        offset += width
    return out


REDUCE_OPS = {"sum": 0, "mean": 1, "prod": 2, "max": 3, "min": 4}


def reduce_trailing(op, a, keep):
    """tfcc::math::reduce_sum / reduce_mean / reduce_prod / reduce_max / reduce_min (tfcc/core/operations/
    tfcc_math.cpp:464-520): the dimensions from `keep` on are reduced and stay in the shape as 1."""
    import torch
    if a.numel() == 0:
        raise InvalidArgumentError("invalid tensor")
    if keep >= a.dim():
        raise InvalidArgumentError("invalid keep dims")
    a = a.contiguous()
    cols = 1
    for d in a.shape[keep:]:
        cols *= d
    out = torch.empty(tuple(a.shape[:keep]) + (1,) * (a.dim() - keep), dtype=torch.float32, device=a.device)
    check(lib().tfcc_rocm_reduce_f32(_stream(), REDUCE_OPS[op], _ptr(a), a.numel() // cols, cols, _ptr(out)))
    return out


def clip(a, lo, hi):
    import torch
    a = a.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_clip_f32(_stream(), _ptr(a), a.numel(), lo, hi, _ptr(out)))
    return out


def leaky_relu(a, alpha):
    import torch
    a = a.contiguous()
    out = torch.empty_like(a)
    check(lib().tfcc_rocm_leaky_relu_f32(_stream(), _ptr(a), a.numel(), alpha, _ptr(out)))
    return out


def broadcast_shapes(s1, s2):
    """_get_broadcast_shape of tfcc/core/operations/tfcc_math.cpp:38-86: (result shape, collapsed s1, collapsed s2).
    Right-aligned; extents must be equal or 1; runs of dimensions of the same kind are merged."""
    s1, s2 = list(s1), list(s2)
    if not s1 or not s2:
        raise InvalidArgumentError("invalid tensor shape")
    result = list(s1 if len(s1) > len(s2) else s2)
    for i in range(min(len(s1), len(s2))):
        l1, l2 = s1[-1 - i], s2[-1 - i]
        if l1 != l2 and l1 != 1 and l2 != 1:
            raise InvalidArgumentError("broadcast failed")
        result[-1 - i] = l2 if l1 == 1 else l1  # the reference takes max(): 0 against 1 would give 1 and read past the empty operand
    kind = lambda l1, l2: 0 if l1 == l2 else (1 if l1 == 1 else 2)  # noqa: E731
    n1, n2 = [], []
    len1, len2 = s1[-1], s2[-1]
    cur = kind(len1, len2)
    for i in range(1, max(len(s1), len(s2))):
        l1 = s1[-1 - i] if i < len(s1) else 1
        l2 = s2[-1 - i] if i < len(s2) else 1
        if kind(l1, l2) != cur:
            n1.insert(0, len1)
            n2.insert(0, len2)
            cur, len1, len2 = kind(l1, l2), l1, l2
        else:
            len1 *= l1
            len2 *= l2
    if len1 != 1 or len2 != 1 or not n1:
        n1.insert(0, len1)
        n2.insert(0, len2)
    return tuple(result), tuple(n1), tuple(n2)


def math_binary(op, a, b):
    """tfcc::math::add / sub / mul / div / pow / max / min (op in BINARY_OPS) with the reference's broadcasting."""
    import torch
    shape, ca, cb = broadcast_shapes(a.shape, b.shape)
    out = torch.empty(shape, dtype=torch.float32, device=a.device)
    if out.numel() == 0:
        return out
    if len(ca) > 6:
        raise NotImplementedError("more than six groups of broadcast dimensions")
    a, b = a.contiguous(), b.contiguous()
    dims = [max(x, y) for x, y in zip(ca, cb)]

    def strides(c):
        st, acc = [0] * len(c), 1
        for d in range(len(c) - 1, -1, -1):
            st[d] = 0 if c[d] == 1 and dims[d] != 1 else acc
            acc *= c[d]
        return st
    n = len(dims)
    check(lib().tfcc_rocm_binary_broadcast_f32(_stream(), BINARY_OPS[op], _ptr(a), _ptr(b), n, (C.c_uint * n)(*dims),
                                               (_U64 * n)(*strides(ca)), (_U64 * n)(*strides(cb)), _ptr(out)))
    return out


COMPARE_OPS = {"equal": 0, "unequal": 1, "greater": 2, "greater_equal": 3, "less": 4, "less_equal": 5}
_C_TYPES = {S8: C.c_int8, U8: C.c_uint8, S16: C.c_int16, U16: C.c_uint16, S32: C.c_int32, U32: C.c_uint32,
            S64: C.c_int64, U64: C.c_uint64, F32: C.c_float, F64: C.c_double}


def compare(op, a, b):
    """tfcc::relation::equal / unequal / greater / greater_equal / less / less_equal (op in COMPARE_OPS): a tensor
    against a Python number (compared directly) or against another tensor of the same element type (the difference,
    taken in the element type with the reference's broadcasting, against 0).  -> uint8 tensor of 0 / 1."""
    import torch
    a = a.contiguous()
    if not isinstance(b, torch.Tensor):
        if a.numel() == 0:
            raise InvalidArgumentError("invalid tensor")
        out = torch.empty(a.shape, dtype=torch.uint8, device=a.device)
        code = _type_code(a.dtype)
        value = _C_TYPES[code](b)
        check(lib().tfcc_rocm_compare_value(_stream(), COMPARE_OPS[op], _ptr(a), code, a.numel(), C.byref(value), _ptr(out)))
        return out
    if a.dtype != b.dtype:
        raise InvalidArgumentError("compare: element types differ")
    if a.numel() == 0 or b.numel() == 0:
        raise InvalidArgumentError("invalid tensor")
    shape, ca, cb = broadcast_shapes(a.shape, b.shape)
    if len(ca) > 6:
        raise NotImplementedError("more than six groups of broadcast dimensions")
    out = torch.empty(shape, dtype=torch.uint8, device=a.device)
    b = b.contiguous()
    dims = [max(x, y) for x, y in zip(ca, cb)]

    def strides(c):
        st, acc = [0] * len(c), 1
        for d in range(len(c) - 1, -1, -1):
            st[d] = 0 if c[d] == 1 and dims[d] != 1 else acc
            acc *= c[d]
        return st
    n = len(dims)
    check(lib().tfcc_rocm_compare(_stream(), COMPARE_OPS[op], _ptr(a), _ptr(b), _type_code(a.dtype), n, (C.c_uint * n)(*dims),
                                  (_U64 * n)(*strides(ca)), (_U64 * n)(*strides(cb)), _ptr(out)))
    return out


def _bits_of(value, dtype):
    import torch
    return int.from_bytes(torch.tensor([value], dtype=dtype).numpy().tobytes(), "little")


def where(condition, x, y):
    """tfcc::nn::where: condition (uint8) != 0 ? x : y; x or y (not both) may be a Python number."""
    import torch
    tensors = [t for t in (x, y) if isinstance(t, torch.Tensor)]
    if not tensors:
        raise InvalidArgumentError("where: x and y are both values")
    if any(t.shape != condition.shape for t in tensors):
        raise InvalidArgumentError("condition x and y has different shape")
    dtype = tensors[0].dtype
    out = torch.empty(condition.shape, dtype=dtype, device=condition.device)
    if out.numel() == 0:
        return out
    condition = condition.contiguous()
    xt = x.contiguous() if isinstance(x, torch.Tensor) else None
    yt = y.contiguous() if isinstance(y, torch.Tensor) else None
    check(lib().tfcc_rocm_where(_stream(), _ptr(condition), _ptr(xt) if xt is not None else None,
                                0 if xt is not None else _bits_of(x, dtype), _ptr(yt) if yt is not None else None,
                                0 if yt is not None else _bits_of(y, dtype), out.element_size(), out.numel(), _ptr(out)))
    return out


def triangle(a, k, upper):
    """tfcc::base::tril (upper False) / triu (upper True) of a matrix."""
    import torch
    if a.dim() != 2:
        raise InvalidArgumentError("invalid shape")
    a = a.contiguous()
    out = torch.empty_like(a)
    if a.numel():
        check(lib().tfcc_rocm_triangle(_stream(), _ptr(a), a.shape[0], a.shape[1], k, 1 if upper else 0, a.element_size(),
                                       _ptr(out)))
    return out


def top_k(a, k):
    """tfcc::math::top_k: (values, positions) of the k largest elements along the last axis, descending; positions
    come back as int64 holding the kernel's uint32 results (torch has no uint32 arithmetic)."""
    import torch
    if a.numel() == 0:
        raise InvalidArgumentError("invalid tensor")
    if a.shape[-1] < k:
        raise InvalidArgumentError("invalid k")
    a = a.contiguous()
    shape = list(a.shape[:-1]) + [k]
    values = torch.empty(shape, dtype=torch.float32, device=a.device)
    positions = torch.empty(shape, dtype=torch.int32, device=a.device)
    check(lib().tfcc_rocm_topk_f32(_stream(), _ptr(a), a.numel() // a.shape[-1], a.shape[-1], k, _ptr(values), _ptr(positions)))
    return values, positions.to(torch.int64) & 0xFFFFFFFF


def argmax(a, axis):
    """tfcc::math::argmax: int64 positions of the first largest element along axis, which stays with length 1."""
    import torch
    if a.numel() == 0:
        raise InvalidArgumentError("invalid tensor")
    if not 0 <= axis < a.dim():
        raise InvalidArgumentError("invalid axis")
    a = a.contiguous()
    s1, _, s3 = _split_at(a.shape, axis)
    shape = list(a.shape)
    shape[axis] = 1
    out = torch.empty(shape, dtype=torch.int64, device=a.device)
    check(lib().tfcc_rocm_argmax_f32(_stream(), _ptr(a), s1, a.shape[axis], s3, _ptr(out)))
    return out


def transpose(a, perm):
    import torch
    a = a.contiguous()
    shape = (C.c_uint * a.dim())(*a.shape)
    p = (C.c_uint * a.dim())(*perm)
    out = torch.empty([a.shape[i] for i in perm], dtype=a.dtype, device=a.device)
    check(lib().tfcc_rocm_transpose_f32(_stream(), _ptr(a), shape, p, a.dim(), _ptr(out)))
    return out
