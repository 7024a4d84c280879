"""ctypes bindings of the CPU oracle (oracle/liboracle.so) and, where it has been built, of the
reference's own kernels (oracle/_ref/libtfcc_ref.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "liboracle.so")
REF_SO = os.path.join(ORACLE_DIR, "_ref", "libtfcc_ref.so")

ROUND_NEAREST_EVEN = 0
ROUND_HALF_AWAY = 1

_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C")
_s8p = np.ctypeslib.ndpointer(np.int8, flags="C")
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C")


def _bind_cells(lib, prefix):
    """The four recurrent-cell entry points, which the oracle and the reference build share."""
    f = getattr(lib, prefix + "lstm_cell")
    f.restype = None
    f.argtypes = [C.c_uint, C.c_uint, _f32p, _f32p, _f32p, _f32p, C.c_float, _f32p, _f32p]
    f = getattr(lib, prefix + "gru_cell_gates")
    f.restype = None
    f.argtypes = [C.c_uint, C.c_uint, C.c_uint, _f32p, _f32p, _f32p, _f32p, _f32p]
    f = getattr(lib, prefix + "gru_cell_candidate")
    f.restype = None
    f.argtypes = [C.c_uint, C.c_uint, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p]
    f = getattr(lib, prefix + "pytorch_gru_cell")
    f.restype = None
    f.argtypes = [C.c_uint, C.c_uint, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p]


def build_oracle():
    """Compile the oracle with the Makefile beside it (a few seconds)."""
    subprocess.check_call(["make", "-s", "-C", ORACLE_DIR], stdout=subprocess.DEVNULL)


def _load_oracle():
    if not os.path.exists(ORACLE_SO):
        build_oracle()
    lib = C.CDLL(ORACLE_SO)
    lib.oracle_matmul_plan.restype = C.c_int
    lib.oracle_matmul_plan.argtypes = [_u32p, C.c_int, _u32p, C.c_int, _u32p, C.c_int, _u32p,
                                       C.POINTER(C.c_int)] + [C.POINTER(C.c_uint)] * 7 + [C.POINTER(C.c_int)]
    lib.oracle_sgemm_strided_batched.restype = None
    lib.oracle_sgemm_strided_batched.argtypes = [_f32p, C.c_uint64, _f32p, C.c_uint64, C.c_void_p,
                                                 C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint,
                                                 C.c_uint, C.c_uint, C.c_uint]
    for name, p in (("row_u8", _u8p), ("row_s8", _s8p), ("col_u8", _u8p), ("col_s8", _s8p)):
        f = getattr(lib, "oracle_reduce_sum_" + name)
        f.restype = None
        f.argtypes = [p, C.c_uint, C.c_uint, C.c_uint, _i32p]
    lib.oracle_qmatmul_offsets.restype = None
    lib.oracle_qmatmul_offsets.argtypes = [C.c_float] * 4 + [C.POINTER(C.c_int32)] * 2
    lib.oracle_qgemm_u8s8s32.restype = None
    lib.oracle_qgemm_u8s8s32.argtypes = [C.c_uint, _u8p, C.c_uint64, _s8p, C.c_uint64, _i32p,
                                         C.c_uint64, _i32p, C.c_uint64, C.c_int32, C.c_int32,
                                         C.c_uint, C.c_uint, C.c_uint, _i32p, C.c_uint64]
    lib.oracle_qmatmul_range.restype = None
    lib.oracle_qmatmul_range.argtypes = [C.c_float] * 4 + [C.POINTER(C.c_float)] * 2
    lib.oracle_quantized_scale_info.restype = None
    lib.oracle_quantized_scale_info.argtypes = [C.c_int, C.c_float, C.c_float,
                                                C.POINTER(C.c_double), C.POINTER(C.c_int64)]
    lib.oracle_dequantized_scale_info.restype = None
    lib.oracle_dequantized_scale_info.argtypes = [C.c_int, C.c_float, C.c_float,
                                                  C.POINTER(C.c_double), C.POINTER(C.c_double)]
    lib.oracle_requantize_one.restype = C.c_int64
    lib.oracle_requantize_one.argtypes = [C.c_int64, C.c_int64, C.c_double, C.c_double, C.c_double,
                                          C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int]
    lib.oracle_requantize_s32_u8.restype = None
    lib.oracle_requantize_s32_u8.argtypes = [_i32p, C.c_uint64] + [C.c_float] * 4 + [C.c_int, C.c_int, _u8p]
    lib.oracle_requantize_s8_u16.restype = None
    lib.oracle_requantize_s8_u16.argtypes = [_s8p, C.c_uint64] + [C.c_float] * 4 + [C.c_int, C.c_int, _u16p]
    for name, p in (("s8", _s8p), ("u8", _u8p), ("s32", _i32p)):
        f = getattr(lib, "oracle_dequantize_" + name)
        f.restype = None
        f.argtypes = [p, C.c_uint64, C.c_float, C.c_float, C.c_int, _f32p]
    for name, p in (("u8", _u8p), ("s8", _s8p)):
        f = getattr(lib, "oracle_quantize_" + name)
        f.restype = None
        f.argtypes = [_f32p, C.c_uint64, C.c_float, C.c_float, C.c_int, p]
    lib.oracle_dequant_per_channel.restype = None
    lib.oracle_dequant_per_channel.argtypes = [_i32p, C.c_uint, C.c_uint, C.c_float, _f32p, _f32p]
    lib.oracle_softmax_lastaxis.restype = None
    lib.oracle_softmax_lastaxis.argtypes = [_f32p, C.c_uint64, C.c_uint, _f32p]
    lib.oracle_layer_norm.restype = None
    lib.oracle_layer_norm.argtypes = [_f32p, _f32p, _f32p, C.c_float, C.c_uint64, C.c_uint, _f32p]
    lib.oracle_gelu_accurate.restype = None
    lib.oracle_gelu_accurate.argtypes = [_f32p, C.c_uint64, _f32p]
    _bind_cells(lib, "oracle_")
    lib.oracle_lstm_sequence.restype = None
    lib.oracle_lstm_sequence.argtypes = [C.c_int] + [C.c_uint] * 4 + [_f32p] * 9
    return lib


_oracle = None


def oracle():
    global _oracle
    if _oracle is None:
        _oracle = _load_oracle()
    return _oracle


_ref = None


def ref():
    """The reference's own kernels, or None where oracle/_ref has not been built."""
    global _ref
    if _ref is None and os.path.exists(REF_SO):
        lib = C.CDLL(REF_SO)
        lib.ref_qmatmul_offsets.restype = None
        lib.ref_qmatmul_offsets.argtypes = [C.c_float] * 4 + [C.POINTER(C.c_int32)] * 2
        lib.ref_qmatmul_range.restype = None
        lib.ref_qmatmul_range.argtypes = [C.c_float] * 4 + [C.POINTER(C.c_float)] * 2
        lib.ref_qgemm_u8s8s32.restype = None
        lib.ref_qgemm_u8s8s32.argtypes = [C.c_uint, _u8p, C.c_uint, _s8p, C.c_uint, _i32p, C.c_uint,
                                          _i32p, C.c_uint, C.c_int32, C.c_int32, C.c_uint, C.c_uint,
                                          C.c_uint, _i32p]
        lib.ref_qgemm_n1.restype = None
        lib.ref_qgemm_n1.argtypes = [_u8p, _i32p, C.c_int32, _s8p, C.c_int32, C.c_int32, C.c_uint,
                                     C.c_uint, _i32p]
        for nm in ("ref_quantized_scale_info_u8", "ref_quantized_scale_info_u16"):
            f = getattr(lib, nm)
            f.restype = None
            f.argtypes = [C.c_float, C.c_float, C.POINTER(C.c_double), C.POINTER(C.c_int64)]
        lib.ref_dequantized_scale_info_s32.restype = None
        lib.ref_dequantized_scale_info_s32.argtypes = [C.c_float, C.c_float, C.POINTER(C.c_double),
                                                       C.POINTER(C.c_double)]
        lib.ref_requantize_s32_u8.restype = None
        lib.ref_requantize_s32_u8.argtypes = [_i32p, C.c_uint64] + [C.c_float] * 4 + [C.c_int, _u8p]
        lib.ref_requantize_s8_u16.restype = None
        lib.ref_requantize_s8_u16.argtypes = [_s8p, C.c_uint64] + [C.c_float] * 4 + [C.c_int, _u16p]
        for name, p in (("s8", _s8p), ("u8", _u8p), ("s32", _i32p)):
            f = getattr(lib, "ref_dequantize_" + name)
            f.restype = None
            f.argtypes = [p, C.c_uint64, C.c_float, C.c_float, C.c_int, _f32p]
        for name, p in (("u8", _u8p), ("s8", _s8p)):
            f = getattr(lib, "ref_quantize_" + name)
            f.restype = None
            f.argtypes = [_f32p, C.c_uint64, C.c_float, C.c_float, C.c_int, p]
        _bind_cells(lib, "ref_")
        _ref = lib
    return _ref


# --------------------------------------------------------------------------------------------
# numpy-level helpers
# --------------------------------------------------------------------------------------------

def matmul_plan(shape_a, shape_b, shape_bias=None):
    """Returns (status, dict) following the reference's validation and stride rules."""
    sa = np.asarray(list(shape_a) or [0], np.uint32)
    sb = np.asarray(list(shape_b) or [0], np.uint32)
    sbias = np.asarray(list(shape_bias) if shape_bias else [0], np.uint32)
    out = np.zeros(max(len(shape_a), len(shape_b), 1), np.uint32)
    rank = C.c_int()
    vals = [C.c_uint() for _ in range(7)]
    empty = C.c_int()
    st = oracle().oracle_matmul_plan(sa, len(shape_a), sb, len(shape_b), sbias,
                                     -1 if shape_bias is None else len(shape_bias), out,
                                     C.byref(rank), *[C.byref(v) for v in vals], C.byref(empty))
    if st != 0:
        return st, None
    names = ("m", "n", "k", "strideA", "strideB", "strideC", "batch")
    d = {k: v.value for k, v in zip(names, vals)}
    d["shape"] = tuple(int(x) for x in out[:rank.value])
    d["empty"] = bool(empty.value)
    return 0, d


def sgemm(a, b, bias=None, want64=False):
    """fp32 matmul with the reference's shape rules, double accumulation."""
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    st, p = matmul_plan(a.shape, b.shape, None if bias is None else bias.shape)
    assert st == 0, st
    c = np.empty(p["shape"], np.float32)
    c64 = np.empty(p["shape"], np.float64) if want64 else None
    if bias is not None:
        bias = np.ascontiguousarray(bias, np.float32)
    oracle().oracle_sgemm_strided_batched(
        a, p["strideA"], b, p["strideB"], None if bias is None else bias.ctypes.data,
        c.ctypes.data, None if c64 is None else c64.ctypes.data, p["strideC"], p["m"], p["n"],
        p["k"], p["batch"])
    return (c, c64) if want64 else c


def reduce_sum(a, row):
    a = np.ascontiguousarray(a)
    r, c = a.shape[-2], a.shape[-1]
    batch = a.size // (r * c)
    out = np.empty(a.shape[:-2] + ((r,) if row else (c,)), np.int32)
    name = "oracle_reduce_sum_%s_%s" % ("row" if row else "col", "u8" if a.dtype == np.uint8 else "s8")
    getattr(oracle(), name)(a, batch, r, c, out)
    return out


def qmatmul_offsets(min_a, max_a, min_b, max_b, lib=None):
    oa, ob = C.c_int32(), C.c_int32()
    f = oracle().oracle_qmatmul_offsets if lib is None else lib.ref_qmatmul_offsets
    f(min_a, max_a, min_b, max_b, C.byref(oa), C.byref(ob))
    return oa.value, ob.value


def qmatmul_range(min_a, max_a, min_b, max_b, lib=None):
    mn, mx = C.c_float(), C.c_float()
    f = oracle().oracle_qmatmul_range if lib is None else lib.ref_qmatmul_range
    f(min_a, max_a, min_b, max_b, C.byref(mn), C.byref(mx))
    return mn.value, mx.value


def _qplan(a, b):
    """Stride / fold rules of the quantized matmul (tfcc_mklquantization.cpp:119-145)."""
    m, k, n = a.shape[-2], a.shape[-1], b.shape[-1]
    shape = (a.shape if a.ndim > b.ndim else b.shape)[:-2] + (m, n)
    batch = int(np.prod(shape[:-2], dtype=np.int64)) if len(shape) > 2 else 1
    strideA = 0 if a.ndim == 2 else m * k
    strideB = 0 if b.ndim == 2 else k * n
    return m, n, k, shape, batch, strideA, strideB


def qgemm(a, b, offset_a, offset_b, rowsum=None, colsum=None, lib=None):
    """uint8 x int8 -> int32 with offsets.  lib = ref() runs the reference's own AVX2 kernel."""
    a = np.ascontiguousarray(a, np.uint8)
    b = np.ascontiguousarray(b, np.int8)
    if rowsum is None:
        rowsum = reduce_sum(a, True)
    if colsum is None:
        colsum = reduce_sum(b, False)
    rowsum = np.ascontiguousarray(rowsum, np.int32)
    colsum = np.ascontiguousarray(colsum, np.int32)
    m, n, k, shape, batch, strideA, strideB = _qplan(a, b)
    sra = 0 if rowsum.ndim == 1 else m
    srb = 0 if colsum.ndim == 1 else n
    if b.ndim == 2:  # single B: fold the batch into M
        m, sra, strideA, batch = m * batch, sra * batch, strideA * batch, 1
    c = np.empty(shape, np.int32)
    if lib is None:
        oracle().oracle_qgemm_u8s8s32(batch, a, strideA, b, strideB, rowsum, sra, colsum, srb,
                                      offset_a, offset_b, m, n, k, c, m * n)
    else:
        lib.ref_qgemm_u8s8s32(batch, a, strideA, b, strideB, rowsum, sra, colsum, srb, offset_a,
                              offset_b, m, n, k, c)
    return c


def quantized_scale_info(bits, mn, mx):
    s, o = C.c_double(), C.c_int64()
    oracle().oracle_quantized_scale_info(bits, mn, mx, C.byref(s), C.byref(o))
    return s.value, o.value


def dequantized_scale_info(bits, mn, mx):
    s, o = C.c_double(), C.c_double()
    oracle().oracle_dequantized_scale_info(bits, mn, mx, C.byref(s), C.byref(o))
    return s.value, o.value


def requantize_s32_u8(a, min_in, max_in, min_out, max_out, rounding=ROUND_NEAREST_EVEN, fma=1):
    a = np.ascontiguousarray(a, np.int32)
    out = np.empty(a.shape, np.uint8)
    oracle().oracle_requantize_s32_u8(a, a.size, min_in, max_in, min_out, max_out, rounding, fma, out)
    return out


def requantize_s8_u16(a, min_in, max_in, min_out, max_out, rounding=ROUND_NEAREST_EVEN, fma=1):
    a = np.ascontiguousarray(a, np.int8)
    out = np.empty(a.shape, np.uint16)
    oracle().oracle_requantize_s8_u16(a, a.size, min_in, max_in, min_out, max_out, rounding, fma, out)
    return out


def dequantize(a, mn, mx, fma=1):
    a = np.ascontiguousarray(a)
    name = {np.dtype(np.int8): "s8", np.dtype(np.uint8): "u8", np.dtype(np.int32): "s32"}[a.dtype]
    out = np.empty(a.shape, np.float32)
    getattr(oracle(), "oracle_dequantize_" + name)(a, a.size, mn, mx, fma, out)
    return out


def quantize(a, mn, mx, dtype, rounding=ROUND_NEAREST_EVEN):
    a = np.ascontiguousarray(a, np.float32)
    out = np.empty(a.shape, dtype)
    name = "u8" if np.dtype(dtype) == np.uint8 else "s8"
    getattr(oracle(), "oracle_quantize_" + name)(a, a.size, mn, mx, rounding, out)
    return out


def dequant_per_channel(acc, scale_a, scale_b):
    acc = np.ascontiguousarray(acc, np.int32)
    scale_b = np.ascontiguousarray(scale_b, np.float32)
    out = np.empty(acc.shape, np.float32)
    oracle().oracle_dequant_per_channel(acc.reshape(-1, acc.shape[-1]), acc.size // acc.shape[-1],
                                        acc.shape[-1], scale_a, scale_b, out)
    return out


def softmax(a):
    a = np.ascontiguousarray(a, np.float32)
    out = np.empty_like(a)
    oracle().oracle_softmax_lastaxis(a, a.size // a.shape[-1], a.shape[-1], out)
    return out


def layer_norm(a, gamma, beta, eps):
    a = np.ascontiguousarray(a, np.float32)
    out = np.empty_like(a)
    oracle().oracle_layer_norm(a, np.ascontiguousarray(gamma, np.float32),
                               np.ascontiguousarray(beta, np.float32), eps,
                               a.size // a.shape[-1], a.shape[-1], out)
    return out


def gelu_accurate(a):
    a = np.ascontiguousarray(a, np.float32)
    out = np.empty_like(a)
    oracle().oracle_gelu_accurate(a, a.size, out)
    return out


def _f32(*arrays):
    return [np.ascontiguousarray(a, np.float32) for a in arrays]


def lstm_cell(state_c, input_value, state_h_value, bias, forget, lib=None, prefix="oracle_"):
    state_c, input_value, state_h_value, bias = _f32(state_c, input_value, state_h_value, bias)
    h, cs = np.empty_like(state_c), np.empty_like(state_c)
    getattr(lib or oracle(), prefix + "lstm_cell")(state_c.shape[0], state_c.shape[1], state_c, input_value,
                                                  state_h_value, bias, forget, h, cs)
    return h, cs


def gru_cell_gates(state, inputs, value, bias, lib=None, prefix="oracle_"):
    state, inputs, value, bias = _f32(state, inputs, value, bias)
    out = np.empty((state.shape[0], inputs.shape[1] + state.shape[1]), np.float32)
    getattr(lib or oracle(), prefix + "gru_cell_gates")(state.shape[0], state.shape[1], inputs.shape[1], state,
                                                       inputs, value, bias, out)
    return out


def gru_cell_candidate(state, value, bias, c_value, c_bias, lib=None, prefix="oracle_"):
    state, value, bias, c_value, c_bias = _f32(state, value, bias, c_value, c_bias)
    out = np.empty_like(state)
    getattr(lib or oracle(), prefix + "gru_cell_candidate")(state.shape[0], state.shape[1], state, value, bias,
                                                           c_value, c_bias, out)
    return out


def pytorch_gru_cell(state, input_value, state_value, gate_bias, ci_bias, ch_bias, lib=None, prefix="oracle_"):
    arrays = _f32(state, input_value, state_value, gate_bias, ci_bias, ch_bias)
    out = np.empty_like(arrays[0])
    getattr(lib or oracle(), prefix + "pytorch_gru_cell")(arrays[0].shape[0], arrays[0].shape[1], *arrays, out)
    return out


def lstm_sequence(a, input_kernel, state_kernel, bias, ih, ic, backward=False):
    """tfcc::rnn::lstm_forward / lstm_backward: (outputs [seq, batch, hidden], h, c)."""
    a, input_kernel, state_kernel, bias, ih, ic = _f32(a, input_kernel, state_kernel, bias, ih, ic)
    seq, batch, length = a.shape
    hidden = ih.shape[1]
    out = np.empty((seq, batch, hidden), np.float32)
    h, c = np.empty_like(ih), np.empty_like(ih)
    oracle().oracle_lstm_sequence(int(backward), seq, batch, length, hidden, a, input_kernel, state_kernel, bias,
                                  ih, ic, out, h, c)
    return out, h, c
