"""ctypes binding of libtfcc_runtime.so (the C ABI of include/tfcc_rocm_runtime.h): the model
runtime on the ROCm device.  `Model` mirrors tfcc::runtime::Model (tfcc_runtime/framework/model.h:37-103)."""
import ctypes as C
import os

from . import modelfile

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtfcc_runtime.so")

_VP = C.c_void_p
SYMBOLS = {
    "tfcc_rocm_runtime_initialize": (C.c_int, []),
    "tfcc_rocm_runtime_initialize_host": (C.c_int, []),
    "tfcc_rocm_runtime_last_error": (C.c_char_p, []),
    "tfcc_rocm_runtime_model_create": (C.c_int, [_VP, C.c_size_t, C.POINTER(_VP)]),
    "tfcc_rocm_runtime_model_destroy": (C.c_int, [_VP]),
    "tfcc_rocm_runtime_model_run": (C.c_int, [_VP, _VP, C.c_size_t, C.POINTER(_VP), C.POINTER(C.c_size_t)]),
    "tfcc_rocm_runtime_buffer_free": (C.c_int, [_VP]),
    "tfcc_rocm_runtime_model_test": (C.c_int, [_VP, _VP, C.c_size_t, C.POINTER(C.c_int), C.POINTER(_VP)]),
    "tfcc_rocm_runtime_set_fusion": (C.c_int, [C.c_int]),
    "tfcc_rocm_runtime_model_step_count": (C.c_int, [_VP, C.POINTER(C.c_size_t)]),
    "tfcc_rocm_runtime_model_set_replay": (C.c_int, [_VP, C.c_int]),
    "tfcc_rocm_runtime_model_time": (C.c_int, [_VP, _VP, C.c_size_t, C.c_int, C.c_int, C.POINTER(C.c_double)]),
}

_lib = None


class RuntimeError_(RuntimeError):
    """tfcc::runtime::RuntimeError and every other exception the runtime raises"""


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError_("%s is missing: build it with `make -C %s`" % (LIB_PATH, os.path.join(_HERE, "host")))
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            f = getattr(handle, name)
            f.restype = res
            f.argtypes = args
        _lib = handle
    return _lib


def check(status):
    if status != 0:
        raise RuntimeError_(lib().tfcc_rocm_runtime_last_error().decode(errors="replace"))


def initialize(host=False):
    """host=True binds the host-memory device (no compute) instead of the GPU"""
    check(lib().tfcc_rocm_runtime_initialize_host() if host else lib().tfcc_rocm_runtime_initialize())


def set_fusion(enable):
    """graphs built afterwards fuse node sequences (default) or run every node as written"""
    check(lib().tfcc_rocm_runtime_set_fusion(1 if enable else 0))


class Model:
    def __init__(self, archive, host=False):
        initialize(host)
        self._h = _VP()
        buf = bytes(archive)
        check(lib().tfcc_rocm_runtime_model_create(buf, len(buf), C.byref(self._h)))

    def close(self):
        if self._h:
            check(lib().tfcc_rocm_runtime_model_destroy(self._h))
            self._h = _VP()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def run_serialized(self, inputs):
        out, n = _VP(), C.c_size_t()
        buf = bytes(inputs)
        check(lib().tfcc_rocm_runtime_model_run(self._h, buf, len(buf), C.byref(out), C.byref(n)))
        try:
            return C.string_at(out, n.value)
        finally:
            lib().tfcc_rocm_runtime_buffer_free(out)

    def run(self, arrays):
        """{name: ndarray} -> {name: ndarray}"""
        return modelfile.decode_outputs(self.run_serialized(modelfile.encode_inputs(arrays)))

    def test(self, npz_bytes):
        passed, report = C.c_int(), _VP()
        buf = bytes(npz_bytes)
        check(lib().tfcc_rocm_runtime_model_test(self._h, buf, len(buf), C.byref(passed), C.byref(report)))
        try:
            return bool(passed.value), C.string_at(report).decode(errors="replace")
        finally:
            lib().tfcc_rocm_runtime_buffer_free(report)

    def step_count(self):
        n = C.c_size_t()
        check(lib().tfcc_rocm_runtime_model_step_count(self._h, C.byref(n)))
        return n.value

    def set_replay(self, enable):
        check(lib().tfcc_rocm_runtime_model_set_replay(self._h, 1 if enable else 0))

    def time(self, arrays, warmup=5, iters=20):
        """microseconds per run of the entrance graph alone, inputs resident on the device"""
        us = C.c_double()
        buf = modelfile.encode_inputs(arrays)
        check(lib().tfcc_rocm_runtime_model_time(self._h, buf, len(buf), warmup, iters, C.byref(us)))
        return us.value
