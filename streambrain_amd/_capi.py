"""ctypes binding of libsbhip.so (the C ABI declared in include/sbhip.h).

Loading fails loudly when the library is missing: there is no CPU fallback of any kind.
"""
import ctypes
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libsbhip.so")

_P = ctypes.c_void_p
_L = ctypes.c_long
_I = ctypes.c_int
_Z = ctypes.c_size_t
_F = ctypes.c_float
_D = ctypes.c_double

# name -> argtypes for every exported entry point (restype is int unless listed in _RESTYPES)
_KERNEL_SIGS = {
    "sb_update_state": lambda R: [_P, _P, _P, _P, _L, _L, _L],
    "sb_softmax_minicolumns": lambda R: [_P, _L, _L, _L],
    "sb_compute_activation": lambda R: [_P, _P, _P, _P, _L, _L, _L, _L],
    "sb_compute_activation_rows": lambda R: [_P, _P, _P, _P, _P, _P, _L, _L, _L, _L, _L, _P],
    "sb_rows_in_blocks": lambda R: [_P, _P, _L, _L],
    "sb_update_weights": lambda R: [_P, _P, _P, _P, _P, R, _P, R, _L, _L, _L],
    "sb_update_counters": lambda R: [_P, _P, _P, _P, _P, R, _L, _L, _L],
    "sb_weights_from_counters": lambda R: [_P, _P, _P, _P, R, _L, _L],
    "sb_weights_masked_from_counters": lambda R: [_P, _P, _P, _P, _P, R, _L, _L, _L],
    "sb_add_bias": lambda R: [_P, _P, _L, _L],
    "sb_update_bias": lambda R: [_P, _P, R, _L],
    "sb_update_bias_regularized": lambda R: [_P, _P, _P, R, R, R, R, _L],
    "sb_update_mask": lambda R: [_P, _P, _P, _P, _P, R, _L, _L, _L, _L, _L],
    "sb_apply_mask": lambda R: [_P, _P, _L, _L, _L],
    "sb_argmax_rows": lambda R: [_P, _L, _L, _P],
    "sb_plastic_train_step": lambda R: [_P, _P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _L, _L, R, R, R,
                                        R, _L],
}
_PLAIN_SIGS = {
    "sb_init": [_I],
    "sb_shutdown": [],
    "sb_abi_version": [],
    "sb_sync": [],
    "sb_malloc": [ctypes.POINTER(_P), _Z],
    "sb_free": [_P],
    "sb_memcpy_h2d": [_P, _P, _Z],
    "sb_memcpy_d2h": [_P, _P, _Z],
    "sb_memcpy_d2d": [_P, _P, _Z],
    "sb_fill_bytes": [_P, _I, _Z],
    "sb_mask_rows": [_P, _P, _P, _L, _L, _L],
    "sb_update_weights_noalloc_f32": [_P, _P, _P, _P, _P, _F, _P, _F, _L, _L, _L],
    "sb_net_create": [ctypes.POINTER(_P), _I],
    "sb_net_destroy": [_P],
    "sb_net_add_dense_layer": [_P, _L, _L, _L, _D, _D, _D, _D],
    "sb_net_add_plastic_layer": [_P, _L, _L, _L, _D, _D, _D, _D, _D, _D, _D],
    "sb_net_randomize_layer": [_P, _I, ctypes.c_uint64, _D],
    "sb_net_set_layer_state": [_P, _I, ctypes.c_char_p, _P, _Z],
    "sb_net_get_layer_state": [_P, _I, ctypes.c_char_p, _P, _Z],
    "sb_net_set_frozen_cache_limit": [_P, _Z],
    "sb_net_set_training_data": [_P, _P, _P, _L, _L, _L],
    "sb_net_training_done": [_P],
    "sb_net_train_epoch": [_P, _I, _L, _P, _P, _L],
    "sb_net_train_batches": [_P, _I, _L, _P, _P, _L, _L, _L, _I],
    "sb_net_layer_activation": [_P, _I, _P, _L, _P],
    "sb_net_layer_train_step": [_P, _I, _P, _P, _L, _L],
    "sb_net_layer_train_finalize": [_P, _I],
    "sb_probe_mfma": [_I, _L, _L, ctypes.POINTER(_D)],
    "sb_profile_start": [],
    "sb_profile_stop": [],
    "sb_profile_kernels": [],
    "sb_profile_get": [_I, ctypes.POINTER(_D), ctypes.POINTER(_L)],
    "sb_net_evaluate": [_P, _P, _P, _L, _L, _L, _L, ctypes.POINTER(ctypes.c_int64),
                        ctypes.POINTER(ctypes.c_int64), _P],
    "sb_net_predict": [_P, _P, _L, _L, _L, _P],
    "sb_net_forward": [_P, _P, _L, _L, _I, _L, _P],
}
_RESTYPES = {"sb_last_error": ctypes.c_char_p, "sb_stream": _P, "sb_allocation_calls": _L}
_OTHER_SIGS = {"sb_profile_kernel_name": ([_I], ctypes.c_char_p),
               "sb_profile_kernel_carried": ([_I], _I),
               "sb_profile_bracket_overhead_us": ([], _D)}


def exported_symbols():
    """Every symbol include/sbhip.h declares."""
    names = list(_PLAIN_SIGS) + list(_RESTYPES) + list(_OTHER_SIGS)
    for base in _KERNEL_SIGS:
        names += [base + "_f32", base + "_f64"]
    return names


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing; build it with `python -m streambrain_amd.build` "
                "(there is no CPU fallback)")
        L = ctypes.CDLL(LIB_PATH)
        for name, args in _PLAIN_SIGS.items():
            f = getattr(L, name)
            f.argtypes = args
            f.restype = _I
        for name, res in _RESTYPES.items():
            f = getattr(L, name)
            f.argtypes = []
            f.restype = res
        for name, (args, res) in _OTHER_SIGS.items():
            f = getattr(L, name)
            f.argtypes = args
            f.restype = res
        for base, sig in _KERNEL_SIGS.items():
            for sfx, R in (("_f32", _F), ("_f64", _D)):
                f = getattr(L, base + sfx)
                f.argtypes = sig(R)
                f.restype = _I
        _lib = L
    return _lib


class SbError(RuntimeError):
    pass


def check(rc):
    if rc < 0:
        raise SbError(f"libsbhip status {rc}: {lib().sb_last_error().decode()}")
    return rc


_initialised = False


def init(device=0):
    global _initialised
    if not _initialised:
        check(lib().sb_init(device))
        _initialised = True


def suffix(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "_f32"
    if dtype == np.float64:
        return "_f64"
    raise Exception("Invalid dtype")


class DeviceArray:
    """A numpy-shaped buffer in HBM owned through sb_malloc / sb_free."""

    def __init__(self, shape, dtype):
        init()
        self.shape = tuple(int(s) for s in np.atleast_1d(shape)) if not isinstance(shape, tuple) else shape
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = _P()
        check(lib().sb_malloc(ctypes.byref(p), self.nbytes))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        check(lib().sb_memcpy_h2d(d.ptr, a.ctypes.data, d.nbytes))
        return d

    def numpy(self):
        out = np.empty(self.shape, dtype=self.dtype)
        check(lib().sb_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))
        return out

    def free(self):
        if self.ptr:
            check(lib().sb_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
