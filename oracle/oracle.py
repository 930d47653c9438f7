"""TEST INFRASTRUCTURE ONLY: ctypes front end of the CPU oracle (libbcpnn_oracle*.so).

The functions mirror the call signatures of the reference's kernel wrapper module
(BCPNN/backend/_kernels/kernels_openmp.py:6-99): numpy arrays in, the same arrays (updated in place)
out, dtype dispatch on float32/float64, "Invalid dtype" otherwise.

Only tests, the smoke test and the bench's cpu_baseline leg may import this module.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIBS = {}

_P = ctypes.c_void_p
_L = ctypes.c_long


def load(fast=False, path=None):
    """The strict build, the portable fast build, or (path) a library built elsewhere from the same source."""
    name = path or ("libbcpnn_oracle_fast.so" if fast else "libbcpnn_oracle.so")
    if name not in _LIBS:
        path = path or os.path.join(_HERE, name)
        if not os.path.exists(path):
            raise RuntimeError(f"{path} missing: run `python oracle/build.py`")
        lib = ctypes.CDLL(path)
        for sfx, R in (("_f32", ctypes.c_float), ("_f64", ctypes.c_double)):
            f = getattr(lib, "oracle_update_state" + sfx)
            f.argtypes = [_P, _P, _P, _P, _L, _L, _L]; f.restype = None
            f = getattr(lib, "oracle_softmax_minicolumns" + sfx)
            f.argtypes = [_P, _L, _L, _L]; f.restype = None
            f = getattr(lib, "oracle_update_weights" + sfx)
            f.argtypes = [R, _P, _P, _P, _P, _P, R, _L, _L, _L, _P, R]; f.restype = R
            f = getattr(lib, "oracle_update_bias" + sfx)
            f.argtypes = [_P, _P, R, _L]; f.restype = None
            f = getattr(lib, "oracle_update_bias_regularized" + sfx)
            f.argtypes = [_P, _P, _P, R, R, R, R, _L]; f.restype = None
            f = getattr(lib, "oracle_update_mask" + sfx)
            f.argtypes = [_P, _P, _P, _P, _P, R, _L, _L, _L, _L, _L, _L, _P, _P, _P, _P, _P]; f.restype = None
            f = getattr(lib, "oracle_apply_mask" + sfx)
            f.argtypes = [_P, _P, _L, _L, _L, _L]; f.restype = None
            f = getattr(lib, "oracle_argmax_rows" + sfx)
            f.argtypes = [_P, _L, _L, _P]; f.restype = None
        _LIBS[name] = lib
    return _LIBS[name]


def _sfx(dtype):
    if dtype == np.float64:
        return "_f64"
    if dtype == np.float32:
        return "_f32"
    raise Exception("Invalid dtype")


def _chk(a, dtype, name):
    if not isinstance(a, np.ndarray) or a.dtype != dtype or not a.flags.c_contiguous:
        raise ValueError(f"{name}: expected C-contiguous ndarray of {np.dtype(dtype)}")
    return a.ctypes.data


class Oracle:
    """One loaded build of the oracle (strict or fast-math)."""

    def __init__(self, fast=False, path=None):
        self.lib = load(fast, path)
        self.fast = fast or path is not None

    # kernels_openmp.py:6-13
    def update_state(self, state, weights, bias, inputs):
        d = state.dtype
        s = _sfx(d)
        B, N = inputs.shape
        M = weights.shape[1]
        assert weights.shape[0] == N and state.shape == (B, M) and bias.shape == (M,)
        getattr(self.lib, "oracle_update_state" + s)(
            _chk(state, d, "state"), _chk(inputs, d, "inputs"), _chk(weights, d, "weights"),
            _chk(bias, d, "bias"), B, N, M)
        return state

    # kernels_numpy.py:18-25 as bound by cpu_backend.py:10,24 (in place here)
    def softmax_minicolumns(self, a, hypercolumns, minicolumns):
        d = a.dtype
        s = _sfx(d)
        assert a.shape[1] == hypercolumns * minicolumns
        getattr(self.lib, "oracle_softmax_minicolumns" + s)(
            _chk(a, d, "a"), a.shape[0], hypercolumns, minicolumns)
        return a

    # kernels_openmp.py:16-25
    def update_weights(self, Ci, Cj, Cij, a_i, a_o, taupdt, weights, cthr):
        d = Ci.dtype
        s = _sfx(d)
        B, N = a_i.shape
        M = a_o.shape[1]
        assert a_o.shape[0] == B and Ci.shape == (N,) and Cj.shape == (M,)
        assert Cij.shape == (N, M) and weights.shape == (N, M)
        getattr(self.lib, "oracle_update_weights" + s)(
            1.0, _chk(Ci, d, "Ci"), _chk(Cj, d, "Cj"), _chk(Cij, d, "Cij"), _chk(a_i, d, "a_i"),
            _chk(a_o, d, "a_o"), taupdt, B, N, M, _chk(weights, d, "weights"), cthr)
        return Ci, Cj, Cij, weights

    # kernels_openmp.py:28-35
    def update_bias(self, bias, Cj, cthr):
        d = bias.dtype
        s = _sfx(d)
        getattr(self.lib, "oracle_update_bias" + s)(_chk(bias, d, "bias"), _chk(Cj, d, "Cj"), cthr,
                                                    bias.shape[0])
        return bias

    # kernels_openmp.py:38-47
    def update_bias_regularized(self, bias, kbi, Cj, cthr, khalf, pmin, taubdt):
        d = bias.dtype
        s = _sfx(d)
        getattr(self.lib, "oracle_update_bias_regularized" + s)(
            _chk(bias, d, "bias"), _chk(kbi, d, "kbi"), _chk(Cj, d, "Cj"), cthr, khalf, pmin, taubdt,
            bias.shape[0])
        return bias, kbi

    # kernels_openmp.py:50-87
    def update_mask(self, wmask, weights, Ci, Cj, Cij, cthr, hypercolumns, minicolumns, h,
                    iterations, trace=None):
        d = weights.dtype
        s = _sfx(d)
        N, M = weights.shape
        assert wmask.shape == (N, hypercolumns) and wmask.dtype == np.uint8
        assert M == hypercolumns * minicolumns and 0 <= h < hypercolumns
        swaps = vals = nsw = runner = stop = None
        if trace is not None:
            swaps = np.zeros([max(iterations, 1), 2], dtype=np.int64)
            vals = np.zeros([max(iterations, 1), 2], dtype=d)
            runner = np.zeros([max(iterations, 1), 2], dtype=d)
            stop = np.zeros([3], dtype=d)
            nsw = ctypes.c_long(0)
        getattr(self.lib, "oracle_update_mask" + s)(
            _chk(wmask, np.uint8, "wmask"), _chk(weights, d, "weights"), _chk(Ci, d, "Ci"),
            _chk(Cj, d, "Cj"), _chk(Cij, d, "Cij"), cthr, N, M, h, hypercolumns, minicolumns,
            iterations,
            swaps.ctypes.data if swaps is not None else None,
            vals.ctypes.data if vals is not None else None,
            ctypes.byref(nsw) if nsw is not None else None,
            runner.ctypes.data if runner is not None else None,
            stop.ctypes.data if stop is not None else None)
        if trace is not None:
            # per swap: the rows picked, their scores, the runners-up on either side (-3e38 / 3e38: none);
            # stop: (vmax0, vmin1) of the iteration that ended the loop by vmax0 < vmin1, or None
            trace["swaps"] = swaps[:nsw.value].copy()
            trace["vals"] = vals[:nsw.value].copy()
            trace["runner"] = runner[:nsw.value].copy()
            trace["stop"] = (float(stop[1]), float(stop[2])) if stop[0] != 0 else None
        return wmask

    # kernels_openmp.py:90-99
    def apply_mask(self, weights, wmask, hypercolumns, minicolumns):
        d = weights.dtype
        s = _sfx(d)
        N, M = weights.shape
        getattr(self.lib, "oracle_apply_mask" + s)(_chk(weights, d, "weights"),
                                                   _chk(wmask, np.uint8, "wmask"), N, M,
                                                   hypercolumns, minicolumns)
        return weights

    # _cpu_base_backend.py:239 (np.argmax over axis 1)
    def argmax_rows(self, act):
        d = act.dtype
        s = _sfx(d)
        out = np.zeros([act.shape[0]], dtype=np.int32)
        getattr(self.lib, "oracle_argmax_rows" + s)(_chk(act, d, "act"), act.shape[0], act.shape[1],
                                                    out.ctypes.data)
        return out
