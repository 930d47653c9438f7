"""numpy-facing front end of the per-kernel C ABI entry points.

Same names, argument order and return values as the reference's kernel wrapper modules
(BCPNN/backend/_kernels/kernels_openmp.py:6-99, kernels_numpy.py:18-25): numpy arrays in, the updated
arrays out, dispatch on float32/float64, Exception("Invalid dtype") otherwise.  Every call copies its
operands to HBM, runs the kernel(s) through libsbhip.so and copies the results back, so this module is
for differential testing of single kernels -- training goes through the device-resident network
object (streambrain_amd.backend.hip_backend), which keeps all state in HBM.
"""
import numpy as np

from . import _capi
from ._capi import DeviceArray, check, lib, suffix


def _dev(a, dtype=None):
    a = np.ascontiguousarray(a if dtype is None else np.asarray(a, dtype=dtype))
    return DeviceArray.from_numpy(a)


def _fn(base, dtype):
    return getattr(lib(), base + suffix(dtype))


def _back(dst, dev):
    """Copy a device result into the caller's array (in-place semantics of the reference)."""
    np.copyto(dst, dev.numpy().reshape(dst.shape))
    return dst


def update_state(state, weights, bias, inputs):
    dt = state.dtype
    f = _fn("sb_update_state", dt)
    B, N = inputs.shape
    M = weights.shape[1]
    assert weights.shape == (N, M) and bias.shape == (M,) and state.shape == (B, M)
    d_act = DeviceArray((B, M), dt)
    d_x, d_w, d_b = _dev(inputs, dt), _dev(weights, dt), _dev(bias, dt)
    check(f(d_act.ptr, d_x.ptr, d_w.ptr, d_b.ptr, B, N, M))
    return _back(state, d_act)


def softmax_minicolumns(a, hypercolumns, minicolumns):
    dt = a.dtype
    f = _fn("sb_softmax_minicolumns", dt)
    assert a.shape[1] == hypercolumns * minicolumns
    d = _dev(a)
    check(f(d.ptr, a.shape[0], hypercolumns, minicolumns))
    return _back(a, d)


def compute_activation(weights, bias, inputs, hypercolumns, minicolumns):
    dt = weights.dtype
    f = _fn("sb_compute_activation", dt)
    B, N = inputs.shape
    M = hypercolumns * minicolumns
    assert weights.shape == (N, M) and bias.shape == (M,)
    d_act = DeviceArray((B, M), dt)
    d_x, d_w, d_b = _dev(inputs, dt), _dev(weights, dt), _dev(bias, dt)
    check(f(d_act.ptr, d_x.ptr, d_w.ptr, d_b.ptr, B, N, hypercolumns, minicolumns))
    return d_act.numpy()


def mask_rows(wmask):
    """Per-hypercolumn lists of the connected rows of wmask[N, H]: (rows[H, cap], counts[H]); rows holds
    ascending indices, then -1 up to cap."""
    wmask = np.ascontiguousarray(wmask, dtype=np.uint8)
    N, H = wmask.shape
    cap = (int(np.count_nonzero(wmask, axis=0).max(initial=0)) + 15) // 16 * 16 + 16
    d_rows = _dev(np.full((H, cap), -2, dtype=np.int32))
    d_cnt = DeviceArray((H,), np.int32)
    d_mask = _dev(wmask)  # kept alive until the results have been copied back
    check(lib().sb_mask_rows(d_rows.ptr, d_cnt.ptr, d_mask.ptr, N, H, cap))
    return d_rows.numpy(), d_cnt.numpy()


def rows_in_blocks(a):
    """a[rows, cols] in blocks of 16 rows, column-major inside a block; rows past the last one zero."""
    a = np.ascontiguousarray(a)
    rows, cols = a.shape
    d = DeviceArray(((rows + 15) // 16 * 16 * cols,), a.dtype)
    d_a = _dev(a)  # kept alive until the kernel has run (the stream is synchronised by the next copy)
    check(_fn("sb_rows_in_blocks", a.dtype)(d.ptr, d_a.ptr, rows, cols))
    check(lib().sb_sync())
    return d


def compute_activation_rows(weights, bias, inputs, wmask, hypercolumns, minicolumns, blocked=False):
    """compute_activation for weights that are zero wherever wmask is 0, over the connected rows only;
    blocked: the kernel reads the inputs from their copy in blocks of 16 rows."""
    dt = weights.dtype
    f = _fn("sb_compute_activation_rows", dt)
    B, N = inputs.shape
    M = hypercolumns * minicolumns
    assert weights.shape == (N, M) and bias.shape == (M,) and wmask.shape == (N, hypercolumns)
    rows, cnt = mask_rows(wmask)
    d_act = DeviceArray((B, M), dt)
    d_x, d_w, d_b = _dev(inputs, dt), _dev(weights, dt), _dev(bias, dt)
    d_rows, d_cnt = _dev(rows), _dev(cnt)
    d_xb = rows_in_blocks(np.asarray(inputs, dtype=dt)) if blocked else None
    check(f(d_act.ptr, d_x.ptr, d_w.ptr, d_b.ptr, d_rows.ptr, d_cnt.ptr, rows.shape[1], B, N,
            hypercolumns, minicolumns, d_xb.ptr if blocked else None))
    return d_act.numpy()


def add_bias(a, x):
    """a[b, :] += x  (kernels_cuda.py:18-26)"""
    dt = a.dtype
    B, M = a.shape
    assert x.shape == (M,)
    d_a, d_x = _dev(a), _dev(x, dt)
    check(_fn("sb_add_bias", dt)(d_a.ptr, d_x.ptr, B, M))
    return _back(a, d_a)


def update_counters(Ci, Cj, Cij, a_i, a_o, taupdt):
    """The trace half of update_weights on its own (kernels_cuda.py:40-48)."""
    dt = Ci.dtype
    B, N = a_i.shape
    M = a_o.shape[1]
    assert a_o.shape[0] == B and Ci.shape == (N,) and Cj.shape == (M,) and Cij.shape == (N, M)
    d_ci, d_cj, d_cij = _dev(Ci), _dev(Cj), _dev(Cij)
    d_x, d_y = _dev(a_i, dt), _dev(a_o, dt)
    check(_fn("sb_update_counters", dt)(d_ci.ptr, d_cj.ptr, d_cij.ptr, d_x.ptr, d_y.ptr, taupdt, B, N, M))
    return _back(Ci, d_ci), _back(Cj, d_cj), _back(Cij, d_cij)


def update_weights(*args):
    """Two call forms, told apart by their length:
    update_weights(Ci, Cj, Cij, a_i, a_o, taupdt, weights, cthr) -- traces and weights in one pass
        (kernels_openmp.py:18-25); returns (Ci, Cj, Cij, weights);
    update_weights(weights, Ci, Cj, Cij, cthr) -- the weights from the traces as they are
        (kernels_cuda.py:51-59); returns weights."""
    if len(args) == 5:
        weights, Ci, Cj, Cij, cthr = args
        dt = weights.dtype
        N, M = weights.shape
        assert Ci.shape == (N,) and Cj.shape == (M,) and Cij.shape == (N, M)
        d_w = DeviceArray((N, M), dt)
        d_ci, d_cj, d_cij = _dev(Ci, dt), _dev(Cj, dt), _dev(Cij, dt)  # kept alive until the copy back
        check(_fn("sb_weights_from_counters", dt)(d_w.ptr, d_ci.ptr, d_cj.ptr, d_cij.ptr, cthr, N, M))
        return _back(weights, d_w)
    Ci, Cj, Cij, a_i, a_o, taupdt, weights, cthr = args
    dt = Ci.dtype
    f = _fn("sb_update_weights", dt)
    B, N = a_i.shape
    M = a_o.shape[1]
    assert a_o.shape[0] == B and Ci.shape == (N,) and Cj.shape == (M,)
    assert Cij.shape == (N, M) and weights.shape == (N, M)
    d_ci, d_cj, d_cij, d_w = _dev(Ci), _dev(Cj), _dev(Cij), _dev(weights)
    d_x, d_y = _dev(a_i, dt), _dev(a_o, dt)
    check(f(d_ci.ptr, d_cj.ptr, d_cij.ptr, d_x.ptr, d_y.ptr, taupdt, d_w.ptr, cthr, B, N, M))
    return _back(Ci, d_ci), _back(Cj, d_cj), _back(Cij, d_cij), _back(weights, d_w)


def update_weights_masked(weights, Ci, Cj, Cij, cthr, wmask, hypercolumns, minicolumns):
    """The weights from the traces as they are, zero under zero mask bytes: update_weights(weights, Ci, Cj,
    Cij, cthr) followed by apply_mask(weights, wmask, hypercolumns, minicolumns) in one pass; returns weights."""
    dt = weights.dtype
    N, M = weights.shape
    assert M == hypercolumns * minicolumns and Ci.shape == (N,) and Cj.shape == (M,) and Cij.shape == (N, M)
    d_w = DeviceArray((N, M), dt)
    d_ci, d_cj, d_cij = _dev(Ci, dt), _dev(Cj, dt), _dev(Cij, dt)
    d_m = _dev(np.asarray(wmask).astype(np.uint8))
    assert d_m.shape == (N, hypercolumns)
    check(_fn("sb_weights_masked_from_counters", dt)(d_w.ptr, d_ci.ptr, d_cj.ptr, d_cij.ptr, d_m.ptr, cthr, N,
                                                     hypercolumns, minicolumns))
    return _back(weights, d_w)


def update_bias(bias, Cj, cthr):
    dt = bias.dtype
    f = _fn("sb_update_bias", dt)
    d_b, d_cj = _dev(bias), _dev(Cj, dt)
    check(f(d_b.ptr, d_cj.ptr, cthr, bias.shape[0]))
    return _back(bias, d_b)


def update_bias_regularized(bias, kbi, Cj, cthr, khalf, pmin, taubdt):
    dt = bias.dtype
    f = _fn("sb_update_bias_regularized", dt)
    d_b, d_k, d_cj = _dev(bias), _dev(kbi), _dev(Cj, dt)
    check(f(d_b.ptr, d_k.ptr, d_cj.ptr, cthr, khalf, pmin, taubdt, bias.shape[0]))
    return _back(bias, d_b), _back(kbi, d_k)


def update_mask(wmask, weights, Ci, Cj, Cij, cthr, hypercolumns, minicolumns, h, iterations):
    dt = weights.dtype
    f = _fn("sb_update_mask", dt)
    N, M = weights.shape
    assert wmask.shape == (N, hypercolumns) and wmask.dtype == np.uint8
    assert M == hypercolumns * minicolumns
    d_m = _dev(wmask)
    d_w, d_ci, d_cj, d_cij = _dev(weights), _dev(Ci, dt), _dev(Cj, dt), _dev(Cij, dt)
    check(f(d_m.ptr, d_w.ptr, d_ci.ptr, d_cj.ptr, d_cij.ptr, cthr, N, hypercolumns, minicolumns, h,
            iterations))
    return _back(wmask, d_m)


def apply_mask(weights, wmask, hypercolumns, minicolumns):
    dt = weights.dtype
    f = _fn("sb_apply_mask", dt)
    N, M = weights.shape
    assert M == hypercolumns * minicolumns
    d_w, d_m = _dev(weights), _dev(np.asarray(wmask).astype(np.uint8))
    check(f(d_w.ptr, d_m.ptr, N, hypercolumns, minicolumns))
    return _back(weights, d_w)


def argmax_rows(act):
    dt = act.dtype
    f = _fn("sb_argmax_rows", dt)
    B, M = act.shape
    d_a = _dev(act)
    d_p = DeviceArray((B,), np.int32)
    check(f(d_a.ptr, B, M, d_p.ptr))
    return d_p.numpy()


def plastic_train_step(state, inputs, outputs, hypercolumns, minicolumns, taupdt, khalf, pmin, taubdt,
                       hypercolumn=None):
    """One StructuralPlasticityLayer.train_step (cpu_backend.py:29-52) on a dict of numpy state arrays
    {weights, bias, Ci, Cj, Cij, kbi, wmask}; returns the updated dict."""
    dt = state["weights"].dtype
    f = _fn("sb_plastic_train_step", dt)
    B, N = inputs.shape
    names = ("weights", "bias", "Ci", "Cj", "Cij", "kbi", "wmask")
    dev = {k: _dev(state[k]) for k in names}
    d_x, d_y = _dev(inputs, dt), _dev(outputs, dt)
    check(f(*(dev[k].ptr for k in names), d_x.ptr, d_y.ptr, B, N, hypercolumns, minicolumns, taupdt,
            khalf, pmin, taubdt, -1 if hypercolumn is None else int(hypercolumn)))
    return {k: dev[k].numpy() for k in names}


def sync():
    _capi.init()
    check(lib().sb_sync())
