"""Size-independent checks at sizes the CPU oracle cannot reach: arrays with more than 2^31 elements
(64-bit indexing in the forward and training kernels), checked on sampled entries against closed forms
computed on the host in float64."""
import ctypes

import numpy as np
import pytest

from helpers import record_error

pytestmark = pytest.mark.gpu


def _slice_to_host(capi, lib, arr, first_elem, count, dtype):
    out = np.empty(count, dtype=dtype)
    capi.check(lib.sb_memcpy_d2h(out.ctypes.data, ctypes.c_void_p(int(arr.ptr) + first_elem * out.itemsize),
                                 out.nbytes))
    return out


def _rows_to_host(capi, lib, arr, rows, row_len, col0, ncols, dtype):
    """arr[rows, col0:col0+ncols] of a device matrix with row_len columns, one small copy per row."""
    out = np.empty((len(rows), ncols), dtype=dtype)
    for k, i in enumerate(rows):
        out[k] = _slice_to_host(capi, lib, arr, int(i) * row_len + col0, ncols, dtype)
    return out


def _check_layer_at_size(dtype, B, N, H, Mc, density, seed):
    """One forward and one fused training step at full size on seeded inputs, checked against closed
    forms evaluated on the host in float64 for sampled rows, and (sparse masks) the row-list forward
    kernel against the dense one and against the host for one hypercolumn."""
    from streambrain_amd import _capi
    from streambrain_amd._capi import DeviceArray
    _capi.init(0)
    lib = _capi.lib()
    sfx = "_f32" if dtype == np.float32 else "_f64"
    fn = lambda name: getattr(lib, name + sfx)
    es = np.dtype(dtype).itemsize
    tol = 1e-5 if dtype == np.float32 else 1e-12
    M = H * Mc
    rng = np.random.default_rng(seed)
    tau, khalf, pmin, taubdt = 0.01, -100.0, 0.05, 0.02
    cthr = tau / 2
    x = (rng.random((B, N), dtype=np.float32) * (rng.random((B, N), dtype=np.float32) < 0.3)).astype(dtype)
    y = rng.random((B, M), dtype=np.float32).astype(dtype)
    y /= y.reshape(B, H, Mc).sum(axis=2).repeat(Mc, axis=1)
    ci = (0.05 + 0.3 * rng.random(N)).astype(dtype)
    cj = np.full(M, 1.0 / Mc, dtype=dtype)
    wmask = (rng.random((N, H), dtype=np.float32) < density).astype(np.uint8)

    d_x, d_y = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y)
    d_ci, d_cj = DeviceArray.from_numpy(ci), DeviceArray.from_numpy(cj)
    d_kbi, d_bias = DeviceArray.from_numpy(np.ones(M, dtype)), DeviceArray.from_numpy(np.zeros(M, dtype))
    d_m = DeviceArray.from_numpy(wmask)
    d_cij, d_w = DeviceArray((N, M), dtype), DeviceArray((N, M), dtype)
    # the same byte everywhere: 0x3a3a3a3a = 7.1e-4 (float), 0x3f3f...3f = 4.8e-4 (double) in every entry
    byte = 0x3a if dtype == np.float32 else 0x3f
    c0 = float(np.frombuffer(bytes([byte] * es), dtype=dtype)[0])
    _capi.check(lib.sb_fill_bytes(d_cij.ptr, byte, N * M * es))
    _capi.check(lib.sb_fill_bytes(d_w.ptr, byte, N * M * es))

    # forward through the constant W: every logit of a row is c0 * sum(x[b]) -> uniform softmax
    d_act = DeviceArray((B, M), dtype)
    _capi.check(fn("sb_compute_activation")(d_act.ptr, d_x.ptr, d_w.ptr, d_bias.ptr, B, N, H, Mc))
    act = d_act.numpy()
    e_uniform = float(np.max(np.abs(act - 1.0 / Mc)))  # (|ref| < 1: the suite's metric is the absolute error)
    record_error("uniform softmax through a constant W", e_uniform, tol)
    assert e_uniform <= tol

    _capi.check(fn("sb_plastic_train_step")(d_w.ptr, d_bias.ptr, d_ci.ptr, d_cj.ptr, d_cij.ptr, d_kbi.ptr,
                                            d_m.ptr, d_x.ptr, d_y.ptr, B, N, H, Mc, tau, khalf, pmin, taubdt,
                                            -1))
    _capi.check(lib.sb_sync())
    ci_new = np.maximum(0, ci.astype(np.float64) * (1 - tau) + x.mean(axis=0, dtype=np.float64) * tau)
    cj_new = np.maximum(0, cj.astype(np.float64) * (1 - tau) + y.mean(axis=0, dtype=np.float64) * tau)
    assert np.max(np.abs(d_ci.numpy() - ci_new)) <= tol / 10 and np.max(np.abs(d_cj.numpy() - cj_new)) <= tol / 10

    def weights_of(i, cols):
        """Closed form of Cij[i, cols] and W[i, cols] after the step."""
        cij = np.maximum(0, c0 * (1 - tau) + (x[:, i].astype(np.float64) @ y[:, cols].astype(np.float64)) / B * tau)
        w = np.log(np.maximum(cij, cthr ** 4) / (ci_new[i] * cj_new[cols]))
        w[cj_new[cols] < cthr] = 0
        if ci_new[i] < cthr:
            w[:] = 0
        return cij, w * np.repeat(wmask[i], Mc)[cols]

    # sampled rows: the first, some in the middle, the row that crosses element 2^31 (if any), the last
    rows = sorted({0, 1, N // 2, min(N - 1, (2 ** 31) // M), min(N - 1, (2 ** 31) // M + 1), N - 2, N - 1})
    every = np.arange(M)
    for i in rows:
        cij_row = _slice_to_host(_capi, lib, d_cij, i * M, M, dtype)
        w_row = _slice_to_host(_capi, lib, d_w, i * M, M, dtype)
        ref_cij, ref_w = weights_of(i, every)
        e_cij = np.max(np.abs(cij_row - ref_cij) / np.maximum(np.abs(ref_cij), 1))
        e_w = np.max(np.abs(w_row - ref_w) / np.maximum(np.abs(ref_w), 1))
        record_error(f"Cij row {i}", e_cij, tol)
        record_error(f"W row {i}", e_w, tol)
        assert e_cij <= tol, f"Cij row {i}"
        assert e_w <= tol, f"W row {i}"

    # forward through the trained, masked W: one hypercolumn against the host (its W columns read back
    # for the connected rows and checked against the closed form), all of it dense kernel against
    # row-list kernel.  The input is scaled down so that sum |x w| of a logit is about 8: a softmax
    # output moves by about its own size times the error of its logit, which is up to eps * sum |x w|.
    h = H // 2
    cols = np.arange(h * Mc, (h + 1) * Mc)
    connected = np.flatnonzero(wmask[:, h])
    sample = connected[:: max(1, len(connected) // 2000)]
    got_w = _rows_to_host(_capi, lib, d_w, sample, M, h * Mc, Mc, dtype)
    for k in range(0, len(sample), max(1, len(sample) // 16)):
        ref_w = weights_of(sample[k], cols)[1]
        e_w = float(np.max(np.abs(got_w[k] - ref_w) / np.maximum(np.abs(ref_w), 1)))
        record_error(f"W of hypercolumn {h}, row {sample[k]}", e_w, tol)
        assert e_w <= tol
    bs = [0, B // 2, B - 1]
    terms = float((x[bs][:, sample].astype(np.float64) @ np.abs(got_w).astype(np.float64)).max())
    terms *= len(connected) / len(sample)
    xs = (x * dtype(8.0 / terms)).astype(dtype)
    d_xs = DeviceArray.from_numpy(xs)
    _capi.check(fn("sb_compute_activation")(d_act.ptr, d_xs.ptr, d_w.ptr, d_bias.ptr, B, N, H, Mc))
    act = d_act.numpy()
    assert np.allclose(act.reshape(B, H, Mc).sum(axis=2), 1.0, atol=100 * tol)
    bias = d_bias.numpy().astype(np.float64)
    if len(sample) == len(connected):  # the logits of the sampled hypercolumn, when all its rows were read
        logits = xs[bs][:, connected].astype(np.float64) @ got_w.astype(np.float64) + bias[cols]
        e = np.exp(logits - logits.max(axis=1, keepdims=True))
        ref = e / e.sum(axis=1, keepdims=True)
        record_error("activation vs host", np.max(np.abs(act[bs][:, cols] - ref)), tol)
        assert np.max(np.abs(act[bs][:, cols] - ref)) <= tol
    if density <= 0.5:
        cap = (int(np.count_nonzero(wmask, axis=0).max()) + 15) // 16 * 16 + 16
        d_rows, d_cnt = DeviceArray((H, cap), np.int32), DeviceArray((H,), np.int32)
        _capi.check(lib.sb_mask_rows(d_rows.ptr, d_cnt.ptr, d_m.ptr, N, H, cap))
        d_act2 = DeviceArray((B, M), dtype)
        _capi.check(fn("sb_compute_activation_rows")(d_act2.ptr, d_xs.ptr, d_w.ptr, d_bias.ptr, d_rows.ptr,
                                                     d_cnt.ptr, cap, B, N, H, Mc, None))
        assert np.array_equal(d_cnt.numpy(), np.count_nonzero(wmask, axis=0))
        record_error("rows vs dense", np.max(np.abs(d_act2.numpy() - act)), tol)
        assert np.max(np.abs(d_act2.numpy() - act)) <= tol
        # ... and the same from the inputs laid out in blocks of 16 rows
        d_xb = DeviceArray(((B + 15) // 16 * 16 * N,), dtype)
        _capi.check(fn("sb_rows_in_blocks")(d_xb.ptr, d_xs.ptr, B, N))
        _capi.check(lib.sb_fill_bytes(d_act2.ptr, 0, B * M * es))
        _capi.check(fn("sb_compute_activation_rows")(d_act2.ptr, d_xs.ptr, d_w.ptr, d_bias.ptr, d_rows.ptr,
                                                     d_cnt.ptr, cap, B, N, H, Mc, d_xb.ptr))
        record_error("blocked rows vs dense", np.max(np.abs(d_act2.numpy() - act)), tol)
        assert np.max(np.abs(d_act2.numpy() - act)) <= tol


def test_more_than_2_31_synapses_f32():
    _check_layer_at_size(np.float32, 16, 33000, 656, 100, 0.5, 11)
    assert 33000 * 65600 > 2 ** 31


def test_wide_layer_f64_full_size():
    """1568 inputs, 100 hypercolumns of 100, batch 512, float64, density 0.1."""
    _check_layer_at_size(np.float64, 512, 1568, 100, 100, 0.1, 12)


def test_stl10_shaped_layer_f32_full_size():
    """55296 inputs, 200 hypercolumns of 100, batch 256, float32, density 0.05 (4.4 GB per matrix)."""
    _check_layer_at_size(np.float32, 256, 55296, 200, 100, 0.05, 13)


def test_largest_layer_f32_full_size():
    """65536 inputs, 1000 hypercolumns of 100, batch 1024, float32, dense mask (26 GB per matrix)."""
    _check_layer_at_size(np.float32, 1024, 65536, 1000, 100, 1.0, 14)
