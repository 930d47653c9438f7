"""Size-independent checks at sizes the CPU oracle cannot reach: arrays with more than 2^31 elements
(64-bit indexing in the forward and training kernels), checked on sampled entries against closed forms
computed on the host in float64."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _slice_to_host(capi, lib, arr, first_elem, count, dtype):
    out = np.empty(count, dtype=dtype)
    capi.check(lib.sb_memcpy_d2h(out.ctypes.data, ctypes.c_void_p(int(arr.ptr) + first_elem * out.itemsize),
                                 out.nbytes))
    return out


def test_more_than_2_31_synapses_f32():
    from streambrain_amd import _capi
    from streambrain_amd._capi import DeviceArray
    _capi.init(0)
    lib = _capi.lib()
    B, N, H, Mc = 16, 33000, 656, 100
    M = H * Mc
    assert N * M > 2 ** 31
    rng = np.random.default_rng(11)
    tau, khalf, pmin, taubdt = 0.01, -100.0, 0.05, 0.02
    cthr = tau / 2
    x = (rng.random((B, N)) * (rng.random((B, N)) < 0.3)).astype(np.float32)
    y = rng.random((B, M)).astype(np.float32)
    y /= y.reshape(B, H, Mc).sum(axis=2).repeat(Mc, axis=1)
    ci = (0.05 + 0.3 * rng.random(N)).astype(np.float32)
    cj = np.full(M, 1.0 / Mc, dtype=np.float32)
    wmask = (rng.random((N, H)) < 0.5).astype(np.uint8)

    d_x, d_y = DeviceArray.from_numpy(x), DeviceArray.from_numpy(y)
    d_ci, d_cj = DeviceArray.from_numpy(ci), DeviceArray.from_numpy(cj)
    d_kbi, d_bias = DeviceArray.from_numpy(np.ones(M, np.float32)), DeviceArray.from_numpy(np.zeros(M, np.float32))
    d_m = DeviceArray.from_numpy(wmask)
    d_cij, d_w = DeviceArray((N, M), np.float32), DeviceArray((N, M), np.float32)
    # every byte 0x3a: the float 0x3a3a3a3a = 7.1e-4 in every entry of Cij and W
    c0 = float(np.frombuffer(bytes([0x3a] * 4), dtype=np.float32)[0])
    _capi.check(lib.sb_fill_bytes(d_cij.ptr, 0x3a, N * M * 4))
    _capi.check(lib.sb_fill_bytes(d_w.ptr, 0x3a, N * M * 4))

    # forward through the constant W: every logit of a row is c0 * sum(x[b]) -> uniform softmax
    d_act = DeviceArray((B, M), np.float32)
    _capi.check(lib.sb_compute_activation_f32(d_act.ptr, d_x.ptr, d_w.ptr, d_bias.ptr, B, N, H, Mc))
    act = d_act.numpy()
    assert np.max(np.abs(act - 1.0 / Mc)) <= 1e-5 / Mc * 10

    _capi.check(lib.sb_plastic_train_step_f32(d_w.ptr, d_bias.ptr, d_ci.ptr, d_cj.ptr, d_cij.ptr, d_kbi.ptr,
                                              d_m.ptr, d_x.ptr, d_y.ptr, B, N, H, Mc, tau, khalf, pmin, taubdt,
                                              -1))
    _capi.check(lib.sb_sync())
    ci_new = np.maximum(0, ci.astype(np.float64) * (1 - tau) + x.astype(np.float64).mean(axis=0) * tau)
    cj_new = np.maximum(0, cj.astype(np.float64) * (1 - tau) + y.astype(np.float64).mean(axis=0) * tau)
    assert np.max(np.abs(d_ci.numpy() - ci_new)) <= 1e-6 and np.max(np.abs(d_cj.numpy() - cj_new)) <= 1e-6
    # sampled rows: the first, some in the middle, the row that crosses element 2^31, the last
    rows = sorted({0, 1, N // 2, (2 ** 31) // M, (2 ** 31) // M + 1, N - 2, N - 1})
    for i in rows:
        cij_row = _slice_to_host(_capi, lib, d_cij, i * M, M, np.float32)
        w_row = _slice_to_host(_capi, lib, d_w, i * M, M, np.float32)
        ref_cij = np.maximum(0, c0 * (1 - tau) + (x[:, i].astype(np.float64) @ y.astype(np.float64)) / B * tau)
        ref_w = np.log(np.maximum(ref_cij, cthr ** 4) / (ci_new[i] * cj_new))
        ref_w[cj_new < cthr] = 0
        if ci_new[i] < cthr:
            ref_w[:] = 0
        ref_w *= np.repeat(wmask[i], Mc)
        assert np.max(np.abs(cij_row - ref_cij) / np.maximum(np.abs(ref_cij), 1)) <= 1e-5, f"Cij row {i}"
        assert np.max(np.abs(w_row - ref_w) / np.maximum(np.abs(ref_w), 1)) <= 2e-5, f"W row {i}"
