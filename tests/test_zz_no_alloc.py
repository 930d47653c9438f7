"""sb_update_weights_noalloc_f32 (the entry point that allocates nothing: its intermediate traces live in
a static device array) against sb_update_weights_f32, through the C ABI: same arguments, bit-identical
results, on two calls in a row of which the second is smaller (the array keeps the first call's
contents), and a clear error beyond the array's size."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _problem(rng, B, N, M):
    f = np.float32
    x = (rng.random((B, N)) * (rng.random((B, N)) < 0.5)).astype(f)
    y = rng.random((B, M)).astype(f)
    Ci = (0.002 + 0.9 * rng.random(N)).astype(f)
    Cj = (0.002 + 0.9 * rng.random(M)).astype(f)
    Cij = (0.5 * rng.random((N, M)) * (rng.random((N, M)) < 0.9)).astype(f)
    W = np.full((N, M), 5.0, dtype=f)
    return x, y, Ci, Cj, Cij, W


def _run(entry, x, y, Ci, Cj, Cij, W, tau, cthr):
    from streambrain_amd._capi import DeviceArray, check
    B, N = x.shape
    M = y.shape[1]
    d = [DeviceArray.from_numpy(a) for a in (Ci, Cj, Cij, x, y, W)]
    check(entry(d[0].ptr, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, tau, d[5].ptr, cthr, B, N, M))
    return d[0].numpy(), d[1].numpy(), d[2].numpy(), d[5].numpy()


def test_noalloc_update_weights_matches_the_allocating_entry_point(oracle):
    from streambrain_amd import _capi
    _capi.init()
    lib = _capi.lib()
    tau = 0.01
    cthr = tau / 2
    rng = np.random.default_rng(77)
    # first a layer with several tile rows and columns, then a smaller one that leaves most of the
    # scratch array holding the first call's values
    for B, N, M in [(128, 1568, 3000), (37, 130, 70)]:
        print(f"noalloc case B={B} N={N} M={M}", flush=True)
        p = _problem(rng, B, N, M)
        ref = _run(lib.sb_update_weights_f32, *p, tau, cthr)
        got = _run(lib.sb_update_weights_noalloc_f32, *p, tau, cthr)
        for name, g, r in zip(("Ci", "Cj", "Cij", "W"), got, ref):
            assert np.array_equal(g, r), f"{name} differs from sb_update_weights_f32 at {(B, N, M)}"
        # and against the CPU restatement of the reference, like the allocating entry point's own test
        o = oracle.update_weights(p[2].copy(), p[3].copy(), p[4].copy(), p[0], p[1], tau, p[5].copy(), cthr)
        assert np.array_equal(got[0], o[0]) and np.array_equal(got[1], o[1])
        assert np.max(np.abs(got[2] - o[2]) / np.maximum(np.abs(o[2]), 1)) <= 1e-5
        assert np.max(np.abs(got[3] - o[3]) / np.maximum(np.abs(o[3]), 1)) <= 1e-5


def test_noalloc_update_weights_rejects_sizes_beyond_its_array():
    from streambrain_amd import _capi
    _capi.init()
    lib = _capi.lib()
    # the size check comes before anything touches the (here null) pointers
    rc = lib.sb_update_weights_noalloc_f32(None, None, None, None, None, 0.01, None, 0.005, 8, 262144, 1)
    assert rc == -4  # SB_ERR_UNSUPPORTED
    assert b"SB_NOALLOC_MAX_UNITS" in lib.sb_last_error()
