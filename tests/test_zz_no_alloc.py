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
    from streambrain_amd import _capi
    lib = _capi.lib()
    check(lib.sb_sync())
    before = lib.sb_allocation_calls()
    check(entry(d[0].ptr, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, tau, d[5].ptr, cthr, B, N, M))
    check(lib.sb_sync())
    allocated = lib.sb_allocation_calls() - before
    return (d[0].numpy(), d[1].numpy(), d[2].numpy(), d[5].numpy()), allocated


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
        # the entry point under test first: nothing the allocating one leaves behind can help it
        got, allocated = _run(lib.sb_update_weights_noalloc_f32, *p, tau, cthr)
        assert allocated == 0, f"{allocated} allocating runtime calls inside the no-alloc entry point"
        ref, _ = _run(lib.sb_update_weights_f32, *p, tau, cthr)
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


def test_noalloc_update_weights_at_the_largest_size_it_takes():
    """N + M == SB_NOALLOC_MAX_UNITS is accepted and uses the array to its last element: the new Cj of the last
    column comes back right."""
    from streambrain_amd import _capi
    from streambrain_amd._capi import DeviceArray, check
    _capi.init()
    lib = _capi.lib()
    f = np.float32
    N, M, B = 4, 262144 - 4, 3
    rng = np.random.default_rng(5)
    x, y = rng.random((B, N)).astype(f), rng.random((B, M)).astype(f)
    Ci, Cj = np.full(N, 0.5, f), np.full(M, 0.25, f)
    Cij, W = np.full((N, M), 0.125, f), np.zeros((N, M), f)
    d = [DeviceArray.from_numpy(a) for a in (Ci, Cj, Cij, x, y, W)]
    before = lib.sb_allocation_calls()
    check(lib.sb_update_weights_noalloc_f32(d[0].ptr, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, 1.0, d[5].ptr, 0.5,
                                            B, N, M))
    check(lib.sb_sync())
    assert lib.sb_allocation_calls() == before
    # taupdt = 1: the new traces are the batch means (sums in batch order, then / B)
    want_cj = ((y[0] + y[1]) + y[2]) / f(B)
    want_ci = ((x[0] + x[1]) + x[2]) / f(B)
    assert np.array_equal(d[1].numpy(), want_cj) and np.array_equal(d[0].numpy(), want_ci)


def test_noalloc_update_weights_is_refused_while_launches_are_bracketed():
    """Between sb_profile_start and sb_profile_stop every launch is bracketed by events the library creates, so
    the entry point that allocates nothing declines: SB_ERR_STATE, nothing launched."""
    from streambrain_amd import _capi
    from streambrain_amd._capi import check
    _capi.init()
    lib = _capi.lib()
    check(lib.sb_profile_start())
    try:
        rc = lib.sb_update_weights_noalloc_f32(None, None, None, None, None, 0.01, None, 0.005, 8, 16, 16)
        assert rc == -3  # SB_ERR_STATE
        assert b"sb_profile" in lib.sb_last_error()
    finally:
        check(lib.sb_profile_stop())
