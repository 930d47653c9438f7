"""GPU parity of every per-kernel C ABI entry point against the CPU oracle on the same seeded inputs.

Tolerance (floating point): |gpu - ref| <= tol * max(|ref|, 1) with tol = 1e-5 (float32) and 1e-12
(float64); masks, class labels and everything integer are compared bit for bit.
"""
import numpy as np
import pytest

from helpers import record_error

pytestmark = pytest.mark.gpu

DT = [np.float32, np.float64]
TOL = {np.float32: 1e-5, np.float64: 1e-12}


def err(a, ref):
    a = np.asarray(a, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(a - ref) / np.maximum(np.abs(ref), 1.0))) if a.size else 0.0


def assert_close(a, ref, dtype, what, scale=1.0):
    e = err(a, ref)
    record_error(what, e, scale * TOL[dtype])
    assert e <= scale * TOL[dtype], f"{what}: error {e:.3e} > {scale * TOL[dtype]:.1e}"


@pytest.fixture(scope="module")
def k():
    from streambrain_amd import kernels_hip
    return kernels_hip


SHAPES = [(1, 1, 1), (3, 5, 7), (16, 64, 64), (17, 33, 65), (128, 257, 130), (96, 1568, 300)]


# ------------------------------------------------------------------------------------ update_state
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,N,M", SHAPES)
def test_update_state(k, oracle, dtype, B, N, M):
    rng = np.random.default_rng(B * 7 + N * 3 + M)
    x = rng.random((B, N)).astype(dtype)
    W = (0.1 * rng.standard_normal((N, M))).astype(dtype)
    b = (0.1 * rng.random(M)).astype(dtype)
    got = k.update_state(np.full((B, M), 3.0, dtype=dtype), W, b, x)
    exact = x.astype(np.float64) @ W.astype(np.float64) + b.astype(np.float64)
    ref = oracle.update_state(np.zeros((B, M), dtype=dtype), W, b, x)
    # both implementations accumulate N products in REAL in different orders; each is held to the
    # tolerance against the float64 product of the same inputs, and they are held to it against each other
    assert_close(got, exact, dtype, "gpu vs exact")
    assert_close(ref, exact, dtype, "oracle vs exact")
    assert_close(got, ref, dtype, "gpu vs oracle")


# ------------------------------------------------------------- forward over the connected rows only
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("rows,cols", [(1, 1), (16, 5), (37, 300), (50, 302), (128, 1568)])
def test_rows_in_blocks(k, dtype, rows, cols):
    rng = np.random.default_rng(rows + cols)
    a = rng.random((rows, cols)).astype(dtype)
    got = k.rows_in_blocks(a).numpy()
    nb = (rows + 15) // 16
    want = np.zeros((nb * 16, cols), dtype=dtype)
    want[:rows] = a
    want = want.reshape(nb, 16, cols).transpose(0, 2, 1).reshape(-1)
    assert np.array_equal(got, want)



@pytest.mark.parametrize("N,H,density", [(1, 1, 1.0), (40, 3, 0.3), (1568, 30, 0.1), (300, 5, 0.0),
                                         (257, 4, 0.05), (64, 2, 1.0)])
def test_mask_rows(k, N, H, density):
    rng = np.random.default_rng(N + H)
    wmask = (rng.random((N, H)) < density).astype(np.uint8)
    if N > 100:
        wmask[:, 1] = 0  # an unconnected hypercolumn
    rows, cnt = k.mask_rows(wmask)
    for h in range(H):
        want = np.flatnonzero(wmask[:, h])
        assert cnt[h] == want.size
        assert np.array_equal(rows[h, :want.size], want)
        assert np.all(rows[h, want.size:] == -1)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,N,H,Mc,density", [(128, 1568, 30, 100, 0.1), (96, 1568, 30, 100, 0.1),
                                              (7, 40, 3, 12, 0.3), (33, 300, 2, 200, 0.2),
                                              (16, 64, 2, 64, 1.0), (20, 100, 2, 256, 0.05),
                                              (5, 50, 3, 12, 0.0), (300, 5000, 4, 100, 0.4),
                                              (20, 6000, 2, 64, 0.5),  # lists longer than one LDS segment
                                              # many tiles: 32 and 64 batch rows per workgroup, ragged
                                              (1000, 300, 32, 100, 0.2), (2030, 200, 64, 100, 0.3),
                                              (12, 40, 2, 224, 0.5),
                                              # many hypercolumns: narrow (12 columns) and full (128) ones, a
                                              # ragged batch, lists longer than one LDS segment
                                              (130, 300, 260, 12, 0.3), (256, 400, 140, 128, 0.2),
                                              (128, 5000, 260, 12, 0.5)])
@pytest.mark.parametrize("blocked", [False, True])
def test_compute_activation_rows(k, oracle, dtype, B, N, H, Mc, density, blocked):
    """The row-list forward kernel against the dense reference computation on the masked weights."""
    rng = np.random.default_rng(B + N + H + Mc)
    M = H * Mc
    wmask = (rng.random((N, H)) < density).astype(np.uint8)
    x = rng.random((B, N)).astype(dtype)
    W = (0.1 * rng.standard_normal((N, M))).astype(dtype) * np.repeat(wmask, Mc, axis=1).astype(dtype)
    b = (0.1 * rng.random(M)).astype(dtype)
    if (dtype == np.float32 and Mc % 4) or (dtype == np.float64 and Mc > 224):
        # outside the kernel's shapes (float32: minicolumns divisible by 4; float64: at most 224 per
        # hypercolumn): the entry point says so, and the network takes the dense kernel for such a layer
        from streambrain_amd._capi import SbError
        with pytest.raises(SbError, match="not supported"):
            k.compute_activation_rows(W, b, x, wmask, H, Mc, blocked=blocked)
        return
    got = k.compute_activation_rows(W, b, x, wmask, H, Mc, blocked=blocked)
    ref = oracle.update_state(np.zeros((B, M), dtype=dtype), W, b, x)
    ref = oracle.softmax_minicolumns(ref, H, Mc)
    assert_close(got, ref, dtype, "gpu vs oracle")
    assert np.allclose(got.reshape(B, H, Mc).sum(2), 1.0, atol=100 * TOL[dtype])
    # and the dense kernel on the same operands
    assert_close(got, k.compute_activation(W, b, x, H, Mc), dtype, "rows vs dense")


# ----------------------------------------------------------------------------------------- softmax
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,H,Mc", [(1, 1, 1), (5, 3, 7), (128, 30, 100), (9, 2, 300), (4, 1, 10)])
def test_softmax_minicolumns(k, oracle, dtype, B, H, Mc):
    rng = np.random.default_rng(B + H + Mc)
    a = (4 * rng.standard_normal((B, H * Mc))).astype(dtype)
    got = k.softmax_minicolumns(a.copy(), H, Mc)
    ref = oracle.softmax_minicolumns(a.copy(), H, Mc)
    assert_close(got, ref, dtype, "softmax")
    assert np.allclose(got.reshape(B, H, Mc).sum(2), 1.0, atol=100 * TOL[dtype])


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,N,H,Mc", [(1, 1, 1, 1), (7, 13, 3, 5), (128, 1568, 30, 100),
                                      (96, 1568, 30, 100), (33, 300, 2, 200), (20, 100, 2, 256),
                                      (16, 64, 2, 300), (40, 3000, 1, 10), (10, 50, 3, 66),
                                      (12, 40, 2, 224),
                                      # many tiles: 32 and 64 batch rows per workgroup, ragged last tile
                                      (1000, 44, 32, 100), (2030, 36, 64, 100)])
def test_compute_activation_fused(k, oracle, dtype, B, N, H, Mc):
    rng = np.random.default_rng(B + N + H + Mc)
    M = H * Mc
    x = rng.random((B, N)).astype(dtype)
    W = (0.1 * rng.standard_normal((N, M))).astype(dtype)
    b = (0.1 * rng.random(M)).astype(dtype)
    got = k.compute_activation(W, b, x, H, Mc)
    ref = oracle.update_state(np.zeros((B, M), dtype=dtype), W, b, x)
    ref = oracle.softmax_minicolumns(ref, H, Mc)
    exact = x.astype(np.float64) @ W.astype(np.float64) + b.astype(np.float64)
    exact = np.exp(exact - exact.reshape(B, H, Mc).max(2, keepdims=True).repeat(Mc, 2).reshape(B, M))
    exact = exact / exact.reshape(B, H, Mc).sum(2, keepdims=True).repeat(Mc, 2).reshape(B, M)
    assert_close(got, exact, dtype, "gpu vs exact")
    assert_close(got, ref, dtype, "gpu vs oracle")


# -------------------------------------------------------------------------- update_weights (fused)
def _trace_problem(rng, B, N, M, dtype):
    x = (rng.random((B, N)) * (rng.random((B, N)) < 0.5)).astype(dtype)
    y = rng.random((B, M)).astype(dtype)
    Ci = (0.002 + 0.9 * rng.random(N)).astype(dtype)
    Cj = (0.002 + 0.9 * rng.random(M)).astype(dtype)
    Cij = (0.5 * rng.random((N, M)) * (rng.random((N, M)) < 0.9)).astype(dtype)
    return x, y, Ci, Cj, Cij


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,N,M", SHAPES + [(128, 1568, 3000), (5, 130, 70), (1024, 64, 64),
                                           # batch of x above 2 MiB: tiles walked in panels of 16 tile
                                           # columns (11 and 8 tile columns: one narrow panel; 18: a full one
                                           # and a rest), of 8 for batches beyond 512 rows (10 tile columns)
                                           (64, 8300, 700), (48, 5600, 512), (64, 8300, 1100), (520, 1100, 600),
                                           # 150 x 141 tiles: the traces come from their own launch (one
                                           # turn of two chunks; two turns; a loop turn ahead of them; that
                                           # launch's blocks of 64 batch rows: a ragged second, four)
                                           (8, 9600, 9000), (40, 9600, 9000), (72, 7040, 6016), (200, 7040, 6016)])
def test_update_weights(k, oracle, dtype, B, N, M):
    rng = np.random.default_rng(B + 2 * N + 3 * M)
    x, y, Ci, Cj, Cij = _trace_problem(rng, B, N, M, dtype)
    tau = 0.01
    cthr = tau / 2  # a few Ci / Cj fall below it: zeroed rows and columns are exercised
    W = np.full((N, M), 5.0, dtype=dtype)
    g = k.update_weights(Ci.copy(), Cj.copy(), Cij.copy(), x, y, tau, W.copy(), cthr)
    r = oracle.update_weights(Ci.copy(), Cj.copy(), Cij.copy(), x, y, tau, W.copy(), cthr)
    # Ci and Cj follow the reference's summation order exactly
    assert np.array_equal(g[0], r[0]), "Ci not bit-exact"
    assert np.array_equal(g[1], r[1]), "Cj not bit-exact"
    assert_close(g[2], r[2], dtype, "Cij")
    assert_close(g[3], r[3], dtype, "W")
    # zeros where the reference has zeros (dead rows and columns).  Among 86 million weights one or two
    # have a logarithm argument within an ulp of 1, where one side's log gives exactly 0 and the other's
    # a value of that last ulp: those are differences inside the tolerance, not of the zero pattern
    differ = (g[3] == 0) != (r[3] == 0)
    record_error(f"W entries whose zero pattern differs ({N} x {M})", int(differ.sum()), 4)
    assert differ.sum() <= 4 and np.all(np.abs(g[3][differ]) + np.abs(r[3][differ]) <= 1e-6), differ.sum()


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B", [1, 7, 8, 9, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 96, 100, 129])
def test_fused_training_pass_at_batch_sizes_around_its_chunks(k, oracle, dtype, B):
    """The fused kernel walks the batch two chunks of 16 (fp64: 8) rows per turn, the last turn padded with
    zero rows, and requests the Cij tile a fixed number of chunks before the end: batch sizes on either side
    of every boundary that schedule has (one turn, two turns, a half-filled last turn, a single row).
    Traces bit for bit, Cij and W at the stated tolerance, W's zeros where the reference has them."""
    rng = np.random.default_rng(1000 + B)
    N, M = 131, 212
    x, y, Ci, Cj, Cij = _trace_problem(rng, B, N, M, dtype)
    tau = 0.01
    cthr = tau / 2
    r = oracle.update_weights(Ci.copy(), Cj.copy(), Cij.copy(), x, y, tau, np.zeros((N, M), dtype=dtype), cthr)
    g = k.update_weights(Ci.copy(), Cj.copy(), Cij.copy(), x, y, tau, np.zeros((N, M), dtype=dtype), cthr)
    assert np.array_equal(g[0], r[0]) and np.array_equal(g[1], r[1])
    assert_close(g[2], r[2], dtype, "Cij")
    assert_close(g[3], r[3], dtype, "W")
    assert np.array_equal(g[3] == 0, r[3] == 0)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,N,M", [(5, 7, 9), (128, 257, 130), (96, 1568, 300), (33, 300, 10), (20, 37, 1032),
                                   (16, 203, 3000)])
def test_update_counters_then_weights(k, oracle, dtype, B, N, M):
    """The two halves of update_weights called one after the other (the cuda kernel set's form) give what
    the fused call gives: traces from update_counters, weights from update_weights(weights, Ci, Cj, Cij,
    cthr)."""
    rng = np.random.default_rng(3 * B + N + M)
    x, y, Ci, Cj, Cij = _trace_problem(rng, B, N, M, dtype)
    tau = 0.01
    cthr = tau / 2
    r = oracle.update_weights(Ci.copy(), Cj.copy(), Cij.copy(), x, y, tau, np.zeros((N, M), dtype=dtype), cthr)
    ci, cj, cij = k.update_counters(Ci.copy(), Cj.copy(), Cij.copy(), x, y, tau)
    assert np.array_equal(ci, r[0]) and np.array_equal(cj, r[1])
    assert_close(cij, r[2], dtype, "Cij")
    W = k.update_weights(np.full((N, M), 5.0, dtype=dtype), ci, cj, cij, cthr)
    assert_close(W, r[3], dtype, "W")
    assert np.array_equal(W == 0, r[3] == 0)
    # and bit for bit what the fused kernel computes from the same traces
    g = k.update_weights(Ci.copy(), Cj.copy(), Cij.copy(), x, y, tau, np.zeros((N, M), dtype=dtype), cthr)
    assert np.array_equal(g[2], cij) and np.array_equal(g[3], W)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("N,H,Mc,density", [(5, 3, 4, 0.5), (37, 5, 12, 0.3), (130, 1, 64, 0.5), (257, 2, 65, 0.4),
                                            (203, 7, 6, 0.0), (203, 7, 6, 1.0), (1568, 30, 100, 0.1)])
def test_weights_masked_from_counters(k, oracle, dtype, N, H, Mc, density):
    """The weight pass with the mask apply fused in (kernels_openmp_internal.cc:192-199 then :322-335 of the
    reference) against the CPU restatement's two calls, and bit for bit against the GPU's own two calls."""
    rng = np.random.default_rng(N + 31 * H + Mc)
    M = H * Mc
    x, y, Ci, Cj, Cij = _trace_problem(rng, 4, N, M, dtype)
    cthr = 0.005
    wmask = (rng.random((N, H)) < density).astype(np.uint8)
    # taupdt = 0 leaves the traces as they are: the restatement's update_weights then is the weight pass alone
    ref = oracle.update_weights(Ci.copy(), Cj.copy(), Cij.copy(), x, y, 0.0, np.zeros((N, M), dtype=dtype), cthr)
    assert np.array_equal(ref[0], Ci) and np.array_equal(ref[2], Cij)
    ref_w = oracle.apply_mask(ref[3].copy(), wmask, H, Mc)
    got = k.update_weights_masked(np.full((N, M), 5.0, dtype=dtype), Ci, Cj, Cij, cthr, wmask, H, Mc)
    assert_close(got, ref_w, dtype, "masked W")
    assert np.array_equal(got == 0, ref_w == 0)
    two = k.apply_mask(k.update_weights(np.full((N, M), 5.0, dtype=dtype), Ci, Cj, Cij, cthr), wmask, H, Mc)
    assert np.array_equal(got, two)


def test_weight_logarithm_f64_within_two_ulp(k):
    """The double-precision weight pass evaluates its logarithm with a short routine of the library's own
    (argument reduction, degree-7 polynomial, hardware reciprocal) instead of the runtime's.  With Ci = Cj = 1 a
    weight is log(max(Cij, cthr^4)): arguments over 60 binades, close to 1 (where the result cancels to nearly
    nothing), at and around powers of two and the reduction's switch at sqrt(1/2), checked against an 80-bit
    logarithm rounded to double.  Measured: 0.75 ulp on the CPU restatement of the same routine."""
    rng = np.random.default_rng(99)
    n = 1 << 18
    arg = np.concatenate([
        np.exp((rng.random(n) - 0.5) * 40.0),
        1.0 + (rng.random(n) - 0.5) * 0.6,
        1.0 + (rng.random(n) - 0.5) * 1e-6,
        np.ldexp(np.sqrt(0.5) * (1.0 + (rng.random(n) - 0.5) * 1e-9), rng.integers(-20, 20, n)),
        np.ldexp(1.0, np.arange(-30, 31)).repeat(3) * np.tile([1 - 2.0 ** -53, 1.0, 1 + 2.0 ** -52], 61),
    ])
    M = 1024
    pad = (-len(arg)) % M
    arg = np.concatenate([arg, np.ones(pad)]).reshape(-1, M)
    N = arg.shape[0]
    cthr = 1e-3  # cthr^4 = 1e-12, below every argument
    assert arg.min() > cthr ** 4
    W = k.update_weights(np.zeros((N, M)), np.ones(N), np.ones(M), arg, cthr)
    ref = np.log(arg.astype(np.longdouble))
    ulp = np.spacing(np.abs(ref.astype(np.float64))).astype(np.longdouble)
    err = float(np.max(np.abs(W.astype(np.longdouble) - ref) / ulp))
    record_error("fp64 weight logarithm, ulp", err, 2.0)
    assert err <= 2.0
    assert np.all(W[arg == 1.0] == 0.0)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,M", [(1, 1), (7, 33), (128, 3000)])
def test_add_bias(k, dtype, B, M):
    rng = np.random.default_rng(B + M)
    a = rng.standard_normal((B, M)).astype(dtype)
    b = rng.standard_normal(M).astype(dtype)
    assert np.array_equal(k.add_bias(a.copy(), b), a + b[None, :])


# -------------------------------------------------------------------------------------------- bias
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("M", [1, 10, 3000])
def test_update_bias(k, oracle, dtype, M):
    rng = np.random.default_rng(M)
    Cj = (rng.random(M) * (rng.random(M) < 0.8)).astype(dtype)
    got = k.update_bias(np.zeros(M, dtype=dtype), Cj, 0.01)
    ref = oracle.update_bias(np.zeros(M, dtype=dtype), Cj, 0.01)
    assert_close(got, ref, dtype, "bias")


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("M", [1, 10, 3000])
def test_update_bias_regularized(k, oracle, dtype, M):
    rng = np.random.default_rng(M + 1)
    Cj = (rng.random(M) * (rng.random(M) < 0.8)).astype(dtype)
    kbi = (1 + rng.standard_normal(M)).astype(dtype)
    args = (0.0035, -139.02586632856327, 0.06195283356566607, 0.02218100432360414)
    gb, gk = k.update_bias_regularized(np.zeros(M, dtype=dtype), kbi.copy(), Cj, *args)
    rb, rk = oracle.update_bias_regularized(np.zeros(M, dtype=dtype), kbi.copy(), Cj, *args)
    assert np.array_equal(gk, rk), "kbi is plain IEEE arithmetic and must be bit-exact"
    assert_close(gb, rb, dtype, "bias")


# -------------------------------------------------------------------------------------------- mask
def _mask_problem(rng, N, H, Mc, dtype, density=0.1):
    M = H * Mc
    wmask = (rng.random((N, H)) < density).astype(np.uint8)
    W = (0.1 * rng.standard_normal((N, M))).astype(dtype)
    Ci = (0.05 + 0.9 * rng.random(N)).astype(dtype)
    Cj = (0.05 + 0.9 * rng.random(M)).astype(dtype)
    Cij = np.minimum(np.minimum(0.9 * Ci[:, None], 0.9 * Cj[None, :]), rng.random((N, M))).astype(dtype)
    return wmask, W, Ci, Cj, Cij


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("N,H,Mc", [(1, 1, 2), (7, 2, 3), (128, 5, 20), (1568, 30, 100), (5000, 3, 4), (9000, 2, 3),
                                    (20000, 2, 3), (40000, 2, 3), (70000, 1, 2)])
@pytest.mark.parametrize("iterations", [0, 1, 16])
def test_update_mask_bit_exact(k, oracle, dtype, N, H, Mc, iterations):
    rng = np.random.default_rng(N + H + Mc)
    wmask, W, Ci, Cj, Cij = _mask_problem(rng, N, H, Mc, dtype)
    h = int(rng.integers(0, H))
    trace = {}
    ref = oracle.update_mask(wmask.copy(), W, Ci, Cj, Cij, 0.01, H, Mc, h, iterations, trace=trace)
    got = k.update_mask(wmask.copy(), W, Ci, Cj, Cij, 0.01, H, Mc, h, iterations)
    assert np.array_equal(got, ref), f"masks differ in {(got != ref).sum()} entries, swaps {trace['swaps']}"
    assert got[:, h].sum() == wmask[:, h].sum()


@pytest.mark.parametrize("dtype", DT)
def test_update_mask_ties_and_degenerate_columns(k, oracle, dtype):
    # all scores equal: last silent row on, last active row off
    wm = np.zeros((6, 1), dtype=np.uint8); wm[[1, 3], 0] = 1
    Ci = np.full(6, 1e-4, dtype=dtype); Cj = np.full(3, 0.3, dtype=dtype)
    Cij = np.full((6, 3), 1e-5, dtype=dtype); W = np.zeros((6, 3), dtype=dtype)
    got = k.update_mask(wm.copy(), W, Ci, Cj, Cij, 0.01, 1, 3, 0, 1)
    assert got[:, 0].tolist() == [0, 1, 0, 0, 0, 1]
    rng = np.random.default_rng(4)
    wmask, W, Ci, Cj, Cij = _mask_problem(rng, 40, 2, 3, dtype, density=0.4)
    for fill in (0, 1):
        w2 = wmask.copy(); w2[:, 1] = fill
        assert np.array_equal(k.update_mask(w2.copy(), W, Ci, Cj, Cij, 0.01, 2, 3, 1, 16), w2)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("N,H,Mc", [(1568, 30, 100), (300, 4, 10), (6000, 3, 8), (12000, 2, 4), (50000, 2, 4)])
@pytest.mark.parametrize("kind", ["dead_rows", "near_equal", "identical_rows", "few_active", "few_silent"])
def test_update_mask_tie_blocks(k, oracle, dtype, N, H, Mc, kind):
    """Score distributions that stress the candidate preselection of the swap loop: large blocks of
    exactly equal scores (dead inputs score 0), many nearly equal scores, tiny groups."""
    rng = np.random.default_rng(N + len(kind))
    wmask, W, Ci, Cj, Cij = _mask_problem(rng, N, H, Mc, dtype, density=0.3)
    h = 1
    if kind == "dead_rows":
        dead = rng.random(N) < 0.6
        Ci[dead] = 0.001  # below cthr: nominator 0, score 0 whatever csum is
    elif kind == "near_equal":
        Ci[:] = 0.4
        # distinct scores, 2e-6 apart (relative): far above rounding noise, far below the preselection's
        # resolution, so dozens of rows share the threshold bucket
        Cij[:] = (Cij[0:1, :] * (1 + 2e-6 * rng.permutation(N)[:, None])).astype(dtype)
        W[:] = W[0:1, :]
    elif kind == "identical_rows":
        Ci[:] = 0.4
        Cij[:] = Cij[0:1, :]
        W[:] = W[0:1, :]
        wmask[:] = 0
        wmask[rng.random(N) < 0.3, h] = 1  # equal csum inside each group: all scores of a group tie
    elif kind == "few_active":
        wmask[:, h] = 0
        wmask[rng.choice(N, 5, replace=False), h] = 1
    elif kind == "few_silent":
        wmask[:, h] = 1
        wmask[rng.choice(N, 7, replace=False), h] = 0
    trace = {}
    ref = oracle.update_mask(wmask.copy(), W, Ci, Cj, Cij, 0.01, H, Mc, h, 16, trace=trace)
    got = k.update_mask(wmask.copy(), W, Ci, Cj, Cij, 0.01, H, Mc, h, 16)
    assert np.array_equal(got, ref), f"masks differ in {(got != ref).sum()} entries, swaps {trace['swaps']}"


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("N", [24, 700, 3000])
def test_update_mask_nan_scores(k, oracle, dtype, N):
    """Rows with Ci = 1 and Cij = Cj give 0 * log(x/0) = NaN nominators.  The reference's sequential
    `>=` / `<=` scan lets a NaN win only when it is the first candidate of its group; the strict-IEEE
    oracle restates exactly that, and the GPU reduction has to reproduce it bit for bit."""
    rng = np.random.default_rng(N)
    H, Mc = 3, 4
    wmask, W, Ci, Cj, Cij = _mask_problem(rng, N, H, Mc, dtype, density=0.3)
    for case in range(6):
        ci, cij, wm = Ci.copy(), Cij.copy(), wmask.copy()
        bad = rng.choice(N, size=max(2, N // 10), replace=False)
        if case % 3 == 1:
            bad[0] = 0  # a NaN on the very first row
        if case % 3 == 2:
            first_active = int(np.flatnonzero(wm[:, 1])[0])
            bad[0] = first_active  # a NaN on the first active row
        ci[bad] = 1.0
        cij[bad, :] = Cj[None, :]
        trace = {}
        ref = oracle.update_mask(wm.copy(), W, ci, Cj, cij, 0.01, H, Mc, 1, 16, trace=trace)
        got = k.update_mask(wm.copy(), W, ci, Cj, cij, 0.01, H, Mc, 1, 16)
        assert np.array_equal(got, ref), f"case {case}: masks differ in {(got != ref).sum()} entries, " \
                                         f"swaps {trace['swaps']}"


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("N,H,Mc", [(1, 1, 1), (13, 4, 5), (1568, 30, 100), (100, 7, 9), (37, 3, 260), (50, 40, 100)])
def test_apply_mask(k, oracle, dtype, N, H, Mc):
    rng = np.random.default_rng(N)
    W = rng.standard_normal((N, H * Mc)).astype(dtype)
    wmask = (rng.random((N, H)) < 0.5).astype(np.uint8)
    assert np.array_equal(k.apply_mask(W.copy(), wmask, H, Mc), oracle.apply_mask(W.copy(), wmask, H, Mc))


@pytest.mark.parametrize("dtype", DT)
def test_argmax_rows(k, oracle, dtype):
    rng = np.random.default_rng(0)
    a = rng.integers(0, 4, (300, 10)).astype(dtype)  # many ties: first maximum must win
    assert np.array_equal(k.argmax_rows(a), oracle.argmax_rows(a))
    b = rng.standard_normal((77, 1000)).astype(dtype)
    assert np.array_equal(k.argmax_rows(b), np.argmax(b, 1))


# ------------------------------------------------------------------------ fused plastic train step
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,N,H,Mc,h", [(16, 40, 3, 8, None), (16, 40, 3, 8, 1), (128, 1568, 30, 100, None),
                                        (128, 1568, 30, 100, 7), (96, 300, 4, 25, 3), (9, 33, 2, 7, 0),
                                        # row counts of the wider swap kernels, whose launch also fixes the weights
                                        # of the rows that changed sides, and past them (a separate fix-up launch)
                                        (16, 3000, 3, 8, 2), (8, 9000, 2, 8, 0), (8, 65600, 2, 4, 1)])
def test_plastic_train_step(k, oracle, dtype, B, N, H, Mc, h):
    _check_plastic_train_step(k, oracle, dtype, B, N, H, Mc, h, np.random.default_rng(B + N + H + Mc))


def _random_shapes(seed, count):
    """Shapes off every tiling's grid: mostly odd widths, batches around the 16- and 32-row boundaries."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        B = int(rng.choice([1, 2, 15, 16, 17, 31, 33, 47, 64, 100, 129]))
        N = int(rng.integers(1, 400))
        H = int(rng.integers(1, 7))
        Mc = int(rng.choice([1, 2, 3, 5, 9, 16, 17, 31, 33, 50, 63, 65, 100, 101, 127, 130]))
        out.append((B, N, H, Mc))
    return out


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,N,H,Mc", _random_shapes(2024, 24))
def test_random_shapes_forward_and_train_step(k, oracle, dtype, B, N, H, Mc):
    rng = np.random.default_rng(B + 3 * N + 5 * H + 7 * Mc)
    M = H * Mc
    x = rng.random((B, N)).astype(dtype)
    W = (0.1 * rng.standard_normal((N, M))).astype(dtype)
    b = (0.1 * rng.random(M)).astype(dtype)
    ref = oracle.softmax_minicolumns(oracle.update_state(np.zeros((B, M), dtype=dtype), W, b, x), H, Mc)
    assert_close(k.compute_activation(W, b, x, H, Mc), ref, dtype, "forward")
    h = int(rng.integers(0, H)) if rng.random() < 0.5 else None
    _check_plastic_train_step(k, oracle, dtype, B, N, H, Mc, h, rng, must_rewire=False)


def _check_plastic_train_step(k, oracle, dtype, B, N, H, Mc, h, rng, must_rewire=True):
    import scipy.special
    M = H * Mc
    tau, khalf, pmin, taubdt = 0.006908854922437549, -139.02586632856327, 0.06195283356566607, \
        0.02218100432360414
    x = (rng.random((B, N)) * (rng.random((B, N)) < 0.3)).astype(dtype)
    y = scipy.special.softmax(rng.standard_normal((B, H, Mc)), axis=2).reshape(B, M).astype(dtype)
    st = {
        "weights": (0.1 * rng.standard_normal((N, M))).astype(dtype),
        "bias": (0.1 * rng.random(M)).astype(dtype),
        "Ci": (0.3 * rng.random(N)).astype(dtype),
        "Cj": np.full(M, 1.0 / Mc, dtype=dtype),
        "kbi": np.ones(M, dtype=dtype),
        "wmask": (rng.random((N, H)) < 0.1).astype(np.uint8),
    }
    st["Cij"] = (st["Ci"][:, None] * st["Cj"][None, :] * (0.5 + rng.random((N, M)))).astype(dtype)
    got = k.plastic_train_step(st, x, y, H, Mc, tau, khalf, pmin, taubdt, h)
    r = {n: v.copy() for n, v in st.items()}
    cthr = tau / 2
    oracle.update_weights(r["Ci"], r["Cj"], r["Cij"], x, y, tau, r["weights"], cthr)
    oracle.update_bias_regularized(r["bias"], r["kbi"], r["Cj"], cthr, khalf, pmin, taubdt)
    if h is not None:
        oracle.update_mask(r["wmask"], r["weights"], r["Ci"], r["Cj"], r["Cij"], cthr, H, Mc, h, 16)
    oracle.apply_mask(r["weights"], r["wmask"], H, Mc)
    assert np.array_equal(got["wmask"], r["wmask"])
    if must_rewire and h is not None and N > 100:
        assert not np.array_equal(r["wmask"], st["wmask"]), "the case is meant to rewire"
    assert np.array_equal(got["Ci"], r["Ci"]) and np.array_equal(got["Cj"], r["Cj"])
    assert np.array_equal(got["kbi"], r["kbi"])
    assert_close(got["Cij"], r["Cij"], dtype, "Cij")
    assert_close(got["bias"], r["bias"], dtype, "bias")
    assert_close(got["weights"], r["weights"], dtype, "W")
    assert np.array_equal(got["weights"] == 0, r["weights"] == 0)
