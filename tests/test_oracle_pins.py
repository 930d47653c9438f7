"""Pins for the CPU oracle: every function is checked against something that does not share its code
-- closed forms, invariants, library routines (numpy float64 matmul, scipy softmax) and brute force
on tiny inputs -- chosen so that a dropped term, a wrong sign or index, or a transposed operand fails.
"""
import numpy as np
import pytest
import scipy.special

DT = [np.float32, np.float64]


def tol(dtype):
    return 1e-5 if dtype == np.float32 else 1e-12


def close(a, ref, dtype, scale=1.0):
    a = np.asarray(a, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return np.all(np.abs(a - ref) <= scale * tol(dtype) * np.maximum(np.abs(ref), 1.0))


# ---------------------------------------------------------------- update_state
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,N,M", [(1, 1, 1), (3, 5, 7), (17, 33, 65), (128, 300, 210)])
def test_update_state_vs_float64_matmul(oracle, dtype, B, N, M):
    rng = np.random.default_rng(B * 1000 + N)
    x = rng.random((B, N)).astype(dtype)
    W = (0.1 * rng.standard_normal((N, M))).astype(dtype)
    b = rng.standard_normal(M).astype(dtype)
    act = np.full((B, M), 7.0, dtype=dtype)  # must be overwritten (beta = 0)
    oracle.update_state(act, W, b, x)
    ref = x.astype(np.float64) @ W.astype(np.float64) + b.astype(np.float64)
    assert close(act, ref, dtype, scale=4.0)


def test_update_state_not_transposed(oracle):
    # x = e_p picks row p of W: a transposed operand or swapped index cannot pass
    N, M = 6, 4
    W = np.arange(N * M, dtype=np.float64).reshape(N, M)
    b = np.zeros(M)
    for p in range(N):
        x = np.zeros((1, N)); x[0, p] = 1.0
        act = np.zeros((1, M))
        oracle.update_state(act, W, b, x)
        assert np.array_equal(act[0], W[p])


# ---------------------------------------------------------------- softmax
@pytest.mark.parametrize("dtype", DT)
def test_softmax_vs_scipy_and_invariants(oracle, dtype):
    rng = np.random.default_rng(3)
    B, H, Mc = 9, 5, 13
    a = (3 * rng.standard_normal((B, H * Mc))).astype(dtype)
    ref = scipy.special.softmax(a.astype(np.float64).reshape(B, H, Mc), axis=2).reshape(B, H * Mc)
    out = oracle.softmax_minicolumns(a.copy(), H, Mc)
    assert close(out, ref, dtype)
    assert np.allclose(out.reshape(B, H, Mc).sum(2), 1.0, atol=10 * tol(dtype))
    shifted = oracle.softmax_minicolumns((a + dtype(5.0)).copy(), H, Mc)
    assert np.allclose(shifted, out, atol=20 * tol(dtype))
    flat = oracle.softmax_minicolumns(np.full((2, H * Mc), 2.5, dtype=dtype), H, Mc)
    assert np.allclose(flat, 1.0 / Mc, rtol=10 * tol(dtype))
    big = oracle.softmax_minicolumns(np.array([[1000.0, 0.0, -1000.0]], dtype=dtype), 1, 3)
    assert np.all(np.isfinite(big)) and big[0, 0] == 1.0


# ---------------------------------------------------------------- update_weights (traces + W)
def _rand_problem(rng, B, N, M, dtype):
    x = rng.random((B, N)).astype(dtype)
    y = rng.random((B, M)).astype(dtype)
    Ci = (0.1 + 0.8 * rng.random(N)).astype(dtype)
    Cj = (0.1 + 0.8 * rng.random(M)).astype(dtype)
    Cij = (0.05 + 0.5 * rng.random((N, M))).astype(dtype)
    return x, y, Ci, Cj, Cij


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("B,N,M", [(1, 1, 1), (4, 3, 5), (7, 19, 35), (32, 40, 70)])
def test_traces_tau_one_is_batch_mean(oracle, dtype, B, N, M):
    # taupdt = 1: the moving average forgets its state, C = batch mean / x^T y / B exactly in real
    # arithmetic.  An x/y transposition or i/j swap changes the matrix.
    rng = np.random.default_rng(B + N + M)
    x, y, Ci, Cj, Cij = _rand_problem(rng, B, N, M, dtype)
    W = np.zeros((N, M), dtype=dtype)
    oracle.update_weights(Ci, Cj, Cij, x, y, 1.0, W, 0.5)
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    assert close(Ci, x64.mean(0), dtype)
    assert close(Cj, y64.mean(0), dtype)
    assert close(Cij, np.einsum("bi,bj->ij", x64, y64) / B, dtype)


@pytest.mark.parametrize("dtype", DT)
def test_traces_are_affine_in_state(oracle, dtype):
    # C' = (1 - tau) C + tau * mean.  With zero activity C' = (1 - tau) C; with the state at zero
    # C' = tau * mean.  The two must add up to the general case (a dropped term breaks this).
    rng = np.random.default_rng(11)
    B, N, M, tau = 6, 10, 12, 0.125  # tau exact in binary so (1 - tau) is too
    x, y, Ci, Cj, Cij = _rand_problem(rng, B, N, M, dtype)
    W = np.zeros((N, M), dtype=dtype)
    z = lambda a: np.zeros_like(a)
    a = [c.copy() for c in (Ci, Cj, Cij)]
    oracle.update_weights(*a, z(x), z(y), tau, W, tau / 2)
    for got, c in zip(a, (Ci, Cj, Cij)):
        assert np.array_equal(got, c * dtype(1 - tau))
    b = [z(c) for c in (Ci, Cj, Cij)]
    oracle.update_weights(*b, x, y, tau, W, tau / 2)
    full = [c.copy() for c in (Ci, Cj, Cij)]
    oracle.update_weights(*full, x, y, tau, W, tau / 2)
    for f, p, q in zip(full, a, b):
        assert close(f, p.astype(np.float64) + q.astype(np.float64), dtype)


@pytest.mark.parametrize("dtype", DT)
def test_traces_one_hot_single_sample(oracle, dtype):
    N, M, tau = 5, 6, 0.25
    for p in range(N):
        for q in range(M):
            x = np.zeros((1, N), dtype=dtype); x[0, p] = 1
            y = np.zeros((1, M), dtype=dtype); y[0, q] = 1
            Ci = np.full(N, 0.5, dtype=dtype); Cj = np.full(M, 0.5, dtype=dtype)
            Cij = np.full((N, M), 0.5, dtype=dtype); W = np.zeros((N, M), dtype=dtype)
            oracle.update_weights(Ci, Cj, Cij, x, y, tau, W, tau / 2)
            exp = np.full((N, M), 0.375); exp[p, q] = 0.625
            assert np.array_equal(Cij, exp.astype(dtype))
            ei = np.full(N, 0.375); ei[p] = 0.625
            ej = np.full(M, 0.375); ej[q] = 0.625
            assert np.array_equal(Ci, ei.astype(dtype)) and np.array_equal(Cj, ej.astype(dtype))


@pytest.mark.parametrize("dtype", DT)
def test_traces_clamped_at_zero(oracle, dtype):
    # negative activity drives the average below zero; the result is clamped (max(0, .))
    x = -np.ones((2, 3), dtype=dtype); y = np.ones((2, 4), dtype=dtype)
    Ci = np.full(3, 0.1, dtype=dtype); Cj = np.full(4, 0.1, dtype=dtype)
    Cij = np.full((3, 4), 0.1, dtype=dtype); W = np.ones((3, 4), dtype=dtype)
    oracle.update_weights(Ci, Cj, Cij, x, y, 0.5, W, 0.25)
    assert np.all(Ci == 0) and np.all(Cij == 0) and np.all(Cj > 0)
    assert np.all(W == 0)  # rows with Ci < cthr are zeroed


@pytest.mark.parametrize("dtype", DT)
def test_softmax_activity_keeps_marginals_consistent(oracle, dtype):
    # with per-hypercolumn normalised y and consistent initial traces (Cj sums to 1 per HC,
    # sum_j Cij[i, HC] = Ci[i]) both identities survive any number of updates
    rng = np.random.default_rng(5)
    B, N, H, Mc, tau = 16, 12, 3, 8, 0.05
    M = H * Mc
    Ci = np.ones(N, dtype=dtype); Cj = np.full(M, 1.0 / Mc, dtype=dtype)
    Cij = np.full((N, M), 1.0 / Mc, dtype=dtype); W = np.zeros((N, M), dtype=dtype)
    for _ in range(5):
        x = rng.random((B, N)).astype(dtype)
        y = scipy.special.softmax(rng.standard_normal((B, H, Mc)), axis=2).reshape(B, M).astype(dtype)
        oracle.update_weights(Ci, Cj, Cij, x, y, tau, W, tau / 2)
    assert np.allclose(Cj.reshape(H, Mc).sum(1), 1.0, atol=50 * tol(dtype))
    assert np.allclose(Cij.reshape(N, H, Mc).sum(2), Ci[:, None], atol=50 * tol(dtype))


@pytest.mark.parametrize("dtype", DT)
def test_weights_special_cases(oracle, dtype):
    # tau = 0 freezes the traces so W is a pure function of (Ci, Cj, Cij, cthr)
    N, M = 4, 5
    x = np.zeros((1, N), dtype=dtype); y = np.zeros((1, M), dtype=dtype)
    cthr = 0.01
    Ci = np.array([0.2, 0.005, 0.5, 0.3], dtype=dtype)          # row 1 below threshold
    Cj = np.array([0.1, 0.4, 0.001, 0.25, 0.6], dtype=dtype)    # col 2 below threshold
    Cij = np.outer(Ci.astype(np.float64), Cj.astype(np.float64)).astype(dtype)  # independent
    Cij[0, 0] = 0.0            # floored at cthr^4
    Cij[2, 1] = 0.4            # arbitrary dependent entry
    W = np.full((N, M), 9.0, dtype=dtype)
    Ci0, Cj0, Cij0 = Ci.copy(), Cj.copy(), Cij.copy()
    oracle.update_weights(Ci, Cj, Cij, x, y, 0.0, W, cthr)
    assert np.array_equal(Ci, Ci0) and np.array_equal(Cj, Cj0) and np.array_equal(Cij, Cij0)
    assert np.all(W[1] == 0) and np.all(W[:, 2] == 0)
    assert abs(W[3, 3]) <= 4 * np.finfo(dtype).eps and abs(W[2, 4]) <= 4 * np.finfo(dtype).eps
    c64 = float(dtype(cthr))
    assert close(W[0, 0], np.log(c64 ** 4 / (float(Ci[0]) * float(Cj[0]))), dtype)
    assert close(np.exp(np.float64(W[2, 1])) * float(Ci[2]) * float(Cj[1]), 0.4, dtype, scale=4)


@pytest.mark.parametrize("dtype", DT)
def test_weights_use_updated_traces(oracle, dtype):
    # W must be computed from the traces AFTER this step's update: with tau = 1 the new traces are
    # the batch statistics, whatever the old state was
    rng = np.random.default_rng(2)
    B, N, M = 8, 5, 6
    x, y, Ci, Cj, Cij = _rand_problem(rng, B, N, M, dtype)
    W = np.zeros((N, M), dtype=dtype)
    oracle.update_weights(Ci, Cj, Cij, x, y, 1.0, W, 1e-3)
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    ref = np.log((x64.T @ y64 / B) / np.outer(x64.mean(0), y64.mean(0)))
    assert close(W, ref, dtype, scale=8)


@pytest.mark.parametrize("dtype", DT)
def test_fast_math_build_stays_within_tolerance(oracle, oracle_fast, dtype):
    rng = np.random.default_rng(8)
    B, N, M = 32, 50, 90
    x, y, Ci, Cj, Cij = _rand_problem(rng, B, N, M, dtype)
    res = []
    for o in (oracle, oracle_fast):
        s = [a.copy() for a in (Ci, Cj, Cij)]
        W = np.zeros((N, M), dtype=dtype)
        o.update_weights(*s, x, y, 0.01, W, 0.005)
        res.append(s + [W])
    for a, b in zip(*res):
        assert close(b, a, dtype, scale=4)


# ---------------------------------------------------------------- bias
@pytest.mark.parametrize("dtype", DT)
def test_update_bias_closed_form(oracle, dtype):
    cthr = 0.05
    Cj = np.array([0.5, 0.05, 0.049, 1.0, 0.0], dtype=dtype)
    bias = np.zeros(5, dtype=dtype)
    oracle.update_bias(bias, Cj, cthr)
    c = float(dtype(cthr))
    exp = np.array([0.5, float(Cj[1]), 2 * c, 1.0, 2 * c])
    assert close(np.exp(bias.astype(np.float64)), exp, dtype, scale=4)
    assert bias[3] == 0


@pytest.mark.parametrize("dtype", DT)
def test_update_bias_regularized_closed_forms(oracle, dtype):
    khalf, pmin, cthr = -100.0, 0.2, 0.01
    p4 = pmin / 4
    Cj = np.array([0.5, 0.051, 0.04, 0.3, 0.005], dtype=dtype)
    kbi0 = np.array([1.0, 2.0, 3.0, -1.0, 0.5], dtype=dtype)
    k = (khalf - 1) * p4 ** 2
    kb = 1 + k / (Cj.astype(np.float64) - p4) ** 2
    kb = np.where((Cj < p4) | (kb < khalf), khalf, kb)
    assert kb[1] == khalf and kb[2] == khalf and kb[0] > khalf  # both clamp branches are exercised
    # taubdt = 0: kbi frozen, bias = kbi * log(Cj or 2 cthr)
    bias = np.zeros(5, dtype=dtype); kbi = kbi0.copy()
    oracle.update_bias_regularized(bias, kbi, Cj, cthr, khalf, pmin, 0.0)
    assert np.array_equal(kbi, kbi0)
    logs = np.log(np.where(Cj < dtype(cthr), 2 * float(dtype(cthr)), Cj.astype(np.float64)))
    assert close(bias, kbi0 * logs, dtype, scale=4)
    # taubdt = 1: kbi = kb
    bias = np.zeros(5, dtype=dtype); kbi = kbi0.copy()
    oracle.update_bias_regularized(bias, kbi, Cj, cthr, khalf, pmin, 1.0)
    assert close(kbi, kb, dtype, scale=200)  # (pj - p4)^-2 amplifies input rounding near the pole
    # general: convex combination
    bias = np.zeros(5, dtype=dtype); kbi = kbi0.copy()
    oracle.update_bias_regularized(bias, kbi, Cj, cthr, khalf, pmin, 0.25)
    assert close(kbi, 0.75 * kbi0 + 0.25 * kb, dtype, scale=200)
    assert close(bias, kbi.astype(np.float64) * logs, dtype, scale=4)


# ---------------------------------------------------------------- mask
def _brute_mask(wmask, W, Ci, Cj, Cij, cthr, H, Mc, h, iterations):
    """Independent pure-Python statement of the rewiring rule, in float64 with Python lists."""
    wm = [[int(v) for v in row] for row in wmask]
    N = len(wm)
    nom = []
    for i in range(N):
        s = 0.0
        for j in range(h * Mc, (h + 1) * Mc):
            if Ci[i] >= cthr and Cj[j] >= cthr:
                pi, pj, pij = float(Ci[i]), float(Cj[j]), float(Cij[i][j])
                s += pij * float(W[i][j]) + (pj - pij) * np.log((pj - pij) / ((1 - pi) * pj))
        nom.append(s)
    for _ in range(iterations):
        score = [nom[i] / (1.0 + sum(wm[i])) for i in range(N)]
        zeros = [i for i in range(N) if wm[i][h] == 0]
        ones = [i for i in range(N) if wm[i][h] == 1]
        if not zeros or not ones:
            break
        vmax = max(score[i] for i in zeros)
        imax = max(i for i in zeros if score[i] == vmax)  # last index among ties
        vmin = min(score[i] for i in ones)
        imin = max(i for i in ones if score[i] == vmin)
        if vmax < vmin:
            break
        wm[imax][h] = 1
        wm[imin][h] = 0
    return np.array(wm, dtype=np.uint8)


def _mask_problem(rng, N, H, Mc, density=0.3):
    M = H * Mc
    wmask = (rng.random((N, H)) < density).astype(np.uint8)
    W = 0.1 * rng.standard_normal((N, M))
    Ci = 0.05 + 0.9 * rng.random(N)
    Cj = 0.05 + 0.9 * rng.random(M)
    Cij = np.minimum(np.minimum(0.9 * Ci[:, None], 0.9 * Cj[None, :]), rng.random((N, M)))
    return wmask, W, Ci, Cj, Cij


@pytest.mark.parametrize("seed", range(6))
def test_update_mask_vs_brute_force(oracle, seed):
    rng = np.random.default_rng(100 + seed)
    N, H, Mc = int(rng.integers(2, 40)), int(rng.integers(1, 5)), int(rng.integers(2, 7))
    wmask, W, Ci, Cj, Cij = _mask_problem(rng, N, H, Mc)
    h = int(rng.integers(0, H))
    for iterations in (0, 1, 3, 16):
        ref = _brute_mask(wmask, W, Ci, Cj, Cij, 0.01, H, Mc, h, iterations)
        got = oracle.update_mask(wmask.copy(), W, Ci, Cj, Cij, 0.01, H, Mc, h, iterations)
        assert np.array_equal(got, ref)
        assert got[:, h].sum() == wmask[:, h].sum()            # column popcount is invariant
        other = [g for g in range(H) if g != h]
        assert np.array_equal(got[:, other], wmask[:, other])  # other hypercolumns untouched
        assert (got != wmask).sum() <= 2 * iterations


@pytest.mark.parametrize("seed", range(6))
def test_update_mask_trace_vs_brute_force(oracle, seed):
    """The optional trace of the rewiring (rows picked, their scores, the runners-up on either side, the
    scores that ended the loop) against a Python scan in float64 on float64 inputs."""
    rng = np.random.default_rng(300 + seed)
    N, H, Mc = int(rng.integers(6, 40)), int(rng.integers(1, 5)), int(rng.integers(2, 7))
    wmask, W, Ci, Cj, Cij = _mask_problem(rng, N, H, Mc)
    h = int(rng.integers(0, H))
    trace = {}
    oracle.update_mask(wmask.copy(), W, Ci, Cj, Cij, 0.01, H, Mc, h, 16, trace=trace)
    wm = wmask.copy().astype(int)
    nom = np.zeros(N)
    for i in range(N):
        for j in range(h * Mc, (h + 1) * Mc):
            if Ci[i] >= 0.01 and Cj[j] >= 0.01:
                nom[i] += Cij[i, j] * W[i, j] + (Cj[j] - Cij[i, j]) * np.log((Cj[j] - Cij[i, j]) / ((1 - Ci[i]) * Cj[j]))
    swaps, stop = [], None
    for _ in range(16):
        score = nom / (1.0 + wm.sum(1))
        zeros, ones = np.flatnonzero(wm[:, h] == 0), np.flatnonzero(wm[:, h] == 1)
        if not len(zeros) or not len(ones):
            break
        imax = max(i for i in zeros if score[i] == score[zeros].max())
        imin = max(i for i in ones if score[i] == score[ones].min())
        if score[imax] < score[imin]:
            stop = (score[imax], score[imin])
            break
        r0 = max((score[i] for i in zeros if i != imax), default=-3e38)
        r1 = min((score[i] for i in ones if i != imin), default=3e38)
        swaps.append((imax, imin, score[imax], score[imin], r0, r1))
        wm[imax, h], wm[imin, h] = 1, 0
    assert trace["swaps"].tolist() == [[a, b] for a, b, *_ in swaps]
    assert np.allclose(trace["vals"], [[c, d] for _, _, c, d, _, _ in swaps] or np.zeros((0, 2)), rtol=1e-12, atol=0)
    assert np.allclose(trace["runner"], [[e, f] for *_, e, f in swaps] or np.zeros((0, 2)), rtol=1e-12, atol=0)
    assert (trace["stop"] is None) == (stop is None)
    if stop is not None:
        assert np.allclose(trace["stop"], stop, rtol=1e-12, atol=0)


def test_update_mask_degenerate_columns_and_ties(oracle):
    rng = np.random.default_rng(4)
    N, H, Mc = 10, 2, 3
    wmask, W, Ci, Cj, Cij = _mask_problem(rng, N, H, Mc)
    for fill in (0, 1):
        wm = wmask.copy(); wm[:, 1] = fill
        assert np.array_equal(oracle.update_mask(wm.copy(), W, Ci, Cj, Cij, 0.01, H, Mc, 1, 16), wm)
    # all scores equal (nominator 0 because every Ci < cthr, and equal row sums): the LAST silent row
    # is switched on and the LAST active row is switched off
    wm = np.zeros((6, 1), dtype=np.uint8); wm[[1, 3], 0] = 1
    Ci = np.full(6, 1e-4); Cj = np.full(3, 0.3); Cij = np.full((6, 3), 1e-5); W = np.zeros((6, 3))
    trace = {}
    got = oracle.update_mask(wm.copy(), W, Ci, Cj, Cij, 0.01, 1, 3, 0, 1, trace=trace)
    assert trace["swaps"].tolist() == [[5, 3]]
    assert got[:, 0].tolist() == [0, 1, 0, 0, 0, 1]


@pytest.mark.parametrize("dtype", DT)
def test_apply_mask_closed_form(oracle, dtype):
    rng = np.random.default_rng(9)
    N, H, Mc = 13, 4, 5
    W = rng.standard_normal((N, H * Mc)).astype(dtype)
    wmask = (rng.random((N, H)) < 0.5).astype(np.uint8)
    ref = W * np.repeat(wmask, Mc, axis=1)
    assert np.array_equal(oracle.apply_mask(W.copy(), wmask, H, Mc), ref.astype(dtype))


@pytest.mark.parametrize("dtype", DT)
def test_argmax_first_maximum(oracle, dtype):
    a = np.array([[1, 3, 3, 2], [5, 5, 5, 5], [0, -1, 4, 4]], dtype=dtype)
    assert oracle.argmax_rows(a).tolist() == [1, 0, 2] == np.argmax(a, axis=1).tolist()
