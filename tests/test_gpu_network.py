"""Network-level GPU parity: the hip backend's DSL (pybind11 object over the C ABI) against the
reference driver's recorded trajectory and against the oracle's cpu-backend restatement, on identical
seeded inputs.  Masks and predicted labels bit-exact; floats within tol * max(|ref|, 1)."""
import os

import numpy as np
import pytest

from helpers import (MNIST_HP, build_two_layer, fixture_config, one_hot_labels, record_error, rel_err,
                     synthetic_images)

pytestmark = pytest.mark.gpu

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "driver_trajectory_f64.npz")


@pytest.fixture(scope="module")
def hb():
    from streambrain_amd.backend import hip_backend
    return hip_backend


def test_reference_trajectory_fixture_f64(hb):
    g = np.load(FIX)
    c = fixture_config(g)
    net = build_two_layer(hb, int(c["n_in"]), int(c["H"]), int(c["Mc"]), int(c["n_out"]), c, np.float64,
                          seed=int(c["net_seed"]))
    l0, l1 = net._layers
    assert np.array_equal(l0.weights, g["init_L0_weights"]) and np.array_equal(l0.wmask, g["init_L0_wmask"])
    assert np.array_equal(l1.weights, g["init_L1_weights"]) and np.array_equal(l1.bias, g["init_L1_bias"])
    net.fit(g["X"], g["Y"], int(c["B"]), [(0, int(c["l1_epochs"]))])
    assert np.array_equal(l0.wmask, g["mid_L0_wmask"])
    for name in ("weights", "bias", "Ci", "Cj", "Cij", "kbi"):
        assert rel_err(getattr(l0, name), g[f"mid_L0_{name}"], f"mid_L0.{name}", 1e-12) <= 1e-12, name
    net.fit(g["X"], g["Y"], int(c["B"]), [(1, int(c["l2_epochs"]))])
    for li, layer in enumerate((l0, l1)):
        for name in ("weights", "bias", "Ci", "Cj", "Cij"):
            assert rel_err(getattr(layer, name), g[f"final_L{li}_{name}"], f"final_L{li}.{name}", 1e-12) <= 1e-12, f"L{li}.{name}"
    correct, total = net.evaluate(g["Xt"], g["Yt"], int(c["B"]))
    assert correct.tolist() == g["correct"].tolist() and total.tolist() == g["total"].tolist()
    assert np.array_equal(net.predict(g["Xt"], int(c["B"])), g["test_predictions"])
    assert rel_err(net.forward(g["Xt"], int(c["B"])), g["test_activations"], "test_activations", 1e-12) <= 1e-12
    np.testing.assert_array_equal(np.random.rand(4), g["rng_probe_after"])


def _run_both(hb, dtype, n_pix, H, Mc, n_out, Ns, Nt, B, e1, e2, hp, data_seed):
    from oracle import cpu_backend as ob
    rng = np.random.default_rng(data_seed)
    X, Y = synthetic_images(rng, Ns, n_pix), one_hot_labels(rng, Ns, n_out)
    Xt, Yt = synthetic_images(rng, Nt, n_pix), one_hot_labels(rng, Nt, n_out)
    nets = []
    for backend in (hb, ob):
        net = build_two_layer(backend, 2 * n_pix, H, Mc, n_out, hp, dtype, seed=0)
        net.fit(X, Y, B, [(0, e1)])
        net.fit(X, Y, B, [(1, e2)])
        nets.append(net)
    return nets, (Xt, Yt)


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
def test_single_step_matches_cpu_backend(hb, dtype, tol):
    # one batch, one epoch per layer: the north-star "after one step" bound
    (g, r), _ = _run_both(hb, dtype, n_pix=100, H=6, Mc=20, n_out=10, Ns=64, Nt=8, B=64, e1=1, e2=1,
                          hp=MNIST_HP, data_seed=7)
    for li in range(2):
        for name in ("Ci", "Cj", "Cij", "weights", "bias") + (("kbi",) if li == 0 else ()):
            e = rel_err(getattr(g._layers[li], name), getattr(r._layers[li], name), f"L{li}.{name}", tol)
            assert e <= tol, f"L{li}.{name}: {e:.3e}"
    assert np.array_equal(g._layers[0].wmask, r._layers[0].wmask)


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
def test_one_step_error_table_at_the_headline_shape(hb, dtype, tol):
    """One training step of each layer at exactly the headline configuration's shape (batch 128,
    1568 -> 30 x 100 -> 10, mask density 0.1) against the cpu-backend restatement: the maximum of
    |gpu - ref| / max(|ref|, 1) per quantity is asserted against the stated tolerance and written to
    parity_one_step_<dtype>.md in $SB_PARITY_OUT (when set), the table the design notes carry."""
    (g, r), _ = _run_both(hb, dtype, n_pix=784, H=30, Mc=100, n_out=10, Ns=128, Nt=8, B=128, e1=1, e2=1,
                          hp=MNIST_HP, data_seed=1001)
    rng = np.random.default_rng(1001)
    X = synthetic_images(rng, 128, 784).astype(dtype)  # the training batch again (same generator state)
    rows = []
    for li in range(2):
        for name in ("Ci", "Cj", "Cij", "weights", "bias") + (("kbi",) if li == 0 else ()):
            e = rel_err(getattr(g._layers[li], name), getattr(r._layers[li], name), f"L{li}.{name}", tol)
            rows.append((f"layer {li} {name}", e))
    act_r = [r._layers[0].compute_activation(X)]
    act_r.append(r._layers[1].compute_activation(act_r[0]))
    for li in range(2):
        e = rel_err(g.forward(X, 128, last_layer=li), act_r[li], f"L{li}.activations", tol)
        rows.append((f"layer {li} activations (after the step)", e))
    assert np.array_equal(g._layers[0].wmask, r._layers[0].wmask)
    assert np.array_equal(g.predict(X, 128), r.predict(X, 128))
    out = os.environ.get("SB_PARITY_OUT")
    if out and os.path.isdir(out):
        with open(os.path.join(out, f"parity_one_step_{np.dtype(dtype).name}.md"), "w") as f:
            f.write(f"| quantity ({np.dtype(dtype).name}, tolerance {tol:.0e}) | max error |\n|---|---|\n")
            for what, e in rows:
                f.write(f"| {what} | {e:.2e} |\n")
    for what, e in rows:
        assert e <= tol, f"{what}: {e:.3e} > {tol:.0e}"


def _compare_states(g, r, tol, names=("Ci", "Cj", "Cij", "weights", "bias")):
    for li in range(2):
        for name in names:
            e = rel_err(getattr(g._layers[li], name), getattr(r._layers[li], name), f"L{li}.{name}", tol)
            assert e <= tol, f"L{li}.{name}: {e:.3e} > {tol:.1e}"


def _mask_diff(a, b):
    return int((a != b).sum())


@pytest.mark.parametrize("B", [16, 20])
def test_small_network_epochs_with_rewiring_f64(hb, B):
    # 3 + 2 epochs, 13 (10) batches with a short last one, rewiring from the second epoch on: in float64
    # the whole trajectory, masks included, is reproduced.  (Batches of 16 let the first layer's forward
    # read its input in blocks of 16 rows, batches of 20 do not.)
    (g, r), (Xt, Yt) = _run_both(hb, np.float64, n_pix=60, H=4, Mc=10, n_out=5, Ns=200, Nt=50, B=B,
                                 e1=3, e2=2, hp=dict(MNIST_HP, l1_density=0.3), data_seed=11)
    assert _mask_diff(g._layers[0].wmask, r._layers[0].wmask) == 0
    _compare_states(g, r, 1e-12)
    assert np.array_equal(g.predict(Xt, 16), r.predict(Xt, 16))
    cg, tg = g.evaluate(Xt, Yt, 16)
    cr, tr = r.evaluate(Xt, Yt, 16)
    assert cg.tolist() == cr.tolist() and tg.tolist() == tr.tolist()


@pytest.mark.parametrize("n_pix,H,Mc,n_out,Ns,B,density", [
    (9, 3, 7, 3, 90, 13, 0.5),      # odd everything: minicolumns not a multiple of the vector width
    (17, 5, 4, 4, 200, 32, 0.2),    # sparse mask, batches of 32 (two row blocks of 16), short last batch
    (4, 2, 2, 2, 192, 64, 0.5),     # three full batches, two minicolumns
    (50, 7, 12, 10, 150, 17, 0.15),  # 9 batches, period 1: a rewiring at every step of the later epochs
    (40, 1, 16, 5, 96, 16, 0.4),    # a single hypercolumn
])
def test_odd_shaped_networks_f64(hb, n_pix, H, Mc, n_out, Ns, B, density):
    # shapes off every tiling's grid, 3 + 2 epochs: whole trajectory in float64, masks included
    (g, r), (Xt, Yt) = _run_both(hb, np.float64, n_pix=n_pix, H=H, Mc=Mc, n_out=n_out, Ns=Ns, Nt=40, B=B,
                                 e1=3, e2=2, hp=dict(MNIST_HP, l1_density=density), data_seed=100 + n_pix)
    assert _mask_diff(g._layers[0].wmask, r._layers[0].wmask) == 0
    _compare_states(g, r, 1e-12)
    assert np.array_equal(g.predict(Xt, B), r.predict(Xt, B))
    assert rel_err(g.forward(Xt, 7), r.forward(Xt.astype(np.float64))) <= 1e-12


def test_classifier_epochs_follow_changes_below_them_f64(hb):
    """While only the output layer trains, the backend keeps the hidden layer's activations of the training
    set instead of recomputing them every epoch.  Whatever changes the hidden layer in between -- its own
    training, state written from outside -- must show in the next classifier epoch as it does in the
    cpu-backend restatement, which recomputes everything."""
    from oracle import cpu_backend as ob
    rng = np.random.default_rng(77)
    n_pix, H, Mc, n_out, Ns, B = 30, 4, 12, 5, 150, 16
    X, Y = synthetic_images(rng, Ns, n_pix), one_hot_labels(rng, Ns, n_out)
    Xt = synthetic_images(rng, 40, n_pix)
    nets = []
    for backend in (hb, ob):
        net = build_two_layer(backend, 2 * n_pix, H, Mc, n_out, dict(MNIST_HP, l1_density=0.4), np.float64, seed=3)
        net.fit(X, Y, B, [(0, 2)])
        net.fit(X, Y, B, [(1, 2)])            # activations kept over these two epochs
        net.fit(X, Y, B, [(0, 1)])            # the hidden layer moves on
        net.fit(X, Y, B, [(1, 1)])
        w = np.array(net._layers[0].weights)  # state written from outside
        w[::3] *= 0.5
        net._layers[0].weights = w
        net.fit(X, Y, B, [(1, 2)])
        net.fit(X[:100], Y[:100], B, [(1, 1)])  # another training set
        nets.append(net)
    g, r = nets
    assert _mask_diff(g._layers[0].wmask, r._layers[0].wmask) == 0
    _compare_states(g, r, 1e-12)
    assert np.array_equal(g.predict(Xt, B), r.predict(Xt, B))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_classifier_epochs_without_the_activation_cache_are_bit_identical(hb, dtype):
    """The cache of the frozen layers' activations is an optimisation with a fallback: when it is not
    affordable (here: a limit of zero bytes, and a limit lowered while a cache is held) every step runs the
    forward passes of the layers below instead.  Both ways give the same bits."""
    rng = np.random.default_rng(78)
    n_pix, H, Mc, n_out, Ns, B = 40, 4, 12, 5, 200, 16
    X, Y = synthetic_images(rng, Ns, n_pix), one_hot_labels(rng, Ns, n_out)
    states = []
    for limit in (None, 0, "lowered"):
        net = build_two_layer(hb, 2 * n_pix, H, Mc, n_out, dict(MNIST_HP, l1_density=0.4), dtype, seed=5)
        if limit == 0:
            net.net.set_frozen_cache_limit(0)
        np.random.seed(11)
        net.fit(X, Y, B, [(0, 1)])
        if limit == "lowered":
            # one epoch with the cache, then the limit drops below what it takes and the rest runs without
            net.net.initiate_training(X.astype(dtype), Y.astype(dtype))
            for epoch in range(3):
                idx = np.random.permutation(Ns).astype(np.int64)
                hc = np.random.permutation(1).astype(np.int64)
                net.net.train_epoch(1, B, idx, hc, epoch)
                if epoch == 0:
                    net.net.set_frozen_cache_limit(1000)
            net.net.training_done()
        else:
            net.fit(X, Y, B, [(1, 3)])
        states.append({name: np.array(getattr(net._layers[1], name)) for name in ("Ci", "Cj", "Cij", "weights", "bias")})
    for other in states[1:]:
        for name, value in states[0].items():
            assert np.array_equal(value, other[name]), name


def test_small_network_one_epoch_f32(hb):
    # float32, one epoch per layer (13 batches, short last one).  Stated drift bound after one epoch:
    # 1e-5 relative (rounding differences of ~1e-7 per step, amplified by the log of small traces).
    (g, r), (Xt, Yt) = _run_both(hb, np.float32, n_pix=60, H=4, Mc=10, n_out=5, Ns=200, Nt=50, B=16,
                                 e1=1, e2=1, hp=dict(MNIST_HP, l1_density=0.3), data_seed=11)
    assert _mask_diff(g._layers[0].wmask, r._layers[0].wmask) == 0
    _compare_states(g, r, 1e-5)
    assert np.array_equal(g.predict(Xt, 16), r.predict(Xt, 16))


def test_mnist_shape_one_epoch_f32(hb):
    # MNIST shape (1568 -> 30x100 -> 10), float32, batch 128, 31 batches (short last one), one epoch
    # per layer.  Stated drift bound after one epoch: 1e-5 relative; predicted labels bit-exact.
    (g, r), (Xt, Yt) = _run_both(hb, np.float32, n_pix=784, H=30, Mc=100, n_out=10, Ns=31 * 128 - 32,
                                 Nt=256, B=128, e1=1, e2=1, hp=MNIST_HP, data_seed=1001)
    assert _mask_diff(g._layers[0].wmask, r._layers[0].wmask) == 0
    _compare_states(g, r, 1e-5)
    assert np.array_equal(g.predict(Xt, 128), r.predict(Xt, 128))
    cg, _ = g.evaluate(Xt, Yt, 128)
    cr, _ = r.evaluate(Xt, Yt, 128)
    assert cg.tolist() == cr.tolist()


def test_dense_hidden_layer_one_epoch_f32(hb):
    # The hidden layer with an all-ones mask (density 1) trained for one epoch on its own activations,
    # float32, batch 128, a short last batch: the reference's cpu-runnable single-layer case on fewer
    # batches (the output layer is only there because fit trains the LAST layer on labels).
    from oracle import cpu_backend as ob
    rng = np.random.default_rng(1000)
    X = synthetic_images(rng, 20 * 128 - 32, 784)
    Y = one_hot_labels(rng, X.shape[0], 10)
    nets = []
    for backend in (hb, ob):
        net = build_two_layer(backend, 1568, 30, 100, 10, MNIST_HP, np.float32, seed=0, density=1.0)
        net.fit(X, Y, 128, [(0, 1)])
        nets.append(net)
    g, r = nets
    assert g._layers[0].wmask.all() and r._layers[0].wmask.all()
    for name in ("Ci", "Cj", "Cij", "weights", "bias", "kbi"):
        e = rel_err(getattr(g._layers[0], name), getattr(r._layers[0], name), name, 1e-5)
        assert e <= 1e-5, f"{name}: {e:.3e}"


def test_full_epoch_drift_f32(hb, oracle_fast):
    """The drift bound after one epoch at the headline configuration's full size: 60000 samples, 469 steps
    of the hidden layer (1568 -> 30 x 100, mask density 0.1, batch 128, short last batch; epoch 0, so no
    rewiring) against the cpu-backend restatement on the reference's own build flags (OpenMP,
    -ffast-math).  Stated drift bound after a full epoch: 5e-5 relative for every trace, the weights and
    the bias (measured: weights 9.4e-6, bias 2.8e-6, kbi 2.2e-6, Ci 8.3e-7, Cij 1.2e-7, Cj 8.2e-8 -- the
    two builds of the restatement themselves differ by as much, since -ffast-math reorders its sums)."""
    from oracle import cpu_backend as ob
    rng = np.random.default_rng(1001)
    X = synthetic_images(rng, 60000, 784).astype(np.float32)
    nets = []
    for backend, kw in ((hb, {}), (ob, {"oracle": oracle_fast})):
        np.random.seed(0)
        net = backend.Network(np.float32)
        hp = MNIST_HP
        net.add_layer(backend.StructuralPlasticityLayer(
            1568, 30, 100, hp["l1_taupdt"], hp["l1_khalf"], hp["l1_pmin"], hp["l1_taubdt"], hp["l1_density"],
            int(hp["l1_mask_iterations"]), (1, 1 / 100, 1 / 100), **kw))
        net.add_layer(backend.DenseLayer(3000, 1, 10, hp["l2_taupdt"], (1 / 100, 1 / 10, 1 / 1000), **kw))
        net.fit(X, np.zeros((60000, 10), np.float32), 128, [(0, 1)])
        nets.append(net)
    g, r = nets
    assert np.array_equal(g._layers[0].wmask, r._layers[0].wmask)
    for name in ("Ci", "Cj", "Cij", "weights", "bias", "kbi"):
        e = rel_err(getattr(g._layers[0], name), getattr(r._layers[0], name), name, 5e-5)
        assert e <= 5e-5, f"{name}: {e:.3e}"


def test_wide_hidden_layer_f64(hb):
    # 1568 -> 100 x 100 -> 10 in float64 with batch 512 (one full and one short batch per epoch): the
    # float64 MFMA path of the trace GEMM and the float64 log / divide of the weight pass.
    (g, r), (Xt, Yt) = _run_both(hb, np.float64, n_pix=784, H=100, Mc=100, n_out=10, Ns=512 + 96, Nt=64,
                                 B=512, e1=1, e2=1, hp=MNIST_HP, data_seed=1002)
    assert _mask_diff(g._layers[0].wmask, r._layers[0].wmask) == 0
    _compare_states(g, r, 1e-12)
    assert np.array_equal(g.predict(Xt, 512), r.predict(Xt, 512))


def _scores_and_rounding_unit(W, Ci, Cj, Cij, wmask, cthr, h, Mc):
    """The rewiring scores of hypercolumn h evaluated in float64 from a float32 state, and per row the size
    of one float32 rounding step of its score: eps32 times the sum over the hypercolumn's columns of
    |pij w| + (pj - pij) (1 + |log y|), over 1 + csum.  (y = (pj - pij) / ((1 - pi) pj) is close to 1, where
    one rounding of y moves log y by eps whatever the size of log y itself.)"""
    cols = slice(h * Mc, (h + 1) * Mc)
    pi, pj = Ci.astype(np.float64)[:, None], Cj.astype(np.float64)[None, cols]
    pij, w = Cij.astype(np.float64)[:, cols], W.astype(np.float64)[:, cols]
    with np.errstate(all="ignore"):
        logy = np.log((pj - pij) / ((1 - pi) * pj))
        live = (pi >= cthr) & (pj >= cthr)
        nom = np.where(live, pij * w + (pj - pij) * logy, 0.0).sum(1)
        mag = np.where(live, np.abs(pij * w) + np.abs(pj - pij) * (1 + np.abs(logy)), 0.0).sum(1)
    den = 1.0 + wmask.sum(1)
    return nom / den, np.finfo(np.float32).eps * mag / den


def test_mnist_shape_rewiring_steps_f32(hb):
    """Second epoch, with rewiring (31 // 31 = 1: hypercolumns rewire on steps 0..29), float32, MNIST shape.
    Over a float32 TRAJECTORY mask equality is not well defined: a swap compares scores that are sums of a
    hundred terms, so state differences at rounding level flip near-ties and two runs fork (the strict-IEEE
    and the -ffast-math build of the cpu restatement disagree in 20 mask entries on this very run).  So the
    runs are walked step by step from identical state: every rewiring step of the restatement's trajectory
    is handed, with the state it started from, to the GPU's fused training step (traces, weights recomputed
    on the device, scores, swaps), and the two masks are compared.  Where they differ, the rows one side
    connected and the other did not (and likewise the rows disconnected) are paired in score order, and
    every pair must be a near-tie: scores within 4 float32 rounding steps of each other.  The device scores a
    row the way the reference does, operation by operation and term by term in column order, so what is left
    to differ between the two sides is the summation order of the batch inside Cij (matrix instructions
    against a sequential loop).  The number of forked steps and the widest such pair are printed and recorded
    (measured: 2 of 30 steps fork, 2 of 480 swaps go to another row, both exact ties of the float64 scores;
    with the weights recomputed through the hardware logarithm and the terms added by a lane butterfly it
    was 19 steps, 34 swaps and up to 17.9 rounding steps)."""
    from oracle import cpu_backend as ob
    from streambrain_amd import kernels_hip as k
    steps = []

    class Recorder(ob.StructuralPlasticityLayer):
        def train_step(self, inputs, outputs, hypercolumn=None):
            if hypercolumn is None:
                return super().train_step(inputs, outputs, None)
            pre = {n: getattr(self, n).copy() for n in ("weights", "bias", "Ci", "Cj", "Cij", "kbi", "wmask")}
            x, y = np.ascontiguousarray(inputs), np.ascontiguousarray(outputs)
            cthr = self.taupdt / 2
            self.k.update_weights(self.Ci, self.Cj, self.Cij, x, y, self.taupdt, self.weights, cthr)
            self.k.update_bias_regularized(self.bias, self.kbi, self.Cj, cthr, self.khalf, self.pmin, self.taubdt)
            score, unit = _scores_and_rounding_unit(self.weights, self.Ci, self.Cj, self.Cij, self.wmask, cthr,
                                                    int(hypercolumn), self.minicolumns)
            trace = {}
            self.k.update_mask(self.wmask, self.weights, self.Ci, self.Cj, self.Cij, cthr, self.hypercolumns,
                               self.minicolumns, int(hypercolumn), 16, trace=trace)
            steps.append((pre, x.copy(), y.copy(), int(hypercolumn), self.wmask.copy(), trace, score, unit))
            self.k.apply_mask(self.weights, self.wmask, self.hypercolumns, self.minicolumns)

    class Backend:
        Network = ob.Network
        StructuralPlasticityLayer = Recorder
        DenseLayer = ob.DenseLayer

    H, Mc, hp = 30, 100, MNIST_HP
    rng = np.random.default_rng(1001)
    X, Y = synthetic_images(rng, 31 * 128 - 32, 784), one_hot_labels(rng, 31 * 128 - 32, 10)
    net = build_two_layer(Backend, 1568, H, Mc, 10, hp, np.float32, seed=0)
    net.fit(X, Y, 128, [(0, 2)])
    assert len(steps) == 30
    forks, swaps_total, differing, widest = 0, 0, 0, 0.0
    for pre, x, y, h, after, trace, score, unit in steps:
        got = k.plastic_train_step(pre, x, y, H, Mc, hp["l1_taupdt"], hp["l1_khalf"], hp["l1_pmin"],
                                   hp["l1_taubdt"], h)["wmask"]
        swaps_total += len(trace["swaps"])
        assert np.array_equal(got.sum(0), after.sum(0))
        other = [g for g in range(H) if g != h]
        assert np.array_equal(got[:, other], pre["wmask"][:, other])
        if np.array_equal(got, after):
            continue
        forks += 1
        before = pre["wmask"][:, h]
        for side in (0, 1):  # rows switched on (were 0), rows switched off (were 1)
            mine = np.flatnonzero((before == side) & (got[:, h] != side) & (after[:, h] == side))
            theirs = np.flatnonzero((before == side) & (after[:, h] != side) & (got[:, h] == side))
            assert len(mine) == len(theirs), f"hypercolumn {h}: the two sides made different numbers of swaps"
            differing += len(mine)
            mine, theirs = mine[np.argsort(score[mine])], theirs[np.argsort(score[theirs])]
            for a, b in zip(mine, theirs):
                gap = abs(score[a] - score[b]) / max(unit[a], unit[b])
                widest = max(widest, gap)
                assert gap <= 4, (f"hypercolumn {h}: rows {a} and {b} were decided differently although their "
                                   f"scores are {gap:.1f} rounding steps apart")
    print(f"rewiring steps: {30 - forks} equal, {forks} forked; {differing} of {swaps_total} swaps went to another "
          f"row, the widest such pair {widest:.1f} float32 rounding steps apart")
    record_error("forked rewiring steps of 30", forks, 30)
    record_error("swaps that went to another row", differing, swaps_total)
    record_error("widest forked pair (rounding steps)", widest, 4)
    assert swaps_total > 250, "the run is meant to rewire"


def test_rewiring_decisions_replayed_f32(hb):
    # Every rewiring decision of a real float32 training run of the oracle (states after the trace and
    # weight update of that step), replayed through the GPU kernel on identical inputs: bit-exact.
    from oracle import cpu_backend as ob
    from streambrain_amd import kernels_hip as k
    captured = []

    class Recorder(ob.StructuralPlasticityLayer):
        def train_step(self, inputs, outputs, hypercolumn=None):
            if hypercolumn is None:
                return super().train_step(inputs, outputs, None)
            cthr = self.taupdt / 2
            self.k.update_weights(self.Ci, self.Cj, self.Cij, np.ascontiguousarray(inputs),
                                  np.ascontiguousarray(outputs), self.taupdt, self.weights, cthr)
            self.k.update_bias_regularized(self.bias, self.kbi, self.Cj, cthr, self.khalf, self.pmin,
                                           self.taubdt)
            before = self.wmask.copy()
            self.k.update_mask(self.wmask, self.weights, self.Ci, self.Cj, self.Cij, cthr,
                               self.hypercolumns, self.minicolumns, int(hypercolumn), 16)
            captured.append((before, self.weights.copy(), self.Ci.copy(), self.Cj.copy(),
                             self.Cij.copy(), cthr, int(hypercolumn), self.wmask.copy()))
            self.k.apply_mask(self.weights, self.wmask, self.hypercolumns, self.minicolumns)

    class Backend:
        Network = ob.Network
        StructuralPlasticityLayer = Recorder
        DenseLayer = ob.DenseLayer

    for n_pix, H, Mc, Ns, B, epochs, hp, seed in [
            (60, 4, 10, 200, 16, 3, dict(MNIST_HP, l1_density=0.3), 11),
            (784, 30, 100, 31 * 128 - 32, 128, 2, MNIST_HP, 1001)]:
        captured.clear()
        rng = np.random.default_rng(seed)
        X, Y = synthetic_images(rng, Ns, n_pix), one_hot_labels(rng, Ns, 5)
        net = build_two_layer(Backend, 2 * n_pix, H, Mc, 5, hp, np.float32, seed=0)
        net.fit(X, Y, B, [(0, epochs)])
        assert len(captured) >= min(H, 8)
        swapped = 0
        for before, W, Ci, Cj, Cij, cthr, h, after in captured:
            got = k.update_mask(before.copy(), W, Ci, Cj, Cij, cthr, H, Mc, h, 16)
            assert _mask_diff(got, after) == 0, f"hypercolumn {h}: {_mask_diff(got, after)} entries differ"
            swapped += _mask_diff(before, after)
        assert swapped > 0


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
def test_layer_level_methods_match_the_cpu_backend(hb, dtype, tol):
    """compute_activation / train_step / train_finalize called on the layers themselves, the way code written
    against the reference's layer classes does (_cpu_base_backend.py:44-68, 126-172; cpu_backend.py:13-52):
    the same calls on both backends from the same seeded state, state compared after every call."""
    from oracle import cpu_backend as ob
    rng = np.random.default_rng(21)
    n_pix, H, Mc, n_out, B = 40, 5, 12, 4, 24
    x = synthetic_images(rng, B, n_pix).astype(dtype)
    labels = one_hot_labels(rng, B, n_out).astype(dtype)
    nets = [build_two_layer(b, 2 * n_pix, H, Mc, n_out, dict(MNIST_HP, l1_density=0.3), dtype, seed=5)
            for b in (hb, ob)]
    (g0, g1), (r0, r1) = nets[0]._layers, nets[1]._layers

    def same(what):
        for li, (gl, rl) in enumerate(((g0, r0), (g1, r1))):
            for name in ("Ci", "Cj", "Cij", "weights", "bias") + (("kbi",) if li == 0 else ()):
                e = rel_err(getattr(gl, name), getattr(rl, name), f"{what} L{li}.{name}", tol)
                assert e <= tol, f"after {what}: L{li}.{name} {e:.3e}"
        assert np.array_equal(g0.wmask, r0.wmask), what

    for step, h in enumerate((None, 2, None, 0)):
        ag, ar = g0.compute_activation(x), r0.compute_activation(x)
        assert ag.shape == ar.shape and ag.dtype == dtype
        assert rel_err(ag, ar, "hidden activation", tol) <= tol
        g0.train_step(x, ar, h)  # both sides train on the same activation
        r0.train_step(x, ar, h)
        same(f"hidden train_step {step}")
        bg, br = g1.compute_activation(ar), r1.compute_activation(ar)
        assert rel_err(bg, br, "output activation", tol) <= tol
        g1.train_step(ar, labels)
        r1.train_step(ar, labels)
        same(f"output train_step {step}")
    g0.train_finalize(), r0.train_finalize(), g1.train_finalize(), r1.train_finalize()
    same("train_finalize")
    assert not np.array_equal(g0.wmask, build_two_layer(ob, 2 * n_pix, H, Mc, n_out, dict(MNIST_HP, l1_density=0.3),
                                                        dtype, seed=5)._layers[0].wmask), "the calls rewired"
    # a layer that has not joined a network says so
    np.random.seed(1)
    loose = hb.DenseLayer(8, 1, 3, 0.01, (0.1, 0.3, 0.03), dtype)
    with pytest.raises(RuntimeError, match="add_layer"):
        loose.compute_activation(np.zeros((2, 8), dtype))
    with pytest.raises(TypeError):
        g1.train_step(ar, labels, 0)


def test_zero_period_schedule_does_not_rewire(hb):
    # 2 batches, 5 hypercolumns: 2 // 6 == 0.  The reference divides by zero here; this backend trains
    # without rewiring.
    rng = np.random.default_rng(3)
    X, Y = synthetic_images(rng, 40, 30), one_hot_labels(rng, 40, 4)
    net = build_two_layer(hb, 60, 5, 6, 4, MNIST_HP, np.float32, seed=0, density=0.3)
    before = net._layers[0].wmask
    net.fit(X, Y, 32, [(0, 3)])
    assert np.array_equal(net._layers[0].wmask, before)
    assert np.all(np.isfinite(net._layers[0].weights))


def test_progress_bar_changes_no_result(hb, monkeypatch):
    """fit with the reference's per-batch progress bar enqueues an epoch in ranges of batches
    (_cpu_base_backend.py:270-312); without tqdm it enqueues the epoch whole.  Same state either way,
    over epochs with rewiring, a short last batch and both layers."""
    rng = np.random.default_rng(8)
    X, Y = synthetic_images(rng, 23 * 32 + 5, 60), one_hot_labels(rng, 23 * 32 + 5, 4)
    states = []
    for bar in (True, False):
        if not bar:
            monkeypatch.setattr(hb, "_tqdm", None)
        assert (hb._tqdm is not None) == bar
        net = build_two_layer(hb, 120, 4, 8, 4, MNIST_HP, np.float32, seed=2, density=0.3)
        np.random.seed(11)
        net.fit(X, Y, 32, [(0, 3), (1, 2)])
        states.append([getattr(l, n) for l in net._layers for n in ("weights", "bias", "Ci", "Cj", "Cij")]
                      + [net._layers[0].wmask, net._layers[0].kbi])
    for a, b in zip(*states):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_evaluate_of_many_batches_equals_single_batches(hb, dtype):
    """evaluate / predict / forward over a set of many batches (uploaded in chunks of whole batches) give what
    the same batches give when they are pushed through one at a time; the last batch is ragged."""
    rng = np.random.default_rng(12)
    n, B = 3000, 128
    X, Y = synthetic_images(rng, n, 784), one_hot_labels(rng, n, 4)
    net = build_two_layer(hb, 1568, 4, 8, 4, MNIST_HP, dtype, seed=5, density=0.3)
    net.fit(X[:512], Y[:512], B, [(0, 2), (1, 1)])  # masked weights: the first layer walks row lists
    whole = net.forward(X, B)
    pred = net.predict(X, B)
    correct, total = net.evaluate(X, Y, B)
    assert whole.shape == (n, 4) and int(total[0]) == n
    for lo in range(0, n, B):
        part = net.forward(X[lo:lo + B], B)
        assert np.array_equal(whole[lo:lo + B], part), lo
    assert np.array_equal(pred, np.argmax(whole, axis=1))
    assert int(correct[0]) == int((pred == np.argmax(Y, axis=1)).sum())


def test_errors_are_python_exceptions(hb):
    net = hb.Network(np.float32)
    with pytest.raises(Exception):
        hb.Network(np.int32)
    net.add_layer(hb.DenseLayer(8, 1, 3, 0.01, (0.1, 0.3, 0.03)))
    with pytest.raises(RuntimeError):
        net.net.train_epoch(0, 4, np.arange(4), None, 0)  # no training data
    with pytest.raises(RuntimeError):
        net.net.get_layer_state(0, "kbi")  # dense layers have no kbi
    with pytest.raises(RuntimeError):
        net.net.set_layer_state(0, "weights", np.zeros((3, 3), np.float32))


def test_checkpoint_round_trip_on_device(hb, tmp_path):
    # state saved from one device-resident network and loaded into another reproduces its outputs
    from streambrain_amd import checkpoint
    rng = np.random.default_rng(5)
    X, Y = synthetic_images(rng, 96, 40), one_hot_labels(rng, 96, 4)
    net = build_two_layer(hb, 80, 3, 8, 4, MNIST_HP, np.float32, seed=3)
    net.fit(X, Y, 32, [(0, 2), (1, 1)])
    checkpoint.save_state(net, tmp_path / "state.npz")
    other = build_two_layer(hb, 80, 3, 8, 4, MNIST_HP, np.float32, seed=4)
    checkpoint.load_state(other, tmp_path / "state.npz")
    for a, b in zip(net._layers, other._layers):
        for name in ("weights", "bias", "Ci", "Cj", "Cij"):
            assert np.array_equal(getattr(a, name), getattr(b, name)), name
    assert np.array_equal(net._layers[0].wmask, other._layers[0].wmask)
    assert np.array_equal(net._layers[0].kbi, other._layers[0].kbi)
    assert np.array_equal(net.forward(X, 32), other.forward(X, 32))
    # and training continues identically from the restored state
    np.random.seed(9)
    net.fit(X, Y, 32, [(0, 1)])
    np.random.seed(9)
    other.fit(X, Y, 32, [(0, 1)])
    assert np.array_equal(net._layers[0].weights, other._layers[0].weights)
    assert np.array_equal(net._layers[0].wmask, other._layers[0].wmask)


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float64, 1e-12)])
def test_forward_over_connected_rows_tracks_the_state(hb, dtype, tol):
    """A sparse layer's forward pass runs over its lists of connected rows once a training step has
    left W masked, and over all rows again after W or the mask has been written from outside: all of
    these must agree with the dense computation on the state read back from the device."""
    from streambrain_amd import kernels_hip as k
    rng = np.random.default_rng(5)
    X = synthetic_images(rng, 3 * 64, 200)
    Y = one_hot_labels(rng, X.shape[0], 10)
    net = build_two_layer(hb, 400, 6, 20, 10, MNIST_HP, dtype, seed=3, density=0.2)
    layer = net._layers[0]
    xt = np.ascontiguousarray(X[:40].astype(dtype))

    def dense(W, b):
        return k.compute_activation(np.ascontiguousarray(W), np.ascontiguousarray(b), xt, 6, 20)

    # before any training step W is the unmasked initial draw: dense path
    assert rel_err(net.forward(xt, last_layer=0), dense(layer.weights, layer.bias)) <= tol
    net.fit(X, Y, 64, [(0, 2)])  # two epochs, the second with rewiring
    W, b, mask = layer.weights, layer.bias, layer.wmask
    assert np.all(W[np.repeat(mask, 20, axis=1) == 0] == 0)
    assert rel_err(net.forward(xt, last_layer=0), dense(W, b)) <= tol  # row lists (after rewiring)
    # a masked W written from outside (a restored checkpoint) is recognised as such ...
    layer.weights = W
    assert rel_err(net.forward(xt, last_layer=0), dense(W, b)) <= tol
    # ... and an unmasked one must be used as it is
    W2 = (W + 0.01).astype(dtype)
    layer.weights = W2
    assert rel_err(net.forward(xt, last_layer=0), dense(W2, b)) <= tol
    # ... and a new mask does not touch W until the next training step
    layer.wmask = np.ascontiguousarray(1 - mask)
    assert rel_err(net.forward(xt, last_layer=0), dense(W2, b)) <= tol
    net.fit(X, Y, 64, [(0, 1)])
    W3, mask3 = layer.weights, layer.wmask
    assert np.all(W3[np.repeat(mask3, 20, axis=1) == 0] == 0)
    assert rel_err(net.forward(xt, last_layer=0), dense(W3, layer.bias)) <= tol


def test_full_size_epochs_keep_the_invariants_f32(hb):
    """The headline configuration at its full size (60000 samples, 1568 -> 30 x 100, batch 128, mask
    density 0.1), two epochs of the hidden layer, the second with rewiring -- out of the oracle's reach
    in test time, so what is checked are the properties the update rules guarantee whatever the data:
    the traces stay probability tables (hypercolumn sums of Cj are 1, hypercolumn sums of Cij rows are
    Ci, everything in [0, 1]), every swap keeps the number of connections of its hypercolumn, W is zero
    exactly where the mask is, the weights are the logarithm of the traces where it is not, and the
    activations of a batch are per-hypercolumn distributions."""
    rng = np.random.default_rng(1001)
    Ns, H, Mc = 60000, 30, 100
    X = synthetic_images(rng, Ns, 784).astype(np.float32)
    Y = one_hot_labels(rng, Ns, 10).astype(np.float32)
    net = build_two_layer(hb, 1568, H, Mc, 10, MNIST_HP, np.float32, seed=0)
    layer = net._layers[0]
    mask0 = layer.wmask.copy()
    net.fit(X, Y, 128, [(0, 2)])
    Ci, Cj, Cij, W, mask = layer.Ci, layer.Cj, layer.Cij, layer.weights, layer.wmask
    assert np.isfinite(W).all() and np.isfinite(Cij).all()
    assert Ci.min() >= 0 and Ci.max() <= 1 + 1e-5 and Cij.min() >= 0
    assert np.allclose(Cj.reshape(H, Mc).sum(1), 1.0, atol=2e-5)
    assert np.allclose(Cij.reshape(1568, H, Mc).sum(2), Ci[:, None], atol=2e-5)
    # rewiring: 30 hypercolumns rewired once each in the second epoch, connection counts unchanged
    assert np.array_equal(mask.sum(0), mask0.sum(0))
    changed = np.flatnonzero((mask != mask0).any(0))
    assert len(changed) >= 20 and np.all((mask != mask0).sum(0) <= 32)
    on = np.repeat(mask, Mc, axis=1) != 0
    assert np.all(W[~on] == 0)
    tau = MNIST_HP["l1_taupdt"]
    cthr = np.float32(tau / 2)
    live = on & (Ci[:, None] >= cthr) & (Cj[None, :] >= cthr)
    ref = np.log(np.maximum(Cij.astype(np.float64), float(cthr) ** 4) / (Ci[:, None].astype(np.float64) * Cj[None, :]))
    assert rel_err(W[live], ref[live]) <= 2e-5
    assert np.all(W[on & ~live] == 0)
    act = net.forward(X[:256], 128, last_layer=0)
    assert np.allclose(act.reshape(256, H, Mc).sum(2), 1.0, atol=1e-5) and act.min() >= 0


def test_example_script_flow_through_the_package(tmp_path, monkeypatch):
    """The flow of the reference's example script (train.py:9-23, 144-202 there) on idx-ubyte files
    written here: read the files, complementary coding, `import BCPNN` with BCPNN_BACKEND=hip, the two
    layers with the script's positional arguments, fit layer by layer, evaluate on both sets.  A learnable
    toy problem (the class is which block of pixels is lit), so the accuracy says the pieces fit together."""
    import importlib
    import sys
    from streambrain_amd import datasets

    rng = np.random.default_rng(3)

    def make(n):
        lab = rng.integers(0, 10, n).astype(np.uint8)
        px = (rng.random((n, 784)) < 0.03) * rng.integers(1, 120, (n, 784))
        for k in range(n):
            c = int(lab[k])
            px[k, 78 * c:78 * c + 78] = rng.integers(150, 256, 78)
        return px.astype(np.uint8), lab

    def write(name, header, payload):
        with open(tmp_path / name, "wb") as f:
            f.write(bytes(header))
            f.write(payload.tobytes())

    for split, n in (("train", 1280), ("t10k", 320)):
        px, lab = make(n)
        write(f"{split}-images", [0, 0, 8, 3] + [0] * 12, px)
        write(f"{split}-labels", [0, 0, 8, 1] + [0] * 4, lab)

    monkeypatch.setenv("BCPNN_BACKEND", "hip")
    sys.modules.pop("BCPNN", None)
    BCPNN = importlib.import_module("BCPNN")
    assert BCPNN.backend() == "hip"

    precision = np.float32
    np.random.seed(0)
    train_x, train_y = datasets.load_mnist(tmp_path / "train-images", tmp_path / "train-labels", precision)
    test_x, test_y = datasets.load_mnist(tmp_path / "t10k-images", tmp_path / "t10k-labels", precision)
    train_x, test_x = datasets.complementary(train_x), datasets.complementary(test_x)
    batch = 128
    hp = MNIST_HP
    net = BCPNN.Network(precision)
    net.add_layer(BCPNN.StructuralPlasticityLayer(784 * 2, 15, 20, hp["l1_taupdt"] * 4, hp["l1_khalf"],
                                                  hp["l1_pmin"], hp["l1_taubdt"], 0.3, 16, (1, 1 / 20, 1 / 20)))
    net.add_layer(BCPNN.DenseLayer(15 * 20, 1, 10, hp["l2_taupdt"] * 40, (1 / 20, 1 / 10, 1 / 200)))
    net.fit(train_x, train_y, batch, [(0, 4), (1, 4)])
    correct, total = net.evaluate(train_x, train_y, batch)
    assert total == 1280 and 0 <= correct <= total
    train_acc = correct / total
    correct, total = net.evaluate(test_x, test_y, batch)
    assert total == 320
    test_acc = correct / total
    assert train_acc > 0.5 and test_acc > 0.5, (train_acc, test_acc)


@pytest.mark.parametrize("precision", [np.float32, np.float64])
def test_backend_object_through_the_reference_methods_alone(precision):
    """The C++ backend object driven the way the reference's full_cuda DSL drives its own
    (full_cuda_backend/__init__.py:69-115 there): add_*_layer with the positional arguments, initiate_training,
    train_layer, training_done, evaluate -> accuracy, and nothing else -- no state is handed in.  The object has
    to bring a usable initial state of its own, as the reference's does (backend_full_cuda_internals.cu:151-155,
    helpers_training.cu:10-32): random weights and bias and a mask of density 0.1.  On the learnable toy problem
    of the example-script test: accuracy far above chance, hidden activations that are not uniform, and mask
    columns that hold about a tenth of the inputs."""
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "streambrain_amd"))
    import _bcpnn_backend_hip_internals as backend
    backend.initialize(0)
    rng = np.random.default_rng(3)

    def make(n):
        lab = rng.integers(0, 10, n)
        px = (rng.random((n, 784)) < 0.03) * rng.integers(1, 120, (n, 784))
        for k in range(n):
            c = int(lab[k])
            px[k, 78 * c:78 * c + 78] = rng.integers(150, 256, 78)
        x = (px / 255.0).astype(precision)
        return np.concatenate([x, 1 - x], axis=1), np.eye(10, dtype=precision)[lab]

    train_x, train_y = make(1280)
    test_x, test_y = make(320)
    hp = MNIST_HP
    H, Mc, N = 15, 20, 784 * 2
    net = backend.PyNetwork_float32() if precision == np.float32 else backend.PyNetwork_float64()
    net.seed(1234)  # (the reference seeds from the clock; a fixed seed keeps the test repeatable)
    net.add_plastic_layer(N, H, Mc, hp["l1_taupdt"] * 4, hp["l1_pmin"], hp["l1_khalf"], hp["l1_taubdt"],
                          1, 1 / Mc, 1 / Mc)
    net.add_dense_layer(H * Mc, 1, 10, hp["l2_taupdt"] * 40, 1 / Mc, 1 / 10, 1 / (10 * Mc))

    # the state the object drew for itself
    W0, b0, mask0 = net.get_layer_state(0, "weights"), net.get_layer_state(0, "bias"), net.get_layer_state(0, "wmask")
    assert abs(float(W0.std()) - 0.1) < 0.005 and abs(float(W0.mean())) < 0.002
    assert 0 <= b0.min() and b0.max() <= 0.1 and b0.std() > 0.01
    counts0 = mask0.sum(axis=0)
    assert np.all(np.abs(counts0 - 0.1 * N) < 5 * np.sqrt(0.09 * N)), counts0
    assert net.get_layer_state(1, "weights").std() > 0.05

    net.initiate_training(train_x, train_y)
    net.train_layer(64, 0, 4)  # 20 batches an epoch: with 15 hypercolumns, one rewiring per batch from epoch 1 on
    net.train_layer(128, 1, 4)
    net.training_done()
    train_acc = net.evaluate(train_x, train_y, 128)
    test_acc = net.evaluate(test_x, test_y, 128)
    assert isinstance(train_acc, float) and 0.0 <= train_acc <= 1.0
    assert train_acc > 0.5 and test_acc > 0.5, (train_acc, test_acc)  # chance: 0.1

    # the hidden layer took sides: its softmax outputs are far from the uniform 1 / Mc
    act = net.forward(test_x, 0, 128).reshape(-1, H, Mc)
    assert np.allclose(act.sum(axis=2), 1, atol=1e-4 if precision == np.float32 else 1e-10)
    assert float(act.max(axis=2).mean()) > 3.0 / Mc, float(act.max(axis=2).mean())
    # rewiring swaps connections, so every mask column still holds what it was drawn with
    mask = net.get_layer_state(0, "wmask")
    assert np.array_equal(mask.sum(axis=0), counts0)
    assert (mask != mask0).any(), "three epochs with rewiring moved no connection"
    # weights are zero exactly under the mask (apply_mask)
    W = net.get_layer_state(0, "weights")
    assert np.all(W[np.repeat(mask, Mc, axis=1) == 0] == 0)

    # two objects with the same seed draw the same state
    a = backend.PyNetwork_float32()
    b = backend.PyNetwork_float32()
    for o in (a, b):
        o.seed(7)
        o.add_plastic_layer(64, 3, 4, 0.01, 0.3, -100, 0.01, 1, 0.25, 0.25)
    for name in ("weights", "bias", "wmask"):
        assert np.array_equal(a.get_layer_state(0, name), b.get_layer_state(0, name))


def test_example_driver_on_files_and_synthetic_data(tmp_path, capsys):
    """`python -m streambrain_amd.train` (the reference's train.py command line, train.py:44-215 there): on
    idx-ubyte files written here with a learnable toy problem it trains, saves, and a second network loaded
    from the file evaluates to the same counts; on synthetic data of the dataset's shape it runs through and
    prints the reference's three result lines."""
    from streambrain_amd import train as driver

    rng = np.random.default_rng(5)

    def write(name, header, payload):
        with open(tmp_path / name, "wb") as f:
            f.write(bytes(header))
            f.write(payload.tobytes())

    for split, n in (("train", 1536), ("t10k", 256)):
        lab = rng.integers(0, 10, n).astype(np.uint8)
        px = ((rng.random((n, 784)) < 0.03) * rng.integers(1, 120, (n, 784)))
        for k in range(n):
            px[k, 78 * int(lab[k]):78 * int(lab[k]) + 78] = rng.integers(150, 256, 78)
        write(f"{split}-images-idx3-ubyte", [0, 0, 8, 3] + [0] * 12, px.astype(np.uint8))
        write(f"{split}-labels-idx1-ubyte", [0, 0, 8, 1] + [0] * 4, lab)

    state = tmp_path / "state.npz"
    train_s, test_s, correct, total = driver.run("mnist", np.float32, 128, data_dir=str(tmp_path),
                                                 epochs=(40, 80), save=str(state))
    assert total == 256 and train_s > 0 and test_s > 0
    assert correct / total > 0.3, correct  # (ten classes)
    # the saved state, loaded into a fresh network and trained for no epoch, evaluates to the same counts
    _, _, correct2, total2 = driver.run("mnist", np.float32, 128, data_dir=str(tmp_path), epochs=(0, 0),
                                        load=str(state))
    assert (correct2, total2) == (correct, total)

    capsys.readouterr()
    driver.main(["fashion_mnist", "double", "64", "--synthetic", "384", "--epochs", "1,1"])
    out = capsys.readouterr().out
    assert "Training duration: " in out and "Testing duration:  " in out and "Accuracy:          " in out
    acc = float(out.split("Accuracy:")[1].split()[0])
    assert 0.0 <= acc <= 1.0
