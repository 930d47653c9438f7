"""The oracle's DSL-level restatement (oracle/cpu_backend.py) against a trajectory recorded from the
reference's own Python driver (tests/golden/driver_trajectory_f64.npz, written by
tests/golden/make_driver_trajectory.py): RNG draw order, batch slicing, rewiring schedule, finalize
cadence, evaluate count -- and, end to end, every kernel of the oracle."""
import os

import numpy as np
import pytest

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "driver_trajectory_f64.npz")


@pytest.fixture(scope="module")
def golden():
    return np.load(FIX)


def build_net(backend, g, dtype=np.float64, **kw):
    c = {k[4:]: g[k].item() for k in g.files if k.startswith("cfg_")}
    np.random.seed(int(c["net_seed"]))
    net = backend.Network(dtype)
    net.add_layer(backend.StructuralPlasticityLayer(
        int(c["n_in"]), int(c["H"]), int(c["Mc"]), c["l1_taupdt"], c["l1_khalf"], c["l1_pmin"],
        c["l1_taubdt"], c["l1_density"], int(c["l1_mask_iterations"]),
        (1, 1 / int(c["Mc"]), 1 / int(c["Mc"])), **kw))
    net.add_layer(backend.DenseLayer(
        int(c["H"]) * int(c["Mc"]), 1, int(c["n_out"]), c["l2_taupdt"],
        (1 / int(c["Mc"]), 1 / int(c["n_out"]), 1 / int(c["Mc"]) / int(c["n_out"])), **kw))
    return net, c


def test_oracle_driver_reproduces_reference_trajectory(golden):
    from oracle import cpu_backend as ob
    g = golden
    net, c = build_net(ob, g)
    l0, l1 = net._layers
    assert np.array_equal(l0.weights, g["init_L0_weights"]) and np.array_equal(l0.bias, g["init_L0_bias"])
    assert np.array_equal(l0.wmask, g["init_L0_wmask"])
    assert np.array_equal(l1.weights, g["init_L1_weights"]) and np.array_equal(l1.bias, g["init_L1_bias"])

    net.fit(g["X"], g["Y"], int(c["B"]), [(0, int(c["l1_epochs"]))])
    assert not np.array_equal(g["mid_L0_wmask"], g["init_L0_wmask"])  # the fixture does rewire
    assert np.array_equal(l0.wmask, g["mid_L0_wmask"])
    for name in ("weights", "bias", "Ci", "Cj", "Cij", "kbi"):
        np.testing.assert_allclose(getattr(l0, name), g[f"mid_L0_{name}"], rtol=1e-10, atol=1e-12,
                                   err_msg=name)
    net.fit(g["X"], g["Y"], int(c["B"]), [(1, int(c["l2_epochs"]))])
    for li, layer in enumerate((l0, l1)):
        for name in ("weights", "bias", "Ci", "Cj", "Cij"):
            np.testing.assert_allclose(getattr(layer, name), g[f"final_L{li}_{name}"], rtol=1e-10,
                                       atol=1e-12, err_msg=f"L{li}.{name}")
    correct, total = net.evaluate(g["Xt"], g["Yt"], int(c["B"]))
    assert correct.tolist() == g["correct"].tolist() and total.tolist() == g["total"].tolist()
    assert np.array_equal(net.predict(g["Xt"], int(c["B"])), g["test_predictions"])
    np.testing.assert_allclose(net.forward(g["Xt"]), g["test_activations"], rtol=1e-10)
    # the global RNG stream has been advanced by exactly the reference's number of draws
    np.testing.assert_array_equal(np.random.rand(4), g["rng_probe_after"])


def test_rewire_schedule_matches_reference_rule():
    from oracle.cpu_backend import rewire_schedule
    perm = list(range(30))[::-1]
    # MNIST shape: 469 batches, 30 hypercolumns -> every 15th step, hypercolumns perm[0..29], then none
    hits = [(i, rewire_schedule(1, i, 469, 30, perm)) for i in range(469)]
    fired = [(i, h) for i, h in hits if h is not None]
    assert [i for i, _ in fired] == list(range(0, 450, 15))
    assert [h for _, h in fired] == perm
    assert all(rewire_schedule(0, i, 469, 30, perm) is None for i in range(469))
    with pytest.raises(ZeroDivisionError):
        rewire_schedule(1, 0, 20, 200, list(range(200)))
