"""Writes tests/golden/driver_trajectory_f64.npz.

The per-batch kernels of the oracle are pinned by closed forms and brute force
(tests/test_oracle_pins.py).  What those cannot pin is the reference's Python DRIVER: the numpy RNG
draw order at layer construction and per epoch, the batch slicing with a short last batch, the
hypercolumn rewiring schedule, the per-epoch finalize and the evaluate count
(BCPNN/backend/_cpu_base_backend.py:175-314).  This script runs that driver ONCE, in the build
container only, on the reference's pure-numpy backend (BCPNN_BACKEND=numpy, float64, a tiny network)
and stores the inputs and the final state as a fixture.  The reference itself never travels.

Known, documented differences between the numpy backend used here and the cpu backend the oracle
restates, none of which is visible in this fixture's final state:
  * dense-layer weights are recomputed at finalize instead of every step -- same final W;
  * the mask score uses `>` instead of `>=` against cthr -- differs only at exact equality;
  * the moving averages are evaluated as (1-t)*C + t*mean -- rounding-level (1e-16) differences.

Usage (build container, reference mounted):  python tests/golden/make_driver_trajectory.py
"""
import os
import sys

import numpy as np

REFERENCE = "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "driver_trajectory_f64.npz")

CFG = dict(n_in=24, H=3, Mc=4, n_out=5, Ns=70, Ntest=23, B=16, l1_epochs=3, l2_epochs=2,
           l1_taupdt=0.02, l1_khalf=-50.0, l1_pmin=0.1, l1_taubdt=0.05, l1_density=0.3,
           l1_mask_iterations=16, l2_taupdt=0.01, data_seed=2024, net_seed=0)


def make_data(cfg):
    rng = np.random.default_rng(cfg["data_seed"])  # separate stream: never touches np.random
    def images(n):
        px = rng.random((n, cfg["n_in"] // 2)) * (rng.random((n, cfg["n_in"] // 2)) < 0.4)
        return np.concatenate([px, 1.0 - px], axis=1)
    def labels(n):
        lab = np.zeros((n, cfg["n_out"]))
        lab[np.arange(n), rng.integers(0, cfg["n_out"], n)] = 1.0
        return lab
    return images(cfg["Ns"]), labels(cfg["Ns"]), images(cfg["Ntest"]), labels(cfg["Ntest"])


def main():
    os.environ["BCPNN_BACKEND"] = "numpy"
    sys.path.insert(0, REFERENCE)
    import BCPNN  # the reference package, numpy backend

    cfg = CFG
    X, Y, Xt, Yt = make_data(cfg)
    np.random.seed(cfg["net_seed"])
    net = BCPNN.Network(np.float64)
    net.add_layer(BCPNN.StructuralPlasticityLayer(
        cfg["n_in"], cfg["H"], cfg["Mc"], cfg["l1_taupdt"], cfg["l1_khalf"], cfg["l1_pmin"],
        cfg["l1_taubdt"], cfg["l1_density"], cfg["l1_mask_iterations"],
        (1, 1 / cfg["Mc"], 1 / cfg["Mc"])))
    net.add_layer(BCPNN.DenseLayer(
        cfg["H"] * cfg["Mc"], 1, cfg["n_out"], cfg["l2_taupdt"],
        (1 / cfg["Mc"], 1 / cfg["n_out"], 1 / cfg["Mc"] / cfg["n_out"])))
    out = {"X": X, "Y": Y, "Xt": Xt, "Yt": Yt}
    for li, layer in enumerate(net._layers):
        out[f"init_L{li}_weights"] = layer.weights.copy()
        out[f"init_L{li}_bias"] = layer.bias.copy()
    out["init_L0_wmask"] = net._layers[0].wmask.copy()
    net.fit(X, Y, cfg["B"], [(0, cfg["l1_epochs"])])
    l0 = net._layers[0]
    for name in ("weights", "bias", "Ci", "Cj", "Cij", "kbi", "wmask"):
        out[f"mid_L0_{name}"] = np.array(getattr(l0, name)).copy()
    net.fit(X, Y, cfg["B"], [(1, cfg["l2_epochs"])])
    for li, layer in enumerate(net._layers):
        for name in ("weights", "bias", "Ci", "Cj", "Cij"):
            out[f"final_L{li}_{name}"] = np.array(getattr(layer, name)).copy()
    correct, total = net.evaluate(Xt, Yt, cfg["B"])
    act = Xt
    for layer in net._layers:
        act = layer.compute_activation(act)
    out["test_activations"] = act
    out["test_predictions"] = np.argmax(act, axis=1).astype(np.int32)
    out["correct"] = np.asarray(correct).copy()
    out["total"] = np.asarray(total).copy()
    out["rng_probe_after"] = np.random.rand(4)  # position of the global stream after the run
    for k, v in cfg.items():
        out["cfg_" + k] = np.asarray(v)
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, {k: v.shape for k, v in out.items() if not k.startswith("cfg_")})


if __name__ == "__main__":
    main()
