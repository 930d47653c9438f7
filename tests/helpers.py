"""Shared builders for the network-level tests."""
import numpy as np

# train.py:77-85 (MNIST hyper-parameters of the reference's example script)
MNIST_HP = dict(l1_taupdt=0.006908854922437549, l1_pmin=0.06195283356566607,
                l1_khalf=-139.02586632856327, l1_taubdt=0.02218100432360414, l1_density=0.1,
                l1_mask_iterations=16, l2_taupdt=0.0007449780036161324)


def fixture_config(g):
    return {k[4:]: g[k].item() for k in g.files if k.startswith("cfg_")}


def build_two_layer(backend, n_in, H, Mc, n_out, hp, dtype, seed=0, density=None):
    """The network of train.py:151-179: a structural-plasticity layer and a 1 x n_out dense layer,
    constructed after np.random.seed(seed) so every backend draws the same initial state."""
    np.random.seed(seed)
    net = backend.Network(dtype)
    net.add_layer(backend.StructuralPlasticityLayer(
        n_in, H, Mc, hp["l1_taupdt"], hp["l1_khalf"], hp["l1_pmin"], hp["l1_taubdt"],
        hp["l1_density"] if density is None else density, int(hp["l1_mask_iterations"]),
        (1, 1 / Mc, 1 / Mc)))
    net.add_layer(backend.DenseLayer(H * Mc, 1, n_out, hp["l2_taupdt"],
                                     (1 / Mc, 1 / n_out, 1 / Mc / n_out)))
    return net


def synthetic_images(rng, n, n_pixels, p_nonzero=0.19):
    """Complementary-coded synthetic images: each pixel nonzero with probability p_nonzero, uniform in
    (0, 1]; the input is (x, 1 - x)."""
    px = (1.0 - rng.random((n, n_pixels))) * (rng.random((n, n_pixels)) < p_nonzero)
    return np.concatenate([px, 1.0 - px], axis=1)


def one_hot_labels(rng, n, n_classes):
    lab = np.zeros((n, n_classes))
    lab[np.arange(n), rng.integers(0, n_classes, n)] = 1.0
    return lab


def rel_err(a, ref, what=None, tol=float("nan")):
    """max |a - ref| / max(|ref|, 1); with `what`, the value is also recorded for the measured-error table."""
    a = np.asarray(a, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    e = float(np.max(np.abs(a - ref) / np.maximum(np.abs(ref), 1.0))) if a.size else 0.0
    if what is not None:
        record_error(what, e, tol)
    return e


# Measured parity errors of the GPU tests, by test id and quantity: (error, tolerance asserted).  The
# session hook in conftest.py writes them out, so the bound a test asserts can be compared with what was
# measured.
MEASURED = {}


def record_error(what, e, tol):
    import os
    test = os.environ.get("PYTEST_CURRENT_TEST", "?").split(" ")[0]
    MEASURED.setdefault(test, []).append((what, float(e), float(tol)))
