"""Example run on one MI355X with the command line of the reference's example script (train.py:44-215
there): `python -m streambrain_amd.train <mnist/fashion_mnist/stl-10> <single/double> <batch size>`.

It builds the reference's two-layer network for the dataset (a structural-plasticity layer of 3000 hidden
units in 15 or 30 hypercolumns, a dense classification layer of 10), trains the hidden layer and then the
classifier for the reference's numbers of epochs with its published hyper-parameters (time constants scaled
by sqrt(batch / 128) as there), evaluates on the test set and prints the three lines the reference prints:
training duration, testing duration, accuracy.  The data files are read from --data-dir with the readers of
`streambrain_amd.datasets` (same file names as the reference: train-images-idx3-ubyte, ..., unlabeled_X.bin,
...).  `--synthetic N` replaces them by N random samples of the dataset's shape, for a run without the files;
`--epochs A,B` shortens the schedule; `--save` / `--load` write / read the network's state as .npz.

One process, one GPU: the reference's MPI launch (mpirun -n R python train.py ...) has no counterpart here.
"""
import argparse
import math
import os
import time
from dataclasses import dataclass

import numpy as np


@dataclass(frozen=True)
class Preset:
    """Hyper-parameters of one dataset (train.py:71-139 of the reference)."""
    hypercolumns: int
    taupdt: float
    pmin: float
    khalf: float
    taubdt: float
    density: float
    mask_iterations: int
    classifier_taupdt: float
    epochs: tuple
    n_inputs: int
    unlabeled_rows: int = 0   # > 0: the hidden layer trains on this many rows of a separate unlabeled file


PRESETS = {
    "mnist": Preset(15, 0.006908854922437549, 0.06195283356566607, -139.02586632856327, 0.02218100432360414,
                    0.1, 16, 0.0007449780036161324, (30, 60), 28 * 28),
    "fashion_mnist": Preset(30, 0.0014712266428529468, 0.10328182984859212, -160.06386313883948,
                            0.0008418555122620076, 0.1, 16, 0.00202951854188782, (30, 60), 28 * 28),
    "stl-10": Preset(15, 0.0006510421564830368, 0.0070169782620369365, 1666.644815059196,
                     0.0024793529936481956, 0.568746541818903, 584, 4.983000352087509e-07, (100, 20),
                     3 * 96 * 96, unlabeled_rows=15000),
}
HIDDEN_UNITS = 3000
CLASSES = 10


def _one_hot(labels, dtype):
    out = np.zeros((labels.shape[0], CLASSES), dtype=dtype)
    out[np.arange(labels.shape[0]), labels] = 1.0
    return out


def synthetic_data(preset, n, dtype, seed=0):
    """(hidden-layer training set, its labels, classifier training set, its labels, test set, its labels) of
    random pixels in [0, 1] and random classes: the shapes of the real files, none of their content."""
    rng = np.random.default_rng(seed)
    def images(rows):
        return rng.random((rows, preset.n_inputs), dtype=np.float32).astype(dtype)
    train_x, train_y = images(n), _one_hot(rng.integers(0, CLASSES, n), dtype)
    test_rows = max(1, n // 6)
    test_x, test_y = images(test_rows), _one_hot(rng.integers(0, CLASSES, test_rows), dtype)
    if preset.unlabeled_rows:
        hidden_x = images(n)
        return hidden_x, np.zeros((n, CLASSES), dtype=dtype), train_x, train_y, test_x, test_y
    return train_x, train_y, train_x, train_y, test_x, test_y


def file_data(name, preset, data_dir, dtype):
    from streambrain_amd import datasets
    path = lambda f: os.path.join(data_dir, f)
    if not preset.unlabeled_rows:
        train_x, train_y = datasets.load_mnist(path("train-images-idx3-ubyte"), path("train-labels-idx1-ubyte"),
                                               dtype=dtype)
        test_x, test_y = datasets.load_mnist(path("t10k-images-idx3-ubyte"), path("t10k-labels-idx1-ubyte"),
                                             dtype=dtype)
        return train_x, train_y, train_x, train_y, test_x, test_y
    hidden_x = datasets.load_stl_10_images(path("unlabeled_X.bin"))[:preset.unlabeled_rows, :]
    return (hidden_x, np.zeros((hidden_x.shape[0], CLASSES)),
            datasets.load_stl_10_images(path("train_X.bin")), datasets.load_stl_10_labels(path("train_y.bin")),
            datasets.load_stl_10_images(path("test_X.bin")), datasets.load_stl_10_labels(path("test_y.bin")))


def build_network(preset, dtype, batch_size):
    """The reference's network for the preset (train.py:144-179 there), on the hip backend."""
    import BCPNN
    scale = math.sqrt(batch_size / 128)
    minicolumns = HIDDEN_UNITS // preset.hypercolumns
    hidden = preset.hypercolumns * minicolumns
    net = BCPNN.Network(dtype)
    net.add_layer(BCPNN.StructuralPlasticityLayer(
        preset.n_inputs, preset.hypercolumns, minicolumns, preset.taupdt * scale, preset.khalf, preset.pmin,
        preset.taubdt, preset.density, preset.mask_iterations,
        (1, 1 / minicolumns, 1 / minicolumns)))
    net.add_layer(BCPNN.DenseLayer(
        hidden, 1, CLASSES, preset.classifier_taupdt * scale,
        (1 / minicolumns, 1 / CLASSES, 1 / minicolumns / CLASSES)))
    return net


def run(dataset, dtype, batch_size, data_dir=".", synthetic=0, epochs=None, save=None, load=None, seed=0):
    """Trains and evaluates; returns (training seconds, testing seconds, correct, total)."""
    if dataset not in PRESETS:
        raise ValueError("Unknown dataset: %r (one of %s)" % (dataset, ", ".join(PRESETS)))
    if batch_size <= 0:
        raise ValueError("batch size must be positive")
    preset = PRESETS[dataset]
    np.random.seed(seed)  # the epoch permutations come from numpy's global generator, as in the reference
    data = (synthetic_data(preset, synthetic, dtype, seed) if synthetic
            else file_data(dataset, preset, data_dir, dtype))
    hidden_x, hidden_y, train_x, train_y, test_x, test_y = data
    net = build_network(preset, dtype, batch_size)
    if load:
        from streambrain_amd import checkpoint
        checkpoint.load_state(net, load)
    hidden_epochs, classifier_epochs = epochs if epochs is not None else preset.epochs
    start = time.time()
    net.fit(hidden_x, hidden_y, batch_size, [(0, hidden_epochs)])
    net.fit(train_x, train_y, batch_size, [(1, classifier_epochs)])
    trained = time.time()
    correct, total = net.evaluate(test_x, test_y, batch_size)
    tested = time.time()
    if save:
        from streambrain_amd import checkpoint
        checkpoint.save_state(net, save)
    return trained - start, tested - trained, int(np.asarray(correct).sum()), int(np.asarray(total).sum())


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m streambrain_amd.train", description=__doc__.split("\n\n")[0])
    ap.add_argument("dataset", choices=sorted(PRESETS))
    ap.add_argument("precision", choices=("single", "double"))
    ap.add_argument("batch_size", type=int)
    ap.add_argument("--data-dir", default=".")
    ap.add_argument("--synthetic", type=int, default=0, metavar="N")
    ap.add_argument("--epochs", default=None, metavar="A,B")
    ap.add_argument("--save", default=None, metavar="FILE.npz")
    ap.add_argument("--load", default=None, metavar="FILE.npz")
    a = ap.parse_args(argv)
    dtype = np.float32 if a.precision == "single" else np.float64
    epochs = tuple(int(e) for e in a.epochs.split(",")) if a.epochs else None
    if epochs is not None and len(epochs) != 2:
        ap.error("--epochs takes two numbers: hidden layer, classifier")
    print('Dataset:', a.dataset, 'Batch size:', a.batch_size, 'precision:', dtype)
    train_s, test_s, correct, total = run(a.dataset, dtype, a.batch_size, a.data_dir, a.synthetic, epochs,
                                          a.save, a.load)
    print('Training duration: ' + str(train_s))
    print('Testing duration:  ' + str(test_s))
    print('Accuracy:          ' + str(correct / total))


if __name__ == "__main__":
    main()
