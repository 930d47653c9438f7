"""The dataset readers against the reference's conventions (train.py:9-41 there) on synthetic files, and
the checkpoint round trip on the CPU oracle's network (same layer attributes as the hip backend)."""
import numpy as np
import pytest

from streambrain_amd import datasets


def _write(path, header, payload):
    with open(path, "wb") as f:
        f.write(bytes(header))
        f.write(np.asarray(payload, dtype=np.uint8).tobytes())


def test_mnist_reader(tmp_path):
    rng = np.random.default_rng(0)
    px = rng.integers(0, 256, size=(7, 28 * 28), dtype=np.uint8)
    lab = rng.integers(0, 10, size=7, dtype=np.uint8)
    # idx3 / idx1 headers: magic, counts, dimensions -- the reader skips 16 and 8 bytes unseen
    _write(tmp_path / "img", [0, 0, 8, 3, 0, 0, 0, 7, 0, 0, 0, 28, 0, 0, 0, 28], px)
    _write(tmp_path / "lab", [0, 0, 8, 1, 0, 0, 0, 7], lab)
    for dtype in (np.float32, np.float64):
        imgs, labels = datasets.load_mnist(tmp_path / "img", tmp_path / "lab", dtype=dtype)
        assert imgs.dtype == dtype and labels.dtype == dtype
        assert imgs.shape == (7, 784) and labels.shape == (7, 10)
        ref = px.astype(dtype)
        ref /= 255.0
        assert np.array_equal(imgs, ref)
        assert np.array_equal(labels.argmax(1), lab) and np.all(labels.sum(1) == 1)


def test_mnist_reader_rejects_ragged_files(tmp_path):
    _write(tmp_path / "img", [0] * 16, np.zeros(784 + 5))
    _write(tmp_path / "lab", [0] * 8, [1])
    with pytest.raises(ValueError):
        datasets.load_mnist(tmp_path / "img", tmp_path / "lab")
    _write(tmp_path / "img", [0] * 16, np.zeros(784 * 2))
    with pytest.raises(ValueError):
        datasets.load_mnist(tmp_path / "img", tmp_path / "lab")  # 1 label, 2 images


def test_stl10_readers(tmp_path):
    rng = np.random.default_rng(1)
    px = rng.integers(0, 256, size=(3, 3 * 96 * 96), dtype=np.uint8)
    lab = np.array([1, 10, 4], dtype=np.uint8)
    _write(tmp_path / "x", [], px)
    _write(tmp_path / "y", [], lab)
    imgs = datasets.load_stl_10_images(tmp_path / "x")
    labels = datasets.load_stl_10_labels(tmp_path / "y")
    assert imgs.dtype == np.float64 and np.array_equal(imgs, px / 255.0)
    assert labels.argmax(1).tolist() == [0, 9, 3]
    _write(tmp_path / "y", [], [0, 3])
    with pytest.raises(ValueError):
        datasets.load_stl_10_labels(tmp_path / "y")


def test_complementary_coding():
    x = np.array([[0.0, 0.25], [1.0, 0.5]])
    assert np.array_equal(datasets.complementary(x), [[0.0, 0.25, 1.0, 0.75], [1.0, 0.5, 0.0, 0.5]])


def test_checkpoint_round_trip(tmp_path):
    from helpers import MNIST_HP, build_two_layer, one_hot_labels, synthetic_images
    from oracle import cpu_backend as ob
    from streambrain_amd import checkpoint
    rng = np.random.default_rng(3)
    X, Y = synthetic_images(rng, 40, 12), one_hot_labels(rng, 40, 3)
    net = build_two_layer(ob, 24, 2, 4, 3, MNIST_HP, np.float32, seed=1)
    net.fit(X, Y, 16, [(0, 2), (1, 1)])
    checkpoint.save_state(net, tmp_path / "state.npz")
    other = build_two_layer(ob, 24, 2, 4, 3, MNIST_HP, np.float32, seed=2)
    checkpoint.load_state(other, tmp_path / "state.npz")
    for a, b in zip(net._layers, other._layers):
        for name in ("weights", "bias", "Ci", "Cj", "Cij"):
            assert np.array_equal(getattr(a, name), getattr(b, name)), name
    assert np.array_equal(net._layers[0].wmask, other._layers[0].wmask)
    assert np.array_equal(net.predict(X, 16), other.predict(X, 16))
    wrong = build_two_layer(ob, 24, 2, 5, 3, MNIST_HP, np.float32, seed=2)
    with pytest.raises(ValueError):
        checkpoint.load_state(wrong, tmp_path / "state.npz")


def test_example_driver_command_line_and_presets():
    """The driver's presets are the reference's published hyper-parameters (train.py:71-139 there; a few
    spot values), its command line rejects what the reference's rejects, and its synthetic data has the
    dataset's shapes."""
    import pytest
    from streambrain_amd import train as driver

    assert set(driver.PRESETS) == {"mnist", "fashion_mnist", "stl-10"}
    m, f, s = (driver.PRESETS[k] for k in ("mnist", "fashion_mnist", "stl-10"))
    assert (m.hypercolumns, f.hypercolumns, s.hypercolumns) == (15, 30, 15)
    assert (m.epochs, f.epochs, s.epochs) == ((30, 60), (30, 60), (100, 20))
    assert m.khalf == -139.02586632856327 and s.mask_iterations == 584 and s.n_inputs == 27648
    assert f.classifier_taupdt == 0.00202951854188782 and s.unlabeled_rows == 15000
    with pytest.raises(SystemExit):
        driver.main(["cifar", "single", "128"])
    with pytest.raises(SystemExit):
        driver.main(["mnist", "half", "128"])
    with pytest.raises(SystemExit):
        driver.main(["mnist", "single", "128", "--epochs", "3"])
    with pytest.raises(ValueError):
        driver.run("mnist", np.float32, 0, synthetic=8)
    hx, hy, tx, ty, ex, ey = driver.synthetic_data(s, 12, np.float64)
    assert hx.shape == (12, 27648) and hy.shape == (12, 10) and not hy.any()
    assert tx.shape == (12, 27648) and ty.sum() == 12 and ex.shape == (2, 27648) and ey.shape == (2, 10)
    hx, hy, tx, ty, ex, ey = driver.synthetic_data(m, 12, np.float32)
    assert hx is tx and hy is ty and hx.dtype == np.float32 and 0 <= hx.min() and hx.max() <= 1
