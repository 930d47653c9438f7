"""Readers for the data files the reference's example script trains on (train.py:9-41 there), with the
same conventions, so a run on real data sees byte-identical inputs:

  MNIST / Fashion-MNIST  idx-ubyte files: 16 header bytes (images) / 8 (labels) are skipped, pixels are
                         divided by 255, labels become one-hot rows of 10;
  STL-10                 flat uint8 files, 3*96*96 bytes per image, pixels / 255; label bytes are 1..10
                         and become one-hot rows of 10 after subtracting 1.

`complementary` appends (1 - x) to every row, the two-minicolumn input coding of the benchmark
configurations.  The files themselves are not shipped (the reference's README says where to fetch
them); nothing here touches the network.
"""
import numpy as np


def load_mnist(image_file, label_file, dtype=np.float64):
    imgs = np.fromfile(image_file, dtype=np.uint8)[16:]
    if imgs.size % (28 * 28):
        raise ValueError(f"{image_file}: {imgs.size} pixel bytes are not a whole number of 28x28 images")
    imgs = imgs.reshape(-1, 28 * 28).astype(dtype)
    imgs /= 255.0
    lab = np.fromfile(label_file, dtype=np.uint8)[8:]
    if lab.shape[0] != imgs.shape[0]:
        raise ValueError(f"{label_file}: {lab.shape[0]} labels for {imgs.shape[0]} images")
    if lab.size and lab.max() > 9:
        raise ValueError(f"{label_file}: label {int(lab.max())} is not a digit class")
    labels = np.zeros((lab.shape[0], 10), dtype=dtype)
    labels[np.arange(lab.shape[0]), lab] = 1.0
    return imgs, labels


def load_stl_10_images(file):
    data = np.fromfile(file, dtype=np.uint8)
    if data.size % (3 * 96 * 96):
        raise ValueError(f"{file}: {data.size} bytes are not a whole number of 3x96x96 images")
    return data.reshape(-1, 3 * 96 * 96) / 255.0


def load_stl_10_labels(file):
    lab = np.fromfile(file, dtype=np.uint8)
    if lab.size and (lab.min() < 1 or lab.max() > 10):
        raise ValueError(f"{file}: labels must be 1..10")
    lab = lab - 1
    labels = np.zeros((lab.shape[0], 10))
    labels[np.arange(lab.shape[0]), lab] = 1.0
    return labels


def complementary(images):
    """(x, 1 - x): every input unit becomes a hypercolumn of two minicolumns."""
    images = np.asarray(images)
    return np.concatenate([images, 1.0 - images], axis=1)
