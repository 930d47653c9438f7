"""Saving and restoring the learned state of a network: the seven arrays of every layer (weights, bias,
Ci, Cj, Cij, kbi, wmask -- the attributes of the reference's layers, _cpu_base_backend.py:24-42,
100-124 there) in one .npz file.  The reference has no checkpoint format of its own; this one holds
plain numpy arrays only, so it loads without executing anything (allow_pickle stays off)."""
import numpy as np

_NAMES = ("weights", "bias", "Ci", "Cj", "Cij", "kbi", "wmask")


def save_state(network, path):
    arrays = {"n_layers": np.asarray(len(network._layers))}
    for li, layer in enumerate(network._layers):
        for name in _NAMES:
            if hasattr(layer, name):
                value = getattr(layer, name)
                if value is not None:
                    arrays[f"L{li}_{name}"] = np.asarray(value)
    np.savez(path, **arrays)


def load_state(network, path):
    """Copies the saved arrays into the layers of `network`, which must have been built with the same
    architecture (shapes are checked)."""
    with np.load(path, allow_pickle=False) as data:
        if int(data["n_layers"]) != len(network._layers):
            raise ValueError(f"{path} holds {int(data['n_layers'])} layers, the network has "
                             f"{len(network._layers)}")
        for li, layer in enumerate(network._layers):
            for name in _NAMES:
                key = f"L{li}_{name}"
                if key not in data.files:
                    continue
                current = np.asarray(getattr(layer, name))
                if current.shape != data[key].shape:
                    raise ValueError(f"{key}: saved shape {data[key].shape}, layer has {current.shape}")
                setattr(layer, name, data[key].astype(current.dtype))
