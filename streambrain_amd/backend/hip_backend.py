"""BCPNN_BACKEND=hip: the layer/network DSL on the MI355X backend object.

Exports the three names every StreamBrain backend module exports -- DenseLayer,
StructuralPlasticityLayer, Network (BCPNN/__init__.py:15-36 star-imports them) -- with the
constructor signatures and call protocol of the reference (BCPNN/backend/_cpu_base_backend.py:7-21,
71-92, 175-205; train.py:151-189 fixes the positional order).

Division of labour, chosen so that results are seed-identical to the reference's cpu backend:
  * Python keeps everything that draws from numpy's global RNG, in the reference's order: initial
    weights / bias / mask at layer construction (_cpu_base_backend.py:31-36, 107-124), and per epoch
    the sample permutation followed by the hypercolumn permutation (:258-264);
  * all state and all arithmetic live on the GPU, in one C++ object per network
    (_bcpnn_backend_hip_internals.PyNetwork_float32/64, the shape of the reference's full_cuda
    backend object, full_cuda_backend/__init__.py:56-115); a whole epoch is enqueued per call.

Semantics follow the cpu backend (cpu_backend.py): fused trace+weight update every step for both
layer types, dense-layer bias at train_finalize (once per epoch), 16 mask iterations regardless of the
constructor argument, rewiring schedule of _cpu_base_backend.py:297-302.  One documented deviation:
when number_of_batches // (hypercolumns + 1) is 0 the reference raises ZeroDivisionError from the
second epoch on; here no rewiring takes place.
"""
import os
import sys

import numpy as np

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if _PKG not in sys.path:
    sys.path.insert(0, _PKG)
try:
    import _bcpnn_backend_hip_internals as _backend
except ImportError as exc:  # no fallback: the GPU module is the backend
    raise ImportError(
        "BCPNN_BACKEND=hip needs the native module _bcpnn_backend_hip_internals and libsbhip.so; "
        "build them with `python -m streambrain_amd.build`") from exc

_backend.initialize(int(os.environ.get("BCPNN_HIP_DEVICE", "0")))

# Progress bars as in the reference's fit (tqdm on rank 0), when tqdm is installed and BCPNN_HIP_PROGRESS is
# not 0.  A bar costs one device synchronization per range of batches, _PROGRESS_RANGES per epoch.
_PROGRESS_RANGES = 20
_tqdm = None
if os.environ.get("BCPNN_HIP_PROGRESS", "1") != "0":
    try:
        from tqdm import tqdm as _tqdm
    except ImportError:
        _tqdm = None


_FLOAT_STATE = ("weights", "bias", "Ci", "Cj", "Cij")


class _DeviceLayer:
    """State lives in numpy until the layer joins a Network, then in HBM; attribute access
    (layer.weights, .bias, .Ci, .Cj, .Cij, .kbi, .wmask) reads it back, assignment writes it."""

    _state_names = _FLOAT_STATE  # arrays in the network dtype
    _all_names = _FLOAT_STATE

    def _init_common(self, in_features, hypercolumns, minicolumns, taupdt, initial_counters, dtype):
        d = self.__dict__
        d["_net"] = None
        d["_index"] = None
        d["_host"] = {}
        self.in_features = in_features
        self.hypercolumns = hypercolumns
        self.minicolumns = minicolumns
        self.out_features = hypercolumns * minicolumns
        self.taupdt = taupdt
        self.initial_counters = initial_counters
        self.dtype = dtype
        n, m = in_features, self.out_features
        host = self._host
        # RNG draw order of the reference: weights, then bias
        host["weights"] = (0.1 * np.random.randn(n, m)).astype(dtype)
        host["bias"] = (0.1 * np.random.rand(m)).astype(dtype)
        host["Ci"] = initial_counters[0] * np.ones([n]).astype(dtype)
        host["Cj"] = initial_counters[1] * np.ones([m]).astype(dtype)
        host["Cij"] = initial_counters[2] * np.ones([n, m]).astype(dtype)

    def __getattr__(self, name):
        # only reached when normal lookup fails, i.e. for the state arrays
        d = self.__dict__
        if name in type(self)._all_names:
            if d.get("_net") is not None:
                return d["_net"].get_layer_state(d["_index"], name)
            host = d.get("_host", {})
            if name in host:
                return host[name]
        raise AttributeError(name)

    def __setattr__(self, name, value):
        if name in type(self)._all_names:
            if self._net is not None:
                self._net.set_layer_state(self._index, name, np.ascontiguousarray(value))
            else:
                self._host[name] = value
            return
        self.__dict__[name] = value

    def convert(self, dtype):
        self.dtype = dtype
        if self._net is None:
            for name in type(self)._state_names:
                self._host[name] = self._host[name].astype(dtype)

    # ---- the layer-level calls of the reference's layers (_cpu_base_backend.py:44-68, 126-172;
    # cpu_backend.py:13-18, 29-52), on the layer's state in HBM
    def _attached(self, what):
        if self._net is None:
            raise RuntimeError(f"{what}: the layer's state lives on the GPU once it has been added to a "
                               "Network (Network.add_layer); add it first")
        return self._net

    def compute_activation(self, inputs):
        net = self._attached("compute_activation")
        return net.layer_activation(self._index, np.ascontiguousarray(inputs, dtype=self.dtype))

    def train_step(self, inputs, outputs, hypercolumn=None):
        net = self._attached("train_step")
        if hypercolumn is not None and not isinstance(self, StructuralPlasticityLayer):
            raise TypeError("train_step: only a StructuralPlasticityLayer takes a hypercolumn")
        net.layer_train_step(self._index, np.ascontiguousarray(inputs, dtype=self.dtype),
                             np.ascontiguousarray(outputs, dtype=self.dtype),
                             -1 if hypercolumn is None else int(hypercolumn))

    def train_finalize(self):
        self._attached("train_finalize").layer_train_finalize(self._index)

    def _upload(self, net, index):
        for name, value in self._host.items():
            net.set_layer_state(index, name, np.ascontiguousarray(value))
        self.__dict__["_net"] = net
        self.__dict__["_index"] = index
        self.__dict__["_host"] = {}


class DenseLayer(_DeviceLayer):
    def __init__(self, in_features, hypercolumns, minicolumns, taupdt, initial_counters,
                 dtype=np.float64):
        self._init_common(in_features, hypercolumns, minicolumns, taupdt, initial_counters, dtype)


class StructuralPlasticityLayer(_DeviceLayer):
    _state_names = _FLOAT_STATE + ("kbi",)
    _all_names = _state_names + ("wmask",)

    def __init__(self, in_features, hypercolumns, minicolumns, taupdt, khalf, pmin, taubdt, density,
                 mask_iterations, initial_counters, dtype=np.float64):
        self._init_common(in_features, hypercolumns, minicolumns, taupdt, initial_counters, dtype)
        self.khalf = khalf
        self.pmin = pmin
        self.taubdt = taubdt
        self.density = density
        self.mask_iterations = mask_iterations  # kept for the signature; the cpu backend uses 16
        self._host["kbi"] = np.ones([self.out_features]).astype(dtype)
        # third draw of the layer: the receptive-field mask
        self._host["wmask"] = (np.random.rand(in_features, hypercolumns) < density).astype(np.uint8)


class Network:
    def __init__(self, dtype):
        self.dtype = dtype
        self._layers = []
        self.world_rank = 0
        self.world_size = 1
        if dtype == np.float32:
            self.net = _backend.PyNetwork_float32()
        elif dtype == np.float64:
            self.net = _backend.PyNetwork_float64()
        else:
            raise Exception("Unsupported dtype")

    def add_layer(self, layer):
        if layer.dtype != self.dtype:
            layer.convert(self.dtype)
        cs = layer.initial_counters
        if isinstance(layer, StructuralPlasticityLayer):
            index = self.net.add_plastic_layer(layer.in_features, layer.hypercolumns,
                                               layer.minicolumns, layer.taupdt, layer.pmin,
                                               layer.khalf, layer.taubdt, cs[0], cs[1], cs[2],
                                               randomize=False)
        elif isinstance(layer, DenseLayer):
            index = self.net.add_dense_layer(layer.in_features, layer.hypercolumns, layer.minicolumns,
                                             layer.taupdt, cs[0], cs[1], cs[2], randomize=False)
        else:
            raise Exception("Unknown layer type:", layer)
        layer._upload(self.net, index)
        self._layers.append(layer)

    def fit(self, training_data, training_labels, maximal_batch_size, schedule):
        # (converted only when needed: the backend object copies the arrays to the device anyway)
        training_data = np.ascontiguousarray(training_data, dtype=self.dtype)
        training_labels = np.ascontiguousarray(training_labels, dtype=self.dtype)
        self.net.initiate_training(training_data, training_labels)
        n_samples = training_data.shape[0]
        for layer, epochs in schedule:
            for epoch in range(epochs):
                print('Layer - %d/%d' % (layer + 1, len(self._layers)), flush=True)
                # the two draws of an epoch, in the reference's order (permutation(n) draws and returns what
                # the reference's permutation(range(n)) does, without building the range element by element)
                idx = np.random.permutation(n_samples).astype(np.int64)
                hypercolumns_shuffled = np.random.permutation(self._layers[layer].hypercolumns).astype(np.int64)
                if _tqdm is None:
                    self.net.train_epoch(layer, maximal_batch_size, idx, hypercolumns_shuffled, epoch)
                    continue
                # the reference's per-batch progress bar (_cpu_base_backend.py:270-277, 311-312): the epoch is
                # enqueued in ranges of batches and the bar advances when the device has finished a range
                number_of_batches = (n_samples + maximal_batch_size - 1) // maximal_batch_size
                per_range = max(1, number_of_batches // _PROGRESS_RANGES)
                with _tqdm(total=number_of_batches) as pbar:
                    pbar.set_description('Epoch %d/%d' % (epoch + 1, epochs))
                    for first in range(0, number_of_batches, per_range):
                        count = min(per_range, number_of_batches - first)
                        self.net.train_batches(layer, maximal_batch_size, idx, hypercolumns_shuffled, epoch,
                                               first, count, first + count == number_of_batches)
                        self.net.synchronize()
                        pbar.update(count)
        self.net.synchronize()
        self.net.training_done()

    def evaluate(self, images, labels, maximal_batch_size):
        images = np.ascontiguousarray(images, dtype=self.dtype)
        labels = np.ascontiguousarray(labels, dtype=self.dtype)
        correct, total = self.net.evaluate_counts(images, labels, maximal_batch_size)
        return np.array([correct]), np.array([total])

    def predict(self, images, maximal_batch_size):
        images = np.ascontiguousarray(images, dtype=self.dtype)
        return self.net.predict(images, maximal_batch_size)

    def forward(self, images, maximal_batch_size=None, last_layer=None):
        images = np.ascontiguousarray(images, dtype=self.dtype)
        if last_layer is None:
            last_layer = len(self._layers) - 1
        return self.net.forward(images, last_layer, maximal_batch_size or max(1, images.shape[0]))
