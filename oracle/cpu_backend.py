"""TEST INFRASTRUCTURE ONLY: restatement of the reference's cpu backend at the DSL level.

Follows BCPNN/backend/_cpu_base_backend.py (layer state and numpy RNG draw order :14-42,:80-124;
convert :53-59,:135-142; Network.add_layer :182-186; fit :188-203; evaluate :205-245;
_train_layer :247-314) with the cpu backend's bindings and cadence from BCPNN/backend/cpu_backend.py
(:7-18 dense layer: fused trace+weight kernel every step, bias only at finalize; :21-52 structural
plasticity layer: fused kernel, regularised bias, mask update with 16 iterations fixed, mask apply).

Every numeric kernel is the C oracle (oracle.py).  Progress bars and printing are left out; they draw
nothing from the RNG.  All random draws use numpy's legacy global stream in the reference's order.
"""
import numpy as np

from .oracle import Oracle


class _LayerBase:
    plastic = False

    def __init__(self, in_features, hypercolumns, minicolumns, taupdt, initial_counters, dtype,
                 oracle):
        self.in_features = in_features
        self.hypercolumns = hypercolumns
        self.minicolumns = minicolumns
        self.out_features = hypercolumns * minicolumns
        self.taupdt = taupdt
        self.dtype = dtype
        self.k = oracle if oracle is not None else Oracle()
        n, m = in_features, self.out_features
        # draw order: weights (randn), then bias (rand)  [_cpu_base_backend.py:31-36, 107-112]
        self.weights = (0.1 * np.random.randn(n, m)).astype(dtype)
        self.bias = (0.1 * np.random.rand(m)).astype(dtype)
        ci0, cj0, cij0 = initial_counters
        self.Ci = ci0 * np.ones([n]).astype(dtype)
        self.Cj = cj0 * np.ones([m]).astype(dtype)
        self.Cij = cij0 * np.ones([n, m]).astype(dtype)

    _state_names = ("weights", "bias", "Ci", "Cj", "Cij")

    def convert(self, dtype):
        self.dtype = dtype
        for name in self._state_names:
            setattr(self, name, np.ascontiguousarray(getattr(self, name).astype(dtype)))

    def compute_activation(self, inputs):
        act = np.zeros([inputs.shape[0], self.out_features], dtype=self.dtype)
        self.k.update_state(act, self.weights, self.bias, np.ascontiguousarray(inputs))
        self.k.softmax_minicolumns(act, self.hypercolumns, self.minicolumns)
        return act


class DenseLayer(_LayerBase):
    def __init__(self, in_features, hypercolumns, minicolumns, taupdt, initial_counters,
                 dtype=np.float64, oracle=None):
        super().__init__(in_features, hypercolumns, minicolumns, taupdt, initial_counters, dtype,
                         oracle)

    def train_step(self, inputs, outputs):  # cpu_backend.py:13-15
        self.k.update_weights(self.Ci, self.Cj, self.Cij, np.ascontiguousarray(inputs),
                              np.ascontiguousarray(outputs), self.taupdt, self.weights,
                              self.taupdt / 2)

    def train_finalize(self):  # cpu_backend.py:17-18
        self.k.update_bias(self.bias, self.Cj, self.taupdt / 2)


class StructuralPlasticityLayer(_LayerBase):
    plastic = True
    _state_names = ("weights", "bias", "Ci", "Cj", "Cij", "kbi")
    MASK_ITERATIONS = 16  # cpu_backend.py:47 ignores the constructor's mask_iterations

    def __init__(self, in_features, hypercolumns, minicolumns, taupdt, khalf, pmin, taubdt, density,
                 mask_iterations, initial_counters, dtype=np.float64, oracle=None):
        super().__init__(in_features, hypercolumns, minicolumns, taupdt, initial_counters, dtype,
                         oracle)
        self.khalf = khalf
        self.pmin = pmin
        self.taubdt = taubdt
        self.density = density
        self.mask_iterations = mask_iterations
        self.kbi = np.ones([self.out_features]).astype(dtype)
        # third draw of the layer: the receptive-field mask  [_cpu_base_backend.py:120-124]
        self.wmask = (np.random.rand(in_features, hypercolumns) < density).astype(np.uint8)

    def train_step(self, inputs, outputs, hypercolumn=None):  # cpu_backend.py:29-52
        cthr = self.taupdt / 2
        self.k.update_weights(self.Ci, self.Cj, self.Cij, np.ascontiguousarray(inputs),
                              np.ascontiguousarray(outputs), self.taupdt, self.weights, cthr)
        self.k.update_bias_regularized(self.bias, self.kbi, self.Cj, cthr, self.khalf, self.pmin,
                                       self.taubdt)
        if hypercolumn is not None:
            self.k.update_mask(self.wmask, self.weights, self.Ci, self.Cj, self.Cij, cthr,
                               self.hypercolumns, self.minicolumns, int(hypercolumn),
                               self.MASK_ITERATIONS)
        self.k.apply_mask(self.weights, self.wmask, self.hypercolumns, self.minicolumns)

    def train_finalize(self):
        pass


def rewire_schedule(epoch, step, number_of_batches, n_hypercolumns, hypercolumns_shuffled):
    """_cpu_base_backend.py:297-302.  Raises ZeroDivisionError, as the reference does, when
    number_of_batches // (n_hypercolumns + 1) == 0 and epoch > 0."""
    if epoch > 0 and step % (number_of_batches // (n_hypercolumns + 1)) == 0:
        slot = step // (number_of_batches // (n_hypercolumns + 1))
        return hypercolumns_shuffled[slot] if slot < n_hypercolumns else None
    return None


class Network:
    def __init__(self, dtype):
        self.dtype = dtype
        self._layers = []

    def add_layer(self, layer):
        if layer.dtype != self.dtype:
            layer.convert(self.dtype)
        self._layers.append(layer)

    def fit(self, training_data, training_labels, maximal_batch_size, schedule):
        data = training_data.astype(self.dtype)
        labels = training_labels.astype(self.dtype)
        for layer, epochs in schedule:
            self._train_layer(layer, maximal_batch_size, data, labels, epochs)

    def forward(self, batch):
        act = batch
        for layer in self._layers:
            act = layer.compute_activation(act)
        return act

    def predict(self, images, maximal_batch_size):
        images = images.astype(self.dtype)
        out = []
        for s in range(0, images.shape[0], maximal_batch_size):
            act = self.forward(images[s:s + maximal_batch_size])
            out.append(np.argmax(act, axis=1))
        return np.concatenate(out).astype(np.int32) if out else np.zeros([0], np.int32)

    def evaluate(self, images, labels, maximal_batch_size):
        images = images.astype(self.dtype)
        labels = labels.astype(self.dtype)
        correct = np.array([0])
        total = np.array([0])
        for s in range(0, images.shape[0], maximal_batch_size):
            act = self.forward(images[s:s + maximal_batch_size])
            lab = labels[s:s + maximal_batch_size]
            correct += (np.argmax(act, axis=1) == np.argmax(lab, axis=1)).sum()
            total += act.shape[0]
        return correct, total

    def _train_layer(self, layer, maximal_batch_size, images, labels, epochs):
        target = self._layers[layer]
        last = layer + 1 == len(self._layers)
        for epoch in range(epochs):
            # draw order per epoch: samples first, then hypercolumns  [_cpu_base_backend.py:258-264]
            idx = np.random.permutation(range(images.shape[0]))
            ep_images = images[idx, :]
            ep_labels = labels[idx, :]
            hc_order = np.random.permutation(range(target.hypercolumns))
            nb = (images.shape[0] + maximal_batch_size - 1) // maximal_batch_size
            for step in range(nb):
                lo = step * maximal_batch_size
                hi = min(lo + maximal_batch_size, images.shape[0])
                prev = None
                act = ep_images[lo:hi, :]
                for l in range(layer + 1):
                    prev = act
                    act = self._layers[l].compute_activation(prev)
                h = rewire_schedule(epoch, step, nb, target.hypercolumns, hc_order)
                if last:
                    target.train_step(prev, ep_labels[lo:hi, :])
                else:
                    target.train_step(prev, act, h)
            # the reference finalizes once per epoch  [_cpu_base_backend.py:314 sits inside the epoch loop]
            target.train_finalize()
