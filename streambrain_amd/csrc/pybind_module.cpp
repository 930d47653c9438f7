// pybind11 module `_bcpnn_backend_hip_internals`: the C++ backend object the Python DSL drives.
//
// It has the interface of the reference's GPU backend module
// (BCPNN/backend/full_cuda_backend/backend_full_cuda_internals.cu:648-781: initialize(),
// PyNetwork_float32 / PyNetwork_float64 with add_dense_layer, add_plastic_layer, initiate_training,
// train_layer, training_done, evaluate) and adds what that interface cannot express but the cpu
// backend's semantics need: seeded initial state (set/get_layer_state), the caller's sample and
// hypercolumn order per epoch (train_epoch), integer results (evaluate_counts, predict).
//
// Host code only: every device operation goes through the C ABI of libsbhip.so (include/sbhip.h).
// Errors become Python RuntimeError instead of the reference's exit().
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>

#include <algorithm>
#include <cstdint>
#include <numeric>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "sbhip.h"

namespace py = pybind11;

namespace {

void check(int rc) {
  if (rc < 0) throw std::runtime_error(std::string("libsbhip: ") + sb_last_error());
}

template <typename REAL>
using carray = py::array_t<REAL, py::array::c_style | py::array::forcecast>;
using iarray = py::array_t<int64_t, py::array::c_style | py::array::forcecast>;

template <typename REAL>
class PyNetwork {
 public:
  PyNetwork() : rng_(std::random_device{}()) {
    check(sb_net_create(&net_, sizeof(REAL) == 4 ? SB_F32 : SB_F64));
  }
  ~PyNetwork() {
    if (net_) sb_net_destroy(net_);
  }
  PyNetwork(const PyNetwork &) = delete;
  PyNetwork &operator=(const PyNetwork &) = delete;

  struct Shape {
    long n_inputs, hypercolumns, minicolumns;
    bool plastic;
  };

  // Like the reference's object (backend_full_cuda_internals.cu:151-155, helpers_training.cu:10-32) a layer
  // starts with random weights, bias and -- plastic layers -- a mask of density 0.1, here from this object's
  // own generator (see seed()); `randomize = false` leaves them at zero / all ones for a caller that sets
  // the state itself right away (set_layer_state).
  static constexpr double kInitialDensity = 0.1;

  int add_dense_layer(size_t n_inputs, size_t n_hypercolumns, size_t n_minicolumns, double taupdt,
                      double initial_Ci, double initial_Cj, double initial_Cij, bool randomize) {
    int idx = sb_net_add_dense_layer(net_, (long)n_inputs, (long)n_hypercolumns, (long)n_minicolumns,
                                     taupdt, initial_Ci, initial_Cj, initial_Cij);
    check(idx);
    shapes_.push_back({(long)n_inputs, (long)n_hypercolumns, (long)n_minicolumns, false});
    if (randomize) check(sb_net_randomize_layer(net_, idx, rng_(), kInitialDensity));
    return idx;
  }

  int add_plastic_layer(size_t n_inputs, size_t n_hypercolumns, size_t n_minicolumns, double taupdt,
                        double pmin, double khalf, double taubdt, double initial_Ci, double initial_Cj,
                        double initial_Cij, bool randomize) {
    int idx = sb_net_add_plastic_layer(net_, (long)n_inputs, (long)n_hypercolumns, (long)n_minicolumns,
                                       taupdt, pmin, khalf, taubdt, initial_Ci, initial_Cj, initial_Cij);
    check(idx);
    shapes_.push_back({(long)n_inputs, (long)n_hypercolumns, (long)n_minicolumns, true});
    if (randomize) check(sb_net_randomize_layer(net_, idx, rng_(), kInitialDensity));
    return idx;
  }

  const Shape &shape_of(int layer) const {
    if (layer < 0 || layer >= (int)shapes_.size()) throw std::runtime_error("layer index out of range");
    return shapes_[layer];
  }

  std::vector<py::ssize_t> state_shape(int layer, const std::string &name) const {
    const Shape &s = shape_of(layer);
    const long M = s.hypercolumns * s.minicolumns;
    if (name == "weights" || name == "Cij") return {s.n_inputs, M};
    if (name == "bias" || name == "Cj" || (name == "kbi" && s.plastic)) return {M};
    if (name == "Ci") return {s.n_inputs};
    if (name == "wmask" && s.plastic) return {s.n_inputs, s.hypercolumns};
    throw std::runtime_error("unknown state array '" + name + "'");
  }

  void set_layer_state(int layer, const std::string &name, py::array value) {
    const auto shape = state_shape(layer, name);
    size_t count = 1;
    for (auto d : shape) count *= (size_t)d;
    if ((size_t)value.size() != count) throw std::runtime_error("state '" + name + "': wrong size");
    if (name == "wmask") {
      auto a = py::array_t<uint8_t, py::array::c_style | py::array::forcecast>::ensure(value);
      if (!a) throw std::runtime_error("wmask must convert to uint8");
      check(sb_net_set_layer_state(net_, layer, name.c_str(), a.data(), count));
    } else {
      auto a = carray<REAL>::ensure(value);
      if (!a) throw std::runtime_error("state must convert to the network dtype");
      check(sb_net_set_layer_state(net_, layer, name.c_str(), a.data(), count * sizeof(REAL)));
    }
  }

  py::array get_layer_state(int layer, const std::string &name) {
    const auto shape = state_shape(layer, name);
    if (name == "wmask") {
      py::array_t<uint8_t> out(shape);
      check(sb_net_get_layer_state(net_, layer, name.c_str(), out.mutable_data(), (size_t)out.size()));
      return std::move(out);
    }
    py::array_t<REAL> out(shape);
    check(sb_net_get_layer_state(net_, layer, name.c_str(), out.mutable_data(),
                                 (size_t)out.size() * sizeof(REAL)));
    return std::move(out);
  }

  void initiate_training(carray<REAL> images, carray<REAL> labels) {
    if (images.ndim() != 2 || labels.ndim() != 2 || images.shape(0) != labels.shape(0))
      throw std::runtime_error("initiate_training: images [Ns, N] and labels [Ns, C] expected");
    check(sb_net_set_training_data(net_, images.data(), labels.data(), images.shape(0), images.shape(1),
                                   labels.shape(1)));
    n_samples_ = images.shape(0);
  }

  void train_epoch(int layer, size_t maximal_batch_size, iarray sample_perm, py::object hc_perm,
                   long epoch) {
    if (sample_perm.ndim() != 1 || sample_perm.shape(0) != n_samples_)
      throw std::runtime_error("train_epoch: sample_perm must have one entry per training sample");
    const int64_t *hc = nullptr;
    iarray hc_arr;
    if (!hc_perm.is_none()) {
      hc_arr = iarray::ensure(hc_perm);
      if (!hc_arr || hc_arr.ndim() != 1 || hc_arr.shape(0) != shape_of(layer).hypercolumns)
        throw std::runtime_error("train_epoch: hc_perm must have one entry per hypercolumn");
      hc = hc_arr.data();
    }
    check(sb_net_train_epoch(net_, layer, (long)maximal_batch_size, sample_perm.data(), hc, epoch));
  }

  // Batches [first_batch, first_batch + n_batches) of an epoch (sb_net_train_batches): what a caller
  // that reports progress between ranges uses instead of train_epoch.
  void train_batches(int layer, size_t maximal_batch_size, iarray sample_perm, py::object hc_perm, long epoch,
                     long first_batch, long n_batches, bool finalize) {
    if (sample_perm.ndim() != 1 || sample_perm.shape(0) != n_samples_)
      throw std::runtime_error("train_batches: sample_perm must have one entry per training sample");
    const int64_t *hc = nullptr;
    iarray hc_arr;
    if (!hc_perm.is_none()) {
      hc_arr = iarray::ensure(hc_perm);
      if (!hc_arr || hc_arr.ndim() != 1 || hc_arr.shape(0) != shape_of(layer).hypercolumns)
        throw std::runtime_error("train_batches: hc_perm must have one entry per hypercolumn");
      hc = hc_arr.data();
    }
    check(sb_net_train_batches(net_, layer, (long)maximal_batch_size, sample_perm.data(), hc, epoch, first_batch,
                               n_batches, finalize ? 1 : 0));
  }

  // The reference's signature: sample and hypercolumn orders come from this object's own generator
  // (time-seeded in the reference, dataloader.h:92 / helpers_random.h:12-23; see seed()).
  void train_layer(size_t maximal_batch_size, size_t layer, size_t epochs) {
    const Shape &s = shape_of((int)layer);
    std::vector<int64_t> perm(n_samples_), hc(s.hypercolumns);
    for (size_t e = 0; e < epochs; e++) {
      std::iota(perm.begin(), perm.end(), 0);
      std::shuffle(perm.begin(), perm.end(), rng_);
      std::iota(hc.begin(), hc.end(), 0);
      std::shuffle(hc.begin(), hc.end(), rng_);
      check(sb_net_train_epoch(net_, (int)layer, (long)maximal_batch_size, perm.data(), hc.data(),
                               (long)e));
    }
  }

  void seed(uint64_t value) { rng_.seed(value); }

  void set_frozen_cache_limit(size_t bytes) { check(sb_net_set_frozen_cache_limit(net_, bytes)); }

  void training_done() {
    check(sb_net_training_done(net_));
    n_samples_ = 0;
  }

  py::tuple evaluate_counts(carray<REAL> images, carray<REAL> labels, size_t batch_size) {
    if (images.ndim() != 2 || labels.ndim() != 2 || images.shape(0) != labels.shape(0))
      throw std::runtime_error("evaluate: images [Ns, N] and labels [Ns, C] expected");
    int64_t correct = 0, total = 0;
    check(sb_net_evaluate(net_, images.data(), labels.data(), images.shape(0), images.shape(1),
                          labels.shape(1), (long)batch_size, &correct, &total, nullptr));
    return py::make_tuple(correct, total);
  }

  // accuracy in [0, 1], as PyNetwork::evaluate of the reference returns it
  double evaluate(carray<REAL> images, carray<REAL> labels, size_t batch_size) {
    py::tuple r = evaluate_counts(images, labels, batch_size);
    const double total = (double)r[1].cast<int64_t>();
    return total > 0 ? (double)r[0].cast<int64_t>() / total : 0.0;
  }

  py::array_t<REAL> forward(carray<REAL> images, int last_layer, size_t batch_size) {
    if (images.ndim() != 2) throw std::runtime_error("forward: images [Ns, N] expected");
    const Shape &s = shape_of(last_layer);
    py::array_t<REAL> out({(py::ssize_t)images.shape(0), (py::ssize_t)(s.hypercolumns * s.minicolumns)});
    check(sb_net_forward(net_, images.data(), images.shape(0), images.shape(1), last_layer,
                         (long)batch_size, out.mutable_data()));
    return out;
  }

  py::array_t<int32_t> predict(carray<REAL> images, size_t batch_size) {
    if (images.ndim() != 2) throw std::runtime_error("predict: images [Ns, N] expected");
    py::array_t<int32_t> out(images.shape(0));
    check(sb_net_predict(net_, images.data(), images.shape(0), images.shape(1), (long)batch_size,
                         out.mutable_data()));
    return out;
  }

  // layer-level calls of the DSL (compute_activation, train_step, train_finalize of one layer)
  py::array_t<REAL> layer_activation(int layer, carray<REAL> inputs) {
    const Shape &s = shape_of(layer);
    if (inputs.ndim() != 2 || inputs.shape(1) != s.n_inputs)
      throw std::runtime_error("compute_activation: inputs [rows, in_features] expected");
    py::array_t<REAL> out({(py::ssize_t)inputs.shape(0), (py::ssize_t)(s.hypercolumns * s.minicolumns)});
    if (inputs.shape(0) > 0)
      check(sb_net_layer_activation(net_, layer, inputs.data(), inputs.shape(0), out.mutable_data()));
    return out;
  }

  void layer_train_step(int layer, carray<REAL> inputs, carray<REAL> outputs, long hypercolumn) {
    const Shape &s = shape_of(layer);
    if (inputs.ndim() != 2 || outputs.ndim() != 2 || inputs.shape(0) != outputs.shape(0) ||
        inputs.shape(1) != s.n_inputs || outputs.shape(1) != s.hypercolumns * s.minicolumns)
      throw std::runtime_error("train_step: inputs [rows, in_features] and outputs [rows, out_features] expected");
    check(sb_net_layer_train_step(net_, layer, inputs.data(), outputs.data(), inputs.shape(0), hypercolumn));
  }

  void layer_train_finalize(int layer) { check(sb_net_layer_train_finalize(net_, layer)); }

  void synchronize() { check(sb_sync()); }
  size_t n_layers() const { return shapes_.size(); }

 private:
  sb_net *net_ = nullptr;
  std::vector<Shape> shapes_;
  long n_samples_ = 0;
  std::mt19937_64 rng_;
};

template <typename REAL>
void bind_network(py::module_ &m, const char *name) {
  using N = PyNetwork<REAL>;
  py::class_<N>(m, name)
      .def(py::init<>())
      .def("add_dense_layer", &N::add_dense_layer, py::arg("n_inputs"), py::arg("n_hypercolumns"),
           py::arg("n_minicolumns"), py::arg("taupdt"), py::arg("initial_Ci"), py::arg("initial_Cj"),
           py::arg("initial_Cij"), py::arg("randomize") = true)
      .def("add_plastic_layer", &N::add_plastic_layer, py::arg("n_inputs"), py::arg("n_hypercolumns"),
           py::arg("n_minicolumns"), py::arg("taupdt"), py::arg("pmin"), py::arg("khalf"), py::arg("taubdt"),
           py::arg("initial_Ci"), py::arg("initial_Cj"), py::arg("initial_Cij"), py::arg("randomize") = true)
      .def("initiate_training", &N::initiate_training)
      .def("train_layer", &N::train_layer)
      .def("training_done", &N::training_done)
      .def("evaluate", &N::evaluate)
      .def("set_layer_state", &N::set_layer_state)
      .def("get_layer_state", &N::get_layer_state)
      .def("train_epoch", &N::train_epoch, py::arg("layer"), py::arg("maximal_batch_size"),
           py::arg("sample_perm"), py::arg("hc_perm"), py::arg("epoch"))
      .def("train_batches", &N::train_batches, py::arg("layer"), py::arg("maximal_batch_size"),
           py::arg("sample_perm"), py::arg("hc_perm"), py::arg("epoch"), py::arg("first_batch"),
           py::arg("n_batches"), py::arg("finalize"))
      .def("evaluate_counts", &N::evaluate_counts)
      .def("forward", &N::forward)
      .def("layer_activation", &N::layer_activation)
      .def("layer_train_step", &N::layer_train_step)
      .def("layer_train_finalize", &N::layer_train_finalize)
      .def("predict", &N::predict)
      .def("seed", &N::seed)
      .def("set_frozen_cache_limit", &N::set_frozen_cache_limit)
      .def("synchronize", &N::synchronize)
      .def("n_layers", &N::n_layers);
}

}  // namespace

PYBIND11_MODULE(_bcpnn_backend_hip_internals, m) {
  m.doc() = "MI355X (gfx950) BCPNN backend: pybind11 front of libsbhip.so";
  m.def("initialize", [](int device) { check(sb_init(device)); }, py::arg("device") = 0);
  m.def("synchronize", []() { check(sb_sync()); });
  m.def("abi_version", []() { return sb_abi_version(); });
  bind_network<float>(m, "PyNetwork_float32");
  bind_network<double>(m, "PyNetwork_float64");
}
