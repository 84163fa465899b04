// rstorch.hpp - C++ host-side mirror of the reference's public API over the HIP backend.
//
// Same names, argument meaning and failure behaviour as the reference crate
// (src/lib.rs:10-14, 53-69): Module / Loss / Optimizer / InitParameters, Identity, Linear, ReLU,
// Sequential, CrossEntropyLoss, SGD, utils::accuracy, and sequential(...) for the macro.
// Where the reference panics (unwrap on a consumed cache, shape mismatch, NaN in softmax) this
// header throws rstorch::Panic.  Array2 is a dense row-major f64 matrix whose storage lives in
// HBM; moving it between layers moves a handle, not data.  Header only; link librstorch_hip.so.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <initializer_list>
#include <memory>
#include <random>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../../include/rstorch_hip.h"

namespace rstorch {

struct Panic : std::runtime_error {
  int status;
  Panic(int s, const std::string& what) : std::runtime_error(what), status(s) {}
};

inline void check(int status) {
  if (status != RST_OK)
    throw Panic(status, std::string(rst_status_string(status)) + ": " + rst_last_error());
}

// ---- engine ---------------------------------------------------------------------------------
class Engine {
 public:
  explicit Engine(int device = 0) { check(rst_engine_create(device, &h_)); }
  ~Engine() { rst_engine_destroy(h_); }
  Engine(const Engine&) = delete;
  Engine& operator=(const Engine&) = delete;
  rst_engine* handle() const { return h_; }
  void synchronize() const { check(rst_engine_synchronize(h_)); }
  static std::shared_ptr<Engine>& global() {
    static std::shared_ptr<Engine> e = std::make_shared<Engine>(0);
    return e;
  }

 private:
  rst_engine* h_ = nullptr;
};

// ---- Array2 (ndarray::Array2<f64> of the reference, src/module/mod.rs:42-49) ----------------
class Array2 {
  struct Storage {
    std::shared_ptr<Engine> engine;
    double* ptr = nullptr;
    ~Storage() {
      if (ptr) rst_free(engine->handle(), ptr);
    }
  };

 public:
  Array2() = default;
  Array2(size_t rows, size_t cols, std::shared_ptr<Engine> e = Engine::global())
      : rows_(rows), cols_(cols), s_(std::make_shared<Storage>()) {
    s_->engine = std::move(e);
    check(rst_malloc(s_->engine->handle(), rows * cols, &s_->ptr));
  }
  static Array2 zeros(size_t rows, size_t cols) { return full(rows, cols, 0.0); }
  static Array2 ones(size_t rows, size_t cols) { return full(rows, cols, 1.0); }
  static Array2 full(size_t rows, size_t cols, double v) {
    Array2 a(rows, cols);
    check(rst_fill(a.engine(), a.data(), a.size(), v));
    return a;
  }
  static Array2 from_host(size_t rows, size_t cols, const double* host) {
    Array2 a(rows, cols);
    check(rst_upload(a.engine(), a.data(), host, a.size()));
    return a;
  }
  // array![[..],[..]] of the reference's tests
  Array2(std::initializer_list<std::initializer_list<double>> rows) {
    std::vector<double> flat;
    size_t r = 0, c = 0;
    for (auto& row : rows) {
      if (r == 0) c = row.size();
      if (row.size() != c) throw Panic(RST_ERR_SHAPE, "ragged initializer");
      flat.insert(flat.end(), row.begin(), row.end());
      ++r;
    }
    *this = from_host(r, c, flat.data());
  }
  static Array2 uniform(size_t rows, size_t cols, uint64_t seed, uint64_t stream, double lo = 0.0,
                        double hi = 1.0) {
    Array2 a(rows, cols);
    check(rst_fill_uniform(a.engine(), a.data(), a.size(), seed, stream, lo, hi));
    return a;
  }
  static Array2 normal(size_t rows, size_t cols, uint64_t seed, uint64_t stream, double mean,
                       double std) {
    Array2 a(rows, cols);
    check(rst_fill_normal(a.engine(), a.data(), a.size(), seed, stream, mean, std));
    return a;
  }
  static Array2 one_hot(size_t rows, size_t cols, uint64_t seed, uint64_t stream) {
    Array2 a(rows, cols);
    check(rst_fill_one_hot(a.engine(), a.data(), rows, cols, seed, stream));
    return a;
  }

  size_t nrows() const { return rows_; }
  size_t ncols() const { return cols_; }
  size_t size() const { return rows_ * cols_; }
  bool empty_handle() const { return !s_; }
  double* data() const { return s_ ? s_->ptr : nullptr; }
  rst_engine* engine() const { return s_->engine->handle(); }
  bool same_shape(const Array2& o) const { return rows_ == o.rows_ && cols_ == o.cols_; }

  Array2 clone() const {
    Array2 out(rows_, cols_, s_->engine);
    check(rst_copy(engine(), out.data(), data(), size()));
    return out;
  }
  std::vector<double> to_host() const {
    std::vector<double> h(size());
    check(rst_download(engine(), h.data(), data(), size()));
    return h;
  }

 private:
  size_t rows_ = 0, cols_ = 0;
  std::shared_ptr<Storage> s_;
};

// ---- Parameter(s): src/module/mod.rs:16-40 ----------------------------------------------------
struct Parameter {
  Array2* parm;
  Array2* grad;
};

class Parameters {
 public:
  Parameters& add(Array2& parm, Array2& grad) {
    parms_.push_back(Parameter{&parm, &grad});
    return *this;
  }
  std::vector<Parameter>& iter() { return parms_; }
  std::vector<Parameter>::iterator begin() { return parms_.begin(); }
  std::vector<Parameter>::iterator end() { return parms_.end(); }
  size_t size() const { return parms_.size(); }
  void append(Parameters&& other) {
    for (auto& p : other.parms_) parms_.push_back(p);
  }

 private:
  std::vector<Parameter> parms_;
};

// ---- Module: src/module/mod.rs:42-56 -----------------------------------------------------------
class Module {
 public:
  virtual ~Module() = default;
  virtual Array2 forward(Array2 input) = 0;
  virtual Array2 backward(Array2 gradient) = 0;
  virtual Parameters parameters() = 0;
  virtual void train() {}
  virtual void eval() {}
  virtual std::string debug() const = 0;  // the reference requires Debug of Sequential's layers
  // Defaulted hooks that let Sequential fuse a Linear with the ReLU next to it.
  virtual int layer_kind() const { return -1; }
};

// ---- initialisers: src/module/init/{mod,he,xavier,sigma}.rs ------------------------------------
class InitParameters {
 public:
  virtual ~InitParameters() = default;
  virtual Array2 weight(size_t input_size, size_t output_size) const = 0;
  virtual Array2 bias(size_t, size_t output_size) const { return Array2::zeros(1, output_size); }
};

inline uint64_t fresh_seed() {
  static std::random_device rd;
  return (uint64_t(rd()) << 32) ^ rd();
}

class Normal : public InitParameters {
 public:
  Normal(double mean, double std) : mean_(mean), std_(std) {
    if (!std::isfinite(std)) throw Panic(RST_ERR_INVALID_ARGUMENT, "std must be finite");
  }
  Array2 weight(size_t in, size_t out) const override {
    static uint64_t stream = 1;
    return Array2::normal(out, in, fresh_seed(), stream++, mean_, sigma(in, out));
  }

 protected:
  virtual double sigma(size_t, size_t) const { return std_; }
  double mean_, std_;
};

class KaimingNormal : public Normal {  // he.rs:12
 public:
  KaimingNormal() : Normal(0.0, 1.0) {}

 protected:
  double sigma(size_t in, size_t) const override { return 1.0 / std::sqrt(double(in)); }
};

class XavierNormal : public Normal {  // xavier.rs:12
 public:
  XavierNormal() : Normal(0.0, 1.0) {}

 protected:
  double sigma(size_t in, size_t out) const override {
    return std::sqrt(2.0 / (double(in) + double(out)));
  }
};

// ---- Identity: src/module/activation/identity.rs -----------------------------------------------
class Identity : public Module {
 public:
  Array2 forward(Array2 input) override { return input; }
  Array2 backward(Array2 gradient) override { return gradient; }
  Parameters parameters() override { return Parameters(); }
  std::string debug() const override { return "Identity"; }
  int layer_kind() const override { return RST_LAYER_IDENTITY; }
};

// ---- ReLU: src/module/activation/relu.rs --------------------------------------------------------
class ReLU : public Module {
 public:
  Array2 forward(Array2 input) override {
    Array2 out(input.nrows(), input.ncols());
    check(rst_relu_forward(input.engine(), input.data(), out.data(), input.size()));
    prev_input_ = std::move(input);
    has_ = true;
    return out;
  }
  Array2 backward(Array2 gradient) override {
    Array2 x = take();
    if (!x.same_shape(gradient)) throw Panic(RST_ERR_SHAPE, "ReLU: gradient shape");
    Array2 out(x.nrows(), x.ncols());
    check(rst_relu_backward(x.engine(), gradient.data(), x.data(), out.data(), x.size()));
    return out;
  }
  Parameters parameters() override { return Parameters(); }
  std::string debug() const override { return "ReLU"; }
  int layer_kind() const override { return RST_LAYER_RELU; }
  // Sequential's fusion: the neighbouring Linear did this layer's work.
  void absorb_forward(const Array2& activation) { prev_input_ = activation; has_ = true; }
  void absorb_backward() { (void)take(); }
  bool has_cache() const { return has_; }

 private:
  Array2 take() {
    if (!has_) throw Panic(RST_ERR_STATE, "ReLU::backward without a forward");
    has_ = false;
    return std::move(prev_input_);
  }
  Array2 prev_input_;
  bool has_ = false;
};

// ---- Softmax: src/module/activation/softmax.rs:5-78 ---------------------------------------------
class Softmax : public Module {
 public:
  Softmax() : axis_(1) {}
  static Softmax with_axis(int axis) { Softmax s; s.axis_ = axis; return s; }
  Array2 forward(Array2 input) override {
    Array2 out(input.nrows(), input.ncols());
    check(rst_softmax_forward(input.engine(), input.data(), out.data(), input.nrows(), input.ncols(), axis_));
    output_ = out;
    has_ = true;
    return out.clone();  // softmax.rs:58-59 keeps the output and returns a clone
  }
  Array2 backward(Array2 gradient) override {
    if (!has_) throw Panic(RST_ERR_STATE, "Softmax::backward without a forward");
    has_ = false;
    Array2 out = std::move(output_);
    if (!out.same_shape(gradient)) throw Panic(RST_ERR_SHAPE, "Softmax: gradient shape");
    Array2 gin(out.nrows(), out.ncols());
    check(rst_softmax_backward(out.engine(), gradient.data(), out.data(), gin.data(), out.nrows(), out.ncols()));
    return gin;
  }
  Parameters parameters() override { return Parameters(); }
  std::string debug() const override { return "Softmax { axis: " + std::to_string(axis_) + " }"; }

 private:
  int axis_;
  Array2 output_;
  bool has_ = false;
};

// ---- Linear: src/module/linear.rs ---------------------------------------------------------------
class Linear : public Module {
 public:
  Linear(size_t input_size, size_t output_size) : Linear(input_size, output_size, KaimingNormal()) {}
  Linear(size_t input_size, size_t output_size, const InitParameters& init)
      : in_(input_size), out_(output_size), weight_(init.weight(input_size, output_size)),
        bias_(init.bias(input_size, output_size)) {
    if (weight_.nrows() != out_ || weight_.ncols() != in_) throw Panic(RST_ERR_SHAPE, "init.weight shape");
    if (bias_.nrows() != 1 || bias_.ncols() != out_) throw Panic(RST_ERR_SHAPE, "init.bias shape");
  }
  static Linear new_with_kernel(size_t i, size_t o, const InitParameters& init) { return Linear(i, o, init); }

  Array2 forward(Array2 input) override { return forward_impl(std::move(input), false); }
  Array2 backward(Array2 gradient) override { return backward_impl(std::move(gradient), false); }

  Array2 forward_impl(Array2 input, bool fuse_relu) {
    if (input.ncols() != in_) throw Panic(RST_ERR_SHAPE, "Linear: input width");
    Array2 out(input.nrows(), out_);
    check(rst_linear_forward(input.engine(), input.data(), weight_.data(), bias_.data(), out.data(),
                             input.nrows(), in_, out_, fuse_relu ? 1 : 0));
    prev_input_ = std::move(input);
    has_input_ = true;
    return out;
  }
  Array2 backward_impl(Array2 gradient, bool mask_by_input) {
    if (!has_input_) throw Panic(RST_ERR_STATE, "Linear::backward without a forward");
    has_input_ = false;
    Array2 x = std::move(prev_input_);
    if (gradient.nrows() != x.nrows() || gradient.ncols() != out_) throw Panic(RST_ERR_SHAPE, "Linear: gradient shape");
    if (!has_grad_) {
      grad_weight_ = Array2(out_, in_);
      grad_bias_ = Array2(1, out_);
      has_grad_ = true;
    }
    Array2 gx(x.nrows(), in_);
    check(rst_linear_backward(x.engine(), gradient.data(), x.data(), weight_.data(), grad_weight_.data(),
                              grad_bias_.data(), gx.data(), mask_by_input ? x.data() : nullptr, x.nrows(),
                              in_, out_));
    return gx;
  }
  Parameters parameters() override {
    if (!has_grad_) throw Panic(RST_ERR_STATE, "Linear::parameters before any backward");
    Parameters p;
    p.add(weight_, grad_weight_).add(bias_, grad_bias_);
    return p;
  }
  std::string debug() const override {
    return "Linear(" + std::to_string(in_) + ", " + std::to_string(out_) + ")";
  }
  int layer_kind() const override { return RST_LAYER_LINEAR; }
  Array2& weight() { return weight_; }
  Array2& bias() { return bias_; }
  Array2& grad_weight() { return grad_weight_; }
  Array2& grad_bias() { return grad_bias_; }

 private:
  size_t in_, out_;
  Array2 weight_, bias_, prev_input_, grad_weight_, grad_bias_;
  bool has_input_ = false, has_grad_ = false;
};

// ---- Sequential: src/module/sequential.rs -------------------------------------------------------
class Sequential : public Module {
 public:
  Sequential() = default;
  explicit Sequential(std::vector<std::unique_ptr<Module>> layers) : layers_(std::move(layers)) {}
  template <class M> void push(M layer) { layers_.push_back(std::make_unique<M>(std::move(layer))); }
  template <class M> void insert(size_t index, M layer) {
    layers_.insert(layers_.begin() + index, std::make_unique<M>(std::move(layer)));
  }
  void push_box(std::unique_ptr<Module> l) { layers_.push_back(std::move(l)); }
  void insert_box(size_t index, std::unique_ptr<Module> l) { layers_.insert(layers_.begin() + index, std::move(l)); }
  size_t len() const { return layers_.size(); }
  bool is_empty() const { return layers_.empty(); }
  std::unique_ptr<Module> remove(size_t index) {
    if (index >= layers_.size()) return nullptr;
    auto l = std::move(layers_[index]);
    layers_.erase(layers_.begin() + index);
    return l;
  }

  Array2 forward(Array2 input) override {
    const int n = int(layers_.size());
    for (int i = 0; i < n; ++i) {
      Module* l = layers_[i].get();
      if (l->layer_kind() == RST_LAYER_LINEAR) {
        int j = next_real(i);
        if (j >= 0 && layers_[j]->layer_kind() == RST_LAYER_RELU) {
          input = static_cast<Linear*>(l)->forward_impl(std::move(input), true);
          static_cast<ReLU*>(layers_[j].get())->absorb_forward(input);
          // Identity layers between the two pass the handle through; the ReLU is done
          for (int k = i + 1; k < j; ++k) input = layers_[k]->forward(std::move(input));
          i = j;
          continue;
        }
      }
      input = l->forward(std::move(input));
    }
    return input;
  }

  Array2 backward(Array2 gradient) override {
    const int n = int(layers_.size());
    for (int i = n - 1; i >= 0; --i) {
      Module* l = layers_[i].get();
      if (l->layer_kind() == RST_LAYER_LINEAR) {
        int j = prev_real(i);
        if (j >= 0 && layers_[j]->layer_kind() == RST_LAYER_RELU &&
            static_cast<ReLU*>(layers_[j].get())->has_cache()) {
          gradient = static_cast<Linear*>(l)->backward_impl(std::move(gradient), true);
          static_cast<ReLU*>(layers_[j].get())->absorb_backward();
          for (int k = i - 1; k > j; --k) gradient = layers_[k]->backward(std::move(gradient));
          i = j;
          continue;
        }
      }
      gradient = l->backward(std::move(gradient));
    }
    return gradient;
  }
  void train() override { for (auto& l : layers_) l->train(); }
  void eval() override { for (auto& l : layers_) l->eval(); }
  Parameters parameters() override {
    Parameters out;
    for (auto& l : layers_) out.append(l->parameters());
    return out;
  }
  std::string debug() const override {
    std::string s = "Sequential { layers: [";
    for (size_t i = 0; i < layers_.size(); ++i) s += (i ? ", " : "") + layers_[i]->debug();
    return s + "] }";
  }

 private:
  int next_real(int i) const {
    for (int j = i + 1; j < int(layers_.size()); ++j)
      if (layers_[j]->layer_kind() != RST_LAYER_IDENTITY) return j;
    return -1;
  }
  int prev_real(int i) const {
    for (int j = i - 1; j >= 0; --j)
      if (layers_[j]->layer_kind() != RST_LAYER_IDENTITY) return j;
    return -1;
  }
  std::vector<std::unique_ptr<Module>> layers_;
};

// sequential!(...): src/module/sequential.rs:62-74
template <class... Layers>
Sequential sequential(Layers... layers) {
  Sequential s;
  (s.push(std::move(layers)), ...);
  return s;
}

// ---- Loss / CrossEntropyLoss: src/loss/{mod,cross_entropy}.rs -----------------------------------
class Loss {
 public:
  virtual ~Loss() = default;
  virtual double forward(Array2 input, Array2 truth) = 0;
  virtual Array2 backward() = 0;
};

class CrossEntropyLoss : public Loss {
 public:
  double forward(Array2 pred, Array2 truth) override {
    if (!pred.same_shape(truth)) throw Panic(RST_ERR_SHAPE, "CrossEntropyLoss: pred/truth shapes");
    Array2 g(pred.nrows(), pred.ncols());
    double loss = 0.0;
    check(rst_cross_entropy(pred.engine(), pred.data(), truth.data(), g.data(), nullptr, pred.nrows(),
                            pred.ncols(), &loss));
    grad_ = std::move(g);
    has_ = true;
    return loss;
  }
  Array2 backward() override {
    if (!has_) throw Panic(RST_ERR_STATE, "CrossEntropyLoss::backward without a forward");
    has_ = false;
    return std::move(grad_);
  }

 private:
  Array2 grad_;
  bool has_ = false;
};

// ---- Optimizer / SGD: src/optim/{mod,sgd}.rs -----------------------------------------------------
class Optimizer {
 public:
  virtual ~Optimizer() = default;
  virtual void step(Module& module) = 0;
};

class SGD : public Optimizer {
 public:
  explicit SGD(double lr) : lr_(lr) {}
  void step(Module& module) override {
    Parameters ps = module.parameters();
    if (ps.size() == 0) return;
    std::vector<double*> parm;
    std::vector<const double*> grad;
    std::vector<size_t> count;
    rst_engine* e = nullptr;
    for (auto& p : ps) {
      if (!p.parm->same_shape(*p.grad)) throw Panic(RST_ERR_SHAPE, "SGD: parameter/gradient shapes");
      parm.push_back(p.parm->data());
      grad.push_back(p.grad->data());
      count.push_back(p.parm->size());
      e = p.parm->engine();
    }
    check(rst_sgd_step(e, parm.data(), grad.data(), count.data(), parm.size(), lr_));
  }

 private:
  double lr_;
};

// ---- utils::accuracy: src/utils.rs:55-65 ----------------------------------------------------------
namespace utils {
inline double accuracy(const Array2& pred, const Array2& truth) {
  if (!pred.same_shape(truth)) throw Panic(RST_ERR_SHAPE, "accuracy: shapes");
  double acc = 0.0;
  check(rst_accuracy(pred.engine(), pred.data(), truth.data(), pred.nrows(), pred.ncols(), &acc));
  return acc;
}
}  // namespace utils

}  // namespace rstorch
