// rstorch.hpp - C++ host-side mirror of the reference's public API over the HIP backend.
//
// Same names, argument meaning and failure behaviour as the reference crate
// (src/lib.rs:10-14, 53-69): Module / Loss / Optimizer / InitParameters, Identity, Linear, ReLU,
// Sequential, CrossEntropyLoss, SGD, utils::accuracy, and sequential(...) for the macro.
// Where the reference panics (unwrap on a consumed cache, shape mismatch, NaN in softmax) this
// header throws rstorch::Panic.  Array2 is a dense row-major f64 matrix whose storage lives in
// HBM; moving it between layers moves a handle, not data.  Header only; link librstorch_hip.so.
//
// A Sequential made only of Identity / Linear / ReLU layers is compiled on its first forward: a
// device model (rst_model) is built over the layer list, the layers' parameters move into its arena
// (the layers keep views), forward becomes one call, and backward launches nothing until
// its results are needed: SGD::step(model) runs it with the update inside the weight-gradient
// launches (the README loop then issues the launches of rst_model_train_step), reading a gradient
// through parameters() or keeping the returned input gradient runs it on its own first.  Everything a
// caller can observe is what the layer-by-layer path computes.  push / insert / remove drop the
// compiled form.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <functional>
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
 public:
  // The device memory behind one or more Array2 handles.  Two kinds fill `ptr` in late: gradient
  // views of a compiled Sequential (before_access first runs the backward pass that is still owed)
  // and the input gradient that Sequential::backward returns (resolver computes it when somebody
  // looks).  Every access goes through Array2::data().
  struct Storage {
    std::shared_ptr<Engine> engine;
    double* ptr = nullptr;
    bool owns = true;                        // false: a view into memory that `keepalive` owns
    // true for the arrays the library rewrites in place (a layer's parameters, which SGD::step
    // updates, and its gradients, which every backward overwrites).  Everything else is written once,
    // by the call that produced it, and never again: such an array is a value, and clone() may hand
    // out a second handle to the same memory instead of copying it.
    bool rewritten_in_place = false;
    std::shared_ptr<void> keepalive;
    std::function<void()> before_access;
    std::function<void(Storage&)> resolver;  // runs once
    // set on the logits a compiled Sequential returns: CrossEntropyLoss::forward hands its work to the
    // compiled form, which knows what follows a loss in a training loop (true: loss and accuracy are
    // there and `grad` is filled)
    std::function<bool(const Array2& pred, const Array2& truth, Array2& grad, double* loss, double* accuracy)> loss_through;
    double* get() {
      if (resolver) {
        auto r = std::move(resolver);
        resolver = nullptr;
        r(*this);
      }
      if (before_access) before_access();
      return ptr;
    }
    void materialise(size_t count) {
      if (rst_malloc(engine->handle(), count, &ptr) != RST_OK) throw Panic(RST_ERR_OUT_OF_MEMORY, rst_last_error());
      owns = true;
    }
    ~Storage() {
      if (ptr && owns) rst_free(engine->handle(), ptr);
    }
  };

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

  // a view of `rows x cols` doubles at `ptr`, owned by whatever `keepalive` keeps alive
  static Array2 view(std::shared_ptr<Engine> e, double* ptr, size_t rows, size_t cols, std::shared_ptr<void> keepalive,
                     std::function<void()> before_access = nullptr) {
    Array2 a;
    a.rows_ = rows; a.cols_ = cols;
    a.s_ = std::make_shared<Storage>();
    a.s_->engine = std::move(e);
    a.s_->ptr = ptr;
    a.s_->owns = false;
    a.s_->keepalive = std::move(keepalive);
    a.s_->before_access = std::move(before_access);
    a.s_->rewritten_in_place = true;  // views are how parameters and gradients of an arena are handed out
    return a;
  }
  // an array whose contents `resolver` produces the first time somebody asks for them
  static Array2 deferred(std::shared_ptr<Engine> e, size_t rows, size_t cols, std::function<void(Storage&)> resolver) {
    Array2 a;
    a.rows_ = rows; a.cols_ = cols;
    a.s_ = std::make_shared<Storage>();
    a.s_->engine = std::move(e);
    a.s_->owns = false;
    a.s_->resolver = std::move(resolver);
    return a;
  }

  size_t nrows() const { return rows_; }
  size_t ncols() const { return cols_; }
  size_t size() const { return rows_ * cols_; }
  bool empty_handle() const { return !s_; }
  double* data() const { return s_ ? s_->get() : nullptr; }
  rst_engine* engine() const { return s_->engine->handle(); }
  const std::shared_ptr<Engine>& engine_ref() const { return s_->engine; }
  const std::shared_ptr<Storage>& storage() const { return s_; }
  bool same_shape(const Array2& o) const { return rows_ == o.rows_ && cols_ == o.cols_; }

  // The reference clones arrays wherever a callee consumes its argument (README.md:66:
  // loss.forward(pred.clone(), y.clone())).  An array that nothing rewrites is a value: its clone is
  // a second handle to the same memory (no copy is launched, and the two stay equal because
  // neither can change).  Parameters and gradients are copied.
  Array2 clone() const {
    if (!s_->rewritten_in_place) {
      (void)data();  // a deferred array is computed before it is shared
      return *this;
    }
    return deep_clone();
  }
  Array2 deep_clone() const {
    Array2 out(rows_, cols_, s_->engine);
    check(rst_copy(engine(), out.data(), data(), size()));
    return out;
  }
  Array2& mark_rewritten_in_place() {
    s_->rewritten_in_place = true;
    return *this;
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
    // the optimiser updates them in place: they must not share memory with what the initialiser
    // returned (which may hand out the same array twice)
    weight_ = weight_.deep_clone().mark_rewritten_in_place();
    bias_ = bias_.deep_clone().mark_rewritten_in_place();
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
      grad_weight_ = Array2(out_, in_).mark_rewritten_in_place();
      grad_bias_ = Array2(1, out_).mark_rewritten_in_place();
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
  size_t input_size() const { return in_; }
  size_t output_size() const { return out_; }

  // A compiled Sequential moves the parameters into its arena: the layer keeps views, `home` names
  // the compiled form (an opaque token that also keeps the arena alive).
  const std::shared_ptr<void>& home() const { return home_; }
  bool has_gradient() const { return has_grad_; }
  void rehome(std::shared_ptr<void> home, Array2 w, Array2 b, Array2 gw, Array2 gb) {
    weight_ = std::move(w); bias_ = std::move(b);
    grad_weight_ = std::move(gw); grad_bias_ = std::move(gb);
    home_ = std::move(home);
  }
  void mark_gradient() { has_grad_ = true; }

 private:
  size_t in_, out_;
  Array2 weight_, bias_, prev_input_, grad_weight_, grad_bias_;
  bool has_input_ = false, has_grad_ = false;
  std::shared_ptr<void> home_;
};

// ---- the compiled form of a Sequential of Identity / Linear / ReLU ------------------------------
namespace detail {

class Plan : public std::enable_shared_from_this<Plan> {
 public:
  // which object `home` tokens of this plan point at
  static std::shared_ptr<Plan> create(const std::vector<std::unique_ptr<Module>>& layers) {
    std::shared_ptr<Plan> p(new Plan());
    p->build(layers);
    return p;
  }
  ~Plan() {
    if (model_) rst_model_destroy(model_);
  }
  bool valid_for(const std::vector<std::unique_ptr<Module>>& layers) const {
    if (layers.size() != key_.size()) return false;
    for (size_t i = 0; i < layers.size(); ++i)
      if (layers[i].get() != key_[i]) return false;
    for (Linear* l : linears_)
      if (l->home().get() != this) return false;
    return true;
  }

  Array2 forward(Array2 input) {
    flush();  // a backward pass nobody looked at would otherwise read the new activations
    if (input.ncols() != in_width_) throw Panic(RST_ERR_SHAPE, "Linear: input width");
    Array2 out(input.nrows(), out_width_, engine_);
    check(rst_model_forward_to(model_, input.data(), input.nrows(), out.data()));
    x_ = std::move(input);
    out_ = out;
    live_ = true;
    // a loss on these logits that the previous step followed up with a backward pass: a training loop
    training_ = loss_seen_ && backward_followed_;
    loss_seen_ = backward_followed_ = false;
    inputs_from_.reset();
    std::weak_ptr<Plan> self = shared_from_this();
    out.storage()->loss_through = [self](const Array2& pred, const Array2& truth, Array2& grad, double* loss, double* acc) {
      auto p = self.lock();
      return p && p->loss_through(pred, truth, grad, loss, acc);
    };
    return out;
  }

  // CrossEntropyLoss::forward on the logits of the latest forward pass.  In a training loop the
  // input gradients of the layers above the first are launched behind the loss, before the host
  // waits for it (rst_model_loss_accuracy_to): the GPU works while the host wakes up, calls
  // model.backward(loss.backward()) and optim.step(model), and that pass then skips them.  They are
  // only kept if the gradient array reaches backward() without anybody having looked at it.
  bool loss_through(const Array2& pred, const Array2& truth, Array2& grad, double* loss, double* acc) {
    if (!live_ || pending_ || pred.storage() != out_.storage() || !pred.same_shape(truth)) return false;
    check(rst_model_loss_accuracy_to(model_, pred.data(), truth.data(), grad.data(), training_ ? 1 : 0, loss, acc));
    loss_seen_ = true;
    if (training_) {
      inputs_from_ = grad.storage();
      std::weak_ptr<Plan> self = shared_from_this();
      grad.storage()->before_access = [self] {
        if (auto p = self.lock()) p->inputs_touched();
      };
    }
    return true;
  }

  Array2 backward(Array2 gradient) {
    if (!live_ || pending_) throw Panic(RST_ERR_STATE, "Sequential::backward without a forward");
    if (gradient.nrows() != x_.nrows() || gradient.ncols() != out_width_) throw Panic(RST_ERR_SHAPE, "Linear: gradient shape");
    std::weak_ptr<Plan> self = shared_from_this();
    Array2 gin = Array2::deferred(engine_, x_.nrows(), in_width_, [self](Array2::Storage& s) {
      if (auto p = self.lock()) p->resolve_input_gradient(s);
      if (!s.ptr) throw Panic(RST_ERR_STATE, "this input gradient was never computed");
    });
    grad_ = std::move(gradient);
    gin_ = gin.storage();
    pending_ = true;
    backward_followed_ = true;
    for (Linear* l : linears_) l->mark_gradient();
    return gin;
  }

  // runs the backward pass that is still owed, without an optimiser step
  void flush() {
    if (pending_) run(false, 0.0);
  }
  // backward + SGD::step in one pass, if a backward is still owed
  bool step_sgd(double lr) {
    if (!pending_) return false;
    run(true, lr);
    return true;
  }

 private:
  Plan() = default;

  void build(const std::vector<std::unique_ptr<Module>>& layers) {
    std::vector<int> kinds;
    std::vector<size_t> in, out;
    for (auto& l : layers) {
      key_.push_back(l.get());
      kinds.push_back(l->layer_kind());
      Linear* lin = l->layer_kind() == RST_LAYER_LINEAR ? static_cast<Linear*>(l.get()) : nullptr;
      in.push_back(lin ? lin->input_size() : 0);
      out.push_back(lin ? lin->output_size() : 0);
      if (lin) linears_.push_back(lin);
    }
    engine_ = linears_[0]->weight().engine_ref();
    in_width_ = linears_.front()->input_size();
    out_width_ = linears_.back()->output_size();
    check(rst_model_create(engine_->handle(), kinds.data(), in.data(), out.data(), kinds.size(), &model_));
    std::shared_ptr<Plan> self = shared_from_this();
    std::weak_ptr<Plan> weak = self;
    auto owed = [weak] { if (auto p = weak.lock()) p->flush(); };
    // a look at (or a write into) a parameter between the loss and the backward pass: input gradients
    // launched ahead were computed with the weights of before
    auto touched = [weak] { if (auto p = weak.lock()) p->parameters_touched(); };
    for (size_t i = 0; i < linears_.size(); ++i) {
      Linear* l = linears_[i];
      double *w, *gw, *b, *gb;
      size_t r, c;
      check(rst_model_parameter(model_, 2 * i, &w, &gw, &r, &c));
      check(rst_model_parameter(model_, 2 * i + 1, &b, &gb, &r, &c));
      const size_t nw = l->input_size() * l->output_size(), nb = l->output_size();
      // (reading the old arrays first runs whatever another compiled Sequential still owes them)
      check(rst_copy(engine_->handle(), w, l->weight().data(), nw));
      check(rst_copy(engine_->handle(), b, l->bias().data(), nb));
      if (l->has_gradient()) {  // gradients computed before the move stay readable
        check(rst_copy(engine_->handle(), gw, l->grad_weight().data(), nw));
        check(rst_copy(engine_->handle(), gb, l->grad_bias().data(), nb));
      }
      l->rehome(self, Array2::view(engine_, w, l->output_size(), l->input_size(), self, touched),
                Array2::view(engine_, b, 1, l->output_size(), self, touched),
                Array2::view(engine_, gw, l->output_size(), l->input_size(), self, owed),
                Array2::view(engine_, gb, 1, l->output_size(), self, owed));
    }
  }

  // somebody looked at (and may have rewritten) the gradient the input gradients were launched from
  void inputs_touched() {
    rst_model_discard_inputs(model_);
    inputs_from_.reset();
  }

  void parameters_touched() {
    if (!inputs_from_.expired()) inputs_touched();
  }

  void resolve_input_gradient(Array2::Storage& s) {
    if (pending_ && gin_.lock().get() == &s) run(false, 0.0);
  }

  void run(bool apply_sgd, double lr) {
    pending_ = false;
    std::shared_ptr<Array2::Storage> gin = gin_.lock();  // still wanted by somebody?
    gin_.reset();
    if (gin) {
      gin->resolver = nullptr;
      gin->materialise(x_.nrows() * in_width_);
    }
    Array2 g = std::move(grad_);
    if (auto from = inputs_from_.lock()) {
      // the gradient the input gradients were launched from, untouched since: our own access keeps them
      if (from == g.storage()) from->before_access = nullptr;
      else inputs_touched();
    }
    inputs_from_.reset();
    check(rst_model_backward_to(model_, g.data(), gin ? gin->ptr : nullptr, apply_sgd ? 1 : 0, lr));
    x_ = Array2();
    out_ = Array2();  // the caches are consumed
    live_ = false;
  }

  rst_model* model_ = nullptr;
  std::shared_ptr<Engine> engine_;
  std::vector<const Module*> key_;
  std::vector<Linear*> linears_;
  size_t in_width_ = 0, out_width_ = 0;
  Array2 x_, out_, grad_;  // the forward pass whose caches are live; the gradient of the owed backward
  std::weak_ptr<Array2::Storage> gin_;  // the input gradient that backward returned, if still held
  std::weak_ptr<Array2::Storage> inputs_from_;  // the loss gradient that input gradients were launched from
  bool live_ = false, pending_ = false;
  bool training_ = false, loss_seen_ = false, backward_followed_ = false;
};

}  // namespace detail

// ---- Sequential: src/module/sequential.rs -------------------------------------------------------
class Sequential : public Module {
 public:
  Sequential() = default;
  explicit Sequential(std::vector<std::unique_ptr<Module>> layers) : layers_(std::move(layers)) {}
  template <class M> void push(M layer) { push_box(std::make_unique<M>(std::move(layer))); }
  template <class M> void insert(size_t index, M layer) { insert_box(index, std::make_unique<M>(std::move(layer))); }
  void push_box(std::unique_ptr<Module> l) {
    drop_plan();
    layers_.push_back(std::move(l));
  }
  void insert_box(size_t index, std::unique_ptr<Module> l) {
    drop_plan();
    layers_.insert(layers_.begin() + index, std::move(l));
  }
  size_t len() const { return layers_.size(); }
  bool is_empty() const { return layers_.empty(); }
  std::unique_ptr<Module> remove(size_t index) {
    if (index >= layers_.size()) return nullptr;
    drop_plan();
    auto l = std::move(layers_[index]);
    layers_.erase(layers_.begin() + index);
    return l;
  }
  // false: always run layer by layer, one call per layer
  void set_compile(bool enabled) {
    if (!enabled) drop_plan();
    compile_ = enabled;
  }
  // backward + SGD::step in one pass if this Sequential is compiled and still owes a backward pass
  bool step_sgd(double lr) { return plan_ && plan_->valid_for(layers_) && plan_->step_sgd(lr); }

  Array2 forward(Array2 input) override {
    if (detail::Plan* plan = compiled()) return plan->forward(std::move(input));
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
    if (plan_ && plan_->valid_for(layers_)) return plan_->backward(std::move(gradient));
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
  // the compiled form, built on demand; null when the layer list has a layer it cannot hold
  detail::Plan* compiled() {
    if (!compile_) return nullptr;
    if (plan_ && plan_->valid_for(layers_)) return plan_.get();
    drop_plan();
    size_t width = 0;
    bool any = false;
    for (auto& l : layers_) {
      const int kind = l->layer_kind();
      if (kind != RST_LAYER_IDENTITY && kind != RST_LAYER_RELU && kind != RST_LAYER_LINEAR) return nullptr;
      if (kind == RST_LAYER_LINEAR) {
        auto* lin = static_cast<Linear*>(l.get());
        // (a width mismatch is left to the layer-by-layer pass, which panics where the reference does)
        if (any && lin->input_size() != width) return nullptr;
        width = lin->output_size();
        any = true;
      }
    }
    if (!any) return nullptr;
    plan_ = detail::Plan::create(layers_);
    return plan_.get();
  }
  void drop_plan() {
    if (plan_) plan_->flush();
    plan_.reset();
  }
  std::shared_ptr<detail::Plan> plan_;
  bool compile_ = true;

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

namespace detail {
// The README loop asks for accuracy(pred, y) right after loss.forward(pred.clone(), y.clone()).  The
// loss computes the arg-max agreement of its two arrays along the way (one launch and one wait for
// both numbers) and leaves it here; accuracy() takes it when it is called on the same memory.  Sound
// because such arrays are values: a clone of an array that nothing rewrites is a second handle to the
// same memory, and neither handle can change it.
struct AccuracyMemo {
  std::weak_ptr<Array2::Storage> pred, truth;
  double value = 0.0;
};
inline AccuracyMemo& accuracy_memo() {
  static thread_local AccuracyMemo memo;
  return memo;
}
}  // namespace detail

class CrossEntropyLoss : public Loss {
 public:
  double forward(Array2 pred, Array2 truth) override {
    if (!pred.same_shape(truth)) throw Panic(RST_ERR_SHAPE, "CrossEntropyLoss: pred/truth shapes");
    Array2 g(pred.nrows(), pred.ncols());
    double loss = 0.0, acc = 0.0;
    const auto& through = pred.storage()->loss_through;  // logits of a compiled Sequential
    if (!(through && through(pred, truth, g, &loss, &acc)))
      check(rst_cross_entropy_accuracy(pred.engine(), pred.data(), truth.data(), g.data(), pred.nrows(),
                                       pred.ncols(), &loss, &acc));
    detail::AccuracyMemo& memo = detail::accuracy_memo();
    memo.pred.reset();
    if (!pred.storage()->rewritten_in_place && !truth.storage()->rewritten_in_place) {
      memo.pred = pred.storage();
      memo.truth = truth.storage();
      memo.value = acc;
    }
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
    // a compiled Sequential that still owes its backward pass runs it with this update inside the
    // weight-gradient launches; the bits are those of the two passes apart
    if (auto* seq = dynamic_cast<Sequential*>(&module))
      if (seq->step_sgd(lr_)) return;
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
  const detail::AccuracyMemo& memo = detail::accuracy_memo();
  if (pred.storage() && memo.pred.lock() == pred.storage() && memo.truth.lock() == truth.storage())
    return memo.value;  // the loss has already counted these two arrays
  double acc = 0.0;
  check(rst_accuracy(pred.engine(), pred.data(), truth.data(), pred.nrows(), pred.ncols(), &acc));
  return acc;
}
}  // namespace utils

}  // namespace rstorch
