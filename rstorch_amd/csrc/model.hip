// Device-resident Sequential of Identity / Linear / ReLU layers with CrossEntropyLoss and SGD:
// the whole training step as an ordered list of launches on the engine's stream, weights,
// gradients and activations staying in HBM between layers.
//
// Fusion plan (decided per call, so it follows whatever layer list the model was built with):
//   forward : a Linear whose next non-Identity layer is a ReLU writes max(z, 0) directly;
//   backward: a Linear whose input came out of a ReLU multiplies its input gradient by
//             (input > 0) in the contraction epilogue, which is that ReLU's backward
//             ([relu(z) > 0] == [z > 0], NaN included, both false);
//   any ReLU not adjacent to a Linear runs the streaming kernels instead.
#include <climits>
#include <cstdlib>
#include <cstring>
#include <new>

#include "common.h"

using namespace rst;

namespace {

constexpr size_t kAlign = 32;  // doubles: every tensor starts on a 256-byte boundary

size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct Layer {
  int kind = RST_LAYER_IDENTITY;
  size_t in = 0, out = 0;  // Linear only
  size_t width_in = 0, width_out = 0;
  // Linear parameters (into the arenas)
  double *w = nullptr, *b = nullptr, *gw = nullptr, *gb = nullptr;
  // forward
  double* out_buf = nullptr;      // Linear: [batch,out]; unfused ReLU: [batch,width]
  const double* input = nullptr;  // what the layer saw in forward (Linear: x; ReLU: pre-activation)
  bool relu_fused = false;        // Linear: the following ReLU was applied in its epilogue
  bool absorbed = false;          // ReLU: forward ran inside the preceding Linear
  const double* mask_source = nullptr;  // ReLU: tensor whose sign gives the backward mask
  // backward
  double* grad_in_buf = nullptr;  // gradient w.r.t. the layer input
  bool backward_absorbed = false; // ReLU: backward ran inside the following Linear's epilogue
};

struct ProfileSlot {
  int kind, layer;
  double flops, bytes;
  hipEvent_t start, stop;
};

}  // namespace

struct rst_model {
  rst_engine* engine = nullptr;
  std::vector<Layer> layers;
  size_t in_width = 0, out_width = 0;
  bool has_linear = false;
  // arenas
  double* parm_arena = nullptr;
  double* grad_arena = nullptr;
  size_t arena_count = 0;    // doubles, padding included
  size_t element_count = 0;  // real parameters
  size_t tensor_count = 0;
  // activations
  size_t batch_capacity = 0;
  size_t batch = 0;
  double* loss_grad = nullptr;  // [batch, out_width]
  // per-row loss terms [batch]: owned by the model, because a recorded step graph keeps the address
  // (a buffer shared through the engine could be reallocated by another caller between two replays)
  double* row_loss = nullptr;
  const double* logits = nullptr;
  // state machine (mirrors the Option::take() caches of the reference)
  bool forward_valid = false;
  bool loss_grad_valid = false;
  bool grads_valid = false;
  // rst_model_loss_accuracy_to has launched the input gradients of every Linear above the first from
  // the gradient at this address; a backward pass from the same address only launches the rest
  bool inputs_done = false;
  const double* inputs_grad = nullptr;
  // the captured training step (one graph launch instead of ~10 kernel launches)
  // (a few graphs are kept: a staged input pipeline alternates between its slots' buffers)
  // 0: plain launches; 1: replay; 2: replay when the step has many launches (deep_enough)
  int graph_mode = 2;
  bool deep_enough = false;
  // what a recorded graph was recorded for: the addresses its kernels were given, the batch and
  // the learning rate
  struct StepGraph {
    hipGraphExec_t exec;
    const double* x;
    const double* truth;
    size_t batch;
    double lr;
    unsigned long long last_use;
    bool matches(const double* a, const double* b, size_t n, double l) const {
      return x == a && truth == b && batch == n && lr == l;
    }
  };
  std::vector<StepGraph> graphs;
  unsigned long long graph_clock = 0;
  // train_step applies the optimiser update inside the weight-gradient launches
  bool fuse_sgd = true;
  // backward launches a layer's weight gradient together with the next layer's input gradient when
  // both are large (C4: a pair takes 0.946 ms against 0.477 + 0.503 ms for the two launches apart)
  bool pair_gradients = true;
  // train_step runs a small classifier head (last Linear, cross entropy, that Linear's input
  // gradient) as one launch when the shape allows it
  // (0: never; 1: the head alone; 2: together with the Linear in front of it when that one is small too)
  int fuse_head = 2;
  // profiling
  bool profiling = false;
  bool slot_open = false;
  bool chain_open = false;  // the last slot's stop event is the latest thing on the stream
  std::vector<ProfileSlot> slots;
  std::vector<hipEvent_t> event_pool;
  size_t events_used = 0;
};

namespace {

// recorded graphs kept per model: a loop that walks a pool of resident batches records one forward
// and one backward graph per batch
constexpr size_t kMaxStepGraphs = 64;

// How a new model launches its step: RSTORCH_GRAPH=0 plainly, =1 as a recorded HIP graph, unset: as a
// graph when the step has many launches (kGraphFromLinears).
int default_graph_mode() {
  const char* v = std::getenv("RSTORCH_GRAPH");
  if (v && v[0] == '0') return 0;
  if (v && v[0] == '1') return 1;
  return 2;
}
// Measured on MI355X, steps per second of the single-call step on one resident batch, Linear+ReLU
// stacks of width 64 and 256 at batch 32 and 1024: with 2 and 4 hidden layers plain launches are 3-20 %
// ahead of the replayed graph (whose launch costs about as much as four plain ones, and 12 us more when
// the host reads the loss after every step), with 8 the two are level at width 64 and the graph is
// 15 % ahead at width 256, with 16 the graph is ahead or level everywhere.
constexpr int kGraphFromLinears = 8;

// What train_step hands to the fused head launch: RSTORCH_HEAD=0 nothing, =1 the head alone, unset or
// anything else also the Linear in front of it.
int default_head_mode() {
  const char* v = std::getenv("RSTORCH_HEAD");
  if (v && v[0] == '0') return 0;
  if (v && v[0] == '1') return 1;
  return 2;
}

// A graph executable is only destroyed once nothing enqueued on the stream can still be running it.
void drop_graph(rst_model* m) {
  if (m->graphs.empty()) return;
  (void)hipStreamSynchronize(m->engine->stream);
  for (auto& g : m->graphs) (void)hipGraphExecDestroy(g.exec);
  m->graphs.clear();
}

int free_activations(rst_model* m) {
  drop_graph(m);  // it holds the addresses of these buffers
  for (auto& l : m->layers) {
    if (l.out_buf) RST_HIP(hipFree(l.out_buf));
    if (l.grad_in_buf) RST_HIP(hipFree(l.grad_in_buf));
    l.out_buf = l.grad_in_buf = nullptr;
  }
  if (m->loss_grad) RST_HIP(hipFree(m->loss_grad));
  if (m->row_loss) RST_HIP(hipFree(m->row_loss));
  m->loss_grad = m->row_loss = nullptr;
  m->batch_capacity = 0;
  return RST_OK;
}

int reserve_activations(rst_model* m, size_t batch) {
  if (batch <= m->batch_capacity) return RST_OK;
  RST_HIP(hipStreamSynchronize(m->engine->stream));
  RST_TRY(free_activations(m));
  for (auto& l : m->layers) {
    if (l.kind == RST_LAYER_IDENTITY) continue;
    size_t n_out = batch * l.width_out, n_in = batch * l.width_in;
    RST_HIP(hipMalloc(&l.out_buf, (n_out ? n_out : 1) * sizeof(double)));
    RST_HIP(hipMalloc(&l.grad_in_buf, (n_in ? n_in : 1) * sizeof(double)));
  }
  size_t n = batch * m->out_width;
  RST_HIP(hipMalloc(&m->loss_grad, (n ? n : 1) * sizeof(double)));
  RST_HIP(hipMalloc(&m->row_loss, (batch ? batch : 1) * sizeof(double)));
  m->batch_capacity = batch;
  return RST_OK;
}

// ---- profiling helpers --------------------------------------------------------------------
constexpr size_t kMaxProfileSlots = 1u << 16;  // records kept between two reads

int prof_begin(rst_model* m, int kind, int layer, double flops, double bytes) {
  m->slot_open = false;
  if (!m->profiling || m->slots.size() >= kMaxProfileSlots) return RST_OK;
  while (m->event_pool.size() < m->events_used + 2) {
    hipEvent_t ev;
    RST_HIP(hipEventCreate(&ev));
    m->event_pool.push_back(ev);
  }
  ProfileSlot s;
  s.kind = kind; s.layer = layer; s.flops = flops; s.bytes = bytes;
  // launches that follow each other inside one call share an event: the stop of one is the start
  // of the next (one marker between two kernels instead of two)
  if (m->chain_open) {
    s.start = m->slots.back().stop;
  } else {
    s.start = m->event_pool[m->events_used++];
    RST_HIP(hipEventRecord(s.start, m->engine->stream));
  }
  s.stop = m->event_pool[m->events_used++];
  m->slots.push_back(s);
  m->slot_open = true;
  return RST_OK;
}

int prof_end(rst_model* m) {
  if (!m->slot_open) return RST_OK;
  m->slot_open = false;
  RST_HIP(hipEventRecord(m->slots.back().stop, m->engine->stream));
  m->chain_open = true;
  return RST_OK;
}

void prof_reset(rst_model* m) {
  m->slots.clear();
  m->events_used = 0;
  m->chain_open = false;
}

int prev_non_identity(const rst_model* m, int i) {
  for (int j = i - 1; j >= 0; --j)
    if (m->layers[j].kind != RST_LAYER_IDENTITY) return j;
  return -1;
}
int next_non_identity(const rst_model* m, int i) {
  for (int j = i + 1; j < (int)m->layers.size(); ++j)
    if (m->layers[j].kind != RST_LAYER_IDENTITY) return j;
  return -1;
}

// final_out != NULL: the last layer that computes anything writes there instead of into the model's
// own buffer (the caller's array that Sequential::forward returns by value; backward reads it again
// as the mask of a trailing ReLU, so it must stay as it is until then).
// The layers that train_step leaves to the fused head launch (do_head): the last Linear and, with
// it, the Linear in front of it.  -1: none.
struct Tail {
  int head = -1, hidden = -1;
  // every Linear but `first` (whose input gradient is the model's): launched ahead of the backward pass
  bool above_first = false;
  int first = -1;
  bool takes(int i) const { return i >= 0 && (i == head || i == hidden || (above_first && i != first)); }
};

// tail: its layers' inputs are noted, nothing is launched for them.
int do_forward(rst_model* m, const double* x, size_t batch, double* final_out = nullptr, Tail tail = Tail()) {
  rst_engine* e = m->engine;
  if (batch > (size_t)INT_MAX) return fail(RST_ERR_UNSUPPORTED, "batch too large");
  RST_TRY(reserve_activations(m, batch));
  m->batch = batch;
  const double* cur = x;
  const int n = (int)m->layers.size();
  int last = -1;  // the last layer with a launch of its own: a Linear, or a ReLU that no Linear absorbs
  for (int i = n - 1; i >= 0 && last < 0; --i) {
    if (m->layers[i].kind == RST_LAYER_LINEAR) last = i;
    if (m->layers[i].kind == RST_LAYER_RELU) {
      const int pv = prev_non_identity(m, i);
      last = (pv >= 0 && m->layers[pv].kind == RST_LAYER_LINEAR) ? pv : i;
    }
  }
  for (auto& l : m->layers) { l.absorbed = false; l.relu_fused = false; l.backward_absorbed = false; }
  for (int i = 0; i < n; ++i) {
    Layer& l = m->layers[i];
    if (l.kind == RST_LAYER_IDENTITY) continue;  // identity.rs:17-19
    double* const dest = (final_out && i == last) ? final_out : l.out_buf;
    if (l.kind == RST_LAYER_LINEAR) {
      const int nx = next_non_identity(m, i);
      const bool fuse = nx >= 0 && m->layers[nx].kind == RST_LAYER_RELU;
      l.input = cur;  // linear.rs:56 keeps the input for backward
      l.relu_fused = fuse;
      if (!tail.takes(i)) {
        GemmDesc d{};
        d.A = cur; d.B = l.w; d.C = dest;
        d.M = (int)batch; d.N = (int)l.out; d.K = (int)l.in;
        d.lda = (long)l.in; d.ldb = (long)l.in; d.ldc = (long)l.out;
        d.a_kc = true; d.b_kc = true;
        d.epilogue = fuse ? EPI_BIAS_RELU : EPI_BIAS;
        d.bias = l.b;
        const double flops = 2.0 * (double)batch * (double)l.in * (double)l.out;
        const double bytes = 8.0 * ((double)batch * l.in + (double)l.in * l.out + (double)batch * l.out);
        d.workspace = e->d_gemm_ws; d.workspace_count = e->gemm_ws_count;
        RST_TRY(prof_begin(m, RST_KERNEL_LINEAR_FORWARD, i, flops, bytes));
        RST_TRY(launch_gemm(e->stream, d));
        RST_TRY(prof_end(m));
      }
      cur = dest;
      if (fuse) {
        Layer& r = m->layers[nx];
        r.absorbed = true;
        r.input = nullptr;
        r.mask_source = dest;  // relu(z) > 0 == z > 0
      }
    } else {  // ReLU
      if (l.absorbed) continue;  // its output already is `cur`
      const size_t cnt = batch * l.width_in;
      l.input = cur;        // relu.rs:20 keeps the pre-activation
      l.mask_source = cur;
      RST_TRY(prof_begin(m, RST_KERNEL_RELU_FORWARD, i, 0.0, 16.0 * (double)cnt));
      RST_TRY(launch_relu_forward(e->stream, cur, dest, cnt));
      RST_TRY(prof_end(m));
      cur = dest;
    }
  }
  m->logits = cur;
  m->forward_valid = true;
  m->loss_grad_valid = false;
  m->inputs_done = false;
  return RST_OK;
}

int do_loss(rst_model* m, const double* truth, double* host_loss) {
  rst_engine* e = m->engine;
  if (!m->forward_valid) return fail(RST_ERR_STATE, "loss before forward");
  if (!truth) return fail(RST_ERR_INVALID_ARGUMENT, "truth is null");
  const size_t rows = m->batch, cols = m->out_width;
  RST_TRY(prof_begin(m, RST_KERNEL_CROSS_ENTROPY, -1, 0.0, 24.0 * (double)rows * (double)cols));
  RST_TRY(engine_cross_entropy(e, m->row_loss, m->logits, truth, m->loss_grad, nullptr, rows, cols, nullptr));
  RST_TRY(prof_end(m));
  m->loss_grad_valid = true;
  if (host_loss) return rst_loss_value(e, host_loss);
  return RST_OK;
}

// The layers that train_step can hand to the fused head launch: the last layer that is not an
// Identity, if it is a Linear whose shape the head kernel takes; and the Linear in front of it, if
// nothing but a ReLU stands between the two and both are small enough for the variant that holds the
// hidden weights in LDS.
Tail tail_layers(const rst_model* m) {
  Tail t;
  if (m->fuse_head == 0) return t;
  const int i = prev_non_identity(m, (int)m->layers.size());
  if (i < 0 || m->layers[i].kind != RST_LAYER_LINEAR) return t;
  if (!head_ce_supported(m->layers[i].out, m->layers[i].in)) return t;
  t.head = i;
  if (m->fuse_head < 2) return t;
  int j = prev_non_identity(m, i);
  if (j >= 0 && m->layers[j].kind == RST_LAYER_RELU) j = prev_non_identity(m, j);
  if (j >= 0 && m->layers[j].kind == RST_LAYER_LINEAR &&
      tail_ce_supported(m->layers[i].out, m->layers[i].in, m->layers[j].in, m->engine->props.sharedMemPerBlock))
    t.hidden = j;
  return t;
}

// Forward of the tail's Linear layers, the loss with its gradient and the input gradients of those
// layers (but not of the model's first Linear, which train_step does not need): one launch.
int do_head(rst_model* m, Tail tail, const double* truth) {
  rst_engine* e = m->engine;
  if (!truth) return fail(RST_ERR_INVALID_ARGUMENT, "truth is null");
  Layer& l = m->layers[tail.head];
  const size_t rows = m->batch;
  auto has_linear_before = [&](int i) {
    for (int k = 0; k < i; ++k)
      if (m->layers[k].kind == RST_LAYER_LINEAR) return true;
    return false;
  };
  auto relu_before = [&](int i) {
    const int pv = prev_non_identity(m, i);
    return pv >= 0 && m->layers[pv].kind == RST_LAYER_RELU;
  };
  const bool wanted = has_linear_before(tail.head);
  double work = (double)rows * (double)l.in * (double)l.out * (wanted ? 4.0 : 2.0);
  double bytes = 8.0 * ((double)rows * l.in * (wanted ? 2.0 : 1.0) + 3.0 * (double)rows * l.out);
  HiddenLayer hidden{};
  if (tail.hidden >= 0) {
    Layer& hl = m->layers[tail.hidden];
    const bool wanted1 = has_linear_before(tail.hidden);
    hidden.input = hl.input;
    hidden.weight = hl.w;
    hidden.bias = hl.b;
    hidden.output = hl.out_buf;
    hidden.input_grad = wanted1 ? hl.grad_in_buf : nullptr;
    hidden.in_features = hl.in;
    hidden.mask_input_grad = relu_before(tail.hidden);
    work += (double)rows * (double)hl.in * (double)hl.out * (wanted1 ? 4.0 : 2.0);
    bytes += 8.0 * ((double)rows * hl.in * (wanted1 ? 2.0 : 1.0) + (double)hl.in * hl.out);
  }
  RST_TRY(prof_begin(m, RST_KERNEL_CROSS_ENTROPY, tail.head, work, bytes));
  RST_TRY(engine_head_cross_entropy(e, m->row_loss, l.input, l.w, l.b, truth, l.out_buf, m->loss_grad,
                                    wanted ? l.grad_in_buf : nullptr, relu_before(tail.head), rows, l.out, l.in,
                                    tail.hidden >= 0 ? &hidden : nullptr));
  RST_TRY(prof_end(m));
  m->loss_grad_valid = true;
  return RST_OK;
}

// grad_input[batch, in] = grad . weight (linear.rs:68), under the mask of a preceding ReLU
GemmDesc input_gradient_desc(rst_model* m, const Layer& l, const double* grad, double* dest, bool mask) {
  GemmDesc dx{};
  dx.A = grad; dx.B = l.w; dx.C = dest;
  dx.M = (int)m->batch; dx.N = (int)l.in; dx.K = (int)l.out;
  dx.lda = (long)l.out; dx.ldb = (long)l.in; dx.ldc = (long)l.in;
  dx.a_kc = true; dx.b_kc = false;
  dx.epilogue = mask ? EPI_MASK : EPI_NONE;
  dx.mask = mask ? l.input : nullptr;  // the ReLU's output is this layer's input
  dx.ldmask = (long)l.in;
  dx.workspace = m->engine->d_gemm_ws; dx.workspace_count = m->engine->gemm_ws_count;
  return dx;
}

// fused_lr != NULL: every weight-gradient launch also applies the SGD update to its layer
// (the input gradient, which needs the old weights, is launched first).
// input_grad_dest != NULL (with need_input_grad): the gradient with respect to the model's input is
// written there (the caller's array that Sequential::backward returns by value) instead of into the
// model's own buffer.
// tail: the input gradients of its layers have been written by do_head already.
int do_backward(rst_model* m, const double* grad, int need_input_grad, const double** input_grad,
                const double* fused_lr, double* input_grad_dest = nullptr, Tail tail = Tail()) {
  rst_engine* e = m->engine;
  if (!m->forward_valid)
    return fail(RST_ERR_STATE, "backward without a forward (the reference panics on a consumed cache)");
  if (!grad) {
    if (!m->loss_grad_valid) return fail(RST_ERR_STATE, "backward from the loss before the loss was computed");
    grad = m->loss_grad;
  }
  const size_t batch = m->batch;
  const double n_rows = (double)batch;
  const double* cur = grad;
  const int n = (int)m->layers.size();
  int first_linear = -1;
  for (int i = 0; i < n; ++i)
    if (m->layers[i].kind == RST_LAYER_LINEAR) { first_linear = i; break; }
  // the layer whose launch produces the gradient with respect to the model's input: the first layer
  // that is not an Identity, or, when that is a ReLU feeding a Linear, the Linear (whose epilogue
  // applies the ReLU's mask)
  int producer = -1;
  if (need_input_grad && input_grad_dest) {
    for (int i = 0; i < n && producer < 0; ++i)
      if (m->layers[i].kind != RST_LAYER_IDENTITY) producer = i;
    if (producer >= 0 && m->layers[producer].kind == RST_LAYER_RELU) {
      const int nx = next_non_identity(m, producer);
      if (nx >= 0 && m->layers[nx].kind == RST_LAYER_LINEAR) producer = nx;
    }
  }

  // a weight gradient that has been described but not launched yet
  struct Pending {
    bool active = false;
    GemmDesc d{};
    int layer = -1;
    double flops = 0.0, bytes = 0.0;
    bool fused_bias = false;
    const double* grad = nullptr;  // gradient w.r.t. that layer's output
  };
  Pending pend;
  // Small weight gradients (a launch each would cost more than their arithmetic) wait here for one
  // shared grid at the end; their operands - the layer's cached input and the gradient buffer of
  // the layer above - stay untouched until then.  Not while profiling: every layer keeps its record.
  std::vector<Pending> held;
  const bool may_hold = !m->profiling;
  // doubles of the split-K workspace that the held ones, plus `extra` if given, take as one group
  auto group_need = [&](const Pending* extra) -> size_t {
    std::vector<GemmDesc> descs;
    for (const Pending& q : held) descs.push_back(q.d);
    if (extra) descs.push_back(extra->d);
    return gemm_group_workspace(descs.data(), (int)descs.size());
  };
  auto launch_pending = [&](const Pending& q) -> int {
    Layer& pl = m->layers[q.layer];
    RST_TRY(prof_begin(m, RST_KERNEL_GRAD_WEIGHT, q.layer, q.flops, q.bytes));
    RST_TRY(launch_gemm(e->stream, q.d));
    RST_TRY(prof_end(m));
    if (!q.fused_bias) {
      RST_TRY(prof_begin(m, RST_KERNEL_GRAD_BIAS, q.layer, 0.0, 8.0 * ((double)batch * pl.out + pl.out)));
      RST_TRY(launch_column_mean(e->stream, q.grad, pl.gb, batch, pl.out, n_rows));
      RST_TRY(prof_end(m));
      if (fused_lr) RST_TRY(launch_sgd_flat(e->stream, pl.b, pl.gb, pl.out, *fused_lr));
    }
    return RST_OK;
  };
  auto flush_held = [&]() -> int {
    if (held.size() == 1) RST_TRY(launch_pending(held[0]));
    if (held.size() > 1) {
      std::vector<GemmDesc> descs;
      for (const Pending& q : held) descs.push_back(q.d);
      RST_TRY(launch_gemm_group(e->stream, descs.data(), (int)descs.size()));
    }
    held.clear();
    return RST_OK;
  };

  auto flush_pending = [&]() -> int {
    if (!pend.active) return RST_OK;
    pend.active = false;
    if (may_hold && pend.fused_bias && can_group_gemm(pend.d)) {
      // a full grid (or a full workspace) goes out, and the next one starts
      if ((int)held.size() == max_gemm_group() || group_need(&pend) > e->gemm_ws_count) RST_TRY(flush_held());
      if (group_need(&pend) <= e->gemm_ws_count) {
        held.push_back(pend);
        return RST_OK;
      }
    }
    return launch_pending(pend);
  };
  for (int i = n - 1; i >= 0; --i) {
    Layer& l = m->layers[i];
    if (l.kind == RST_LAYER_IDENTITY) continue;  // identity.rs:22-24
    double* const gin = (i == producer) ? input_grad_dest : l.grad_in_buf;
    if (l.kind == RST_LAYER_RELU) {
      if (l.backward_absorbed) continue;
      const size_t cnt = batch * l.width_in;
      RST_TRY(prof_begin(m, RST_KERNEL_RELU_BACKWARD, i, 0.0, 24.0 * (double)cnt));
      RST_TRY(launch_relu_backward(e->stream, cur, l.mask_source, gin, cnt));
      RST_TRY(prof_end(m));
      cur = gin;
      continue;
    }
    // Linear: linear.rs:60-69.  The input gradient goes first: it reads the weights, which the
    // weight-gradient launch may update in place when the optimiser step is fused in.  The weight
    // gradient itself is held back one layer: it does not depend on anything the next layer down
    // computes, so it can share a grid with that layer's input gradient (launch_gemm_pair).
    const double mnk = (double)batch * (double)l.in * (double)l.out;
    const bool wanted = need_input_grad || i != first_linear;
    const int pv = prev_non_identity(m, i);
    const bool mask = pv >= 0 && m->layers[pv].kind == RST_LAYER_RELU;
    GemmDesc dx{};
    double dx_bytes = 0.0;
    if (wanted) {
      dx = input_gradient_desc(m, l, cur, gin, mask);
      dx_bytes = 8.0 * ((double)batch * l.out + (double)l.in * l.out +
                        (double)batch * l.in * (mask ? 2.0 : 1.0));
    }
    if (tail.takes(i)) {
      RST_TRY(flush_pending());  // (the head's weight gradient, when this is the layer in front of it)
    } else if (pend.active && wanted && m->pair_gradients && can_pair_gemm(dx, pend.d)) {
      RST_TRY(prof_begin(m, RST_KERNEL_GRAD_PAIR, i, 2.0 * mnk + pend.flops, dx_bytes + pend.bytes));
      RST_TRY(launch_gemm_pair(e->stream, dx, pend.d));
      RST_TRY(prof_end(m));
      pend.active = false;
    } else {
      RST_TRY(flush_pending());
      if (wanted) {
        RST_TRY(prof_begin(m, RST_KERNEL_GRAD_INPUT, i, 2.0 * mnk, dx_bytes));
        RST_TRY(launch_gemm(e->stream, dx));
        RST_TRY(prof_end(m));
      }
    }
    if (wanted && mask) m->layers[pv].backward_absorbed = true;
    {
      GemmDesc& d = pend.d;
      d = GemmDesc{};
      d.A = cur; d.B = l.input; d.C = l.gw;
      d.M = (int)l.out; d.N = (int)l.in; d.K = (int)batch;
      d.lda = (long)l.out; d.ldb = (long)l.in; d.ldc = (long)l.in;
      d.a_kc = false; d.b_kc = false;
      d.epilogue = EPI_DIVIDE; d.divisor = n_rows;
      // the bias gradient (linear.rs:65-67) is accumulated by the same launch
      pend.fused_bias = l.in > 0 && batch > 0;
      d.colsum = pend.fused_bias ? l.gb : nullptr;
      d.colsum_div = n_rows;
      if (fused_lr) {
        d.sgd_parm = l.w;
        d.sgd_bias = pend.fused_bias ? l.b : nullptr;
        d.sgd_lr = *fused_lr;
      }
      d.workspace = e->d_gemm_ws; d.workspace_count = e->gemm_ws_count;
      pend.bytes = 8.0 * ((double)batch * l.out + (double)batch * l.in + (double)l.in * l.out);
      if (fused_lr) pend.bytes += 16.0 * ((double)l.in * l.out + l.out);  // read and write the parameters
      pend.flops = 2.0 * mnk;
      pend.layer = i;
      pend.grad = cur;
      pend.active = true;
    }
    if (!wanted) { cur = nullptr; break; }
    cur = gin;
  }
  RST_TRY(flush_pending());
  RST_TRY(flush_held());
  if (input_grad) *input_grad = cur;
  // the caches are consumed (Option::take in linear.rs:61, relu.rs:26, cross_entropy.rs:46)
  m->forward_valid = false;
  m->loss_grad_valid = false;
  m->grads_valid = true;
  m->inputs_done = false;
  return RST_OK;
}

// The part of a backward pass that changes nothing a caller can see: the input gradients of every
// Linear above the first, from `grad`, into the model's own buffers.  For small models only - every
// weight gradient waits for the shared grid at the end of backward anyway, so launching these first
// leaves the order of the launches as it is - whose ReLU layers all sit right below a Linear.
bool inputs_ahead_possible(rst_model* m) {
  if (!m->forward_valid || m->profiling || m->batch == 0) return false;
  const int n = (int)m->layers.size();
  int linears = 0;
  for (int i = 0; i < n; ++i) {
    const Layer& l = m->layers[i];
    if (l.kind == RST_LAYER_RELU) {
      const int nx = next_non_identity(m, i);
      if (nx < 0 || m->layers[nx].kind != RST_LAYER_LINEAR) return false;  // (a launch of its own in backward)
    }
    if (l.kind != RST_LAYER_LINEAR) continue;
    ++linears;
    GemmDesc d{};
    d.A = m->loss_grad; d.B = l.input; d.C = l.gw;
    d.M = (int)l.out; d.N = (int)l.in; d.K = (int)m->batch;
    d.lda = (long)l.out; d.ldb = (long)l.in; d.ldc = (long)l.in;
    d.a_kc = false; d.b_kc = false;
    d.epilogue = EPI_DIVIDE; d.divisor = (double)m->batch;
    d.workspace = m->engine->d_gemm_ws; d.workspace_count = m->engine->gemm_ws_count;
    if (l.in == 0 || !can_group_gemm(d)) return false;
  }
  return linears >= 2;
}

int do_backward_inputs(rst_model* m, const double* grad) {
  rst_engine* e = m->engine;
  const int n = (int)m->layers.size();
  int first_linear = -1;
  for (int i = 0; i < n; ++i)
    if (m->layers[i].kind == RST_LAYER_LINEAR) { first_linear = i; break; }
  const double* cur = grad;
  for (int i = n - 1; i > first_linear; --i) {
    Layer& l = m->layers[i];
    if (l.kind != RST_LAYER_LINEAR) continue;  // (every ReLU is taken by the Linear above it)
    const int pv = prev_non_identity(m, i);
    const bool mask = pv >= 0 && m->layers[pv].kind == RST_LAYER_RELU;
    RST_TRY(launch_gemm(e->stream, input_gradient_desc(m, l, cur, l.grad_in_buf, mask)));
    if (mask) m->layers[pv].backward_absorbed = true;
    cur = l.grad_in_buf;
  }
  m->inputs_done = true;
  m->inputs_grad = grad;
  return RST_OK;
}

int do_sgd(rst_model* m, double lr) {
  if (!m->has_linear) return RST_OK;
  if (!m->grads_valid)
    return fail(RST_ERR_STATE, "optimizer step before any backward (the reference panics unwrapping the gradient)");
  RST_TRY(prof_begin(m, RST_KERNEL_SGD, -1, 0.0, 24.0 * (double)m->element_count));
  RST_TRY(launch_sgd_flat(m->engine->stream, m->parm_arena, m->grad_arena, m->arena_count, lr));
  RST_TRY(prof_end(m));
  return RST_OK;
}

}  // namespace

extern "C" {

int rst_model_create(rst_engine* e, const int* kinds, const size_t* in_features,
                     const size_t* out_features, size_t layer_count, rst_model** out) {
  RST_TRY(engine_activate(e));
  if (!out) return fail(RST_ERR_INVALID_ARGUMENT, "out is null");
  *out = nullptr;
  if (layer_count && !kinds) return fail(RST_ERR_INVALID_ARGUMENT, "kinds is null");
  rst_model* m = new (std::nothrow) rst_model();
  if (!m) return fail(RST_ERR_OUT_OF_MEMORY, "host allocation failed");
  m->engine = e;
  m->graph_mode = default_graph_mode();
  m->fuse_head = default_head_mode();
  m->layers.resize(layer_count);
  size_t offset = 0;
  size_t width = 0;
  bool width_known = false;
  for (size_t i = 0; i < layer_count; ++i) {
    Layer& l = m->layers[i];
    l.kind = kinds[i];
    if (l.kind == RST_LAYER_LINEAR) {
      if (!in_features || !out_features) { delete m; return fail(RST_ERR_INVALID_ARGUMENT, "feature arrays are null"); }
      l.in = in_features[i];
      l.out = out_features[i];
      if (l.in > (size_t)INT_MAX || l.out > (size_t)INT_MAX) { delete m; return fail(RST_ERR_UNSUPPORTED, "layer too wide"); }
      if (width_known && width != l.in) {
        int status = fail(RST_ERR_SHAPE, "layer %zu expects %zu inputs but receives %zu", i, l.in, width);
        delete m;
        return status;
      }
      if (!m->has_linear) m->in_width = l.in;
      m->has_linear = true;
      width = l.out;
      width_known = true;
      offset = round_up(offset, kAlign) + l.in * l.out;
      offset = round_up(offset, kAlign) + l.out;
      m->element_count += l.in * l.out + l.out;
      m->tensor_count += 2;
    } else if (l.kind != RST_LAYER_IDENTITY && l.kind != RST_LAYER_RELU) {
      int status = fail(RST_ERR_INVALID_ARGUMENT, "layer %zu has unknown kind %d", i, l.kind);
      delete m;
      return status;
    }
  }
  if (!m->has_linear) {
    delete m;
    return fail(RST_ERR_UNSUPPORTED, "a device model needs at least one Linear layer to fix its width");
  }
  m->out_width = width;
  m->deep_enough = m->tensor_count / 2 >= (size_t)kGraphFromLinears;
  // widths flowing through every layer
  width = m->in_width;
  for (auto& l : m->layers) {
    l.width_in = width;
    if (l.kind == RST_LAYER_LINEAR) width = l.out;
    l.width_out = width;
  }
  m->arena_count = round_up(offset, kAlign);
  hipError_t err = hipMalloc(&m->parm_arena, m->arena_count * sizeof(double));
  if (err == hipSuccess) err = hipMalloc(&m->grad_arena, m->arena_count * sizeof(double));
  if (err != hipSuccess) {
    int status = fail_hip(err, "parameter arena allocation", __FILE__, __LINE__);
    rst_model_destroy(m);
    return status;
  }
  int status = launch_fill(e->stream, m->parm_arena, m->arena_count, 0.0);
  if (status == RST_OK) status = launch_fill(e->stream, m->grad_arena, m->arena_count, 0.0);
  if (status != RST_OK) { rst_model_destroy(m); return status; }
  offset = 0;
  for (auto& l : m->layers) {
    if (l.kind != RST_LAYER_LINEAR) continue;
    offset = round_up(offset, kAlign);
    l.w = m->parm_arena + offset; l.gw = m->grad_arena + offset;
    offset += l.in * l.out;
    offset = round_up(offset, kAlign);
    l.b = m->parm_arena + offset; l.gb = m->grad_arena + offset;
    offset += l.out;
  }
  *out = m;
  return RST_OK;
}

int rst_model_destroy(rst_model* m) {
  if (!m) return RST_OK;
  (void)hipSetDevice(m->engine->device);
  (void)hipStreamSynchronize(m->engine->stream);
  (void)free_activations(m);
  drop_graph(m);
  if (m->parm_arena) (void)hipFree(m->parm_arena);
  if (m->grad_arena) (void)hipFree(m->grad_arena);
  for (hipEvent_t ev : m->event_pool) (void)hipEventDestroy(ev);
  delete m;
  return RST_OK;
}

int rst_model_parameter_count(rst_model* m, size_t* tensor_count, size_t* element_count) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  if (tensor_count) *tensor_count = m->tensor_count;
  if (element_count) *element_count = m->element_count;
  return RST_OK;
}

int rst_model_parameter(rst_model* m, size_t index, double** parm, double** grad, size_t* rows,
                        size_t* cols) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  size_t k = 0;
  for (auto& l : m->layers) {
    if (l.kind != RST_LAYER_LINEAR) continue;
    if (index == k || index == k + 1) {
      const bool is_w = index == k;
      if (parm) *parm = is_w ? l.w : l.b;
      if (grad) *grad = is_w ? l.gw : l.gb;
      if (rows) *rows = is_w ? l.out : 1;
      if (cols) *cols = is_w ? l.in : l.out;
      return RST_OK;
    }
    k += 2;
  }
  return fail(RST_ERR_INVALID_ARGUMENT, "parameter index %zu out of range (%zu tensors)", index, k);
}

static int transfer_parameters(rst_model* m, double* host_dst, const double* host_src, size_t count) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  RST_TRY(engine_activate(m->engine));
  if (count != m->element_count)
    return fail(RST_ERR_SHAPE, "the model has %zu parameters, the buffer holds %zu", m->element_count, count);
  if (!host_dst && !host_src) return fail(RST_ERR_INVALID_ARGUMENT, "host buffer is null");
  size_t off = 0;
  for (auto& l : m->layers) {
    if (l.kind != RST_LAYER_LINEAR) continue;
    double* tensors[2] = {l.w, l.b};
    size_t counts[2] = {l.in * l.out, l.out};
    for (int t = 0; t < 2; ++t) {
      if (host_dst) RST_TRY(rst_download(m->engine, host_dst + off, tensors[t], counts[t]));
      else RST_TRY(rst_upload(m->engine, tensors[t], host_src + off, counts[t]));
      off += counts[t];
    }
  }
  return RST_OK;
}

int rst_model_export_parameters(rst_model* m, double* host_dst, size_t count) {
  return transfer_parameters(m, host_dst, nullptr, count);
}

int rst_model_import_parameters(rst_model* m, const double* host_src, size_t count) {
  if (!host_src) return fail(RST_ERR_INVALID_ARGUMENT, "host buffer is null");
  return transfer_parameters(m, nullptr, host_src, count);
}

int rst_model_init_kaiming(rst_model* m, uint64_t seed, uint64_t first_stream) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  RST_TRY(engine_activate(m->engine));
  uint64_t stream = first_stream;
  for (auto& l : m->layers) {
    if (l.kind != RST_LAYER_LINEAR) continue;
    const double sigma = 1.0 / sqrt((double)l.in);  // he.rs:12
    RST_TRY(launch_fill_normal(m->engine->stream, l.w, l.in * l.out, seed, stream, 0.0, sigma));
    RST_TRY(launch_fill(m->engine->stream, l.b, l.out, 0.0));  // init/mod.rs:15-17
    stream += 2;
  }
  return RST_OK;
}

int rst_model_forward(rst_model* m, const double* x, size_t batch, const double** logits) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->chain_open = false;  // whatever ran on the stream since the last profiled launch is not ours
  RST_TRY(engine_activate(m->engine));
  if (!x && batch) return fail(RST_ERR_INVALID_ARGUMENT, "x is null");
  RST_TRY(do_forward(m, x, batch));
  if (logits) *logits = m->logits;
  return RST_OK;
}

int rst_model_loss(rst_model* m, const double* truth, double* host_loss) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->chain_open = false;  // whatever ran on the stream since the last profiled launch is not ours
  RST_TRY(engine_activate(m->engine));
  return do_loss(m, truth, host_loss);
}

int rst_model_backward(rst_model* m, const double* grad, int need_input_grad,
                       const double** input_grad) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->chain_open = false;
  RST_TRY(engine_activate(m->engine));
  return do_backward(m, grad, need_input_grad, input_grad, nullptr);
}

int rst_model_sgd_step(rst_model* m, double lr) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->chain_open = false;  // whatever ran on the stream since the last profiled launch is not ours
  RST_TRY(engine_activate(m->engine));
  return do_sgd(m, lr);
}

}  // extern "C"

namespace {

int run_step(rst_model* m, const double* x, const double* truth, size_t batch, double lr) {
  const Tail tail = tail_layers(m);
  RST_TRY(do_forward(m, x, batch, nullptr, tail));
  if (tail.head >= 0) {
    RST_TRY(do_head(m, tail, truth));
  } else {
    RST_TRY(do_loss(m, truth, nullptr));
  }
  if (m->fuse_sgd) {  // SGD::step rides in the epilogues of the weight-gradient launches
    RST_TRY(do_backward(m, nullptr, 0, nullptr, &lr, nullptr, tail));
  } else {
    RST_TRY(do_backward(m, nullptr, 0, nullptr, nullptr, nullptr, tail));
    RST_TRY(do_sgd(m, lr));
  }
  return RST_OK;
}

// Records what `run` launches into a graph.  Everything the launches allocate lazily is reserved
// first, because allocation is not allowed while the stream is capturing.  The graph holds kernel
// nodes only (no memset nodes).  `key` says what the graph was recorded for.
template <class Run>
int capture_graph(rst_model* m, rst_model::StepGraph key, Run run, hipGraphExec_t* out) {
  rst_engine* e = m->engine;
  RST_TRY(reserve_activations(m, key.batch));  // drops every graph if the buffers move
  RST_HIP(hipStreamBeginCapture(e->stream, hipStreamCaptureModeThreadLocal));
  const int status = run();
  hipGraph_t graph = nullptr;
  const hipError_t end = hipStreamEndCapture(e->stream, &graph);
  if (status != RST_OK) {
    if (graph) (void)hipGraphDestroy(graph);
    return status;
  }
  if (end != hipSuccess) return fail_hip(end, "hipStreamEndCapture", __FILE__, __LINE__);
  hipGraphExec_t exec = nullptr;
  const hipError_t inst = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (inst != hipSuccess) return fail_hip(inst, "hipGraphInstantiate", __FILE__, __LINE__);
  if (m->graphs.size() >= kMaxStepGraphs) {  // evict the least recently used
    size_t victim = 0;
    for (size_t i = 1; i < m->graphs.size(); ++i)
      if (m->graphs[i].last_use < m->graphs[victim].last_use) victim = i;
    (void)hipStreamSynchronize(e->stream);  // it may be the graph launched a moment ago
    (void)hipGraphExecDestroy(m->graphs[victim].exec);
    m->graphs.erase(m->graphs.begin() + victim);
  }
  key.exec = exec;
  key.last_use = ++m->graph_clock;
  m->graphs.push_back(key);
  *out = exec;
  return RST_OK;
}

// the recorded graph for `key`, if there is one
hipGraphExec_t find_graph(rst_model* m, const rst_model::StepGraph& key) {
  for (auto& g : m->graphs)
    if (g.matches(key.x, key.truth, key.batch, key.lr)) {
      g.last_use = ++m->graph_clock;
      return g.exec;
    }
  return nullptr;
}

bool use_graphs(const rst_model* m) {
  return !m->profiling && (m->graph_mode == 1 || (m->graph_mode == 2 && m->deep_enough));
}

}  // namespace

extern "C" {

int rst_model_train_step(rst_model* m, const double* x, const double* truth, size_t batch,
                         double lr, double* host_loss) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->chain_open = false;
  rst_engine* e = m->engine;
  RST_TRY(engine_activate(e));
  if (!x || !truth) return fail(RST_ERR_INVALID_ARGUMENT, "x or truth is null");
  if (batch == 0) return fail(RST_ERR_SHAPE, "training step on an empty batch");
  if (use_graphs(m)) {
    const rst_model::StepGraph key{nullptr, x, truth, batch, lr, 0};
    hipGraphExec_t exec = find_graph(m, key);
    if (!exec) RST_TRY(capture_graph(m, key, [&] { return run_step(m, x, truth, batch, lr); }, &exec));
    RST_HIP(hipGraphLaunch(exec, e->stream));
    // the state the eager calls leave behind
    m->batch = batch;
    m->forward_valid = false;
    m->loss_grad_valid = false;
    m->grads_valid = true;
    e->loss_valid = true;
    e->loss_ticket = 0;  // a replayed loss announces no ticket: its reader waits for the stream
  } else {
    RST_TRY(run_step(m, x, truth, batch, lr));
  }
  if (host_loss) return rst_loss_value(e, host_loss);
  return RST_OK;
}

// These two launch plainly, never from a recorded graph: their caller reads a scalar (the loss)
// between them, so what counts is how soon the first kernel starts after the call, and a graph
// launch of three or four small kernels starts later than the first of as many plain launches
// (the README loop at batch 32 through the C++ mirror: 22.1 k steps/s with plain launches, 17.7 k
// with one graph per pass; 6.4 k against 6.1 k at batch 8192).
int rst_model_forward_to(rst_model* m, const double* x, size_t batch, double* logits_out) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->chain_open = false;
  RST_TRY(engine_activate(m->engine));
  if (batch && (!x || !logits_out)) return fail(RST_ERR_INVALID_ARGUMENT, "x or logits_out is null");
  return do_forward(m, x, batch, logits_out);
}

int rst_model_backward_to(rst_model* m, const double* grad, double* input_grad_out, int apply_sgd,
                          double lr) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->chain_open = false;
  RST_TRY(engine_activate(m->engine));
  if (!grad) return fail(RST_ERR_INVALID_ARGUMENT, "grad is null");
  const int need = input_grad_out != nullptr;
  const bool fused = apply_sgd != 0 && m->fuse_sgd;
  Tail done;
  if (m->inputs_done && m->inputs_grad == grad && m->forward_valid && !m->profiling) {
    // the input gradients above the first Linear are in their buffers already
    done.above_first = true;
    for (int i = 0; i < (int)m->layers.size() && done.first < 0; ++i)
      if (m->layers[i].kind == RST_LAYER_LINEAR) done.first = i;
  }
  RST_TRY(do_backward(m, grad, need, nullptr, fused ? &lr : nullptr, input_grad_out, done));
  if (apply_sgd && !fused) RST_TRY(do_sgd(m, lr));
  return RST_OK;
}

int rst_model_loss_accuracy_to(rst_model* m, const double* pred, const double* truth, double* grad_out,
                               int inputs_ahead, double* host_loss, double* host_accuracy) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  rst_engine* e = m->engine;
  RST_TRY(engine_activate(e));
  if (!pred || !truth || !grad_out || !host_loss)
    return fail(RST_ERR_INVALID_ARGUMENT, "loss_accuracy_to: null operand");
  if (!m->forward_valid || pred != m->logits)
    return fail(RST_ERR_STATE, "pred is not what the model's latest forward pass wrote");
  const size_t rows = m->batch, cols = m->out_width;
  bool hits_done = false;
  RST_TRY(engine_cross_entropy(e, nullptr, pred, truth, grad_out, nullptr, rows, cols, nullptr,
                               host_accuracy ? &hits_done : nullptr));
  m->inputs_done = false;
  // behind the loss on the stream, ahead of the host's wait for it
  struct Ahead {
    rst_model* m;
    const double* grad;
    static int run(void* p) {
      Ahead* a = static_cast<Ahead*>(p);
      return do_backward_inputs(a->m, a->grad);
    }
  } ahead{m, grad_out};
  const bool go = inputs_ahead != 0 && inputs_ahead_possible(m);
  if (host_accuracy && !hits_done) RST_TRY(engine_accuracy(e, pred, truth, rows, cols, go ? &Ahead::run : nullptr, &ahead));
  else if (go) RST_TRY(do_backward_inputs(m, grad_out));
  const int status = rst_loss_value(e, host_loss);
  if (host_accuracy) *host_accuracy = (double)(*static_cast<volatile unsigned long long*>(e->h_hits)) / (double)rows;
  return status;
}

int rst_model_discard_inputs(rst_model* m) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->inputs_done = false;
  return RST_OK;
}

int rst_model_fuse_sgd(rst_model* m, int enabled) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->fuse_sgd = enabled != 0;
  drop_graph(m);
  return RST_OK;
}

int rst_model_fuse_head(rst_model* m, int enabled) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->fuse_head = enabled <= 0 ? 0 : enabled == 1 ? 1 : 2;
  drop_graph(m);
  return RST_OK;
}

int rst_model_pair_gradients(rst_model* m, int enabled) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->pair_gradients = enabled != 0;
  drop_graph(m);
  return RST_OK;
}

int rst_model_graph_enable(rst_model* m, int enabled) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->graph_mode = enabled == 0 ? 0 : enabled == 1 ? 1 : 2;
  if (!use_graphs(m)) drop_graph(m);
  return RST_OK;
}

int rst_model_graph_active(rst_model* m, int* active) {
  if (!m || !active) return fail(RST_ERR_INVALID_ARGUMENT, "model or result is null");
  *active = use_graphs(m) ? 1 : 0;
  return RST_OK;
}

}  // extern "C"

extern "C" {

int rst_model_profile_enable(rst_model* m, int enabled) {
  if (!m) return fail(RST_ERR_INVALID_ARGUMENT, "model is null");
  m->profiling = enabled != 0;
  prof_reset(m);
  return RST_OK;
}

int rst_model_profile_read(rst_model* m, rst_kernel_record* host_records, size_t capacity,
                           size_t* count) {
  if (!m || !count) return fail(RST_ERR_INVALID_ARGUMENT, "null argument");
  RST_TRY(engine_activate(m->engine));
  RST_HIP(hipStreamSynchronize(m->engine->stream));
  *count = m->slots.size();
  for (size_t i = 0; i < m->slots.size() && i < capacity && host_records; ++i) {
    float ms = 0.f;
    RST_HIP(hipEventElapsedTime(&ms, m->slots[i].start, m->slots[i].stop));
    host_records[i].kind = m->slots[i].kind;
    host_records[i].layer = m->slots[i].layer;
    host_records[i].ms = (double)ms;
    host_records[i].flops = m->slots[i].flops;
    host_records[i].bytes = m->slots[i].bytes;
  }
  prof_reset(m);  // reading consumes the records; their events go back to the pool
  return RST_OK;
}

}  // extern "C"
