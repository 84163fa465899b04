/*
 * rstorch_hip.h - C ABI of the MI355X (gfx950) backend for the rstorch f64 training step.
 *
 * The reference crate is pure Rust and has no FFI of its own; its hot path sits behind the
 * traits `Module` (src/module/mod.rs:42-56), `Loss` (src/loss/mod.rs:6-11) and `Optimizer`
 * (src/optim/mod.rs:6-8).  These entry points are what a Rust (or C++/Python) implementation
 * of those traits binds with `extern "C"`: plain pointers and sizes only.
 *
 * Conventions
 *   - every matrix is dense row-major f64 without strides (the reference's Array2<f64>);
 *     `double*` arguments are DEVICE pointers unless the name says `host`;
 *   - every function returns an rst_status; on failure rst_last_error() gives a message for
 *     the calling thread and rst_last_hip_error() the hipError_t, if HIP raised it.  The
 *     reference panics in these situations (unwrap on a consumed cache, ndarray shape
 *     mismatch, NaN in softmax); a binding turns the status into its own panic/exception;
 *   - work is enqueued on the engine's stream and runs asynchronously; only the calls that
 *     hand a value back to the host (downloads, the scalar loss) wait for it;
 *   - one engine is used from one thread at a time (the reference is single-threaded,
 *     nothing in it is Send/Sync).
 */
#ifndef RSTORCH_HIP_H
#define RSTORCH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum rst_status {
  RST_OK = 0,
  RST_ERR_INVALID_ARGUMENT = 1, /* null pointer, zero handle, bad enum */
  RST_ERR_SHAPE = 2,            /* operand shapes do not agree (ndarray would panic) */
  RST_ERR_STATE = 3,            /* backward before forward, step before backward, ... */
  RST_ERR_HIP = 4,              /* a HIP call failed; see rst_last_hip_error() */
  RST_ERR_NAN = 5,              /* NaN logits: the reference panics in softmax.rs:38 */
  RST_ERR_OUT_OF_MEMORY = 6,
  RST_ERR_UNSUPPORTED = 7
} rst_status;

typedef struct rst_engine rst_engine; /* one GPU + one stream + small scratch buffers */
typedef struct rst_model rst_model;   /* a device-resident Sequential of Identity/Linear/ReLU */
typedef struct rst_event rst_event;   /* a timestamp on the engine's stream */

/* ---- errors ---------------------------------------------------------------------------- */
const char* rst_last_error(void);
int rst_last_hip_error(void);
const char* rst_status_string(int status);

/* ---- engine ---------------------------------------------------------------------------- */
/* Opens device `device`, creates the stream every later call is ordered on. */
int rst_engine_create(int device, rst_engine** out);
int rst_engine_destroy(rst_engine* engine);
/* Blocks until everything enqueued so far has finished. */
int rst_engine_synchronize(rst_engine* engine);
/* The hipStream_t, for callers that order their own HIP work against the engine's. */
void* rst_engine_stream(rst_engine* engine);
/* Device name and number of compute units (for reports). */
int rst_engine_device_info(rst_engine* engine, char* name, size_t name_capacity,
                           int* compute_units, size_t* total_memory_bytes);

/* ---- device memory (counts are numbers of doubles) -------------------------------------- */
/* rst_free keeps the block in a per-engine cache for the next rst_malloc of the same size (no
 * device synchronisation on either call); rst_engine_trim returns the cache to the driver. */
int rst_malloc(rst_engine* engine, size_t count, double** out);
int rst_free(rst_engine* engine, double* ptr);
int rst_engine_trim(rst_engine* engine);
int rst_upload(rst_engine* engine, double* dst, const double* host_src, size_t count);
int rst_download(rst_engine* engine, double* host_dst, const double* src, size_t count);
int rst_copy(rst_engine* engine, double* dst, const double* src, size_t count);
int rst_fill(rst_engine* engine, double* dst, size_t count, double value);

/* ---- timing on the engine's stream ------------------------------------------------------ */
int rst_event_create(rst_engine* engine, rst_event** out);
/* May be called after the event's engine has been destroyed (record and elapsed may not). */
int rst_event_destroy(rst_event* event);
int rst_event_record(rst_event* event);
/* Work enqueued on `engine` after this call starts only once `event` (recorded on any engine of the
 * same GPU) has happened; the host does not wait.  How two engines - two streams - hand buffers to
 * each other, e.g. a loader engine that refills an input array while the training engine works. */
int rst_event_wait(rst_engine* engine, rst_event* event);
/* Waits for `stop` and returns the time between the two records in milliseconds. */
int rst_event_elapsed_ms(rst_event* start, rst_event* stop, double* host_ms);

/* ---- Linear (replaces src/module/linear.rs:43-57 and :60-69) ----------------------------- */
/* out[batch,out_features] = x[batch,in_features] . weight[out_features,in_features]^T, then
 * + bias[1,out_features] (bias may be NULL).  With fuse_relu != 0 the ReLU that follows the
 * layer (src/module/activation/relu.rs:19-22) is applied in the same kernel: out = max(z, 0). */
int rst_linear_forward(rst_engine* engine, const double* x, const double* weight,
                       const double* bias, double* out, size_t batch, size_t in_features,
                       size_t out_features, int fuse_relu);
/* n = batch.  grad_weight[out,in] = (grad^T . x) / n;  grad_bias[1,out] = colsum(grad) / n
 * (NULL: skipped);  grad_input[batch,in] = grad . weight, not scaled (NULL: skipped).
 * relu_mask_source (may be NULL) is the [batch,in] pre-activation or output of a ReLU that
 * fed this layer: grad_input is then multiplied by (source > 0 ? 1 : 0), which is that ReLU's
 * backward (src/module/activation/relu.rs:25-27) fused into the epilogue. */
int rst_linear_backward(rst_engine* engine, const double* grad, const double* x,
                        const double* weight, double* grad_weight, double* grad_bias,
                        double* grad_input, const double* relu_mask_source, size_t batch,
                        size_t in_features, size_t out_features);

/* ---- ReLU, unfused (src/module/activation/relu.rs:19-27) --------------------------------- */
int rst_relu_forward(rst_engine* engine, const double* x, double* out, size_t count);
/* out = grad * (x > 0 ? 1 : 0); x may be the pre-activation or the ReLU output. */
int rst_relu_backward(rst_engine* engine, const double* grad, const double* x, double* out,
                      size_t count);

/* ---- softmax over each row (src/module/activation/softmax.rs:45-53, axis 1) -------------- */
/* Returns RST_ERR_NAN when a logit is NaN (checked when the call returns: this call waits). */
int rst_softmax_rows(rst_engine* engine, const double* x, double* out, size_t rows, size_t cols);

/* The Softmax MODULE (src/module/activation/softmax.rs:55-78; not on the training path, which
 * uses the free function through CrossEntropyLoss).  forward: softmax along `axis` (1: rows,
 * 0: columns; Softmax::with_axis).  backward: ONE cols x cols matrix for the whole batch,
 * jacobian = -(output^T . output) with each diagonal entry d replaced by d*(1-d), and
 * grad_input = grad . jacobian - literally what the reference computes. */
int rst_softmax_forward(rst_engine* engine, const double* x, double* out, size_t rows, size_t cols,
                        int axis);
int rst_softmax_backward(rst_engine* engine, const double* grad, const double* output,
                         double* grad_input, size_t rows, size_t cols);

/* ---- CrossEntropyLoss (src/loss/cross_entropy.rs:34-47) ---------------------------------- */
/* One pass: prob = softmax(pred); loss = -(sum truth*ln(prob)) / rows; grad_out = prob - truth
 * (what `backward()` returns; NOT divided by rows).  prob_out may be NULL.  host_loss may be
 * NULL, in which case nothing waits and the loss stays in the engine (rst_loss_value). */
int rst_cross_entropy(rst_engine* engine, const double* pred, const double* truth,
                      double* grad_out, double* prob_out, size_t rows, size_t cols,
                      double* host_loss);
/* rst_cross_entropy with host_loss, and rst_accuracy(pred, truth) (src/utils.rs:55-65) with it: what
 * the README loop asks for back to back (README.md:66-67), answered after ONE wait.  Rows of up to
 * 512 logits (256 when the arrays are not 16-byte aligned or the width is odd) are counted by the
 * cross-entropy launches themselves; for wider rows the arg-max launch follows on the stream.  Same
 * loss bits as rst_cross_entropy, same count as rst_accuracy. */
int rst_cross_entropy_accuracy(rst_engine* engine, const double* pred, const double* truth,
                               double* grad_out, size_t rows, size_t cols, double* host_loss,
                               double* host_accuracy);
/* The loss of the latest rst_cross_entropy on this engine; waits for it.  RST_ERR_NAN if a
 * logit was NaN. */
int rst_loss_value(rst_engine* engine, double* host_loss);

/* No counterpart in the reference.  For callers that cannot allocate device memory at the time of
 * the call (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * the same computation and the same bits as rst_cross_entropy without prob_out, but the per-row
 * loss terms, the loss word and the NaN flags live in a fixed array inside the library's device
 * image (RST_STATIC_CROSS_ENTROPY_MAX_ROWS doubles + 256 bytes on every GPU the library runs on,
 * held until the process ends) instead of engine buffers that grow on demand.  The call allocates
 * and frees nothing.  More rows than the maximum: RST_ERR_UNSUPPORTED.  Every call on one GPU
 * shares that GPU's array: calls that overlap there (two engines, two threads) race. */
#define RST_STATIC_CROSS_ENTROPY_MAX_ROWS 65536
int rst_cross_entropy_static(rst_engine* engine, const double* pred, const double* truth,
                             double* grad_out, size_t rows, size_t cols, double* host_loss);

/* ---- SGD (src/optim/sgd.rs:19-24) -------------------------------------------------------- */
/* parm[i] = parm[i] - (lr * grad[i]) for every tensor in ONE launch: the product is rounded,
 * then the difference (no fused multiply-add), as in the reference.  The arrays are HOST
 * arrays of `tensor_count` device pointers / element counts. */
int rst_sgd_step(rst_engine* engine, double* const* host_parm_ptrs,
                 const double* const* host_grad_ptrs, const size_t* host_counts,
                 size_t tensor_count, double lr);
/* Same update over one contiguous range (a parameter arena). */
int rst_sgd_step_flat(rst_engine* engine, double* parm, const double* grad, size_t count,
                      double lr);

/* ---- accuracy (src/utils.rs:44-65) ------------------------------------------------------- */
/* Fraction of rows whose arg-max column (first maximum wins) agrees between pred and truth. */
int rst_accuracy(rst_engine* engine, const double* pred, const double* truth, size_t rows,
                 size_t cols, double* host_accuracy);

/* ---- synthetic data and initialisers (src/module/init/{mod,he,xavier,sigma}.rs) ----------- */
/* value(seed, stream, index) is a pure function (counter-based generator), so a tensor does
 * not depend on launch geometry.  The reference draws from an unseedable thread RNG; these
 * give the same distributions reproducibly: KaimingNormal is std = 1/sqrt(in_features). */
int rst_fill_uniform(rst_engine* engine, double* dst, size_t count, uint64_t seed,
                     uint64_t stream, double lo, double hi);
int rst_fill_normal(rst_engine* engine, double* dst, size_t count, uint64_t seed,
                    uint64_t stream, double mean, double std);
/* dst[rows,cols] = one-hot rows with labels uniform over the columns (src/utils.rs:38-42). */
int rst_fill_one_hot(rst_engine* engine, double* dst, size_t rows, size_t cols, uint64_t seed,
                     uint64_t stream);

/* ---- input staging (the step before the path: src/data/data_loader.rs:192-207 builds a batch
 *      on the host, src/utils.rs:38-42 expands labels to one-hot rows) ------------------------ */
typedef struct rst_stager rst_stager;
/* `depth` slots of pinned host memory + device memory and a copy stream of its own: the transfer
 * of batch k+1 overlaps the training step on batch k.  x is [rows <= max_rows, x_cols] f64. */
int rst_stager_create(rst_engine* engine, size_t max_rows, size_t x_cols, size_t classes,
                      int depth, rst_stager** out);
int rst_stager_destroy(rst_stager* stager);
/* Copies the host batch into the next free slot and starts its transfer; does not wait for the
 * GPU.  Labels are class indices; the dense one-hot truth [rows, classes] is built on the device.
 * RST_ERR_STATE when all slots are submitted and none has been taken with rst_stager_next. */
int rst_stager_submit_labels(rst_stager* stager, const double* host_x, const uint32_t* host_labels,
                             size_t rows);
/* The same in two halves, without the intermediate copy: rst_stager_acquire_host returns the
 * pinned buffers of the next free slot (x: max_rows * x_cols doubles, labels: max_rows u32; it
 * waits until the slot's previous transfer has left them) for the caller's loader to fill in
 * place, rst_stager_commit_labels(rows) starts the transfer of what was written. */
int rst_stager_acquire_host(rst_stager* stager, double** host_x, uint32_t** host_labels);
int rst_stager_commit_labels(rst_stager* stager, size_t rows);
/* Same with a dense (possibly soft-label) truth matrix [rows, classes]. */
int rst_stager_submit_dense(rst_stager* stager, const double* host_x, const double* host_truth,
                            size_t rows);
/* Hands out the oldest submitted batch: the engine's stream waits for its transfer (the host does
 * not).  The device arrays stay valid until `depth` further submits; work that reads them must
 * be enqueued on the engine before the submit that reuses their slot. */
int rst_stager_next(rst_stager* stager, const double** x_dev, const double** truth_dev,
                    size_t* rows);

/* ---- device-resident Sequential (src/module/sequential.rs:78-109) ------------------------ */
enum { RST_LAYER_IDENTITY = 0, RST_LAYER_LINEAR = 1, RST_LAYER_RELU = 2 };

/* kinds[i] is one of RST_LAYER_*; in_features/out_features are read for LINEAR entries.
 * All weights, biases and their gradients live in two contiguous device arenas (parameters
 * and gradients, same layout), zero-initialised. */
int rst_model_create(rst_engine* engine, const int* kinds, const size_t* in_features,
                     const size_t* out_features, size_t layer_count, rst_model** out);
int rst_model_destroy(rst_model* model);
/* Number of parameter tensors (2 per Linear) and total number of f64 parameters. */
int rst_model_parameter_count(rst_model* model, size_t* tensor_count, size_t* element_count);
/* Tensor `index` in the reference's order (per Linear in layer order: weight (out,in), then
 * bias (1,out); src/module/linear.rs:71-78): device pointers of the parameter and its gradient. */
int rst_model_parameter(rst_model* model, size_t index, double** parm, double** grad,
                        size_t* rows, size_t* cols);
/* Every parameter packed without padding into / out of one host array of `count` =
 * element_count doubles, tensors in the order of rst_model_parameter (a checkpoint; the reference
 * has no serialisation, its weights are reachable only through parameters(), mod.rs:16-40). */
int rst_model_export_parameters(rst_model* model, double* host_dst, size_t count);
int rst_model_import_parameters(rst_model* model, const double* host_src, size_t count);
/* KaimingNormal weights (std = 1/sqrt(in)), zero biases (src/module/init/mod.rs:15-17,
 * he.rs:11-14); tensor i uses generator stream `first_stream + i`. */
int rst_model_init_kaiming(rst_model* model, uint64_t seed, uint64_t first_stream);
/* forward: x[batch, in] -> *logits (device pointer owned by the model, [batch, out]).
 * Linear+ReLU pairs run as one kernel; the input is referenced, not copied, until backward. */
int rst_model_forward(rst_model* model, const double* x, size_t batch, const double** logits);
/* CrossEntropyLoss::forward on the logits of the last forward (truth[batch, classes], dense).
 * host_loss may be NULL (no wait).  Keeps prob - truth for rst_model_backward. */
int rst_model_loss(rst_model* model, const double* truth, double* host_loss);
/* Sequential::backward.  grad == NULL: start from the gradient rst_model_loss kept
 * (loss.backward()); otherwise from grad[batch, out].  need_input_grad == 0 skips the first
 * Linear's input gradient, which the README loop discards; otherwise *input_grad receives it. */
int rst_model_backward(rst_model* model, const double* grad, int need_input_grad,
                       const double** input_grad);
/* The same two passes for a host-side Sequential that hands arrays over BY VALUE, as the reference's
 * Module::forward / backward do (src/module/mod.rs:45-47, sequential.rs:78-90): the logits and the
 * input gradient are written into arrays the caller owns instead of buffers the model reuses.
 * rst_model_forward_to: logits_out[batch, out].  The model keeps x and logits_out by address until
 * the backward pass (a trailing ReLU reads logits_out again as its mask): the caller keeps both
 * alive and unchanged until then.
 * rst_model_backward_to: grad[batch, out] is the gradient with respect to the logits (what
 * loss.backward() returned); input_grad_out[batch, in] may be NULL, which skips the first Linear's
 * input gradient (the README loop drops it).  apply_sgd != 0 also runs SGD::step(lr): inside the
 * weight-gradient launches (see rst_model_fuse_sgd), i.e. `model.backward(g); optim.step(&mut model)`
 * as one pass with the same bits as the two calls apart.
 * Both launch plainly (no recorded graph): their caller reads the loss between them, so the first
 * kernel of each pass should start as soon as the call is made. */
int rst_model_forward_to(rst_model* model, const double* x, size_t batch, double* logits_out);
int rst_model_backward_to(rst_model* model, const double* grad, double* input_grad_out, int apply_sgd,
                          double lr);
/* The loss and the accuracy of the logits that the model's latest rst_model_forward_to wrote
 * (pred must be that address), for the loop of README.md:64-74, whose host waits for the loss
 * between the forward and the backward pass: rst_cross_entropy_accuracy(pred, truth, grad_out, ...)
 * and, with inputs_ahead != 0, the part of the coming backward pass that changes nothing a caller
 * can see - the input gradients of every Linear above the first, from grad_out, into the model's own
 * buffers - launched behind the loss kernels BEFORE the host waits, so that the GPU has work while the
 * host wakes up and enqueues the rest.  Same kernels on the same operands as rst_model_backward_to
 * would launch: a following rst_model_backward_to(model, grad_out, ...) skips them and its results
 * are the same to the bit; with any other grad address it computes everything itself.  The caller
 * promises that grad_out is not rewritten in between, or calls rst_model_discard_inputs.  Only small
 * models take part (every weight gradient waits for the shared grid at the end of backward anyway,
 * every ReLU sits right below a Linear, profiling is off); for the others inputs_ahead is ignored.
 * host_accuracy may be NULL (the loss alone, as rst_cross_entropy). */
int rst_model_loss_accuracy_to(rst_model* model, const double* pred, const double* truth,
                               double* grad_out, int inputs_ahead, double* host_loss,
                               double* host_accuracy);
int rst_model_discard_inputs(rst_model* model);
/* SGD::step over every parameter of the model (one launch over the arena). */
int rst_model_sgd_step(rst_model* model, double lr);
/* forward, loss, backward, step: the README loop body (README.md:64-74) without accuracy,
 * i.e. what the reference's private BasicModel::step (src/model.rs:19-27) does.
 * host_loss may be NULL: then the call returns without waiting for the GPU. */
int rst_model_train_step(rst_model* model, const double* x, const double* truth, size_t batch,
                         double lr, double* host_loss);
/* By default rst_model_train_step applies SGD::step inside the weight-gradient launches (each
 * stores its gradient, then updates the parameter at the same index: parm - (lr * grad), two
 * roundings, the same bits as the separate pass; the layer's input gradient, which needs the
 * old weights, is launched first).  enabled == 0 runs the optimiser as its own pass over the
 * parameter arena, as rst_model_sgd_step does. */
int rst_model_fuse_sgd(rst_model* model, int enabled);
/* enabled != 0: the backward pass holds each layer's weight gradient back until the next layer's
 * input gradient is due and launches the two, which do not depend on each other, as one grid when
 * both are large products (a 256-tile input gradient alone leaves one workgroup per CU).
 * Results are identical either way.  On by default (measured on MI355X at C4's hidden width:
 * 0.946 ms per pair against 0.477 + 0.503 ms for the two launches one after the other). */
int rst_model_pair_gradients(rst_model* model, int enabled);
/* How much of a small classifier's tail rst_model_train_step runs as ONE launch.
 * enabled >= 1: when the model ends in a Linear with at most 16 outputs on at most 288 inputs, that
 * Linear's forward (src/module/linear.rs:44-58), the cross entropy with its gradient
 * (src/loss/cross_entropy.rs:34-47), the Linear's input gradient (linear.rs:68, masked by a preceding
 * ReLU, relu.rs:25-28) and the final sum of the loss are one launch instead of four.
 * enabled >= 2 (the default): when, besides, the Linear in front of it - with nothing but a ReLU
 * between the two - has at most 112 inputs and 112 outputs, its forward and its input gradient run in
 * the same launch too (its weights sit in LDS; both products run on the matrix cores), which saves two
 * more launches.
 * enabled == 0: the separate launches.  The environment variable RSTORCH_HEAD (0, 1; anything else: 2)
 * sets the level new models start with.
 * The fused sums are taken in another order than those of the contraction kernels (the head: 16 lanes
 * share a row, each adding every 16th term, then the lanes' sums; the hidden layer: four interleaved
 * partial sums per output), so results differ from the unfused launches by rounding (1e-15 relative);
 * they are deterministic and do not depend on the number of compute units or on the order in which
 * workgroups finish.  The separate calls (rst_model_forward / _loss / _backward, and the *_to variants)
 * are not affected. */
int rst_model_fuse_head(rst_model* model, int enabled);
/* How rst_model_train_step launches its kernels.
 * enabled == 1: it records them into a HIP graph the first time it sees a given (x, truth, batch, lr)
 * and replays the graph afterwards; a different argument re-records (the 64 most recently used graphs
 * of a model are kept).  enabled == 0: plain launches (profiling does so by itself).
 * enabled == 2, the default: the graph for models of eight Linear layers or more, plain launches for
 * shallower ones - measured on MI355X, a replayed graph of the four or five launches of a shallow
 * model's step starts later than the first of as many plain launches and costs the host 12 us more
 * when it reads the loss after every step (the README network at batch 32 with the loss read every
 * step: 30.0 k steps/s plain, 19.3 k replayed), while from about 25 small launches per step on the
 * graph is ahead.  The environment variable RSTORCH_GRAPH (0 or 1) fixes the mode new models start
 * with.  rst_model_graph_active tells whether the model's next step would be replayed. */
int rst_model_graph_enable(rst_model* model, int enabled);
int rst_model_graph_active(rst_model* model, int* active);
/* Environment variables read once per process.  RSTORCH_GRAPH=0 / 1: new models launch plainly / replay
 * a recorded graph, whatever their depth.
 * The next two change which kernel a product runs on and therefore the ORDER of its summation
 * (results stay within rounding, 1e-13 relative, of each other; every setting is deterministic and
 * independent of the number of compute units):
 *   RSTORCH_DMA_GROUP=0  small weight gradients never share the grid of K-sliced 128x128 tiles,
 *                    =1  they do whenever they can (unset: the measured rule);
 *   RSTORCH_DMA64=0      no product goes to the 64x64 direct-to-LDS kernel, =1 every eligible one;
 *   RSTORCH_HEAD=0 / 1   new models keep the classifier's tail as separate launches / fuse the head alone
 *                        (rst_model_fuse_head). */
/* Per-launch timing of the model's kernels: when enabled an event is recorded on the engine's
 * stream after every launch (and one before the first launch of a call); a launch's duration runs
 * from the previous event to its own, so it includes the few microseconds between the previous
 * kernel's end and its own start.  While enabled, every layer's weight gradient is a launch of
 * its own.  Small ones otherwise share one grid at the end of backward: bit-identical to the
 * launches of their own as long as the shared grid runs 32x32 tiles, equal within rounding (1e-13
 * relative) when the batch is long enough (from about 4096 rows) for the shared grid of K-sliced
 * 128x128 tiles, which cuts the batch into other slices than a lone launch does and so adds in
 * another order.  Records
 * accumulate over calls (up to 65536) until rst_model_profile_read, which waits for the stream,
 * copies up to `capacity` of them (host_records == NULL: only counts) and clears the list. */
typedef struct rst_kernel_record {
  int kind;          /* RST_KERNEL_* */
  int layer;         /* layer index, -1 for loss / optimiser */
  double ms;         /* launch duration */
  double flops;      /* algorithmic flops (2*M*N*K for the contractions, else 0) */
  double bytes;      /* algorithmic HBM bytes */
} rst_kernel_record;
enum {
  RST_KERNEL_LINEAR_FORWARD = 0,
  RST_KERNEL_GRAD_WEIGHT = 1,
  RST_KERNEL_GRAD_BIAS = 2,
  RST_KERNEL_GRAD_INPUT = 3,
  RST_KERNEL_RELU_FORWARD = 4,
  RST_KERNEL_RELU_BACKWARD = 5,
  RST_KERNEL_CROSS_ENTROPY = 6,
  RST_KERNEL_LOSS_REDUCE = 7,
  RST_KERNEL_SGD = 8,
  RST_KERNEL_GRAD_PAIR = 9   /* one layer's input gradient and the weight gradient of the layer above, one grid */
};
int rst_model_profile_enable(rst_model* model, int enabled);
int rst_model_profile_read(rst_model* model, rst_kernel_record* host_records, size_t capacity,
                           size_t* count);

#ifdef __cplusplus
}
#endif
#endif /* RSTORCH_HIP_H */
