// Host-side mirror of rust-autograd's operator interface for the GPU path.
//
// The reference is Rust; this is its C++ counterpart for the same path: `Op` with
// `compute(ComputeContext&)` / `grad(GradientContext&)` (src/op.rs:90-101), a lazy `Graph` of
// `Tensor` handles built with `TensorBuilder` (src/tensor.rs:609-803), reverse-mode `grad()`
// (src/gradient.rs:20-247, src/tensor_ops/mod.rs:94-114), the evaluator (src/evaluation.rs:
// 251-363), `VariableEnvironment` (src/variable.rs) and the `Adam` optimizer
// (src/optimizers/adam.rs).  Arrays live in device memory; every op's numerics is one or more
// calls into the C ABI of libag_hip.so.  Only what the conv / matmul / pool / reduce / Adam path
// and its immediate neighbours need is here; it is not a port of the crate.
#pragma once
#include <stdexcept>
#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <string>
#include <unordered_map>
#include <vector>

namespace ag {
namespace host {

// ---------------------------------------------------------------------------------------------
// errors                                                                        src/op.rs:66-73
// ---------------------------------------------------------------------------------------------
enum class ErrorKind { None = 0, NdArrayError = 1, IncompatibleShape = 2, TypeUnsupported = 3, InvalidDims = 4,
                       OutOfBounds = 5, Hip = 100 };

struct OpError {
    ErrorKind kind = ErrorKind::None;
    std::string message;
    bool ok() const { return kind == ErrorKind::None; }
    static OpError none() { return OpError{}; }
    static OpError make(ErrorKind k, std::string m) { return OpError{k, std::move(m)}; }
};

// Misuse of the API ("Bad op impl: ..." panics of the reference) is reported by throwing this.
struct Panic : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// A file that cannot be read, written or parsed while saving or loading variables; the reference
// returns these as `Err(Box<dyn Error>)` (src/variable.rs:487, 549, 556).
struct PersistError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// ---------------------------------------------------------------------------------------------
// device arrays
// ---------------------------------------------------------------------------------------------
using Shape = std::vector<int64_t>;

struct DeviceBlock;  // one allocation of the caching arena

// Contiguous row-major f32 array in device memory.  Copies share the block (cheap views);
// `deep_copy()` allocates.  A default-constructed array has rank 0 and no storage.
class NdArray {
  public:
    NdArray() = default;
    static NdArray empty(const Shape &shape);
    static NdArray zeros(const Shape &shape);
    static NdArray filled(const Shape &shape, float value);
    static NdArray from_host(const Shape &shape, const float *data);
    static NdArray scalar(float v) { return filled({}, v); }
    // A 0-dimensional 0.0 that every caller shares (the reference's NdArray::zeros(vec![]) of an op
    // without a result, src/op.rs:290-294); nothing writes to it.
    static NdArray shared_zero();
    // Extents without elements: shape() and ndim() answer, there is no storage behind them (ptr() is null).
    static NdArray extents_only(const Shape &shape);
    // Identity of the allocation behind the array (views of one allocation compare equal).
    const void *allocation() const { return block_.get(); }

    const Shape &shape() const { return shape_; }
    int ndim() const { return (int)shape_.size(); }
    size_t len() const;
    float *ptr() const;
    bool defined() const { return block_ != nullptr; }
    NdArray reshaped(const Shape &shape) const;  // same storage, new extents (len must match)
    NdArray deep_copy() const;
    std::vector<float> to_host() const;  // synchronises the stream
    void copy_from_host(const float *data);  // overwrites the elements in place; synchronises
    // Called before the calling thread enqueues work that reads / overwrites the elements: if another thread's
    // stream used the array last, the caller's stream is ordered after it (a no-op for a thread's own arrays).
    void will_read() const;
    void will_write() const;
    // A rearranged copy of the elements that one op made for its kernels and a later op can use again instead of making
    // its own (the zero-bordered upstream gradient, which both gradients of a column-free convolution read).  One slot
    // per allocation, found again by `key` (whatever identifies the arrangement and anything else it was made from);
    // dropped when the array is overwritten (will_write) or freed.  `derived` returns an undefined array when the slot
    // holds nothing for the key.
    NdArray derived(const std::vector<int64_t> &key) const;
    void set_derived(std::vector<int64_t> key, const NdArray &copy) const;
    // Counts the in-place overwrites of the allocation (a key component for copies derived from a second array).
    int64_t version() const;

  private:
    Shape shape_;
    std::shared_ptr<DeviceBlock> block_;
};

int64_t reused_copies();  // NdArray::derived hits of the calling thread so far
// The evaluator's shortcuts -- a node evaluated in its producer's launch (Op::fuses_with_producer), a rearranged copy
// found again (NdArray::derived) -- can be switched off, process-wide, to compare against the plain node-by-node
// evaluation; results are the same bits either way.  On by default.
void set_shortcuts(bool on);
bool shortcuts_enabled();
void *current_stream();  // hipStream_t of the calling thread: every op it evaluates is ordered on it
void synchronize();

// ---------------------------------------------------------------------------------------------
// graph                                                        src/tensor.rs, src/graph.rs
// ---------------------------------------------------------------------------------------------
class Graph;
class Op;
class Context;
using TensorID = int;
using VariableID = int;

struct Tensor {  // a (graph, id) handle, like the reference's Tensor<'graph, F>
    Graph *graph = nullptr;
    TensorID id = -1;
    bool valid() const { return graph && id >= 0; }
};

struct IncomingTensor {  // src/tensor.rs:542-550
    TensorID id;
    bool allow_mut;
    int array_selector;
};

struct TensorInternal {  // src/tensor.rs:408-441
    TensorID id = -1;
    std::unique_ptr<Op> op;
    std::vector<IncomingTensor> incoming_nodes;
    int topo_rank = 0;
    std::string placeholder_name;  // empty = not a placeholder
    bool is_placeholder = false;
    bool is_differentiable = true;
    std::optional<std::vector<IncomingTensor>> backprop_inputs;
    std::optional<Shape> known_shape;  // -1 = unknown extent
    VariableID variable_id = -1;

    bool is_source() const { return incoming_nodes.empty(); }
    bool is_variable() const { return variable_id >= 0; }
    const std::vector<IncomingTensor> &get_backprop_inputs() const
    {
        return backprop_inputs ? *backprop_inputs : incoming_nodes;
    }
};

// ---------------------------------------------------------------------------------------------
// Op and its contexts                                                     src/op.rs:90-434
// ---------------------------------------------------------------------------------------------
// In-place Adam updates of one evaluation, collected so that they go out as one launch over all
// parameters instead of one per AdamOp node.  The evaluator flushes the batch before any node that
// reads an array the batch writes, so every node sees what it would have seen had each update run
// at its own node.
struct AdamJob {
    NdArray p, g, m, v, t;
    float alpha, eps, b1, b2;
};
class DeferredUpdates {
  public:
    void add(AdamJob job);                     // flushes first if the job touches an array of the batch
    bool writes(const NdArray &a) const;       // is `a` one of the batch's param / m / v / t arrays?
    bool reads(const NdArray &a) const;        // is `a` one of the batch's gradient arrays?
    bool empty() const { return jobs_.empty(); }
    void flush();

  private:
    std::vector<AdamJob> jobs_;
};

class ComputeContext {
  public:
    enum class InputKind { NonVariable, RdOnlyVariable, RdWrVariable };
    struct Input {
        NdArray array;
        InputKind kind;
        bool taken = false;
    };
    explicit ComputeContext(std::vector<Input> xs, DeferredUpdates *deferred = nullptr)
        : xs_(std::move(xs)), deferred_(deferred) {}

    // Each input may be grabbed once; variable inputs registered with allow_mut must be grabbed
    // with input_mut (src/op.rs:206-259).
    NdArray input(size_t i);
    NdArray input_mut(size_t i);
    size_t num_inputs() const { return xs_.size(); }
    // Extents of an input without grabbing it (a fusing op decides by them whether it will run).
    const Shape &input_shape(size_t i) const { return xs_.at(i).array.shape(); }

    void append_output(NdArray y) { ys_.push_back(std::move(y)); }
    // A view of an input: copied first when any input is a variable (src/op.rs:273-287).
    void append_output_view(const NdArray &y);
    void append_empty_output() { ys_.push_back(NdArray::shared_zero()); }  // src/op.rs:290-294
    // An Adam update: joins the evaluation's batch, or runs at once when there is none.
    void adam_update(AdamJob job);

    std::vector<NdArray> &outputs() { return ys_; }
    void *stream() const { return current_stream(); }

  private:
    std::vector<Input> xs_;
    std::vector<NdArray> ys_;
    DeferredUpdates *deferred_;
};

class GradientContext {
  public:
    GradientContext(Tensor gy, Tensor y, Graph *g) : gy_(gy), y_(y), graph_(g) {}
    Tensor output_grad() const { return gy_; }
    Tensor output() const { return y_; }
    Tensor input(size_t i) const;
    std::vector<Tensor> inputs() const;
    size_t num_inputs() const;
    Graph *graph() const { return graph_; }
    void append_input_grad(std::optional<Tensor> gx) { gxs_.push_back(gx); }
    std::vector<std::optional<Tensor>> &input_grads() { return gxs_; }

  private:
    Tensor gy_, y_;
    Graph *graph_;
    std::vector<std::optional<Tensor>> gxs_;
};

class Op {
  public:
    virtual ~Op() = default;
    virtual const char *name() const = 0;
    virtual OpError compute(ComputeContext &ctx) const = 0;
    virtual void grad(GradientContext &ctx) const = 0;
    // Evaluation-time fusion with the op that produces input 0 (no counterpart in the reference, whose evaluator
    // runs every node on its own, src/evaluation.rs:310-329).  When the evaluator reaches a node whose first input has
    // not been computed yet and fuses_with_producer(that input's op) holds, it gathers the PRODUCER's inputs instead
    // and calls compute_with_producer: the op may then write the producer's outputs (`producer_outputs`) and its own
    // (ctx) in one pass and return true, or touch nothing and return false, upon which both nodes are evaluated the
    // ordinary way.  The results must have the bits of the two nodes evaluated in turn.
    virtual bool fuses_with_producer(const Op &) const { return false; }
    virtual bool compute_with_producer(ComputeContext &, const Op &, std::vector<NdArray> *, OpError *) const { return false; }
};

class TensorBuilder {  // src/tensor.rs:609-803
  public:
    explicit TensorBuilder(Graph *g) : graph_(g) {}
    TensorBuilder &append_input(Tensor t, bool allow_mut) { return append_input_with_selector(t, allow_mut, 0); }
    TensorBuilder &append_input_with_selector(Tensor t, bool allow_mut, int selector);
    TensorBuilder &append_backprop_input(Tensor t);
    TensorBuilder &set_differentiable(bool d) { differentiable_ = d; return *this; }
    TensorBuilder &set_variable(VariableID v) { variable_id_ = v; return *this; }
    TensorBuilder &set_placeholder_name(std::string n) { placeholder_ = std::move(n); is_placeholder_ = true; return *this; }
    TensorBuilder &set_known_shape(const Shape &s) { known_shape_ = s; return *this; }
    Tensor build(std::unique_ptr<Op> op);

  private:
    Graph *graph_;
    std::vector<IncomingTensor> in_nodes_;
    std::optional<std::vector<IncomingTensor>> backprop_inputs_;
    bool differentiable_ = true;
    VariableID variable_id_ = -1;
    std::string placeholder_;
    bool is_placeholder_ = false;
    std::optional<Shape> known_shape_;
};

// ---------------------------------------------------------------------------------------------
// variables                                                              src/variable.rs
// ---------------------------------------------------------------------------------------------
// Host-memory image of a saved environment: what the reference serialises (src/variable.rs:470-480).
struct SavedArray {
    Shape dim;
    std::vector<float> data;  // row-major
};
struct SavedEnvironment {
    std::vector<SavedArray> array_list;
    std::map<std::string, int> name_to_id;  // "namespace\x01name" -> index into array_list
};
std::string to_json(const SavedEnvironment &env);     // the text serde_json writes for it
SavedEnvironment from_json(const std::string &text);  // throws PersistError
SavedEnvironment read_saved_environment(const std::string &path);
void write_saved_environment(const SavedEnvironment &env, const std::string &path);

class VariableEnvironment {
  public:
    // `namespace_id` "" is the default namespace.  Names are unique inside a namespace.
    VariableID set(const std::string &namespace_id, const std::string &name, NdArray array);
    VariableID set_anonymous(NdArray array);
    std::optional<VariableID> find(const std::string &namespace_id, const std::string &name) const;
    NdArray &array(VariableID id);
    size_t size() const { return arrays_.size(); }
    std::vector<std::pair<std::string, VariableID>> names_in(const std::string &namespace_id) const;

    // Runs `f` with a fresh graph bound to this environment (src/variable.rs:670-683).
    void run(const std::function<void(Context &)> &f);

    // Persistence in the reference's JSON format (src/variable.rs:483-500, 549-554).  `initialize`
    // replaces this environment's arrays and names with the saved ones.  Throw PersistError.
    void save(const std::string &path) const;
    static VariableEnvironment load(const std::string &path);
    void initialize(const std::string &path);

  private:
    std::vector<NdArray> arrays_;
    std::map<std::string, VariableID> name_to_id_;  // "namespace\x01name", src/variable.rs:225-229
};

struct EvalResult {
    OpError error;  // error.ok() => array holds the value
    NdArray array;
};

class Graph {
  public:
    TensorBuilder builder() { return TensorBuilder(this); }
    TensorInternal &node(TensorID id) { return *nodes_.at((size_t)id); }
    const TensorInternal &node(TensorID id) const { return *nodes_.at((size_t)id); }
    size_t num_nodes() const { return nodes_.size(); }
    Tensor tensor(TensorID id) { return Tensor{this, id}; }
    TensorID install(std::unique_ptr<TensorInternal> n);  // src/graph.rs:27-47 (node-count guards)

  private:
    std::vector<std::unique_ptr<TensorInternal>> nodes_;
};

class Evaluator;

class Context : public Graph {  // src/graph.rs Context: graph + variable environment
  public:
    explicit Context(VariableEnvironment *env) : env_(env) {}
    VariableEnvironment &env() { return *env_; }
    Tensor variable(VariableID id);                                              // src/graph.rs variable_by_id
    Tensor variable(const std::string &name, const std::string &namespace_id = "");
    Tensor placeholder(const std::string &name, const Shape &shape);             // src/graph.rs:178-199
    Evaluator evaluator();
    // Graph::eval (src/evaluation.rs:251-363)
    std::vector<EvalResult> eval(const std::vector<Tensor> &tensors,
                                 const std::vector<std::pair<std::string, NdArray>> &feeds);
    // Pairs of nodes that the evaluations of this context so far ran in one pass (Op::compute_with_producer).
    size_t fused_pairs() const { return fused_pairs_; }

  private:
    size_t fused_pairs_ = 0;
    VariableEnvironment *env_;
    std::unordered_map<VariableID, TensorID> var_nodes_;
};

class Evaluator {  // src/evaluation.rs:100-181
  public:
    explicit Evaluator(Context *c) : ctx_(c) {}
    Evaluator &push(Tensor t) { targets_.push_back(t); return *this; }
    Evaluator &extend(const std::vector<Tensor> &ts) { targets_.insert(targets_.end(), ts.begin(), ts.end()); return *this; }
    Evaluator &feed(const std::string &name, NdArray value) { feeds_.emplace_back(name, std::move(value)); return *this; }
    std::vector<EvalResult> run() { return ctx_->eval(targets_, feeds_); }

  private:
    Context *ctx_;
    std::vector<Tensor> targets_;
    std::vector<std::pair<std::string, NdArray>> feeds_;
};

// ---------------------------------------------------------------------------------------------
// tensor_ops: the functional API for this path                   src/tensor_ops/mod.rs
// ---------------------------------------------------------------------------------------------
namespace tensor_ops {
Tensor conv2d(Tensor x, Tensor w, int pad, int stride);                                   // :2733
Tensor dilated_conv2d(Tensor x, Tensor w, int pad, int stride, int dilate);               // :2763
// The same operator made to write the im2col columns as its second output like the reference,
// whatever the geometry (by default large stride-1 / stride-2 convolutions take the column-free path).
Tensor conv2d_with_columns(Tensor x, Tensor w, int pad, int stride, int dilate);
Tensor conv2d_transpose(Tensor x, Tensor w, int pad, int stride);                         // :2799
Tensor dilated_conv2d_transpose(Tensor x, Tensor w, int pad, int stride, int dilate);     // :2834
Tensor max_pool2d(Tensor x, int pool_size, int pad, int stride);                          // :2869
Tensor matmul(Tensor a, Tensor b);                                                        // :1870
Tensor batch_matmul(Tensor a, Tensor b);                                                  // :2007
Tensor batch_matmul_t(Tensor a, Tensor b, bool trans_a, bool trans_b);                    // :1967
Tensor reduce_sum(Tensor x, const std::vector<int> &axes, bool keep_dims);                // :1195
Tensor reduce_mean(Tensor x, const std::vector<int> &axes, bool keep_dims);               // :1227
Tensor sum_all(Tensor x);                                                                 // :1149
Tensor relu(Tensor x);
Tensor add(Tensor a, Tensor b);   // same shape, or b = [1, cols] / [cols] broadcast over the rows of a 2-D a
Tensor mul(Tensor a, Tensor b);   // same shape
Tensor add_n(const std::vector<Tensor> &xs);                                              // :831
Tensor nth_tensor(Tensor x, int n);                                                       // :545
Tensor reshape(Tensor x, const Shape &shape);  // one extent may be -1
Tensor sparse_softmax_cross_entropy(Tensor logits, Tensor labels);
Tensor scalar(float v, Graph *g);
Tensor zeros_like(Tensor x);      // zeros(shape(x)): what grad() returns for a non-differentiable x
Tensor stop_gradient(Tensor x);
std::vector<Tensor> grad(const std::vector<Tensor> &ys, const std::vector<Tensor> &xs);   // :94
std::vector<Tensor> grad_with_default(const std::vector<Tensor> &ys, const std::vector<Tensor> &xs,
                                      const std::vector<Tensor> &ys_grads);                  // :130
}  // namespace tensor_ops

// ---------------------------------------------------------------------------------------------
// optimizers                                        src/optimizers/mod.rs, src/optimizers/adam.rs
// ---------------------------------------------------------------------------------------------
namespace optimizers {
// (variables, gradients) of every variable of `namespace_id` the losses depend on (mod.rs:21-46).
std::pair<std::vector<Tensor>, std::vector<Tensor>> grad_helper(const std::vector<Tensor> &losses, Context &ctx,
                                                                const std::string &namespace_id = "");

class Adam {
  public:
    // Allocates m, v (zeros) and t (= 1) for every listed variable in `adam_namespace_id`
    // under the names "<id>m", "<id>v", "<id>t" (adam.rs:75-112).
    Adam(float alpha, float eps, float b1, float b2, const std::vector<VariableID> &vars, VariableEnvironment &env,
         std::string adam_namespace_id);
    static Adam with_defaults(const std::vector<VariableID> &vars, VariableEnvironment &env,
                              std::string adam_namespace_id)
    {
        return Adam(0.001f, 1e-08f, 0.9f, 0.999f, vars, env, std::move(adam_namespace_id));
    }
    std::vector<Tensor> compute_updates(const std::vector<Tensor> &params, const std::vector<Tensor> &grads,
                                        Context &ctx) const;                                     // adam.rs:116-153
    void update(const std::vector<Tensor> &params, const std::vector<Tensor> &grads, Context &ctx,
                const std::vector<std::pair<std::string, NdArray>> &feeds) const;                // mod.rs:66-85
    Tensor get_update_op(const std::vector<Tensor> &params, const std::vector<Tensor> &grads, Context &ctx) const;

  private:
    float alpha_, eps_, b1_, b2_;
    std::string ns_;
};
}  // namespace optimizers

}  // namespace host
}  // namespace ag
