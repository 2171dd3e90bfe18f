// Device arrays, graph construction, the evaluator and the variable environment.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <stdexcept>

#include "ag_hip.h"
#include "ag_host.hpp"

namespace ag {
namespace host {

// ---------------------------------------------------------------------------------------------
// Streams.  The reference evaluates a graph on the thread that owns it (Graph is neither Send nor Sync,
// src/graph.rs:17-47); here every host thread that evaluates graphs has a stream of its own (non-blocking, default
// priority), created at its first use and handed to a later thread when this one ends.  Everything a thread enqueues
// -- kernels, feeds, read-backs -- is ordered on its stream, so evaluations on different threads overlap on the
// device and none of them waits for the null stream.
// ---------------------------------------------------------------------------------------------
namespace {
void check(hipError_t e, const char *what)
{
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

struct StreamPool {  // streams of threads that have ended (never destroyed: the runtime may outlive or precede us at exit)
    std::mutex mu;
    std::vector<hipStream_t> idle;
};
StreamPool &stream_pool()
{
    static StreamPool *p = new StreamPool;  // leaked on purpose: thread-local destructors may run after statics elsewhere
    return *p;
}
struct ThreadStream {
    hipStream_t stream = nullptr;
    hipEvent_t handoff = nullptr;  // marks "everything enqueued so far" on another thread's stream
    hipStream_t get()
    {
        if (!stream) {
            StreamPool &pool = stream_pool();
            {
                std::lock_guard<std::mutex> lk(pool.mu);
                if (!pool.idle.empty()) {
                    stream = pool.idle.back();
                    pool.idle.pop_back();
                }
            }
            if (!stream) check(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");
        }
        return stream;
    }
    ~ThreadStream()
    {
        if (!stream) return;
        StreamPool &pool = stream_pool();
        std::lock_guard<std::mutex> lk(pool.mu);
        pool.idle.push_back(stream);  // its arena blocks stay with it
    }
};
thread_local ThreadStream t_stream;

// Orders the calling thread's stream after everything enqueued so far on `other`.
void wait_for_stream(hipStream_t other)
{
    hipStream_t mine = t_stream.get();
    if (other == mine) return;
    if (!t_stream.handoff) check(hipEventCreateWithFlags(&t_stream.handoff, hipEventDisableTiming), "hipEventCreate");
    check(hipEventRecord(t_stream.handoff, other), "hipEventRecord");
    check(hipStreamWaitEvent(mine, t_stream.handoff, 0), "hipStreamWaitEvent");
}
}  // namespace

void *current_stream() { return t_stream.get(); }

void synchronize() { check(hipStreamSynchronize(t_stream.get()), "hipStreamSynchronize"); }

// ---------------------------------------------------------------------------------------------
// caching device arena: freed blocks are kept in per-size free lists, so a training loop that
// rebuilds its graph every step (as the reference does, src/variable.rs:670-683) stops calling
// hipMalloc after the first step.  The lists are per stream: a block goes back to the list of the stream it
// was allocated for and is handed out again only to work on that stream, which is ordered after whatever used
// the block before.
// ---------------------------------------------------------------------------------------------
struct DeviceBlock {
    void *ptr = nullptr;   // what the array uses
    void *base = nullptr;  // what hipMalloc returned
    size_t bytes = 0;
    hipStream_t owner = nullptr;  // the stream whose free list the block returns to
    // Hand-offs between threads: the stream that last wrote the block and the streams that have read it since.
    // A thread that touches a block last used on another thread's stream first orders its own stream after that
    // one (NdArray::will_read / will_write); the callers serialise their accesses, as the reference's borrow rules
    // make them.  `constant`: written once, synchronously, before anyone else sees it (the shared zero).
    std::mutex mu;
    hipStream_t writer = nullptr;
    std::vector<hipStream_t> readers;
    bool constant = false;
    // NdArray::derived / set_derived / version
    std::vector<int64_t> derived_key;
    NdArray derived;
    int64_t version = 0;
    ~DeviceBlock();
};

namespace {
// Large blocks start a rotating multiple of 4 KiB into their allocation.  hipMalloc hands out addresses with the
// same low 21 bits, and an elementwise kernel that streams several such arrays in lockstep then sends all of its
// streams to the same DRAM banks at the same time (the pooling backward over gy, the tap bytes and gx moves
// between 0.83 and 0.91 of its best with the placement).
constexpr size_t kStaggerFrom = (size_t)1 << 20, kStaggerStep = 4096, kStaggerSlots = 16;

struct Arena {
    struct Free {
        void *base, *ptr;
    };
    std::mutex mu;
    std::map<hipStream_t, std::multimap<size_t, Free>> free_blocks;
    size_t next_slot = 0;
    ~Arena()
    {
        for (auto &per_stream : free_blocks)
            for (auto &kv : per_stream.second) (void)hipFree(kv.second.base);
    }
    static size_t round_up(size_t bytes)
    {
        const size_t q = bytes < (1u << 20) ? 256 : (1u << 16);
        return (bytes + q - 1) / q * q;
    }
    bool take(hipStream_t st, size_t bytes, Free *out)
    {
        std::lock_guard<std::mutex> lk(mu);
        auto &list = free_blocks[st];
        auto it = list.lower_bound(bytes);
        if (it != list.end() && it->first <= bytes + bytes / 8) {
            *out = it->second;
            list.erase(it);
            return true;
        }
        return false;
    }
    size_t stagger()
    {
        std::lock_guard<std::mutex> lk(mu);
        return (next_slot++ % kStaggerSlots) * kStaggerStep;
    }
    void give(hipStream_t st, size_t bytes, Free f)
    {
        std::lock_guard<std::mutex> lk(mu);
        free_blocks[st].emplace(bytes, f);
    }
};
Arena &arena()
{
    static Arena a;
    return a;
}
std::shared_ptr<DeviceBlock> allocate(size_t bytes)
{
    auto blk = std::make_shared<DeviceBlock>();
    blk->bytes = Arena::round_up(bytes ? bytes : 4);
    blk->owner = blk->writer = t_stream.get();
    Arena::Free f;
    if (arena().take(blk->owner, blk->bytes, &f)) {
        blk->base = f.base;
        blk->ptr = f.ptr;
        return blk;
    }
    const bool large = blk->bytes >= kStaggerFrom;
    check(hipMalloc(&blk->base, blk->bytes + (large ? kStaggerStep * kStaggerSlots : 0)), "hipMalloc");
    blk->ptr = static_cast<char *>(blk->base) + (large ? arena().stagger() : 0);
    return blk;
}
size_t product(const Shape &s)
{
    size_t n = 1;
    for (int64_t d : s) n *= (size_t)d;
    return n;
}
}  // namespace

DeviceBlock::~DeviceBlock()
{
    if (!base) return;
    // The block returns to its owner's list.  If other streams used it last, the owner must not reuse it before
    // they are done: the thread that drops the last reference orders the owner after them here.
    std::vector<hipStream_t> others;
    if (writer && writer != owner) others.push_back(writer);
    for (hipStream_t r : readers)
        if (r != owner) others.push_back(r);
    for (hipStream_t o : others) {
        hipEvent_t ev = nullptr;
        if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) == hipSuccess) {
            (void)hipEventRecord(ev, o);
            (void)hipStreamWaitEvent(owner, ev, 0);
            (void)hipEventDestroy(ev);
        }
    }
    arena().give(owner, bytes, Arena::Free{base, ptr});
}

void NdArray::will_read() const
{
    if (!block_ || block_->constant) return;
    hipStream_t mine = t_stream.get(), w;
    {
        std::lock_guard<std::mutex> lk(block_->mu);
        w = block_->writer;
        if (w == mine && block_->readers.empty()) return;  // the usual case: a thread's own array
        if (std::find(block_->readers.begin(), block_->readers.end(), mine) == block_->readers.end()) block_->readers.push_back(mine);
    }
    if (w && w != mine) wait_for_stream(w);
}

void NdArray::will_write() const
{
    if (!block_ || block_->constant) return;
    hipStream_t mine = t_stream.get();
    std::vector<hipStream_t> before;
    NdArray dropped;  // (released outside the lock)
    {
        std::lock_guard<std::mutex> lk(block_->mu);
        ++block_->version;
        std::swap(dropped, block_->derived);
        block_->derived_key.clear();
        if (block_->writer == mine && block_->readers.empty()) return;
        if (block_->writer && block_->writer != mine) before.push_back(block_->writer);
        for (hipStream_t r : block_->readers)
            if (r != mine) before.push_back(r);
        block_->writer = mine;
        block_->readers.clear();
    }
    for (hipStream_t o : before) wait_for_stream(o);
}

static thread_local int64_t t_reused_copies = 0;

static std::atomic<bool> g_shortcuts{true};
void set_shortcuts(bool on) { g_shortcuts.store(on); }
bool shortcuts_enabled() { return g_shortcuts.load(std::memory_order_relaxed); }

NdArray NdArray::derived(const std::vector<int64_t> &key) const
{
    NdArray d;
    if (!block_ || !shortcuts_enabled()) return d;
    {
        std::lock_guard<std::mutex> lk(block_->mu);
        if (block_->derived.defined() && block_->derived_key == key) d = block_->derived;
    }
    if (d.defined()) {
        d.will_read();
        ++t_reused_copies;
    }
    return d;
}

int64_t reused_copies() { return t_reused_copies; }

void NdArray::set_derived(std::vector<int64_t> key, const NdArray &copy) const
{
    if (!block_ || block_->constant) return;
    NdArray old = copy;  // (the previous occupant is released outside the lock)
    std::lock_guard<std::mutex> lk(block_->mu);
    std::swap(block_->derived, old);
    block_->derived_key = std::move(key);
}

int64_t NdArray::version() const
{
    if (!block_) return 0;
    std::lock_guard<std::mutex> lk(block_->mu);
    return block_->version;
}

size_t NdArray::len() const { return product(shape_); }

float *NdArray::ptr() const { return block_ ? static_cast<float *>(block_->ptr) : nullptr; }

NdArray NdArray::extents_only(const Shape &shape)
{
    NdArray a;
    a.shape_ = shape;
    return a;
}

NdArray NdArray::empty(const Shape &shape)
{
    for (int64_t d : shape)
        if (d < 0) throw Panic("NdArray: negative extent");
    NdArray a;
    a.shape_ = shape;
    a.block_ = allocate(product(shape) * sizeof(float));
    return a;
}

NdArray NdArray::filled(const Shape &shape, float value)
{
    NdArray a = empty(shape);
    if (ag_fill_f32(current_stream(), a.ptr(), value, a.len()) != AG_OK) throw std::runtime_error(ag_last_error());
    return a;
}

NdArray NdArray::zeros(const Shape &shape) { return filled(shape, 0.f); }

NdArray NdArray::shared_zero()
{
    // written once and complete before anyone else sees it: threads read it without ordering their streams
    static const NdArray zero = [] {
        NdArray z = zeros({});
        synchronize();
        z.block_->constant = true;
        return z;
    }();
    return zero;
}

// ---------------------------------------------------------------------------------------------
// Host-to-device uploads go through a page-locked staging ring: the caller's array is copied into
// it on the host and the DMA is enqueued without waiting, so a feed costs a memcpy instead of a
// pageable-memory transfer plus a device synchronisation.  The caller's buffer is free for reuse
// when upload() returns.  Arrays larger than the ring take the synchronous path.
// ---------------------------------------------------------------------------------------------
namespace {
class StagingRing {
  public:
    static constexpr size_t kBytes = 16u << 20;
    ~StagingRing()
    {
        if (base_) {
            (void)hipStreamSynchronize(stream_);  // transfers out of the ring may still be in flight when a thread ends
            (void)hipHostFree(base_);
        }
        if (drained_) (void)hipEventDestroy(drained_);
    }
    // Device-to-host through the same ring; returns after the data has arrived in `dst`.
    void download(void *dst, const void *src, size_t bytes)
    {
        hipStream_t st = static_cast<hipStream_t>(current_stream());
        if (bytes > kBytes) {
            check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, st), "hipMemcpy D2H");
            synchronize();
            return;
        }
        std::lock_guard<std::mutex> lk(mu_);
        reserve();
        // the synchronisation below drains every earlier transfer, so the whole ring is free
        check(hipMemcpyAsync(base_, src, bytes, hipMemcpyDeviceToHost, st), "hipMemcpy D2H");
        synchronize();
        used_ = 0;
        pending_ = false;
        std::memcpy(dst, base_, bytes);
    }
    void upload(void *dst, const void *src, size_t bytes)
    {
        hipStream_t st = static_cast<hipStream_t>(current_stream());
        if (bytes > kBytes) {
            check(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, st), "hipMemcpy H2D");
            synchronize();
            return;
        }
        std::lock_guard<std::mutex> lk(mu_);
        reserve();
        const size_t need = (bytes + 255) / 256 * 256;
        if (used_ + need > kBytes) {
            // wrap: every transfer enqueued so far must have left the ring
            if (pending_) check(hipEventSynchronize(drained_), "hipEventSynchronize");
            used_ = 0;
            pending_ = false;
        }
        char *slot = static_cast<char *>(base_) + used_;
        std::memcpy(slot, src, bytes);
        check(hipMemcpyAsync(dst, slot, bytes, hipMemcpyHostToDevice, st), "hipMemcpy H2D");
        check(hipEventRecord(drained_, st), "hipEventRecord");
        used_ += need;
        pending_ = true;
    }

  private:
    void reserve()
    {
        if (base_) return;
        check(hipHostMalloc(&base_, kBytes, hipHostMallocDefault), "hipHostMalloc");
        check(hipEventCreateWithFlags(&drained_, hipEventDisableTiming), "hipEventCreate");
        stream_ = static_cast<hipStream_t>(current_stream());
    }
    std::mutex mu_;
    hipStream_t stream_ = nullptr;
    void *base_ = nullptr;
    hipEvent_t drained_ = nullptr;
    size_t used_ = 0;
    bool pending_ = false;
};
StagingRing &staging()
{
    // one ring per host thread, like the stream its transfers are ordered on: a slot is reused once the
    // transfers that THIS thread enqueued have left it
    thread_local StagingRing r;
    return r;
}
}  // namespace

NdArray NdArray::from_host(const Shape &shape, const float *data)
{
    NdArray a = empty(shape);
    if (a.len()) staging().upload(a.ptr(), data, a.len() * sizeof(float));
    return a;
}

void NdArray::copy_from_host(const float *data)
{
    will_write();
    if (len()) staging().upload(ptr(), data, len() * sizeof(float));
}

NdArray NdArray::reshaped(const Shape &shape) const
{
    if (product(shape) != len()) throw Panic("NdArray::reshaped: element count differs");
    NdArray a = *this;
    a.shape_ = shape;
    return a;
}

NdArray NdArray::deep_copy() const
{
    NdArray a = empty(shape_);
    will_read();
    if (len())
        check(hipMemcpyAsync(a.ptr(), ptr(), len() * sizeof(float), hipMemcpyDeviceToDevice,
                             static_cast<hipStream_t>(current_stream())),
              "hipMemcpy D2D");
    return a;
}

std::vector<float> NdArray::to_host() const
{
    if (!block_ && len()) throw Panic("NdArray::to_host: extents without elements");
    std::vector<float> out(len());
    will_read();
    if (len()) staging().download(out.data(), ptr(), len() * sizeof(float));
    else synchronize();
    return out;
}

// ---------------------------------------------------------------------------------------------
// ComputeContext / GradientContext                                        src/op.rs:186-434
// ---------------------------------------------------------------------------------------------
NdArray ComputeContext::input(size_t i)
{
    if (i >= xs_.size()) throw Panic("Bad op impl: input index out of range.");
    Input &x = xs_[i];
    if (x.kind == InputKind::RdWrVariable)
        throw Panic("Bad op impl: cannot perform mutable borrowing for input(" + std::to_string(i) +
                    "). Use input_mut() instead.");
    if (x.taken)
        throw Panic("Bad op impl: input(" + std::to_string(i) + ")/input_mut(" + std::to_string(i) +
                    ") cannot be called twice");
    x.taken = true;
    x.array.will_read();
    return x.array;
}

NdArray ComputeContext::input_mut(size_t i)
{
    if (i >= xs_.size()) throw Panic("Bad op impl: " + std::to_string(i) + "'s input doesn't exist.");
    Input &x = xs_[i];
    if (x.kind != InputKind::RdWrVariable)
        throw Panic("Bad op impl: cannot perform mutable borrowing for input(" + std::to_string(i) + ")");
    if (x.taken)
        throw Panic("Bad op impl: input(" + std::to_string(i) + ")/input_mut(" + std::to_string(i) +
                    ") cannot be called twice");
    x.taken = true;
    x.array.will_write();
    return x.array;
}

void ComputeContext::adam_update(AdamJob job)
{
    if (deferred_) {
        deferred_->add(std::move(job));
        return;
    }
    DeferredUpdates one;
    one.add(std::move(job));
    one.flush();
}

bool DeferredUpdates::writes(const NdArray &a) const
{
    const void *id = a.allocation();
    for (const AdamJob &j : jobs_)
        if (id == j.p.allocation() || id == j.m.allocation() || id == j.v.allocation() || id == j.t.allocation()) return true;
    return false;
}

bool DeferredUpdates::reads(const NdArray &a) const
{
    for (const AdamJob &j : jobs_)
        if (a.allocation() == j.g.allocation()) return true;
    return false;
}

void DeferredUpdates::add(AdamJob job)
{
    bool clash = false;
    for (const AdamJob &j : jobs_) {
        // another optimizer's coefficients, or a gradient that the batch is about to overwrite / a
        // parameter that the batch still reads as a gradient
        clash |= j.alpha != job.alpha || j.eps != job.eps || j.b1 != job.b1 || j.b2 != job.b2;
        clash |= job.p.allocation() == j.g.allocation() || job.m.allocation() == j.g.allocation() ||
                 job.v.allocation() == j.g.allocation() || job.t.allocation() == j.g.allocation();
    }
    clash |= writes(job.p) || writes(job.g) || writes(job.m) || writes(job.v) || writes(job.t);
    if (clash || (int)jobs_.size() == ag_adam_update_multi_max()) flush();
    jobs_.push_back(std::move(job));
}

void DeferredUpdates::flush()
{
    if (jobs_.empty()) return;
    std::vector<float *> p, m, v, t;
    std::vector<const float *> g;
    std::vector<size_t> n;
    for (const AdamJob &j : jobs_) {
        p.push_back(j.p.ptr());
        g.push_back(j.g.ptr());
        m.push_back(j.m.ptr());
        v.push_back(j.v.ptr());
        t.push_back(j.t.ptr());
        n.push_back(j.p.len());
    }
    const AdamJob &h = jobs_.front();
    const ag_status_t st = ag_adam_update_multi_f32(current_stream(), (int)jobs_.size(), p.data(), g.data(), m.data(),
                                                    v.data(), t.data(), n.data(), h.alpha, h.eps, h.b1, h.b2);
    jobs_.clear();
    if (st != AG_OK) throw std::runtime_error(ag_last_error());
}

void ComputeContext::append_output_view(const NdArray &y)
{
    bool contains_variable_input = false;
    for (const Input &x : xs_) contains_variable_input |= x.kind != InputKind::NonVariable;
    ys_.push_back(contains_variable_input ? y.deep_copy() : y);
}

Tensor GradientContext::input(size_t i) const
{
    const TensorInternal &n = graph_->node(y_.id);
    if (i >= n.incoming_nodes.size()) throw Panic("bad Op::grad impl");
    return graph_->tensor(n.incoming_nodes[i].id);
}

std::vector<Tensor> GradientContext::inputs() const
{
    std::vector<Tensor> r;
    for (const IncomingTensor &in : graph_->node(y_.id).incoming_nodes) r.push_back(graph_->tensor(in.id));
    return r;
}

size_t GradientContext::num_inputs() const { return graph_->node(y_.id).incoming_nodes.size(); }

// ---------------------------------------------------------------------------------------------
// graph building                                            src/tensor.rs:609-803, src/graph.rs
// ---------------------------------------------------------------------------------------------
TensorID Graph::install(std::unique_ptr<TensorInternal> n)
{
    const size_t count = nodes_.size();
    if (count == 50000)  // src/graph.rs:30-36
        std::fprintf(stderr, "Current graph size is 50,000! Graph should be reset regularly.\n");
    if (count > 500000) throw Panic("Maximum graph size exceeded: 500,000. Use Graph::clear and so on.");
    n->id = (TensorID)count;
    nodes_.push_back(std::move(n));
    return (TensorID)count;
}

TensorBuilder &TensorBuilder::append_input_with_selector(Tensor t, bool allow_mut, int selector)
{
    if (t.graph != graph_) throw Panic("Detected tensors belonging to different graphs");
    in_nodes_.push_back(IncomingTensor{t.id, allow_mut, selector});
    return *this;
}

TensorBuilder &TensorBuilder::append_backprop_input(Tensor t)
{
    if (t.graph != graph_) throw Panic("Detected tensors belonging to different graphs");
    if (!backprop_inputs_) backprop_inputs_.emplace();
    backprop_inputs_->push_back(IncomingTensor{t.id, false, 0});
    return *this;
}

Tensor TensorBuilder::build(std::unique_ptr<Op> op)
{
    int rank = 0;
    for (const IncomingTensor &in : in_nodes_) rank = std::max(rank, graph_->node(in.id).topo_rank + 1);
    // (a back-prop input that is not an input -- the sum behind a fused AddReLU -- must also rank below this node,
    // or the gradient builder's heap could reach it before this node has handed it its gradient)
    if (backprop_inputs_)
        for (const IncomingTensor &in : *backprop_inputs_) rank = std::max(rank, graph_->node(in.id).topo_rank + 1);
    auto n = std::make_unique<TensorInternal>();
    n->op = std::move(op);
    n->incoming_nodes = std::move(in_nodes_);
    n->topo_rank = rank;
    n->placeholder_name = std::move(placeholder_);
    n->is_placeholder = is_placeholder_;
    n->is_differentiable = differentiable_;
    n->backprop_inputs = std::move(backprop_inputs_);
    n->known_shape = std::move(known_shape_);
    n->variable_id = variable_id_;
    const TensorID id = graph_->install(std::move(n));
    return Tensor{graph_, id};
}

// ---------------------------------------------------------------------------------------------
// source ops                                               src/tensor_ops/basic_source_ops.rs
// ---------------------------------------------------------------------------------------------
namespace {
struct SourceOp : Op {
    const char *label;
    explicit SourceOp(const char *l) : label(l) {}
    const char *name() const override { return label; }
    OpError compute(ComputeContext &) const override
    {
        throw Panic(std::string(label) + ": source nodes are never computed");
    }
    void grad(GradientContext &) const override {}
};
}  // namespace

Tensor Context::variable(VariableID id)
{
    if (id < 0 || (size_t)id >= env_->size()) throw Panic("variable array not found");
    auto it = var_nodes_.find(id);
    if (it != var_nodes_.end()) return tensor(it->second);
    Tensor t = builder().set_variable(id).build(std::make_unique<SourceOp>("Variable"));
    var_nodes_[id] = t.id;
    return t;
}

Tensor Context::variable(const std::string &name, const std::string &namespace_id)
{
    auto id = env_->find(namespace_id, name);
    if (!id) throw Panic("variable array not found in namespace '" + namespace_id + "': " + name);
    return variable(*id);
}

Tensor Context::placeholder(const std::string &name, const Shape &shape)
{
    for (int64_t d : shape)
        if (d == 0 || d < -1) throw Panic("Given shape contains invalid dim size(s)");  // src/tensor.rs KnownShape::new
    return builder().set_placeholder_name(name).set_known_shape(shape).build(std::make_unique<SourceOp>("Placeholder"));
}

Evaluator Context::evaluator() { return Evaluator(this); }

// ---------------------------------------------------------------------------------------------
// evaluator                                                      src/evaluation.rs:183-363
// ---------------------------------------------------------------------------------------------
namespace {
struct StorageEntry {
    OpError error;
    std::vector<NdArray> outputs;
};

const NdArray *find_placeholder(const std::vector<std::pair<std::string, NdArray>> &feeds, const TensorInternal &n)
{
    // src/evaluation.rs:225-249: the feed must exist and match the placeholder's known shape
    for (const auto &f : feeds)
        if (f.first == n.placeholder_name) {
            if (n.known_shape) {
                const Shape &ks = *n.known_shape;
                bool ok = ks.size() == f.second.shape().size();
                for (size_t i = 0; ok && i < ks.size(); ++i) ok = ks[i] <= 0 || ks[i] == f.second.shape()[i];
                if (!ok) throw Panic("Shape error: placeholder '" + n.placeholder_name + "' was fed an array of another shape");
            }
            return &f.second;
        }
    throw Panic("Placeholder unfilled: " + n.placeholder_name);
}

// AG_HOST_TRACE=1 in the environment lists every evaluated node on stderr (op, inputs, output shapes)
bool trace_enabled()
{
    static const bool on = [] {
        const char *e = std::getenv("AG_HOST_TRACE");
        return e && std::string(e) == "1";
    }();
    return on;
}

void trace_node(const TensorInternal &n, const std::vector<NdArray> &outputs, const OpError &status)
{
    std::string line = "[ag_host] #" + std::to_string(n.id) + " " + n.op->name() + "(";
    for (size_t i = 0; i < n.incoming_nodes.size(); ++i)
        line += (i ? ", #" : "#") + std::to_string(n.incoming_nodes[i].id);
    line += ") ->";
    for (const NdArray &y : outputs) {
        line += " [";
        for (size_t i = 0; i < y.shape().size(); ++i) line += (i ? "," : "") + std::to_string(y.shape()[i]);
        line += "]";
    }
    if (!status.ok()) line += " error: " + status.message;
    std::fprintf(stderr, "%s\n", line.c_str());
}
}  // namespace

std::vector<EvalResult> Context::eval(const std::vector<Tensor> &tensors,
                                      const std::vector<std::pair<std::string, NdArray>> &feeds)
{
    std::unordered_map<TensorID, StorageEntry> storage;  // every output lives until eval returns
    DeferredUpdates deferred;                            // in-place optimizer updates, batched
    // A node that panics ends the evaluation; the updates queued by the nodes before it have already happened
    // as far as the reference is concerned (each AdamOp runs at its own node), so they are applied on the way out.
    struct FlushOnUnwind {
        DeferredUpdates &d;
        bool armed = true;
        ~FlushOnUnwind()
        {
            if (!armed) return;
            try {
                d.flush();
            } catch (...) {
            }
        }
    } flush_on_unwind{deferred};
    auto would_not_visit = [&](const TensorInternal &n) {
        return n.is_placeholder || n.is_variable() || storage.count(n.id) != 0;
    };
    std::vector<std::pair<TensorID, bool>> dfs;
    for (const Tensor &t : tensors) {
        if (t.graph != this) throw Panic("Detected tensors belonging to different graphs");
        dfs.emplace_back(t.id, false);
    }
    // Inputs of a node, from the feeds, the environment and what has been computed; the first error among them
    // is the node's own (src/evaluation.rs:283-309).
    auto gather = [&](const TensorInternal &n, std::vector<ComputeContext::Input> *inputs) {
        OpError status;
        for (const IncomingTensor &in : n.incoming_nodes) {
            const TensorInternal &src = node(in.id);
            if (src.is_placeholder) {
                inputs->push_back({*find_placeholder(feeds, src), ComputeContext::InputKind::NonVariable});
            } else if (src.is_variable()) {
                inputs->push_back({env_->array(src.variable_id), in.allow_mut ? ComputeContext::InputKind::RdWrVariable
                                                                              : ComputeContext::InputKind::RdOnlyVariable});
            } else {
                const StorageEntry &e = storage.at(in.id);
                if (!e.error.ok()) {
                    status = e.error;
                    break;
                }
                if ((size_t)in.array_selector >= e.outputs.size())
                    throw Panic("Bad op impl: output selector out of range");
                inputs->push_back({e.outputs[(size_t)in.array_selector], ComputeContext::InputKind::NonVariable});
            }
        }
        return status;
    };
    auto flush_if_touched = [&](const std::vector<ComputeContext::Input> &inputs) {
        if (deferred.empty()) return;
        for (const ComputeContext::Input &x : inputs)
            if (deferred.writes(x.array) || (x.kind == ComputeContext::InputKind::RdWrVariable && deferred.reads(x.array))) {
                deferred.flush();
                return;
            }
    };
    // Runs one node the ordinary way and files its result.
    auto run_node = [&](const TensorInternal &n) {
        std::vector<ComputeContext::Input> inputs;
        OpError status = gather(n, &inputs);
        StorageEntry entry;
        if (status.ok()) {
            flush_if_touched(inputs);
            ComputeContext cc(std::move(inputs), &deferred);
            status = n.op->compute(cc);
            if (status.ok()) {
                if (cc.outputs().empty()) throw Panic("Bad op implementation: empty return value");
                entry.outputs = std::move(cc.outputs());
            }
            if (trace_enabled()) trace_node(n, entry.outputs, status);
        }
        entry.error = status;
        storage.emplace(n.id, std::move(entry));
    };
    // The producer of a node's first input when the two can be evaluated in one pass (Op::fuses_with_producer).
    auto fusable_producer = [&](const TensorInternal &n) -> const TensorInternal * {
        if (!shortcuts_enabled()) return nullptr;
        if (n.incoming_nodes.empty() || n.incoming_nodes[0].array_selector != 0 || n.incoming_nodes[0].allow_mut) return nullptr;
        const TensorInternal &p = node(n.incoming_nodes[0].id);
        if (p.is_placeholder || p.is_variable() || !p.op || !n.op->fuses_with_producer(*p.op)) return nullptr;
        for (const IncomingTensor &in : p.incoming_nodes)
            if (in.allow_mut) return nullptr;
        return &p;
    };
    // Which of the nodes this evaluation will reach are such producers, and of which node: whoever asks for the
    // producer first is sent to that node instead, so the pair runs fused whatever the order of the walk.
    std::unordered_map<TensorID, TensorID> fused_into;
    {
        std::vector<TensorID> stack;
        std::unordered_map<TensorID, bool> seen;
        for (const Tensor &t : tensors) stack.push_back(t.id);
        while (!stack.empty()) {
            const TensorID id = stack.back();
            stack.pop_back();
            if (seen[id]) continue;
            seen[id] = true;
            const TensorInternal &n = node(id);
            if (n.is_placeholder || n.is_variable()) continue;
            if (const TensorInternal *p = fusable_producer(n)) fused_into.emplace(p->id, id);
            for (const IncomingTensor &in : n.incoming_nodes) stack.push_back(in.id);
        }
    }
    while (!dfs.empty()) {
        const auto [id, should_visit] = dfs.back();
        dfs.pop_back();
        const TensorInternal &n = node(id);
        if (!should_visit) {
            if (auto it = fused_into.find(id); it != fused_into.end() && !would_not_visit(n) && storage.count(it->second) == 0) {
                dfs.emplace_back(it->second, false);  // the node that computes this one along with itself
                continue;
            }
        }
        if (should_visit) {
            if (would_not_visit(n)) continue;
            if (const TensorInternal *p = fusable_producer(n); p && storage.count(p->id) == 0) {
                // the producer has not run: both nodes in one pass, from the producer's inputs (which the first visit
                // below has put in front of this node)
                std::vector<ComputeContext::Input> inputs;
                OpError status = gather(*p, &inputs);
                bool fused = false;
                if (status.ok()) {
                    flush_if_touched(inputs);
                    ComputeContext cc(std::move(inputs), &deferred);
                    StorageEntry pe, ne;
                    fused = n.op->compute_with_producer(cc, *p->op, &pe.outputs, &status);
                    if (fused) {
                        ++fused_pairs_;
                        if (status.ok()) {
                            if (cc.outputs().empty() || pe.outputs.empty()) throw Panic("Bad op implementation: empty return value");
                            ne.outputs = std::move(cc.outputs());
                        } else {
                            pe.outputs.clear();
                        }
                        if (trace_enabled()) {
                            trace_node(*p, pe.outputs, status);
                            trace_node(n, ne.outputs, status);
                        }
                        pe.error = ne.error = status;
                        storage.emplace(p->id, std::move(pe));
                        storage.emplace(id, std::move(ne));
                    }
                }
                if (fused) continue;
                run_node(*p);  // not this time (extents the fused form does not take, or an input in error)
            }
            run_node(n);
        } else {
            dfs.emplace_back(id, true);
            const TensorInternal *p = fusable_producer(n);
            for (size_t i = 0; i < n.incoming_nodes.size(); ++i) {
                const TensorInternal &src = node(n.incoming_nodes[i].id);
                if (would_not_visit(src)) continue;
                if (i == 0 && p) {
                    // evaluate what the producer reads, not the producer: it is computed together with this node
                    for (const IncomingTensor &in : p->incoming_nodes)
                        if (!would_not_visit(node(in.id))) dfs.emplace_back(in.id, false);
                } else {
                    dfs.emplace_back(n.incoming_nodes[i].id, false);
                }
            }
        }
    }
    flush_on_unwind.armed = false;
    deferred.flush();
    std::vector<EvalResult> ret;
    for (const Tensor &t : tensors) {
        const TensorInternal &n = node(t.id);
        EvalResult r;
        if (n.is_variable()) {
            r.array = env_->array(n.variable_id).deep_copy();
        } else if (n.is_placeholder) {
            r.array = find_placeholder(feeds, n)->deep_copy();
        } else {
            const StorageEntry &e = storage.at(t.id);
            r.error = e.error;
            if (e.error.ok()) r.array = e.outputs.at(0);
        }
        ret.push_back(std::move(r));
    }
    return ret;
}

// ---------------------------------------------------------------------------------------------
// variable environment                                                    src/variable.rs
// ---------------------------------------------------------------------------------------------
static std::string full_name(const std::string &ns, const std::string &name) { return ns + '\x01' + name; }

VariableID VariableEnvironment::set(const std::string &namespace_id, const std::string &name, NdArray array)
{
    // register_variable (src/variable.rs:347-358): a name that is already taken is bound to the new
    // array; the old array stays in the list under its id
    const VariableID id = (VariableID)arrays_.size();
    arrays_.push_back(std::move(array));
    name_to_id_[full_name(namespace_id, name)] = id;
    return id;
}

VariableID VariableEnvironment::set_anonymous(NdArray array)
{
    arrays_.push_back(std::move(array));
    return (VariableID)arrays_.size() - 1;
}

std::optional<VariableID> VariableEnvironment::find(const std::string &namespace_id, const std::string &name) const
{
    auto it = name_to_id_.find(full_name(namespace_id, name));
    if (it == name_to_id_.end()) return std::nullopt;
    return it->second;
}

NdArray &VariableEnvironment::array(VariableID id)
{
    if (id < 0 || (size_t)id >= arrays_.size()) throw Panic("variable array not found");
    return arrays_[(size_t)id];
}

std::vector<std::pair<std::string, VariableID>> VariableEnvironment::names_in(const std::string &namespace_id) const
{
    std::vector<std::pair<std::string, VariableID>> r;
    const std::string prefix = namespace_id + '\x01';
    for (const auto &kv : name_to_id_)
        if (kv.first.compare(0, prefix.size(), prefix) == 0) r.emplace_back(kv.first.substr(prefix.size()), kv.second);
    std::sort(r.begin(), r.end(), [](const auto &a, const auto &b) { return a.second < b.second; });
    return r;
}

void VariableEnvironment::run(const std::function<void(Context &)> &f)
{
    Context ctx(this);
    f(ctx);
}

}  // namespace host
}  // namespace ag
