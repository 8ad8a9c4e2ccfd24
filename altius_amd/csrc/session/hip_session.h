// The session: same construction and run interface as the reference's
// InterpreterSessionBuilder / InterpreterSession
// (crates/session_interpreter/src/builder.rs:12-66, session.rs:49-134), with the
// kernels running on an MI355X and tensors resident in device memory between nodes.
//
//   HipSessionBuilder(model).with_intra_op_num_threads(n).with_profiling_enabled(b).build()
//   session.run(inputs) -> outputs        inputs/outputs are host Tensors, positional
//   session.model()
//
// Failures come back as a SessionError value; nothing panics or aborts.
#pragma once

#include <map>
#include <set>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../core/model.h"
#include "../core/shape.h"
#include "../device/ctx.h"
#include "plan.h"

namespace altius {

// altius_session::SessionError (crates/session/src/lib.rs:14-35): Shape and Message
// keep their meaning; Hip stands for failures of the device runtime.
struct SessionError {
    enum Kind { Shape, Message, Hip, OutOfMemory, Argument } kind = Message;
    std::string message;
    int code() const;  // the AHIP_ERR_* code of this kind
    std::string to_string() const;
};

// Device memory reused between nodes and runs: freed blocks are kept in
// size-bucketed lists and handed out again, so a steady-state run allocates nothing.
class BufferPool {
public:
    explicit BufferPool(DeviceCtx *ctx) : ctx_(ctx) {}
    ~BufferPool();
    int acquire(size_t bytes, void **ptr, size_t *bucket);
    void release(void *ptr, size_t bucket);
    // Takes one particular cached block out of the free list (true if it was there): the caller owns it now.
    bool take(void *ptr, size_t bucket);
    void trim();  // returns every cached block to the device (a no-op while trimming is held off)
    // Recorded HIP graphs address cached blocks directly: while one exists nothing may be freed.
    void hold_memory(bool hold) { hold_ = hold; }
    size_t bytes_reserved() const { return reserved_; }
    size_t device_allocations() const { return allocations_; }

private:
    static size_t bucket_of(size_t bytes);
    DeviceCtx *ctx_;
    std::map<size_t, std::vector<void *>> free_;
    size_t reserved_ = 0;
    size_t allocations_ = 0;
    bool hold_ = false;
};

// A block of pooled device memory; goes back to its pool when the last tensor using it is dropped.
struct DeviceBlock {
    BufferPool *pool = nullptr;
    void *ptr = nullptr;
    size_t bucket = 0;
    DeviceBlock() = default;
    DeviceBlock(const DeviceBlock &) = delete;
    DeviceBlock &operator=(const DeviceBlock &) = delete;
    ~DeviceBlock() {
        if (pool && ptr) pool->release(ptr, bucket);
    }
};

// DeviceTensor::pending_op of the placeholder a deferred attention product leaves behind (no memory).
constexpr int PENDING_ATTENTION = 1000;

struct DeviceTensor;
// An Add of two tensors of one shape that has not run yet: the tensor's block is reserved for the sum, the operands
// are kept alive, and either the LayerNormalization behind it computes the sum on its way (writing it here as well),
// or the first other reader makes it run.  Shared by every alias of the tensor.
struct PendingAdd {
    std::shared_ptr<DeviceBlock> a_block, b_block;
    const float *a = nullptr, *b = nullptr;
    size_t elems = 0;
    bool done = false;
};

struct DeviceTensor {
    FixedDimensions dims;
    TensorElemType elem_ty = TensorElemType::F32;
    void *ptr = nullptr;
    // Keeps the memory alive.  Reshape / Flatten / Squeeze / Unsqueeze / Identity outputs share
    // their input's block (the reference shares the buffer the same way, tensor.rs:340-342).
    std::shared_ptr<DeviceBlock> block;
    // The contents on the host, when they are known there: initializers and the small integer
    // tensors of shape arithmetic.  Shape inference and the host evaluator read these.
    std::shared_ptr<const Tensor> host;
    // Element strides when the tensor is a strided view of its block (a lazily taken Split part or
    // Transpose); empty for the usual dense row-major layout.  Only operators that read views in
    // place ever see one: every other reader gets a dense copy first.
    std::vector<int64_t> strides;
    // An activation (AHIP_GELU / AHIP_RELU) that has not been applied yet: the tensor holds the
    // activation's input, and its one reader, a MatMul, applies it while splitting the operand.
    int pending_op = -1;
    // An activation (AHIP_GELU / AHIP_RELU) that the MatMul which produced the tensor has already applied while
    // writing it: the activation node that follows passes the tensor on.
    int applied_op = -1;
    // The block does not hold fp32 values but the tensor's three bf16 planes, laid out as the first operand of the
    // tall bf16 product that is its only reader; the LayerNormalization that produced the tensor wrote them instead
    // of the fp32 result.
    bool planes = false;
    size_t planes_rows = 0, planes_k = 0;  // the [rows, k] operand the planes were written for
    // Set while the tensor's values are still owed by an Add that was deferred (see PendingAdd).
    std::shared_ptr<PendingAdd> pending_add;
    bool owes_add() const { return pending_add && !pending_add->done; }
    size_t nbytes() const { return dims.total_elems() * elem_size(elem_ty); }
};

class HipSession {
public:
    ~HipSession();
    HipSession(const HipSession &) = delete;
    HipSession &operator=(const HipSession &) = delete;

    const Model &model() const { return model_; }

    // Binds inputs[i] to graph.inputs[i], runs every node of the plan on the
    // device, and returns graph.outputs in order.  Calls are serialised.
    bool run(const std::vector<Tensor> &inputs, std::vector<Tensor> *outputs, SessionError *err);

    // Not in the reference: the same run on tensors that already live on the session's GPU.
    // inputs[i] describes caller-owned device memory (ptr, dims, element type; no block), read in
    // stream order: it must hold its data before the call and stay valid until synchronize().
    // Outputs are device tensors whose memory belongs to the session's pool (or, for an output
    // that is a reshaped view of an input, the caller's own pointer); they hold results once
    // synchronize() has returned.  Nothing crosses PCIe and the call does not wait for the GPU.
    bool run_device(const std::vector<DeviceTensor> &inputs, std::vector<DeviceTensor> *outputs, SessionError *err);
    // Waits for the session's stream and reports errors that kernels leave in device flags.
    bool synchronize(SessionError *err);
    // Drops a tensor run_device() returned; its block goes back to the pool for later nodes.
    void release(DeviceTensor *t);

    // Per-operator device time of the last run, in milliseconds (filled when
    // profiling is enabled), keyed by Op::name().
    const std::map<std::string, double> &last_profile() const { return profile_; }
    double last_run_ms() const { return last_run_ms_; }
    // Device time of the last run's kernels alone (between the uploads and the downloads), from two
    // events on the session's stream.
    double last_device_ms() const { return last_device_ms_; }
    size_t device_allocations() const { return pool_->device_allocations(); }
    // Nodes of the last node-by-node run that produced a view or wrote a following Transpose's layout.
    size_t copies_avoided() const { return copies_avoided_; }
    // Runs served by replaying a captured HIP graph since the session was built.
    size_t graph_replays() const { return graph_replays_; }
    const std::vector<NodeExecutionPlan> &execution_plan() const { return plan_; }
    const InferredShapes &inferred_shapes() const { return inferred_; }

private:
    friend class HipSessionBuilder;
    HipSession() = default;

    bool run_node(NodeId id, std::map<ValueId, DeviceTensor> &values, SessionError *err);
    // A fresh pooled tensor of the given shape (contents unspecified).
    bool allocate(const TypedFixedShape &shape, DeviceTensor *out, SessionError *err);
    // A pooled block of the given size behind a tensor whose shape the caller sets (operand planes).
    bool allocate_bytes(size_t nbytes, DeviceTensor *out, SessionError *err);
    bool defers_add(NodeId id, const std::vector<DeviceTensor *> &in, const std::vector<TypedFixedShape> &shapes) const;
    // Uploads a host tensor into a fresh pooled tensor that remembers its host contents.
    bool upload(const Tensor &t, DeviceTensor *out, SessionError *err);
    // Makes t.host available by reading a small tensor back (synchronises the stream).
    bool fetch_host(DeviceTensor *t, SessionError *err);
    bool run_fused_elemwise(const Node &node, const Op &op, const std::vector<DeviceTensor *> &in,
                            const std::vector<TypedFixedShape> &shapes, std::vector<DeviceTensor> *outs, SessionError *err);
    bool run_device_op(const Node &node, const Op &op, const std::vector<DeviceTensor *> &in,
                       const std::vector<TypedFixedShape> &shapes, std::vector<DeviceTensor> *outs, SessionError *err);

    // A run recorded as a HIP graph for one set of input shapes: replaying it issues every kernel
    // of the plan with one launch.  The graph refers to pool blocks by address, which stays valid
    // because the pool never returns memory to the device while a graph exists.
    struct CapturedRun {
        hipGraphExec_t exec = nullptr;
        std::vector<DeviceTensor> inputs;   // persistent device copies of the graph inputs
        std::vector<DeviceTensor> outputs;  // where the recorded kernels leave the graph outputs
        // Every other block the recorded kernels read or write (the run's intermediates): kept out of the pool
        // while the graph exists, so that no later run -- a device-resident one whose outputs the caller holds
        // included -- is handed memory that a replay overwrites.
        std::vector<std::shared_ptr<DeviceBlock>> blocks;
        bool has_gather = false;
        bool unusable = false;              // capture was tried and refused; run eagerly from now on
    };
    bool check_input(size_t i, TensorElemType elem_ty, const FixedDimensions &dims, SessionError *err) const;
    bool try_capture(const std::string &key, const std::vector<Tensor> &inputs, SessionError *err);
    bool replay(CapturedRun &run, const std::vector<Tensor> &inputs, std::vector<Tensor> *outputs, SessionError *err);
    void drop_graphs();
    // Decides at build time which Split / Transpose nodes hand out views and which MatMul nodes
    // write their result in the layout a following Transpose would produce.
    void plan_views(bool fused_attention);
    // Replaces a view by a dense copy of itself.
    bool materialize(DeviceTensor *t, SessionError *err);
    // How a MatMul reads an operand that may be a strided view: its last two axes as a matrix with one unit
    // stride (a unit row stride means the stored matrix is the transposed one), the leading axes as batches.
    struct MatOperand {
        size_t rows = 0, cols = 0, ld = 0, batch = 1;
        bool stored_transposed = false;
        std::vector<size_t> bdims;
        std::vector<int64_t> bstr;
    };
    // Fills *o; a view the GEMM's addressing cannot express is replaced by a dense copy first.
    bool describe_operand(DeviceTensor *t, MatOperand *o, SessionError *err);
    // MatMul -> Softmax -> MatMul as one kernel (plan_views finds the triples): the first MatMul leaves a
    // placeholder and its operands here, the Softmax passes the placeholder on, the second MatMul launches.
    struct PendingAttention {
        DeviceTensor q, k;
        MatOperand Q, K;
        std::vector<size_t> bd;  // batch axes (extent-1 axes dropped), at most two
        FixedDimensions score_dims;
        DeviceTensor mask;       // the Softmax's absorbed mask (one value per key), if any
        size_t mask_outer_stride = 0;
    };
    struct AttentionPlan {
        NodeId softmax, tail;
        int scale_op = 0;
        float scale = 1.0f;
        bool has_mask = false;
    };
    // Undoes a deferral: runs the first product of a pending attention into real scores.
    bool flush_attention(ValueId scores, DeviceTensor *placeholder, SessionError *err);
    bool try_defer_attention(const Node &node, const Op &op, const std::vector<DeviceTensor *> &in,
                             const std::vector<TypedFixedShape> &shapes, std::vector<DeviceTensor> *outs, SessionError *err);
    bool run_attention_tail(const Op &op, const std::vector<DeviceTensor *> &in, DeviceTensor *out, SessionError *err);
    // Runs the activation a tensor still owes (pending_op) into a new buffer.
    bool apply_pending(DeviceTensor *t, SessionError *err);

    Model model_;
    std::vector<NodeExecutionPlan> plan_;
    InferredShapes inferred_;
    bool enable_profiling_ = false;
    size_t intra_op_num_threads_ = 1;
    DeviceCtx ctx_;
    std::unique_ptr<BufferPool> pool_;
    std::map<ValueId, DeviceTensor> inits_;  // uploaded once at build
    std::map<std::string, double> profile_;
    double last_run_ms_ = 0;
    double last_device_ms_ = 0;
    bool span_pending_ = false;  // run_device() recorded the span; synchronize() reads it
    bool device_timing_ = true;  // record the span at all
    hipEvent_t span_begin_ = nullptr, span_end_ = nullptr;  // bracket the kernels of a run
    std::mutex mutex_;
    bool graph_replay_ = false;
    bool capturing_ = false;        // a stream capture is in progress: nothing may synchronise
    std::vector<std::pair<void *, size_t>> capture_allocs_;  // (block, bucket) of every allocation made while recording
    bool capture_refused_ = false;  // a node needed the host during capture
    std::map<std::string, CapturedRun> graphs_;
    std::map<std::string, int> eager_runs_;  // per input signature: eager runs so far (the pool is warm after one)
    size_t graph_replays_ = 0;
    uint64_t seen_ws_generation_ = 0;  // recorded launches hold the GEMM workspace's address: graphs are dropped when it moves
    size_t copies_avoided_ = 0;
    NodeId current_node_ = 0;  // the node run_device_op is working on
    std::map<NodeId, AttentionPlan> attn_head_;                  // first MatMul of a fusable attention -> the rest
    std::set<NodeId> attn_softmax_, attn_tail_;
    std::map<ValueId, PendingAttention> pending_attn_;
    // What follows a MatMul whose result has one reader and can be done while the product is written (fp32 kernel):
    // a Gelu / Relu node, or an Add of a tensor of the result's shape (a residual connection).
    struct MatMulPost {
        int act = 0;            // AHIP_GELU / AHIP_RELU, 0: none
        bool has_add = false;
        NodeId add_node = 0;
        size_t add_input = 0;   // which input of the Add is the product
        ValueId residual = 0;   // the Add's other input
    };
    std::map<NodeId, MatMulPost> matmul_post_;
    std::map<NodeId, size_t> absorbed_add_;                     // Add nodes whose sum a MatMul wrote in this run -> input holding it
    const std::map<ValueId, DeviceTensor> *values_ = nullptr;   // the running call's values, for run_device_op
    std::set<NodeId> deferred_unary_;                           // Gelu / Relu nodes folded into the MatMul that reads them
    // LayerNormalization -> MatMul(weights) with a single reader: where the product takes the bf16 route the
    // normalisation writes the operand planes the product reads instead of fp32 values (next_n: columns of the weights).
    struct PlanesPlan {
        NodeId consumer = 0;
        size_t next_n = 0;
    };
    std::map<NodeId, PlanesPlan> planes_out_;
    std::set<NodeId> planes_consumer_;
    // The second product of an attention -> Transpose (written in place) -> Reshape -> MatMul(weights): the attention kernel
    // writes that last product's operand planes; the two nodes between pass them on.
    std::map<NodeId, PlanesPlan> attn_planes_;
    std::set<NodeId> planes_pass_;
    std::map<NodeId, NodeId> add_into_ln_;  // Add nodes (a residual connection) -> the planes-writing LayerNormalization that reads the sum
    // Runs a deferred Add into the tensor's block.
    bool flush_add(DeviceTensor *t, SessionError *err);
    std::set<NodeId> lazy_views_;                               // Split / Transpose nodes whose outputs are views
    std::map<NodeId, std::vector<int64_t>> matmul_out_perm_;    // MatMul nodes -> perm of the Transpose they feed
};

class HipSessionBuilder {
public:
    explicit HipSessionBuilder(Model model) : model_(std::move(model)) {}
    // Accepted for interface parity; the device kernels do not use host threads.
    HipSessionBuilder &with_intra_op_num_threads(size_t n) {
        intra_op_num_threads_ = n;
        return *this;
    }
    HipSessionBuilder &with_profiling_enabled(bool enable) {
        enable_profiling_ = enable;
        return *this;
    }
    // Not in the reference: record each distinct input-shape signature as a HIP graph on its second
    // run and replay it afterwards (one launch per run instead of one per node).  Off by default.
    // Graphs whose shapes or operands need the host during the run, and profiled sessions, keep
    // running node by node.
    HipSessionBuilder &with_graph_replay(bool enable) {
        graph_replay_ = enable;
        return *this;
    }
    // Not in the reference: the kernel large single-batch MatMul / Gemm products take (AHIP_GEMM_FP32, the
    // default and the reference's semantics for infinite operands, AHIP_GEMM_AUTO or AHIP_GEMM_BF16X3).
    // Float initializers are declared constant to the GEMM, so a weight operand's bf16 planes are made on
    // its first use and kept.
    HipSessionBuilder &with_gemm_algorithm(int algorithm) {
        gemm_algorithm_ = algorithm;
        return *this;
    }
    // Not in the reference: Split and Transpose nodes whose results only MatMuls read (possibly through
    // reshapes) hand out strided views instead of copies, and a MatMul read only by a Transpose writes
    // that Transpose's layout directly (default on; off makes every node copy, as the reference does).
    HipSessionBuilder &with_strided_views(bool enable) {
        strided_views_ = enable;
        return *this;
    }
    // Not in the reference: MatMul -> Softmax -> MatMul as one attention kernel (default off: its sums run in
    // another order than the three operators', 2e-4 relative).  Needs strided views.
    HipSessionBuilder &with_fused_attention(bool enable) {
        fused_attention_ = enable;
        return *this;
    }
    // Not in the reference: whether a run is bracketed by two events on the session's stream, which is what
    // last_device_ms() reports (default on).  Off saves two event records per run, on the host and in the queue: a
    // caller that runs small graphs back to back and does not ask for the device time turns it off.
    HipSessionBuilder &with_device_timing(bool enable) {
        device_timing_ = enable;
        return *this;
    }
    // Not in the reference: which GPU to run on (default 0).
    HipSessionBuilder &with_device(int device) {
        device_ = device;
        return *this;
    }
    // Infers shapes, builds the execution plan, creates the device context and
    // uploads the initializers.  Returns nullptr and fills *err on failure.
    std::unique_ptr<HipSession> build(SessionError *err);

private:
    Model model_;
    size_t intra_op_num_threads_ = 1;
    bool enable_profiling_ = false;
    int device_ = 0;
    bool graph_replay_ = false;
    int gemm_algorithm_ = AHIP_GEMM_FP32;
    bool strided_views_ = true;
    bool fused_attention_ = false;
    bool device_timing_ = true;
};

}  // namespace altius
