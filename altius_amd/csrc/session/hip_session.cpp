#include "hip_session.h"

#include <algorithm>
#include <chrono>

#include "../device/host_pool.h"

namespace altius {

int SessionError::code() const {
    switch (kind) {
    case Shape: return AHIP_ERR_SHAPE;
    case Message: return AHIP_ERR_UNSUPPORTED;
    case Hip: return AHIP_ERR_HIP;
    case OutOfMemory: return AHIP_ERR_OOM;
    case Argument: return AHIP_ERR_ARG;
    }
    return AHIP_ERR_ARG;
}

std::string SessionError::to_string() const {
    switch (kind) {
    case Shape: return "Shape: " + message;
    case Message: return "Something went wrong: " + message;
    case Hip: return "Hip: " + message;
    case OutOfMemory: return "OutOfMemory: " + message;
    case Argument: return "Argument: " + message;
    }
    return message;
}

namespace {

bool fail(SessionError *err, SessionError::Kind kind, std::string msg) {
    if (err) {
        err->kind = kind;
        err->message = std::move(msg);
    }
    return false;
}

// Turns an AHIP_ERR_* code from the device layer into a SessionError.
bool fail_code(SessionError *err, int code, const std::string &msg) {
    SessionError::Kind k = SessionError::Hip;
    if (code == AHIP_ERR_OOM) k = SessionError::OutOfMemory;
    else if (code == AHIP_ERR_UNSUPPORTED) k = SessionError::Message;
    else if (code == AHIP_ERR_SHAPE) k = SessionError::Shape;
    else if (code == AHIP_ERR_ARG) k = SessionError::Argument;
    return fail(err, k, msg);
}

}  // namespace

// ---- BufferPool ------------------------------------------------------------------

size_t BufferPool::bucket_of(size_t bytes) {
    if (bytes == 0) bytes = 1;
    const size_t small = 256, large = (size_t)1 << 20;
    const size_t unit = bytes <= large ? small : large;
    return (bytes + unit - 1) / unit * unit;
}

BufferPool::~BufferPool() { trim(); }

int BufferPool::acquire(size_t bytes, void **ptr, size_t *bucket) {
    const size_t b = bucket_of(bytes);
    auto it = free_.find(b);
    if (it != free_.end() && !it->second.empty()) {
        *ptr = it->second.back();
        it->second.pop_back();
        *bucket = b;
        return AHIP_OK;
    }
    hipError_t e = hipMalloc(ptr, b);
    if (e == hipErrorOutOfMemory) {  // give cached blocks back and retry once
        (void)hipGetLastError();
        (void)hipStreamSynchronize(ctx_->stream);
        trim();
        e = hipMalloc(ptr, b);
    }
    int rc = ctx_->check(e, "hipMalloc");
    if (rc) return rc;
    reserved_ += b;
    allocations_++;
    *bucket = b;
    return AHIP_OK;
}

void BufferPool::release(void *ptr, size_t bucket) {
    if (ptr) free_[bucket].push_back(ptr);
}

void BufferPool::trim() {
    for (auto &kv : free_) {
        for (void *p : kv.second) {
            (void)hipFree(p);
            reserved_ -= kv.first;
        }
        kv.second.clear();
    }
}

// ---- HipSessionBuilder ----------------------------------------------------------------

std::unique_ptr<HipSession> HipSessionBuilder::build(SessionError *err) {
    std::unique_ptr<HipSession> s(new HipSession());
    s->model_ = std::move(model_);
    s->enable_profiling_ = enable_profiling_;
    s->intra_op_num_threads_ = intra_op_num_threads_;

    ShapeError serr;
    if (!infer_shapes(s->model_, &s->inferred_, nullptr, &serr)) {
        fail(err, SessionError::Shape, serr.message);
        return nullptr;
    }
    s->plan_ = create_execution_plan(s->model_);

    std::string derr;
    int rc = create_device_ctx(device_, nullptr, true, &s->ctx_, &derr);
    if (rc) {
        fail_code(err, rc, derr);
        return nullptr;
    }
    s->pool_.reset(new BufferPool(&s->ctx_));

    // Initializers live on the device for the lifetime of the session.
    for (const auto &kv : s->model_.graph.inits) {
        const Tensor &t = kv.second;
        DeviceTensor d;
        d.dims = t.dims();
        d.elem_ty = t.elem_ty();
        const size_t bytes = d.nbytes();
        if (t.nbytes() != bytes) {
            fail(err, SessionError::Argument, "initializer data does not match its shape");
            return nullptr;
        }
        rc = s->pool_->acquire(bytes, &d.ptr, &d.bucket);
        if (rc) {
            fail_code(err, rc, s->ctx_.last_error);
            return nullptr;
        }
        if (bytes) {
            rc = s->ctx_.check(hipMemcpyAsync(d.ptr, t.data_as_bytes(), bytes, hipMemcpyHostToDevice, s->ctx_.stream),
                               "hipMemcpyAsync(initializer)");
            if (rc) {
                fail_code(err, rc, s->ctx_.last_error);
                return nullptr;
            }
        }
        s->inits_[kv.first] = d;
    }
    rc = s->ctx_.check(hipStreamSynchronize(s->ctx_.stream), "hipStreamSynchronize(build)");
    if (rc) {
        fail_code(err, rc, s->ctx_.last_error);
        return nullptr;
    }
    return s;
}

// ---- HipSession -------------------------------------------------------------------------

HipSession::~HipSession() {
    if (pool_) {
        (void)hipSetDevice(ctx_.device);
        (void)hipStreamSynchronize(ctx_.stream);
        for (auto &kv : inits_) pool_->release(kv.second.ptr, kv.second.bucket);
        inits_.clear();
        pool_.reset();
        destroy_device_ctx(&ctx_);
    }
}

void HipSession::release(DeviceTensor &t) {
    if (t.pooled && t.ptr) pool_->release(t.ptr, t.bucket);
    t.ptr = nullptr;
    t.pooled = false;
}

bool HipSession::run(const std::vector<Tensor> &inputs, std::vector<Tensor> *outputs, SessionError *err) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (!outputs) return fail(err, SessionError::Argument, "run: null output vector");
    outputs->clear();
    profile_.clear();
    const Graph &g = model_.graph;
    if (inputs.size() < g.inputs.size())
        return fail(err, SessionError::Argument,
                    "run: " + std::to_string(inputs.size()) + " inputs given, the graph has " +
                        std::to_string(g.inputs.size()));
    if (hipSetDevice(ctx_.device) != hipSuccess) return fail(err, SessionError::Hip, "hipSetDevice failed");

    const auto t0 = std::chrono::steady_clock::now();
    std::map<ValueId, DeviceTensor> values;
    auto cleanup = [&]() {
        (void)hipStreamSynchronize(ctx_.stream);  // nothing still reads a block that goes back to the pool
        for (auto &kv : values) release(kv.second);
    };

    // Upload the inputs (positional, session.rs:81-83).
    for (size_t i = 0; i < g.inputs.size(); i++) {
        const Tensor &t = inputs[i];
        if (!t.has_data()) {
            cleanup();
            return fail(err, SessionError::Argument, "run: input " + std::to_string(i) + " has no data");
        }
        DeviceTensor d;
        d.dims = t.dims();
        d.elem_ty = t.elem_ty();
        int rc = pool_->acquire(d.nbytes(), &d.ptr, &d.bucket);
        if (rc) {
            cleanup();
            return fail_code(err, rc, ctx_.last_error);
        }
        d.pooled = true;
        values[g.inputs[i]] = d;
        if (d.nbytes()) {
            rc = ctx_.check(hipMemcpyAsync(d.ptr, t.data_as_bytes(), d.nbytes(), hipMemcpyHostToDevice, ctx_.stream),
                            "hipMemcpyAsync(input)");
            if (rc) {
                cleanup();
                return fail_code(err, rc, ctx_.last_error);
            }
        }
    }

    // One event per node boundary when profiling.
    std::vector<hipEvent_t> events;
    if (enable_profiling_) {
        events.resize(plan_.size() + 1);
        for (auto &e : events) {
            if (hipEventCreate(&e) != hipSuccess) {
                cleanup();
                return fail(err, SessionError::Hip, "hipEventCreate failed");
            }
        }
        (void)hipEventRecord(events[0], ctx_.stream);
    }
    auto destroy_events = [&]() {
        for (auto e : events) (void)hipEventDestroy(e);
    };

    // The hot loop (session.rs:86-92).
    for (size_t i = 0; i < plan_.size(); i++) {
        if (!run_node(plan_[i].node_id, values, err)) {
            cleanup();
            destroy_events();
            return false;
        }
        if (enable_profiling_) (void)hipEventRecord(events[i + 1], ctx_.stream);
        for (ValueId v : plan_[i].free_vals) {
            auto it = values.find(v);
            if (it != values.end()) {
                release(it->second);  // stream order makes immediate reuse safe
                values.erase(it);
            }
        }
    }

    // Download the outputs (session.rs:127-133).
    for (ValueId v : g.outputs) {
        const DeviceTensor *d = nullptr;
        auto it = values.find(v);
        if (it != values.end()) d = &it->second;
        else {
            auto ii = inits_.find(v);
            if (ii != inits_.end()) d = &ii->second;
        }
        if (!d) {
            cleanup();
            destroy_events();
            return fail(err, SessionError::Message, "run: graph output was not produced");
        }
        Tensor t = Tensor::uninit_of_type(d->elem_ty, d->dims, pinned_host_block);
        if (!t.has_data()) {
            cleanup();
            destroy_events();
            return fail(err, SessionError::OutOfMemory, "run: out of host memory for an output tensor");
        }
        if (d->nbytes()) {
            int rc = ctx_.check(hipMemcpyAsync(t.data_as_bytes_mut(), d->ptr, d->nbytes(), hipMemcpyDeviceToHost,
                                               ctx_.stream),
                                "hipMemcpyAsync(output)");
            if (rc) {
                cleanup();
                destroy_events();
                return fail_code(err, rc, ctx_.last_error);
            }
        }
        outputs->push_back(std::move(t));
    }
    int rc = ctx_.check(hipStreamSynchronize(ctx_.stream), "hipStreamSynchronize(run)");
    if (rc) {
        cleanup();
        destroy_events();
        return fail_code(err, rc, ctx_.last_error);
    }
    if (enable_profiling_) {
        for (size_t i = 0; i < plan_.size(); i++) {
            float ms = 0;
            if (hipEventElapsedTime(&ms, events[i], events[i + 1]) == hipSuccess)
                profile_[model_.graph.nodes[plan_[i].node_id].op.name()] += ms;
        }
        destroy_events();
    }
    for (auto &kv : values) release(kv.second);
    last_run_ms_ = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    return true;
}

bool HipSession::run_node(NodeId id, std::map<ValueId, DeviceTensor> &values, SessionError *err) {
    const Node &node = model_.graph.nodes[id];
    const std::string opname = node.op.name();

    // Inputs: run-time values first, then initializers.
    std::vector<const DeviceTensor *> in;
    for (ValueId v : node.inputs) {
        auto it = values.find(v);
        if (it != values.end()) {
            in.push_back(&it->second);
            continue;
        }
        auto ii = inits_.find(v);
        if (ii == inits_.end()) return fail(err, SessionError::Message, opname + ": an input value is missing");
        in.push_back(&ii->second);
    }

    // Output shapes: inferred at build time if possible, else now (session.rs:149-158).
    Op op = node.op;
    std::vector<TypedFixedShape> shapes;
    auto cached = inferred_.find(id);
    if (cached != inferred_.end()) {
        op = cached->second.first;
        shapes = cached->second.second;
    } else {
        std::vector<Tensor> meta;
        meta.reserve(in.size());
        for (auto *d : in) meta.push_back(Tensor::empty_of_type(d->elem_ty, d->dims));
        std::vector<const Tensor *> ptrs;
        for (auto &m : meta) ptrs.push_back(&m);
        ShapeError serr;
        if (!compute_output_shapes(model_, op, ptrs, node.outputs.size(), &shapes, &serr))
            return fail(err, SessionError::Shape, serr.message);
    }
    if (shapes.size() < node.outputs.size() || node.outputs.empty())
        return fail(err, SessionError::Message, opname + ": output count mismatch");

    // Every kernel here computes in fp32.
    for (auto *d : in)
        if (d->elem_ty != TensorElemType::F32)
            return fail(err, SessionError::Message,
                        opname + ": input type " + elem_name(d->elem_ty) + " is not supported (f32 only)");

    // Allocate the output, pre-sized, contents unspecified (session.rs:159-162).
    DeviceTensor out;
    out.dims = shapes[0].dims;
    out.elem_ty = shapes[0].elem_ty;
    int rc = pool_->acquire(out.nbytes(), &out.ptr, &out.bucket);
    if (rc) return fail_code(err, rc, ctx_.last_error);
    out.pooled = true;
    float *o = static_cast<float *>(out.ptr);
    auto f = [](const DeviceTensor *d) { return static_cast<const float *>(d->ptr); };
    auto bail = [&](SessionError::Kind k, const std::string &msg) {
        release(out);
        return fail(err, k, msg);
    };

    switch (op.kind) {
    case OpKind::Identity:
        if (out.nbytes())
            rc = ctx_.check(hipMemcpyAsync(out.ptr, in[0]->ptr, out.nbytes(), hipMemcpyDeviceToDevice, ctx_.stream),
                            "hipMemcpyAsync(Identity)");
        break;
    case OpKind::Add:
    case OpKind::Sub:
    case OpKind::Mul:
    case OpKind::Div:
    case OpKind::Pow: {
        auto as = in[0]->dims.strides_for_broadcasting_to(out.dims);
        auto bs = in[1]->dims.strides_for_broadcasting_to(out.dims);
        if (!as || !bs) return bail(SessionError::Shape, opname + ": operands do not broadcast to the output shape");
        const size_t rank = out.dims.len();
        if (rank > (size_t)MAX_RANK) return bail(SessionError::Message, opname + ": rank above 8 is not supported");
        int64_t dims[MAX_RANK], sa[MAX_RANK], sb[MAX_RANK];
        for (size_t i = 0; i < rank; i++) {
            dims[i] = (int64_t)out.dims[i];
            sa[i] = (int64_t)(*as)[i];
            sb[i] = (int64_t)(*bs)[i];
        }
        const int bop = op.kind == OpKind::Add   ? AHIP_ADD
                        : op.kind == OpKind::Sub ? AHIP_SUB
                        : op.kind == OpKind::Mul ? AHIP_MUL
                        : op.kind == OpKind::Div ? AHIP_DIV
                                                 : AHIP_POW;
        rc = launch_binary(ctx_, bop, o, f(in[0]), f(in[1]), (int)rank, dims, sa, sb);
        break;
    }
    case OpKind::Sqrt: rc = launch_unary(ctx_, AHIP_SQRT, o, f(in[0]), out.dims.total_elems(), 0, 0); break;
    case OpKind::ReLU: rc = launch_unary(ctx_, AHIP_RELU, o, f(in[0]), out.dims.total_elems(), 0, 0); break;
    case OpKind::Gelu: rc = launch_unary(ctx_, AHIP_GELU, o, f(in[0]), out.dims.total_elems(), 0, 0); break;
    case OpKind::Sigmoid: rc = launch_unary(ctx_, AHIP_SIGMOID, o, f(in[0]), out.dims.total_elems(), 0, 0); break;
    case OpKind::Erf: rc = launch_unary(ctx_, AHIP_ERF, o, f(in[0]), out.dims.total_elems(), 0, 0); break;
    case OpKind::Tanh: rc = launch_unary(ctx_, AHIP_TANH, o, f(in[0]), out.dims.total_elems(), 0, 0); break;
    case OpKind::HardSigmoid:
        rc = launch_unary(ctx_, AHIP_HARDSIGMOID, o, f(in[0]), out.dims.total_elems(), op.alpha, op.beta);
        break;
    case OpKind::Softmax: {
        const size_t rank = in[0]->dims.len();
        if (rank == 0) return bail(SessionError::Message, "Softmax: rank-0 input");
        if (!(op.axis == -1 || op.axis == (int64_t)rank - 1))  // session.rs:999
            return bail(SessionError::Message, "Softmax: only the last axis is supported");
        const size_t len = in[0]->dims[rank - 1];
        rc = launch_softmax(ctx_, o, f(in[0]), len ? out.dims.total_elems() / len : 0, len);
        break;
    }
    case OpKind::LayerNormalization: {
        const size_t rank = in[0]->dims.len();
        if (rank == 0) return bail(SessionError::Message, "LayerNormalization: rank-0 input");
        if (!(op.axis == -1 || op.axis == (int64_t)rank - 1))
            return bail(SessionError::Message, "LayerNormalization: Axis must be the last dimension.");
        if (op.stash_type != 1) return bail(SessionError::Message, "LayerNormalization: Stash type must be 1.");
        const size_t len = in[0]->dims[rank - 1];
        if (in[1]->dims.total_elems() != len || in[2]->dims.total_elems() != len)
            return bail(SessionError::Shape, "LayerNormalization: scale and bias must hold one value per column");
        rc = launch_layernorm(ctx_, o, f(in[0]), f(in[1]), f(in[2]), len ? out.dims.total_elems() / len : 0, len,
                              op.epsilon);
        break;
    }
    case OpKind::ReduceMean:
    case OpKind::ReduceMax: {
        const FixedDimensions &d = in[0]->dims;
        const size_t rank = d.len();
        std::vector<size_t> axes;
        if (op.axes.empty()) {
            if (op.kind == OpKind::ReduceMean) {  // nothing is reduced: the output is the input
                if (out.nbytes())
                    rc = ctx_.check(hipMemcpyAsync(out.ptr, in[0]->ptr, out.nbytes(), hipMemcpyDeviceToDevice,
                                                   ctx_.stream),
                                    "hipMemcpyAsync(ReduceMean)");
                break;
            }
            for (size_t i = 0; i < rank; i++) axes.push_back(i);
        } else {
            for (int64_t a : op.axes) axes.push_back((size_t)(a < 0 ? a + (int64_t)rank : a));
        }
        size_t outer = 1, red = 1, inner = 1;
        if (rank > 0) {
            std::sort(axes.begin(), axes.end());
            axes.erase(std::unique(axes.begin(), axes.end()), axes.end());
            for (size_t i = 1; i < axes.size(); i++)
                if (axes[i] != axes[i - 1] + 1)
                    return bail(SessionError::Message, opname + ": reduced axes must be adjacent");
            for (size_t i = 0; i < axes.front(); i++) outer *= d[i];
            for (size_t i = axes.front(); i <= axes.back(); i++) red *= d[i];
            for (size_t i = axes.back() + 1; i < rank; i++) inner *= d[i];
        }
        rc = launch_reduce(ctx_, op.kind == OpKind::ReduceMean ? AHIP_REDUCE_MEAN : AHIP_REDUCE_MAX, o, f(in[0]),
                           outer, red, inner);
        break;
    }
    default:
        return bail(SessionError::Message, opname + ": Kernel not implemented");
    }
    if (rc) {
        release(out);
        return fail_code(err, rc, ctx_.last_error);
    }
    // A node may be listed with more outputs than this backend produces; only the first is bound.
    auto old = values.find(node.outputs[0]);
    if (old != values.end()) release(old->second);
    values[node.outputs[0]] = out;
    return true;
}

}  // namespace altius
