#include "hip_session.h"

#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <functional>
#include <limits>

#include "../device/host_pool.h"
#include "host_eval.h"
#include "views.h"

namespace altius {

using namespace detail;

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


// ---- BufferPool ------------------------------------------------------------------

size_t BufferPool::bucket_of(size_t bytes) {
    if (bytes == 0) bytes = 1;
    const size_t small = 256, large = (size_t)1 << 20;
    const size_t unit = bytes <= large ? small : large;
    return (bytes + unit - 1) / unit * unit;
}

BufferPool::~BufferPool() {
    hold_ = false;
    trim();
}

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

bool BufferPool::take(void *ptr, size_t bucket) {
    auto it = free_.find(bucket);
    if (it == free_.end()) return false;
    auto pos = std::find(it->second.begin(), it->second.end(), ptr);
    if (pos == it->second.end()) return false;
    it->second.erase(pos);
    return true;
}

void BufferPool::trim() {
    if (hold_) return;
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
    s->graph_replay_ = graph_replay_ && !enable_profiling_;
    s->device_timing_ = device_timing_;

    ShapeError serr;
    if (!infer_shapes(s->model_, &s->inferred_, nullptr, &serr)) {
        fail(err, SessionError::Shape, serr.message);
        return nullptr;
    }
    s->plan_ = create_execution_plan(s->model_);
    if (strided_views_) s->plan_views(fused_attention_);

    std::string derr;
    int rc = create_device_ctx(device_, nullptr, true, &s->ctx_, &derr);
    if (rc) {
        fail_code(err, rc, derr);
        return nullptr;
    }
    // Every input of a node was written by the node in front and is, up to the size of the caches, still in them.
    if (!getenv("AHIP_STREAMING_THRESHOLD_MIB")) s->ctx_.nt_threshold_bytes = SESSION_NT_THRESHOLD_BYTES;
    s->ctx_.nt_load_threshold_bytes = s->ctx_.nt_threshold_bytes;
    if (gemm_algorithm_ != AHIP_GEMM_AUTO && gemm_algorithm_ != AHIP_GEMM_FP32 && gemm_algorithm_ != AHIP_GEMM_BF16X3) {
        destroy_device_ctx(&s->ctx_);
        fail(err, SessionError::Argument, "unknown GEMM algorithm");
        return nullptr;
    }
    s->ctx_.gemm_algorithm = gemm_algorithm_;
    s->pool_.reset(new BufferPool(&s->ctx_));
    if (hipEventCreate(&s->span_begin_) != hipSuccess || hipEventCreate(&s->span_end_) != hipSuccess) {
        fail(err, SessionError::Hip, "hipEventCreate failed");
        return nullptr;
    }

    // Initializers live on the device for the lifetime of the session; their host contents stay
    // reachable for shape inference and shape arithmetic.
    for (const auto &kv : s->model_.graph.inits) {
        const Tensor &t = kv.second;
        if (t.nbytes() != t.dims().total_elems() * elem_size(t.elem_ty())) {
            fail(err, SessionError::Argument, "initializer data does not match its shape");
            return nullptr;
        }
        DeviceTensor d;
        if (!s->upload(t, &d, err)) return nullptr;
        if (t.elem_ty() == TensorElemType::F32 && d.ptr && d.nbytes()) gemm_register_constant(s->ctx_, d.ptr, d.nbytes());
        s->inits_[kv.first] = std::move(d);
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
        drop_graphs();
        if (span_begin_) (void)hipEventDestroy(span_begin_);
        if (span_end_) (void)hipEventDestroy(span_end_);
        inits_.clear();  // blocks go back to the pool before it is destroyed
        pool_.reset();
        destroy_device_ctx(&ctx_);
    }
}

bool HipSession::allocate(const TypedFixedShape &shape, DeviceTensor *out, SessionError *err) {
    out->dims = shape.dims;
    out->elem_ty = shape.elem_ty;
    out->host.reset();
    auto block = std::make_shared<DeviceBlock>();
    const int rc = pool_->acquire(out->nbytes(), &block->ptr, &block->bucket);
    if (rc) return fail_code(err, rc, ctx_.last_error);
    block->pool = pool_.get();
    if (capturing_) capture_allocs_.emplace_back(block->ptr, block->bucket);
    out->ptr = block->ptr;
    out->block = std::move(block);
    return true;
}

// Whether this Add (planned as the residual connection in front of a planes-writing LayerNormalization) can leave its
// sum to that kernel in this run: two dense f32 tensors of the result's shape, 16-byte aligned, nothing else owed, and
// the LayerNormalization's own conditions (row length, the product behind it on the bf16 route).
bool HipSession::defers_add(NodeId id, const std::vector<DeviceTensor *> &in, const std::vector<TypedFixedShape> &shapes) const {
    if (in.size() != 2 || !in[0] || !in[1] || shapes.empty()) return false;
    auto ln = planes_out_.find(add_into_ln_.at(id));
    if (ln == planes_out_.end() || matmul_out_perm_.count(ln->second.consumer)) return false;
    const FixedDimensions &d = shapes[0].dims;
    for (const DeviceTensor *t : {in[0], in[1]})
        if (t->elem_ty != TensorElemType::F32 || t->host || !(t->dims == d) || !t->strides.empty() || t->pending_op >= 0 || t->applied_op >= 0 ||
            t->planes || t->owes_add() || !t->ptr || (reinterpret_cast<uintptr_t>(t->ptr) & 15u))
            return false;
    if (d.len() < 2) return false;
    const size_t len = d[d.len() - 1], rows = len ? d.total_elems() / len : 0;
    return layernorm_planes_fits(rows, len) && gemm_takes_split(ctx_, rows, ln->second.next_n, len);
}

bool HipSession::allocate_bytes(size_t nbytes, DeviceTensor *out, SessionError *err) {
    auto block = std::make_shared<DeviceBlock>();
    const int rc = pool_->acquire(nbytes, &block->ptr, &block->bucket);
    if (rc) return fail_code(err, rc, ctx_.last_error);
    block->pool = pool_.get();
    if (capturing_) capture_allocs_.emplace_back(block->ptr, block->bucket);
    out->ptr = block->ptr;
    out->block = std::move(block);
    return true;
}

bool HipSession::upload(const Tensor &t, DeviceTensor *out, SessionError *err) {
    if (!allocate(TypedFixedShape{t.dims(), t.elem_ty()}, out, err)) return false;
    if (out->nbytes()) {
        const int rc = ctx_.check(hipMemcpyAsync(out->ptr, t.data_as_bytes(), out->nbytes(), hipMemcpyHostToDevice, ctx_.stream),
                                  "hipMemcpyAsync(upload)");
        if (rc) return fail_code(err, rc, ctx_.last_error);
    }
    out->host = std::make_shared<const Tensor>(t);  // shares the bytes; keeps them alive while the copy is in flight
    return true;
}

bool HipSession::fetch_host(DeviceTensor *t, SessionError *err) {
    if (t->host) return true;
    if (capturing_) {  // a read-back would synchronise the capturing stream
        capture_refused_ = true;
        return fail(err, SessionError::Message, "graph capture: a node needs tensor contents on the host");
    }
    Tensor h = Tensor::uninit_of_type(t->elem_ty, t->dims);
    if (!h.has_data()) return fail(err, SessionError::OutOfMemory, "out of host memory");
    if (t->nbytes()) {
        int rc = ctx_.check(hipMemcpyAsync(h.data_as_bytes_mut(), t->ptr, t->nbytes(), hipMemcpyDeviceToHost, ctx_.stream),
                            "hipMemcpyAsync(shape operand)");
        if (!rc) rc = ctx_.check(hipStreamSynchronize(ctx_.stream), "hipStreamSynchronize(shape operand)");
        if (rc) return fail_code(err, rc, ctx_.last_error);
    }
    t->host = std::make_shared<const Tensor>(std::move(h));
    return true;
}

// The shapes cached at build time were derived from the declared input shapes: kernels sized by
// them must never see a tensor of another extent.
bool HipSession::check_input(size_t i, TensorElemType elem_ty, const FixedDimensions &dims, SessionError *err) const {
    const auto &declared = model_.graph.values[model_.graph.inputs[i]].shape;
    if (!declared) return true;
    const auto fixed = declared->dims.as_fixed_dims();
    if (fixed && *fixed == dims && declared->elem_ty == elem_ty) return true;
    return fail(err, SessionError::Shape,
                "run: input " + std::to_string(i) + " is " + elem_name(elem_ty) + dims.to_string() +
                    " but the graph declares " + elem_name(declared->elem_ty) + (fixed ? fixed->to_string() : "a dynamic shape"));
}

bool HipSession::run(const std::vector<Tensor> &inputs, std::vector<Tensor> *outputs, SessionError *err) {
    std::lock_guard<std::mutex> lock(mutex_);
    const auto t0 = std::chrono::steady_clock::now();
    if (!outputs) return fail(err, SessionError::Argument, "run: null output vector");
    outputs->clear();
    profile_.clear();
    const Graph &g = model_.graph;
    if (inputs.size() < g.inputs.size())
        return fail(err, SessionError::Argument,
                    "run: " + std::to_string(inputs.size()) + " inputs given, the graph has " +
                        std::to_string(g.inputs.size()));
    if (hipSetDevice(ctx_.device) != hipSuccess) return fail(err, SessionError::Hip, "hipSetDevice failed");
    for (size_t i = 0; i < g.inputs.size(); i++)
        if (!check_input(i, inputs[i].elem_ty(), inputs[i].dims(), err)) return false;

    if (graph_replay_) {
        if (seen_ws_generation_ != ctx_.gemm_ws_generation) {  // the GEMM workspace moved: recorded launches point at the old one
            drop_graphs();
            seen_ws_generation_ = ctx_.gemm_ws_generation;
        }
        std::string key;
        for (size_t i = 0; i < g.inputs.size(); i++)
            key += std::to_string((int)inputs[i].elem_ty()) + inputs[i].dims().to_string() + ";";
        auto it = graphs_.find(key);
        if (it == graphs_.end() && eager_runs_[key] >= 1) {
            if (!try_capture(key, inputs, err)) return false;
            it = graphs_.find(key);
        }
        if (it != graphs_.end() && !it->second.unusable) {
            if (!replay(it->second, inputs, outputs, err)) return false;
            last_run_ms_ = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
            return true;
        }
        eager_runs_[key]++;
    }

    std::map<ValueId, DeviceTensor> values;
    copies_avoided_ = 0;
    pending_attn_.clear();
    absorbed_add_.clear();
    std::vector<hipEvent_t> events;
    // Nothing may still read a block when it goes back to the pool for another run, and input
    // tensors must outlive their uploads: every exit path synchronises first.
    auto finish = [&](bool ok) {
        (void)hipStreamSynchronize(ctx_.stream);
        for (auto e : events) (void)hipEventDestroy(e);
        values.clear();
        return ok;
    };

    // Upload the inputs (positional, session.rs:81-83).
    for (size_t i = 0; i < g.inputs.size(); i++) {
        const Tensor &t = inputs[i];
        if (!t.has_data()) return finish(fail(err, SessionError::Argument, "run: input " + std::to_string(i) + " has no data"));
        DeviceTensor d;
        if (!upload(t, &d, err)) return finish(false);
        // Only small integer inputs keep their host view (shape arithmetic may read them).
        if (t.elem_ty() == TensorElemType::F32 || t.dims().total_elems() > 4096) d.host.reset();
        values[g.inputs[i]] = std::move(d);
    }

    // One event per node boundary when profiling.
    if (enable_profiling_) {
        events.resize(plan_.size() + 1);
        for (size_t i = 0; i < events.size(); i++) {
            if (hipEventCreate(&events[i]) != hipSuccess) {
                events.resize(i);
                return finish(fail(err, SessionError::Hip, "hipEventCreate failed"));
            }
        }
        (void)hipEventRecord(events[0], ctx_.stream);
    }

    // The hot loop (session.rs:86-92).
    if (device_timing_) (void)hipEventRecord(span_begin_, ctx_.stream);
    for (size_t i = 0; i < plan_.size(); i++) {
        if (!run_node(plan_[i].node_id, values, err)) return finish(false);
        if (enable_profiling_) (void)hipEventRecord(events[i + 1], ctx_.stream);
        // Stream order makes immediate reuse safe.  A value that is also a graph output stays: the
        // plan lists it when another node reads it, but it is still owed to the caller.
        for (ValueId v : plan_[i].free_vals)
            if (std::find(g.outputs.begin(), g.outputs.end(), v) == g.outputs.end()) values.erase(v);
    }

    if (device_timing_) (void)hipEventRecord(span_end_, ctx_.stream);

    // Download the outputs (session.rs:127-133).
    for (ValueId v : g.outputs) {
        const DeviceTensor *d = nullptr;
        auto it = values.find(v);
        if (it != values.end() && (!materialize(&it->second, err) || !apply_pending(&it->second, err))) return finish(false);  // never planned; dense for the caller
        if (it != values.end()) d = &it->second;
        else {
            auto ii = inits_.find(v);
            if (ii != inits_.end()) d = &ii->second;
        }
        if (!d) return finish(fail(err, SessionError::Message, "run: graph output was not produced"));
        Tensor t = Tensor::uninit_of_type(d->elem_ty, d->dims, pinned_host_block);
        if (!t.has_data()) return finish(fail(err, SessionError::OutOfMemory, "run: out of host memory for an output tensor"));
        if (d->nbytes()) {
            const int rc = ctx_.check(hipMemcpyAsync(t.data_as_bytes_mut(), d->ptr, d->nbytes(), hipMemcpyDeviceToHost, ctx_.stream),
                                      "hipMemcpyAsync(output)");
            if (rc) return finish(fail_code(err, rc, ctx_.last_error));
        }
        outputs->push_back(std::move(t));
    }
    int rc = ctx_.check(hipStreamSynchronize(ctx_.stream), "hipStreamSynchronize(run)");
    if (!rc) rc = check_device_flags(ctx_);
    if (rc) {
        outputs->clear();
        return finish(fail_code(err, rc, ctx_.last_error));
    }
    float span_ms = 0;
    last_device_ms_ = device_timing_ && hipEventElapsedTime(&span_ms, span_begin_, span_end_) == hipSuccess ? span_ms : 0;
    if (enable_profiling_) {
        for (size_t i = 0; i < plan_.size(); i++) {
            float ms = 0;
            if (hipEventElapsedTime(&ms, events[i], events[i + 1]) == hipSuccess)
                profile_[model_.graph.nodes[plan_[i].node_id].op.name()] += ms;
        }
    }
    finish(true);
    last_run_ms_ = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    return true;
}

bool HipSession::run_device(const std::vector<DeviceTensor> &inputs, std::vector<DeviceTensor> *outputs, SessionError *err) {
    std::lock_guard<std::mutex> lock(mutex_);
    const auto t0 = std::chrono::steady_clock::now();
    if (!outputs) return fail(err, SessionError::Argument, "run_device: null output vector");
    outputs->clear();
    profile_.clear();
    const Graph &g = model_.graph;
    if (inputs.size() < g.inputs.size())
        return fail(err, SessionError::Argument,
                    "run_device: " + std::to_string(inputs.size()) + " inputs given, the graph has " +
                        std::to_string(g.inputs.size()));
    if (hipSetDevice(ctx_.device) != hipSuccess) return fail(err, SessionError::Hip, "hipSetDevice failed");

    std::map<ValueId, DeviceTensor> values;
    copies_avoided_ = 0;
    pending_attn_.clear();
    absorbed_add_.clear();
    for (size_t i = 0; i < g.inputs.size(); i++) {
        if (!inputs[i].ptr && inputs[i].nbytes())
            return fail(err, SessionError::Argument, "run_device: input " + std::to_string(i) + " has no device pointer");
        if (!check_input(i, inputs[i].elem_ty, inputs[i].dims, err)) return false;
        DeviceTensor d;
        d.dims = inputs[i].dims;
        d.elem_ty = inputs[i].elem_ty;
        d.ptr = inputs[i].ptr;  // the caller's memory: no block, never returned to the pool
        values[g.inputs[i]] = std::move(d);
    }
    // A failed run leaves nothing behind; blocks released while kernels are still queued are only
    // handed to later work on the same stream.
    if (device_timing_) (void)hipEventRecord(span_begin_, ctx_.stream);
    for (size_t i = 0; i < plan_.size(); i++) {
        if (!run_node(plan_[i].node_id, values, err)) return false;
        for (ValueId v : plan_[i].free_vals)
            if (std::find(g.outputs.begin(), g.outputs.end(), v) == g.outputs.end()) values.erase(v);
    }
    if (device_timing_) (void)hipEventRecord(span_end_, ctx_.stream);
    for (ValueId v : g.outputs) {
        const DeviceTensor *d = nullptr;
        auto it = values.find(v);
        if (it != values.end() && (!materialize(&it->second, err) || !apply_pending(&it->second, err))) return false;  // never planned; dense for the caller
        if (it != values.end()) d = &it->second;
        else {
            auto ii = inits_.find(v);
            if (ii != inits_.end()) d = &ii->second;
        }
        if (!d) {
            outputs->clear();
            return fail(err, SessionError::Message, "run_device: graph output was not produced");
        }
        outputs->push_back(*d);
    }
    span_pending_ = device_timing_;
    last_run_ms_ = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    return true;
}

bool HipSession::synchronize(SessionError *err) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (hipSetDevice(ctx_.device) != hipSuccess) return fail(err, SessionError::Hip, "hipSetDevice failed");
    int rc = ctx_.check(hipStreamSynchronize(ctx_.stream), "hipStreamSynchronize");
    if (!rc) rc = check_device_flags(ctx_);
    if (rc) return fail_code(err, rc, ctx_.last_error);
    if (span_pending_) {
        span_pending_ = false;
        float span_ms = 0;
        last_device_ms_ = hipEventElapsedTime(&span_ms, span_begin_, span_end_) == hipSuccess ? span_ms : 0;
    }
    return true;
}

void HipSession::release(DeviceTensor *t) {
    std::lock_guard<std::mutex> lock(mutex_);
    *t = DeviceTensor();
}

void HipSession::drop_graphs() {
    for (auto &kv : graphs_)
        if (kv.second.exec) (void)hipGraphExecDestroy(kv.second.exec);
    graphs_.clear();
    if (pool_) pool_->hold_memory(false);
}

// Records the node loop for these input shapes.  Returns false only for errors that should fail
// the run; a refused capture marks the signature unusable and returns true.
bool HipSession::try_capture(const std::string &key, const std::vector<Tensor> &inputs, SessionError *err) {
    const Graph &g = model_.graph;
    CapturedRun run;
    std::map<ValueId, DeviceTensor> values;
    copies_avoided_ = 0;
    pending_attn_.clear();
    absorbed_add_.clear();
    for (size_t i = 0; i < g.inputs.size(); i++) {
        DeviceTensor d;
        if (!allocate(TypedFixedShape{inputs[i].dims(), inputs[i].elem_ty()}, &d, err)) return false;
        run.inputs.push_back(d);
        values[g.inputs[i]] = d;
    }
    if (hipStreamBeginCapture(ctx_.stream, hipStreamCaptureModeRelaxed) != hipSuccess) {
        (void)hipGetLastError();
        graphs_[key].unusable = true;
        return true;
    }
    capturing_ = true;
    capture_refused_ = false;
    capture_allocs_.clear();
    ctx_.flags_armed = false;
    bool ok = true;
    SessionError local;
    for (size_t i = 0; i < plan_.size() && ok; i++) {
        ok = run_node(plan_[i].node_id, values, &local);
        if (!ok) break;
        for (ValueId v : plan_[i].free_vals)
            if (std::find(g.outputs.begin(), g.outputs.end(), v) == g.outputs.end()) values.erase(v);
    }
    capturing_ = false;
    hipGraph_t graph = nullptr;
    const hipError_t end = hipStreamEndCapture(ctx_.stream, &graph);
    run.has_gather = ctx_.flags_armed;
    ctx_.flags_armed = false;
    // A capture that had to grow the pool recorded kernels against fresh blocks: still valid, the
    // blocks stay in the pool.  A capture that failed for any reason leaves the eager path in charge.
    if (ok && end == hipSuccess && graph) {
        for (ValueId v : g.outputs) {
            auto it = values.find(v);
            if (it != values.end() && (!materialize(&it->second, err) || !apply_pending(&it->second, err))) ok = false;
            const DeviceTensor *d = it != values.end() ? &it->second : nullptr;
            if (!d) {
                auto ii = inits_.find(v);
                if (ii != inits_.end()) d = &ii->second;
            }
            if (!d) {
                ok = false;
                break;
            }
            run.outputs.push_back(*d);  // holds the block: the recorded kernels write here on every replay
        }
    }
    if (ok && end == hipSuccess && graph && hipGraphInstantiate(&run.exec, graph, nullptr, nullptr, 0) == hipSuccess) {
        (void)hipGraphDestroy(graph);
        // The recorded kernels address their intermediates directly.  Those blocks went back to the pool as the
        // plan freed them (and were reused inside the recording, which stream order allows); take every one of
        // them out of the pool for as long as the graph lives.
        values.clear();
        pending_attn_.clear();
        std::sort(capture_allocs_.begin(), capture_allocs_.end());
        capture_allocs_.erase(std::unique(capture_allocs_.begin(), capture_allocs_.end()), capture_allocs_.end());
        for (const auto &a : capture_allocs_)
            if (pool_->take(a.first, a.second)) {
                auto block = std::make_shared<DeviceBlock>();
                block->pool = pool_.get();
                block->ptr = a.first;
                block->bucket = a.second;
                run.blocks.push_back(std::move(block));
            }
        capture_allocs_.clear();
        graphs_[key] = std::move(run);
        pool_->hold_memory(true);
        return true;
    }
    (void)hipGetLastError();
    if (graph) (void)hipGraphDestroy(graph);
    if (!ok && !capture_refused_) {  // a real error (unsupported operator, bad shapes): report it as the eager run would
        if (err) *err = local;
        return false;
    }
    graphs_[key].unusable = true;
    return true;
}

bool HipSession::replay(CapturedRun &run, const std::vector<Tensor> &inputs, std::vector<Tensor> *outputs, SessionError *err) {
    int rc = AHIP_OK;
    for (size_t i = 0; i < run.inputs.size(); i++)
        if (!inputs[i].has_data()) return fail(err, SessionError::Argument, "run: input " + std::to_string(i) + " has no data");
    for (size_t i = 0; i < run.inputs.size() && !rc; i++)
        if (run.inputs[i].nbytes())
            rc = ctx_.check(hipMemcpyAsync(run.inputs[i].ptr, inputs[i].data_as_bytes(), run.inputs[i].nbytes(), hipMemcpyHostToDevice,
                                           ctx_.stream),
                            "hipMemcpyAsync(input)");
    if (device_timing_) (void)hipEventRecord(span_begin_, ctx_.stream);
    if (!rc) rc = ctx_.check(hipGraphLaunch(run.exec, ctx_.stream), "hipGraphLaunch");
    if (device_timing_) (void)hipEventRecord(span_end_, ctx_.stream);
    for (size_t i = 0; i < run.outputs.size() && !rc; i++) {
        Tensor t = Tensor::uninit_of_type(run.outputs[i].elem_ty, run.outputs[i].dims, pinned_host_block);
        if (!t.has_data()) {
            (void)hipStreamSynchronize(ctx_.stream);
            outputs->clear();
            return fail(err, SessionError::OutOfMemory, "run: out of host memory for an output tensor");
        }
        if (run.outputs[i].nbytes())
            rc = ctx_.check(hipMemcpyAsync(t.data_as_bytes_mut(), run.outputs[i].ptr, run.outputs[i].nbytes(), hipMemcpyDeviceToHost,
                                           ctx_.stream),
                            "hipMemcpyAsync(output)");
        outputs->push_back(std::move(t));
    }
    const int rs = ctx_.check(hipStreamSynchronize(ctx_.stream), "hipStreamSynchronize(run)");
    if (!rc) rc = rs;
    if (!rc && run.has_gather) {
        ctx_.flags_armed = true;
        rc = check_device_flags(ctx_);
    }
    if (rc) {
        outputs->clear();
        return fail_code(err, rc, ctx_.last_error);
    }
    float span_ms = 0;
    last_device_ms_ = device_timing_ && hipEventElapsedTime(&span_ms, span_begin_, span_end_) == hipSuccess ? span_ms : 0;
    graph_replays_++;
    return true;
}

bool HipSession::run_node(NodeId id, std::map<ValueId, DeviceTensor> &values, SessionError *err) {
    const Node &node = model_.graph.nodes[id];
    auto opname = [&]() { return std::string(node.op.name()); };  // for messages only

    // Inputs: run-time values first, then initializers.  An input whose value is never produced
    // and carries the empty name is an omitted optional input (the reference binds a dummy tensor).
    std::vector<DeviceTensor *> in;
    for (ValueId v : node.inputs) {
        auto it = values.find(v);
        if (it != values.end()) {
            in.push_back(&it->second);
            continue;
        }
        auto ii = inits_.find(v);
        if (ii != inits_.end()) {
            in.push_back(&ii->second);
            continue;
        }
        const auto &name = model_.graph.values[v].name;
        if (name && name->empty()) {
            in.push_back(nullptr);
            continue;
        }
        return fail(err, SessionError::Message, opname() + ": an input value is missing");
    }
    if (node.outputs.empty()) return fail(err, SessionError::Message, opname() + ": node without outputs");
    // Strided views are read in place by the operators that can; every other reader gets a dense
    // copy, which also replaces the view for whoever reads the value later.
    if (!reads_views(node.op.kind))
        for (auto *d : in)
            if (d && !d->strides.empty() && !materialize(d, err)) return false;
    // Operand planes have exactly one planned reader: the product behind the LayerNormalization that wrote them.
    for (size_t i = 0; i < in.size(); i++)
        if (in[i] && in[i]->planes && !(i == 0 && (planes_consumer_.count(id) || planes_pass_.count(id))))
            return fail(err, SessionError::Message, "internal: operand planes reached an operator that cannot read them");
    // A deferred Add runs now unless the reader is the LayerNormalization that can compute the sum itself.
    for (size_t i = 0; i < in.size(); i++)
        if (in[i] && in[i]->owes_add() && !(i == 0 && planes_out_.count(id)) && !flush_add(in[i], err)) return false;
    // An activation still owed is applied by the MatMul that reads the tensor as its first operand, or here.
    for (size_t i = 0; i < in.size(); i++)
        if (in[i] && in[i]->pending_op >= 0 && !(node.op.kind == OpKind::MatMul && i == 0) &&
            !(in[i]->pending_op == PENDING_ATTENTION && i == 0 && attn_softmax_.count(id)) &&
            !(in[i]->pending_op == PENDING_ATTENTION ? flush_attention(node.inputs[i], in[i], err) : apply_pending(in[i], err)))
            return false;

    // Output shapes: inferred at build time if possible, else now (session.rs:149-158).  Operands
    // whose contents decide a shape are read from their host copy, fetched on demand.
    Op inferred_op;
    std::vector<TypedFixedShape> inferred_shapes;
    const Op *op_used = &inferred_op;
    const std::vector<TypedFixedShape> *shapes_used = &inferred_shapes;
    auto cached = inferred_.find(id);
    if (cached != inferred_.end()) {  // no copies on this path: it is the one every node of a planned graph takes
        op_used = &cached->second.first;
        shapes_used = &cached->second.second;
    } else if (capturing_) {
        capture_refused_ = true;
        return fail(err, SessionError::Message, "graph capture: a node's shape is not known before the run");
    } else {
        static const Tensor absent;
        for (int attempt = 0;; attempt++) {
            std::vector<Tensor> meta;
            meta.reserve(in.size());
            for (auto *d : in) meta.push_back(!d ? absent : d->host ? *d->host : Tensor::empty_of_type(d->elem_ty, d->dims));
            std::vector<const Tensor *> ptrs;
            for (auto &m : meta) ptrs.push_back(&m);
            ShapeError serr;
            inferred_op = node.op;
            if (compute_output_shapes(model_, inferred_op, ptrs, node.outputs.size(), &inferred_shapes, &serr)) break;
            if (!serr.needs_data || attempt > 0) return fail(err, SessionError::Shape, serr.message);
            // Read back the small operands (shape vectors, Resize scales) and try once more.
            for (size_t i = 1; i < in.size(); i++)
                if (in[i] && !in[i]->host && in[i]->dims.total_elems() <= 4096 && !fetch_host(in[i], err)) return false;
        }
    }
    const Op &op = *op_used;
    const std::vector<TypedFixedShape> &shapes = *shapes_used;
    if (shapes.size() < node.outputs.size()) return fail(err, SessionError::Message, opname() + ": output count mismatch");

    std::vector<DeviceTensor> outs;
    values_ = &values;

    auto absorbed = absorbed_add_.find(id);
    if (absorbed != absorbed_add_.end() && absorbed->second < in.size() && in[absorbed->second]) {
        // The MatMul that produced one operand has added the other one already.
        DeviceTensor o = *in[absorbed->second];
        absorbed_add_.erase(absorbed);
        o.dims = shapes[0].dims;
        copies_avoided_++;
        outs.push_back(std::move(o));
    } else if ((op.kind == OpKind::Gelu || op.kind == OpKind::ReLU) && in[0] && in[0]->applied_op == (op.kind == OpKind::Gelu ? AHIP_GELU : AHIP_RELU)) {
        // The MatMul that produced the operand has applied this activation already.
        DeviceTensor o = *in[0];
        o.dims = shapes[0].dims;
        o.applied_op = -1;
        copies_avoided_++;
        outs.push_back(std::move(o));
    } else
    // Reshape family: the output is the input's memory under another shape.
    if (is_alias_op(op.kind) && in[0]) {
        std::vector<int64_t> view_strides;
        if (!in[0]->strides.empty()) {
            if (!reshape_strides(in[0]->dims, in[0]->strides, shapes[0].dims, &view_strides)) {
                if (!materialize(in[0], err)) return false;
                view_strides.clear();
            } else if (is_dense(shapes[0].dims, view_strides)) {
                view_strides.clear();
            }
        }
        DeviceTensor o = *in[0];
        o.dims = shapes[0].dims;
        o.strides = view_strides;
        if (in[0]->host) {
            Tensor h = in[0]->host->reshaped(shapes[0].dims);
            o.host = h.has_data() || shapes[0].dims.total_elems() == 0 ? std::make_shared<const Tensor>(std::move(h)) : nullptr;
        }
        outs.push_back(std::move(o));
    } else if (attn_softmax_.count(id) && in[0] && in[0]->pending_op == PENDING_ATTENTION) {
        // The Softmax of a deferred attention: its work happens in the second product's kernel.
        auto it = pending_attn_.find(node.inputs[0]);
        if (it == pending_attn_.end()) return fail(err, SessionError::Message, "Softmax: deferred attention operands are missing");
        // An absorbed mask must be one value per key: a single row, or one row per outermost batch.
        bool fits = true;
        DeviceTensor *mask_t = nullptr;
        size_t mask_stride = 0;
        if (op.prologue_mask) {
            const size_t n_in = 1 + (op.prologue_scale ? 1 : 0) + 1;
            mask_t = in.size() >= n_in ? in[n_in - 1] : nullptr;
            const FixedDimensions &sd = it->second.score_dims;
            const size_t tk = sd[sd.len() - 1];
            fits = mask_t && mask_t->elem_ty == TensorElemType::F32 && mask_t->strides.empty() && mask_t->pending_op < 0 &&
                   (reinterpret_cast<uintptr_t>(mask_t->ptr) & 3u) == 0;
            const size_t m_elems = fits ? mask_t->dims.total_elems() : 0;
            if (fits && m_elems == tk) {
                mask_stride = 0;
            } else if (fits && !it->second.bd.empty() && m_elems == sd[0] * tk && sd[0] == it->second.bd[0] && mask_t->dims.len() >= 1 &&
                       mask_t->dims[mask_t->dims.len() - 1] == tk) {
                mask_stride = tk;
            } else {
                fits = false;
            }
        }
        if (fits) {
            PendingAttention pa = std::move(it->second);
            pending_attn_.erase(it);
            if (mask_t) pa.mask = *mask_t, pa.mask_outer_stride = mask_stride;
            pending_attn_[node.outputs[0]] = std::move(pa);
            DeviceTensor o = *in[0];
            o.dims = shapes[0].dims;
            copies_avoided_++;
            outs.push_back(std::move(o));
        } else {
            // This Softmax is not one the attention kernel can absorb: compute the scores after all and go on as usual.
            if (!flush_attention(node.inputs[0], in[0], err)) return false;
            copies_avoided_--;
            current_node_ = id;
            if (!run_device_op(node, op, in, shapes, &outs, err)) return false;
        }
    } else if (add_into_ln_.count(id) && defers_add(id, in, shapes)) {
        // A residual Add whose sum the LayerNormalization behind it computes on its way: reserve the sum's block,
        // keep the operands, run nothing yet.
        DeviceTensor o;
        if (!allocate(shapes[0], &o, err)) return false;
        auto p = std::make_shared<PendingAdd>();
        p->a_block = in[0]->block, p->b_block = in[1]->block;
        p->a = static_cast<const float *>(in[0]->ptr), p->b = static_cast<const float *>(in[1]->ptr);
        p->elems = shapes[0].dims.total_elems();
        o.pending_add = std::move(p);
        copies_avoided_++;
        outs.push_back(std::move(o));
    } else if (deferred_unary_.count(id) && in[0] && !in[0]->host && in[0]->elem_ty == TensorElemType::F32 && in[0]->pending_op < 0) {
        DeviceTensor o = *in[0];
        o.dims = shapes[0].dims;
        o.pending_op = op.kind == OpKind::Gelu ? AHIP_GELU : AHIP_RELU;
        copies_avoided_++;
        outs.push_back(std::move(o));
    } else if (op.kind == OpKind::Transpose && in[0] && !in[0]->host && (lazy_views_.count(id) || !in[0]->strides.empty())) {
        // The permuted strides describe the result in place.  Dense again (the Transpose that a MatMul
        // wrote ahead of): a plain tensor.  Otherwise a view when every reader takes views, else a
        // strided copy.
        const std::vector<int64_t> s = strides_of(*in[0]);
        if (op.perm.size() != s.size()) return fail(err, SessionError::Shape, "Transpose: perm does not match the rank");
        std::vector<int64_t> ps(s.size());
        for (size_t i = 0; i < s.size(); i++) ps[i] = s[(size_t)op.perm[i]];
        if (is_dense(shapes[0].dims, ps) || lazy_views_.count(id)) {
            copies_avoided_++;
            DeviceTensor o = *in[0];
            o.dims = shapes[0].dims;
            o.strides = is_dense(shapes[0].dims, ps) ? std::vector<int64_t>() : ps;
            outs.push_back(std::move(o));
        } else {
            DeviceTensor o;
            if (!allocate(shapes[0], &o, err)) return false;
            std::vector<int64_t> d;
            for (auto x : o.dims.as_vec()) d.push_back((int64_t)x);
            const std::vector<int64_t> os = dense_strides(o.dims);
            const int rc = launch_copy_strided(ctx_, o.ptr, in[0]->ptr, (int)elem_size(o.elem_ty), (int)d.size(), d.data(), os.data(), ps.data());
            if (rc) return fail_code(err, rc, ctx_.last_error);
            outs.push_back(std::move(o));
        }
    } else if (op.kind == OpKind::Split && in[0] && !in[0]->host && lazy_views_.count(id)) {
        const size_t rank = in[0]->dims.len();
        const size_t axis = (size_t)(op.axis < 0 ? op.axis + (int64_t)rank : op.axis);
        if (axis >= rank) return fail(err, SessionError::Shape, "Split: axis out of range");
        const std::vector<int64_t> s = strides_of(*in[0]);
        size_t start = 0;
        copies_avoided_++;
        for (size_t p = 0; p < node.outputs.size(); p++) {
            DeviceTensor o = *in[0];
            o.dims = shapes[p].dims;
            o.ptr = static_cast<char *>(in[0]->ptr) + start * (size_t)s[axis] * elem_size(o.elem_ty);
            o.strides = is_dense(o.dims, s) ? std::vector<int64_t>() : s;
            start += o.dims[axis];
            outs.push_back(std::move(o));
        }
    } else {
        // Shape arithmetic: integer tensors whose operands the host already knows (or can read back
        // cheaply) are computed there and uploaded; Shape and Constant always are.
        bool on_host = false;
        if (host_evaluable(op)) {
            const bool int_out = shapes[0].elem_ty != TensorElemType::F32;
            bool small = shapes[0].dims.total_elems() <= 4096;
            bool ints_in = true;
            for (auto *d : in)
                if (d) {
                    small = small && d->dims.total_elems() <= 4096;
                    ints_in = ints_in && d->elem_ty != TensorElemType::F32;
                }
            if (op.kind == OpKind::Shape || op.kind == OpKind::Constant) {
                on_host = true;
            } else if (small && ints_in && (int_out || op.kind == OpKind::Cast)) {
                on_host = true;
                for (auto *d : in)
                    if (d && !fetch_host(d, err)) return false;
            }
        }
        if (on_host && capturing_) {
            capture_refused_ = true;
            return fail(err, SessionError::Message, "graph capture: a node is evaluated on the host");
        }
        if (on_host) {
            std::vector<const Tensor *> hin;
            static const Tensor no_data;
            for (auto *d : in) hin.push_back(!d ? nullptr : d->host ? d->host.get() : &no_data);
            // Shape reads only the dims of its operand.
            std::vector<Tensor> dims_only;
            if (op.kind == OpKind::Shape && in[0] && !in[0]->host) {
                dims_only.push_back(Tensor::empty_of_type(in[0]->elem_ty, in[0]->dims));
                hin[0] = &dims_only[0];
            }
            std::vector<Tensor> results;
            std::string msg;
            if (!evaluate_on_host(model_, op, hin, shapes, &results, &msg)) return fail(err, SessionError::Message, msg);
            for (const Tensor &t : results) {
                DeviceTensor d;
                if (!upload(t, &d, err)) return false;
                outs.push_back(std::move(d));
            }
        } else if (current_node_ = id, !run_device_op(node, op, in, shapes, &outs, err)) {
            return false;
        }
    }
    for (size_t i = 0; i < node.outputs.size() && i < outs.size(); i++) values[node.outputs[i]] = std::move(outs[i]);
    return true;
}

// Op::FusedElemwise: the whole chain in one kernel when its operands fit the kernel's geometry and
// every step has a step code there; otherwise the steps run one after the other through their own
// kernels, which gives the same bits.
bool HipSession::run_fused_elemwise(const Node &node, const Op &op, const std::vector<DeviceTensor *> &in,
                                    const std::vector<TypedFixedShape> &shapes, std::vector<DeviceTensor> *outs, SessionError *err) {
    if (!op.fused || op.fused->chain.empty()) return fail(err, SessionError::Message, "FusedElemwise: empty chain");
    const FusedElemwise &f = *op.fused;
    if (in.size() < f.input_map.size()) return fail(err, SessionError::Message, "FusedElemwise: too few inputs");
    for (size_t i = 0; i < f.input_map.size(); i++)
        if (!in[i]) return fail(err, SessionError::Message, "FusedElemwise: an input value is missing");
    auto outer_index = [&](ValueId v) -> int {
        for (size_t i = 0; i < f.input_map.size(); i++)
            if (f.input_map[i] == v) return (int)i;
        return -1;
    };

    // Translate the chain into the kernel's steps while following the shapes operator by operator
    // (Pow's scalar-exponent path depends on the operand extents of its own node).
    std::vector<ahip_fused_step> steps;
    bool one_kernel = f.input_map.size() <= AHIP_FUSED_MAX_INPUTS && f.chain.size() <= AHIP_FUSED_MAX_STEPS &&
                      shapes[0].elem_ty == TensorElemType::F32 && shapes[0].dims.len() <= (size_t)MAX_RANK;
    for (size_t i = 0; i < f.input_map.size() && one_kernel; i++) one_kernel = in[i]->elem_ty == TensorElemType::F32;
    FixedDimensions prev_dims;
    ValueId prev_id = 0;
    for (size_t t = 0; t < f.chain.size() && one_kernel; t++) {
        const auto &step = f.chain[t];
        ahip_fused_step s{};
        std::vector<FixedDimensions> operand_dims;
        int sel[2] = {AHIP_FUSED_ACC, AHIP_FUSED_ACC};
        if (step.inputs.empty() || step.inputs.size() > 2 || step.outputs.size() != 1) {
            one_kernel = false;
            break;
        }
        for (size_t k = 0; k < step.inputs.size(); k++) {
            const int idx = outer_index(step.inputs[k]);
            if (idx >= 0) {
                sel[k] = idx;
                operand_dims.push_back(in[idx]->dims);
            } else if (t > 0 && step.inputs[k] == prev_id) {
                operand_dims.push_back(prev_dims);
            } else {
                return fail(err, SessionError::Message, "FusedElemwise: a step reads a value that is neither an input nor the previous result");
            }
        }
        s.lhs = sel[0];
        s.rhs = sel[1];
        switch (step.op.kind) {
        case OpKind::Add: s.op = AHIP_ADD; break;
        case OpKind::Sub: s.op = AHIP_SUB; break;
        case OpKind::Mul: s.op = AHIP_MUL; break;
        case OpKind::Div: s.op = AHIP_DIV; break;
        case OpKind::Pow: s.op = AHIP_POW; break;
        case OpKind::Sqrt: s.is_unary = 1; s.op = AHIP_SQRT; break;
        case OpKind::ReLU: s.is_unary = 1; s.op = AHIP_RELU; break;
        case OpKind::Gelu: s.is_unary = 1; s.op = AHIP_GELU; break;
        case OpKind::Sigmoid: s.is_unary = 1; s.op = AHIP_SIGMOID; break;
        case OpKind::Erf: s.is_unary = 1; s.op = AHIP_ERF; break;
        case OpKind::Tanh: s.is_unary = 1; s.op = AHIP_TANH; break;
        case OpKind::Exp: s.is_unary = 1; s.op = AHIP_EXP; break;
        case OpKind::Round: s.is_unary = 1; s.op = AHIP_ROUND; break;
        case OpKind::HardSigmoid: s.is_unary = 1; s.op = AHIP_HARDSIGMOID; s.alpha = step.op.alpha; s.beta = step.op.beta; break;
        case OpKind::LeakyReLU: s.is_unary = 1; s.op = AHIP_LEAKYRELU; s.alpha = step.op.alpha; break;
        default: one_kernel = false; break;  // Greater, or anything without a step code
        }
        if (!one_kernel) break;
        if ((s.is_unary != 0) != (step.inputs.size() == 1)) {
            one_kernel = false;
            break;
        }
        if (s.is_unary) {
            prev_dims = operand_dims[0];
        } else {
            auto b = operand_dims[0].broadcast(operand_dims[1]);
            if (!b) return fail(err, SessionError::Shape, std::string("FusedElemwise: ") + step.op.name() + " operands do not broadcast");
            // launch_binary's rule: one exponent for a base of more than one element.
            s.pow_scalar_exponent = s.op == AHIP_POW && operand_dims[1].total_elems() == 1 && operand_dims[0].total_elems() > 1;
            prev_dims = *b;
        }
        prev_id = step.outputs[0];
        steps.push_back(s);
    }
    if (one_kernel && prev_dims != shapes[0].dims) one_kernel = false;

    if (one_kernel) {
        DeviceTensor out;
        if (!allocate(shapes[0], &out, err)) return false;
        std::vector<std::vector<int64_t>> strides(f.input_map.size());
        std::vector<const int64_t *> stride_ptrs;
        std::vector<const float *> ptrs;
        for (size_t i = 0; i < f.input_map.size(); i++) {
            auto st = in[i]->dims.strides_for_broadcasting_to(out.dims);
            if (!st) return fail(err, SessionError::Shape, "FusedElemwise: an operand does not broadcast to the output shape");
            for (auto x : st->as_vec()) strides[i].push_back((int64_t)x);
            stride_ptrs.push_back(strides[i].data());
            ptrs.push_back(static_cast<const float *>(in[i]->ptr));
        }
        std::vector<int64_t> dims;
        for (auto x : out.dims.as_vec()) dims.push_back((int64_t)x);
        const int rc = launch_fused_elemwise(ctx_, static_cast<float *>(out.ptr), (int)dims.size(), dims.data(), (int)ptrs.size(), ptrs.data(),
                                             stride_ptrs.data(), (int)steps.size(), steps.data());
        if (rc == AHIP_OK) {
            outs->push_back(std::move(out));
            return true;
        }
        if (rc != AHIP_ERR_UNSUPPORTED) return fail_code(err, rc, ctx_.last_error);
        // geometry the kernel does not take: fall through to the operator-by-operator route
    }

    DeviceTensor prev;
    bool have_prev = false;
    prev_id = 0;
    for (const auto &step : f.chain) {
        if (step.outputs.size() != 1) return fail(err, SessionError::Message, "FusedElemwise: a step must have one output");
        std::vector<DeviceTensor *> ins;
        std::vector<Tensor> meta;
        meta.reserve(step.inputs.size());
        for (ValueId v : step.inputs) {
            const int idx = outer_index(v);
            if (idx >= 0) ins.push_back(in[idx]);
            else if (have_prev && v == prev_id) ins.push_back(&prev);
            else return fail(err, SessionError::Message, "FusedElemwise: a step reads a value that is neither an input nor the previous result");
            meta.push_back(Tensor::empty_of_type(ins.back()->elem_ty, ins.back()->dims));
        }
        std::vector<const Tensor *> meta_ptrs;
        for (auto &m : meta) meta_ptrs.push_back(&m);
        Op step_op = step.op;
        std::vector<TypedFixedShape> step_shapes;
        ShapeError serr;
        if (!compute_output_shapes(model_, step_op, meta_ptrs, 1, &step_shapes, &serr)) return fail(err, SessionError::Shape, serr.message);
        Node step_node(step_op);
        step_node.inputs = step.inputs;
        step_node.outputs = step.outputs;
        std::vector<DeviceTensor> step_outs;
        if (!run_device_op(step_node, step_op, ins, step_shapes, &step_outs, err)) return false;
        if (step_outs.empty()) return fail(err, SessionError::Message, "FusedElemwise: a step produced nothing");
        prev = std::move(step_outs[0]);  // the previous intermediate goes back to the pool; stream order keeps it readable
        have_prev = true;
        prev_id = step.outputs[0];
    }
    outs->push_back(std::move(prev));
    return true;
}

bool HipSession::run_device_op(const Node &node, const Op &op, const std::vector<DeviceTensor *> &in,
                               const std::vector<TypedFixedShape> &shapes, std::vector<DeviceTensor> *outs, SessionError *err) {
    struct LazyName {  // the operator's name, made where a message needs it
        const Op &op;
        std::string operator+(const char *rest) const { return std::string(op.name()) + rest; }
        std::string operator+(const std::string &rest) const { return std::string(op.name()) + rest; }
    } opname{op};
    auto need = [&](size_t n) {
        if (in.size() >= n) {
            bool all = true;
            for (size_t i = 0; i < n; i++) all = all && in[i];
            if (all) return true;
        }
        return fail(err, SessionError::Message, opname + ": expected " + std::to_string(n) + " inputs");
    };
    auto need_f32 = [&](std::initializer_list<size_t> which) {
        for (size_t i : which)
            if (in[i]->elem_ty != TensorElemType::F32)
                return fail(err, SessionError::Message,
                            opname + ": input type " + elem_name(in[i]->elem_ty) + " is not supported (f32 only)");
        return true;
    };
    auto f = [](const DeviceTensor *d) { return static_cast<const float *>(d->ptr); };
    auto esize = [](const DeviceTensor *d) { return (int)elem_size(d->elem_ty); };
    auto i64v = [](const FixedDimensions &d) {
        std::vector<int64_t> v;
        for (auto x : d.as_vec()) v.push_back((int64_t)x);
        return v;
    };
    auto done = [&](int rc) { return rc ? fail_code(err, rc, ctx_.last_error) : true; };

    if (op.kind == OpKind::FusedElemwise) return run_fused_elemwise(node, op, in, shapes, outs, err);

    // Split produces one tensor per part; everything else one output.
    if (op.kind == OpKind::Split) {
        if (!need(1)) return false;
        const size_t rank = in[0]->dims.len();
        const size_t axis = (size_t)(op.axis < 0 ? op.axis + (int64_t)rank : op.axis);
        const std::vector<int64_t> in_str = strides_of(*in[0]);  // a view's own strides
        size_t start = 0;
        for (size_t p = 0; p < node.outputs.size(); p++) {
            DeviceTensor o;
            if (!allocate(shapes[p], &o, err)) return false;
            const std::vector<int64_t> d = i64v(o.dims), os = i64v(o.dims.strides());
            const char *src = static_cast<const char *>(in[0]->ptr) + start * (size_t)in_str[axis] * (size_t)esize(in[0]);
            if (!done(launch_copy_strided(ctx_, o.ptr, src, esize(in[0]), (int)rank, d.data(), os.data(), in_str.data()))) return false;
            start += o.dims[axis];
            outs->push_back(std::move(o));
        }
        return true;
    }

    if (op.kind == OpKind::MatMul && attn_head_.count(current_node_)) {
        const size_t before = outs->size();
        if (!try_defer_attention(node, op, in, shapes, outs, err)) return false;
        if (outs->size() > before) return true;  // deferred; otherwise this product runs as usual
    }

    DeviceTensor out;
    if (!allocate(shapes[0], &out, err)) return false;
    float *o = static_cast<float *>(out.ptr);
    const size_t n_out = out.dims.total_elems();
    int rc = AHIP_OK;

    switch (op.kind) {
    case OpKind::Identity:
        if (!need(1)) return false;
        if (out.nbytes())
            rc = ctx_.check(hipMemcpyAsync(out.ptr, in[0]->ptr, out.nbytes(), hipMemcpyDeviceToDevice, ctx_.stream), "hipMemcpyAsync(Identity)");
        break;
    case OpKind::Add:
    case OpKind::Sub:
    case OpKind::Mul:
    case OpKind::Div:
    case OpKind::Pow: {
        if (!need(2) || !need_f32({0, 1})) return false;
        auto as = in[0]->dims.strides_for_broadcasting_to(out.dims);
        auto bs = in[1]->dims.strides_for_broadcasting_to(out.dims);
        if (!as || !bs) return fail(err, SessionError::Shape, opname + ": operands do not broadcast to the output shape");
        if (out.dims.len() > (size_t)MAX_RANK) return fail(err, SessionError::Message, opname + ": rank above 8 is not supported");
        const std::vector<int64_t> dims = i64v(out.dims), sa = i64v(*as), sb = i64v(*bs);
        const int bop = op.kind == OpKind::Add   ? AHIP_ADD
                        : op.kind == OpKind::Sub ? AHIP_SUB
                        : op.kind == OpKind::Mul ? AHIP_MUL
                        : op.kind == OpKind::Div ? AHIP_DIV
                                                 : AHIP_POW;
        rc = launch_binary(ctx_, bop, o, f(in[0]), f(in[1]), (int)dims.size(), dims.data(), sa.data(), sb.data());
        break;
    }
    case OpKind::Sqrt:
    case OpKind::ReLU:
    case OpKind::Gelu:
    case OpKind::Sigmoid:
    case OpKind::Erf:
    case OpKind::Tanh:
    case OpKind::Exp:
    case OpKind::Round:
    case OpKind::HardSigmoid:
    case OpKind::LeakyReLU: {
        if (!need(1) || !need_f32({0})) return false;
        int uop = AHIP_SQRT;
        float a = 0, b = 0;
        switch (op.kind) {
        case OpKind::Sqrt: uop = AHIP_SQRT; break;
        case OpKind::ReLU: uop = AHIP_RELU; break;
        case OpKind::Gelu: uop = AHIP_GELU; break;
        case OpKind::Sigmoid: uop = AHIP_SIGMOID; break;
        case OpKind::Erf: uop = AHIP_ERF; break;
        case OpKind::Tanh: uop = AHIP_TANH; break;
        case OpKind::Exp: uop = AHIP_EXP; break;
        case OpKind::Round: uop = AHIP_ROUND; break;
        case OpKind::HardSigmoid: uop = AHIP_HARDSIGMOID; a = op.alpha; b = op.beta; break;
        default: uop = AHIP_LEAKYRELU; a = op.alpha; break;
        }
        rc = launch_unary(ctx_, uop, o, f(in[0]), n_out, a, b);
        break;
    }
    case OpKind::Clip: {  // bounds are optional scalar inputs (opset >= 11); the host needs their values
        if (!need(1) || !need_f32({0})) return false;
        float lo = -std::numeric_limits<float>::infinity(), hi = std::numeric_limits<float>::infinity();
        for (size_t k = 1; k <= 2; k++) {
            if (k >= in.size() || !in[k] || in[k]->dims.total_elems() == 0) continue;
            if (in[k]->elem_ty != TensorElemType::F32 || in[k]->dims.total_elems() != 1)
                return fail(err, SessionError::Message, "Clip: bounds must be f32 scalars");
            if (!fetch_host(in[k], err)) return false;
            (k == 1 ? lo : hi) = *in[k]->host->data_f32();
        }
        rc = launch_unary(ctx_, AHIP_CLIP, o, f(in[0]), n_out, lo, hi);
        break;
    }
    case OpKind::Softmax: {
        if (!need(1) || !need_f32({0})) return false;
        const size_t rank = in[0]->dims.len();
        if (rank == 0) return fail(err, SessionError::Message, "Softmax: rank-0 input");
        if (!(op.axis == -1 || op.axis == (int64_t)rank - 1))  // session.rs:999
            return fail(err, SessionError::Message, "Softmax: only the last axis is supported");
        const size_t len = in[0]->dims[rank - 1];
        const size_t rows = len ? n_out / len : 0;
        if (!op.prologue_scale && !op.prologue_mask) {
            rc = launch_softmax(ctx_, o, f(in[0]), rows, len);
            break;
        }
        // Softmax that absorbed its scale and mask (fuse_softmax_prologue): inputs x, scale?, mask?.
        const size_t n_in = 1 + (op.prologue_scale ? 1 : 0) + (op.prologue_mask ? 1 : 0);
        if (!need(n_in)) return false;
        DeviceTensor *scale_t = op.prologue_scale ? in[1] : nullptr;
        DeviceTensor *mask_t = op.prologue_mask ? in[n_in - 1] : nullptr;
        float scale = 1.0f;
        if (scale_t) {
            if (scale_t->elem_ty != TensorElemType::F32 || scale_t->dims.total_elems() != 1)
                return fail(err, SessionError::Shape, "Softmax: the absorbed scale must be one f32 value");
            if (!fetch_host(scale_t, err)) return false;
            scale = scale_t->host->data_f32()[0];
        }
        size_t rows_per_mask = 0;
        if (mask_t) {
            if (mask_t->elem_ty != TensorElemType::F32) return fail(err, SessionError::Message, "Softmax: the absorbed mask must be f32");
            const size_t m_elems = mask_t->dims.total_elems();
            if (len == 0 || m_elems % len != 0 || m_elems == 0 || rows % (m_elems / len) != 0 ||
                (m_elems / len != 1 && m_elems / len != in[0]->dims[0]))
                return fail(err, SessionError::Shape, "Softmax: the absorbed mask does not fit the scores");
            rows_per_mask = rows / (m_elems / len);
        }
        rc = launch_softmax_prologue(ctx_, o, f(in[0]), rows, len, op.prologue_scale, scale, mask_t ? f(mask_t) : nullptr, rows_per_mask);
        if (rc == AHIP_ERR_UNSUPPORTED) {
            // Geometry the one-kernel route does not take: the same operators one after the other, in place.
            const std::vector<int64_t> xd = i64v(out.dims), xs = i64v(out.dims.strides());
            const std::vector<int64_t> zero(xd.size(), 0);
            const float *cur = f(in[0]);
            rc = AHIP_OK;
            if (scale_t) {
                rc = launch_binary(ctx_, op.prologue_scale == 1 ? AHIP_MUL : AHIP_DIV, o, cur, f(scale_t), (int)xd.size(), xd.data(), xs.data(), zero.data());
                cur = o;
            }
            if (!rc && mask_t) {
                auto ms = mask_t->dims.strides_for_broadcasting_to(out.dims);
                if (!ms) return fail(err, SessionError::Shape, "Softmax: the absorbed mask does not broadcast to the scores");
                const std::vector<int64_t> msv = i64v(*ms);
                rc = launch_binary(ctx_, AHIP_ADD, o, cur, f(mask_t), (int)xd.size(), xd.data(), xs.data(), msv.data());
                cur = o;
            }
            if (!rc) rc = launch_softmax(ctx_, o, cur, rows, len);
        }
        break;
    }
    case OpKind::LayerNormalization: {
        if (!need(3) || !need_f32({0, 1, 2})) return false;
        const size_t rank = in[0]->dims.len();
        if (rank == 0) return fail(err, SessionError::Message, "LayerNormalization: rank-0 input");
        if (!(op.axis == -1 || op.axis == (int64_t)rank - 1))
            return fail(err, SessionError::Message, "LayerNormalization: Axis must be the last dimension.");
        if (op.stash_type != 1) return fail(err, SessionError::Message, "LayerNormalization: Stash type must be 1.");
        const size_t len = in[0]->dims[rank - 1];
        if (in[1]->dims.total_elems() != len || in[2]->dims.total_elems() != len)
            return fail(err, SessionError::Shape, "LayerNormalization: scale and bias must hold one value per column");
        {
            // Read only by a product with a weight matrix that takes the bf16 route: write that product's operand planes.
            auto pp = planes_out_.find(current_node_);
            const size_t rows = len ? n_out / len : 0;
            auto a16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
            if (pp != planes_out_.end() && in[0]->strides.empty() && layernorm_planes_fits(rows, len) && a16(in[0]->ptr) && a16(in[1]->ptr) &&
                a16(in[2]->ptr) && matmul_out_perm_.count(pp->second.consumer) == 0 && gemm_takes_split(ctx_, rows, pp->second.next_n, len)) {
                DeviceTensor planes;
                if (!allocate_bytes(gemm_planes_bytes(rows, len), &planes, err)) return false;
                if (in[0]->owes_add()) {  // the residual Add in front was left to this kernel: it writes the sum too
                    PendingAdd &pa = *in[0]->pending_add;
                    rc = launch_layernorm_planes(ctx_, planes.ptr, static_cast<float *>(in[0]->ptr), pa.a, pa.b, f(in[1]), f(in[2]), rows, len,
                                                 op.epsilon);
                    pa.done = true;
                    pa.a_block.reset();
                    pa.b_block.reset();
                } else {
                    rc = launch_layernorm_planes(ctx_, planes.ptr, nullptr, f(in[0]), nullptr, f(in[1]), f(in[2]), rows, len, op.epsilon);
                }
                out.block = planes.block;  // the fp32 block goes back to the pool unused
                out.ptr = planes.ptr;
                out.planes = true;
                out.planes_rows = rows, out.planes_k = len;
                copies_avoided_++;  // the operand split of the product behind (and the fp32 tensor between them)
                break;
            }
        }
        if (!flush_add(in[0], err)) return false;
        rc = launch_layernorm(ctx_, o, f(in[0]), f(in[1]), f(in[2]), len ? n_out / len : 0, len, op.epsilon);
        break;
    }
    case OpKind::ReduceMean:
    case OpKind::ReduceMax: {
        if (!need(1) || !need_f32({0})) return false;
        const FixedDimensions &d = in[0]->dims;
        const size_t rank = d.len();
        std::vector<size_t> axes;
        if (op.axes.empty()) {
            if (op.kind == OpKind::ReduceMean) {  // nothing is reduced: the output is the input
                if (out.nbytes())
                    rc = ctx_.check(hipMemcpyAsync(out.ptr, in[0]->ptr, out.nbytes(), hipMemcpyDeviceToDevice, ctx_.stream),
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
                if (axes[i] != axes[i - 1] + 1) return fail(err, SessionError::Message, opname + ": reduced axes must be adjacent");
            for (size_t i = 0; i < axes.front(); i++) outer *= d[i];
            for (size_t i = axes.front(); i <= axes.back(); i++) red *= d[i];
            for (size_t i = axes.back() + 1; i < rank; i++) inner *= d[i];
        }
        rc = launch_reduce(ctx_, op.kind == OpKind::ReduceMean ? AHIP_REDUCE_MEAN : AHIP_REDUCE_MAX, o, f(in[0]), outer, red, inner);
        break;
    }
    case OpKind::GlobalAveragePool: {  // sum of each H*W plane, then a true division by H*W (session.rs:265-297)
        if (!need(1) || !need_f32({0})) return false;
        const FixedDimensions &d = in[0]->dims;
        const size_t planes = d[0] * d[1], area = d[2] * d[3];
        if (area == 0) return fail(err, SessionError::Shape, "GlobalAveragePool: empty plane");
        rc = launch_reduce(ctx_, AHIP_REDUCE_SUM, o, f(in[0]), planes, area, 1);
        if (!rc) rc = launch_unary(ctx_, AHIP_DIV_BY, o, o, planes, (float)area, 0);
        break;
    }
    case OpKind::BatchNormalization: {
        if (!need(5) || !need_f32({0, 1, 2, 3, 4})) return false;
        if (op.training_mode) return fail(err, SessionError::Message, "BatchNormalization: Training mode is not supported.");
        const FixedDimensions &d = in[0]->dims;
        if (d.len() < 2) return fail(err, SessionError::Message, "BatchNormalization: input rank must be at least 2");
        const size_t c = d[1];
        for (size_t k = 1; k < 5; k++)
            if (in[k]->dims.total_elems() != c) return fail(err, SessionError::Shape, "BatchNormalization: one value per channel is needed");
        size_t hw = 1;
        for (size_t i = 2; i < d.len(); i++) hw *= d[i];
        rc = launch_batchnorm(ctx_, o, f(in[0]), f(in[1]), f(in[2]), f(in[3]), f(in[4]), d[0], c, hw, op.epsilon);
        break;
    }
    case OpKind::Transpose: {
        if (!need(1)) return false;
        const std::vector<int64_t> d = i64v(in[0]->dims);
        rc = launch_transpose(ctx_, out.ptr, in[0]->ptr, esize(in[0]), (int)d.size(), d.data(), op.perm.data());
        break;
    }
    case OpKind::Concat: {
        if (!need(1)) return false;
        const size_t rank = out.dims.len();
        const size_t axis = (size_t)(op.axis < 0 ? op.axis + (int64_t)rank : op.axis);
        const std::vector<int64_t> out_str = i64v(out.dims.strides());
        size_t at = 0;
        for (auto *t : in) {
            if (!t) return fail(err, SessionError::Message, "Concat: an input value is missing");
            if (t->elem_ty != out.elem_ty) return fail(err, SessionError::Message, "Concat: inputs differ in element type");
            const std::vector<int64_t> d = i64v(t->dims), is = i64v(t->dims.strides());
            char *dst = static_cast<char *>(out.ptr) + at * (size_t)out_str[axis] * (size_t)esize(t);
            rc = launch_copy_strided(ctx_, dst, t->ptr, esize(t), (int)rank, d.data(), out_str.data(), is.data());
            if (rc) break;
            at += t->dims[axis];
        }
        break;
    }
    case OpKind::Slice: {
        if (!need(3)) return false;
        std::vector<int64_t> starts, ends, axes, steps;
        auto read = [&](size_t k, std::vector<int64_t> *v) {
            if (k >= in.size() || !in[k] || in[k]->dims.total_elems() == 0) return true;
            if (!fetch_host(in[k], err)) return false;
            const Tensor &t = *in[k]->host;
            const size_t n = t.dims().total_elems();
            for (size_t i = 0; i < n; i++)
                v->push_back(t.elem_ty() == TensorElemType::I64 ? reinterpret_cast<const int64_t *>(t.data_as_bytes())[i]
                                                                 : (int64_t)reinterpret_cast<const int32_t *>(t.data_as_bytes())[i]);
            return true;
        };
        if (!read(1, &starts) || !read(2, &ends) || !read(3, &axes) || !read(4, &steps)) return false;
        if (axes.empty())
            for (size_t i = 0; i < starts.size(); i++) axes.push_back((int64_t)i);
        if (steps.empty()) steps.assign(starts.size(), 1);
        const FixedDimensions &d = in[0]->dims;
        std::vector<int64_t> in_str = i64v(d.strides());
        const std::vector<int64_t> base_str = in_str;
        size_t base = 0;
        for (size_t i = 0; i < starts.size(); i++) {
            const size_t ax = (size_t)(axes[i] < 0 ? axes[i] + (int64_t)d.len() : axes[i]);
            const int64_t n = (int64_t)d[ax];
            int64_t s = starts[i] < 0 ? starts[i] + n : starts[i];
            s = std::min(std::max<int64_t>(s, 0), n);
            base += (size_t)s * (size_t)base_str[ax];
            in_str[ax] = base_str[ax] * steps[i];
        }
        const std::vector<int64_t> od = i64v(out.dims), os = i64v(out.dims.strides());
        const char *src = static_cast<const char *>(in[0]->ptr) + base * (size_t)esize(in[0]);
        rc = launch_copy_strided(ctx_, out.ptr, src, esize(in[0]), (int)od.size(), od.data(), os.data(), in_str.data());
        break;
    }
    case OpKind::Expand: {
        if (!need(1)) return false;
        auto is = in[0]->dims.strides_for_broadcasting_to(out.dims);
        if (!is) return fail(err, SessionError::Shape, "Expand: the input does not broadcast to the output shape");
        const std::vector<int64_t> od = i64v(out.dims), os = i64v(out.dims.strides()), ist = i64v(*is);
        rc = launch_copy_strided(ctx_, out.ptr, in[0]->ptr, esize(in[0]), (int)od.size(), od.data(), os.data(), ist.data());
        break;
    }
    case OpKind::Tile: {  // each axis becomes (repeat, extent) with stride 0 on the repeat
        if (!need(1)) return false;
        const FixedDimensions &d = in[0]->dims;
        if (d.len() * 2 > (size_t)MAX_RANK) return fail(err, SessionError::Message, "Tile: rank above 4 is not supported");
        std::vector<int64_t> dims, os, is;
        const std::vector<int64_t> in_str = i64v(d.strides()), out_str = i64v(out.dims.strides());
        for (size_t i = 0; i < d.len(); i++) {
            const int64_t reps = d[i] ? (int64_t)(out.dims[i] / d[i]) : 0;
            dims.push_back(reps);
            os.push_back(out_str[i] * (int64_t)d[i]);
            is.push_back(0);
            dims.push_back((int64_t)d[i]);
            os.push_back(out_str[i]);
            is.push_back(in_str[i]);
        }
        rc = launch_copy_strided(ctx_, out.ptr, in[0]->ptr, esize(in[0]), (int)dims.size(), dims.data(), os.data(), is.data());
        break;
    }
    case OpKind::Gather: {
        if (!need(2)) return false;
        if (in[1]->elem_ty != TensorElemType::I64 && in[1]->elem_ty != TensorElemType::I32)
            return fail(err, SessionError::Message, "Gather: indices must be i32 or i64");
        const size_t rank = in[0]->dims.len();
        const size_t axis = (size_t)(op.axis < 0 ? op.axis + (int64_t)rank : op.axis);
        size_t outer, len, inner;
        split_at(in[0]->dims, axis, &outer, &len, &inner);
        ctx_.flags_armed = true;
        rc = launch_gather(ctx_, out.ptr, in[0]->ptr, in[1]->ptr, esize(in[1]), esize(in[0]), outer, len, in[1]->dims.total_elems(), inner,
                           ctx_.flags);
        break;
    }
    case OpKind::Where: {
        if (!need(3)) return false;
        if (in[0]->elem_ty != TensorElemType::Bool) return fail(err, SessionError::Message, "Where: the condition must be bool");
        if (in[1]->elem_ty != in[2]->elem_ty) return fail(err, SessionError::Message, "Where: x and y differ in element type");
        auto cs = in[0]->dims.strides_for_broadcasting_to(out.dims), xs = in[1]->dims.strides_for_broadcasting_to(out.dims),
             ys = in[2]->dims.strides_for_broadcasting_to(out.dims);
        if (!cs || !xs || !ys) return fail(err, SessionError::Shape, "Where: operands do not broadcast to the output shape");
        const std::vector<int64_t> d = i64v(out.dims), c = i64v(*cs), x = i64v(*xs), y = i64v(*ys);
        rc = launch_where(ctx_, out.ptr, in[0]->ptr, in[1]->ptr, in[2]->ptr, esize(in[1]), (int)d.size(), d.data(), c.data(), x.data(), y.data());
        break;
    }
    case OpKind::Greater: {
        if (!need(2) || !need_f32({0, 1})) return false;
        auto as = in[0]->dims.strides_for_broadcasting_to(out.dims), bs = in[1]->dims.strides_for_broadcasting_to(out.dims);
        if (!as || !bs) return fail(err, SessionError::Shape, "Greater: operands do not broadcast to the output shape");
        const std::vector<int64_t> d = i64v(out.dims), a = i64v(*as), b = i64v(*bs);
        rc = launch_greater(ctx_, static_cast<uint8_t *>(out.ptr), f(in[0]), f(in[1]), (int)d.size(), d.data(), a.data(), b.data());
        break;
    }
    case OpKind::Cast:
        if (!need(1)) return false;
        rc = launch_cast(ctx_, out.ptr, in[0]->ptr, (int)in[0]->elem_ty, (int)out.elem_ty, n_out);
        break;
    case OpKind::Conv2d: {  // conv2d::compute (conv2d.rs:26-211)
        if (!need(2) || !need_f32({0, 1})) return false;
        const FixedDimensions &x = in[0]->dims, &w = in[1]->dims;
        if (x.len() != 4 || w.len() != 4 || op.padding.size() != 4) return fail(err, SessionError::Shape, "Conv2d: four-dimensional input, weight and padding are needed");
        const size_t group = (size_t)op.group;
        if (group == 0 || x[1] % group || w[0] % group || w[1] != x[1] / group || w[2] != (size_t)op.kernel_shape[0] || w[3] != (size_t)op.kernel_shape[1])
            return fail(err, SessionError::Shape, "Conv2d: weight " + w.to_string() + " does not fit input " + x.to_string() + " with group " + std::to_string(group));
        const float *bias = nullptr;
        if (in.size() > 2 && in[2]) {
            if (in[2]->elem_ty != TensorElemType::F32 || in[2]->dims.total_elems() != w[0]) return fail(err, SessionError::Shape, "Conv2d: bias must hold one f32 per output channel");
            bias = f(in[2]);
        }
        DeviceTensor col;
        const size_t oh = out.dims[2], ow = out.dims[3];
        if (!allocate(TypedFixedShape{FixedDimensions({x[0], x[1], w[2], w[3], oh, ow}), TensorElemType::F32}, &col, err)) return false;
        rc = launch_conv2d(ctx_, o, f(in[0]), f(in[1]), bias, static_cast<float *>(col.ptr), x[0], x[1], x[2], x[3], w[0], oh, ow, w[2], w[3],
                           (size_t)op.strides[0], (size_t)op.strides[1], (size_t)op.dilations[0], (size_t)op.dilations[1],
                           (size_t)op.padding[0], (size_t)op.padding[1], group);
        break;  // `col` goes back to the pool here; stream order keeps it intact until the GEMMs have read it
    }
    case OpKind::MaxPool: {  // compute_max_pool (session.rs:324-382)
        if (!need(1) || !need_f32({0})) return false;
        const FixedDimensions &x = in[0]->dims;
        if (x.len() != 4 || op.padding.size() != 4) return fail(err, SessionError::Shape, "MaxPool: four-dimensional input and padding are needed");
        rc = launch_maxpool(ctx_, o, f(in[0]), x[0] * x[1], x[2], x[3], out.dims[2], out.dims[3], (size_t)op.kernel_shape[0],
                            (size_t)op.kernel_shape[1], (size_t)op.strides[0], (size_t)op.strides[1], (size_t)op.padding[0], (size_t)op.padding[1]);
        break;
    }
    case OpKind::Resize: {  // compute_resize (session.rs:1056-1132): batch and channels keep their extents
        if (!need(1) || !need_f32({0})) return false;
        const FixedDimensions &x = in[0]->dims;
        if (x.len() != 4 || out.dims[0] != x[0] || out.dims[1] != x[1])
            return fail(err, SessionError::Message, "Resize: only the two spatial axes of an NCHW tensor can be resized");
        rc = launch_resize(ctx_, o, f(in[0]), x[0] * x[1], x[2], x[3], out.dims[2], out.dims[3], op.mode == "nearest");
        break;
    }
    case OpKind::MatMul: {  // compute_mat_mul (session.rs:621-684), with NumPy broadcasting of the batch axes
        if (!need(2) || !need_f32({0, 1})) return false;
        // An operand may be a strided view (a head of a [b, t, h, d] tensor taken by Split / Reshape /
        // Transpose without a copy).  Its matrix must have one unit stride; a unit row stride means the
        // stored matrix is the transposed one.  A view the kernel's addressing cannot express is copied.
        if (in[0]->dims.len() < 2 || in[1]->dims.len() < 2) return fail(err, SessionError::Shape, "MatMul: operands of rank < 2");
        if (in[0]->pending_op == PENDING_ATTENTION) {  // the second product of a deferred attention: everything happens here
            if (!run_attention_tail(op, in, &out, err)) return false;
            break;
        }
        if (in[0]->planes) {
            // The first operand arrives as the planes the LayerNormalization in front wrote: [rows, k] x weights [k, n] on the bf16 route.
            const FixedDimensions &ad = in[0]->dims, &bdm = in[1]->dims;
            size_t rows = 1;
            for (size_t i = 0; i + 1 < ad.len(); i++) rows *= ad[i];
            const size_t kk = ad[ad.len() - 1];
            if (op.trans_a || bdm.len() != 2 || !in[1]->strides.empty() || matmul_out_perm_.count(current_node_) ||
                (op.trans_b ? bdm[1] : bdm[0]) != kk || in[0]->planes_rows != rows || in[0]->planes_k != kk)
                return fail(err, SessionError::Message, "internal: operand planes reached a product of another form");
            const size_t nn = op.trans_b ? bdm[0] : bdm[1];
            const float *bias_p = nullptr;
            if (in.size() > 2 && in[2]) {
                if (in[2]->elem_ty != TensorElemType::F32 || in[2]->dims.total_elems() != nn)
                    return fail(err, SessionError::Shape, "MatMul: the absorbed bias must hold one f32 value per output column");
                bias_p = f(in[2]);
            }
            rc = launch_gemm_split(ctx_, o, nullptr, f(in[1]), bias_p, rows, nn, kk, 0, op.trans_b ? 1 : 0, kk, op.trans_b ? kk : nn, nn, 0, 1, 1.0f,
                                   bias_p ? 1.0f : 0.0f, 0, in[0]->ptr);
            break;
        }
        // The activation the first operand still owes is folded into the bf16 route's operand split when this
        // product is one tall sgemm that takes that route; otherwise it runs now.
        int a_op = 0;
        if (in[0]->pending_op >= 0) {
            const FixedDimensions &ad = in[0]->dims, &bdm = in[1]->dims;
            size_t rows = 1;
            for (size_t i = 0; i + 1 < ad.len(); i++) rows *= ad[i];
            const bool tall = !op.trans_a && bdm.len() == 2 && in[0]->strides.empty() && in[1]->strides.empty() &&
                              matmul_out_perm_.count(current_node_) == 0;
            const size_t nn = op.trans_b ? bdm[0] : bdm[1];
            if (tall && gemm_takes_split(ctx_, rows, nn, ad[ad.len() - 1])) {
                a_op = in[0]->pending_op;
            } else if (!apply_pending(in[0], err)) {
                return false;
            }
        }
        MatOperand A, B;
        if (!describe_operand(in[0], &A, err) || !describe_operand(in[1], &B, err)) return false;
        // trans_a / trans_b (fuse_transpose_matmul): the logical operand is the transpose of the tensor.
        const int ta = (op.trans_a ? 1 : 0) ^ (A.stored_transposed ? 1 : 0), tb = (op.trans_b ? 1 : 0) ^ (B.stored_transposed ? 1 : 0);
        const size_t m = op.trans_a ? A.cols : A.rows, k = op.trans_a ? A.rows : A.cols;
        const size_t n = op.trans_b ? B.rows : B.cols;
        size_t batch = 1;
        std::vector<size_t> bd;
        for (size_t i = 0; i + 2 < out.dims.len(); i++) batch *= out.dims[i], bd.push_back(out.dims[i]);
        // A third input is a bias row absorbed by fuse_matmul_bias: added in the epilogue (1 * acc + 1 * bias,
        // the one addition the separate Add performs).
        const float *bias = nullptr;
        if (in.size() > 2 && in[2]) {
            if (in[2]->elem_ty != TensorElemType::F32 || in[2]->dims.total_elems() != n)
                return fail(err, SessionError::Shape, "MatMul: the absorbed bias must hold one f32 value per output column");
            bias = f(in[2]);
        }
        const float beta = bias ? 1.0f : 0.0f;
        // The result in the layout of the Transpose that reads it (plan_views): the buffer is dense in the
        // transposed shape, and this node's value is a view of it.
        std::vector<int64_t> c_str = dense_strides(out.dims);
        auto pv = matmul_out_perm_.find(current_node_);
        if (pv != matmul_out_perm_.end() && pv->second.size() == out.dims.len()) {
            FixedDimensions td = out.dims;
            for (size_t i = 0; i < td.len(); i++) td[i] = out.dims[(size_t)pv->second[i]];
            const std::vector<int64_t> ts = dense_strides(td);
            for (size_t i = 0; i < td.len(); i++) c_str[(size_t)pv->second[i]] = ts[i];
            if (!is_dense(out.dims, c_str)) out.strides = c_str;
        }
        const bool plain = in[0]->strides.empty() && in[1]->strides.empty() && out.strides.empty();
        if (plain && B.batch == 1 && A.batch == batch && !ta) {
            // [.., m, k] x [k, n]: one tall sgemm, as the reference does (session.rs:653-660)
            // On the fp32 kernel, the activation or the residual Add behind the product is done as it is written.
            auto mp = matmul_post_.find(current_node_);
            if (!a_op && mp != matmul_post_.end() && !gemm_takes_split(ctx_, batch * m, n, k)) {
                GemmPost post;
                if (mp->second.act) {
                    post.act = mp->second.act;
                } else if (mp->second.has_add && values_) {
                    const DeviceTensor *x = nullptr;
                    auto xv = values_->find(mp->second.residual);
                    if (xv != values_->end()) x = &xv->second;
                    else if (auto xi = inits_.find(mp->second.residual); xi != inits_.end()) x = &xi->second;
                    if (x && x->ptr && x->elem_ty == TensorElemType::F32 && x->strides.empty() && x->pending_op < 0 && x->applied_op < 0 &&
                        x->dims == out.dims)
                        post.residual = static_cast<const float *>(x->ptr);
                }
                if (post.act || post.residual) {
                    const size_t none[2] = {0, 0};
                    rc = launch_gemm_batch2(ctx_, o, f(in[0]), f(in[1]), bias, 1, 1, batch * m, n, k, 0, tb, A.ld, B.ld, n, none, none, none, 0, 1, 1.0f,
                                            beta, &post);
                    if (!rc && post.act) out.applied_op = post.act;
                    if (!rc && post.residual) absorbed_add_[mp->second.add_node] = mp->second.add_input;
                    break;
                }
            }
            if (a_op) rc = launch_gemm_split(ctx_, o, f(in[0]), f(in[1]), bias, batch * m, n, k, 0, tb, A.ld, B.ld, n, 0, 1, 1.0f, beta, a_op);
            else rc = launch_gemm(ctx_, o, f(in[0]), f(in[1]), bias, 1, batch * m, n, k, 0, tb, A.ld, B.ld, n, 0, 0, 0, 0, 1, 1.0f, beta);
            break;
        }
        if (a_op) return fail(err, SessionError::Message, "MatMul: an activation was left pending on a product that cannot fold it");
        if (out.dims.len() < 2) return fail(err, SessionError::Shape, "MatMul: result of rank < 2");
        if (!((A.batch == batch || A.batch == 1) && (B.batch == batch || B.batch == 1)))
            return fail(err, SessionError::Message, "MatMul: batch axes that broadcast against each other partially are not supported");
        // Batch strides per output batch axis for each operand (0 = shared); a dense operand counts its
        // matrices in the output's batch order whatever its own leading shape.
        auto batch_strides = [&](const MatOperand &x, const DeviceTensor *t, std::vector<int64_t> *s) -> bool {
            s->assign(bd.size(), 0);
            if (x.batch == 1) return true;
            if (t->strides.empty()) {
                int64_t acc = (int64_t)(x.rows * x.cols);
                for (size_t i = bd.size(); i-- > 0;) (*s)[i] = acc, acc *= (int64_t)bd[i];
                return true;
            }
            if (x.bdims != bd) return false;
            *s = x.bstr;
            return true;
        };
        std::vector<int64_t> as, bs;
        for (int attempt = 0;; attempt++) {
            const std::vector<int64_t> cs(c_str.begin(), c_str.begin() + (long)bd.size());
            const size_t ldc = out.dims[out.dims.len() - 2] > 1 ? (size_t)c_str[out.dims.len() - 2] : n;
            bool ok = batch_strides(A, in[0], &as) && batch_strides(B, in[1], &bs);
            std::vector<size_t> d = bd;
            std::vector<int64_t> sa = as, sb = bs, sc = cs;
            if (ok) {
                // Drop axes of extent 1, then fold neighbours that every operand strides uniformly.
                for (size_t i = d.size(); i-- > 0;)
                    if (d[i] == 1) d.erase(d.begin() + (long)i), sa.erase(sa.begin() + (long)i), sb.erase(sb.begin() + (long)i), sc.erase(sc.begin() + (long)i);
                for (size_t i = d.size(); i-- > 1;) {
                    auto folds = [&](const std::vector<int64_t> &v) { return v[i - 1] == (int64_t)d[i] * v[i]; };
                    if (folds(sa) && folds(sb) && folds(sc)) {
                        d[i - 1] *= d[i];
                        sa[i - 1] = sa[i], sb[i - 1] = sb[i], sc[i - 1] = sc[i];
                        d.erase(d.begin() + (long)i), sa.erase(sa.begin() + (long)i), sb.erase(sb.begin() + (long)i), sc.erase(sc.begin() + (long)i);
                    }
                }
                ok = d.size() <= 2;
            }
            if (ok) {
                while (d.size() < 2) d.push_back(1), sa.push_back(0), sb.push_back(0), sc.push_back(0);
                const size_t a2[2] = {(size_t)sa[0], (size_t)sa[1]}, b2[2] = {(size_t)sb[0], (size_t)sb[1]}, c2[2] = {(size_t)sc[0], (size_t)sc[1]};
                rc = launch_gemm_batch2(ctx_, o, f(in[0]), f(in[1]), bias, d[0], d[1], m, n, k, ta, tb, A.ld, B.ld, ldc, a2, b2, c2, 0, 1, 1.0f, beta);
                break;
            }
            // Not expressible: dense copies of the operands and a dense result instead.
            if (attempt > 0 || (in[0]->strides.empty() && in[1]->strides.empty() && out.strides.empty()))
                return fail(err, SessionError::Message, "MatMul: more than two independent batch axes");
            if (!materialize(in[0], err) || !materialize(in[1], err)) return false;
            if (!describe_operand(in[0], &A, err) || !describe_operand(in[1], &B, err)) return false;
            out.strides.clear();
            c_str = dense_strides(out.dims);
        }
        break;
    }
    case OpKind::Gemm: {  // compute_gemm (session.rs:686-794)
        if (!need(2) || !need_f32({0, 1})) return false;
        const FixedDimensions &a = in[0]->dims, &b = in[1]->dims;
        const size_t m = op.trans_a ? a[1] : a[0], k = op.trans_a ? a[0] : a[1], n = op.trans_b ? b[0] : b[1];
        const float *c0 = nullptr;
        size_t rs = 0, cs = 0;
        if (in.size() > 2 && in[2]) {
            if (in[2]->elem_ty != TensorElemType::F32) return fail(err, SessionError::Message, "Gemm: C must be f32");
            auto st = in[2]->dims.strides_for_broadcasting_to(out.dims);
            if (!st) return fail(err, SessionError::Shape, "Gemm: C does not broadcast to the output");
            rs = (*st)[0];
            cs = (*st)[1];
            c0 = f(in[2]);
        }
        rc = launch_gemm(ctx_, o, f(in[0]), f(in[1]), c0, 1, m, n, k, op.trans_a, op.trans_b, a[1], b[1], n, 0, 0, 0, rs, cs, op.alpha,
                         c0 ? op.beta : 0.0f);
        break;
    }
    default: return fail(err, SessionError::Message, opname + ": Kernel not implemented");
    }
    if (rc) return fail_code(err, rc, ctx_.last_error);
    outs->push_back(std::move(out));
    return true;
}

}  // namespace altius
