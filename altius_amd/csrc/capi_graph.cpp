// C ABI: graph IR, analysis, fusion passes, host tensors and the session.
#include <condition_variable>
#include <cstring>
#include <mutex>
#include <new>
#include <string>

#include "../../include/altius_hip.h"
#include "core/model.h"
#include "core/optimize.h"
#include "core/shape.h"
#include "capi_guard.h"
#include "device/ctx.h"
#include "device/host_pool.h"
#include "onnx/load.h"
#include "session/hip_session.h"
#include "session/plan.h"

using namespace altius;

struct ahip_model {
    Model m;
};
struct ahip_tensor {
    Tensor t;
};
struct ahip_session_builder {
    Model model;
    size_t threads = 1;
    bool profiling = false;
    int device = 0;
    bool graph_replay = false;
    int gemm_algorithm = AHIP_GEMM_FP32;
    bool strided_views = true;
    bool fused_attention = false;
    bool device_timing = true;
};
// InterpreterSession::run takes &self and keeps its intermediates in a map per calling thread
// (crates/session_interpreter/src/session.rs:56,75-78), so several threads may run one session at once.  Here a
// HipSession is one stream, one buffer pool and one set of uploaded initializers, used by one call at a time; a
// session therefore holds several of them ("lanes"): lane 0 is built with the session, further ones from the same
// model and switches the first time a call finds every lane busy.
constexpr size_t MAX_LANES = 16;
struct ahip_session {
    std::shared_ptr<HipSession> s;  // lane 0; shared with the device tensors the session has handed out
    ahip_model view;  // what ahip_session_model hands out (a copy of the session's model)
    std::vector<std::pair<std::string, double>> profile;
    ahip_session_builder settings;                    // to build further lanes (its model is left empty: `view` holds it)
    std::mutex lanes_mutex;                           // guards lanes, busy, building and profile
    std::condition_variable lane_freed;
    std::vector<std::shared_ptr<HipSession>> lanes;   // lanes[0] == s
    std::vector<bool> busy;
    size_t last_lane = 0;                             // the lane that served the call that finished last: the statistics read it
    bool lanes_full = false;                          // a further lane could not be built (memory): concurrent calls wait instead
    size_t building = 0;                              // lanes under construction
};

namespace {

int fail(int code, const std::string &msg);

// A lane nobody is using: a free one, a newly built one while fewer than MAX_LANES exist, else whichever frees up first.
// The lane comes back as a pointer of its own, since another thread may grow `lanes` while this one runs.
int acquire_lane(ahip_session *session, size_t *index, std::shared_ptr<HipSession> *lane_out) {
    std::unique_lock<std::mutex> lock(session->lanes_mutex);
    for (;;) {
        for (size_t i = 0; i < session->lanes.size(); i++)
            if (!session->busy[i]) {
                session->busy[i] = true;
                *index = i;
                *lane_out = session->lanes[i];
                return AHIP_OK;
            }
        if (!session->lanes_full && session->lanes.size() + session->building < MAX_LANES) break;
        session->lane_freed.wait(lock);
    }
    session->building++;
    lock.unlock();
    const ahip_session_builder &b = session->settings;
    HipSessionBuilder hb(session->view.m);
    hb.with_intra_op_num_threads(b.threads).with_profiling_enabled(b.profiling).with_device(b.device).with_graph_replay(b.graph_replay).with_device_timing(b.device_timing)
        .with_gemm_algorithm(b.gemm_algorithm).with_strided_views(b.strided_views).with_fused_attention(b.fused_attention);
    SessionError err;
    std::shared_ptr<HipSession> lane;
    try {
        lane = hb.build(&err);
    } catch (...) {
        lock.lock();
        session->building--;
        session->lane_freed.notify_all();
        throw;
    }
    lock.lock();
    session->building--;
    if (!lane) {
        // Every lane holds its own copy of the weights: the GPU may simply have no room for another.  The lanes that
        // exist still serve every call, one after the other.
        session->lanes_full = true;
        session->lane_freed.notify_all();
        for (;;) {
            for (size_t i = 0; i < session->lanes.size(); i++)
                if (!session->busy[i]) {
                    session->busy[i] = true;
                    *index = i;
                    *lane_out = session->lanes[i];
                    return AHIP_OK;
                }
            session->lane_freed.wait(lock);
        }
    }
    session->lanes.push_back(lane);
    session->busy.push_back(true);
    *index = session->lanes.size() - 1;
    *lane_out = std::move(lane);
    return AHIP_OK;
}

// The lane whose run finished last, for the statistics calls.  A lane that is running is waited for: its counters
// are written by the run.
std::shared_ptr<HipSession> last_lane_idle(const ahip_session *session_c) {
    ahip_session *session = const_cast<ahip_session *>(session_c);
    std::unique_lock<std::mutex> lock(session->lanes_mutex);
    while (session->busy[session->last_lane]) session->lane_freed.wait(lock);
    return session->lanes[session->last_lane];
}

// The device-resident calls keep their tensors in lane 0's pool and order their work on lane 0's stream.
void acquire_first_lane(ahip_session *session) {
    std::unique_lock<std::mutex> lock(session->lanes_mutex);
    while (session->busy[0]) session->lane_freed.wait(lock);
    session->busy[0] = true;
}

void release_lane(ahip_session *session, size_t index, bool keep_profile) {
    std::lock_guard<std::mutex> lock(session->lanes_mutex);
    if (keep_profile) session->profile.assign(session->lanes[index]->last_profile().begin(), session->lanes[index]->last_profile().end());
    session->busy[index] = false;
    session->last_lane = index;
    session->lane_freed.notify_all();
}

}  // namespace

struct ahip_device_tensor {
    DeviceTensor t;
    std::shared_ptr<HipSession> owner;  // keeps the pool (and the device context) alive
    ~ahip_device_tensor() {
        if (owner) owner->release(&t);
    }
};

namespace {

int fail(int code, const std::string &msg) {
    set_global_error(msg);
    return code;
}

bool valid_elem_type(int t) { return t >= AHIP_BOOL && t <= AHIP_I64; }

Op op_from_c(int kind, const ahip_op_attrs *a, int64_t opset_version) {
    Op op(static_cast<OpKind>(kind));
    if (!a) {
        // No attribute block: the operator starts from the defaults the ONNX loader gives it
        // (Gemm alpha = beta = 1, LeakyRelu alpha = 0.01, Flatten axis = 1, ...).
        const char *onnx = onnx_type_of(op.kind);
        if (onnx) op_from_onnx_type(onnx, opset_version, &op);
        return op;
    }
    op.axis = a->axis;
    op.axes.assign(a->axes, a->axes + (a->n_axes < 0 ? 0 : a->n_axes > AHIP_MAX_RANK ? AHIP_MAX_RANK : a->n_axes));
    op.keep_dims = a->keep_dims != 0;
    op.alpha = a->alpha;
    op.beta = a->beta;
    op.epsilon = a->epsilon;
    op.stash_type = a->stash_type;
    return op;
}

void op_to_c(const Op &op, ahip_op_attrs *a) {
    ahip_op_attrs_default(a);
    a->axis = op.axis;
    a->n_axes = (int32_t)std::min<size_t>(op.axes.size(), AHIP_MAX_RANK);
    for (int i = 0; i < a->n_axes; i++) a->axes[i] = op.axes[i];
    a->keep_dims = op.keep_dims ? 1 : 0;
    a->alpha = op.alpha;
    a->beta = op.beta;
    a->epsilon = op.epsilon;
    a->stash_type = op.stash_type;
}

bool valid_value(const ahip_model *m, int64_t id) { return id >= 0 && (size_t)id < m->m.graph.values.size(); }

template <class F> int run_pass(ahip_model *model, int *count, F pass, const char *name) try {
    if (!model) return fail(AHIP_ERR_ARG, std::string(name) + ": null model");
    const size_t n = pass(model->m);
    if (count) *count = (int)n;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary(name);
}

}  // namespace

extern "C" {

void ahip_op_attrs_default(ahip_op_attrs *a) {
    if (!a) return;
    std::memset(a, 0, sizeof(*a));
    a->axis = -1;
    a->n_axes = 0;
    a->keep_dims = 1;
    a->alpha = 0.2f;
    a->beta = 0.5f;
    a->epsilon = 1e-5f;
    a->stash_type = 1;
}

const char *ahip_op_name(int op_kind) { return op_kind_name(static_cast<OpKind>(op_kind)); }

int ahip_model_new(int64_t opset_version, ahip_model **model) try {
    if (!model) return fail(AHIP_ERR_ARG, "ahip_model_new: null output pointer");
    *model = new (std::nothrow) ahip_model();
    if (!*model) return fail(AHIP_ERR_OOM, "ahip_model_new: out of host memory");
    (*model)->m.opset_version = opset_version;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_new");
}

int ahip_model_clone(const ahip_model *model, ahip_model **copy) try {
    if (!model || !copy) return fail(AHIP_ERR_ARG, "ahip_model_clone: null argument");
    *copy = new (std::nothrow) ahip_model(*model);
    if (!*copy) return fail(AHIP_ERR_OOM, "ahip_model_clone: out of host memory");
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_clone");
}

void ahip_model_free(ahip_model *model) { delete model; }

int ahip_model_new_value(ahip_model *model, const char *name, int64_t *value_id) try {
    if (!model || !value_id) return fail(AHIP_ERR_ARG, "ahip_model_new_value: null argument");
    *value_id = (int64_t)(name ? model->m.graph.values.new_val_named(name) : model->m.graph.values.new_val());
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_new_value");
}

int ahip_model_new_value_shaped(ahip_model *model, const char *name, int elem_type, int rank, const int64_t *dims,
                                int64_t *value_id) try {
    if (!model || !value_id || rank < 0 || (rank && !dims) || !valid_elem_type(elem_type))
        return fail(AHIP_ERR_ARG, "ahip_model_new_value_shaped: invalid argument");
    std::vector<Dimension> d;
    for (int i = 0; i < rank; i++)
        d.push_back(dims[i] < 0 ? Dimension::Dynamic("dim" + std::to_string(i)) : Dimension::Fixed((size_t)dims[i]));
    TypedShape ts{Dimensions(std::move(d)), static_cast<TensorElemType>(elem_type)};
    *value_id = (int64_t)model->m.graph.values.new_val_named_and_shaped(name ? name : "", std::move(ts));
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_new_value_shaped");
}

int ahip_model_add_initializer(ahip_model *model, int64_t value_id, int elem_type, int rank, const int64_t *dims,
                               const void *data, size_t nbytes) try {
    if (!model || rank < 0 || (rank && !dims) || !valid_elem_type(elem_type) || !valid_value(model, value_id))
        return fail(AHIP_ERR_ARG, "ahip_model_add_initializer: invalid argument");
    for (int i = 0; i < rank; i++)
        if (dims[i] < 0) return fail(AHIP_ERR_ARG, "ahip_model_add_initializer: negative dimension");
    FixedDimensions fd = FixedDimensions::from_i64(dims, (size_t)rank);
    const TensorElemType ty = static_cast<TensorElemType>(elem_type);
    if (nbytes != fd.total_elems() * elem_size(ty) || (nbytes && !data))
        return fail(AHIP_ERR_ARG, "ahip_model_add_initializer: data size does not match the shape");
    model->m.graph.inits[(ValueId)value_id] = Tensor::from_raw(std::move(fd), ty, data, nbytes);
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_add_initializer");
}

int ahip_model_add_node(ahip_model *model, int op_kind, const ahip_op_attrs *attrs, const char *name, int n_inputs,
                        const int64_t *inputs, int n_outputs, const int64_t *outputs, int64_t *node_id) try {
    if (!model || op_kind < 0 || op_kind >= AHIP_OP_COUNT || n_inputs < 0 || n_outputs < 0 ||
        (n_inputs && !inputs) || (n_outputs && !outputs))
        return fail(AHIP_ERR_ARG, "ahip_model_add_node: invalid argument");
    Node node(op_from_c(op_kind, attrs, model->m.opset_version));
    if (name) node.with_name(name);
    for (int i = 0; i < n_inputs; i++) {
        if (!valid_value(model, inputs[i])) return fail(AHIP_ERR_ARG, "ahip_model_add_node: unknown input value");
        node.with_in((ValueId)inputs[i]);
    }
    for (int i = 0; i < n_outputs; i++) {
        if (!valid_value(model, outputs[i])) return fail(AHIP_ERR_ARG, "ahip_model_add_node: unknown output value");
        node.with_out((ValueId)outputs[i]);
    }
    const NodeId id = model->m.graph.add_node(std::move(node));
    if (node_id) *node_id = (int64_t)id;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_add_node");
}

int ahip_model_add_input(ahip_model *model, int64_t value_id) try {
    if (!model || !valid_value(model, value_id)) return fail(AHIP_ERR_ARG, "ahip_model_add_input: invalid argument");
    model->m.graph.inputs.push_back((ValueId)value_id);
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_add_input");
}

int ahip_model_add_output(ahip_model *model, int64_t value_id) try {
    if (!model || !valid_value(model, value_id)) return fail(AHIP_ERR_ARG, "ahip_model_add_output: invalid argument");
    model->m.graph.outputs.push_back((ValueId)value_id);
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_add_output");
}

int ahip_model_lookup_named_value(const ahip_model *model, const char *name, int64_t *value_id) try {
    if (!model || !name || !value_id) return fail(AHIP_ERR_ARG, "ahip_model_lookup_named_value: null argument");
    auto id = model->m.lookup_named_value(name);
    if (!id) return fail(AHIP_ERR_ARG, std::string("no value named '") + name + "'");
    *value_id = (int64_t)*id;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_lookup_named_value");
}

int ahip_model_graph_io(const ahip_model *model, int which, int64_t *value_ids, int capacity, int *n) try {
    if (!model || !n || (which != 0 && which != 1) || capacity < 0 || (capacity && !value_ids))
        return fail(AHIP_ERR_ARG, "ahip_model_graph_io: invalid argument");
    const auto &v = which == 0 ? model->m.graph.inputs : model->m.graph.outputs;
    *n = (int)v.size();
    for (int i = 0; i < capacity && i < (int)v.size(); i++) value_ids[i] = (int64_t)v[i];
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_graph_io");
}

int ahip_model_topo_sort(const ahip_model *model, int64_t *node_ids, int capacity, int *n) try {
    if (!model || !n || capacity < 0 || (capacity && !node_ids))
        return fail(AHIP_ERR_ARG, "ahip_model_topo_sort: invalid argument");
    const auto order = model->m.topo_sort_nodes();
    *n = (int)order.size();
    for (int i = 0; i < capacity && i < (int)order.size(); i++) node_ids[i] = (int64_t)order[i];
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_topo_sort");
}

int ahip_model_node_info(const ahip_model *model, int64_t node_id, int *op_kind, ahip_op_attrs *attrs, int *n_inputs,
                         int64_t *inputs, int *n_outputs, int64_t *outputs, int io_capacity) try {
    if (!model || node_id < 0 || (size_t)node_id >= model->m.graph.nodes.size() || io_capacity < 0)
        return fail(AHIP_ERR_ARG, "ahip_model_node_info: invalid argument");
    const Node &node = model->m.graph.nodes[(size_t)node_id];
    if (op_kind) *op_kind = (int)node.op.kind;
    if (attrs) op_to_c(node.op, attrs);
    if (n_inputs) *n_inputs = (int)node.inputs.size();
    if (n_outputs) *n_outputs = (int)node.outputs.size();
    if (inputs)
        for (int i = 0; i < io_capacity && i < (int)node.inputs.size(); i++) inputs[i] = (int64_t)node.inputs[i];
    if (outputs)
        for (int i = 0; i < io_capacity && i < (int)node.outputs.size(); i++) outputs[i] = (int64_t)node.outputs[i];
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_node_info");
}

int ahip_model_infer_value_shape(const ahip_model *model, int64_t value_id, int *elem_type, int *rank,
                                 int64_t *dims) try {
    if (!model || !rank || !dims || !valid_value(model, value_id))
        return fail(AHIP_ERR_ARG, "ahip_model_infer_value_shape: invalid argument");
    std::map<ValueId, TypedFixedShape> shapes;
    ShapeError err;
    if (!infer_shapes(model->m, nullptr, &shapes, &err)) return fail(AHIP_ERR_SHAPE, err.message);
    auto it = shapes.find((ValueId)value_id);
    if (it == shapes.end()) return fail(AHIP_ERR_ARG, "the shape of this value is not known before run time");
    if (it->second.dims.len() > AHIP_MAX_RANK) return fail(AHIP_ERR_UNSUPPORTED, "rank above AHIP_MAX_RANK");
    if (elem_type) *elem_type = (int)it->second.elem_ty;
    *rank = (int)it->second.dims.len();
    for (size_t i = 0; i < it->second.dims.len(); i++) dims[i] = (int64_t)it->second.dims[i];
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_infer_value_shape");
}

int ahip_model_execution_plan(const ahip_model *model, int64_t *node_ids, int *free_offsets, int node_capacity,
                              int64_t *free_vals, int free_capacity, int *n_nodes, int *n_free) try {
    if (!model || !n_nodes || !n_free || node_capacity < 0 || free_capacity < 0)
        return fail(AHIP_ERR_ARG, "ahip_model_execution_plan: invalid argument");
    const auto plan = create_execution_plan(model->m);
    int nf = 0;
    for (size_t i = 0; i < plan.size(); i++) {
        if ((int)i < node_capacity) {
            if (node_ids) node_ids[i] = (int64_t)plan[i].node_id;
            if (free_offsets) free_offsets[i] = nf;
        }
        for (ValueId v : plan[i].free_vals) {
            if (nf < free_capacity && free_vals) free_vals[nf] = (int64_t)v;
            nf++;
        }
    }
    if (free_offsets && (int)plan.size() <= node_capacity) free_offsets[plan.size()] = nf;
    *n_nodes = (int)plan.size();
    *n_free = nf;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_execution_plan");
}

// ---- ONNX loader, value / node inspection, attributes by name ------------------------------

namespace {

int load_error_code(const ModelLoadError &e) {
    switch (e.kind) {
    case ModelLoadError::Io: return AHIP_ERR_IO;
    case ModelLoadError::Todo: return AHIP_ERR_UNSUPPORTED;
    default: return AHIP_ERR_ARG;
    }
}

Node *live_node(ahip_model *m, int64_t id) {
    if (!m || id < 0 || (size_t)id >= m->m.graph.nodes.size() || m->m.graph.nodes[(size_t)id].deleted) return nullptr;
    return &m->m.graph.nodes[(size_t)id];
}
const Node *live_node_c(const ahip_model *m, int64_t id) { return live_node(const_cast<ahip_model *>(m), id); }

int no_attr(const char *fn, const Node &n, const char *name) {
    return fail(AHIP_ERR_ARG, std::string(fn) + ": " + n.op.name() + " has no attribute '" + name + "' of that kind");
}

}  // namespace

int ahip_model_load_onnx(const char *path, ahip_model **model) try {
    if (!path || !model) return fail(AHIP_ERR_ARG, "ahip_model_load_onnx: null argument");
    *model = nullptr;
    ahip_model *m = new (std::nothrow) ahip_model();
    if (!m) return fail(AHIP_ERR_OOM, "ahip_model_load_onnx: out of host memory");
    ModelLoadError e;
    if (!load_onnx(path, &m->m, &e)) {
        delete m;
        return fail(load_error_code(e), e.to_string());
    }
    *model = m;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_load_onnx");
}

int ahip_model_load_onnx_buffer(const void *data, size_t bytes, ahip_model **model) try {
    if (!model || (!data && bytes)) return fail(AHIP_ERR_ARG, "ahip_model_load_onnx_buffer: null argument");
    *model = nullptr;
    ahip_model *m = new (std::nothrow) ahip_model();
    if (!m) return fail(AHIP_ERR_OOM, "ahip_model_load_onnx_buffer: out of host memory");
    ModelLoadError e;
    if (!load_onnx_from_buffer(data, bytes, &m->m, &e)) {
        delete m;
        return fail(load_error_code(e), e.to_string());
    }
    *model = m;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_load_onnx_buffer");
}

int64_t ahip_model_opset_version(const ahip_model *model) { return model ? model->m.opset_version : -1; }
int64_t ahip_model_num_values(const ahip_model *model) { return model ? (int64_t)model->m.graph.values.size() : -1; }
int64_t ahip_model_num_nodes(const ahip_model *model) { return model ? (int64_t)model->m.graph.nodes.size() : -1; }

int ahip_model_value_info(const ahip_model *model, int64_t value_id, const char **name, int *elem_type, int *rank,
                          int64_t *dims, int dims_capacity) try {
    if (!model || !valid_value(model, value_id) || dims_capacity < 0 || (dims_capacity && !dims))
        return fail(AHIP_ERR_ARG, "ahip_model_value_info: invalid argument");
    const Value &v = model->m.graph.values[(ValueId)value_id];
    if (name) *name = v.name ? v.name->c_str() : nullptr;
    if (!v.shape) {
        if (rank) *rank = -1;
        return AHIP_OK;
    }
    if (elem_type) *elem_type = (int)v.shape->elem_ty;
    const auto &dv = v.shape->dims.as_vec();
    if (rank) *rank = (int)dv.size();
    for (int i = 0; i < dims_capacity && i < (int)dv.size(); i++) dims[i] = dv[(size_t)i].fixed ? (int64_t)dv[(size_t)i].value : -1;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_value_info");
}

int ahip_model_initializer(const ahip_model *model, int64_t value_id, ahip_tensor **tensor) try {
    if (!model || !tensor || !valid_value(model, value_id)) return fail(AHIP_ERR_ARG, "ahip_model_initializer: invalid argument");
    auto it = model->m.graph.inits.find((ValueId)value_id);
    if (it == model->m.graph.inits.end()) return fail(AHIP_ERR_ARG, "ahip_model_initializer: the value has no initializer");
    ahip_tensor *t = new (std::nothrow) ahip_tensor();
    if (!t) return fail(AHIP_ERR_OOM, "ahip_model_initializer: out of host memory");
    t->t = it->second;  // shares the bytes
    *tensor = t;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_model_initializer");
}

const char *ahip_model_node_name(const ahip_model *model, int64_t node_id) {
    const Node *n = live_node_c(model, node_id);
    return n && n->name ? n->name->c_str() : nullptr;
}

int ahip_node_set_attr_int(ahip_model *model, int64_t node_id, const char *name, int64_t value) try {
    Node *n = live_node(model, node_id);
    if (!n || !name) return fail(AHIP_ERR_ARG, "ahip_node_set_attr_int: invalid argument");
    return n->op.set_int(name, value) ? AHIP_OK : no_attr("ahip_node_set_attr_int", *n, name);
} catch (...) {
    return altius::caught_at_boundary("ahip_node_set_attr_int");
}
int ahip_node_set_attr_float(ahip_model *model, int64_t node_id, const char *name, float value) try {
    Node *n = live_node(model, node_id);
    if (!n || !name) return fail(AHIP_ERR_ARG, "ahip_node_set_attr_float: invalid argument");
    return n->op.set_float(name, value) ? AHIP_OK : no_attr("ahip_node_set_attr_float", *n, name);
} catch (...) {
    return altius::caught_at_boundary("ahip_node_set_attr_float");
}
int ahip_node_set_attr_ints(ahip_model *model, int64_t node_id, const char *name, const int64_t *values, int count) try {
    Node *n = live_node(model, node_id);
    if (!n || !name || count < 0 || (count && !values)) return fail(AHIP_ERR_ARG, "ahip_node_set_attr_ints: invalid argument");
    return n->op.set_ints(name, std::vector<int64_t>(values, values + count)) ? AHIP_OK
                                                                               : no_attr("ahip_node_set_attr_ints", *n, name);
} catch (...) {
    return altius::caught_at_boundary("ahip_node_set_attr_ints");
}
int ahip_node_set_attr_string(ahip_model *model, int64_t node_id, const char *name, const char *value) try {
    Node *n = live_node(model, node_id);
    if (!n || !name || !value) return fail(AHIP_ERR_ARG, "ahip_node_set_attr_string: invalid argument");
    return n->op.set_string(name, value) ? AHIP_OK : no_attr("ahip_node_set_attr_string", *n, name);
} catch (...) {
    return altius::caught_at_boundary("ahip_node_set_attr_string");
}
int ahip_node_set_attr_tensor(ahip_model *model, int64_t node_id, const char *name, const ahip_tensor *value) try {
    Node *n = live_node(model, node_id);
    if (!n || !name || !value) return fail(AHIP_ERR_ARG, "ahip_node_set_attr_tensor: invalid argument");
    if (n->op.kind != OpKind::Constant || std::string(name) != "value") return no_attr("ahip_node_set_attr_tensor", *n, name);
    n->op.value = std::make_shared<Tensor>(value->t);
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_node_set_attr_tensor");
}
int ahip_node_get_attr_int(const ahip_model *model, int64_t node_id, const char *name, int64_t *value) try {
    const Node *n = live_node_c(model, node_id);
    if (!n || !name || !value) return fail(AHIP_ERR_ARG, "ahip_node_get_attr_int: invalid argument");
    return n->op.get_int(name, value) ? AHIP_OK : no_attr("ahip_node_get_attr_int", *n, name);
} catch (...) {
    return altius::caught_at_boundary("ahip_node_get_attr_int");
}
int ahip_node_get_attr_float(const ahip_model *model, int64_t node_id, const char *name, float *value) try {
    const Node *n = live_node_c(model, node_id);
    if (!n || !name || !value) return fail(AHIP_ERR_ARG, "ahip_node_get_attr_float: invalid argument");
    return n->op.get_float(name, value) ? AHIP_OK : no_attr("ahip_node_get_attr_float", *n, name);
} catch (...) {
    return altius::caught_at_boundary("ahip_node_get_attr_float");
}
int ahip_node_get_attr_ints(const ahip_model *model, int64_t node_id, const char *name, int64_t *values, int capacity,
                            int *count) try {
    const Node *n = live_node_c(model, node_id);
    if (!n || !name || capacity < 0 || (capacity && !values)) return fail(AHIP_ERR_ARG, "ahip_node_get_attr_ints: invalid argument");
    std::vector<int64_t> v;
    if (!n->op.get_ints(name, &v)) return no_attr("ahip_node_get_attr_ints", *n, name);
    for (int i = 0; i < capacity && i < (int)v.size(); i++) values[i] = v[(size_t)i];
    if (count) *count = (int)v.size();
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_node_get_attr_ints");
}
int ahip_node_get_attr_string(const ahip_model *model, int64_t node_id, const char *name, char *value, int capacity,
                              int *length) try {
    const Node *n = live_node_c(model, node_id);
    if (!n || !name || capacity < 0 || (capacity && !value)) return fail(AHIP_ERR_ARG, "ahip_node_get_attr_string: invalid argument");
    std::string v;
    if (!n->op.get_string(name, &v)) return no_attr("ahip_node_get_attr_string", *n, name);
    if (capacity > 0) {
        const size_t k = std::min<size_t>(v.size(), (size_t)capacity - 1);
        std::memcpy(value, v.data(), k);
        value[k] = 0;
    }
    if (length) *length = (int)v.size();
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_node_get_attr_string");
}
int ahip_node_get_attr_tensor(const ahip_model *model, int64_t node_id, const char *name, ahip_tensor **value) try {
    const Node *n = live_node_c(model, node_id);
    if (!n || !name || !value) return fail(AHIP_ERR_ARG, "ahip_node_get_attr_tensor: invalid argument");
    if (n->op.kind != OpKind::Constant || std::string(name) != "value" || !n->op.value)
        return no_attr("ahip_node_get_attr_tensor", *n, name);
    ahip_tensor *t = new (std::nothrow) ahip_tensor();
    if (!t) return fail(AHIP_ERR_OOM, "ahip_node_get_attr_tensor: out of host memory");
    t->t = *n->op.value;
    *value = t;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_node_get_attr_tensor");
}

int ahip_fuse_layer_norm(ahip_model *model, int *count) { return run_pass(model, count, fuse_layer_norm, "ahip_fuse_layer_norm"); }
int ahip_fuse_gelu(ahip_model *model, int *count) { return run_pass(model, count, fuse_gelu, "ahip_fuse_gelu"); }
int ahip_fuse_fast_gelu(ahip_model *model, int *count) { return run_pass(model, count, fuse_fast_gelu, "ahip_fuse_fast_gelu"); }
int ahip_eliminate_identity(ahip_model *model, int *count) { return run_pass(model, count, eliminate_identity, "ahip_eliminate_identity"); }
int ahip_fuse_transpose_matmul(ahip_model *model, int *count) { return run_pass(model, count, fuse_transpose_matmul, "ahip_fuse_transpose_matmul"); }
int ahip_fuse_matmul_bias(ahip_model *model, int *count) { return run_pass(model, count, fuse_matmul_bias, "ahip_fuse_matmul_bias"); }
int ahip_fuse_softmax_prologue(ahip_model *model, int *count) { return run_pass(model, count, fuse_softmax_prologue, "ahip_fuse_softmax_prologue"); }
int ahip_fuse_elemwise_ops(ahip_model *model, int rule, int *count) try {
    if (!model) return fail(AHIP_ERR_ARG, "ahip_fuse_elemwise_ops: null model");
    if (rule != AHIP_FUSE_REFERENCE_RULE && rule != AHIP_FUSE_EXTENDED_RULE) return fail(AHIP_ERR_ARG, "ahip_fuse_elemwise_ops: unknown rule");
    size_t n = 0;
    std::string msg;
    if (!fuse_elemwise_ops(model->m, static_cast<ElemwiseFusionRule>(rule), &n, &msg)) return fail(AHIP_ERR_SHAPE, msg);
    if (count) *count = (int)n;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_fuse_elemwise_ops");
}

// ---- tensors -----------------------------------------------------------------------

int ahip_tensor_new(int elem_type, int rank, const int64_t *dims, const void *data, size_t nbytes,
                    ahip_tensor **tensor) try {
    if (!tensor || rank < 0 || (rank && !dims) || !valid_elem_type(elem_type))
        return fail(AHIP_ERR_ARG, "ahip_tensor_new: invalid argument");
    for (int i = 0; i < rank; i++)
        if (dims[i] < 0) return fail(AHIP_ERR_ARG, "ahip_tensor_new: negative dimension");
    FixedDimensions fd = FixedDimensions::from_i64(dims, (size_t)rank);
    const TensorElemType ty = static_cast<TensorElemType>(elem_type);
    const size_t want = fd.total_elems() * elem_size(ty);
    if (data && nbytes != want) return fail(AHIP_ERR_ARG, "ahip_tensor_new: data size does not match the shape");
    ahip_tensor *t = new (std::nothrow) ahip_tensor();
    if (!t) return fail(AHIP_ERR_OOM, "ahip_tensor_new: out of host memory");
    // Tensors made here are the ones handed to ahip_session_run: pinned storage when a device is there.
    t->t = data ? Tensor::from_raw(std::move(fd), ty, data, want, altius::pinned_host_block)
                : Tensor::zeros_of_type(ty, std::move(fd), altius::pinned_host_block);
    if (!t->t.has_data()) {
        delete t;
        return fail(AHIP_ERR_OOM, "ahip_tensor_new: out of host memory");
    }
    *tensor = t;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_tensor_new");
}

void *ahip_tensor_data_mut(ahip_tensor *tensor) { return tensor ? tensor->t.data_as_bytes_mut() : nullptr; }

int ahip_host_pool_stats(size_t *live_bytes, size_t *cached_bytes, size_t *pinned_allocations, size_t *reuses) try {
    const altius::HostPoolStats st = altius::host_pool_stats();
    if (live_bytes) *live_bytes = st.live_bytes;
    if (cached_bytes) *cached_bytes = st.cached_bytes;
    if (pinned_allocations) *pinned_allocations = st.pinned_allocations;
    if (reuses) *reuses = st.reuses;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_host_pool_stats");
}

size_t ahip_host_pool_trim(void) { return altius::host_pool_trim(); }

void ahip_tensor_free(ahip_tensor *tensor) { delete tensor; }
int ahip_tensor_elem_type(const ahip_tensor *tensor) { return tensor ? (int)tensor->t.elem_ty() : -1; }
int ahip_tensor_rank(const ahip_tensor *tensor) { return tensor ? (int)tensor->t.dims().len() : -1; }
int ahip_tensor_dims(const ahip_tensor *tensor, int64_t *dims, int capacity) try {
    if (!tensor || capacity < 0 || (capacity && !dims)) return fail(AHIP_ERR_ARG, "ahip_tensor_dims: invalid argument");
    const auto &d = tensor->t.dims();
    for (int i = 0; i < capacity && i < (int)d.len(); i++) dims[i] = (int64_t)d[i];
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_tensor_dims");
}
size_t ahip_tensor_nbytes(const ahip_tensor *tensor) { return tensor ? tensor->t.nbytes() : 0; }
const void *ahip_tensor_data(const ahip_tensor *tensor) { return tensor ? tensor->t.data_as_bytes() : nullptr; }

// ---- session ---------------------------------------------------------------------------

int ahip_session_builder_new(const ahip_model *model, ahip_session_builder **builder) try {
    if (!model || !builder) return fail(AHIP_ERR_ARG, "ahip_session_builder_new: null argument");
    ahip_session_builder *b = new (std::nothrow) ahip_session_builder();
    if (!b) return fail(AHIP_ERR_OOM, "ahip_session_builder_new: out of host memory");
    b->model = model->m;
    *builder = b;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_new");
}

void ahip_session_builder_free(ahip_session_builder *builder) { delete builder; }

int ahip_session_builder_with_intra_op_num_threads(ahip_session_builder *builder, size_t n) try {
    if (!builder) return fail(AHIP_ERR_ARG, "null builder");
    builder->threads = n;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_with_intra_op_num_threads");
}

int ahip_session_builder_with_profiling_enabled(ahip_session_builder *builder, int enable) try {
    if (!builder) return fail(AHIP_ERR_ARG, "null builder");
    builder->profiling = enable != 0;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_with_profiling_enabled");
}

int ahip_session_builder_with_device(ahip_session_builder *builder, int device) try {
    if (!builder) return fail(AHIP_ERR_ARG, "null builder");
    builder->device = device;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_with_device");
}

int ahip_session_builder_with_device_timing(ahip_session_builder *builder, int enable) try {
    if (!builder) return fail(AHIP_ERR_ARG, "ahip_session_builder_with_device_timing: null builder");
    builder->device_timing = enable != 0;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_with_device_timing");
}

int ahip_session_builder_with_graph_replay(ahip_session_builder *builder, int enable) try {
    if (!builder) return fail(AHIP_ERR_ARG, "null builder");
    builder->graph_replay = enable != 0;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_with_graph_replay");
}

int ahip_session_builder_with_gemm_algorithm(ahip_session_builder *builder, int algorithm) try {
    if (!builder) return fail(AHIP_ERR_ARG, "null builder");
    if (algorithm != AHIP_GEMM_AUTO && algorithm != AHIP_GEMM_FP32 && algorithm != AHIP_GEMM_BF16X3)
        return fail(AHIP_ERR_ARG, "ahip_session_builder_with_gemm_algorithm: unknown algorithm");
    builder->gemm_algorithm = algorithm;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_with_gemm_algorithm");
}

int ahip_session_builder_with_strided_views(ahip_session_builder *builder, int enable) try {
    if (!builder) return fail(AHIP_ERR_ARG, "null builder");
    builder->strided_views = enable != 0;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_with_strided_views");
}

int ahip_session_builder_with_fused_attention(ahip_session_builder *builder, int enable) try {
    if (!builder) return fail(AHIP_ERR_ARG, "null builder");
    builder->fused_attention = enable != 0;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_with_fused_attention");
}

int ahip_session_copies_avoided(const ahip_session *session, size_t *count) try {
    if (!session || !count) return fail(AHIP_ERR_ARG, "ahip_session_copies_avoided: null argument");
    *count = last_lane_idle(session)->copies_avoided();
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_copies_avoided");
}

int ahip_session_graph_replays(const ahip_session *session, size_t *count) try {
    if (!session || !count) return fail(AHIP_ERR_ARG, "ahip_session_graph_replays: null argument");
    *count = last_lane_idle(session)->graph_replays();
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_graph_replays");
}

int ahip_session_builder_build(ahip_session_builder *builder, ahip_session **session) try {
    if (!builder || !session) return fail(AHIP_ERR_ARG, "ahip_session_builder_build: null argument");
    *session = nullptr;
    HipSessionBuilder b(builder->model);
    b.with_intra_op_num_threads(builder->threads).with_profiling_enabled(builder->profiling).with_device(builder->device).with_graph_replay(builder->graph_replay).with_gemm_algorithm(builder->gemm_algorithm).with_strided_views(builder->strided_views).with_fused_attention(builder->fused_attention).with_device_timing(builder->device_timing);
    SessionError err;
    std::unique_ptr<HipSession> s = b.build(&err);
    if (!s) return fail(err.code(), err.to_string());
    ahip_session *out = new (std::nothrow) ahip_session();
    if (!out) return fail(AHIP_ERR_OOM, "ahip_session_builder_build: out of host memory");
    out->view.m = s->model();
    out->s = std::move(s);
    out->settings.threads = builder->threads;
    out->settings.profiling = builder->profiling;
    out->settings.device = builder->device;
    out->settings.graph_replay = builder->graph_replay;
    out->settings.device_timing = builder->device_timing;
    out->settings.gemm_algorithm = builder->gemm_algorithm;
    out->settings.strided_views = builder->strided_views;
    out->settings.fused_attention = builder->fused_attention;
    out->lanes.push_back(out->s);
    out->busy.push_back(false);
    *session = out;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_builder_build");
}

int ahip_session_lanes(ahip_session *session, size_t *count) try {
    if (!session || !count) return fail(AHIP_ERR_ARG, "ahip_session_lanes: null argument");
    std::lock_guard<std::mutex> lock(session->lanes_mutex);
    *count = session->lanes.size();
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_lanes");
}

void ahip_session_free(ahip_session *session) { delete session; }

int ahip_session_run(ahip_session *session, int n_inputs, const ahip_tensor *const *inputs, int output_capacity,
                     ahip_tensor **outputs, int *n_outputs) try {
    if (!session || n_inputs < 0 || (n_inputs && !inputs) || output_capacity < 0 || (output_capacity && !outputs) ||
        !n_outputs)
        return fail(AHIP_ERR_ARG, "ahip_session_run: invalid argument");
    std::vector<Tensor> in;
    for (int i = 0; i < n_inputs; i++) {
        if (!inputs[i]) return fail(AHIP_ERR_ARG, "ahip_session_run: null input tensor");
        in.push_back(inputs[i]->t);  // shares the bytes, no copy
    }
    std::vector<Tensor> out;
    SessionError err;
    size_t lane_index = 0;
    std::shared_ptr<HipSession> lane;
    if (const int rc = acquire_lane(session, &lane_index, &lane)) return rc;
    bool ok = false;
    try {
        ok = lane->run(in, &out, &err);
    } catch (...) {
        release_lane(session, lane_index, false);
        throw;
    }
    release_lane(session, lane_index, ok);
    if (!ok) return fail(err.code(), err.to_string());
    *n_outputs = (int)out.size();
    if ((int)out.size() > output_capacity) return fail(AHIP_ERR_ARG, "ahip_session_run: output capacity too small");
    for (size_t i = 0; i < out.size(); i++) {
        ahip_tensor *t = new (std::nothrow) ahip_tensor();
        if (!t) {
            for (size_t j = 0; j < i; j++) delete outputs[j];
            return fail(AHIP_ERR_OOM, "ahip_session_run: out of host memory");
        }
        t->t = std::move(out[i]);
        outputs[i] = t;
    }
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_run");
}

int ahip_session_run_device(ahip_session *session, int n_inputs, const void *const *device_ptrs, const int *elem_types,
                            const int *ranks, const int64_t *const *dims, int output_capacity,
                            ahip_device_tensor **outputs, int *n_outputs) try {
    if (!session || n_inputs < 0 || (n_inputs && (!device_ptrs || !elem_types || !ranks || !dims)) || output_capacity < 0 ||
        (output_capacity && !outputs) || !n_outputs)
        return fail(AHIP_ERR_ARG, "ahip_session_run_device: invalid argument");
    std::vector<DeviceTensor> in(n_inputs);
    for (int i = 0; i < n_inputs; i++) {
        if (!valid_elem_type(elem_types[i])) return fail(AHIP_ERR_ARG, "ahip_session_run_device: unknown element type");
        if (ranks[i] < 0 || ranks[i] > AHIP_MAX_RANK || (ranks[i] && !dims[i]))
            return fail(AHIP_ERR_ARG, "ahip_session_run_device: bad rank or null dims");
        for (int k = 0; k < ranks[i]; k++)
            if (dims[i][k] < 0) return fail(AHIP_ERR_ARG, "ahip_session_run_device: negative dimension");
        in[i].dims = FixedDimensions::from_i64(dims[i], (size_t)ranks[i]);
        in[i].elem_ty = static_cast<TensorElemType>(elem_types[i]);
        in[i].ptr = const_cast<void *>(device_ptrs[i]);
    }
    std::vector<DeviceTensor> out;
    SessionError err;
    acquire_first_lane(session);
    bool ok = false;
    try {
        ok = session->s->run_device(in, &out, &err);
    } catch (...) {
        release_lane(session, 0, false);
        throw;
    }
    release_lane(session, 0, false);
    if (!ok) return fail(err.code(), err.to_string());
    *n_outputs = (int)out.size();
    auto drop_all = [&](size_t made) {
        for (size_t j = 0; j < made; j++) delete outputs[j];
        for (auto &t : out) session->s->release(&t);
    };
    if ((int)out.size() > output_capacity) {
        drop_all(0);
        return fail(AHIP_ERR_ARG, "ahip_session_run_device: output capacity too small");
    }
    for (size_t i = 0; i < out.size(); i++) {
        ahip_device_tensor *t = new (std::nothrow) ahip_device_tensor();
        if (!t) {
            drop_all(i);
            return fail(AHIP_ERR_OOM, "ahip_session_run_device: out of host memory");
        }
        t->t = std::move(out[i]);
        t->owner = session->s;
        outputs[i] = t;
    }
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_run_device");
}

int ahip_session_synchronize(ahip_session *session) try {
    if (!session) return fail(AHIP_ERR_ARG, "ahip_session_synchronize: null session");
    // Every lane's stream: a call that another thread made on a lane of its own is waited for as well.
    std::vector<std::shared_ptr<HipSession>> lanes;
    {
        std::lock_guard<std::mutex> lock(session->lanes_mutex);
        lanes = session->lanes;
    }
    for (auto &lane : lanes) {
        SessionError err;
        if (!lane->synchronize(&err)) return fail(err.code(), err.to_string());
    }
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_synchronize");
}

void ahip_device_tensor_free(ahip_device_tensor *tensor) { delete tensor; }
void *ahip_device_tensor_ptr(const ahip_device_tensor *tensor) { return tensor ? tensor->t.ptr : nullptr; }
int ahip_device_tensor_elem_type(const ahip_device_tensor *tensor) { return tensor ? (int)tensor->t.elem_ty : -1; }
int ahip_device_tensor_rank(const ahip_device_tensor *tensor) { return tensor ? (int)tensor->t.dims.len() : -1; }
size_t ahip_device_tensor_nbytes(const ahip_device_tensor *tensor) { return tensor ? tensor->t.nbytes() : 0; }
int ahip_device_tensor_dims(const ahip_device_tensor *tensor, int64_t *dims, int capacity) try {
    if (!tensor || capacity < 0 || (capacity && !dims)) return fail(AHIP_ERR_ARG, "ahip_device_tensor_dims: invalid argument");
    for (int i = 0; i < capacity && i < (int)tensor->t.dims.len(); i++) dims[i] = (int64_t)tensor->t.dims[i];
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_device_tensor_dims");
}

const ahip_model *ahip_session_model(const ahip_session *session) { return session ? &session->view : nullptr; }

int ahip_session_profile(const ahip_session *session, int index, const char **op_name, double *ms, int *count) try {
    if (!session) return fail(AHIP_ERR_ARG, "ahip_session_profile: null session");
    // The names handed out point into `profile`, which the next profiled run replaces: as before, the caller reads
    // them before it runs again; the lock keeps a run on another thread from replacing it in mid-read.
    std::lock_guard<std::mutex> lock(const_cast<ahip_session *>(session)->lanes_mutex);
    if (count) *count = (int)session->profile.size();
    if (index < 0 || index >= (int)session->profile.size()) {
        if (op_name || ms) return fail(AHIP_ERR_ARG, "ahip_session_profile: index out of range");
        return AHIP_OK;
    }
    if (op_name) *op_name = session->profile[index].first.c_str();
    if (ms) *ms = session->profile[index].second;
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_profile");
}

int ahip_session_last_device_ms(const ahip_session *session, double *ms) try {
    if (!session || !ms) return fail(AHIP_ERR_ARG, "ahip_session_last_device_ms: null argument");
    *ms = last_lane_idle(session)->last_device_ms();
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_last_device_ms");
}

int ahip_session_last_run_ms(const ahip_session *session, double *ms) try {
    if (!session || !ms) return fail(AHIP_ERR_ARG, "ahip_session_last_run_ms: null argument");
    *ms = last_lane_idle(session)->last_run_ms();
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_last_run_ms");
}

int ahip_session_device_allocations(const ahip_session *session, size_t *count) try {
    if (!session || !count) return fail(AHIP_ERR_ARG, "ahip_session_device_allocations: null argument");
    *count = last_lane_idle(session)->device_allocations();
    return AHIP_OK;
} catch (...) {
    return altius::caught_at_boundary("ahip_session_device_allocations");
}

}  // extern "C"
