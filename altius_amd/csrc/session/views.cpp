// The session's copy avoidance: strided views (Split / Transpose results that only MatMuls read), operand
// descriptions for the GEMM, activations deferred into the next product's operand split, and
// MatMul -> Softmax -> MatMul deferred into the one-kernel attention.  Counterparts in the reference always
// copy: compute_transpose (crates/session_interpreter/src/session.rs:1179-1278), compute_split (1488-1548),
// compute_mat_mul (621-684), compute_softmax (990-1026).
#include <algorithm>
#include <functional>

#include "views.h"

namespace altius {

using namespace detail;

bool HipSession::materialize(DeviceTensor *t, SessionError *err) {
    if (t->strides.empty()) return true;
    DeviceTensor dense;
    if (!allocate(TypedFixedShape{t->dims, t->elem_ty}, &dense, err)) return false;
    std::vector<int64_t> d;
    for (auto x : t->dims.as_vec()) d.push_back((int64_t)x);
    const std::vector<int64_t> os = dense_strides(t->dims);
    const int rc = launch_copy_strided(ctx_, dense.ptr, t->ptr, (int)elem_size(t->elem_ty), (int)d.size(), d.data(), os.data(),
                                       t->strides.data());
    if (rc) return fail_code(err, rc, ctx_.last_error);
    dense.host = t->host;
    *t = std::move(dense);
    return true;
}

bool HipSession::flush_add(DeviceTensor *t, SessionError *err) {
    if (!t->owes_add()) return true;
    PendingAdd &p = *t->pending_add;
    const int64_t n = (int64_t)p.elems, one = 1;
    const int rc = launch_binary(ctx_, AHIP_ADD, static_cast<float *>(t->ptr), p.a, p.b, 1, &n, &one, &one);
    if (rc) return fail_code(err, rc, ctx_.last_error);
    p.done = true;
    p.a_block.reset();
    p.b_block.reset();
    return true;
}

bool HipSession::apply_pending(DeviceTensor *t, SessionError *err) {
    if (!flush_add(t, err)) return false;
    if (t->pending_op < 0) return true;
    if (t->pending_op == PENDING_ATTENTION)  // callers that know the value's id flush it instead (flush_attention)
        return fail(err, SessionError::Message, "internal: a deferred attention product was read by an operator that cannot finish it");
    if (!materialize(t, err)) return false;
    DeviceTensor done;
    if (!allocate(TypedFixedShape{t->dims, t->elem_ty}, &done, err)) return false;
    const int rc = launch_unary(ctx_, t->pending_op, static_cast<float *>(done.ptr), static_cast<const float *>(t->ptr),
                                t->dims.total_elems(), 0.0f, 0.0f);
    if (rc) return fail_code(err, rc, ctx_.last_error);
    *t = std::move(done);
    return true;
}

bool HipSession::describe_operand(DeviceTensor *t, MatOperand *o, SessionError *err) {
    for (int attempt = 0; attempt < 2; attempt++) {
        const size_t r = t->dims.len();
        const std::vector<int64_t> st = strides_of(*t);
        o->rows = t->dims[r - 2], o->cols = t->dims[r - 1];
        const int64_t sr = st[r - 2], sc = st[r - 1];
        bool ok = true;
        if (sc == 1 || o->cols == 1) {
            o->stored_transposed = false;
            o->ld = o->rows == 1 ? o->cols : (size_t)sr;
            ok = o->ld >= o->cols;
        } else if (sr == 1 || o->rows == 1) {
            o->stored_transposed = true;
            o->ld = o->cols == 1 ? o->rows : (size_t)sc;
            ok = o->ld >= o->rows;
        } else {
            ok = false;
        }
        o->batch = 1;
        o->bdims.clear(), o->bstr.clear();
        for (size_t i = 0; i + 2 < r; i++) {
            o->batch *= t->dims[i];
            o->bdims.push_back(t->dims[i]);
            o->bstr.push_back(st[i]);
            ok = ok && st[i] >= 0;
        }
        if (ok) return true;
        if (t->strides.empty()) break;
        if (!materialize(t, err)) return false;
    }
    return fail(err, SessionError::Message, "MatMul: an operand's layout could not be read");
}

namespace {
// Batch strides of an operand over the batch axes bd (extent-1 axes already dropped from both): a dense
// operand counts its matrices in bd's order whatever its own leading shape.
bool operand_batch_strides(const std::vector<size_t> &bd, const std::vector<size_t> &own_dims, const std::vector<int64_t> &own_strides,
                           bool dense, size_t matrix_elems, size_t batch, std::vector<int64_t> *out) {
    out->assign(bd.size(), 0);
    if (batch == 1) return true;
    if (dense) {
        int64_t acc = (int64_t)matrix_elems;
        for (size_t i = bd.size(); i-- > 0;) (*out)[i] = acc, acc *= (int64_t)bd[i];
        return true;
    }
    std::vector<size_t> d;
    std::vector<int64_t> s;
    for (size_t i = 0; i < own_dims.size(); i++)
        if (own_dims[i] != 1) d.push_back(own_dims[i]), s.push_back(own_strides[i]);
    if (d != bd) return false;
    *out = s;
    return true;
}
bool aligned_operand(const void *p, size_t ld, const std::vector<int64_t> &bs) {
    bool ok = (reinterpret_cast<uintptr_t>(p) & 15u) == 0 && ld % 4 == 0;
    for (int64_t s : bs) ok = ok && s % 4 == 0;
    return ok;
}
}  // namespace

bool HipSession::flush_attention(ValueId scores, DeviceTensor *placeholder, SessionError *err) {
    auto it = pending_attn_.find(scores);
    if (it == pending_attn_.end()) return fail(err, SessionError::Message, "internal: no operands kept for a deferred attention product");
    PendingAttention pa = std::move(it->second);
    pending_attn_.erase(it);
    DeviceTensor out;
    if (!allocate(TypedFixedShape{pa.score_dims, TensorElemType::F32}, &out, err)) return false;
    const size_t tq = pa.Q.stored_transposed ? pa.Q.cols : pa.Q.rows, tk = pa.K.stored_transposed ? pa.K.cols : pa.K.rows;
    auto two = [](const std::vector<int64_t> &s, size_t out2[2]) {
        out2[0] = s.size() > 0 ? (size_t)s[0] : 0;
        out2[1] = s.size() > 1 ? (size_t)s[1] : 0;
    };
    const size_t outer = pa.bd.size() > 0 ? pa.bd[0] : 1, inner = pa.bd.size() > 1 ? pa.bd[1] : 1;
    size_t q2[2], k2[2], c2[2] = {inner * tq * tk, pa.bd.size() > 1 ? tq * tk : 0};
    two(pa.Q.bstr, q2), two(pa.K.bstr, k2);
    // Q rows [tq, 64] times the transpose of K rows [tk, 64].
    const int rc = launch_gemm_batch2(ctx_, static_cast<float *>(out.ptr), static_cast<const float *>(pa.q.ptr),
                                      static_cast<const float *>(pa.k.ptr), nullptr, outer, inner, tq, tk, 64, 0, 1, pa.Q.ld, pa.K.ld, tk, q2,
                                      k2, c2, 0, 1, 1.0f, 0.0f);
    if (rc) return fail_code(err, rc, ctx_.last_error);
    *placeholder = std::move(out);
    return true;
}

// The first product of MatMul -> Softmax -> MatMul: if the one-kernel attention can take it (64-wide heads,
// at most two batch axes, aligned operands), leave a placeholder and remember Q and K.
bool HipSession::try_defer_attention(const Node &node, const Op &op, const std::vector<DeviceTensor *> &in,
                                     const std::vector<TypedFixedShape> &shapes, std::vector<DeviceTensor> *outs, SessionError *err) {
    if (in.size() != 2 || !in[0] || !in[1] || in[0]->elem_ty != TensorElemType::F32 || in[1]->elem_ty != TensorElemType::F32) return true;
    if (in[0]->dims.len() < 2 || in[1]->dims.len() < 2 || in[0]->pending_op >= 0 || in[1]->pending_op >= 0) return true;
    PendingAttention pa;
    if (!describe_operand(in[0], &pa.Q, err) || !describe_operand(in[1], &pa.K, err)) return false;
    // Q as stored rows [tq, d]; the logical second operand is K^T, so K must be stored as rows [tk, d].
    const bool q_rows = !((op.trans_a ? 1 : 0) ^ (pa.Q.stored_transposed ? 1 : 0));
    const bool k_rows = ((op.trans_b ? 1 : 0) ^ (pa.K.stored_transposed ? 1 : 0)) != 0;
    if (!q_rows || !k_rows) return true;
    const size_t tq = pa.Q.stored_transposed ? pa.Q.cols : pa.Q.rows, d = pa.Q.stored_transposed ? pa.Q.rows : pa.Q.cols;
    const size_t tk = pa.K.stored_transposed ? pa.K.cols : pa.K.rows, dk = pa.K.stored_transposed ? pa.K.rows : pa.K.cols;
    if (d != 64 || dk != 64 || tk == 0 || tq == 0) return true;
    const FixedDimensions &od = shapes[0].dims;
    size_t batch = 1;
    for (size_t i = 0; i + 2 < od.len(); i++) {
        batch *= od[i];
        if (od[i] != 1) pa.bd.push_back(od[i]);
    }
    if (pa.bd.size() > 2 || pa.Q.batch != batch || pa.K.batch != batch) return true;
    std::vector<int64_t> qs, ks;
    if (!operand_batch_strides(pa.bd, pa.Q.bdims, pa.Q.bstr, in[0]->strides.empty(), tq * d, pa.Q.batch, &qs) ||
        !operand_batch_strides(pa.bd, pa.K.bdims, pa.K.bstr, in[1]->strides.empty(), tk * d, pa.K.batch, &ks))
        return true;
    if (!aligned_operand(in[0]->ptr, pa.Q.ld, qs) || !aligned_operand(in[1]->ptr, pa.K.ld, ks)) return true;
    pa.Q.bstr = qs, pa.K.bstr = ks;  // now per axis of bd
    pa.q = *in[0], pa.k = *in[1];
    pa.score_dims = od;
    pending_attn_[node.outputs[0]] = std::move(pa);
    DeviceTensor o;
    o.dims = od;
    o.elem_ty = TensorElemType::F32;
    o.pending_op = PENDING_ATTENTION;
    copies_avoided_++;
    outs->push_back(std::move(o));
    return true;
}

// The second product: O = Softmax(scale(Q K^T)) V in one kernel, into `out` (dense, or in the layout of the
// Transpose behind this node).
bool HipSession::run_attention_tail(const Op &op, const std::vector<DeviceTensor *> &in, DeviceTensor *out, SessionError *err) {
    const Node &node = model_.graph.nodes[current_node_];
    auto it = pending_attn_.find(node.inputs[0]);
    if (it == pending_attn_.end()) return fail(err, SessionError::Message, "MatMul: deferred attention operands are missing");
    PendingAttention pa = std::move(it->second);
    pending_attn_.erase(it);
    // Which attention this is (for the scale): the head that names this node as its tail.
    const AttentionPlan *plan = nullptr;
    for (const auto &kv : attn_head_)
        if (kv.second.tail == current_node_) plan = &kv.second;
    if (!plan) return fail(err, SessionError::Message, "MatMul: no attention plan for this node");
    if (op.trans_a || in.size() != 2 || !in[1] || in[1]->elem_ty != TensorElemType::F32 || in[1]->dims.len() < 2)
        return fail(err, SessionError::Message, "MatMul: the second product of an attention has an unexpected form");
    const size_t tq = pa.Q.stored_transposed ? pa.Q.cols : pa.Q.rows, tk = pa.K.stored_transposed ? pa.K.cols : pa.K.rows;
    MatOperand V;
    std::vector<int64_t> vs;
    for (int attempt = 0;; attempt++) {
        if (!describe_operand(in[1], &V, err)) return false;
        const bool v_rows = !((op.trans_b ? 1 : 0) ^ (V.stored_transposed ? 1 : 0));
        size_t batch = 1;
        for (size_t x : pa.bd) batch *= x;
        bool ok = v_rows && V.rows == tk && V.cols == 64 && (V.batch == batch || V.batch == 1) &&
                  operand_batch_strides(pa.bd, V.bdims, V.bstr, in[1]->strides.empty(), tk * 64, V.batch, &vs) &&
                  aligned_operand(in[1]->ptr, V.ld, vs);
        if (ok) break;
        if (attempt > 0 || in[1]->strides.empty())
            return fail(err, SessionError::Message, "MatMul: the values of an attention do not fit its keys");
        if (!materialize(in[1], err)) return false;
    }
    // Output strides: dense, or the Transpose's layout behind this node.
    std::vector<int64_t> c_str = dense_strides(out->dims);
    auto pv = matmul_out_perm_.find(current_node_);
    if (pv != matmul_out_perm_.end() && pv->second.size() == out->dims.len()) {
        FixedDimensions td = out->dims;
        for (size_t i = 0; i < td.len(); i++) td[i] = out->dims[(size_t)pv->second[i]];
        const std::vector<int64_t> ts = dense_strides(td);
        std::vector<int64_t> cand = c_str;
        for (size_t i = 0; i < td.len(); i++) cand[(size_t)pv->second[i]] = ts[i];
        bool aligned = true;
        for (size_t i = 0; i + 1 < cand.size(); i++) aligned = aligned && (out->dims[i] == 1 || cand[i] % 4 == 0);
        if (aligned && !is_dense(out->dims, cand)) out->strides = c_str = cand;
    }
    const size_t rank = out->dims.len();
    std::vector<int64_t> os;
    for (size_t i = 0; i + 2 < rank; i++)
        if (out->dims[i] != 1) os.push_back(c_str[i]);
    const size_t ldo = out->dims[rank - 2] > 1 ? (size_t)c_str[rank - 2] : 64;
    auto two = [](const std::vector<int64_t> &s, size_t out2[2]) {
        out2[0] = s.size() > 0 ? (size_t)s[0] : 0;
        out2[1] = s.size() > 1 ? (size_t)s[1] : 0;
    };
    size_t q2[2], k2[2], v2[2], o2[2];
    two(pa.Q.bstr, q2), two(pa.K.bstr, k2), two(vs, v2), two(os, o2);
    const size_t outer = pa.bd.size() > 0 ? pa.bd[0] : 1, inner = pa.bd.size() > 1 ? pa.bd[1] : 1;
    // O as the operand planes of the product behind it: O is [outer, inner, tq, 64] written as [outer, tq, inner * 64]
    // (the Transpose's layout), which that product reads as [outer * tq, inner * 64].
    void *planes_ptr = nullptr;
    auto ap = attn_planes_.find(current_node_);
    if (ap != attn_planes_.end() && pa.bd.size() == 2 && rank == 4 && !out->strides.empty() && ldo == inner * 64 && o2[0] == tq * ldo && o2[1] == 64 &&
        attention_writes_planes(ctx_, outer, inner, tq) && gemm_takes_split(ctx_, outer * tq, ap->second.next_n, inner * 64)) {
        DeviceTensor planes;
        if (!allocate_bytes(gemm_planes_bytes(outer * tq, inner * 64), &planes, err)) return false;
        out->block = planes.block;  // the fp32 block goes back to the pool unused
        out->ptr = planes.ptr;
        out->planes = true;
        out->planes_rows = outer * tq, out->planes_k = inner * 64;
        planes_ptr = planes.ptr;
        copies_avoided_++;  // the operand split of the product behind
    }
    const int rc = launch_attention(ctx_, planes_ptr ? nullptr : static_cast<float *>(out->ptr), static_cast<const float *>(pa.q.ptr),
                                    static_cast<const float *>(pa.k.ptr), static_cast<const float *>(in[1]->ptr), outer, inner, tq, tk, 64,
                                    pa.Q.ld, pa.K.ld, V.ld, ldo, q2, k2, v2, o2, plan->scale_op, plan->scale,
                                    pa.mask.ptr ? static_cast<const float *>(pa.mask.ptr) : nullptr, pa.mask_outer_stride, planes_ptr);
    if (rc) return fail_code(err, rc, ctx_.last_error);
    return true;
}

// A Split or Transpose hands out views when everything downstream of it can read them in place:
// MatMul operands, possibly through reshapes and further transposes.  A MatMul whose only reader is
// a Transpose that keeps the last axis writes its result directly in that Transpose's layout.
void HipSession::plan_views(bool fused_attention) {
    const auto users = model_.get_value_users();
    const auto parents = model_.get_value_parents();
    const Graph &g = model_.graph;
    auto is_output = [&](ValueId v) { return std::find(g.outputs.begin(), g.outputs.end(), v) != g.outputs.end(); };
    std::function<bool(ValueId, int)> view_ok = [&](ValueId v, int depth) -> bool {
        if (depth > 8 || is_output(v)) return false;
        auto it = users.find(v);
        if (it == users.end() || it->second.empty()) return false;
        for (NodeId u : it->second) {
            const Node &n = g.nodes[u];
            if (n.op.kind == OpKind::MatMul) {
                if (n.inputs.size() > 2 && n.inputs[2] == v) return false;
            } else if (is_alias_op(n.op.kind) || n.op.kind == OpKind::Transpose) {
                if (n.inputs.empty() || n.inputs[0] != v || n.outputs.empty()) return false;
                for (size_t i = 1; i < n.inputs.size(); i++)
                    if (n.inputs[i] == v) return false;
                if (!view_ok(n.outputs[0], depth + 1)) return false;
            } else {
                return false;
            }
        }
        return true;
    };
    for (const NodeExecutionPlan &step : plan_) {
        const NodeId id = step.node_id;
        const Node &n = g.nodes[id];
        if (n.op.kind == OpKind::Split || n.op.kind == OpKind::Transpose) {
            bool all = !n.outputs.empty();
            for (ValueId v : n.outputs) all = all && view_ok(v, 0);
            if (all) lazy_views_.insert(id);
        } else if ((n.op.kind == OpKind::Gelu || n.op.kind == OpKind::ReLU) && n.outputs.size() == 1 && n.inputs.size() == 1 &&
                   !is_output(n.outputs[0])) {
            // The activation between two products: its only reader is a MatMul's first operand.
            auto it = users.find(n.outputs[0]);
            if (it == users.end() || it->second.size() != 1) continue;
            const Node &mm = g.nodes[*it->second.begin()];
            if (mm.op.kind != OpKind::MatMul || mm.inputs.size() < 2 || mm.inputs[0] != n.outputs[0]) continue;
            bool elsewhere = false;
            for (size_t i = 1; i < mm.inputs.size(); i++) elsewhere = elsewhere || mm.inputs[i] == n.outputs[0];
            if (!elsewhere) deferred_unary_.insert(id);
        } else if (n.op.kind == OpKind::LayerNormalization && n.outputs.size() == 1 && n.inputs.size() == 3 && !is_output(n.outputs[0])) {
            // LayerNormalization read only by a product with a weight matrix: it can write that product's operand planes.
            auto it = users.find(n.outputs[0]);
            if (it == users.end() || it->second.size() != 1) continue;
            const Node &mm = g.nodes[*it->second.begin()];
            if (mm.op.kind != OpKind::MatMul || mm.inputs.size() < 2 || mm.inputs[0] != n.outputs[0] || mm.op.trans_a) continue;
            bool elsewhere = false;
            for (size_t i = 1; i < mm.inputs.size(); i++) elsewhere = elsewhere || mm.inputs[i] == n.outputs[0];
            auto w = g.inits.find(mm.inputs[1]);
            if (elsewhere || w == g.inits.end() || w->second.dims().len() != 2 || w->second.elem_ty() != TensorElemType::F32) continue;
            PlanesPlan pp;
            pp.consumer = *it->second.begin();
            pp.next_n = mm.op.trans_b ? w->second.dims()[0] : w->second.dims()[1];
            planes_out_[id] = pp;
            planes_consumer_.insert(pp.consumer);
            // The residual Add in front of it (two tensors of one shape) can leave its sum to this kernel.
            auto par = parents.find(n.inputs[0]);
            if (par != parents.end()) {
                const Node &add = g.nodes[par->second];
                if (add.op.kind == OpKind::Add && add.inputs.size() == 2 && add.outputs.size() == 1 && add.inputs[0] != add.inputs[1])
                    add_into_ln_[par->second] = id;
            }
        } else if (n.op.kind == OpKind::MatMul && n.outputs.size() == 1 && !is_output(n.outputs[0])) {
            auto it = users.find(n.outputs[0]);
            if (it == users.end() || it->second.size() != 1) continue;
            // MatMul -> Gelu / Relu, or MatMul -> Add(residual): done by the product's own kernel when it is the fp32 one.
            {
                const NodeId uid = *it->second.begin();
                const Node &u = g.nodes[uid];
                MatMulPost mp;
                if ((u.op.kind == OpKind::Gelu || u.op.kind == OpKind::ReLU) && u.inputs.size() == 1 && u.outputs.size() == 1) {
                    mp.act = u.op.kind == OpKind::Gelu ? AHIP_GELU : AHIP_RELU;
                    matmul_post_[id] = mp;
                } else if (u.op.kind == OpKind::Add && u.inputs.size() == 2 && u.outputs.size() == 1 && u.inputs[0] != u.inputs[1]) {
                    mp.has_add = true;
                    mp.add_node = uid;
                    mp.add_input = u.inputs[0] == n.outputs[0] ? 0 : 1;
                    mp.residual = u.inputs[1 - mp.add_input];
                    matmul_post_[id] = mp;
                }
            }
            // MatMul -> Softmax(last axis, optional scalar scale, no mask) -> MatMul(first operand): one attention kernel.
            if (fused_attention) {
                const NodeId sid = *it->second.begin();
                const Node &sm = g.nodes[sid];
                if (sm.op.kind == OpKind::Softmax && n.inputs.size() == 2 && !sm.inputs.empty() && sm.inputs[0] == n.outputs[0] &&
                    sm.outputs.size() == 1 && !is_output(sm.outputs[0])) {
                    bool last_axis = sm.op.axis == -1;
                    auto sh = inferred_.find(sid);
                    if (!last_axis && sh != inferred_.end() && !sh->second.second.empty())
                        last_axis = sm.op.axis == (int64_t)sh->second.second[0].dims.len() - 1;
                    AttentionPlan ap;
                    ap.has_mask = sm.op.prologue_mask != 0;
                    bool scale_ok = true;
                    if (sm.op.prologue_scale) {
                        auto init = sm.inputs.size() > 1 ? g.inits.find(sm.inputs[1]) : g.inits.end();
                        scale_ok = init != g.inits.end() && init->second.elem_ty() == TensorElemType::F32 &&
                                   init->second.dims().total_elems() == 1 && init->second.has_data();
                        if (scale_ok) ap.scale_op = sm.op.prologue_scale, ap.scale = init->second.data_f32()[0];
                    }
                    auto su = users.find(sm.outputs[0]);
                    if (last_axis && scale_ok && su != users.end() && su->second.size() == 1) {
                        const NodeId tid = *su->second.begin();
                        const Node &mm = g.nodes[tid];
                        if (mm.op.kind == OpKind::MatMul && mm.inputs.size() == 2 && mm.inputs[0] == sm.outputs[0] &&
                            mm.inputs[1] != sm.outputs[0] && !mm.op.trans_a) {
                            ap.softmax = sid, ap.tail = tid;
                            attn_head_[id] = ap;
                            attn_softmax_.insert(sid);
                            attn_tail_.insert(tid);
                            continue;
                        }
                    }
                }
            }
            const Node &t = g.nodes[*it->second.begin()];
            if (t.op.kind != OpKind::Transpose || t.inputs.size() != 1) continue;
            const auto &perm = t.op.perm;
            if (perm.size() < 3 || perm.back() != (int64_t)perm.size() - 1) continue;
            matmul_out_perm_[id] = perm;
        }
    }
    // An attention whose result goes, through the Transpose it is written ahead of and one Reshape, into a product with a
    // weight matrix and nowhere else: the attention kernel can write that product's operand planes.
    for (NodeId tid : attn_tail_) {
        auto pv = matmul_out_perm_.find(tid);
        if (pv == matmul_out_perm_.end() || pv->second != std::vector<int64_t>{0, 2, 1, 3}) continue;
        auto single_user = [&](ValueId v, NodeId *u) {
            auto it = users.find(v);
            if (it == users.end() || it->second.size() != 1 || is_output(v)) return false;
            *u = *it->second.begin();
            return true;
        };
        NodeId tr, rs, mm;
        if (!single_user(g.nodes[tid].outputs[0], &tr) || g.nodes[tr].op.kind != OpKind::Transpose || g.nodes[tr].outputs.size() != 1) continue;
        if (!single_user(g.nodes[tr].outputs[0], &rs) || g.nodes[rs].op.kind != OpKind::Reshape || g.nodes[rs].outputs.size() != 1 ||
            g.nodes[rs].inputs.empty() || g.nodes[rs].inputs[0] != g.nodes[tr].outputs[0])
            continue;
        if (!single_user(g.nodes[rs].outputs[0], &mm)) continue;
        const Node &m = g.nodes[mm];
        if (m.op.kind != OpKind::MatMul || m.inputs.size() < 2 || m.inputs[0] != g.nodes[rs].outputs[0] || m.op.trans_a ||
            planes_consumer_.count(mm) || matmul_out_perm_.count(mm))
            continue;
        bool elsewhere = false;
        for (size_t i = 1; i < m.inputs.size(); i++) elsewhere = elsewhere || m.inputs[i] == m.inputs[0];
        auto w = g.inits.find(m.inputs[1]);
        if (elsewhere || w == g.inits.end() || w->second.dims().len() != 2 || w->second.elem_ty() != TensorElemType::F32) continue;
        // The planes are laid out for [b * t, h * 64] x weights [h * 64, n]: the attention's result must be [b, h, t, 64],
        // the Reshape must merge exactly the heads into the last axis (any other valid reshape, [b, t * h, 64] say, would
        // read the planes with another geometry), and the weights must have h * 64 rows.  Shapes that are not known
        // before the run leave the plan out.
        auto at = inferred_.find(tid), rt = inferred_.find(rs);
        if (at == inferred_.end() || rt == inferred_.end() || at->second.second.empty() || rt->second.second.empty()) continue;
        const FixedDimensions &ad = at->second.second[0].dims, &rd = rt->second.second[0].dims;
        if (ad.len() != 4 || ad[3] != 64 || rd.len() < 2) continue;
        const size_t merged = ad[1] * 64, rows = ad[0] * ad[2];
        size_t lead = 1;
        for (size_t i = 0; i + 1 < rd.len(); i++) lead *= rd[i];
        if (rd[rd.len() - 1] != merged || lead != rows || (m.op.trans_b ? w->second.dims()[1] : w->second.dims()[0]) != merged) continue;
        PlanesPlan pp;
        pp.consumer = mm;
        pp.next_n = m.op.trans_b ? w->second.dims()[0] : w->second.dims()[1];
        attn_planes_[tid] = pp;
        planes_consumer_.insert(mm);
        planes_pass_.insert(tr);
        planes_pass_.insert(rs);
    }
}

}  // namespace altius
