// Pattern fusion over the node list of a session's graph.
//
// The reference executes an ONNX graph node by node, one kernel each
// (runtime/src/core/instance.rs:25-37). Decoder graphs repeat a few chains of small element-wise
// nodes in every layer; on this GPU each launch costs ~2 us whatever it moves, so those chains
// dominate a decode step. This pass finds them and replaces each by ONE node backed by a fused
// kernel that rounds every intermediate like the separate kernels do (the attention MatMul
// instead drops two copies: the grouped-query Expand and the K transpose become GEMM strides):
//
//   rmlk.RMSNorm           Pow(x,2) ReduceMean(-1) Add(eps) Sqrt Div|(Div(1,.) Mul) Mul(gamma)
//   rmlk.AddRMSNorm        Add(a,b) followed by rmlk.RMSNorm: the sum is an output too
//   rmlk.SwiGLU            Sigmoid(g) Mul(g,.) Mul(.,u)
//   rmlk.ScaleMaskSoftmax  Div|Mul(x,c) Add(mask) Softmax(-1)
//   rmlk.Rotary            [Transpose(0,2,1,3)] Slice Slice Neg Concat Mul Mul Add
//   rmlk.HeadRows          up to four streams of rows (rmlk.Rotary, or a ScatterND fed by one or by
//                          a head Transpose) behind one projection, one launch
//   rmlk.AttnMatMul        MatMul(a, [Transpose(0,1,3,2)] [Reshape Expand Unsqueeze] (kv))
//   rmlk.Attention         rmlk.AttnMatMul -> rmlk.ScaleMaskSoftmax -> rmlk.AttnMatMul [-> Transpose]
//   rmlk.MatMulGroup       MatMul(a, W1), MatMul(a, W2), ... on the same a with constant 2-D weights
//   rmlk.MatMulGroupSwiGLU a [gate | up] rmlk.MatMulGroup feeding only an rmlk.SwiGLU
//   rmlk.MatMulAddRMSNorm  MatMul(a, W) feeding the residual Add of an rmlk.AddRMSNorm
//   rmlk.MatMulConst       any other MatMul(a, W) with constant 2-D W
//
// The nodes over constant weights store them K-contiguous ([n][k]) and release the row-major
// initializers: one-row inputs and many-row inputs read the same copy.
//
// A fused node keeps the nodes it replaced as its `body` (the nodes over constant weights: product
// nodes over the K-contiguous weights, or nothing where every case is covered). What cannot be decided while building
// (shapes are only known at run time) is checked when the node runs; if the fused kernel does not
// cover the case, the body runs instead, node by node, so the graph's meaning never changes.
#include <algorithm>
#include <cmath>
#include <set>

#include "core.hpp"

namespace rmlk {
namespace rt {

namespace {

struct Matcher {
    Session &s;
    rmlk_graph &g;
    std::vector<std::vector<int>> users;   // value id -> consumer node indices
    std::vector<bool> removed;

    explicit Matcher(Session &session) : s(session), g(session.graph_copy) {
        users.assign(g.values.size(), {});
        removed.assign(g.nodes.size(), false);
        for (size_t n = 0; n < g.nodes.size(); ++n)
            for (int v : g.nodes[n].inputs)
                if (v >= 0) users[v].push_back(static_cast<int>(n));
    }

    int producer(int v) const {
        if (v < 0) return -1;
        const Value &val = g.values[v];
        if (val.is_input || val.is_initializer) return -1;
        int p = val.producer;
        return p >= 0 && !removed[p] ? p : -1;
    }
    const Node *produced_by(int v, const char *op) const {
        int p = producer(v);
        return p >= 0 && g.nodes[p].op == op ? &g.nodes[p] : nullptr;
    }
    // every consumer of v is one of `inside`, and v is not a graph output
    bool only_used_by(int v, std::initializer_list<const Node *> inside) const {
        if (g.values[v].is_output) return false;
        for (int u : users[v]) {
            bool ok = false;
            for (const Node *n : inside)
                if (n == &g.nodes[u]) ok = true;
            if (!ok) return false;
        }
        return true;
    }
    bool const_float(int v, float *out) const {
        if (v < 0 || !g.values[v].is_initializer) return false;
        const Tensor &t = s.values[v];
        if (t.dtype != RMLK_FLOAT || t.numel() != 1 || !t.host || !t.host->is_float) return false;
        *out = static_cast<float>(t.host->f[0]);
        return true;
    }
    bool const_ints(int v, std::vector<int64_t> *out) const {
        if (v < 0 || !g.values[v].is_initializer) return false;
        const Tensor &t = s.values[v];
        if (!t.host || t.host->is_float) return false;
        if (t.dtype != RMLK_INT64 && t.dtype != RMLK_INT32) return false;
        *out = t.host->i;
        return true;
    }
    static int64_t attr_int(const Node &n, const char *name, int64_t dflt) {
        auto it = n.attrs.find(name);
        return it == n.attrs.end() ? dflt : it->second.i;
    }
    int index_of(const Node *n) const { return static_cast<int>(n - g.nodes.data()); }

    // Replace `parts` (graph order) by one node at the position of the last of them.
    void replace(const std::vector<const Node *> &parts, Node fused) {
        std::vector<int> idx;
        for (const Node *n : parts) idx.push_back(index_of(n));
        std::sort(idx.begin(), idx.end());
        for (int i : idx) fused.body.push_back(g.nodes[i]);
        for (int i : idx) {
            removed[i] = true;
            for (int v : g.nodes[i].inputs) {
                if (v < 0) continue;
                auto &u = users[v];
                u.erase(std::remove(u.begin(), u.end(), i), u.end());
            }
        }
        const int at = idx.back();
        g.nodes[at] = std::move(fused);
        removed[at] = false;
        // consumers: the fused node now reads its inputs at `at`
        for (int v : g.nodes[at].inputs)
            if (v >= 0) users[v].push_back(at);
        for (int v : g.nodes[at].outputs) g.values[v].producer = at;
    }

    static Attr a_int(int64_t v) {
        Attr a;
        a.kind = Attr::Int;
        a.i = v;
        return a;
    }
    static Attr a_float(float v) {
        Attr a;
        a.kind = Attr::Float;
        a.f = v;
        return a;
    }

    // ---- RMSNorm, anchored at the final Mul ------------------------------------------------------
    bool match_rmsnorm(const Node &m2) {
        if (m2.op != "Mul" || m2.inputs.size() != 2) return false;
        for (int side = 0; side < 2; ++side) {
            const int normed = m2.inputs[side], gamma = m2.inputs[1 - side];
            if (normed < 0 || gamma < 0) continue;
            const Node *sqrt_n = nullptr, *div_n = nullptr, *mul_n = nullptr;
            int x = -1;
            bool recip = false;
            if (const Node *d = produced_by(normed, "Div")) {
                // x / sqrt(var)
                if (d->inputs.size() != 2) continue;
                sqrt_n = produced_by(d->inputs[1], "Sqrt");
                if (!sqrt_n) continue;
                div_n = d;
                x = d->inputs[0];
            } else if (const Node *m = produced_by(normed, "Mul")) {
                // x * (1 / sqrt(var))
                if (m->inputs.size() != 2) continue;
                for (int k = 0; k < 2 && !div_n; ++k) {
                    const Node *d = produced_by(m->inputs[k], "Div");
                    float one;
                    if (d && d->inputs.size() == 2 && const_float(d->inputs[0], &one) &&
                        one == 1.0f && (sqrt_n = produced_by(d->inputs[1], "Sqrt"))) {
                        div_n = d;
                        mul_n = m;
                        x = m->inputs[1 - k];
                    }
                }
                if (!div_n) continue;
                recip = true;
            } else {
                continue;
            }
            const Node *add_n = produced_by(sqrt_n->inputs[0], "Add");
            if (!add_n || add_n->inputs.size() != 2) continue;
            float eps = 0.f;
            const Node *mean_n = nullptr;
            for (int k = 0; k < 2 && !mean_n; ++k)
                if (const_float(add_n->inputs[1 - k], &eps))
                    mean_n = produced_by(add_n->inputs[k], "ReduceMean");
            if (!mean_n) continue;
            if (attr_int(*mean_n, "keepdims", 1) != 1) continue;
            int64_t axis = 0;
            {
                std::vector<int64_t> axes;
                auto it = mean_n->attrs.find("axes");
                if (it != mean_n->attrs.end()) axes = it->second.ints;
                else if (mean_n->inputs.size() > 1 && !const_ints(mean_n->inputs[1], &axes)) continue;
                if (axes.size() != 1) continue;
                axis = axes[0];
            }
            const Node *pow_n = produced_by(mean_n->inputs[0], "Pow");
            float two;
            if (!pow_n || pow_n->inputs.size() != 2 || pow_n->inputs[0] != x ||
                !const_float(pow_n->inputs[1], &two) || two != 2.0f)
                continue;
            // every intermediate feeds the chain only
            if (!only_used_by(pow_n->outputs[0], {mean_n}) ||
                !only_used_by(mean_n->outputs[0], {add_n}) ||
                !only_used_by(add_n->outputs[0], {sqrt_n}) ||
                !only_used_by(sqrt_n->outputs[0], {div_n}))
                continue;
            if (recip) {
                if (!only_used_by(div_n->outputs[0], {mul_n}) ||
                    !only_used_by(mul_n->outputs[0], {&m2}))
                    continue;
            } else if (!only_used_by(div_n->outputs[0], {&m2})) {
                continue;
            }
            Node f;
            f.op = "rmlk.RMSNorm";
            f.inputs = {x, gamma};
            f.outputs = m2.outputs;
            f.attrs["epsilon"] = a_float(eps);
            f.attrs["reciprocal"] = a_int(recip ? 1 : 0);
            f.attrs["axis"] = a_int(axis);
            std::vector<const Node *> parts = {pow_n, mean_n, add_n, sqrt_n, div_n, &m2};
            if (mul_n) parts.push_back(mul_n);
            replace(parts, std::move(f));
            return true;
        }
        return false;
    }

    // ---- SwiGLU, anchored at the outer Mul -------------------------------------------------------
    bool match_swiglu(const Node &m2) {
        if (m2.op != "Mul" || m2.inputs.size() != 2) return false;
        for (int side = 0; side < 2; ++side) {
            const int silu = m2.inputs[side], up = m2.inputs[1 - side];
            const Node *m1 = produced_by(silu, "Mul");
            if (!m1 || m1->inputs.size() != 2 || up < 0) continue;
            for (int k = 0; k < 2; ++k) {
                const Node *sg = produced_by(m1->inputs[k], "Sigmoid");
                const int gate = m1->inputs[1 - k];
                if (!sg || sg->inputs[0] != gate) continue;
                if (!only_used_by(sg->outputs[0], {m1}) || !only_used_by(m1->outputs[0], {&m2}))
                    continue;
                Node f;
                f.op = "rmlk.SwiGLU";
                f.inputs = {gate, up};
                f.outputs = m2.outputs;
                replace({sg, m1, &m2}, std::move(f));
                return true;
            }
        }
        return false;
    }

    // ---- scale + mask + softmax, anchored at Softmax ----------------------------------------------
    bool match_softmax(const Node &sm) {
        if (sm.op != "Softmax" || sm.inputs.size() != 1) return false;
        const Node *add_n = produced_by(sm.inputs[0], "Add");
        if (!add_n || add_n->inputs.size() != 2) return false;
        for (int side = 0; side < 2; ++side) {
            const int scaled = add_n->inputs[side], mask = add_n->inputs[1 - side];
            if (mask < 0) continue;
            const Node *sc = produced_by(scaled, "Div");
            bool is_mul = false;
            int x = -1;
            float c = 0.f;
            if (sc) {
                if (sc->inputs.size() != 2 || !const_float(sc->inputs[1], &c)) continue;
                x = sc->inputs[0];
            } else if ((sc = produced_by(scaled, "Mul"))) {
                if (sc->inputs.size() != 2) continue;
                if (const_float(sc->inputs[1], &c)) x = sc->inputs[0];
                else if (const_float(sc->inputs[0], &c)) x = sc->inputs[1];
                else continue;
                is_mul = true;
            } else {
                continue;
            }
            if (x < 0) continue;
            if (!only_used_by(sc->outputs[0], {add_n}) || !only_used_by(add_n->outputs[0], {&sm}))
                continue;
            Node f;
            f.op = "rmlk.ScaleMaskSoftmax";
            f.inputs = {x, mask};
            f.outputs = sm.outputs;
            f.attrs["scale"] = a_float(c);
            f.attrs["scale_is_mul"] = a_int(is_mul ? 1 : 0);
            f.attrs["axis"] = a_int(attr_int(sm, "axis", -1));
            replace({sc, add_n, &sm}, std::move(f));
            return true;
        }
        return false;
    }

    // one-element constant input `i` of a Slice
    bool slice_param(const Node &sl, size_t i, int64_t *out) const {
        std::vector<int64_t> v;
        if (sl.inputs.size() <= i || !const_ints(sl.inputs[i], &v) || v.size() != 1) return false;
        *out = v[0];
        return true;
    }

    // ---- rotary embedding, anchored at the final Add ---------------------------------------------
    bool match_rotary(const Node &add) {
        if (add.op != "Add" || add.inputs.size() != 2) return false;
        for (int side = 0; side < 2; ++side) {
            const Node *ma = produced_by(add.inputs[side], "Mul");       // x * cos
            const Node *mr = produced_by(add.inputs[1 - side], "Mul");   // rotate_half(x) * sin
            if (!ma || !mr || ma == mr || ma->inputs.size() != 2 || mr->inputs.size() != 2) continue;
            for (int k = 0; k < 2; ++k) {
                const Node *cat = produced_by(mr->inputs[k], "Concat");
                const int sin_v = mr->inputs[1 - k];
                if (!cat || cat->inputs.size() != 2 || sin_v < 0) continue;
                const Node *neg = produced_by(cat->inputs[0], "Neg");
                const Node *s1 = produced_by(cat->inputs[1], "Slice");
                if (!neg || !s1) continue;
                const Node *s2 = produced_by(neg->inputs[0], "Slice");
                if (!s2 || s1 == s2) continue;
                const int x = s1->inputs[0];
                if (x < 0 || s2->inputs[0] != x) continue;
                int cos_v = -1;
                if (ma->inputs[0] == x) cos_v = ma->inputs[1];
                else if (ma->inputs[1] == x) cos_v = ma->inputs[0];
                if (cos_v < 0 || cos_v == x) continue;
                // Slice(x, [0], [h], [ax]) and Slice(x, [h], [>= 2h], [ax]), unit steps
                int64_t b1, e1, a1, b2, e2, a2, st;
                if (!slice_param(*s1, 1, &b1) || !slice_param(*s1, 2, &e1) ||
                    !slice_param(*s1, 3, &a1) || !slice_param(*s2, 1, &b2) ||
                    !slice_param(*s2, 2, &e2) || !slice_param(*s2, 3, &a2))
                    continue;
                if (s1->inputs.size() > 4 && s1->inputs[4] >= 0 &&
                    (!slice_param(*s1, 4, &st) || st != 1))
                    continue;
                if (s2->inputs.size() > 4 && s2->inputs[4] >= 0 &&
                    (!slice_param(*s2, 4, &st) || st != 1))
                    continue;
                if (b1 != 0 || e1 <= 0 || b2 != e1 || e2 < 2 * e1 || a1 != a2) continue;
                const int64_t cat_axis = attr_int(*cat, "axis", 0);
                if (!only_used_by(s1->outputs[0], {cat}) || !only_used_by(s2->outputs[0], {neg}) ||
                    !only_used_by(neg->outputs[0], {cat}) || !only_used_by(cat->outputs[0], {mr}) ||
                    !only_used_by(ma->outputs[0], {&add}) || !only_used_by(mr->outputs[0], {&add}))
                    continue;
                std::vector<const Node *> parts = {s1, s2, neg, cat, ma, mr, &add};
                int src = x;
                int64_t pre = 0;
                // a head-split Transpose feeding only this pattern is read through strides instead
                if (const Node *tr = produced_by(x, "Transpose")) {
                    auto it = tr->attrs.find("perm");
                    const std::vector<int64_t> want = {0, 2, 1, 3};
                    if (it != tr->attrs.end() && it->second.ints == want &&
                        only_used_by(x, {s1, s2, ma})) {
                        parts.push_back(tr);
                        src = tr->inputs[0];
                        pre = 1;
                    }
                }
                Node f;
                f.op = "rmlk.Rotary";
                f.inputs = {src, cos_v, sin_v};
                f.outputs = add.outputs;
                f.attrs["half"] = a_int(e1);
                f.attrs["end"] = a_int(e2);
                f.attrs["slice_axis"] = a_int(a1);
                f.attrs["concat_axis"] = a_int(cat_axis);
                f.attrs["transposed_input"] = a_int(pre);
                replace(parts, std::move(f));
                return true;
            }
        }
        return false;
    }

    static Attr a_ints(const std::vector<int64_t> &v) {
        Attr a;
        a.kind = Attr::Ints;
        a.ints = v;
        return a;
    }

    // ---- attention MatMul whose second operand is a transposed and / or group-expanded cache -------
    bool match_attn_matmul(const Node &mm) {
        if (mm.op != "MatMul" || mm.inputs.size() != 2 || mm.inputs[0] < 0) return false;
        std::vector<const Node *> parts;
        int cur = mm.inputs[1];
        const Node *user = &mm;
        bool transposed = false, expanded = false;
        std::vector<int64_t> expand_shape, reshape_shape;
        if (const Node *tr = produced_by(cur, "Transpose")) {
            auto it = tr->attrs.find("perm");
            const std::vector<int64_t> want = {0, 1, 3, 2};
            if (it != tr->attrs.end() && it->second.ints == want && only_used_by(cur, {user})) {
                transposed = true;
                parts.push_back(tr);
                cur = tr->inputs[0];
                user = tr;
            }
        }
        if (const Node *rs = produced_by(cur, "Reshape")) {
            const Node *ex = rs->inputs.size() == 2 ? produced_by(rs->inputs[0], "Expand") : nullptr;
            const Node *us = ex && ex->inputs.size() == 2 ? produced_by(ex->inputs[0], "Unsqueeze")
                                                          : nullptr;
            std::vector<int64_t> axes;
            bool axes_ok = false;
            if (us) {
                auto it = us->attrs.find("axes");
                if (it != us->attrs.end()) axes = it->second.ints;
                else if (us->inputs.size() > 1) const_ints(us->inputs[1], &axes);
                axes_ok = axes.size() == 1 && (axes[0] == 2 || axes[0] == -3);
            }
            if (us && axes_ok && attr_int(*rs, "allowzero", 0) == 0 &&
                const_ints(ex->inputs[1], &expand_shape) && const_ints(rs->inputs[1], &reshape_shape) &&
                only_used_by(cur, {user}) && only_used_by(rs->inputs[0], {rs}) &&
                only_used_by(ex->inputs[0], {ex})) {
                expanded = true;
                parts.push_back(rs);
                parts.push_back(ex);
                parts.push_back(us);
                cur = us->inputs[0];
            }
        }
        if (!transposed && !expanded) return false;
        parts.push_back(&mm);
        Node f;
        f.op = "rmlk.AttnMatMul";
        f.inputs = {mm.inputs[0], cur};
        f.outputs = mm.outputs;
        f.attrs["transposed"] = a_int(transposed ? 1 : 0);
        f.attrs["expanded"] = a_int(expanded ? 1 : 0);
        f.attrs["expand_shape"] = a_ints(expand_shape);
        f.attrs["reshape_shape"] = a_ints(reshape_shape);
        replace(parts, std::move(f));
        return true;
    }

    // ---- residual Add in front of an RMSNorm node: one pass, two outputs ---------------------------
    int form_add_rmsnorm() {
        int formed = 0;
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n] || g.nodes[n].op != "rmlk.RMSNorm") continue;
            const Node &norm = g.nodes[n];
            const int x = norm.inputs[0], gamma = norm.inputs[1];
            const Node *add = produced_by(x, "Add");
            if (!add || add->inputs.size() != 2 || add->inputs[0] < 0 || add->inputs[1] < 0) continue;
            // the fused node sits where the Add was: gamma must exist there already
            const int at = index_of(add);
            const Value &gv = g.values[gamma];
            if (!gv.is_initializer && !gv.is_input && !(gv.producer >= 0 && gv.producer < at)) continue;
            Node f;
            f.op = "rmlk.AddRMSNorm";
            f.inputs = {add->inputs[0], add->inputs[1], gamma};
            f.outputs = {x, norm.outputs[0]};
            f.attrs = norm.attrs;
            f.body = {*add, norm};
            auto &ux = users[x];
            ux.erase(std::remove(ux.begin(), ux.end(), static_cast<int>(n)), ux.end());
            auto &ug = users[gamma];
            ug.erase(std::remove(ug.begin(), ug.end(), static_cast<int>(n)), ug.end());
            ug.push_back(at);
            removed[n] = true;
            g.nodes[at] = std::move(f);
            for (int v : g.nodes[at].outputs) g.values[v].producer = at;
            ++formed;
        }
        return formed;
    }

    // ---- scores -> softmax -> context, all three already fused nodes: one attention node -----------
    int form_attention() {
        int formed = 0;
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n] || g.nodes[n].op != "rmlk.ScaleMaskSoftmax") continue;
            const Node &sm = g.nodes[n];
            const Node *qk = produced_by(sm.inputs[0], "rmlk.AttnMatMul");
            if (!qk || attr_int(*qk, "transposed", 0) != 1 || !only_used_by(qk->outputs[0], {&sm}))
                continue;
            const int probs = sm.outputs[0];
            if (g.values[probs].is_output || users[probs].size() != 1) continue;
            const Node &pv = g.nodes[users[probs][0]];
            // the context product: with the KV repeat folded in, or (one query head per KV head) plain
            const bool plain = pv.op == "MatMul" && pv.inputs.size() == 2;
            if (!plain && (pv.op != "rmlk.AttnMatMul" || attr_int(pv, "transposed", 0) != 0)) continue;
            if (pv.inputs[0] != probs || pv.inputs[1] == probs || pv.inputs[1] < 0) continue;
            Node f;
            f.op = "rmlk.Attention";
            f.inputs = {qk->inputs[0], qk->inputs[1], sm.inputs[1], pv.inputs[1]};
            f.outputs = pv.outputs;
            f.attrs["scale"] = sm.attrs.at("scale");
            f.attrs["scale_is_mul"] = sm.attrs.at("scale_is_mul");
            f.attrs["axis"] = sm.attrs.at("axis");
            for (const char *name : {"expanded", "expand_shape", "reshape_shape"}) {
                f.attrs[std::string("k_") + name] = qk->attrs.at(name);
                if (!plain) f.attrs[std::string("v_") + name] = pv.attrs.at(name);
            }
            // a Transpose to [B, S, H, D] behind the context (on the way to the output projection) is
            // a matter of where the kernel writes
            std::vector<const Node *> parts = {qk, &sm, &pv};
            const int ctx = pv.outputs[0];
            if (!g.values[ctx].is_output && users[ctx].size() == 1) {
                const Node &tr = g.nodes[users[ctx][0]];
                auto it = tr.attrs.find("perm");
                const std::vector<int64_t> want = {0, 2, 1, 3};
                if (tr.op == "Transpose" && it != tr.attrs.end() && it->second.ints == want) {
                    f.outputs = tr.outputs;
                    f.attrs["seq_major_output"] = a_int(1);
                    parts.push_back(&tr);
                }
            }
            replace(parts, std::move(f));
            ++formed;
        }
        return formed;
    }

    // ---- streams of head rows behind a projection: one launch -------------------------------------
    // A stream is an rmlk.Rotary node, or a ScatterND (reduction none) whose updates come from an
    // rmlk.Rotary node or from a head Transpose (0,2,1,3) that feed nothing else. Streams that follow
    // one another in the node list are gathered (up to four) into one rmlk.HeadRows node at the
    // position of the last, as long as nothing in between reads the result of an earlier one.
    int form_head_rows() {
        struct Stream {
            int kind;                  // see op_fused_head_rows
            int last;                  // node index of the stream's last node
            std::vector<int> nodes;
            std::vector<int> inputs;
            int output;
            int64_t transposed, half, end, slice_axis, concat_axis;
        };
        std::vector<Stream> streams;
        std::vector<bool> taken(g.nodes.size(), false);
        auto rotary_stream = [&](const Node &rot, Stream *st) {
            st->inputs = {rot.inputs[0], rot.inputs[1], rot.inputs[2]};
            st->transposed = attr_int(rot, "transposed_input", 0);
            st->half = attr_int(rot, "half", 0);
            st->end = attr_int(rot, "end", 0);
            st->slice_axis = attr_int(rot, "slice_axis", 0);
            st->concat_axis = attr_int(rot, "concat_axis", 0);
        };
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n] || g.nodes[n].op != "ScatterND") continue;
            const Node &sc = g.nodes[n];
            auto red = sc.attrs.find("reduction");
            if (red != sc.attrs.end() && red->second.s != "none") continue;
            if (sc.inputs.size() != 3 || sc.inputs[0] < 0 || sc.inputs[1] < 0 || sc.inputs[2] < 0) continue;
            const int upd = sc.inputs[2];
            if (upd == sc.inputs[0] || upd == sc.inputs[1]) continue;
            Stream st{};
            st.last = static_cast<int>(n);
            st.output = sc.outputs[0];
            if (const Node *rot = produced_by(upd, "rmlk.Rotary")) {
                if (!only_used_by(upd, {&sc})) continue;
                st.kind = 1;
                rotary_stream(*rot, &st);
                st.nodes = {index_of(rot), static_cast<int>(n)};
            } else if (const Node *tr = produced_by(upd, "Transpose")) {
                auto it = tr->attrs.find("perm");
                const std::vector<int64_t> want = {0, 2, 1, 3};
                if (it == tr->attrs.end() || it->second.ints != want || !only_used_by(upd, {&sc}) ||
                    tr->inputs[0] < 0)
                    continue;
                st.kind = 2;
                st.transposed = 1;
                st.inputs = {tr->inputs[0]};
                st.nodes = {index_of(tr), static_cast<int>(n)};
            } else {
                continue;
            }
            st.inputs.push_back(sc.inputs[0]);
            st.inputs.push_back(sc.inputs[1]);
            taken[st.nodes[0]] = true;
            streams.push_back(std::move(st));
        }
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n] || taken[n] || g.nodes[n].op != "rmlk.Rotary") continue;
            Stream st{};
            st.kind = 0;
            st.last = static_cast<int>(n);
            st.output = g.nodes[n].outputs[0];
            rotary_stream(g.nodes[n], &st);
            st.nodes = {static_cast<int>(n)};
            streams.push_back(std::move(st));
        }
        std::sort(streams.begin(), streams.end(),
                  [](const Stream &a, const Stream &b) { return a.last < b.last; });
        int formed = 0;
        size_t i = 0;
        while (i < streams.size()) {
            // grow the group while every earlier member's result is first read after the newcomer
            size_t j = i + 1;
            auto safe = [&](size_t upto) {
                for (size_t m = i; m < upto; ++m) {
                    for (int u : users[streams[m].output])
                        if (u <= streams[upto].last) return false;
                }
                return true;
            };
            while (j < streams.size() && j - i < 4 && safe(j)) ++j;
            const size_t count = j - i;
            const bool worth = count > 1 || streams[i].kind != 0;
            if (worth) {
                Node f;
                f.op = "rmlk.HeadRows";
                std::vector<int64_t> kinds, tr, half, end, sa, ca;
                std::vector<const Node *> parts;
                for (size_t m = i; m < j; ++m) {
                    const Stream &st = streams[m];
                    kinds.push_back(st.kind);
                    tr.push_back(st.transposed);
                    half.push_back(st.half);
                    end.push_back(st.end);
                    sa.push_back(st.slice_axis);
                    ca.push_back(st.concat_axis);
                    f.inputs.insert(f.inputs.end(), st.inputs.begin(), st.inputs.end());
                    f.outputs.push_back(st.output);
                    for (int k : st.nodes) parts.push_back(&g.nodes[k]);
                }
                f.attrs["kinds"] = a_ints(kinds);
                f.attrs["transposed"] = a_ints(tr);
                f.attrs["half"] = a_ints(half);
                f.attrs["end"] = a_ints(end);
                f.attrs["slice_axis"] = a_ints(sa);
                f.attrs["concat_axis"] = a_ints(ca);
                replace(parts, std::move(f));
                ++formed;
            }
            i = j;
        }
        return formed;
    }

    // ---- norms whose only reader is a product that can apply them itself (one-row inputs) -----------
    int mark_deferred_norms() {
        int marked = 0;
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n]) continue;
            Node &p = g.nodes[n];
            int normed = -1;
            if (p.op == "rmlk.RMSNorm") normed = p.outputs[0];
            else if (p.op == "rmlk.MatMulAddRMSNorm") normed = p.outputs[1];
            if (normed < 0 || g.values[normed].is_output || users[normed].size() != 1) continue;
            const Node &cons = g.nodes[users[normed][0]];
            const bool aware = (cons.op == "rmlk.MatMulGroup" || cons.op == "rmlk.MatMulGroupSwiGLU" ||
                                cons.op == "rmlk.MatMulConst") &&
                               cons.inputs.size() == 2 && cons.inputs[0] == normed && cons.inputs[1] != normed;
            if (!aware) continue;
            p.attrs["defer_norm"] = a_int(1);
            ++marked;
        }
        // (the same question for the gate / up product with its activation: does its result only feed
        // one product, the down projection? Then it may store that result as bfloat16 pieces as well.)
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n]) continue;
            Node &p = g.nodes[n];
            if (p.op != "rmlk.MatMulGroupSwiGLU") continue;
            const int act = p.outputs[0];
            if (g.values[act].is_output || users[act].size() != 1) continue;
            const Node &cons = g.nodes[users[act][0]];
            const bool product = (cons.op == "rmlk.MatMulAddRMSNorm" || cons.op == "rmlk.MatMulConst") &&
                                 cons.inputs.size() >= 2 && cons.inputs[0] == act && cons.inputs[1] != act;
            if (product) p.attrs["reader_is_product"] = a_int(1);
        }
        // (and for the attention node whose [B, S, H, D] result reaches the output projection through
        // a Reshape)
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n]) continue;
            Node &p = g.nodes[n];
            if (p.op != "rmlk.Attention") continue;
            const auto major = p.attrs.find("seq_major_output");
            if (major == p.attrs.end() || major->second.i == 0) continue;
            int value = p.outputs[0];
            for (int hop = 0; hop < 2; ++hop) {
                if (g.values[value].is_output || users[value].size() != 1) break;
                const Node &cons = g.nodes[users[value][0]];
                if (cons.op == "Reshape" && cons.inputs[0] == value) {
                    value = cons.outputs[0];
                    continue;
                }
                if ((cons.op == "rmlk.MatMulAddRMSNorm" || cons.op == "rmlk.MatMulConst") && cons.inputs.size() >= 2 &&
                    cons.inputs[0] == value && cons.inputs[1] != value)
                    p.attrs["reader_is_product"] = a_int(1);
                break;
            }
        }
        return marked;
    }

    // ---- joint one-row products whose members only feed one row-stream node -----------------------
    // (through a Reshape each: the q/k/v projection in front of rmlk.HeadRows). For a one-row input
    // such a product is left to the row-stream node, which runs it and its own work as one launch.
    int mark_deferred_products() {
        int marked = 0;
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n]) continue;
            Node &p = g.nodes[n];
            if (p.op != "rmlk.MatMulGroup") continue;
            int reader = -1;
            bool ok = true;
            for (int o : p.outputs) {
                if (g.values[o].is_output || users[o].size() != 1) { ok = false; break; }
                const Node &r = g.nodes[users[o][0]];
                if (r.op != "Reshape" || r.inputs.empty() || r.inputs[0] != o || r.outputs.size() != 1) { ok = false; break; }
                const int v = r.outputs[0];
                if (g.values[v].is_output || users[v].size() != 1) { ok = false; break; }
                const int h = users[v][0];
                if (g.nodes[h].op != "rmlk.HeadRows" || (reader >= 0 && h != reader)) { ok = false; break; }
                reader = h;
            }
            if (!ok || reader < 0) continue;
            p.attrs["defer_product"] = a_int(1);
            ++marked;
        }
        return marked;
    }

    // ---- a producer whose split-K combine can move into the consumer -----------------------------
    // (Tried for one-row inputs as well and dropped, both slower than what they replace: MatMul ->
    // AddRMSNorm, where the norm owns a row with ONE block that then adds up 32-64 slabs by itself;
    // and one kernel for scores -> softmax -> context of a decode step with one block per KV head,
    // where eight blocks cannot hide the HBM latency of a cold cache.)
    int form_splitk_epilogues() {
        int formed = 0;
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n]) continue;
            const Node &cons = g.nodes[n];
            if (cons.op == "rmlk.AddRMSNorm") {
                // a projection with constant 2-D weights feeding the residual Add: with many rows the
                // GEMM's split-K slabs are added up by the norm kernel (a one-row product keeps its
                // own combine, see above)
                for (int side = 0; side < 2; ++side) {
                    const Node *mm = produced_by(cons.inputs[side], "MatMul");
                    if (!mm || mm->inputs.size() != 2 || mm->inputs[0] < 0 || mm->inputs[1] < 0) continue;
                    const int w = mm->inputs[1];
                    if (!g.values[w].is_initializer || !s.values[w].defined() ||
                        s.values[w].dtype != RMLK_FLOAT || s.values[w].rank() != 2)
                        continue;
                    if (!only_used_by(mm->outputs[0], {&cons}) ||
                        cons.inputs[0] == cons.inputs[1])
                        continue;
                    const int wt = transposed_copy(w);
                    if (wt < 0) continue;   // (K no multiple of 4: the separate nodes stay)
                    Node f;
                    f.op = "rmlk.MatMulAddRMSNorm";
                    f.inputs = {mm->inputs[0], wt, cons.inputs[1 - side], cons.inputs[2]};
                    users[wt].push_back(static_cast<int>(n));
                    f.outputs = cons.outputs;
                    f.attrs = cons.attrs;
                    Node prod;   // the product on its own, for the cases the joint kernels decline
                    prod.op = "rmlk.MatMulConst";
                    prod.inputs = {mm->inputs[0], wt};
                    prod.outputs = mm->outputs;
                    Node norm = cons;
                    f.body = {prod, norm};
                    const int mi = index_of(mm);
                    const int act = mm->inputs[0];
                    for (int v : mm->inputs) {
                        auto &u = users[v];
                        u.erase(std::remove(u.begin(), u.end(), mi), u.end());
                    }
                    users[act].push_back(static_cast<int>(n));
                    removed[mi] = true;
                    g.nodes[n] = std::move(f);
                    release_unused(w);
                    ++formed;
                    break;
                }
                continue;
            }
            if (cons.op == "rmlk.SwiGLU") {
                const Node *grp = produced_by(cons.inputs[0], "rmlk.MatMulGroup");
                if (!grp || grp != produced_by(cons.inputs[1], "rmlk.MatMulGroup") ||
                    grp->outputs.size() != 2 || cons.inputs[0] == cons.inputs[1])
                    continue;
                if (!only_used_by(grp->outputs[0], {&cons}) || !only_used_by(grp->outputs[1], {&cons}))
                    continue;
                Node f;
                f.op = "rmlk.MatMulGroupSwiGLU";
                f.inputs = grp->inputs;
                f.outputs = cons.outputs;
                f.attrs = grp->attrs;
                f.attrs["gate_first"] = a_int(cons.inputs[0] == grp->outputs[0] ? 1 : 0);
                Node swiglu = cons;
                f.body = {*grp, swiglu};
                const int gi = index_of(grp);
                for (int v : grp->inputs) {
                    auto &u = users[v];
                    u.erase(std::remove(u.begin(), u.end(), gi), u.end());
                    u.push_back(static_cast<int>(n));
                }
                removed[gi] = true;
                g.nodes[n] = std::move(f);
                ++formed;
            }
        }
        return formed;
    }

    // The constant 2-D float matrix `w` ([k][n]) stored K-contiguous ([n][k]) as a new initializer;
    // -1 when w is not such a matrix or k is no multiple of 4. Every product of a fused node reads
    // its weights in this one form: a one-row product with a wavefront per output column and no
    // split-K combine, the GEMMs as their transposed-B variants (same sums in the same order as
    // over the row-major form). The row-major original is released once no node reads it.
    std::unordered_map<int, int> transposed_of;
    void release_unused(int w) {
        if (w >= 0 && users[w].empty() && !g.values[w].is_output && !g.values[w].is_input) s.values[w].reset();
    }
    // A float matrix [rows, k] in its own allocation.
    Tensor weight_matrix(int64_t rows, int64_t k, const char *what) {
        Tensor tt;
        tt.dtype = RMLK_FLOAT;
        tt.shape = {rows, k};
        auto buf = std::make_shared<Buffer>();
        buf->bytes = tt.nbytes();
        buf->owned_raw = true;
        check_hip(hipMalloc(&buf->ptr, buf->bytes), what);
        tt.buf = buf;
        return tt;
    }
    // The K-contiguous float matrix `tt` as the session holds it: itself, or (a session built with
    // 16-bit weight storage, rows of whole 128-bit units) rounded once to that type, the float form
    // released.
    // True when every value of the float matrix comes back from `storage` with the bits it has.
    int32_t *fit_flag = nullptr;   // device
    ~Matcher() {
        if (fit_flag) (void)hipFree(fit_flag);
    }
    bool fits(const Tensor &tt, int32_t storage) {
        if (!fit_flag) check_hip(hipMalloc(reinterpret_cast<void **>(&fit_flag), sizeof(int32_t)), "hipMalloc");
        int32_t one = 1;
        check_hip(hipMemcpy(fit_flag, &one, sizeof(one), hipMemcpyHostToDevice), "hipMemcpy");
        check_status(rmlk_hip_weights_fit(s.stream, storage, tt.numel(), tt.data(), fit_flag), "16-bit weights");
        check_hip(hipStreamSynchronize(s.stream), "hipStreamSynchronize");
        check_hip(hipMemcpy(&one, fit_flag, sizeof(one), hipMemcpyDeviceToHost), "hipMemcpy");
        return one != 0;
    }
    Tensor as_stored(const Tensor &tt) {
        check_hip(hipStreamSynchronize(s.stream), "hipStreamSynchronize");
        if (tt.shape[1] % 8 != 0) return tt;
        int32_t storage = s.weight_storage;
        if (storage == RMLK_FLOAT && s.lossless_16bit) {
            // (bfloat16 first: what checkpoints of this model family are trained and released in)
            if (fits(tt, RMLK_BFLOAT16)) storage = RMLK_BFLOAT16;
            else if (fits(tt, RMLK_FLOAT16)) storage = RMLK_FLOAT16;
        }
        if (storage == RMLK_FLOAT) return tt;
        ++s.weights_16bit;
        Tensor st;
        st.dtype = storage;
        st.shape = tt.shape;
        auto buf = std::make_shared<Buffer>();
        buf->bytes = st.nbytes();
        buf->owned_raw = true;
        check_hip(hipMalloc(&buf->ptr, buf->bytes), "hipMalloc (16-bit weights)");
        st.buf = buf;
        check_status(rmlk_hip_store_weights(s.stream, st.dtype, tt.numel(), tt.data(), st.data()), "16-bit weights");
        check_hip(hipStreamSynchronize(s.stream), "hipStreamSynchronize");
        return st;
    }
    int transposed_copy(int w) {
        auto it = transposed_of.find(w);
        if (it != transposed_of.end()) return it->second;
        if (w < 0 || !g.values[w].is_initializer) return -1;
        const Tensor &t = s.values[w];
        if (!t.defined() || t.dtype != RMLK_FLOAT || t.rank() != 2 || t.shape[0] == 0 || t.shape[1] == 0 ||
            t.shape[0] % 4 != 0)
            return -1;
        Tensor tt = weight_matrix(t.shape[1], t.shape[0], "hipMalloc (K-contiguous weights)");
        rmlk_dims in_shape = to_dims(t.shape);
        const int64_t perm[2] = {1, 0};
        check_status(rmlk_hip_transpose(s.stream, RMLK_FLOAT, &in_shape, perm, t.data(), tt.data()),
                     "K-contiguous weights");
        tt = as_stored(tt);
        const int id = static_cast<int>(g.values.size());
        Value v;
        v.name = "rmlk.k_contiguous." + std::to_string(w);
        v.dtype = tt.dtype;
        v.shape = tt.shape;
        v.is_initializer = true;
        g.values.push_back(v);
        g.by_name[v.name] = id;
        s.values.push_back(tt);
        users.emplace_back();
        transposed_of[w] = id;
        return id;
    }

    // ---- remaining MatMuls with constant 2-D weights (the lm-head) --------------------------------
    int form_const_matmuls() {
        int formed = 0;
        for (size_t n = 0; n < g.nodes.size(); ++n) {
            if (removed[n] || g.nodes[n].op != "MatMul") continue;
            const Node &mm = g.nodes[n];
            if (mm.inputs.size() != 2 || mm.inputs[0] < 0) continue;
            const int wt = transposed_copy(mm.inputs[1]);
            if (wt < 0) continue;
            const int w = mm.inputs[1];
            Node f;
            f.op = "rmlk.MatMulConst";
            f.inputs = {mm.inputs[0], wt};
            f.outputs = mm.outputs;
            users[wt].push_back(static_cast<int>(n));
            auto &u = users[w];
            u.erase(std::remove(u.begin(), u.end(), static_cast<int>(n)), u.end());
            g.nodes[n] = std::move(f);
            release_unused(w);
            ++formed;
        }
        return formed;
    }

    // ---- MatMuls that share their first operand and have constant 2-D weights (q/k/v, gate/up) ----
    // The weights are laid one below the other in ONE K-contiguous device matrix [N1 + N2 + .., K]
    // while building (the separate matrices are released unless something else reads them). A
    // one-row input then takes a single weight-streaming launch whose result is handed out as
    // views; more rows take one GEMM whose tiles write to the members' outputs, or one GEMM per
    // member on its block of rows, i.e. exactly the separate products. Nothing is left for a
    // fallback body.
    int form_matmul_groups() {
        int formed = 0;
        const size_t n_nodes = g.nodes.size();
        for (size_t first = 0; first < n_nodes; ++first) {
            if (removed[first] || g.nodes[first].op != "MatMul") continue;
            auto weight_ok = [&](const Node &mm, int64_t *k, int64_t *n) {
                if (mm.inputs.size() != 2 || mm.inputs[0] < 0 || mm.inputs[1] < 0) return false;
                const int w = mm.inputs[1];
                if (!g.values[w].is_initializer) return false;
                const Tensor &t = s.values[w];
                if (!t.defined() || t.dtype != RMLK_FLOAT || t.rank() != 2 || t.shape[1] % 4 != 0 ||
                    t.shape[0] % 4 != 0 || t.shape[0] == 0 || t.shape[1] == 0)
                    return false;
                *k = t.shape[0];
                *n = t.shape[1];
                return true;
            };
            int64_t k0, n0;
            if (!weight_ok(g.nodes[first], &k0, &n0)) continue;
            const int a = g.nodes[first].inputs[0];
            std::vector<size_t> members = {first};
            std::vector<int64_t> widths = {n0};
            for (size_t j = first + 1; j < n_nodes; ++j) {
                if (removed[j] || g.nodes[j].op != "MatMul" || g.nodes[j].inputs.empty() ||
                    g.nodes[j].inputs[0] != a)
                    continue;
                int64_t k, n;
                if (!weight_ok(g.nodes[j], &k, &n) || k != k0) continue;
                members.push_back(j);
                widths.push_back(n);
            }
            if (members.size() < 2) continue;
            int64_t total = 0;
            for (int64_t w : widths) total += w;
            // the joint weight matrix
            Tensor joint = weight_matrix(total, k0, "hipMalloc (joint weights)");
            int64_t off = 0;
            for (size_t i = 0; i < members.size(); ++i) {
                // member i transposed into its block of rows
                const Tensor &w = s.values[g.nodes[members[i]].inputs[1]];
                rmlk_dims in_shape = to_dims(w.shape);
                const int64_t perm[2] = {1, 0};
                check_status(rmlk_hip_transpose(s.stream, RMLK_FLOAT, &in_shape, perm, w.data(),
                                                static_cast<float *>(joint.data()) + off * k0),
                             "joint weights");
                off += widths[i];
            }
            joint = as_stored(joint);
            const int joint_id = static_cast<int>(g.values.size());
            Value jv;
            jv.name = "rmlk.joint_weights." + std::to_string(first);
            jv.dtype = joint.dtype;
            jv.shape = joint.shape;
            jv.is_initializer = true;
            g.values.push_back(jv);
            g.by_name[jv.name] = joint_id;
            s.values.push_back(joint);
            users.emplace_back();
            Node f;
            f.op = "rmlk.MatMulGroup";
            f.inputs = {a, joint_id};
            f.attrs["widths"] = a_ints(widths);
            for (size_t i = 0; i < members.size(); ++i) {
                const Node &mm = g.nodes[members[i]];
                f.outputs.push_back(mm.outputs[0]);
                const int w = mm.inputs[1];
                removed[members[i]] = true;
                for (int v : mm.inputs) {
                    auto &u = users[v];
                    u.erase(std::remove(u.begin(), u.end(), static_cast<int>(members[i])), u.end());
                }
                // release a weight nobody else reads (another member may share it)
                if (users[w].empty() && !g.values[w].is_output) s.values[w].reset();
            }
            g.nodes[first] = std::move(f);
            removed[first] = false;
            users[a].push_back(static_cast<int>(first));
            users[joint_id].push_back(static_cast<int>(first));
            for (int v : g.nodes[first].outputs) g.values[v].producer = static_cast<int>(first);
            ++formed;
        }
        return formed;
    }
};

// Run the nodes a fused node replaced, one kernel each.
void run_body(OpContext &c) {
    Session &s = c.session;
    std::unordered_map<int, Tensor> local;
    // the fused node's own inputs come from its context (a body may be nested inside another body,
    // whose intermediates are not session values)
    for (size_t i = 0; i < c.node.inputs.size(); ++i)
        if (c.node.inputs[i] >= 0 && c.in[i]) local[c.node.inputs[i]] = *c.in[i];
    auto lookup = [&](int v) -> Tensor * {
        auto it = local.find(v);
        return it != local.end() ? &it->second : &s.values[v];
    };
    for (const Node &n : c.node.body) {
        OpContext sub{s, n, c.node_index, {}, {}, c.stream};
        for (int v : n.inputs) sub.in.push_back(v < 0 ? nullptr : lookup(v));
        std::vector<Tensor> outs(n.outputs.size());
        for (size_t o = 0; o < outs.size(); ++o) sub.out.push_back(&outs[o]);
        find_op(n.op)(sub);
        for (size_t o = 0; o < outs.size(); ++o) local[n.outputs[o]] = outs[o];
    }
    for (size_t o = 0; o < c.node.outputs.size(); ++o) *c.out[o] = local[c.node.outputs[o]];
}

void require_float(int32_t dt) {
    if (dt != RMLK_FLOAT) fail_unsupported(dt);
}


float attr_float(const OpContext &c, const char *name) {
    const Attr *a = c.attr(name);
    return a ? a->f : 0.f;
}

// status of a fused kernel: UNSUPPORTED means "not this layout", anything else is an error
bool took_fast_path(int32_t st, const char *what) {
    if (st == RMLK_ERR_UNSUPPORTED) return false;
    check_status(st, what);
    return true;
}

// ---- many-row products over bfloat16 weights on the bf16 matrix cores ----------------------------
// With Session::bf16_pieces a product of 64 and more rows over a weight matrix held as bfloat16
// values splits its first operand into three bfloat16 pieces (exactly) and multiplies those
// (rmlk_hip_matmul_bf16x3). The pieces live in the session workspace, behind `own` bytes that the
// caller wants there for itself.
bool wants_pieces(const OpContext &c, int64_t m, int64_t k, int32_t w_dtype) {
    // (the kernels address the pieces with 32 bits: no workspace is asked for an operand they refuse)
    return c.session.bf16_pieces && w_dtype == RMLK_BFLOAT16 && m >= 64 && k % 32 == 0 &&
           rmlk_hip_bf16x3_pieces_size(m, k) < (static_cast<size_t>(1) << 32);
}

// Splits a [m, k] (dense rows); returns the pieces, null when the split does not take the operand.
// *own_out: the caller's part of the workspace. `src`: the tensor a belongs to, which may carry its
// pieces already (a norm that stored them for this reader).
void *split_pieces(OpContext &c, const void *a, int64_t m, int64_t k, size_t own, void **own_out,
                   const char *what, const Tensor *src = nullptr) {
    if (src && src->pieces && src->data() == a && src->pieces->nbytes() == rmlk_hip_bf16x3_pieces_size(m, k)) {
        if (own_out) *own_out = own ? c.scratch(own) : nullptr;
        return src->pieces->data();
    }
    const size_t own_bytes = (own + 255) / 256 * 256;
    char *ws = static_cast<char *>(c.scratch(own_bytes + rmlk_hip_bf16x3_pieces_size(m, k)));
    if (own_out) *own_out = ws;
    void *pieces = ws + own_bytes;
    return took_fast_path(rmlk_hip_bf16x3_split(c.stream, m, k, a, k, pieces), what) ? pieces : nullptr;
}

// A many-row norm (or gate / up product: mark `reader_is_product`) whose result has one reader, a
// product (the `defer_norm` mark of the fusion pass), in a session that multiplies over bfloat16 weights on the bf16 matrix cores: room for the pieces of
// its [rows, cols] result, which the norm kernel then writes itself. Undefined when not wanted.
Tensor room_for_pieces(OpContext &c, int64_t rows, int64_t cols, const char *mark = "defer_norm") {
    Tensor t;
    if (!c.session.bf16_pieces || c.session.weights_16bit == 0 || c.attr_int(mark, 0) == 0 || rows < 64 ||
        cols % 32 != 0)
        return t;
    const size_t bytes = rmlk_hip_bf16x3_pieces_size(rows, cols);
    if (bytes >= (static_cast<size_t>(1) << 32)) return t;
    std::vector<Tensor *> keep = c.out;
    c.out = {&t};
    c.alloc_output(0, RMLK_UINT8, {static_cast<int64_t>(bytes)});
    c.out = keep;
    return t;
}

// ---- one-row RMSNorm left to the product that reads it ------------------------------------------
// A norm node marked `defer_norm` (its result feeds exactly one product over K-contiguous constant
// weights) does not run for a one-row input: its output is a view of the row BEFORE the norm that
// carries the norm's parameters (Tensor::pending_norm), and the product's kernel normalises the
// row while it loads it (rmlk_hip_gemv_kmajor_normed). One launch less per norm of a decode step.
constexpr int64_t kMaxDeferredNormCols = 8192;   // what the product kernels accept
constexpr int64_t kMaxDeferredNormWidth = 16384; // output columns up to which a product applies the norm

bool may_defer_norm(const OpContext &c, const Tensor &row, const Tensor &gamma) {
    const int64_t cols = row.shape.empty() ? 0 : row.shape.back();
    return c.attr_int("defer_norm", 0) != 0 && row.dtype == RMLK_FLOAT && gamma.dtype == RMLK_FLOAT &&
           cols > 0 && row.numel() == cols && cols % 4 == 0 && cols <= kMaxDeferredNormCols &&
           gamma.numel() == cols;
}

void defer_norm(OpContext &c, int out_index, const Tensor &row, const Tensor &gamma) {
    Tensor &y = c.view_output(out_index, row, row.shape);
    auto pn = std::make_shared<PendingNorm>();
    pn->gamma = gamma;
    pn->eps = attr_float(c, "epsilon");
    pn->reciprocal = static_cast<int32_t>(c.attr_int("reciprocal", 0));
    y.pending_norm = pn;
}

// The consumer's side: input 0 with a pending norm is replaced by the computed norm (a tensor of
// the context's own) when the consumer is not going to apply it itself.
void compute_pending_norm(OpContext &c) {
    const Tensor &row = c.input(0);
    const PendingNorm &pn = *row.pending_norm;
    c.temps.emplace_back();
    Tensor *store = &c.temps.back();
    {
        std::vector<Tensor *> keep = c.out;
        c.out = {store};
        c.alloc_output(0, RMLK_FLOAT, row.shape);
        c.out = keep;
    }
    const int64_t cols = row.shape.back();
    check_status(rmlk_hip_rmsnorm(c.stream, RMLK_FLOAT, row.numel() / cols, cols, row.data(), pn.gamma.data(),
                                  pn.eps, pn.reciprocal, store->data()),
                 "rmlk.RMSNorm (deferred)");
    c.in[0] = store;
}

// The Unsqueeze -> Expand -> Reshape chain folded into an attention product must repeat every KV
// head of kv [B, G, L, D] `rep` times in place ([B, G * rep, L, D]); false when the recorded shapes
// say anything else.
bool kv_repeat(const std::vector<int64_t> &e, const std::vector<int64_t> &r, const Tensor &kv, int64_t *rep) {
    const int64_t in5[5] = {kv.shape[0], kv.shape[1], 1, kv.shape[2], kv.shape[3]};
    if (e.size() != 5 || r.size() != 4) return false;
    for (int d = 0; d < 5; ++d)
        if (d != 2 && e[d] != 1 && e[d] != in5[d]) return false;
    *rep = e[2];
    if (*rep < 1) return false;
    // the Reshape must give [B, G * rep, L, D] (0 copies a dim, one -1 is inferred)
    const int64_t ex5[5] = {in5[0], in5[1], *rep, in5[3], in5[4]};
    const int64_t want[4] = {ex5[0], ex5[1] * *rep, ex5[3], ex5[4]};
    int64_t total = 1, known = 1;
    for (int64_t d : ex5) total *= d;
    int infer = -1;
    int64_t got[4];
    for (int d = 0; d < 4; ++d) {
        if (r[d] == -1) {
            if (infer >= 0) return false;
            infer = d;
            got[d] = 1;
        } else if (r[d] == 0) {
            got[d] = ex5[d];
            known *= got[d];
        } else {
            got[d] = r[d];
            known *= got[d];
        }
    }
    if (infer >= 0) {
        if (known <= 0 || total % known != 0) return false;
        got[infer] = total / known;
    }
    for (int d = 0; d < 4; ++d)
        if (got[d] != want[d]) return false;
    return true;
}

// Element strides of `mask` per dim of `shape` when it broadcasts INTO that shape with a full last
// dim; false otherwise.
bool mask_strides(const Tensor &mask, const std::vector<int64_t> &shape, rmlk_dims *out) {
    const int rank = static_cast<int>(shape.size());
    if (mask.rank() == 0 || mask.rank() > rank || mask.shape.back() != shape.back()) return false;
    std::vector<int64_t> st(rank, 0), dense = dense_strides(mask.shape);
    const int shift = rank - mask.rank();
    for (int d = 0; d < mask.rank(); ++d) {
        const int64_t md = mask.shape[d], xd = shape[d + shift];
        if (md == xd) st[d + shift] = md == 1 ? 0 : dense[d];
        else if (md == 1) st[d + shift] = 0;
        else return false;
    }
    st[rank - 1] = 1;
    *out = to_dims(st);
    return true;
}

}  // namespace

void op_fused_rmsnorm(OpContext &c) {
    const Tensor &x = c.input(0), &gamma = c.input(1);
    const int rank = x.rank();
    bool ok = x.dtype == RMLK_FLOAT && gamma.dtype == RMLK_FLOAT && rank >= 1 && x.numel() > 0;
    if (ok) {
        const int64_t axis = c.attr_int("axis", -1);
        ok = axis == -1 || axis == rank - 1;
    }
    if (ok) {
        // gamma broadcasts along the rows only: [cols] or [1, .., 1, cols]
        ok = gamma.rank() >= 1 && gamma.rank() <= rank && gamma.shape.back() == x.shape.back() &&
             gamma.numel() == x.shape.back();
    }
    if (ok && may_defer_norm(c, x, gamma)) {
        defer_norm(c, 0, x, gamma);
        return;
    }
    if (ok) {
        const int64_t cols = x.shape.back(), rows = x.numel() / cols;
        Tensor &y = c.alloc_output(0, RMLK_FLOAT, x.shape);
        if (Tensor pieces = room_for_pieces(c, rows, cols); pieces.defined()) {
            if (took_fast_path(rmlk_hip_rmsnorm_pieces(c.stream, rows, cols, x.data(), 1, 0, nullptr, gamma.data(),
                                                       attr_float(c, "epsilon"),
                                                       static_cast<int32_t>(c.attr_int("reciprocal", 0)), nullptr,
                                                       y.data(), pieces.data()),
                               "rmlk.RMSNorm")) {
                y.pieces = std::make_shared<const Tensor>(std::move(pieces));
                return;
            }
        }
        if (took_fast_path(rmlk_hip_rmsnorm(c.stream, RMLK_FLOAT, rows, cols, x.data(), gamma.data(),
                                            attr_float(c, "epsilon"),
                                            static_cast<int32_t>(c.attr_int("reciprocal", 0)),
                                            y.data()),
                           "rmlk.RMSNorm"))
            return;
    }
    run_body(c);
}

void op_fused_swiglu(OpContext &c) {
    const Tensor &g = c.input(0), &u = c.input(1);
    if (g.dtype == RMLK_FLOAT && u.dtype == RMLK_FLOAT && g.shape == u.shape) {
        Tensor &y = c.alloc_output(0, RMLK_FLOAT, g.shape);
        if (took_fast_path(rmlk_hip_swiglu(c.stream, RMLK_FLOAT, g.numel(), g.data(), u.data(),
                                           y.data()),
                           "rmlk.SwiGLU"))
            return;
    }
    run_body(c);
}

void op_fused_softmax(OpContext &c) {
    const Tensor &x = c.input(0), &mask = c.input(1);
    const int rank = x.rank();
    bool ok = x.dtype == RMLK_FLOAT && mask.dtype == RMLK_FLOAT && rank >= 1 &&
              mask.rank() <= rank && x.numel() > 0;
    if (ok) {
        const int64_t axis = c.attr_int("axis", -1);
        ok = axis == -1 || axis == rank - 1;
    }
    rmlk_dims ms{};
    if (ok) ok = mask_strides(mask, x.shape, &ms);
    if (ok) {
        rmlk_dims xs = to_dims(x.shape);
        Tensor &y = c.alloc_output(0, RMLK_FLOAT, x.shape);
        if (took_fast_path(rmlk_hip_scale_mask_softmax(
                               c.stream, RMLK_FLOAT, &xs, &ms,
                               static_cast<int32_t>(c.attr_int("scale_is_mul", 0)),
                               attr_float(c, "scale"), x.data(), mask.data(), y.data()),
                           "rmlk.ScaleMaskSoftmax"))
            return;
    }
    run_body(c);
}

namespace {

// Layout of one stream of head rows: the logical [B,H,S,D] shape of `src` (seen through a
// Transpose 0,2,1,3 when `pre`), its element strides, and, with rotary tables, their broadcast
// strides into that shape. False when the rotary kernels do not cover the case.
struct RowLayout {
    std::vector<int64_t> shape, xst;
    rmlk_dims cs{}, ss{};
};
bool row_layout(const Tensor &src, bool pre, RowLayout *out) {
    if (src.dtype != RMLK_FLOAT || src.rank() != 4 || src.numel() == 0) return false;
    std::vector<int64_t> dense = dense_strides(src.shape);
    if (pre) {  // logical x = Transpose(src, 0,2,1,3)
        out->shape = {src.shape[0], src.shape[2], src.shape[1], src.shape[3]};
        out->xst = {dense[0], dense[2], dense[1], dense[3]};
    } else {
        out->shape = src.shape;
        out->xst = dense;
    }
    return true;
}
bool rotary_layout(const Tensor &src, const Tensor &cos_t, const Tensor &sin_t, bool pre, int64_t half,
                   int64_t end, int64_t slice_axis, int64_t concat_axis, RowLayout *out) {
    if (cos_t.dtype != RMLK_FLOAT || sin_t.dtype != RMLK_FLOAT || cos_t.rank() > 4 || sin_t.rank() > 4 ||
        !row_layout(src, pre, out))
        return false;
    const std::vector<int64_t> &shape = out->shape;
    const int64_t d = shape[3];
    auto axis_ok = [](int64_t a) { return a == 3 || a == -1; };
    if (d != 2 * half || end < d || !axis_ok(slice_axis) || !axis_ok(concat_axis)) return false;
    auto table_strides = [&](const Tensor &t, rmlk_dims *st_out) {
        // broadcast INTO `shape`, last dim full
        std::vector<int64_t> st(4, 0), dense = dense_strides(t.shape);
        const int shift = 4 - t.rank();
        for (int k = 0; k < t.rank(); ++k) {
            const int64_t td = t.shape[k], xd = shape[k + shift];
            if (td == xd) st[k + shift] = td == 1 ? 0 : dense[k];
            else if (td != 1) return false;
        }
        if (t.rank() == 0 || t.shape.back() != shape[3]) return false;
        st[3] = 1;
        *st_out = to_dims(st);
        return true;
    };
    return table_strides(cos_t, &out->cs) && table_strides(sin_t, &out->ss);
}

}  // namespace

void op_fused_rotary(OpContext &c) {
    const Tensor &src = c.input(0), &cos_t = c.input(1), &sin_t = c.input(2);
    RowLayout lay;
    if (rotary_layout(src, cos_t, sin_t, c.attr_int("transposed_input", 0) != 0, c.attr_int("half", 0),
                      c.attr_int("end", 0), c.attr_int("slice_axis", 0), c.attr_int("concat_axis", 0),
                      &lay)) {
        rmlk_dims sd = to_dims(lay.shape), xs = to_dims(lay.xst);
        Tensor &y = c.alloc_output(0, RMLK_FLOAT, lay.shape);
        if (took_fast_path(rmlk_hip_rotary(c.stream, RMLK_FLOAT, &sd, &xs, &lay.cs, &lay.ss, src.data(),
                                           cos_t.data(), sin_t.data(), y.data()),
                           "rmlk.Rotary"))
            return;
    }
    run_body(c);
}

// A one-row product that was left to its reader and has to be stored after all.
void store_product(OpContext &c, PendingProduct &pp) {
    if (pp.m > 0) {
        // many rows, partial sums not added up: the members' outputs by the grouped product
        std::vector<void *> outs;
        for (Tensor &t : pp.outs) outs.push_back(t.data());
        const size_t ws_bytes = rmlk_hip_matmul_grouped_workspace_size(
            RMLK_FLOAT, pp.m, pp.k, static_cast<int32_t>(pp.widths.size()), pp.widths.data());
        void *ws = ws_bytes ? c.scratch(ws_bytes) : nullptr;
        check_status(rmlk_hip_matmul_grouped(c.stream, RMLK_FLOAT, pp.m, pp.k, pp.x.data(), pp.k, pp.wt.dtype, pp.wt.data(),
                                             pp.k, 1, static_cast<int32_t>(pp.widths.size()), pp.widths.data(),
                                             outs.data(), ws, ws_bytes),
                     "rmlk.MatMulGroup (deferred)");
        pp.computed = true;
        return;
    }
    int32_t st;
    if (pp.norm)
        st = rmlk_hip_gemv_kmajor_normed(c.stream, RMLK_FLOAT, pp.total, pp.k, pp.x.data(), pp.norm->gamma.data(),
                                         pp.norm->eps, pp.norm->reciprocal, pp.wt.dtype, pp.wt.data(), pp.k, pp.row.data());
    else
        st = rmlk_hip_gemv_kmajor(c.stream, RMLK_FLOAT, pp.total, pp.k, pp.x.data(), pp.wt.dtype, pp.wt.data(), pp.k,
                                  pp.row.data());
    if (st == RMLK_ERR_UNSUPPORTED && pp.norm) {
        // (a row the one-row kernels refuse to normalise: norm, then product)
        Tensor normed;
        std::vector<Tensor *> keep = c.out;
        c.out = {&normed};
        c.alloc_output(0, RMLK_FLOAT, pp.x.shape);
        c.out = keep;
        check_status(rmlk_hip_rmsnorm(c.stream, RMLK_FLOAT, 1, pp.k, pp.x.data(), pp.norm->gamma.data(),
                                      pp.norm->eps, pp.norm->reciprocal, normed.data()),
                     "rmlk.RMSNorm (deferred)");
        st = rmlk_hip_gemv_kmajor(c.stream, RMLK_FLOAT, pp.total, pp.k, normed.data(), pp.wt.dtype, pp.wt.data(), pp.k,
                                  pp.row.data());
    }
    check_status(st, "rmlk.MatMulGroup (deferred)");
    pp.computed = true;
}

// Streams of head rows (rmlk.HeadRows): per stream, by `kinds`,
//   0  rmlk.Rotary                                 inputs src, cos, sin
//   1  rmlk.Rotary -> ScatterND(data, idx, .)      inputs src, cos, sin, data, idx
//   2  Transpose(0,2,1,3) -> ScatterND(data, idx, .)   inputs src, data, idx
// one output each, all in one launch. The ScatterND destinations follow op_scatter_nd (in place
// where the data tensor may be overwritten, else a copy first).
void op_fused_head_rows(OpContext &c) {
    const std::vector<int64_t> kinds = c.attr_ints("kinds"), pre = c.attr_ints("transposed"),
                               half = c.attr_ints("half"), end = c.attr_ints("end"),
                               slice_axis = c.attr_ints("slice_axis"),
                               concat_axis = c.attr_ints("concat_axis");
    const size_t n = kinds.size();
    std::vector<RowLayout> lay(n);
    std::vector<int> first_input(n);
    bool ok = n > 0 && n <= 4;
    int at = 0;
    int64_t d_common = -1;
    for (size_t i = 0; i < n && ok; ++i) {
        first_input[i] = at;
        const Tensor &src = c.input(at);
        int data_at = -1;
        if (kinds[i] == 2) {
            ok = row_layout(src, pre[i] != 0, &lay[i]);
            data_at = at + 1;
            at += 3;
        } else {
            ok = rotary_layout(src, c.input(at + 1), c.input(at + 2), pre[i] != 0, half[i], end[i],
                               slice_axis[i], concat_axis[i], &lay[i]);
            if (kinds[i] == 1) data_at = at + 3;
            at += kinds[i] == 1 ? 5 : 3;
        }
        if (!ok) break;
        const int64_t d = lay[i].shape[3];
        ok = d % 2 == 0 && (d_common < 0 || d == d_common);
        d_common = d;
        if (ok && data_at >= 0) {
            // ScatterND(reduction none) writing whole rows: one index tuple per row, in row order
            const Tensor &data = c.input(data_at), &idx = c.input(data_at + 1);
            ok = data.dtype == RMLK_FLOAT && idx.dtype == RMLK_INT64 && data.rank() >= 2 &&
                 data.rank() <= 5 && idx.rank() == 4 && idx.shape[3] == data.rank() - 1 &&
                 data.shape.back() == d && idx.shape[0] == lay[i].shape[0] &&
                 idx.shape[1] == lay[i].shape[1] && idx.shape[2] == lay[i].shape[2] &&
                 data.numel() > 0;
        }
    }
    // Sources that are members of a one-row product left to this node (op_fused_matmul_group): the
    // product and the row streams run as one launch when every source is a member of the same
    // product and a [1, H, 1, D] tensor with its heads side by side; otherwise the product is
    // computed first, and everything below finds its rows in memory.
    std::shared_ptr<PendingProduct> product;
    bool one_launch = ok, from_slabs = false;
    std::vector<int64_t> slab_col(n, 0);
    {
        std::vector<std::shared_ptr<PendingProduct>> seen;
        int at_src = 0;
        for (size_t i = 0; i < n; ++i) {
            const Tensor &src = c.input(at_src);
            at_src += kinds[i] == 2 ? 3 : (kinds[i] == 1 ? 5 : 3);
            const std::shared_ptr<PendingProduct> &pp = src.pending_product;
            if (!pp || pp->computed) {
                one_launch = false;
                continue;
            }
            if (std::find(seen.begin(), seen.end(), pp) == seen.end()) seen.push_back(pp);
            if (ok) {
                const std::vector<int64_t> &sh = lay[i].shape, &xs = lay[i].xst;
                if (sh[0] != 1 || sh[2] != 1 || xs[1] != sh[3] || xs[3] != 1) one_launch = false;
            }
        }
        if (seen.size() != 1) one_launch = false;
        // a many-row product whose partial sums were left in their slabs: every source is a member
        // of it, seen as [B, S, H, D] rows of the joint matrix
        if (ok && seen.size() == 1 && seen[0]->m > 0) {
            const PendingProduct &pp = *seen[0];
            from_slabs = true;
            int at_m = 0;
            for (size_t i = 0; i < n && from_slabs; ++i) {
                const Tensor &src = c.input(at_m);
                at_m += kinds[i] == 2 ? 3 : (kinds[i] == 1 ? 5 : 3);
                int member = -1;
                int64_t col = 0;
                for (size_t j = 0; j < pp.outs.size(); ++j) {
                    if (src.pending_product && pp.outs[j].buf == src.buf && pp.outs[j].offset == src.offset) {
                        member = static_cast<int>(j);
                        break;
                    }
                    col += pp.widths[j];
                }
                from_slabs = member >= 0 && pre[i] != 0 && src.rank() == 4 &&
                             src.shape[0] * src.shape[1] == pp.m && src.shape[2] * src.shape[3] == pp.widths[member];
                slab_col[i] = col;
            }
            one_launch = false;
        }
        if (one_launch || from_slabs) {
            product = seen[0];
        } else {
            for (const std::shared_ptr<PendingProduct> &pp : seen) store_product(c, *pp);
        }
    }
    if (!ok) {
        run_body(c);
        return;
    }
    std::vector<rmlk_row_stream> streams(n);
    std::vector<int64_t> first_col(n, 0);
    std::vector<void *> copy_dst;
    std::vector<const void *> copy_src;
    std::vector<size_t> copy_bytes;
    for (size_t i = 0; i < n; ++i) {
        rmlk_row_stream &st = streams[i];
        st = rmlk_row_stream{};
        int in = first_input[i];
        if (product && !from_slabs)
            first_col[i] = static_cast<int64_t>(c.input(in).offset - product->row.offset) / static_cast<int64_t>(sizeof(float));
        st.shape = to_dims(lay[i].shape);
        st.x_stride = to_dims(lay[i].xst);
        st.x = c.input(in++).data();
        if (from_slabs) {
            // logical [B, H, S, D] over the rows (b, s) of the joint matrix, `total` columns wide
            const PendingProduct &pp = *product;
            const int64_t seq = lay[i].shape[2], d = lay[i].shape[3];
            st.x_stride = to_dims({seq * pp.total, d, pp.total, 1});
            st.x = static_cast<const float *>(pp.slabs.data()) + slab_col[i];
            st.partials = pp.splits;
            st.partial_stride = pp.slab;
        }
        if (kinds[i] != 2) {
            st.cos = c.input(in++).data();
            st.sin = c.input(in++).data();
            st.cos_stride = lay[i].cs;
            st.sin_stride = lay[i].ss;
        }
        if (kinds[i] == 0) {
            st.out = c.alloc_output(static_cast<int>(i), RMLK_FLOAT, lay[i].shape).data();
        } else {
            const Tensor &data = c.input(in), &idx = c.input(in + 1);
            st.data_shape = to_dims(data.shape);
            st.tuple_size = static_cast<int32_t>(data.rank() - 1);
            st.idx = static_cast<const int64_t *>(idx.data());
            // a destination that has to be a copy of its data tensor: the copies of all streams go
            // out as one launch below
            bool copy_here = false;
            Tensor &dest = scatter_destination(c, in, static_cast<int>(i), &copy_here);
            st.out = dest.data();
            if (copy_here && data.nbytes() > 0) {
                copy_dst.push_back(dest.data());
                copy_src.push_back(data.data());
                copy_bytes.push_back(data.nbytes());
            }
        }
    }
    if (!copy_dst.empty())
        check_status(rmlk_hip_memcpy_dtod_many(c.stream, static_cast<int32_t>(copy_dst.size()), copy_dst.data(),
                                               copy_src.data(), copy_bytes.data()),
                     "ScatterND copy");
    if (product && from_slabs) {
        if (took_fast_path(rmlk_hip_head_rows(c.stream, RMLK_FLOAT, static_cast<int32_t>(n), streams.data(),
                                              c.error_flag()),
                           "rmlk.HeadRows (over partial sums)")) {
            product->computed = true;   // consumed: nothing else reads its members
            return;
        }
        // the kernel refuses these operands: the members stored after all, then the streams over them
        store_product(c, *product);
        for (size_t i = 0; i < n; ++i) {
            streams[i].x = c.input(first_input[i]).data();
            streams[i].x_stride = to_dims(lay[i].xst);
            streams[i].partials = 0;
            streams[i].partial_stride = 0;
        }
    } else if (product) {
        const PendingProduct &pp = *product;
        const int32_t st = rmlk_hip_gemv_kmajor_head_rows(
            c.stream, RMLK_FLOAT, pp.k, pp.x.data(), pp.norm ? pp.norm->gamma.data() : nullptr,
            pp.norm ? pp.norm->eps : 0.f, pp.norm ? pp.norm->reciprocal : 0, pp.wt.dtype, pp.wt.data(), pp.k,
            static_cast<int32_t>(n), streams.data(), first_col.data(), c.error_flag());
        if (took_fast_path(st, "rmlk.HeadRows (with its projection)")) {
            product->computed = true;   // consumed: nothing else reads its members
            return;
        }
        // the one-row kernels refuse these operands: the product on its own, then the streams
        store_product(c, *product);
    }
    if (took_fast_path(rmlk_hip_head_rows(c.stream, RMLK_FLOAT, static_cast<int32_t>(n), streams.data(),
                                          c.error_flag()),
                       "rmlk.HeadRows"))
        return;
    run_body(c);
}

// MatMul(a [B,H,S,K], f(kv [B,G,L,D])) where f repeats every cache head H / G times (Unsqueeze,
// Expand, Reshape) and / or swaps the last two dims: one strided GEMM with batch B * G and
// M = (H / G) * S reads the cache in place; neither the repeated nor the transposed copy is made.
void op_fused_attn_matmul(OpContext &c) {
    const Tensor &a = c.input(0), &kv = c.input(1);
    const bool transposed = c.attr_int("transposed", 0) != 0;
    const bool expanded = c.attr_int("expanded", 0) != 0;
    bool ok = a.dtype == RMLK_FLOAT && kv.dtype == RMLK_FLOAT && a.rank() == 4 && kv.rank() == 4 &&
              a.numel() > 0 && kv.numel() > 0;
    int64_t rep = 1;
    if (ok && expanded) ok = kv_repeat(c.attr_ints("expand_shape"), c.attr_ints("reshape_shape"), kv, &rep);
    if (ok) {
        const int64_t bsz = kv.shape[0], grp = kv.shape[1], len = kv.shape[2], dim = kv.shape[3];
        const int64_t heads = a.shape[1], seq = a.shape[2], ka = a.shape[3];
        const int64_t n = transposed ? len : dim, k = transposed ? dim : len;
        ok = a.shape[0] == bsz && heads == grp * rep && ka == k;
        if (ok) {
            const int64_t batch = bsz * grp, m = rep * seq;
            Tensor &y = c.alloc_output(0, RMLK_FLOAT, {bsz, heads, seq, n});
            const size_t ws_bytes = rmlk_hip_matmul_workspace_size(RMLK_FLOAT, batch, m, n, k);
            void *ws = ws_bytes ? c.scratch(ws_bytes) : nullptr;
            check_status(rmlk_hip_matmul(c.stream, RMLK_FLOAT, batch, m, n, k, a.data(), k, m * k, 0,
                                         kv.data(), dim, len * dim, transposed ? 1 : 0, y.data(), n,
                                         m * n, ws, ws_bytes),
                         "rmlk.AttnMatMul");
            return;
        }
    }
    run_body(c);
}

// scores -> scale, mask, softmax -> context of grouped-query attention: one kernel when there are
// enough query rows to fill its tiles, the split-key pair of kernels for a decode step (a handful
// of rows), the three nodes otherwise.
void op_fused_attention(OpContext &c) {
    const Tensor &q = c.input(0), &k = c.input(1), &mask = c.input(2), &v = c.input(3);
    bool ok = q.dtype == RMLK_FLOAT && k.dtype == RMLK_FLOAT && v.dtype == RMLK_FLOAT &&
              mask.dtype == RMLK_FLOAT && q.rank() == 4 && k.rank() == 4 && v.shape == k.shape &&
              q.numel() > 0 && k.numel() > 0;
    if (ok) {
        const int64_t axis = c.attr_int("axis", -1);
        ok = axis == -1 || axis == 3;
    }
    int64_t rep_k = 1, rep_v = 1;
    if (ok && c.attr_int("k_expanded", 0) != 0)
        ok = kv_repeat(c.attr_ints("k_expand_shape"), c.attr_ints("k_reshape_shape"), k, &rep_k);
    if (ok && c.attr_int("v_expanded", 0) != 0)
        ok = kv_repeat(c.attr_ints("v_expand_shape"), c.attr_ints("v_reshape_shape"), v, &rep_v);
    rmlk_dims ms{};
    if (ok) {
        const int64_t bsz = k.shape[0], grp = k.shape[1], len = k.shape[2], dim = k.shape[3];
        const int64_t heads = q.shape[1], seq = q.shape[2];
        ok = rep_k == rep_v && q.shape[0] == bsz && heads == grp * rep_k && q.shape[3] == dim &&
             mask_strides(mask, {bsz, heads, seq, len}, &ms);
        const size_t few_bytes =
            ok ? rmlk_hip_attention_few_rows_workspace_size(RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim) : 0;
        if (ok && few_bytes) {
            // a decode step: keys split over blocks, partial softmaxes merged by a second kernel
            const bool seq_major = c.attr_int("seq_major_output", 0) != 0;
            void *ws = c.scratch(few_bytes);
            Tensor &y = seq_major ? c.alloc_output(0, RMLK_FLOAT, {bsz, seq, heads, dim})
                                  : c.alloc_output(0, RMLK_FLOAT, {bsz, heads, seq, dim});
            const int32_t scale_is_mul = static_cast<int32_t>(c.attr_int("scale_is_mul", 0));
            // the last block of a KV head merges its chunks when the session's counters cover the heads
            const int32_t st =
                bsz * grp <= Session::kBlockCounters
                    ? rmlk_hip_attention_few_rows_one_launch(c.stream, RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim,
                                                             q.data(), k.data(), v.data(), mask.data(), &ms,
                                                             scale_is_mul, attr_float(c, "scale"), seq_major ? 1 : 0,
                                                             ws, few_bytes, c.session.block_counters, y.data())
                    : rmlk_hip_attention_few_rows(c.stream, RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim, q.data(),
                                                  k.data(), v.data(), mask.data(), &ms, scale_is_mul,
                                                  attr_float(c, "scale"), seq_major ? 1 : 0, ws, few_bytes,
                                                  y.data());
            if (took_fast_path(st, "rmlk.Attention")) return;
        }
        ok = ok && rep_k * seq >= 32;
        if (ok) {
            const bool seq_major = c.attr_int("seq_major_output", 0) != 0;
            Tensor &y = seq_major ? c.alloc_output(0, RMLK_FLOAT, {bsz, seq, heads, dim})
                                  : c.alloc_output(0, RMLK_FLOAT, {bsz, heads, seq, dim});
            // The map of (query tile, key chunk) pairs the mask leaves visible, kept for the other
            // attention nodes of this run that read the same mask (a pool buffer that lives until the
            // run ends; the session's workspace is overwritten by the products in between).
            const int mask_value = c.node.inputs.size() > 2 ? c.node.inputs[2] : -1;
            const size_t shared_bytes =
                mask_value >= 0 ? rmlk_hip_attention_map_size(RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim, &ms) : 0;
            // (the result's pieces for the output projection behind it, stored by the same launch)
            Tensor pieces = seq_major ? room_for_pieces(c, bsz * seq, heads * dim, "reader_is_product") : Tensor();
            if (shared_bytes) {
                Session::AttentionMap &am = c.session.attention_map;
                const int64_t sizes[6] = {bsz, grp, rep_k, seq, len, dim};
                bool same = am.map.defined() && am.mask_value == mask_value && am.strides.rank == ms.rank &&
                            am.map.nbytes() == shared_bytes;
                for (int i = 0; i < 6 && same; ++i) same = am.sizes[i] == sizes[i];
                for (int i = 0; i < ms.rank && same; ++i) same = am.strides.v[i] == ms.v[i];
                int32_t st = RMLK_OK;
                if (!same) {
                    am.map.reset();
                    std::vector<Tensor *> keep = c.out;
                    c.out = {&am.map};
                    c.alloc_output(0, RMLK_UINT8, {static_cast<int64_t>(shared_bytes)});
                    c.out = keep;
                    am.mask_value = mask_value;
                    am.strides = ms;
                    for (int i = 0; i < 6; ++i) am.sizes[i] = sizes[i];
                    st = rmlk_hip_attention_map(c.stream, RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim, mask.data(), &ms,
                                                am.map.data(), shared_bytes);
                    if (st) am.map.reset();
                }
                if (!st && pieces.defined()) {
                    if (took_fast_path(rmlk_hip_attention_mapped_pieces(
                                           c.stream, RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim, q.data(), k.data(),
                                           v.data(), mask.data(), &ms,
                                           static_cast<int32_t>(c.attr_int("scale_is_mul", 0)), attr_float(c, "scale"),
                                           am.map.data(), shared_bytes, y.data(), pieces.data()),
                                       "rmlk.Attention")) {
                        y.pieces = std::make_shared<const Tensor>(std::move(pieces));
                        return;
                    }
                } else if (!st && took_fast_path(rmlk_hip_attention_mapped(
                                                     c.stream, RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim, q.data(),
                                                     k.data(), v.data(), mask.data(), &ms,
                                                     static_cast<int32_t>(c.attr_int("scale_is_mul", 0)),
                                                     attr_float(c, "scale"), seq_major ? 1 : 0, am.map.data(),
                                                     shared_bytes, y.data()),
                                                 "rmlk.Attention")) {
                    return;
                }
            }
            // room for the map of (query tile, key chunk) pairs the mask leaves visible, when it pays
            const size_t map_bytes = rmlk_hip_attention_workspace_size(RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim, &ms);
            void *map = map_bytes ? c.scratch(map_bytes) : nullptr;
            if (pieces.defined()) {
                if (took_fast_path(rmlk_hip_attention_ws_pieces(c.stream, RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim,
                                                                q.data(), k.data(), v.data(), mask.data(), &ms,
                                                                static_cast<int32_t>(c.attr_int("scale_is_mul", 0)),
                                                                attr_float(c, "scale"), map, map_bytes, y.data(),
                                                                pieces.data()),
                                   "rmlk.Attention")) {
                    y.pieces = std::make_shared<const Tensor>(std::move(pieces));
                    return;
                }
            }
            if (took_fast_path(rmlk_hip_attention_ws(c.stream, RMLK_FLOAT, bsz, grp, rep_k, seq, len, dim,
                                                     q.data(), k.data(), v.data(), mask.data(), &ms,
                                                     static_cast<int32_t>(c.attr_int("scale_is_mul", 0)),
                                                     attr_float(c, "scale"), seq_major ? 1 : 0, map, map_bytes,
                                                     y.data()),
                               "rmlk.Attention"))
                return;
        }
    }
    run_body(c);
}

void op_fused_add_rmsnorm(OpContext &c) {
    const Tensor &a = c.input(0), &b = c.input(1), &gamma = c.input(2);
    const int rank = a.rank();
    bool ok = a.dtype == RMLK_FLOAT && b.dtype == RMLK_FLOAT && gamma.dtype == RMLK_FLOAT &&
              a.shape == b.shape && rank >= 1 && a.numel() > 0;
    if (ok) {
        const int64_t axis = c.attr_int("axis", -1);
        ok = (axis == -1 || axis == rank - 1) && gamma.rank() >= 1 && gamma.rank() <= rank &&
             gamma.shape.back() == a.shape.back() && gamma.numel() == a.shape.back();
    }
    if (ok) {
        const int64_t cols = a.shape.back(), rows = a.numel() / cols;
        Tensor &sum = c.alloc_output(0, RMLK_FLOAT, a.shape);
        Tensor &y = c.alloc_output(1, RMLK_FLOAT, a.shape);
        if (took_fast_path(rmlk_hip_add_rmsnorm(c.stream, RMLK_FLOAT, rows, cols, a.data(), b.data(),
                                                gamma.data(), attr_float(c, "epsilon"),
                                                static_cast<int32_t>(c.attr_int("reciprocal", 0)),
                                                sum.data(), y.data()),
                           "rmlk.AddRMSNorm"))
            return;
    }
    run_body(c);
}

// MatMul(a, W) -> Add(residual) -> RMSNorm, W constant and stored K-contiguous (wt [n, k]). Many
// rows: the GEMM leaves its split-K slabs in the workspace and the norm kernel adds them up while it
// forms the residual row. One row: the product with the residual added, the norm left to its reader.
void op_fused_matmul_add_rmsnorm(OpContext &c) {
    const Tensor &a = c.input(0), &wt = c.input(1), &res = c.input(2), &gamma = c.input(3);
    const int64_t n = wt.shape[0], k = wt.shape[1];
    bool ok = a.dtype == RMLK_FLOAT && res.dtype == RMLK_FLOAT && gamma.dtype == RMLK_FLOAT && a.rank() >= 2 &&
              a.numel() > 0 && a.shape.back() == k;
    if (ok) {
        std::vector<int64_t> out_shape(a.shape.begin(), a.shape.end() - 1);
        out_shape.push_back(n);
        const int64_t axis = c.attr_int("axis", -1);
        ok = res.shape == out_shape && (axis == -1 || axis == res.rank() - 1) && gamma.rank() >= 1 &&
             gamma.rank() <= res.rank() && gamma.numel() == n && gamma.shape.back() == n;
    }
    if (ok && a.numel() == k) {
        // one row: no combine launch, then Add + norm
        if (may_defer_norm(c, res, gamma)) {
            // the product with the residual added is the row; the norm is left to the product
            // that reads it
            Tensor &sum = c.alloc_output(0, RMLK_FLOAT, res.shape);
            if (took_fast_path(rmlk_hip_gemv_kmajor_add(c.stream, RMLK_FLOAT, n, k, a.data(), wt.dtype, wt.data(), k,
                                                        res.data(), sum.data()),
                               "rmlk.MatMulAddRMSNorm")) {
                defer_norm(c, 1, sum, gamma);
                return;
            }
        }
        float *prod = static_cast<float *>(c.scratch(static_cast<size_t>(n) * sizeof(float)));
        if (took_fast_path(rmlk_hip_gemv_kmajor(c.stream, RMLK_FLOAT, n, k, a.data(), wt.dtype, wt.data(), k, prod),
                           "rmlk.MatMulAddRMSNorm")) {
            Tensor &sum = c.alloc_output(0, RMLK_FLOAT, res.shape);
            Tensor &y = c.alloc_output(1, RMLK_FLOAT, res.shape);
            if (took_fast_path(rmlk_hip_add_rmsnorm(c.stream, RMLK_FLOAT, 1, n, prod, res.data(), gamma.data(),
                                                    attr_float(c, "epsilon"),
                                                    static_cast<int32_t>(c.attr_int("reciprocal", 0)),
                                                    sum.data(), y.data()),
                               "rmlk.MatMulAddRMSNorm"))
                return;
        }
    }
    if (ok && wants_pieces(c, a.numel() / k, k, wt.dtype)) {
        const int64_t m = a.numel() / k;
        const int32_t splits = rmlk_hip_bf16x3_splits(m, n, k);
        void *slabs = nullptr;
        void *pieces = splits > 0 ? split_pieces(c, a.data(), m, k, static_cast<size_t>(splits) * m * n * sizeof(float),
                                                 &slabs, "rmlk.MatMulAddRMSNorm", &a)
                                  : nullptr;
        if (pieces && took_fast_path(rmlk_hip_matmul_bf16x3(c.stream, m, n, k, pieces, wt.data(), k, splits, slabs, n,
                                                            m * n),
                                     "rmlk.MatMulAddRMSNorm")) {
            Tensor &sum = c.alloc_output(0, RMLK_FLOAT, res.shape);
            Tensor &y = c.alloc_output(1, RMLK_FLOAT, res.shape);
            if (Tensor normed = room_for_pieces(c, m, n); normed.defined()) {
                if (took_fast_path(rmlk_hip_rmsnorm_pieces(c.stream, m, n, slabs, splits, m * n, res.data(), gamma.data(),
                                                           attr_float(c, "epsilon"),
                                                           static_cast<int32_t>(c.attr_int("reciprocal", 0)),
                                                           sum.data(), y.data(), normed.data()),
                                   "rmlk.MatMulAddRMSNorm")) {
                    y.pieces = std::make_shared<const Tensor>(std::move(normed));
                    ++c.session.products_bf16_pieces;
                    return;
                }
            }
            if (took_fast_path(rmlk_hip_splitk_add_rmsnorm(c.stream, RMLK_FLOAT, m, n, slabs, splits, m * n, res.data(),
                                                           gamma.data(), attr_float(c, "epsilon"),
                                                           static_cast<int32_t>(c.attr_int("reciprocal", 0)),
                                                           sum.data(), y.data()),
                               "rmlk.MatMulAddRMSNorm")) {
                ++c.session.products_bf16_pieces;
                return;
            }
        }
    }
    if (ok) {
        const int64_t m = a.numel() / k;
        const size_t bytes = rmlk_hip_matmul_partials_workspace_size(RMLK_FLOAT, m, n, k);
        if (bytes) {
            void *ws = c.scratch(bytes);
            int32_t splits = 0;
            if (took_fast_path(rmlk_hip_matmul_partials(c.stream, RMLK_FLOAT, m, n, k, a.data(), k, wt.dtype,
                                                        wt.data(), k, 1, ws, bytes, &splits),
                               "rmlk.MatMulAddRMSNorm")) {
                Tensor &sum = c.alloc_output(0, RMLK_FLOAT, res.shape);
                Tensor &y = c.alloc_output(1, RMLK_FLOAT, res.shape);
                if (took_fast_path(rmlk_hip_splitk_add_rmsnorm(
                                       c.stream, RMLK_FLOAT, m, n, ws, splits, m * n, res.data(), gamma.data(),
                                       attr_float(c, "epsilon"),
                                       static_cast<int32_t>(c.attr_int("reciprocal", 0)), sum.data(), y.data()),
                                   "rmlk.MatMulAddRMSNorm"))
                    return;
            }
        }
    }
    run_body(c);   // the product (rmlk.MatMulConst), then rmlk.AddRMSNorm
}

// a [.., k] . wt^T for any number of rows: the general product with a K-contiguous second operand
// (`wt`: n rows of k), into the dense [m, n] at `out`.
// `w_dtype`: how the weights are stored (float, or the 16-bit type the session was built with).
void product_over_kmajor(OpContext &c, const void *a, int64_t m, int64_t k, int32_t w_dtype, const void *wt,
                         int64_t n, void *out, const char *what, const Tensor *a_tensor = nullptr) {
    if (wants_pieces(c, m, k, w_dtype) && rmlk_hip_bf16x3_splits(m, n, k) > 0) {
        void *pieces = split_pieces(c, a, m, k, 0, nullptr, what, a_tensor);
        if (pieces && took_fast_path(rmlk_hip_matmul_bf16x3(c.stream, m, n, k, pieces, wt, k, 1, out, n, 0), what)) {
            ++c.session.products_bf16_pieces;
            return;
        }
    }
    const size_t ws_bytes = rmlk_hip_matmul_workspace_size(RMLK_FLOAT, 1, m, n, k);
    void *ws = ws_bytes ? c.scratch(ws_bytes) : nullptr;
    if (w_dtype == RMLK_FLOAT) {
        check_status(rmlk_hip_matmul(c.stream, RMLK_FLOAT, 1, m, n, k, a, k, 0, 0, wt, k, 0, 1, out, n, 0, ws,
                                     ws_bytes),
                     what);
        return;
    }
    // (the grouped product with one member is the general product over stored weights)
    void *outs[1] = {out};
    check_status(rmlk_hip_matmul_grouped(c.stream, RMLK_FLOAT, m, k, a, k, w_dtype, wt, k, 1, 1, &n, outs, ws,
                                         ws_bytes),
                 what);
}

// What MatMul checks of a first operand [.., k]; returns its rows.
int64_t rows_of(const Tensor &a, int64_t k) {
    require_float(a.dtype);
    if (a.rank() == 0) fail_op("ZeroRank");
    if (a.shape.back() != k) fail_op("IncompatibleDimForMul");
    return k ? a.numel() / k : 0;
}

// MatMul(a, W) with constant 2-D W stored K-contiguous (wt [n, k]): a one-row input takes the kernel
// with a wavefront per output column (no split-K, no combine launch), anything else the general
// product with a transposed second operand.
void op_fused_matmul_const(OpContext &c) {
    const Tensor &wt = c.input(1);
    const int64_t n = wt.shape[0], k = wt.shape[1];
    const int64_t m = rows_of(c.input(0), k);
    std::vector<int64_t> shape(c.input(0).shape.begin(), c.input(0).shape.end() - 1);
    shape.push_back(n);
    Tensor &y = c.alloc_output(0, RMLK_FLOAT, shape);
    if (m == 0) return;
    if (m == 1) {
        const Tensor &a = c.input(0);
        // (a very wide product -- the lm-head -- has thousands of blocks that would each normalise
        // the row: there the separate norm launch is cheaper)
        if (a.pending_norm && n < kMaxDeferredNormWidth) {
            const PendingNorm &pn = *a.pending_norm;
            if (took_fast_path(rmlk_hip_gemv_kmajor_normed(c.stream, RMLK_FLOAT, n, k, a.data(), pn.gamma.data(),
                                                           pn.eps, pn.reciprocal, wt.dtype, wt.data(), k, y.data()),
                               "rmlk.MatMulConst"))
                return;
        }
        if (c.input(0).pending_norm) compute_pending_norm(c);
        if (took_fast_path(rmlk_hip_gemv_kmajor(c.stream, RMLK_FLOAT, n, k, c.input(0).data(), wt.dtype, wt.data(), k, y.data()),
                           "rmlk.MatMulConst"))
            return;
    }
    if (c.input(0).pending_norm) compute_pending_norm(c);
    product_over_kmajor(c, c.input(0).data(), m, k, wt.dtype, wt.data(), n, y.data(), "rmlk.MatMulConst", &c.input(0));
}

// swiglu(a . Wg, a . Wu) with [Wg | Wu] constant and stored K-contiguous as one matrix (wt [2 n, k]).
void op_fused_matmul_group_swiglu(OpContext &c) {
    const Tensor &wt = c.input(1);
    const std::vector<int64_t> widths = c.attr_ints("widths");
    const int64_t k = wt.shape[1];
    if (c.input(0).pending_norm) {
        const Tensor &row = c.input(0);
        const PendingNorm &pn = *row.pending_norm;
        if (row.dtype == RMLK_FLOAT && row.rank() >= 1 && row.shape.back() == k && row.numel() == k &&
            widths.size() == 2 && widths[0] == widths[1]) {
            const int64_t n = widths[0];
            const bool gate_first = c.attr_int("gate_first", 1) != 0;
            std::vector<int64_t> shape(row.shape.begin(), row.shape.end() - 1);
            shape.push_back(n);
            Tensor &y = c.alloc_output(0, RMLK_FLOAT, shape);
            if (took_fast_path(rmlk_hip_gemv_kmajor_swiglu_normed(
                                   c.stream, RMLK_FLOAT, n, k, row.data(), pn.gamma.data(), pn.eps, pn.reciprocal,
                                   wt.dtype, wt.data(), k, gate_first ? 0 : n, gate_first ? n : 0, y.data()),
                               "rmlk.MatMulGroupSwiGLU"))
                return;
        }
        compute_pending_norm(c);
    }
    const Tensor &a = c.input(0);
    const bool same_width = a.dtype == RMLK_FLOAT && a.rank() >= 1 && a.shape.back() == k && k > 0 &&
                            widths.size() == 2 && widths[0] == widths[1];
    if (same_width && a.numel() / k >= 128) {
        // many rows: one GEMM over [gate | up] with the activation applied to the accumulators
        const int64_t n = widths[0], m = a.numel() / k;
        const bool gate_first = c.attr_int("gate_first", 1) != 0;
        std::vector<int64_t> shape(a.shape.begin(), a.shape.end() - 1);
        shape.push_back(n);
        Tensor &y = c.alloc_output(0, RMLK_FLOAT, shape);
        if (wants_pieces(c, m, k, wt.dtype)) {
            void *pieces = split_pieces(c, a.data(), m, k, 0, nullptr, "rmlk.MatMulGroupSwiGLU", &a);
            // (the activation's pieces for the down projection behind it, stored by the same launch)
            Tensor act = pieces ? room_for_pieces(c, m, n, "reader_is_product") : Tensor();
            if (pieces && took_fast_path(rmlk_hip_matmul_bf16x3_swiglu(c.stream, m, n, k, pieces, wt.data(), k,
                                                                       gate_first ? 0 : n, gate_first ? n : 0,
                                                                       y.data(), n, act.defined() ? act.data() : nullptr),
                                         "rmlk.MatMulGroupSwiGLU")) {
                if (act.defined()) y.pieces = std::make_shared<const Tensor>(std::move(act));
                ++c.session.products_bf16_pieces;
                return;
            }
        }
        if (took_fast_path(rmlk_hip_matmul_swiglu(c.stream, RMLK_FLOAT, m, n, k, a.data(), k, wt.dtype, wt.data(), k, 1,
                                                  gate_first ? 0 : n, gate_first ? n : 0, y.data(), n),
                           "rmlk.MatMulGroupSwiGLU"))
            return;
    }
    if (same_width && a.numel() == k) {
        // one row: gate, up and the activation in one launch
        const int64_t n = widths[0];
        const bool gate_first = c.attr_int("gate_first", 1) != 0;
        std::vector<int64_t> shape(a.shape.begin(), a.shape.end() - 1);
        shape.push_back(n);
        Tensor &y = c.alloc_output(0, RMLK_FLOAT, shape);
        if (took_fast_path(rmlk_hip_gemv_kmajor_swiglu(c.stream, RMLK_FLOAT, n, k, a.data(), wt.dtype, wt.data(), k,
                                                       gate_first ? 0 : n, gate_first ? n : 0, y.data()),
                           "rmlk.MatMulGroupSwiGLU"))
            return;
    }
    run_body(c);   // rmlk.MatMulGroup, then rmlk.SwiGLU
}

// MatMul(a, W_i) for every member of a group, the W_i stored K-contiguous one below the other in one
// joint matrix (wt [N1 + N2 + .., k]).
void op_fused_matmul_group(OpContext &c) {
    const Tensor &wt = c.input(1);
    const std::vector<int64_t> widths = c.attr_ints("widths");
    const int64_t k = wt.shape[1], total = wt.shape[0];
    std::shared_ptr<const PendingNorm> pending = c.input(0).pending_norm;
    if (pending && !(c.input(0).numel() == k && total < kMaxDeferredNormWidth)) {
        compute_pending_norm(c);
        pending.reset();
    }
    const Tensor &a = c.input(0);
    const int64_t m = rows_of(a, k);
    std::vector<int64_t> lead(a.shape.begin(), a.shape.end() - 1);   // 1-D a: the row dim is dropped
    auto out_shape = [&](int64_t n) {
        std::vector<int64_t> sh = lead;
        sh.push_back(n);
        return sh;
    };
    const char *rows = static_cast<const char *>(wt.data());
    const int64_t row_bytes = k * static_cast<int64_t>(dtype_size(wt.dtype));
    if (m == 1) {
        // one launch over the joint matrix; the members' results are slices of its output row
        Tensor row;
        {
            std::vector<Tensor *> keep = c.out;
            c.out = {&row};
            c.alloc_output(0, RMLK_FLOAT, {total});
            c.out = keep;
        }
        auto hand_out = [&](const std::shared_ptr<PendingProduct> &pp) {
            int64_t off = 0;
            for (size_t i = 0; i < widths.size(); ++i) {
                Tensor v;
                v.dtype = RMLK_FLOAT;
                v.shape = out_shape(widths[i]);
                v.buf = row.buf;
                v.offset = row.offset + static_cast<size_t>(off) * sizeof(float);
                v.pending_product = pp;
                *c.out[i] = v;
                off += widths[i];
            }
        };
        if (c.attr_int("defer_product", 0) != 0) {
            // left to the row-stream node behind it (op_fused_head_rows)
            auto pp = std::make_shared<PendingProduct>();
            pp->x = a;
            pp->x.pending_norm.reset();
            pp->norm = pending;
            pp->wt = wt;
            pp->row = row;
            pp->k = k;
            pp->total = total;
            hand_out(pp);
            return;
        }
        bool done = false;
        if (pending) {
            done = took_fast_path(rmlk_hip_gemv_kmajor_normed(c.stream, RMLK_FLOAT, total, k, a.data(),
                                                              pending->gamma.data(), pending->eps,
                                                              pending->reciprocal, wt.dtype, wt.data(), k,
                                                              row.data()),
                                  "rmlk.MatMulGroup");
            if (!done) compute_pending_norm(c);   // what follows reads input 0 through the context
        }
        const Tensor &a1 = c.input(0);
        if (!done && !took_fast_path(rmlk_hip_gemv_kmajor(c.stream, RMLK_FLOAT, total, k, a1.data(), wt.dtype, wt.data(), k,
                                                          row.data()),
                                     "rmlk.MatMulGroup"))
            product_over_kmajor(c, a1.data(), 1, k, wt.dtype, wt.data(), total, row.data(), "rmlk.MatMulGroup");
        hand_out(nullptr);
        return;
    }
    if (widths.size() <= 4 && c.attr_int("defer_product", 0) != 0) {
        // Everything that reads the members is one row-stream node: the product runs now, but its
        // split-K partial sums stay where they are - that node adds them up while it reads its rows,
        // which saves the combine launch and a round trip of the product through memory.
        const int32_t x3_splits = wants_pieces(c, m, k, wt.dtype) ? rmlk_hip_bf16x3_splits(m, total, k) : 0;
        const size_t bytes = x3_splits > 0 ? static_cast<size_t>(x3_splits) * m * total * sizeof(float)
                                           : rmlk_hip_matmul_partials_workspace_size(RMLK_FLOAT, m, total, k);
        if (bytes) {
            auto pp = std::make_shared<PendingProduct>();
            {
                std::vector<Tensor *> keep = c.out;
                c.out = {&pp->slabs};
                c.alloc_output(0, RMLK_UINT8, {static_cast<int64_t>(bytes)});
                c.out = keep;
            }
            int32_t splits = 0;
            bool multiplied = false;
            if (x3_splits > 0) {
                void *pieces = split_pieces(c, a.data(), m, k, 0, nullptr, "rmlk.MatMulGroup", &a);
                multiplied = pieces && took_fast_path(rmlk_hip_matmul_bf16x3(c.stream, m, total, k, pieces, wt.data(), k,
                                                                             x3_splits, pp->slabs.data(), total,
                                                                             m * total),
                                                      "rmlk.MatMulGroup");
                if (multiplied) {
                    splits = x3_splits;
                    ++c.session.products_bf16_pieces;
                }
            }
            // (should the pieces be refused after all, the fp32 kernels take over where the slabs
            // allocated for them are large enough for theirs)
            if (multiplied ||
                (bytes >= rmlk_hip_matmul_partials_workspace_size(RMLK_FLOAT, m, total, k) &&
                 took_fast_path(rmlk_hip_matmul_partials(c.stream, RMLK_FLOAT, m, total, k, a.data(), k, wt.dtype,
                                                         wt.data(), k, 1, pp->slabs.data(), bytes, &splits),
                                "rmlk.MatMulGroup"))) {
                pp->x = a;
                pp->wt = wt;
                pp->k = k;
                pp->total = total;
                pp->m = m;
                pp->splits = splits;
                pp->slab = m * total;
                pp->widths = widths;
                for (size_t i = 0; i < widths.size(); ++i) {
                    Tensor &y = c.alloc_output(static_cast<int>(i), RMLK_FLOAT, out_shape(widths[i]));
                    y.pending_product = pp;
                    pp->outs.push_back(y);
                    pp->outs.back().pending_product.reset();   // (no cycle: the copies only name the memory)
                }
                return;
            }
        }
    }
    if (widths.size() <= 4) {
        // one launch whose tiles write to the members' outputs (or the members one by one, as the
        // kernel library sees fit)
        std::vector<void *> outs;
        for (size_t i = 0; i < widths.size(); ++i)
            outs.push_back(c.alloc_output(static_cast<int>(i), RMLK_FLOAT, out_shape(widths[i])).data());
        if (wants_pieces(c, m, k, wt.dtype) && rmlk_hip_bf16x3_splits(m, total, k) > 0) {
            // one split of the operand, one product over the joint matrix whose column blocks go to
            // the members' outputs
            void *pieces = split_pieces(c, a.data(), m, k, 0, nullptr, "rmlk.MatMulGroup", &a);
            if (pieces && took_fast_path(rmlk_hip_matmul_bf16x3_grouped(c.stream, m, k, pieces, wt.data(), k,
                                                                        static_cast<int32_t>(widths.size()),
                                                                        widths.data(), outs.data()),
                                         "rmlk.MatMulGroup")) {
                ++c.session.products_bf16_pieces;
                return;
            }
        }
        const size_t ws_bytes = rmlk_hip_matmul_grouped_workspace_size(
            RMLK_FLOAT, m, k, static_cast<int32_t>(widths.size()), widths.data());
        void *ws = ws_bytes ? c.scratch(ws_bytes) : nullptr;
        check_status(rmlk_hip_matmul_grouped(c.stream, RMLK_FLOAT, m, k, a.data(), k, wt.dtype, wt.data(), k, 1,
                                             static_cast<int32_t>(widths.size()), widths.data(),
                                             outs.data(), ws, ws_bytes),
                     "rmlk.MatMulGroup");
        return;
    }
    int64_t off = 0;
    for (size_t i = 0; i < widths.size(); ++i) {
        Tensor &y = c.alloc_output(static_cast<int>(i), RMLK_FLOAT, out_shape(widths[i]));
        if (y.numel() > 0)
            product_over_kmajor(c, a.data(), m, k, wt.dtype, rows + off * row_bytes, widths[i], y.data(), "rmlk.MatMulGroup");
        off += widths[i];
    }
}

// Rewrite the session's node list; returns how many fused nodes were formed.
int fuse_patterns(Session &s) {
    Matcher m(s);
    int formed = 0;
    for (size_t n = 0; n < m.g.nodes.size(); ++n) {
        if (m.removed[n]) continue;
        // the node object may be overwritten by replace(): match on a copy of its header
        const Node &node = m.g.nodes[n];
        if (node.op == "Mul") {
            if (m.match_rmsnorm(node) || m.match_swiglu(node)) ++formed;
        } else if (node.op == "Softmax") {
            if (m.match_softmax(node)) ++formed;
        } else if (node.op == "Add") {
            if (m.match_rotary(node)) ++formed;
        } else if (node.op == "MatMul") {
            if (m.match_attn_matmul(node)) ++formed;
        }
    }
    formed += m.form_attention();
    formed += m.form_head_rows();
    formed += m.form_add_rmsnorm();
    formed += m.form_matmul_groups();
    formed += m.form_splitk_epilogues();
    formed += m.form_const_matmuls();
    if (formed) m.mark_deferred_norms();   // an attribute on existing fused nodes, not a node of its own
    if (formed) m.mark_deferred_products();
    if (!formed) return 0;
    std::vector<Node> kept;
    kept.reserve(m.g.nodes.size());
    for (size_t n = 0; n < m.g.nodes.size(); ++n)
        if (!m.removed[n]) kept.push_back(std::move(m.g.nodes[n]));
    m.g.nodes = std::move(kept);
    for (Value &v : m.g.values) v.producer = -1;
    for (size_t n = 0; n < m.g.nodes.size(); ++n)
        for (int v : m.g.nodes[n].outputs) m.g.values[v].producer = static_cast<int>(n);
    return formed;
}

}  // namespace rt
}  // namespace rmlk
