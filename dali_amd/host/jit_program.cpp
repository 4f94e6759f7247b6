// The program a fused kernel is generated from: nodes of the expression in evaluation order, the buffers and scalars
// they read, and the classification of every node over the collapsed 2-D index domain [R, C] (full element, one value
// per row, scalar). Counterpart of the reference's node numbering in compute_node_compilation_info
// (dali/array/jit/jit.cpp:552-587).
#include "jit_internal.h"

namespace dali {
namespace jit {

int64_t numel_of(const std::vector<int>& shape) {
    int64_t n = 1;
    for (int s : shape) n *= s;
    return n;
}

std::string array_key(const Expr* b, Cls cls, bool gather) {
    std::ostringstream ss;
    ss << (const void*)b->memory.get() << "|" << b->offset << "|" << (int)b->dtype << "|" << (int)cls << "|" << gather << "|";
    for (int s : b->shape) ss << s << ",";
    ss << "|";
    for (int s : b->strides) ss << s << ",";
    return ss.str();
}

int add_node(Program& P, const Array& a) {
    std::shared_ptr<Expr> eptr = a.expression();
    const Expr* e = eptr.get();
    auto it = P.memo.find(e);
    if (it != P.memo.end()) return it->second;
    PNode n;
    n.kind = e->kind;
    n.dtype = e->dtype;
    n.name = e->name;
    n.shape = e->shape;
    n.axis = e->axis;
    n.depth = e->depth;
    n.src = eptr;
    for (const Array& arg : e->args) n.args.push_back(add_node(P, arg));
    std::ostringstream key;
    key << (int)n.kind << "|" << n.name << "|" << (int)n.dtype << "|" << n.axis << "|" << n.depth << "|";
    for (int s : n.shape) key << s << ",";
    key << "|";
    for (int a2 : n.args) key << a2 << ",";
    if (n.kind == Kind::BUFFER) key << "|" << array_key(e, Cls::FULL, false);
    if (n.kind == Kind::SCALAR) {
        // every literal keeps its own slot: values are launch arguments, not code
        n.scalar = (int)P.scalars.size();
        ScalarArg s;
        s.dtype = e->dtype;
        s.d = e->dvalue;
        s.f = (float)e->dvalue;
        s.i = e->ivalue;
        s.src = e;
        P.scalars.push_back(s);
        key << "|s" << n.scalar;
    }
    auto sit = P.structural.find(key.str());
    if (sit != P.structural.end()) {
        P.memo[e] = sit->second;
        return sit->second;
    }
    int id = (int)P.nodes.size();
    P.nodes.push_back(n);
    P.memo[e] = id;
    P.structural[key.str()] = id;
    return id;
}

// Collapse dims [0, upto) of a strided shape into one index; false when they do not nest.
bool collapse_dims(const std::vector<int>& shape, const std::vector<int>& st, int upto, int64_t* stride) {
    int64_t extent = 1, s = 0;
    for (int d = upto - 1; d >= 0; --d) {
        if (shape[d] == 1) continue;
        if (extent == 1) {
            s = st[d];
            extent = shape[d];
        } else {
            if ((int64_t)st[d] != s * extent) return false;
            extent *= shape[d];
        }
    }
    *stride = extent == 1 ? 0 : s;
    return true;
}

// Register a buffer as a kernel argument in class `cls`; returns -1 when its layout does not fit the class.
int add_array(Program& P, const std::shared_ptr<Expr>& b, Cls cls, bool gather, const Domain& dom, bool is_dest) {
    ArrayArg a;
    a.buf = b;
    a.cls = cls;
    a.gather_source = gather;
    a.is_dest = is_dest;
    auto st = strides_of(b.get());
    int nd = (int)b->shape.size();
    int64_t n = numel_of(b->shape);
    if (gather) {
        if (nd != 2) return -1;
        a.nd = 2;
        a.sizes = b->shape;
        a.strides = st;
        a.row_stride = st[0];
        a.col_stride = st[1];
        a.strided = !b->strides.empty();
    } else if (cls == Cls::FULL && dom.flat) {
        if (n != dom.C) return -1;
        auto c = contiguous_strides(b->shape);
        for (int d = 0; d < nd; ++d)
            if (b->shape[d] != 1 && st[d] != c[d]) return -1;
        a.nd = 1;
        a.sizes = {(int)dom.C};
        a.strided = false;
        a.row_stride = 0;
        a.col_stride = 1;
    } else if (cls == Cls::FULL) {
        // [R, C] or, broadcast along the rows, [1, C] (row stride 0)
        int64_t last = nd ? b->shape[nd - 1] : 1;
        bool col_vector = false;
        if (n == dom.R * dom.C && (last == dom.C || dom.C == 1)) {
        } else if (n == dom.C && last == dom.C) {
            col_vector = true;
        } else {
            return -1;
        }
        int64_t rs = 0;
        if (dom.C == 1 && last != 1) {
            // degenerate domain: every dim is a row dim
            if (!collapse_dims(b->shape, st, nd, &rs)) return -1;
            a.col_stride = 1;
        } else {
            if (!collapse_dims(b->shape, st, nd - 1, &rs)) return -1;
            a.col_stride = (nd && b->shape[nd - 1] != 1) ? st[nd - 1] : 1;
        }
        a.row_stride = col_vector ? 0 : rs;
        if (dom.R == 1) a.row_stride = 0;
        a.nd = 2;
        a.sizes = {(int)dom.R, (int)dom.C};
        a.strided = !(a.col_stride == 1 && (dom.R == 1 || a.row_stride == dom.C));
        a.strides = {(int)a.row_stride, (int)a.col_stride};
    } else if (cls == Cls::ROW) {
        if (n != dom.R) return -1;
        int64_t s = 0;
        if (!collapse_dims(b->shape, st, nd, &s)) return -1;
        if (dom.R == 1) s = 1;
        a.nd = 1;
        a.sizes = {(int)dom.R};
        a.row_stride = s;
        a.strided = s != 1;
        a.strides = {(int)s};
    } else {
        if (n != 1) return -1;
        a.nd = 1;
        a.sizes = {1};
        a.strided = false;
    }
    if (!is_dest) {
        std::string key = array_key(b.get(), cls, gather);
        for (size_t i = 0; i < P.arrays.size(); ++i)
            if (!P.arrays[i].is_dest && P.arrays[i].row_index < 0 &&
                array_key(P.arrays[i].buf.get(), P.arrays[i].cls, P.arrays[i].gather_source) == key)
                return (int)i;
    }
    P.arrays.push_back(a);
    return (int)P.arrays.size() - 1;
}

// Assign index classes top-down; false when the tree does not fit the row model.
bool classify(Program& P, int id, Cls want, const Domain& dom) {
    PNode& n = P.nodes[id];
    if (n.kind == Kind::SCALAR) {
        n.cls = Cls::SCAL;
        n.cls_set = true;
        return true;
    }
    if (n.cls_set) return n.cls == want;
    n.cls = want;
    n.cls_set = true;
    int nd = (int)n.shape.size();
    switch (n.kind) {
        case Kind::BUFFER: {
            int idx = add_array(P, n.src, want, false, dom, false);
            if (idx < 0) return false;
            P.nodes[id].array = idx;
            return true;
        }
        case Kind::ELEMENTWISE: {
            std::vector<int> args = n.args;
            for (int a : args) {
                Cls w = want;
                if (P.nodes[a].shape.empty() && nd > 0) w = Cls::SCAL;
                if (numel_of(P.nodes[a].shape) == 1 && numel_of(n.shape) != 1) w = Cls::SCAL;
                if (!classify(P, a, w, dom)) return false;
            }
            return true;
        }
        case Kind::BROADCAST: {
            int c = n.args[0];
            const std::vector<int>& s = P.nodes[c].shape;
            if ((int)s.size() != nd) return false;
            bool lead_equal = true, lead_ones = true;
            for (int i = 0; i + 1 < nd; ++i) {
                if (s[i] != n.shape[i]) lead_equal = false;
                if (s[i] != 1) lead_ones = false;
            }
            bool last_equal = nd == 0 || s[nd - 1] == n.shape[nd - 1];
            bool last_one = nd == 0 || s[nd - 1] == 1;
            Cls w;
            if (dom.flat) {
                if (numel_of(s) != 1) return false;
                w = Cls::SCAL;
            } else if (want == Cls::FULL) {
                if (lead_equal && last_equal) w = Cls::FULL;
                else if (lead_equal && last_one) w = Cls::ROW;
                else if (lead_ones && last_equal) w = Cls::FULL;  // [1, C]: row-broadcast column vector
                else if (lead_ones && last_one) w = Cls::SCAL;
                else return false;
                if (dom.C == 1 && !(lead_equal && last_equal)) {
                    // degenerate domain: only scalar broadcasts are expressible
                    if (numel_of(s) == 1) w = Cls::SCAL; else return false;
                }
            } else if (want == Cls::ROW) {
                if (numel_of(s) == numel_of(n.shape)) w = Cls::ROW;
                else if (numel_of(s) == 1) w = Cls::SCAL;
                else return false;
            } else {
                w = Cls::SCAL;
            }
            return classify(P, c, w, dom);
        }
        case Kind::EXPAND_DIMS: {
            int c = n.args[0];
            Cls w = want;
            if (!dom.flat && want == Cls::FULL && n.axis == nd - 1 && dom.C != 1) return false;
            return classify(P, c, w, dom);
        }
        case Kind::AXIS_REDUCE:
        case Kind::ARG_AXIS_REDUCE: {
            if (dom.flat) return false;
            if (want == Cls::SCAL && dom.R == 1) {
                // single-row domain: the row value is also the scalar
            } else if (want == Cls::FULL && dom.C == 1) {
                // single-column domain: one element per row, the row value is the element
            } else if (want != Cls::ROW) {
                return false;
            }
            int c = n.args[0];
            const std::vector<int>& s = P.nodes[c].shape;
            if (s.empty() || s.back() != dom.C || numel_of(s) != dom.R * dom.C) return false;
            return classify(P, c, Cls::FULL, dom);
        }
        case Kind::GATHER_FROM_ROWS: {
            if (want != Cls::ROW && !(want == Cls::FULL && dom.C == 1)) return false;
            int src = n.args[0], idx = n.args[1];
            if (P.nodes[src].kind != Kind::BUFFER) return false;
            if (P.nodes[src].shape.size() != 2 || P.nodes[src].shape[0] < dom.R) return false;
            if (numel_of(P.nodes[idx].shape) != dom.R) return false;
            int ai = add_array(P, P.nodes[src].src, Cls::FULL, true, dom, false);
            if (ai < 0) return false;
            P.nodes[id].array = ai;  // the gather node owns the source presentation
            return classify(P, idx, Cls::ROW, dom);
        }
        case Kind::GATHER: {
            // out[r, c] = source[indices[r], c]: the source is an ordinary FULL leaf whose row pointer goes
            // through the index (dali/array/op/gather.cpp:49-52)
            if (want != Cls::FULL || dom.flat) return false;
            int src = n.args[0], idx = n.args[1];
            if (P.nodes[src].kind != Kind::BUFFER || P.nodes[idx].kind != Kind::BUFFER) return false;
            const std::vector<int>& ss = P.nodes[src].shape;
            if (ss.size() != 2 || ss[1] != dom.C || numel_of(P.nodes[idx].shape) != dom.R) return false;
            if (P.nodes[idx].dtype != DTYPE_INT32) return false;
            if (!classify(P, idx, Cls::ROW, dom)) return false;
            ArrayArg a;
            a.buf = P.nodes[src].src;
            a.cls = Cls::FULL;
            a.nd = 2;
            a.sizes = ss;
            auto st = strides_of(a.buf.get());
            a.row_stride = st[0];
            a.col_stride = st[1];
            a.strided = !(st[1] == 1 && st[0] == dom.C);
            a.strides = {st[0], st[1]};
            a.row_index = P.nodes[idx].array;
            for (size_t i = 0; i < P.arrays.size(); ++i)
                if (!P.arrays[i].is_dest && P.arrays[i].row_index == a.row_index &&
                    array_key(P.arrays[i].buf.get(), Cls::FULL, false) == array_key(a.buf.get(), Cls::FULL, false)) {
                    P.nodes[id].array = (int)i;
                    return true;
                }
            P.arrays.push_back(a);
            P.nodes[id].array = (int)P.arrays.size() - 1;
            return true;
        }
        case Kind::ONE_HOT: {
            if (want != Cls::FULL || n.depth != dom.C) return false;
            if (!classify(P, n.args[0], Cls::SCAL, dom)) return false;
            if (!classify(P, n.args[1], Cls::SCAL, dom)) return false;
            if (numel_of(P.nodes[n.args[2]].shape) != dom.R) return false;
            return classify(P, n.args[2], Cls::ROW, dom);
        }
        default:
            return false;
    }
}

void compute_dep(Program& P, int id, std::vector<bool>& seen) {
    if (seen[id]) return;
    seen[id] = true;
    PNode& n = P.nodes[id];
    int dep = 0;
    for (int a : n.args) {
        compute_dep(P, a, seen);
        const PNode& c = P.nodes[a];
        dep = std::max(dep, is_reduce(c.kind) ? c.phase + 1 : c.dep);
    }
    n.dep = dep;
    if (is_reduce(n.kind)) n.phase = dep;
}

// nodes reachable from `roots` without crossing reduce nodes or kept nodes
void body_nodes(const Program& P, int id, std::set<int>& out, bool top) {
    const PNode& n = P.nodes[id];
    if (is_reduce(n.kind) || (!top && n.kept)) {
        out.insert(id);
        return;
    }
    if (out.count(id)) return;
    out.insert(id);
    for (int a : n.args) body_nodes(P, a, out, false);
}

bool contains_expensive(const Program& P, int id) {
    const PNode& n = P.nodes[id];
    if (is_reduce(n.kind)) return false;
    if (n.kind == Kind::ELEMENTWISE && expensive_functor(n.name)) return true;
    for (int a : n.args)
        if (contains_expensive(P, a)) return true;
    return false;
}

void count_uses(Program& P, const std::vector<int>& roots) {
    for (auto& n : P.nodes) n.uses = 0;
    std::vector<bool> seen(P.nodes.size(), false);
    std::function<void(int)> walk = [&](int id) {
        P.nodes[id].uses++;
        if (seen[id]) return;
        seen[id] = true;
        for (int a : P.nodes[id].args) walk(a);
    };
    for (int r : roots) walk(r);
}

int pow2ceil(int v) {
    int p = 1;
    while (p < v) p <<= 1;
    return p;
}

std::string signature(const Program& P, const std::vector<Output>& outs) {
    std::ostringstream ss;
    for (const PNode& n : P.nodes) {
        ss << (int)n.kind << ":" << n.name << ":" << (int)n.dtype << ":" << (int)n.cls << ":" << n.array << ":" << n.scalar << ":" << n.axis << ":" << n.kept << ":" << n.shape.size() << "(";
        for (int a : n.args) ss << a << ",";
        ss << ");";
    }
    ss << "#";
    for (const ArrayArg& a : P.arrays) ss << a.nd << (a.strided ? "s" : "c") << (int)a.cls << (a.gather_source ? "g" : "") << (a.row_index >= 0 ? "i" + std::to_string(a.row_index) : std::string()) << (int)a.buf->dtype << ";";
    ss << "#";
    for (const ScalarArg& s : P.scalars) ss << (int)s.dtype << ";";
    ss << "#";
    for (const Output& o : outs) ss << o.root << ">" << o.array << ":" << (int)o.op << ":" << (int)o.cls << ":" << o.total_red << ";";
    return ss.str();
}

void fill_plan_arrays(KernelSpec& K, const Program& P, const std::vector<int>& shape_ndims) {
    for (const ArrayArg& a : P.arrays) {
        K.array_ndim.push_back(a.nd);
        K.array_strided.push_back(a.strided ? 1 : 0);
        K.array_elsize.push_back(size_of_dtype(a.buf->dtype));
    }
    for (const ScalarArg& s : P.scalars) K.scalar_dtype.push_back((int)s.dtype);
    K.shape_ndim = shape_ndims;
    std::memset(&K.plan, 0, sizeof(K.plan));
    K.plan.n_arrays = (int)P.arrays.size();
    K.plan.n_scalars = (int)P.scalars.size();
    K.plan.n_shapes = (int)shape_ndims.size();
    K.plan.array_ndim = K.array_ndim.data();
    K.plan.array_strided = K.array_strided.data();
    K.plan.array_elsize = K.array_elsize.data();
    K.plan.scalar_dtype = K.scalar_dtype.data();
    K.plan.shape_ndim = K.shape_ndim.data();
}

}  // namespace jit

}  // namespace dali
