// The generic N-D map: operands with arbitrary strides and broadcasts that the 2-D kernels cannot address, indexed
// by decomposing the linear output index (the reference's index_to_dim path, dali/array/jit/array_view.h).
#include "jit_internal.h"

namespace dali {
namespace jit {

// Fallback for layouts the 2-D model cannot express (N-D strided views, broadcasts
// over inner axes): one thread per destination element, every operand addressed
// through per-axis strides in the destination's index space (stride 0 along
// broadcast axes). No reductions; reductions over such operands are planned after
// a copy to contiguous memory through this kernel.
struct NdLeaf {
    std::vector<int> strides;  // per destination axis
};

static bool nd_collect(Program& P, int id, const std::vector<int>& axis_map, int out_nd, std::vector<std::vector<int>>& leaf_strides) {
    PNode& n = P.nodes[id];
    switch (n.kind) {
        case Kind::SCALAR:
            n.cls = Cls::SCAL;
            return true;
        case Kind::BUFFER: {
            auto st = strides_of(n.src.get());
            std::vector<int> eff(out_nd, 0);
            for (size_t d = 0; d < n.shape.size(); ++d) {
                int o = axis_map[d];
                if (o < 0) {
                    if (n.shape[d] != 1) return false;
                    continue;
                }
                if (n.shape[d] != 1) eff[o] += st[d];
            }
            ArrayArg a;
            a.buf = n.src;
            a.cls = Cls::FULL;
            a.nd = std::max(1, out_nd);
            a.strided = true;
            a.strides = eff;
            if (a.strides.empty()) a.strides = {0};
            // identical presentation of the same memory shares one argument slot
            for (size_t i = 0; i < P.arrays.size(); ++i) {
                const ArrayArg& b = P.arrays[i];
                if (!b.is_dest && b.buf->memory.get() == a.buf->memory.get() && b.buf->offset == a.buf->offset &&
                    b.buf->dtype == a.buf->dtype && b.strides == a.strides) {
                    n.array = (int)i;
                    n.cls = Cls::FULL;
                    return true;
                }
            }
            P.arrays.push_back(a);
            leaf_strides.push_back(eff);
            n.array = (int)P.arrays.size() - 1;
            n.cls = Cls::FULL;
            return true;
        }
        case Kind::ELEMENTWISE: {
            std::vector<int> args = n.args;
            for (int a : args) {
                std::vector<int> m = axis_map;
                size_t and_ = P.nodes[a].shape.size();
                if (and_ == 0) m.clear();
                else if (and_ != n.shape.size()) return false;
                if (!nd_collect(P, a, m, out_nd, leaf_strides)) return false;
            }
            return true;
        }
        case Kind::BROADCAST: {
            int c = n.args[0];
            if (P.nodes[c].shape.size() != n.shape.size()) return false;
            return nd_collect(P, c, axis_map, out_nd, leaf_strides);
        }
        case Kind::EXPAND_DIMS: {
            std::vector<int> m = axis_map;
            m.erase(m.begin() + n.axis);
            return nd_collect(P, n.args[0], m, out_nd, leaf_strides);
        }
        default:
            return false;
    }
}

// VEC > 1: the destination and every operand have stride 1 or 0 (UNIT[a] false: a broadcast) along the last axis, whose
// extent is a multiple of VEC; a thread decomposes one index for VEC adjacent elements and moves them as one vector at
// element alignment. NARROW: fewer than 2^31 elements, the decomposition runs in 32-bit arithmetic.
static std::string gen_generic_kernel(const Program& P, const std::vector<Output>& outs, const IvLayout& L, int nd, int VEC, const std::vector<bool>& UNIT, bool NARROW,
                               const std::string& kname) {
    std::ostringstream ss;
    RowParams rp;
    rp.cached = false;
    rp.VEC = VEC;
    const std::string it = NARROW ? "unsigned int" : "long";
    ss << device_prelude();
    ss << kargs_struct(P, L);
    ss << "extern \"C\" __global__ __launch_bounds__(256) void " << kname << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n";
    ss << "  constexpr int ND = " << nd << ", VEC = " << VEC << ";\n";
    ss << "  long total = 1;\n  _Pragma(\"unroll\") for (int d = 0; d < ND; ++d) total *= A.iv[" << L.shape_pos[0] << " + d];\n  total /= VEC;\n";
    ss << "  const long row = 0; (void)row;\n";
    ss << "  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {\n";
    ss << "    int idx[ND];\n    " << it << " rem = (" << it << ")i;\n";
    ss << "    _Pragma(\"unroll\") for (int d = ND - 1; d >= 0; --d) { const " << it << " ext = (" << it << ")A.iv[" << L.shape_pos[0]
       << " + d] / (d == ND - 1 ? VEC : 1); idx[d] = (int)(rem % ext) * (d == ND - 1 ? VEC : 1); rem /= ext; }\n";
    for (size_t a = 0; a < P.arrays.size(); ++a) {
        ss << "    long off" << a << " = 0;\n    _Pragma(\"unroll\") for (int d = 0; d < ND; ++d) off" << a << " += (long)idx[d] * A.iv[" << L.stride_pos[a] << " + d];\n";
        const ArrayArg& arr = P.arrays[a];
        std::string t = ctype(arr.buf->dtype);
        if (arr.is_dest) continue;
        if (VEC > 1 && UNIT[a])
            ss << "    const dali_vec<" << t << ", VEC> xv" << a << " = dali_loadu<" << t << ", VEC>((const " << t << "*)A.p[" << a << "] + off" << a << ");\n    const " << t
               << "* x" << a << " = xv" << a << ".v;\n";
        else if (VEC > 1)
            ss << "    " << t << " x" << a << "[VEC];\n    { const " << t << " one = ((const " << t << "*)A.p[" << a << "])[off" << a
               << "]; _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) x" << a << "[j] = one; }\n";
        else
            ss << "    const " << t << " x" << a << "[1] = { ((const " << t << "*)A.p[" << a << "])[off" << a << "] };\n";
    }
    std::vector<int> first_body(P.nodes.size(), -1);
    BodyEmitter be(P, rp, true, 0, &first_body);
    std::ostringstream pre, body, post;
    for (const Output& o : outs) {
        std::string t = ctype(P.arrays[o.array].buf->dtype);
        const std::string ptr = "((" + t + "*)A.p[" + std::to_string(o.array) + "] + off" + std::to_string(o.array) + ")";
        const std::string ov = "o" + std::to_string(o.array);
        pre << "    dali_vec<" << t << ", VEC> " << ov << ";\n";
        if (o.op != OPERATOR_T_EQL) pre << "    " << ov << " = dali_loadu<" << t << ", VEC>(" << ptr << ");\n";
        std::string v = be.value(o.root);
        body << "      " << ov << ".v[j] = " << op_combine(o.op, ov + ".v[j]", "(" + t + ")(" + v + ")") << ";\n";
        post << "    dali_storeu<" << t << ", VEC>(" << ptr << ", " << ov << ");\n";
    }
    ss << pre.str() << "    _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n      const int col = idx[ND - 1] + j; (void)col;\n";
    ss << be.stmts.str() << body.str() << "    }\n" << post.str() << "  }\n}\n";
    return ss.str();
}

bool try_generic(const std::vector<DestSpec>& specs) {
    const std::vector<int>& shape = specs[0].dest.shape();
    int nd = std::max<int>(1, (int)shape.size());
    if (nd > 8) return false;
    for (const DestSpec& s : specs)
        if (s.dest.shape() != shape) return false;
    Program P;
    std::vector<Output> outs;
    std::vector<std::vector<int>> leaf_strides;
    for (const DestSpec& s : specs) {
        ArrayArg a;
        a.buf = s.dest.expression();
        a.cls = Cls::FULL;
        a.is_dest = true;
        a.nd = nd;
        a.strided = true;
        a.strides = strides_of(a.buf.get());
        if (a.strides.empty()) a.strides = {0};
        P.arrays.push_back(a);
        Output o;
        o.array = (int)P.arrays.size() - 1;
        o.op = s.op;
        o.cls = Cls::FULL;
        o.root = -1;
        outs.push_back(o);
    }
    std::vector<int> roots;
    for (size_t i = 0; i < specs.size(); ++i) {
        int r = add_node(P, specs[i].root);
        outs[i].root = r;
        roots.push_back(r);
        std::vector<int> ident(shape.size());
        for (size_t d = 0; d < shape.size(); ++d) ident[d] = (int)d;
        const std::vector<int>& rs = P.nodes[r].shape;
        if (rs.size() != shape.size() && !rs.empty()) return false;
        if (rs.empty()) ident.clear();
        if (!nd_collect(P, r, ident, nd, leaf_strides)) return false;
    }
    count_uses(P, roots);
    // every array is presented with the destination's extents and its own strides
    std::vector<int> ext = shape;
    if (ext.empty()) ext = {1};
    for (ArrayArg& a : P.arrays) a.sizes = ext;
    // four adjacent elements of the last axis per thread when every array runs along it with stride 1 (or 0)
    int VEC = ext.back() % 4 == 0 ? 4 : 1;
    std::vector<bool> UNIT(P.arrays.size(), true);
    for (size_t a = 0; a < P.arrays.size(); ++a) {
        const int last = P.arrays[a].strides.empty() ? 0 : P.arrays[a].strides.back();
        UNIT[a] = last == 1;
        if (last != 1 && (last != 0 || P.arrays[a].is_dest)) VEC = 1;
    }
    const bool NARROW = numel_of(ext) < ((int64_t)1 << 31);
    std::ostringstream params;
    params << nd << "," << VEC << "," << NARROW << ",";
    for (size_t a = 0; a < UNIT.size(); ++a) params << (VEC > 1 && UNIT[a] ? 'u' : 'b');
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash("generic", signature(P, outs), params.str());
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    std::vector<int> shape_ndims = {nd};
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = "generic";
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = 256;
        K->plan.grid_kind = DALI_HIP_GRID_ELEMS;
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = nd;
        K->plan.work_per_block = 256 * VEC;
        K->plan.max_blocks = 65536;
    }
    std::vector<std::vector<int>> shapes = {ext};
    load_and_launch(*K, [&]() { return gen_generic_kernel(P, outs, L, nd, VEC, UNIT, NARROW, K->name); }, P, shapes);
    return true;
}

}  // namespace jit

}  // namespace dali
