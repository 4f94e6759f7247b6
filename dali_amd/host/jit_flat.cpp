// The flat kernel: a contiguous elementwise map over operands of one element count, 128-bit accesses, one tile of
// BT * UNROLL vectors per workgroup (the loop the reference's elementwise kernel leaves to the host compiler,
// dali/array/jit/elementwise_kernel_utils.cpp).
#include "jit_internal.h"

namespace dali {
namespace jit {

// All operands contiguous with the same element count (or single elements): one
// 1-D map, each block covering one tile of BT*UNROLL vectors.
bool flat_eligible(const Array& a, int64_t n, std::set<const Expr*>& seen) {
    auto e = a.expression();
    if (seen.count(e.get())) return true;
    seen.insert(e.get());
    switch (e->kind) {
        case Kind::SCALAR: return true;
        case Kind::BUFFER: return (numel_of(e->shape) == n && a.contiguous_memory()) || numel_of(e->shape) == 1;
        case Kind::ELEMENTWISE:
            for (const Array& x : e->args) {
                int64_t xn = numel_of(x.shape());
                if (xn != n && xn != 1) return false;
                if (!flat_eligible(x, n, seen)) return false;
            }
            return true;
        case Kind::EXPAND_DIMS:
            return flat_eligible(e->args[0], n, seen);
        case Kind::BROADCAST:
            return numel_of(e->args[0].shape()) == 1 && flat_eligible(e->args[0], n, seen);
        default: return false;
    }
}

// UNALIGNED: some operand starts off a 16-byte boundary (element-aligned vector accesses). REST: the element count is
// no multiple of VEC; the first block's leading threads take one of the last N % VEC elements each.
static std::string gen_flat_kernel(const Program& P, const std::vector<Output>& outs, const IvLayout& L, int VEC, int BT, int UNROLL, bool UNALIGNED, bool REST,
                            const std::string& kname, bool NT_STORES, bool NT_LOADS) {
    std::ostringstream ss;
    RowParams rp;
    rp.cached = false;
    rp.VEC = VEC;
    ss << device_prelude();
    ss << kargs_struct(P, L);
    ss << "extern \"C\" __global__ __launch_bounds__(" << BT << ") void " << kname << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n";
    ss << "  constexpr int VEC = " << VEC << ", BT = " << BT << ", UNROLL = " << UNROLL << ";\n";
    ss << "  const long N = A.iv[" << L.shape_pos[0] << "];\n  const long C = N; const long row = 0; (void)C; (void)row;\n";
    ss << "  const long NCH = N / VEC;\n";
    emit_row_prologue(ss, P, L);
    std::vector<int> full_leaves;
    for (size_t i = 0; i < P.arrays.size(); ++i)
        if (!P.arrays[i].is_dest && P.arrays[i].cls == Cls::FULL) full_leaves.push_back((int)i);
    ss << "  const long base = (long)blockIdx.x * (BT * UNROLL) + threadIdx.x;\n";
    for (int i : full_leaves) ss << "  " << ctype(P.arrays[i].buf->dtype) << " x" << i << "s[UNROLL][VEC];\n";
    ss << "  _Pragma(\"unroll\") for (int u = 0; u < UNROLL; ++u) {\n    const long ch = base + (long)u * BT;\n    if (ch < NCH) {\n";
    for (int i : full_leaves) emit_leaf_load(ss, P.arrays[i], i, VEC, "x" + std::to_string(i) + "s[u]", "      ", NT_LOADS, UNALIGNED);
    ss << "    }\n  }\n";
    ss << "  _Pragma(\"unroll\") for (int u = 0; u < UNROLL; ++u) {\n    const long ch = base + (long)u * BT;\n    if (ch < NCH) {\n";
    for (int i : full_leaves) ss << "      const " << ctype(P.arrays[i].buf->dtype) << "* x" << i << " = x" << i << "s[u];\n";
    std::vector<int> first_body(P.nodes.size(), -1);
    BodyEmitter be(P, rp, true, 0, &first_body);
    std::ostringstream pre, body, post;
    for (const Output& o : outs) {
        const ArrayArg& d = P.arrays[o.array];
        std::string t = ctype(d.buf->dtype);
        std::string ov = "o" + std::to_string(o.array);
        pre << "      dali_vec<" << t << ", VEC> " << ov << ";\n";
        if (o.op != OPERATOR_T_EQL) pre << "      " << ov << " = " << (UNALIGNED ? "dali_loadu<" : "dali_load<") << t << ", VEC>(q" << o.array << " + ch * VEC);\n";
        post << "      " << (UNALIGNED ? (NT_STORES ? "dali_storeu_nt<" : "dali_storeu<") : (NT_STORES ? "dali_store_nt<" : "dali_store<")) << t << ", VEC>(q" << o.array << " + ch * VEC, " << ov << ");\n";
        std::string v = be.value(o.root);
        body << "        " << ov << ".v[j] = " << op_combine(o.op, ov + ".v[j]", "(" + t + ")(" + v + ")") << ";\n";
    }
    ss << pre.str() << "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n        const int col = (int)(ch * VEC + j); (void)col;\n";
    ss << be.stmts.str() << body.str() << "      }\n" << post.str() << "    }\n  }\n";
    if (REST) {
        ss << "  if (blockIdx.x == 0 && threadIdx.x < (unsigned)(N - NCH * VEC)) {\n    const long rest = NCH * VEC + threadIdx.x;\n";
        for (int i : full_leaves) ss << "    " << ctype(P.arrays[i].buf->dtype) << " x" << i << "[VEC];\n    x" << i << "[0] = q" << i << "[rest];\n";
        ss << "    constexpr int j = 0; (void)j;\n    const int col = (int)rest; (void)col;\n" << be.stmts.str();
        for (const Output& o : outs) {
            std::string t = ctype(P.arrays[o.array].buf->dtype);
            const std::string dp = "q" + std::to_string(o.array) + "[rest]";
            ss << "    " << dp << " = " << op_combine(o.op, dp, "(" + t + ")(" + be.value(o.root) + ")") << ";\n";
        }
        ss << "  }\n";
    }
    ss << "}\n";
    return ss.str();
}

bool try_flat(const std::vector<DestSpec>& specs) {
    int64_t n = numel_of(specs[0].dest.shape());
    for (const DestSpec& s : specs) {
        if (numel_of(s.dest.shape()) != n || !s.dest.contiguous_memory()) return false;
        std::set<const Expr*> seen;
        if (!flat_eligible(s.root, n, seen)) return false;
    }
    if (n == 0) return true;
    Domain dom;
    dom.R = 1;
    dom.C = n;
    dom.flat = true;
    Program P;
    std::vector<Output> outs;
    for (const DestSpec& s : specs) {
        int ai = add_array(P, s.dest.expression(), Cls::FULL, false, dom, true);
        if (ai < 0) return false;
        Output o;
        o.array = ai;
        o.op = s.op;
        o.cls = Cls::FULL;
        o.root = -1;
        outs.push_back(o);
    }
    std::vector<int> roots;
    for (size_t i = 0; i < specs.size(); ++i) {
        outs[i].root = add_node(P, specs[i].root);
        roots.push_back(outs[i].root);
        if (!classify(P, outs[i].root, Cls::FULL, dom)) return false;
    }
    count_uses(P, roots);
    int max_el = 4;
    for (const ArrayArg& a : P.arrays) max_el = std::max(max_el, size_of_dtype(a.buf->dtype));
    bool aligned = true;
    for (const ArrayArg& a : P.arrays)
        if (a.cls == Cls::FULL && a.buf->offset % 4 != 0) aligned = false;
    int VEC = n >= 16 ? 4 : 1, BT = 256, UNROLL = max_el == 8 ? 2 : 4;
    static const int unroll_env = env_int("DALI_HIP_FLAT_UNROLL", 0);
    if (unroll_env > 0) UNROLL = unroll_env;
    const bool UNALIGNED = VEC > 1 && !aligned, REST = VEC > 1 && n % VEC != 0;
    std::ostringstream params;
    // Streaming policy of a map, measured on 64M floats (copy / a + b / a chain of five operands): inputs bypass cache
    // allocation (plain loads: 0.73 instead of 0.87 of the HBM peak), outputs leave with plain stores (non-temporal stores:
    // 0.78). Kernels that reduce over cached rows are the other way round for their stores, and so is a map whose outputs
    // fit the second-level caches (32 MiB between them): with plain stores the whole output is still dirty in cache when
    // the last wave ends and the write-back is added to the kernel's time (4M floats over sixteen rotating buffer
    // pairs: copy 7.0 us, with non-temporal stores 6.0; a + b 9.2 -> 9.0; the same from cache-resident pairs: no loss).
    static const int nt_env = env_int("DALI_HIP_FLAT_NT_STORES", -1);
    static const int ntl_env = env_int("DALI_HIP_FLAT_NT_LOADS", 1);
    long out_bytes = 0;
    for (const Output& o : outs) out_bytes += n * (long)size_of_dtype(P.arrays[o.array].buf->dtype);
    const bool NT_STORES = nt_env < 0 ? out_bytes <= (32L << 20) : nt_env != 0, NT_LOADS = ntl_env != 0;
    params << VEC << "," << BT << "," << UNROLL << "," << UNALIGNED << REST << "," << NT_STORES << NT_LOADS;
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash("flat", signature(P, outs), params.str());
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    std::vector<int> shape_ndims = {1};
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = "flat";
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = BT;
        K->plan.grid_kind = DALI_HIP_GRID_ELEMS;
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = 1;
        K->plan.work_per_block = BT * UNROLL * VEC;
    }
    std::vector<std::vector<int>> shapes = {{(int)n}};
    load_and_launch(*K, [&]() { return gen_flat_kernel(P, outs, L, VEC, BT, UNROLL, UNALIGNED, REST, K->name, NT_STORES, NT_LOADS); }, P, shapes);
    return true;
}

}  // namespace jit

}  // namespace dali
