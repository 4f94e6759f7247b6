// The full reduction (dali/array/jit/all_reduce_kernel_utils.cpp): two stages through the library workspace in one
// launch (the last workgroup to finish folds the partial results), optional scalar epilogue.
#include "jit_internal.h"

namespace dali {
namespace jit {

// root = [epilogue over] ALL_REDUCE / ARG_ALL_REDUCE (contiguous elementwise arg).
// Stage 1: every block reduces a strided share of the vectors and writes one
// partial into the workspace; the block that takes the last ticket combines the
// partials in block order (so the result does not depend on scheduling), applies
// the scalar epilogue and resets the ticket counter.
static std::string gen_all_kernel(const Program& P, int red_id, int root_id, int dest_array, OPERATOR_T op, const IvLayout& L, int VEC, int BT,
                           int UNROLL, int TAIL, bool NT, bool UNALIGNED, bool REST, const std::string& kname) {
    const PNode& red = P.nodes[red_id];
    bool is_arg = red.kind == Kind::ARG_ALL_REDUCE;
    std::string t = ctype(P.nodes[red.args[0]].dtype);
    std::string dt = ctype(P.arrays[dest_array].buf->dtype);
    RowParams rp;
    rp.cached = false;
    rp.VEC = VEC;
    int NW = BT / 64;
    std::ostringstream ss;
    ss << device_prelude();
    ss << kargs_struct(P, L);
    ss << "struct dali_partial { " << t << " v; int i; };\n";
    ss << "extern \"C\" __global__ __launch_bounds__(" << BT << ") void " << kname << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n";
    ss << "  constexpr int VEC = " << VEC << ", BT = " << BT << ";\n";
    ss << "  const long N = A.iv[" << L.shape_pos[0] << "];\n  const long C = N; const long row = 0; (void)C; (void)row;\n";
    ss << "  const long NCH = N / VEC;\n";
    emit_row_prologue(ss, P, L);
    std::vector<int> full_leaves;
    for (size_t i = 0; i < P.arrays.size(); ++i)
        if (!P.arrays[i].is_dest && P.arrays[i].cls == Cls::FULL) full_leaves.push_back((int)i);
    ss << "  " << t << " acc = " << red.name << "::init<" << t << ">();\n  int acci = 0; (void)acci;\n";
    // UNROLL independent vector loads in flight per thread before any of them is consumed
    ss << "  constexpr int UNROLL = " << UNROLL << ";\n";
    ss << "  for (long base = (long)blockIdx.x * (BT * UNROLL) + threadIdx.x; base < NCH; base += (long)gridDim.x * (BT * UNROLL)) {\n";
    for (int i : full_leaves) ss << "    " << ctype(P.arrays[i].buf->dtype) << " x" << i << "s[UNROLL][VEC];\n";
    ss << "    _Pragma(\"unroll\") for (int u = 0; u < UNROLL; ++u) {\n      const long ch = base + (long)u * BT;\n      if (ch < NCH) {\n";
    for (int i : full_leaves) emit_leaf_load(ss, P.arrays[i], i, VEC, "x" + std::to_string(i) + "s[u]", "        ", NT, UNALIGNED);
    ss << "      }\n    }\n";
    ss << "    _Pragma(\"unroll\") for (int u = 0; u < UNROLL; ++u) {\n      const long ch = base + (long)u * BT;\n      if (ch < NCH) {\n";
    for (int i : full_leaves) ss << "        const " << ctype(P.arrays[i].buf->dtype) << "* x" << i << " = x" << i << "s[u];\n";
    ss << "        _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n          const int col = (int)(ch * VEC + j); (void)col;\n";
    std::vector<int> first_body(P.nodes.size(), -1);
    {
        BodyEmitter be(P, rp, true, 0, &first_body);
        std::string v = be.value(red.args[0]);
        std::string update;
        if (!is_arg)
            update = "acc = " + red.name + "::step<" + t + ">(acc, " + v + ");\n";
        else
            update = "{ const " + t + " cand = " + v + "; if (" + red.name + "::better<" + t + ">(cand, acc)) { acc = cand; acci = col; } }\n";
        ss << be.stmts.str() << "          " << update;
        ss << "        }\n      }\n    }\n  }\n";
        if (REST) {
            // the last N % VEC elements: one each to the leading threads of the first block, after their vectors (so a
            // thread still meets its elements in increasing order)
            ss << "  if (blockIdx.x == 0 && threadIdx.x < (unsigned)(N - NCH * VEC)) {\n    const long rest = NCH * VEC + threadIdx.x;\n";
            for (int i : full_leaves) ss << "    " << ctype(P.arrays[i].buf->dtype) << " x" << i << "[VEC];\n    x" << i << "[0] = q" << i << "[rest];\n";
            ss << "    constexpr int j = 0; (void)j;\n    const int col = (int)rest; (void)col;\n" << be.stmts.str() << "    " << update << "  }\n";
        }
    }
    ss << "  __shared__ " << t << " smv[" << NW << "]; __shared__ int smi[" << NW << "]; __shared__ int is_last;\n";
    if (!is_arg)
        ss << "  acc = dali_block_reduce<" << red.name << ", " << t << ", " << NW << ">(acc, smv);\n";
    else
        ss << "  dali_block_arg_reduce<" << red.name << ", " << t << ", " << NW << ">(acc, acci, smv, smi);\n";
    ss << "  unsigned int* counters = (unsigned int*)A.ws;\n";
    ss << "  dali_partial* partials = (dali_partial*)((char*)A.ws + " << 16384 * 4 << ");\n";
    // Cross-block hand-off without cache-wide fences: partials are written with agent-scope
    // atomic stores (written through to the device coherence point, never left dirty in one
    // XCD's L2), s_waitcnt 0 holds the ticket back until those stores are acknowledged, and the
    // last block reads them with agent-scope atomic loads (which do not hit stale lines).
    ss << "  if (threadIdx.x == 0) {\n    dali_publish(&partials[blockIdx.x].v, acc); dali_publish(&partials[blockIdx.x].i, acci);\n"
          "    is_last = dali_take_ticket(&counters[0]) == gridDim.x - 1;\n  }\n  __syncthreads();\n";
    ss << "  if (!is_last) return;\n";
    ss << "  acc = " << red.name << "::init<" << t << ">(); acci = 0;\n";
    ss << "  // fixed combination order: thread k folds partials k, k+BT, ... (all loads issued first), then the block folds in wave order\n";
    ss << "  {\n    constexpr int TAIL = " << TAIL << ";\n    " << t << " pv[TAIL]; int pi[TAIL];\n";
    ss << "    _Pragma(\"unroll\") for (int k = 0; k < TAIL; ++k) {\n      const unsigned int b = threadIdx.x + k * BT;\n"
          "      if (b < gridDim.x) { pv[k] = dali_observe(&partials[b].v); pi[k] = dali_observe(&partials[b].i); }\n    }\n";
    ss << "    _Pragma(\"unroll\") for (int k = 0; k < TAIL; ++k) {\n      const unsigned int b = threadIdx.x + k * BT;\n      if (b < gridDim.x) {\n";
    if (!is_arg)
        ss << "        acc = " << red.name << "::step<" << t << ">(acc, pv[k]);\n";
    else
        ss << "        if (" << red.name << "::better<" << t << ">(pv[k], acc) || (pv[k] == acc && pi[k] < acci)) { acc = pv[k]; acci = pi[k]; }\n";
    ss << "      }\n    }\n  }\n  __syncthreads();\n";

    if (!is_arg)
        ss << "  acc = dali_block_reduce<" << red.name << ", " << t << ", " << NW << ">(acc, smv);\n";
    else
        ss << "  dali_block_arg_reduce<" << red.name << ", " << t << ", " << NW << ">(acc, acci, smv, smi);\n";
    ss << "  if (threadIdx.x == 0) {\n    dali_publish(&counters[0], 0u);\n";
    // the reference stores a flat arg index in the input dtype
    if (!is_arg)
        ss << "    const " << ctype(red.dtype) << " red" << red_id << " = acc;\n";
    else
        ss << "    const " << ctype(red.dtype) << " red" << red_id << " = (" << ctype(red.dtype) << ")acci;\n";
    {
        BodyEmitter be(P, rp, false, 1, &first_body);
        std::string v = be.value(root_id);
        ss << be.stmts.str();
        ss << "    q" << dest_array << "[0] = " << op_combine(op, "q" + std::to_string(dest_array) + "[0]", "(" + dt + ")(" + v + ")") << ";\n";
    }
    ss << "  }\n}\n";
    return ss.str();
}

// does the subtree contain any reduce node?
bool has_kind(const Array& a, const std::function<bool(Kind)>& pred, std::set<const Expr*>& seen) {
    auto e = a.expression();
    if (seen.count(e.get())) return false;
    seen.insert(e.get());
    if (pred(e->kind)) return true;
    for (const Array& x : e->args)
        if (has_kind(x, pred, seen)) return true;
    return false;
}

bool has_kind(const Array& a, const std::function<bool(Kind)>& pred) {
    std::set<const Expr*> seen;
    return has_kind(a, pred, seen);
}

// find the unique ALL_REDUCE under a scalar epilogue; nullptr when the root does not have that shape
void find_all_reduces(const Array& a, std::vector<Array>& out, std::set<const Expr*>& seen) {
    auto e = a.expression();
    if (seen.count(e.get())) return;
    seen.insert(e.get());
    if (is_all_reduce(e->kind)) {
        out.push_back(a);
        return;
    }
    for (const Array& x : e->args) find_all_reduces(x, out, seen);
}

bool try_all(const DestSpec& spec) {
    std::vector<Array> reds;
    std::set<const Expr*> seen;
    find_all_reduces(spec.root, reds, seen);
    if (reds.size() != 1) return false;
    if (numel_of(spec.dest.shape()) != 1) return false;
    Array red = reds[0];
    Array arg = red.expression()->args[0];
    int64_t n = numel_of(arg.shape());
    if (n == 0) return false;
    std::set<const Expr*> s2;
    if (!flat_eligible(arg, n, s2)) return false;
    Domain dom;
    dom.R = 1;
    dom.C = n;
    dom.flat = true;
    Program P;
    int dest_array = add_array(P, spec.dest.expression(), Cls::SCAL, false, dom, true);
    if (dest_array < 0) return false;
    int root_id = add_node(P, spec.root);
    int red_id = P.memo[red.expression().get()];
    // classify: epilogue nodes are scalars, the reduced argument is the flat domain
    std::function<bool(int)> cls_epi = [&](int id) -> bool {
        PNode& nd = P.nodes[id];
        if (id == red_id) {
            nd.cls = Cls::SCAL;
            nd.cls_set = true;
            return classify(P, nd.args[0], Cls::FULL, dom);
        }
        if (numel_of(nd.shape) != 1) return false;
        if (nd.kind == Kind::SCALAR) { nd.cls = Cls::SCAL; nd.cls_set = true; return true; }
        if (nd.kind == Kind::BUFFER) {
            nd.cls = Cls::SCAL;
            nd.cls_set = true;
            int ai = add_array(P, nd.src, Cls::SCAL, false, dom, false);
            if (ai < 0) return false;
            P.nodes[id].array = ai;
            return true;
        }
        if (nd.kind != Kind::ELEMENTWISE && nd.kind != Kind::EXPAND_DIMS && nd.kind != Kind::BROADCAST) return false;
        nd.cls = Cls::SCAL;
        nd.cls_set = true;
        std::vector<int> args = nd.args;
        for (int a : args)
            if (!cls_epi(a)) return false;
        return true;
    };
    if (!cls_epi(root_id)) return false;
    count_uses(P, {root_id});
    bool aligned = true;
    for (const ArrayArg& a : P.arrays)
        if (a.cls == Cls::FULL && a.buf->offset % 4 != 0) aligned = false;
    int VEC = n >= 16 ? 4 : 1, BT = 256;
    const bool UNALIGNED = VEC > 1 && !aligned, REST = VEC > 1 && n % VEC != 0;
    int max_el_all = 4;
    for (const ArrayArg& a : P.arrays) max_el_all = std::max(max_el_all, size_of_dtype(a.buf->dtype));
    static const int unroll_env = env_int("DALI_HIP_ALL_UNROLL", 0), tail_env = env_int("DALI_HIP_ALL_TAIL", 0);
    const int UNROLL = unroll_env > 0 ? unroll_env : (max_el_all == 8 ? 4 : 8);  // vector loads in flight per thread
    const int TAIL = tail_env > 0 ? tail_env : 2, MAX_BLOCKS = TAIL * BT;  // 512 blocks; the last one folds every partial in one unrolled pass
    std::vector<Output> outs(1);
    outs[0].root = root_id;
    outs[0].array = dest_array;
    outs[0].op = spec.op;
    outs[0].cls = Cls::SCAL;
    std::ostringstream params;
    const bool NT = n * (int64_t)max_el_all >= ((int64_t)64 << 20);
    params << VEC << "," << BT << "," << red_id << "," << UNROLL << "," << TAIL << "," << NT << "," << UNALIGNED << REST;
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash("all", signature(P, outs), params.str());
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    std::vector<int> shape_ndims = {1};
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = "all";
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = BT;
        K->plan.grid_kind = DALI_HIP_GRID_ALL;
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = 1;
        K->plan.work_per_block = BT * VEC * UNROLL;
        K->plan.max_blocks = MAX_BLOCKS;
        K->plan.ws_elsize = 16;
    }
    std::vector<std::vector<int>> shapes = {{(int)n}};
    load_and_launch(*K, [&]() { return gen_all_kernel(P, red_id, root_id, dest_array, spec.op, L, VEC, BT, UNROLL, TAIL, NT, UNALIGNED, REST, K->name); }, P, shapes);
    return true;
}

}  // namespace jit

}  // namespace dali
