// The column kernel: reduction over the leading axis (or a middle axis) of a row-major array, coalesced along the
// kept axis, two stages through the library workspace in one launch.
#include "jit_internal.h"

namespace dali {
namespace jit {

// root = AXIS_REDUCE (optionally under EXPAND_DIMS) over an elementwise argument
// whose buffers are [K, X] views with unit stride along the KEPT axis K: the
// transposed view op::axis_reduce builds for a leading-axis reduction
// (dali/array/op/reducer_operation.cpp:642-655). Lanes own VEC adjacent kept
// columns (coalesced 128-bit loads along memory rows), the waves of a block and
// the blocks along grid.y split the reduced axis; partials go through the
// workspace and the last block of each column strip folds them in y order.
struct ColLeaf {
    int array;
};

// Kept axes [0, split) of a [kept..., reduced] view must merge into one batch axis and kept axes
// [split, n_kept) into one unit-stride axis; the reduced (last) axis may have any stride.
static bool col_buffer_layout(const Expr* e, const std::vector<int>& shape, int split, int64_t* batch_stride) {
    auto st = strides_of(e);
    const int nk = (int)shape.size() - 1;
    int64_t expect = 1;
    for (int d = nk - 1; d >= split; --d) {
        if (shape[d] == 1) continue;
        if (st[d] != expect) return false;
        expect *= shape[d];
    }
    int64_t bs = 0;
    bool first = true;  // (a flag of its own: with a reversed axis the expected stride is itself negative)
    for (int d = split - 1; d >= 0; --d) {
        if (shape[d] == 1) continue;
        if (first) {
            bs = st[d];
            first = false;
        } else if (st[d] != expect) {
            return false;
        }
        expect = (int64_t)st[d] * shape[d];
    }
    if (batch_stride) *batch_stride = bs;
    return true;
}

// [kept..., 1] against [kept..., X]
bool col_kept_vector(const std::vector<int>& s, const std::vector<int>& shape) {
    if (s.size() != shape.size() || s.empty() || s.back() != 1 || shape.back() == 1) return false;
    for (size_t d = 0; d + 1 < s.size(); ++d)
        if (s[d] != shape[d]) return false;
    return true;
}

static bool col_eligible(const Array& a, const std::vector<int>& shape, int split, std::set<const Expr*>& seen) {
    auto e = a.expression();
    if (seen.count(e.get())) return true;
    seen.insert(e.get());
    switch (e->kind) {
        case Kind::SCALAR: return true;
        case Kind::BUFFER: {
            if (numel_of(e->shape) == 1) return true;
            if (e->shape == shape) return col_buffer_layout(e.get(), shape, split, nullptr);
            // one value per kept index, constant along the reduced axis ([kept..., 1] under a broadcast)
            if (col_kept_vector(e->shape, shape)) return col_buffer_layout(e.get(), e->shape, split, nullptr);
            return false;
        }
        case Kind::ELEMENTWISE:
            for (const Array& x : e->args) {
                if (numel_of(x.shape()) != numel_of(shape) && numel_of(x.shape()) != 1) return false;
                if (!col_eligible(x, shape, split, seen)) return false;
            }
            return true;
        case Kind::BROADCAST: {
            const Array& in = e->args[0];
            if (numel_of(in.shape()) == 1) return col_eligible(in, shape, split, seen);
            return e->shape == shape && in.is_buffer() && col_kept_vector(in.shape(), shape) && col_eligible(in, shape, split, seen);
        }
        default: return false;
    }
}

// The first split of the kept axes into [batch..., unit-stride run...] that every operand of a
// [kept..., reduced] argument fits (0: no batch axis); -1 when there is none.
int col_split_of(const Array& arg) {
    const int nk = arg.ndim() - 1;
    for (int sp = 0; sp < nk; ++sp) {
        std::set<const Expr*> seen;
        if (col_eligible(arg, arg.shape(), sp, seen)) return sp;
    }
    return -1;
}

static std::string gen_col_kernel(const Program& P, int red_id, int dest_array, OPERATOR_T op, const IvLayout& L, int VEC, int UNR, int TAIL, int RG, bool NT,
                           int IL, bool BATCHED, bool UNALIGNED, bool SHIFT, const std::string& kname) {
    // UNALIGNED: memory rows start off a 16-byte boundary (element-aligned vector loads). SHIFT: K is no multiple of
    // VEC; the lane whose vector would cross the end of the kept axis moves it back to end at K, reduces those VEC
    // columns like any other lane and stores only the ones its left neighbour does not own.
    const std::string ld = UNALIGNED ? (NT ? "dali_loadu_nt<" : "dali_loadu<") : (NT ? "dali_load_nt<" : "dali_load<");
    const PNode& red = P.nodes[red_id];
    const bool ARG = red.kind == Kind::ARG_AXIS_REDUCE;  // carries (value, row index); ties keep the lower index
    // softmax statistics: the accumulator is a (maximum, sum of exponentials) pair fed with plain values; the destination
    // holds the K maxima followed by the K sums
    const bool PAIR = red.name == "reducers::maxsumexp";
    std::string t = PAIR ? std::string("dali_ms") : ctype(P.nodes[red.args[0]].dtype);
    const std::string feed = PAIR ? red.name + "::feed(" : red.name + "::step<" + t + ">(";
    std::string dt = ctype(P.arrays[dest_array].buf->dtype);
    const std::string Rd = red.name;
    // fold candidate (cv, ci) into (av, ai)
    auto take = [&](const std::string& av, const std::string& ai, const std::string& cv, const std::string& ci) {
        return "if (" + Rd + "::better<" + t + ">(" + cv + ", " + av + ") || (" + cv + " == " + av + " && " + ci + " < " + ai + ")) { " + av + " = " + cv + "; " + ai + " = " + ci + "; }";
    };
    RowParams rp;
    rp.cached = false;
    rp.VEC = VEC;
    std::ostringstream ss;
    ss << device_prelude();
    ss << kargs_struct(P, L);
    ss << "extern \"C\" __global__ __launch_bounds__(256) void " << kname << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n";
    // the 256 threads form RG row groups of TPP threads; a group reads TPP*VEC adjacent kept columns of one memory row
    ss << "  constexpr int VEC = " << VEC << ", NWAVE = " << RG << ", TPP = " << 256 / RG << ", UNR = " << UNR << ", TAIL = " << TAIL << ";\n";
    ss << "  const long K = A.iv[" << L.shape_pos[0] << "], X = A.iv[" << L.shape_pos[0] + 1 << "];\n";
    ss << "  const long row = 0; const long C = K; (void)row; (void)C;\n";
    ss << "  const int lane = threadIdx.x % TPP, wave = threadIdx.x / TPP;\n";
    ss << "  const long k0 = ((long)blockIdx.x * TPP + lane) * VEC;\n";
    ss << "  const bool k_ok = k0 < K;\n";
    ss << "  const long ks = " << (SHIFT ? "k_ok && k0 + VEC > K ? K - VEC : k0" : "k0") << ";  // first kept column this lane reads\n";
    // BATCHED: the kept index runs over [batch, unit-stride run]; a lane's VEC kept elements lie in one run, and
    // the second shape entry holds the run length followed by one batch stride per array
    if (BATCHED) ss << "  const long k_run = A.iv[" << L.shape_pos[1] << "], k_batch = k0 / k_run, k_in = k0 - k_batch * k_run;\n";
    std::vector<int> kept_vectors;  // operands with one value per kept index
    for (size_t i = 0; i < P.arrays.size(); ++i) {
        const ArrayArg& a = P.arrays[i];
        std::string ty = ctype(a.buf->dtype);
        if (a.is_dest) {
            ss << "  " << ty << "* q" << i << " = (" << ty << "*)A.p[" << i << "];\n  const long ds" << i << " = " << (a.strided ? "A.iv[" + std::to_string(L.stride_pos[i]) + "]" : "1") << ";\n";
        } else if (a.cls == Cls::FULL || a.cls == Cls::ROW) {
            if (BATCHED)
                ss << "  const " << ty << "* q" << i << " = (const " << ty << "*)A.p[" << i << "] + (k_ok ? k_batch * (long)A.iv[" << L.shape_pos[1] + 1 + i
                   << "] + k_in : 0);\n";
            else
                ss << "  const " << ty << "* q" << i << " = (const " << ty << "*)A.p[" << i << "] + (k_ok ? ks : 0);\n";
            if (a.cls == Cls::FULL) {
                ss << "  const long ld" << i << " = A.iv[" << L.stride_pos[i] + 1 << "];\n";
            } else {
                kept_vectors.push_back((int)i);
                ss << "  " << ty << " rl" << i << "v[VEC];\n  _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) rl" << i << "v[j] = k_ok ? q" << i << "[j] : (" << ty << ")0;\n";
            }
        } else {
            ss << "  const " << ty << " sl" << i << " = ((const " << ty << "*)A.p[" << i << "])[0];\n";
        }
    }
    std::vector<int> full_leaves;
    for (size_t i = 0; i < P.arrays.size(); ++i)
        if (!P.arrays[i].is_dest && P.arrays[i].cls == Cls::FULL) full_leaves.push_back((int)i);
    ss << "  " << t << " acc[VEC];\n  _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) acc[j] = " << red.name << "::init<" << t << ">();\n";
    if (ARG) ss << "  int acci[VEC];\n  _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) acci[j] = 0;\n";
    // contiguous share of the reduced axis for this y-block, interleaved over its waves
    // Which memory rows a y-block reads. 0: one contiguous share of the reduced axis. 1: single rows dealt
    // round-robin. 2: chunks of UNR*NWAVE consecutive rows dealt round-robin, so that the grid as a whole reads
    // one contiguous band of memory at any moment while the loads of one lane stay within a few pages.
    if (IL == 2) {
        ss << "  constexpr long XS = NWAVE;\n";
        ss << "  const long n_chunks = X / (UNR * NWAVE);\n";
        ss << "  const long x_end = X;\n";
        ss << "  if (k_ok) {\n";
    } else if (IL == 1) {
        ss << "  const long XS = (long)gridDim.y * NWAVE;\n";
        ss << "  const long x_end = X;\n";
        ss << "  if (k_ok) {\n    long x = (long)blockIdx.y * NWAVE + wave;\n";
    } else {
        ss << "  constexpr long XS = NWAVE;\n";
        ss << "  const long per_y = (X + gridDim.y - 1) / gridDim.y;\n";
        ss << "  const long x_begin = (long)blockIdx.y * per_y, x_end = x_begin + per_y < X ? x_begin + per_y : X;\n";
        ss << "  if (k_ok) {\n    long x = x_begin + wave;\n";
    }
    std::vector<int> first_body(P.nodes.size(), -1);
    // main loop: UNR independent row fetches in flight per lane
    if (IL == 2)
        ss << "    for (long ch = blockIdx.y; ch < n_chunks; ch += gridDim.y) {\n      const long x = ch * (UNR * NWAVE) + wave;\n";
    else
        ss << "    for (; x + (UNR - 1) * XS < x_end; x += UNR * XS) {\n";
    for (int i : full_leaves) {
        std::string ty = ctype(P.arrays[i].buf->dtype);
        ss << "      " << ty << " x" << i << "s[UNR][VEC];\n";
        ss << "      _Pragma(\"unroll\") for (int u = 0; u < UNR; ++u) { dali_vec<" << ty << ", VEC> tmp = " << ld << ty << ", VEC>(q" << i
           << " + (x + u * XS) * ld" << i << "); _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) x" << i << "s[u][j] = tmp.v[j]; }\n";
    }
    if (PAIR) ss << "      float vv[VEC][UNR];\n";
    ss << "      _Pragma(\"unroll\") for (int u = 0; u < UNR; ++u) {\n";
    for (int i : full_leaves) ss << "        const " << ctype(P.arrays[i].buf->dtype) << "* x" << i << " = x" << i << "s[u];\n";
    ss << "        _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n          const int col = 0; (void)col;\n";
    for (int i : kept_vectors) ss << "          const " << ctype(P.arrays[i].buf->dtype) << " rl" << i << " = rl" << i << "v[j];\n";
    {
        BodyEmitter be(P, rp, true, 0, &first_body);
        std::string v = be.value(red.args[0]);
        if (ARG)
            // a thread meets its rows in increasing order: a strictly better value is the first index of its kind
            ss << be.stmts.str() << "          { const " << t << " cv = " << v << "; if (" << Rd << "::better<" << t << ">(cv, acc[j])) { acc[j] = cv; acci[j] = (int)(x + u * XS); } }\n        }\n      }\n";
        else
            if (PAIR)
                ss << be.stmts.str() << "          vv[j][u] = " << v << ";\n        }\n      }\n      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) acc[j] = "
                   << red.name << "::feed_n<UNR>(acc[j], vv[j]);\n";
            else
            ss << be.stmts.str() << "          acc[j] = " << feed << "acc[j], " << v << ");\n        }\n      }\n";
    }
    if (IL == 2)
        ss << "    }\n    for (long x = n_chunks * (UNR * NWAVE) + (long)blockIdx.y * NWAVE + wave; x < x_end; x += (long)gridDim.y * NWAVE) {\n";
    else
        ss << "    }\n    for (; x < x_end; x += XS) {\n";
    for (int i : full_leaves) {
        std::string ty = ctype(P.arrays[i].buf->dtype);
        ss << "      " << ty << " x" << i << "[VEC];\n";
        ss << "      { dali_vec<" << ty << ", VEC> tmp = " << ld << ty << ", VEC>(q" << i << " + x * ld" << i << "); _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) x" << i << "[j] = tmp.v[j]; }\n";
    }
    ss << "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n        const int col = 0; (void)col;\n";
    for (int i : kept_vectors) ss << "        const " << ctype(P.arrays[i].buf->dtype) << " rl" << i << " = rl" << i << "v[j];\n";
    {
        BodyEmitter be(P, rp, true, 0, &first_body);
        std::string v = be.value(red.args[0]);
        if (ARG)
            ss << be.stmts.str() << "        { const " << t << " cv = " << v << "; if (" << Rd << "::better<" << t << ">(cv, acc[j])) { acc[j] = cv; acci[j] = (int)x; } }\n      }\n";
        else
            ss << be.stmts.str() << "        acc[j] = " << feed << "acc[j], " << v << ");\n      }\n";
    }
    ss << "    }\n  }\n";
    // fold the row groups of the block in group order
    ss << "  __shared__ " << t << " sm[NWAVE][TPP * VEC];\n  __shared__ int is_last;\n";
    if (ARG) ss << "  __shared__ int smi[NWAVE][TPP * VEC];\n";
    auto emit_group_fold = [&](const std::string& ind) {
        ss << ind << "if (NWAVE > 1) {\n" << ind << "  _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) { sm[wave][lane * VEC + j] = acc[j];" << (ARG ? " smi[wave][lane * VEC + j] = acci[j];" : "")
           << " }\n" << ind << "  __syncthreads();\n";
        ss << ind << "  if (wave == 0) {\n" << ind << "    _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n" << ind << "      " << t << " r = sm[0][lane * VEC + j];\n";
        if (ARG) {
            ss << ind << "      int ri = smi[0][lane * VEC + j];\n";
            ss << ind << "      _Pragma(\"unroll\") for (int w = 1; w < NWAVE; ++w) { const " << t << " ov = sm[w][lane * VEC + j]; const int oi = smi[w][lane * VEC + j]; " << take("r", "ri", "ov", "oi") << " }\n";
            ss << ind << "      acc[j] = r; acci[j] = ri;\n";
        } else {
            ss << ind << "      _Pragma(\"unroll\") for (int w = 1; w < NWAVE; ++w) r = " << red.name << "::step<" << t << ">(r, sm[w][lane * VEC + j]);\n" << ind << "      acc[j] = r;\n";
        }
        ss << ind << "    }\n" << ind << "  }\n" << ind << "}\n";
    };
    emit_group_fold("  ");
    auto emit_store = [&](const std::string& indent) {
        if (PAIR) {
            ss << indent << "_Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) if (ks + j >= k0 && ks + j < K) { " << dt << "* dp = q" << dest_array << " + (ks + j) * ds"
               << dest_array << "; dp[0] = acc[j].m; dp[K * ds" << dest_array << "] = acc[j].l; }\n";
            return;
        }
        ss << indent << "_Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) if (ks + j >= k0 && ks + j < K) { " << dt << "* dp = q" << dest_array << " + (ks + j) * ds" << dest_array
           << "; *dp = " << op_combine(op, "(*dp)", std::string("(") + dt + ")" + (ARG ? "acci[j]" : "acc[j]")) << "; }\n";
    };
    ss << "  if (gridDim.y == 1) {\n    if (wave == 0 && k_ok) {\n";
    emit_store("      ");
    ss << "    }\n    return;\n  }\n";
    ss << "  unsigned int* counters = (unsigned int*)A.ws;\n";
    ss << "  " << t << "* partials = (" << t << "*)((char*)A.ws + " << 16384 * 4 << ");\n";
    ss << "  const long KP = (long)gridDim.x * TPP * VEC;  // padded kept extent of one row of partials\n";
    ss << "  const long pcol = ((long)blockIdx.x * TPP + lane) * VEC;\n";
    // same fence-free hand-off as the full reduction: agent-scope atomic stores, wait for their
    // acknowledgement, then the ticket; the last block of the strip observes with agent-scope loads
    if (ARG) ss << "  int* pidx = (int*)(partials + (long)gridDim.y * KP);  // the indices follow the values\n";
    ss << "  if (wave == 0) {\n    _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) { dali_publish(partials + (long)blockIdx.y * KP + pcol + j, acc[j]);"
       << (ARG ? " dali_publish(pidx + (long)blockIdx.y * KP + pcol + j, acci[j]);" : "") << " }\n"
          "    dali_stores_acknowledged();\n  }\n  __syncthreads();\n";
    ss << "  if (threadIdx.x == 0) is_last = dali_take_ticket(&counters[blockIdx.x]) == gridDim.y - 1;\n  __syncthreads();\n";
    ss << "  if (!is_last) return;\n";
    // every row group of the last block folds a contiguous share of the partial rows in y order (TAIL of them in
    // flight at a time); the groups are then joined in group order through LDS
    ss << "  _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) acc[j] = " << red.name << "::init<" << t << ">();\n";
    if (ARG) ss << "  _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) acci[j] = 2147483647;\n";
    ss << "  const unsigned int y_per = (gridDim.y + NWAVE - 1) / NWAVE;\n";
    ss << "  const unsigned int y_begin = wave * y_per, y_end = y_begin + y_per < gridDim.y ? y_begin + y_per : gridDim.y;\n";
    ss << "  for (unsigned int y0 = y_begin; y0 < y_end; y0 += TAIL) {\n    dali_vec<" << t << ", VEC> pv[TAIL];\n";
    if (ARG) ss << "    dali_vec<int, VEC> pi[TAIL];\n";
    ss << "    _Pragma(\"unroll\") for (int k = 0; k < TAIL; ++k) if (y0 + k < y_end) {\n"
          "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) { pv[k].v[j] = dali_observe(partials + (long)(y0 + k) * KP + pcol + j);"
       << (ARG ? " pi[k].v[j] = dali_observe(pidx + (long)(y0 + k) * KP + pcol + j);" : "") << " }\n    }\n";
    if (ARG)
        // the y-blocks hold interleaved chunks of rows: equal values are settled by the index itself
        ss << "    _Pragma(\"unroll\") for (int k = 0; k < TAIL; ++k) if (y0 + k < y_end) {\n      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) { "
           << take("acc[j]", "acci[j]", "pv[k].v[j]", "pi[k].v[j]") << " }\n    }\n  }\n";
    else
        ss << "    _Pragma(\"unroll\") for (int k = 0; k < TAIL; ++k) if (y0 + k < y_end) {\n      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) acc[j] = "
           << red.name << "::step<" << t << ">(acc[j], pv[k].v[j]);\n    }\n  }\n";
    emit_group_fold("  ");
    ss << "  if (wave == 0 && k_ok) {\n";
    emit_store("    ");
    ss << "  }\n  if (threadIdx.x == 0) dali_publish(&counters[blockIdx.x], 0u);\n}\n";
    return ss.str();
}

bool try_col(const DestSpec& spec) {
    Array root = spec.root;
    while (root.expression()->kind == Kind::EXPAND_DIMS) root = root.expression()->args[0];
    auto re = root.expression();
    if (re->kind != Kind::AXIS_REDUCE && re->kind != Kind::ARG_AXIS_REDUCE) return false;
    const bool is_arg = re->kind == Kind::ARG_AXIS_REDUCE;
    Array arg = re->args[0];
    if (arg.ndim() < 2) return false;
    const std::vector<int> arg_shape = arg.shape();
    const int nk = arg.ndim() - 1;
    int64_t X = arg_shape[nk], K = numel_of(arg_shape) / std::max<int64_t>(1, X);
    if (K <= 1 || X == 0 || K * X >= ((int64_t)1 << 31)) return false;
    // the kept axes [batch..., unit-stride run...]: the first split every operand fits (0: no batch axis)
    const int split = col_split_of(arg);
    if (split < 0) return false;
    int64_t k_run = 1;
    for (int d = split; d < nk; ++d) k_run *= arg_shape[d];
    const bool BATCHED = k_run != K;
    const bool pair = re->name == "reducers::maxsumexp";  // K maxima followed by K sums of exponentials, float only
    if (pair && (is_arg || spec.op != OPERATOR_T_EQL || arg.dtype() != DTYPE_FLOAT || spec.dest.dtype() != DTYPE_FLOAT || !spec.dest.contiguous_memory())) return false;
    if (numel_of(spec.dest.shape()) != (pair ? 2 * K : K)) return false;
    Domain dom;
    dom.R = K;  // ROW-class destination has K entries
    dom.C = X;
    Program P;
    // (the pair form presents the first half of its destination, the maxima; the kernel stores the sums K entries further on)
    int dest_array = add_array(P, pair ? spec.dest.reshape({2, (int)K})[0].expression() : spec.dest.expression(), Cls::ROW, false, dom, true);
    if (dest_array < 0) return false;
    int red_id = add_node(P, root);
    // classify the argument tree: [K, X] buffers are FULL with the kept stride in strides[0]
    std::vector<int> batch_strides = {0};  // one per array of the program (the destination's is not used)
    std::function<bool(int)> cls = [&](int id) -> bool {
        PNode& nd = P.nodes[id];
        if (nd.cls_set) return true;
        nd.cls_set = true;
        if (nd.kind == Kind::SCALAR) { nd.cls = Cls::SCAL; return true; }
        if (nd.kind == Kind::BUFFER) {
            int64_t bs = 0;
            ArrayArg a;
            a.buf = nd.src;
            if (numel_of(nd.shape) == 1) {
                a.cls = Cls::SCAL;
                a.nd = 1;
                a.sizes = {1};
                nd.cls = Cls::SCAL;
            } else if (col_kept_vector(nd.shape, arg_shape)) {
                // one value per kept index: read once per lane, ahead of the loop over the reduced axis
                col_buffer_layout(nd.src.get(), nd.shape, split, &bs);
                a.cls = Cls::ROW;
                a.nd = 1;
                a.sizes = {(int)K};
                nd.cls = Cls::ROW;
            } else {
                auto st = strides_of(nd.src.get());
                col_buffer_layout(nd.src.get(), arg_shape, split, &bs);
                a.cls = Cls::FULL;
                a.nd = 2;
                a.sizes = {(int)K, (int)X};
                a.strided = true;
                a.strides = {nk == 1 ? st[0] : 1, st[nk]};
                a.row_stride = a.strides[0];
                a.col_stride = st[nk];
                nd.cls = Cls::FULL;
            }
            std::string key = array_key(nd.src.get(), a.cls, false);
            for (size_t i = 0; i < P.arrays.size(); ++i)
                if (!P.arrays[i].is_dest && array_key(P.arrays[i].buf.get(), P.arrays[i].cls, false) == key) {
                    P.nodes[id].array = (int)i;
                    return true;
                }
            P.arrays.push_back(a);
            batch_strides.resize(P.arrays.size(), 0);
            batch_strides.back() = (int)bs;
            P.nodes[id].array = (int)P.arrays.size() - 1;
            return true;
        }
        nd.cls = numel_of(nd.shape) == 1 ? Cls::SCAL : Cls::FULL;
        std::vector<int> args = nd.args;
        for (int a : args)
            if (!cls(a)) return false;
        return true;
    };
    P.nodes[red_id].cls = Cls::ROW;
    P.nodes[red_id].cls_set = true;
    if (!cls(P.nodes[red_id].args[0])) return false;
    count_uses(P, {red_id});
    // a lane's vector lies within one unit-stride run; without a batch axis the last vector may be moved back instead
    const bool vec = BATCHED ? k_run % 4 == 0 : K >= 16;
    bool aligned = true;
    for (const ArrayArg& a : P.arrays)
        if (!a.is_dest && a.cls == Cls::FULL && (a.buf->offset % 4 != 0 || a.col_stride % 4 != 0)) aligned = false;
    for (int bs : batch_strides)
        if (bs % 4 != 0) aligned = false;
    int VEC = vec ? 4 : 1;
    const bool UNALIGNED = VEC > 1 && !aligned, SHIFT = VEC > 1 && K % VEC != 0;
    static const int IL = env_int("DALI_HIP_COL_INTERLEAVE", 2);
    static const int rg_env = env_int("DALI_HIP_COL_RG", 0), tail_env = env_int("DALI_HIP_COL_TAIL", 16);
    static const int unr_env = env_int("DALI_HIP_COL_UNR", 8), rows_env = env_int("DALI_HIP_COL_ROWS", 0);
    static const int blocks_env = env_int("DALI_HIP_COL_BLOCKS", 0);
    // One 256-thread workgroup per CU keeps eight loads per lane in flight and is best for a bare reduction; with
    // transcendental arithmetic on every element a single wave per SIMD cannot overlap it with its loads, and two
    // workgroups per CU are better (sum(exp(x)) along the leading axis of [8192,8192]: 61 -> 45 us; bare sum 40.6 -> 42.1)
    // (small problems keep one: [4096,1024] 13 us against 20 us with the extra partial results to fold)
    const bool streaming = K * X * (int64_t)size_of_dtype(arg.dtype()) >= ((int64_t)64 << 20);
    const int max_blocks = blocks_env > 0 ? blocks_env : (streaming && (pair || contains_expensive(P, P.nodes[red_id].args[0])) ? 512 : 256);
    const int UNR = unr_env;
    // four row groups of one wave each: a wave reads 1 KiB pieces of memory rows, a block owns a 256-column strip.
    // Narrow strips and few y-blocks measured best (8192x8192: 53 us with 1024-column strips x 32 y-blocks,
    // 41 us with 256-column strips x 8 y-blocks).
    int RG = 4;
    if (rg_env > 0) RG = rg_env;
    const int TAIL = tail_env;
    std::vector<Output> outs(1);
    outs[0].root = red_id;
    outs[0].array = dest_array;
    outs[0].op = spec.op;
    outs[0].cls = Cls::ROW;
    std::ostringstream params;
    const bool NT = K * X * (int64_t)size_of_dtype(arg.dtype()) >= ((int64_t)64 << 20);
    static const int maxy_env = env_int("DALI_HIP_COL_MAXY", 256);
    params << VEC << "," << UNR << "," << TAIL << "," << RG << "," << NT << "," << IL << "," << BATCHED << UNALIGNED << SHIFT << "," << max_blocks;
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash("col", signature(P, outs), params.str());
    std::shared_ptr<KernelSpec>& Kp = specs_cache[h];
    std::vector<int> shape_ndims = {2};
    batch_strides.resize(P.arrays.size(), 0);
    if (BATCHED) shape_ndims.push_back(1 + (int)batch_strides.size());
    IvLayout L = layout_iv(P, shape_ndims);
    if (!Kp) {
        Kp = std::make_shared<KernelSpec>();
        Kp->hash = h;
        Kp->kind = "col";
        Kp->name = kernel_name(Kp->kind, h);
        fill_plan_arrays(*Kp, P, shape_ndims);
        Kp->plan.block_threads = 256;
        Kp->plan.grid_kind = DALI_HIP_GRID_COLS;
        Kp->plan.work_begin = L.shape_pos[0];
        Kp->plan.work_count = 1;
        Kp->plan.work_per_block = (256 / RG) * VEC;
        Kp->plan.work2_begin = L.shape_pos[0] + 1;
        Kp->plan.work2_per_block = rows_env > 0 ? rows_env : UNR * RG;  // fewest reduced rows per y-block
        Kp->plan.max_blocks2 = maxy_env;
        Kp->plan.max_blocks = max_blocks;  // the y split fills what the column strips leave
        Kp->plan.ws_elsize = pair ? 8 : size_of_dtype(arg.dtype()) + (is_arg ? 4 : 0);  // a partial is a value, plus its index
    }
    std::vector<std::vector<int>> shapes = {{(int)K, (int)X}};
    if (BATCHED) {
        shapes.push_back({(int)k_run});
        shapes.back().insert(shapes.back().end(), batch_strides.begin(), batch_strides.end());
    }
    load_and_launch(*Kp, [&]() { return gen_col_kernel(P, red_id, dest_array, spec.op, L, VEC, UNR, TAIL, RG, NT, IL, BATCHED, UNALIGNED, SHIFT, Kp->name); }, P, shapes);
    return true;
}

}  // namespace jit

}  // namespace dali
