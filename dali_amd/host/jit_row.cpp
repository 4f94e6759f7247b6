// The row kernel: reductions over the trailing axis with their results broadcast back onto the row (softmax,
// log-sum-exp, argmax, cross-entropy), and the strided / broadcasting 2-D map (no reduction phase). A row lives in the
// registers of TPR threads; wave64 cross-lane reductions, one LDS hop across waves.
#include "jit_internal.h"

namespace dali {
namespace jit {


// The statistics of a softmax or a log-sum-exp as two reduction phases: a maximum over the row, then the sum of
// exp(x - that maximum) over the same values x. Gives the two reduction nodes and the node of x.
static bool max_then_sum_of_exp(const RowPlan& rpn, int* max_id, int* sum_id, int* arg_id) {
    const Program& P = rpn.P;
    if (rpn.n_phases < 2 || rpn.phase_reduces[0].size() != 1 || rpn.phase_reduces[1].size() != 1) return false;
    const int m_id = rpn.phase_reduces[0][0], s_id = rpn.phase_reduces[1][0];
    const PNode& mx = P.nodes[m_id];
    const PNode& sm = P.nodes[s_id];
    auto through_views = [&](int id) {
        while (P.nodes[id].kind == Kind::BROADCAST || P.nodes[id].kind == Kind::EXPAND_DIMS) id = P.nodes[id].args[0];
        return id;
    };
    if (mx.kind != Kind::AXIS_REDUCE || mx.name != "reducers::maximum" || sm.kind != Kind::AXIS_REDUCE || sm.name != "reducers::sum" ||
        mx.dtype != DTYPE_FLOAT || sm.dtype != DTYPE_FLOAT)
        return false;
    const PNode& ex = P.nodes[sm.args[0]];
    if (ex.kind != Kind::ELEMENTWISE || ex.name != "functor::exp" || ex.args.size() != 1) return false;
    const PNode& sub = P.nodes[ex.args[0]];
    if (sub.kind != Kind::ELEMENTWISE || sub.name != "functor::subtract" || sub.args.size() != 2 || sub.args[0] != mx.args[0] ||
        through_views(sub.args[1]) != m_id || P.nodes[mx.args[0]].dtype != DTYPE_FLOAT)
        return false;
    *max_id = m_id;
    *sum_id = s_id;
    *arg_id = mx.args[0];
    return true;
}

static std::string gen_row_kernel(const RowPlan& rpn, const IvLayout& L, const std::string& kname) {
    const Program& P = rpn.P;
    const RowParams& rp = rpn.rp;
    std::ostringstream ss;
    ss << device_prelude();
    ss << kargs_struct(P, L);
    ss << "extern \"C\" __global__ __launch_bounds__(" << rp.BT << ") ";
    if (rp.waves_per_eu > 0) ss << "__attribute__((amdgpu_waves_per_eu(" << rp.waves_per_eu << ", " << rp.waves_per_eu << "))) ";
    ss << "void " << kname << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n";
    ss << "  constexpr int VEC = " << rp.VEC << ", TPR = " << rp.TPR << ", RPB = " << rp.RPB << ";\n";
    if (rp.cached) ss << "  constexpr int EPT = " << rp.EPT << ";\n";
    ss << "  const int tid = threadIdx.x;\n  const int tr = tid % TPR;\n";
    if (rp.band > 1) {
        // the shape entry is {strips, bands, R, C}: neighbouring workgroups take neighbouring strips of TPR vectors of the
        // same band of rows, so that the device as a whole reads whole rows (all memory channels) at any moment
        ss << "  constexpr int BAND = " << rp.band << ";\n";
        ss << "  const unsigned int strips = A.iv[" << L.shape_pos[0] << "];\n";
        ss << "  const long R = A.iv[" << L.shape_pos[0] + 2 << "], C = A.iv[" << L.shape_pos[0] + 3 << "];\n";
        ss << "  long row = (long)(blockIdx.x / strips) * BAND;  // first row of this workgroup's band\n  constexpr bool row_ok = true; (void)row_ok;\n";
        ss << "  const int CH = (int)(C / VEC); (void)CH;\n";
        ss << "  const int ch = (int)(blockIdx.x % strips) * TPR + tr;\n";
    } else if (rp.split) {
        // the shape entry is {S, R, C}: workgroup b works on piece b % S of row b / S
        ss << "  const int S = A.iv[" << L.shape_pos[0] << "];\n";
        ss << "  const long R = A.iv[" << L.shape_pos[0] + 1 << "], C = A.iv[" << L.shape_pos[0] + 2 << "];\n";
        ss << "  long row = blockIdx.x / (unsigned)S;\n  const int seg = (int)(blockIdx.x - (unsigned)row * (unsigned)S);\n";
        ss << "  constexpr bool row_ok = true;\n  (void)R;\n";
        ss << "  const int CH = (int)(C / VEC); (void)CH;\n";
        ss << "  const int CHS = (CH + S - 1) / S, ch_begin = seg * CHS, ch_end = ch_begin + CHS < CH ? ch_begin + CHS : CH;\n";
    } else {
    ss << "  const long R = A.iv[" << L.shape_pos[0] << "], C = A.iv[" << L.shape_pos[0] + 1 << "];\n";
    ss << "  long row = (long)blockIdx.x * RPB + tid / TPR;\n";
    if (rp.RPB == 1)
        ss << "  constexpr bool row_ok = true;  // one row per workgroup: the grid has exactly R of them\n  (void)R;\n";
    else
        ss << "  const bool row_ok = row < R;\n  if (!row_ok) row = R - 1;\n";
    if (!rp.peel) ss << "  const int CH = (int)(C / VEC); (void)CH;\n";
    }
    emit_row_prologue(ss, P, L);
    // FULL leaves (inputs)
    std::vector<int> full_leaves;
    for (size_t i = 0; i < P.arrays.size(); ++i)
        if (!P.arrays[i].is_dest && P.arrays[i].cls == Cls::FULL && !P.arrays[i].gather_source) full_leaves.push_back((int)i);
    // vector accesses go through v<i>: the row pointer, moved to the row's first 16-byte boundary when the rows are peeled
    const std::string vp = rp.peel ? "v" : "q";
    if (rp.peel) {
        int first = -1;
        for (size_t i = 0; i < P.arrays.size() && first < 0; ++i)
            if (P.arrays[i].cls == Cls::FULL && !P.arrays[i].gather_source) first = (int)i;
        // (rows as wide as a wave or wider: up to the first 128-byte boundary, so that a wave's kilobyte is eight whole cache lines)
        ss << "  const int head = (int)((0u - (unsigned int)((unsigned long)q" << first << " >> 2)) & " << (rp.TPR >= 64 && rpn.dom.C >= 8192 ? 31 : 3) << "u);  // elements in front of the row's first boundary\n";
        ss << "  const int CH = (int)((C - head) / VEC); (void)CH;\n";
        for (size_t i = 0; i < P.arrays.size(); ++i)
            if (P.arrays[i].cls == Cls::FULL && !P.arrays[i].gather_source)
                ss << "  " << (P.arrays[i].is_dest ? "" : "const ") << ctype(P.arrays[i].buf->dtype) << "* v" << i << " = q" << i << " + head;\n";
    }
    // an operand broadcast along the rows ([1, C]: row stride 0): with peeled rows its vectors start wherever the rows' do, at
    // element alignment, and it is read by every row, so it stays in the caches
    auto along_rows = [&](int i) { const ArrayArg& a = P.arrays[i]; return rp.peel && !a.is_dest && a.strided && a.strides[0] == 0; };
    const std::string col_of_ch = rp.peel ? "head + ch * VEC + j" : "ch * VEC + j";
    // ragged rows: the C % VEC elements past the last whole vector go one to a thread, through the same bodies
    // (slot EPT of the register cache, j = 0)
    const bool tail = rp.ragged && rp.tail;
    // (peeled rows: thread tr < head takes element tr, the others the elements behind the last vector, head + CH * VEC + (tr - head))
    if (tail) ss << "  const bool tail_on = tr < (int)(C - (long)CH * VEC)" << (rp.split ? " && seg == S - 1" : "") << ";\n  const int tail_col = "
                 << (rp.peel ? "tr < head ? tr : CH * VEC + tr" : "CH * VEC + tr") << ";\n";
    // register-cached rows whose length fills every chunk need no chunk guard
    const std::string chunk_guard = rp.cached && rp.exact ? "    {\n" : "    if (ch < CH) {\n";

    if (rp.cached && rp.EPT_L > 0) {
        // Hybrid row cache: a thread keeps its first EPT_R vectors in registers and the other EPT_L in LDS (its own
        // 16 bytes per slot, so no barrier is involved); two 1024-thread workgroups then fit a CU where the registers
        // alone allow one, and one row's arithmetic overlaps the other's loads. `x<i>(e, j)` picks the storage; `e` is
        // a constant after unrolling, so the selection folds away.
        ss << "  constexpr int EPT_L = " << rp.EPT_L << ", EPT_R = EPT - EPT_L;\n";
        for (int i : full_leaves) {
            const std::string t = ctype(P.arrays[i].buf->dtype);
            ss << "  " << t << " xr" << i << "[EPT_R + 1][VEC];\n";
            ss << "  __shared__ __attribute__((aligned(16))) " << t << " xl" << i << "[EPT_L][" << rp.BT << " * VEC];\n";
            ss << "#define x" << i << "(e, j) ((e) < EPT_R ? xr" << i << "[(e) < EPT_R ? (e) : 0][j] : ((e) >= EPT ? xr" << i << "[EPT_R][j] : xl" << i
               << "[(e) >= EPT_R && (e) < EPT ? (e) - EPT_R : 0][tid * VEC + (j)]))\n";
        }
        ss << "  _Pragma(\"unroll\") for (int e = 0; e < EPT; ++e) {\n    const int ch = tr + e * TPR;\n" << chunk_guard;
        for (int i : full_leaves) {
            const std::string t = ctype(P.arrays[i].buf->dtype);
            ss << "      " << t << " ld" << i << "[VEC];\n";
            emit_leaf_load(ss, P.arrays[i], i, rp.VEC, "ld" + std::to_string(i), "      ", rp.nt_loads && !along_rows(i), rp.ragged && (!rp.peel || along_rows(i)), vp);
            ss << "      if (e < EPT_R) {\n        _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) xr" << i << "[e < EPT_R ? e : 0][j] = ld" << i << "[j];\n      } else {\n";
            ss << "        dali_vec<" << t << ", VEC> lv; _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) lv.v[j] = ld" << i << "[j];\n";
            ss << "        dali_store<" << t << ", VEC>(&xl" << i << "[e >= EPT_R ? e - EPT_R : 0][tid * VEC], lv);\n      }\n";
        }
        ss << "    }\n  }\n";
        if (tail) {
            ss << "  if (tail_on) {\n";
            for (int i : full_leaves) ss << "    xr" << i << "[EPT_R][0] = q" << i << "[tail_col];\n";
            ss << "  }\n";
        }
    } else if (rp.cached) {
        for (int i : full_leaves) {
            ss << "  " << ctype(P.arrays[i].buf->dtype) << " x" << i << "[EPT + " << (tail ? 1 : 0) << "][VEC];\n";
        }
        ss << "  _Pragma(\"unroll\") for (int e = 0; e < EPT; ++e) {\n    const int ch = tr + e * TPR;\n" << chunk_guard;
        for (int i : full_leaves) emit_leaf_load(ss, P.arrays[i], i, rp.VEC, "x" + std::to_string(i) + "[e]", "      ", rp.nt_loads && !along_rows(i), rp.ragged && (!rp.peel || along_rows(i)), vp);
        ss << "    }\n  }\n";
        if (tail) {
            ss << "  if (tail_on) {\n";
            for (int i : full_leaves) ss << "    x" << i << "[EPT][0] = q" << i << "[tail_col];\n";
            ss << "  }\n";
        }
    }
    if (rp.cached) {
        for (size_t id = 0; id < P.nodes.size(); ++id)
            if (P.nodes[id].kept) ss << "  " << ctype(P.nodes[id].dtype) << " t" << id << "[EPT + " << (tail ? 1 : 0) << "][VEC];\n";
    }
    // opens the tail element's scope: the names a body refers to (e, j, col, x<i>) stand for that one element
    auto open_tail = [&](std::ostringstream& o, const std::string& cond) {
        o << "  if (" << cond << ") {\n";
        if (rp.cached) {
            o << "    constexpr int e = EPT; (void)e;\n";
        } else {
            for (int i : full_leaves) o << "    " << ctype(P.arrays[i].buf->dtype) << " x" << i << "[VEC];\n    x" << i << "[0] = q" << i << "[tail_col];\n";
        }
        o << "    constexpr int j = 0; (void)j;\n    const int col = tail_col; (void)col;\n";
    };
    auto open_loop = [&](std::ostringstream& o) {
        if (rp.cached) {
            o << "  _Pragma(\"unroll\") for (int e = 0; e < EPT; ++e) {\n    const int ch = tr + e * TPR;\n" << chunk_guard;
        } else {
            if (rp.split)
                o << (rpn.n_phases > 0 ? "  _Pragma(\"unroll 4\")\n" : "") << "  for (int ch = ch_begin + tr; ch < ch_end; ch += TPR) {\n    {\n";
            else
                o << "  for (int ch = tr; ch < CH; ch += TPR) {\n    {\n";
            for (int i : full_leaves) {
                o << "      " << ctype(P.arrays[i].buf->dtype) << " x" << i << "[VEC];\n";
                emit_leaf_load(o, P.arrays[i], i, rp.VEC, "x" + std::to_string(i), "      ", rp.nt_loads && !along_rows(i), rp.ragged && (!rp.peel || along_rows(i)), vp);
            }
        }
    };

    // A loop whose body divides by row constants is emitted twice behind one wave-uniform test: with the
    // reciprocals (product + FMA correction per element) when every divisor of the wave's rows has a normal
    // reciprocal, with plain quotients otherwise. Neither copy has a branch per element.
    int div_plans = 0;
    auto emit_with_division_plan = [&](std::ostringstream& o, const std::function<void(std::ostringstream&, int, std::vector<std::string>*)>& emit_loop) {
        std::vector<std::string> divisors;
        std::ostringstream probe;
        emit_loop(probe, 1, &divisors);
        if (divisors.empty()) {
            emit_loop(o, 0, nullptr);
            return;
        }
        const int plan = div_plans++;
        o << "  bool div_ok" << plan << " = true;\n";
        o << "  {\n";
        // the reciprocals live in this scope together with both copies of the loop
        for (size_t k = 0; k < divisors.size(); ++k)
            o << "  const float dr" << k << " = 1.0f / " << divisors[k] << ";\n  div_ok" << plan << " = div_ok" << plan << " && dali_div_ok(" << divisors[k] << ");\n";
        o << "  if (__all(div_ok" << plan << ")) {\n" << probe.str() << "  } else {\n";
        std::vector<std::string> again;
        emit_loop(o, 2, &again);
        o << "  }\n  }\n";
    };

    // Rows that are streamed (too long for the registers): a maximum followed by the sum of exp(x - maximum), the statistics
    // of a softmax or a log-sum-exp, are taken in ONE walk over the row. A thread keeps the largest value it has met and the
    // sum of the exponentials relative to it, and scales the sum when a larger value arrives; the threads' sums are scaled
    // to the row's maximum before they are added. The row is then read twice in all (statistics, output) instead of three times
    // ([1024,128256]: 361 -> 292 us, [512,151936]: 209 -> 167 us).
    int online_max = -1, online_sum = -1, online_arg = -1;
    static const int online_env = env_int("DALI_HIP_ROW_ONLINE_SOFTMAX", 1);
    // (pieces of rows: each piece ends with its own maximum and its own sum relative to it, which is what its workgroup writes)
    if (online_env && !rp.cached) max_then_sum_of_exp(rpn, &online_max, &online_sum, &online_arg);
    // reduction phases
    for (int p = 0; p < rpn.n_phases; ++p) {
        if (online_max >= 0 && p == 0) {
            const std::string m = "acc" + std::to_string(online_max), l = "acc" + std::to_string(online_sum);
            ss << "  float " << m << " = reducers::maximum::init<float>();\n  float " << l << " = 0.0f;\n";
            BodyEmitter be(P, rp, true, 0, &rpn.first_body);
            const std::string v = be.value(online_arg);
            const std::string update = "{ const float xv = " + v + "; if (xv > " + m + ") { " + l + " = " + l + " * functor::exp<float>::Map(functor::subtract<float>::Map(" + m +
                                       ", xv)) + 1.0f; " + m + " = xv; } else { " + l + " += functor::exp<float>::Map(functor::subtract<float>::Map(xv, " + m + ")); } }";
            open_loop(ss);
            ss << "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n        const int col = " << col_of_ch << "; (void)col;\n";
            ss << be.stmts.str() << "        " << update << "\n      }\n    }\n  }\n";
            if (tail) {
                open_tail(ss, "tail_on");
                ss << be.stmts.str() << "    " << update << "\n  }\n";
            }
            const std::string rm = "red" + std::to_string(online_max), rs = "red" + std::to_string(online_sum);
            if (rp.NW == 1) {
                ss << "  const float " << rm << " = dali_group_reduce<reducers::maximum, float, " << std::min(rp.TPR, 64) << ">(" << m << ");\n";
                ss << "  " << l << " *= functor::exp<float>::Map(functor::subtract<float>::Map(" << m << ", " << rm << "));\n";
                ss << "  const float " << rs << " = dali_group_reduce<reducers::sum, float, " << std::min(rp.TPR, 64) << ">(" << l << ");\n";
            } else {
                ss << "  __shared__ float sm" << online_max << "[" << rp.NW << "];\n  __shared__ float sm" << online_sum << "[" << rp.NW << "];\n";
                ss << "  const float " << rm << " = dali_block_reduce<reducers::maximum, float, " << rp.NW << ">(" << m << ", sm" << online_max << ");\n";
                ss << "  " << l << " *= functor::exp<float>::Map(functor::subtract<float>::Map(" << m << ", " << rm << "));\n";
                ss << "  const float " << rs << " = dali_block_reduce<reducers::sum, float, " << rp.NW << ">(" << l << ", sm" << online_sum << ");\n";
            }
            p = 1;  // both phases are done
            continue;
        }
        const std::vector<int>& reds = rpn.phase_reduces[p];
        for (int id : reds) {
            const PNode& n = P.nodes[id];
            std::string t = ctype(P.nodes[n.args[0]].dtype);
            ss << "  " << t << " acc" << id << " = " << n.name << "::init<" << t << ">();\n";
            if (n.kind == Kind::ARG_AXIS_REDUCE) ss << "  int acci" << id << " = 0;\n";
        }
        auto emit_phase_loop = [&](std::ostringstream& o, int div_mode, std::vector<std::string>* divisors) {
            open_loop(o);
            o << "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n        const int col = " << col_of_ch << "; (void)col;\n";
            BodyEmitter be(P, rp, true, p, &rpn.first_body);
            be.div_mode = div_mode;
            be.divisors = divisors;
            std::vector<std::string> updates;
            for (int id : reds) {
                const PNode& n = P.nodes[id];
                std::string t = ctype(P.nodes[n.args[0]].dtype);
                std::string v = be.value(n.args[0]);
                if (n.kind == Kind::AXIS_REDUCE) {
                    updates.push_back("acc" + std::to_string(id) + " = " + n.name + "::step<" + t + ">(acc" + std::to_string(id) + ", " + v + ");");
                } else {
                    updates.push_back("{ const " + t + " cand = " + v + "; if (" + n.name + "::better<" + t + ">(cand, acc" + std::to_string(id) +
                                      ")) { acc" + std::to_string(id) + " = cand; acci" + std::to_string(id) + " = col; } }");
                }
            }
            o << be.stmts.str();
            for (auto& u : updates) o << "        " << u << "\n";
            o << "      }\n    }\n  }\n";
            if (tail) {
                open_tail(o, "tail_on");
                o << be.stmts.str();
                for (auto& u : updates) o << "    " << u << "\n";
                o << "  }\n";
            }
        };
        emit_with_division_plan(ss, emit_phase_loop);
        for (int id : reds) {
            const PNode& n = P.nodes[id];
            std::string t = ctype(P.nodes[n.args[0]].dtype);
            if (n.kind == Kind::AXIS_REDUCE) {
                if (rp.NW == 1) {
                    ss << "  const " << t << " red" << id << " = dali_group_reduce<" << n.name << ", " << t << ", " << std::min(rp.TPR, 64) << ">(acc" << id << ");\n";
                } else {
                    ss << "  __shared__ " << t << " sm" << id << "[" << rp.NW << "];\n";
                    ss << "  const " << t << " red" << id << " = dali_block_reduce<" << n.name << ", " << t << ", " << rp.NW << ">(acc" << id << ", sm" << id << ");\n";
                }
            } else {
                if (rp.NW == 1) {
                    ss << "  dali_group_arg_reduce<" << n.name << ", " << t << ", " << std::min(rp.TPR, 64) << ">(acc" << id << ", acci" << id << ");\n";
                } else {
                    ss << "  __shared__ " << t << " sm" << id << "[" << rp.NW << "]; __shared__ int smi" << id << "[" << rp.NW << "];\n";
                    ss << "  dali_block_arg_reduce<" << n.name << ", " << t << ", " << rp.NW << ">(acc" << id << ", acci" << id << ", sm" << id << ", smi" << id << ");\n";
                }
                ss << "  const int red" << id << " = acci" << id << ";\n";
            }
        }
    }

    // totals over the rows: value per row -> workgroup (wave order) -> workspace slot -> last workgroup folds the slots
    std::vector<const Output*> totals;
    for (const Output& o : rpn.outputs)
        if (o.total_red >= 0) totals.push_back(&o);
    const int NWB = rp.BT / 64;
    // The slot and the ticket go out before the rows are written: the wave that draws the ticket waits for its earlier
    // memory operations, and after the output loop those would be a whole row of stores (the workgroup would keep
    // its place on the compute unit until they are acknowledged).
    auto emit_totals_publish = [&]() {
        ss << "  constexpr int BT = " << rp.BT << ";\n";
        ss << "  unsigned int* counters = (unsigned int*)A.ws;\n  char* slots = (char*)A.ws + " << 16384 * 4 << ";\n";
        ss << "  __shared__ int is_last;\n";
        for (size_t k = 0; k < totals.size(); ++k) {
            const PNode& red = P.nodes[totals[k]->total_red];
            const std::string t = ctype(P.nodes[red.args[0]].dtype);
            ss << "  " << t << " tot" << k << " = " << red.name << "::init<" << t << ">();\n";
            ss << "  __shared__ " << t << " smt" << k << "[" << NWB << "];\n";
        }
        ss << "  if (tr == 0 && row_ok) {\n";
        {
            BodyEmitter be(P, rp, false, rpn.n_phases, &rpn.first_body);
            std::ostringstream body;
            for (size_t k = 0; k < totals.size(); ++k) body << "    tot" << k << " = " << be.value(P.nodes[totals[k]->total_red].args[0]) << ";\n";
            ss << be.stmts.str() << body.str();
        }
        ss << "  }\n";
        for (size_t k = 0; k < totals.size() && rp.RPB > 1; ++k) {  // (one row per workgroup: thread 0 holds its value already)
            const PNode& red = P.nodes[totals[k]->total_red];
            const std::string t = ctype(P.nodes[red.args[0]].dtype);
            ss << "  tot" << k << " = dali_block_reduce<" << red.name << ", " << t << ", " << NWB << ">(tot" << k << ", smt" << k << ");\n";
        }
        ss << "  if (tid == 0) {\n";
        for (size_t k = 0; k < totals.size(); ++k) {
            const std::string t = ctype(P.nodes[P.nodes[totals[k]->total_red].args[0]].dtype);
            ss << "    dali_publish((" << t << "*)(slots + ((size_t)" << k << " * gridDim.x + blockIdx.x) * 8), tot" << k << ");\n";
        }
        ss << "    is_last = dali_last_arrival(counters, blockIdx.x, gridDim.x);\n  }\n";
    };
    auto emit_totals_fold = [&]() {
        ss << "  __syncthreads();\n  if (!is_last) return;\n";
        // fixed order: thread t folds slots t, t + BT, ... (eight loads in flight at a time), then the workgroup folds in wave order
        for (size_t k = 0; k < totals.size(); ++k) {
            const PNode& red = P.nodes[totals[k]->total_red];
            const std::string t = ctype(P.nodes[red.args[0]].dtype);
            ss << "  tot" << k << " = " << red.name << "::init<" << t << ">();\n";
            ss << "  for (unsigned int base = tid; base < gridDim.x; base += BT * 8) {\n    " << t << " pv[8];\n";
            ss << "    _Pragma(\"unroll\") for (int u = 0; u < 8; ++u) { const unsigned int b = base + u * BT; if (b < gridDim.x) pv[u] = dali_observe((const " << t
               << "*)(slots + ((size_t)" << k << " * gridDim.x + b) * 8)); }\n";
            ss << "    _Pragma(\"unroll\") for (int u = 0; u < 8; ++u) { const unsigned int b = base + u * BT; if (b < gridDim.x) tot" << k << " = " << red.name
               << "::step<" << t << ">(tot" << k << ", pv[u]); }\n  }\n";
            ss << "  __syncthreads();\n";
            ss << "  tot" << k << " = dali_block_reduce<" << red.name << ", " << t << ", " << NWB << ">(tot" << k << ", smt" << k << ");\n";
        }
        ss << "  if (tid == 0) {\n    dali_publish(&counters[0], 0u);\n";
        {
            BodyEmitter be(P, rp, false, rpn.n_phases + 1, &rpn.first_body);
            std::ostringstream body;
            for (size_t k = 0; k < totals.size(); ++k) {
                const Output& o = *totals[k];
                const PNode& red = P.nodes[o.total_red];
                ss << "    const " << ctype(red.dtype) << " red" << o.total_red << " = tot" << k << ";\n";
            }
            for (size_t k = 0; k < totals.size(); ++k) {
                const Output& o = *totals[k];
                const std::string dt = ctype(P.arrays[o.array].buf->dtype);
                const std::string v = be.value(o.root);
                body << "    q" << o.array << "[0] = " << op_combine(o.op, "q" + std::to_string(o.array) + "[0]", "(" + dt + ")(" + v + ")") << ";\n";
            }
            ss << be.stmts.str() << body.str();
        }
        ss << "  }\n";
    };
    if (!totals.empty()) emit_totals_publish();

    if (rp.band > 1) {
        // Operands that are broadcast along the rows (row stride 0) are loaded once per column chunk, what depends on them
        // alone (the reciprocal of such a divisor) is computed there, and the workgroup then walks its band of rows.
        auto is_colvec = [&](int i) { const ArrayArg& a = P.arrays[i]; return a.cls == Cls::FULL && !a.is_dest && a.strided && a.strides[0] == 0; };
        std::function<bool(int)> invariant = [&](int id) -> bool {
            const PNode& n = P.nodes[id];
            switch (n.kind) {
                case Kind::SCALAR: return true;
                case Kind::BUFFER: return P.arrays[n.array].cls == Cls::SCAL || is_colvec(n.array);
                case Kind::ELEMENTWISE: case Kind::BROADCAST: case Kind::EXPAND_DIMS:
                    for (int a : n.args) if (!invariant(a)) return false;
                    return true;
                default: return false;
            }
        };
        auto row_stride = [&](int i) { return P.arrays[i].strided ? "(long)A.iv[" + std::to_string(L.stride_pos[i]) + "]" : std::string("C"); };
        std::vector<int> divs;
        {
            BodyEmitter probe(P, rp, true, rpn.n_phases, &rpn.first_body);
            probe.band_divisors = &divs;
            probe.band_invariant = invariant;
            probe.div_mode = 1;
            for (const Output& o : rpn.outputs) (void)probe.value(o.root);
        }
        ss << "  if (ch < CH) {\n";
        for (int i : full_leaves)
            if (is_colvec(i)) {
                ss << "    " << ctype(P.arrays[i].buf->dtype) << " x" << i << "[VEC];\n";
                emit_leaf_load(ss, P.arrays[i], i, rp.VEC, "x" + std::to_string(i), "    ", false, rp.ragged);
            }
        if (!divs.empty()) ss << "    bool hok = true;\n";
        for (size_t k = 0; k < divs.size(); ++k) {
            ss << "    float hv" << k << "[VEC], hr" << k << "[VEC];\n    _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n      const int col = ch * VEC + j; (void)col;\n";
            BodyEmitter hb(P, rp, true, rpn.n_phases, &rpn.first_body);
            const std::string v = hb.value(divs[k]);
            ss << hb.stmts.str() << "      hv" << k << "[j] = " << v << "; hr" << k << "[j] = 1.0f / hv" << k << "[j]; hok = hok && dali_div_ok(hv" << k << "[j]);\n    }\n";
        }
        auto emit_rows = [&](int div_mode) {
            // U rows at a time: their loads are all issued before the first row is worked on
            const int U = rp.band_unroll;
            auto row_pointer = [&](size_t i, const std::string& rr, const char* indent) {
                const ArrayArg& a = P.arrays[i];
                ss << indent << (a.is_dest ? "" : "const ") << ctype(a.buf->dtype) << "* w" << i << " = q" << i << " + (long)(" << rr << ") * " << row_stride((int)i) << ";\n";
            };
            ss << "    for (int r0 = 0; r0 < BAND; r0 += " << U << ") {\n      if (row + r0 >= R) break;\n";
            for (int i : full_leaves)
                if (!is_colvec(i)) ss << "      " << ctype(P.arrays[i].buf->dtype) << " x" << i << "u[" << U << "][VEC];\n";
            ss << "      _Pragma(\"unroll\") for (int u = 0; u < " << U << "; ++u) {\n        if (row + r0 + u < R) {\n";
            for (int i : full_leaves)
                if (!is_colvec(i)) {
                    row_pointer((size_t)i, "r0 + u", "          ");
                    emit_leaf_load(ss, P.arrays[i], i, rp.VEC, "x" + std::to_string(i) + "u[u]", "          ", rp.nt_loads, rp.ragged, "w");
                }
            ss << "        }\n      }\n";
            ss << "      _Pragma(\"unroll\") for (int u = 0; u < " << U << "; ++u) {\n      const int rr = r0 + u;\n      if (row + rr >= R) break;\n";
            for (size_t i = 0; i < P.arrays.size(); ++i) {
                const ArrayArg& a = P.arrays[i];
                const std::string t = ctype(a.buf->dtype);
                if (a.cls == Cls::FULL && a.is_dest)
                    row_pointer(i, "rr", "      ");
                else if (a.cls == Cls::ROW && !a.is_dest)
                    ss << "      const " << t << " rl" << i << " = ((const " << t << "*)A.p[" << i << "])[(row + rr)" << (a.strided ? " * (long)A.iv[" + std::to_string(L.stride_pos[i]) + "]" : std::string()) << "];\n";
            }
            for (int i : full_leaves)
                if (!is_colvec(i)) ss << "      const " << ctype(P.arrays[i].buf->dtype) << "* x" << i << " = x" << i << "u[u];\n";
            BodyEmitter be(P, rp, true, rpn.n_phases, &rpn.first_body);
            std::vector<int> again;
            be.band_divisors = &again;
            be.band_invariant = invariant;
            be.div_mode = div_mode;
            std::ostringstream pre, body, post;
            for (const Output& o : rpn.outputs) {
                const ArrayArg& d = P.arrays[o.array];
                const std::string t = ctype(d.buf->dtype), ov = "o" + std::to_string(o.array), w = "w" + std::to_string(o.array);
                const std::string ldf = rp.ragged ? "dali_loadu<" : "dali_load<";
                const std::string stf = rp.ragged ? (rp.nt_stores ? "dali_storeu_nt<" : "dali_storeu<") : (rp.nt_stores ? "dali_store_nt<" : "dali_store<");
                pre << "      dali_vec<" << t << ", VEC> " << ov << ";\n";
                if (o.op != OPERATOR_T_EQL) pre << "      " << ov << " = " << ldf << t << ", VEC>(" << w << " + (long)ch * VEC);\n";
                post << "      " << stf << t << ", VEC>(" << w << " + (long)ch * VEC, " << ov << ");\n";
                body << "        " << ov << ".v[j] = " << op_combine(o.op, ov + ".v[j]", "(" + t + ")(" + be.value(o.root) + ")") << ";\n";
            }
            ss << pre.str() << "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n        const int col = ch * VEC + j; (void)col;\n" << be.stmts.str() << body.str()
               << "      }\n" << post.str() << "      }\n    }\n";
        };
        if (divs.empty()) {
            emit_rows(0);
        } else {
            ss << "    if (__all(hok)) {\n";
            emit_rows(1);
            ss << "    } else {\n";
            emit_rows(2);
            ss << "    }\n";
        }
        ss << "  }\n}\n";
        return ss.str();
    }

    // output body: FULL destinations
    bool any_full = false;
    for (const Output& o : rpn.outputs) any_full = any_full || o.cls == Cls::FULL;
    if (any_full) {
        auto emit_output_loop = [&](std::ostringstream& os, int div_mode, std::vector<std::string>* divisors) {
            open_loop(os);
            os << "      if (row_ok) {\n";
            BodyEmitter be(P, rp, true, rpn.n_phases, &rpn.first_body);
            be.div_mode = div_mode;
            be.divisors = divisors;
            std::ostringstream pre, body, post;
            for (const Output& o : rpn.outputs) {
                if (o.cls != Cls::FULL) continue;
                const ArrayArg& d = P.arrays[o.array];
                std::string t = ctype(d.buf->dtype);
                std::string ov = "o" + std::to_string(o.array);
                if (rp.VEC > 1 && rp.peel) {
                    pre << "        dali_vec<" << t << ", VEC> " << ov << ";\n";
                    if (o.op != OPERATOR_T_EQL) pre << "        " << ov << " = dali_load<" << t << ", VEC>(v" << o.array << " + (long)ch * VEC);\n";
                    post << "        " << (rp.nt_stores ? "dali_store_nt<" : "dali_store<") << t << ", VEC>(v" << o.array << " + (long)ch * VEC, " << ov << ");\n";
                } else if (rp.VEC > 1 && rp.ragged) {
                    pre << "        dali_vec<" << t << ", VEC> " << ov << ";\n";
                    if (o.op != OPERATOR_T_EQL) pre << "        " << ov << " = dali_loadu<" << t << ", VEC>(q" << o.array << " + (long)ch * VEC);\n";
                    post << "        " << (rp.nt_stores ? "dali_storeu_nt<" : "dali_storeu<") << t << ", VEC>(q" << o.array << " + (long)ch * VEC, " << ov << ");\n";
                } else if (rp.VEC > 1) {
                    pre << "        dali_vec<" << t << ", VEC> " << ov << ";\n";
                    if (o.op != OPERATOR_T_EQL) pre << "        " << ov << " = dali_load<" << t << ", VEC>(q" << o.array << " + (long)ch * VEC);\n";
                    post << "        " << (rp.nt_stores ? "dali_store_nt<" : "dali_store<") << t << ", VEC>(q" << o.array << " + (long)ch * VEC, " << ov << ");\n";
                } else {
                    std::string cs = d.strided ? " * cs" + std::to_string(o.array) : "";
                    pre << "        dali_vec<" << t << ", 1> " << ov << ";\n";
                    if (o.op != OPERATOR_T_EQL) pre << "        " << ov << ".v[0] = q" << o.array << "[(long)ch" << cs << "];\n";
                    post << "        q" << o.array << "[(long)ch" << cs << "] = " << ov << ".v[0];\n";
                }
                std::string v = be.value(o.root);
                body << "          " << ov << ".v[j] = " << op_combine(o.op, ov + ".v[j]", "(" + t + ")(" + v + ")") << ";\n";
            }
            os << pre.str();
            os << "        _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n          const int col = " << col_of_ch << "; (void)col;\n";
            os << be.stmts.str() << body.str();
            os << "        }\n" << post.str();
            os << "      }\n    }\n  }\n";
            if (tail) {
                open_tail(os, "tail_on && row_ok");
                os << be.stmts.str();
                for (const Output& o : rpn.outputs) {
                    if (o.cls != Cls::FULL) continue;
                    std::string t = ctype(P.arrays[o.array].buf->dtype);
                    const std::string dp = "q" + std::to_string(o.array) + "[tail_col]";
                    os << "    " << dp << " = " << op_combine(o.op, dp, "(" + t + ")(" + be.value(o.root) + ")") << ";\n";
                }
                os << "  }\n";
            }
        };
        emit_with_division_plan(ss, emit_output_loop);
    }
    // ROW / SCAL destinations: one thread per row writes
    bool any_row = false;
    for (const Output& o : rpn.outputs) any_row = any_row || (o.cls != Cls::FULL && o.total_red < 0);
    if (any_row) {
        // (pieces of rows reduced on their own: every piece writes its result, piece `seg` into element `seg` behind the row's first)
        const bool pieces = rp.split && rpn.n_phases > 0;
        const std::string slot = pieces ? "[seg]" : "[0]";
        ss << "  if (tr == 0 && row_ok" << (rp.split && !pieces ? " && seg == 0" : "") << ") {\n";
        BodyEmitter be(P, rp, false, rpn.n_phases, &rpn.first_body);
        std::ostringstream body;
        for (const Output& o : rpn.outputs) {
            if (o.cls == Cls::FULL || o.total_red >= 0) continue;
            std::string t = ctype(P.arrays[o.array].buf->dtype);
            std::string v = be.value(o.root);
            body << "    q" << o.array << slot << " = " << op_combine(o.op, "q" + std::to_string(o.array) + slot, "(" + t + ")(" + v + ")") << ";\n";
        }
        ss << be.stmts.str() << body.str() << "  }\n";
    }
    if (!totals.empty()) emit_totals_fold();
    ss << "}\n";
    return ss.str();
}

static bool vec4_ok(const Program& P, const Domain& dom) {
    if (dom.C % 4 != 0) return false;
    for (const ArrayArg& a : P.arrays) {
        if (a.gather_source || a.cls != Cls::FULL) continue;
        if (a.col_stride != 1) return false;
        if (a.row_stride % 4 != 0) return false;
        if (a.buf->offset % 4 != 0) return false;
    }
    return true;
}

// Rows of unit column stride whose length, row stride or offset is no multiple of four elements: vector accesses at
// element alignment with a partial last chunk, instead of one element per access.
static bool ragged_ok(const Program& P, const Domain& dom) {
    if (dom.C < 16) return false;
    for (const ArrayArg& a : P.arrays) {
        if (a.gather_source || a.cls != Cls::FULL) continue;
        if (a.col_stride != 1) return false;
    }
    return true;
}

// every vector-accessed array starts its rows at the same distance from a 16-byte boundary: 4-byte elements, offsets and row
// strides congruent modulo 4 (buffers themselves are 256-byte aligned); positions matter to nothing but the element values
// (no argmax / argmin, whose ties go by the order in which a thread visits its elements)
static bool peel_ok(const Program& P, const Domain& dom) {
    if (dom.C < 64) return false;
    long off = -1, rs = -1;
    for (const ArrayArg& a : P.arrays) {
        if (a.gather_source || a.cls != Cls::FULL) continue;
        if (a.col_stride != 1 || size_of_dtype(a.buf->dtype) != 4 || a.row_index >= 0) return false;
        if (!a.is_dest && a.strided && a.strides[0] == 0) continue;  // broadcast along the rows: read at element alignment
        const long o = (long)(a.buf->offset % 4), r = (long)(a.row_stride % 4);
        if (off < 0) { off = o; rs = r; }
        if (o != off || r != rs) return false;
    }
    for (const PNode& n : P.nodes)
        if (n.kind == Kind::ARG_AXIS_REDUCE || n.kind == Kind::ARG_ALL_REDUCE || n.kind == Kind::GATHER) return false;
    return off >= 0;
}

// `totals`: further requests whose destination holds one element and whose root is [scalar arithmetic over] one full
// reduction of an expression with one value per row of `dom` (the mean of the row losses next to the gradient of a
// cross-entropy). They ride along in the same launch: every workgroup publishes the combination of its rows' values,
// the workgroup that draws the last ticket folds those in workgroup order, applies the scalar arithmetic and stores.
bool try_row(const std::vector<DestSpec>& specs, const Domain& dom, const std::vector<DestSpec>* totals, int segments) {
    RowPlan rpn;
    Program& P = rpn.P;
    rpn.dom = dom;
    // destinations first (dali/array/jit/jit.cpp:1159-1164: dest, then leaves)
    std::vector<int> roots;
    for (const DestSpec& s : specs) {
        int64_t n = numel_of(s.dest.shape());
        Cls cls;
        int last = s.dest.ndim() ? s.dest.shape().back() : 1;
        if (n == dom.R * dom.C && (last == dom.C || dom.C == 1)) cls = Cls::FULL;
        else if (n == dom.R) cls = Cls::ROW;
        else return false;
        if (dom.C == 1 && n == dom.R) cls = Cls::FULL;
        int ai = add_array(P, s.dest.expression(), cls, false, dom, true);
        if (ai < 0) return false;
        Output o;
        o.array = ai;
        o.op = s.op;
        o.cls = cls;
        o.root = -1;
        rpn.outputs.push_back(o);
    }
    const size_t n_totals = totals ? totals->size() : 0;
    for (size_t k = 0; k < n_totals; ++k) {
        const DestSpec& s = (*totals)[k];
        if (numel_of(s.dest.shape()) != 1) return false;
        int ai = add_array(P, s.dest.expression(), Cls::SCAL, false, dom, true);
        if (ai < 0) return false;
        Output o;
        o.array = ai;
        o.op = s.op;
        o.cls = Cls::SCAL;
        o.root = -1;
        rpn.outputs.push_back(o);
    }
    for (size_t i = 0; i < specs.size(); ++i) {
        int r = add_node(P, specs[i].root);
        rpn.outputs[i].root = r;
        roots.push_back(r);
    }
    for (size_t k = 0; k < n_totals; ++k) {
        int r = add_node(P, (*totals)[k].root);
        rpn.outputs[specs.size() + k].root = r;
        roots.push_back(r);
    }
    for (size_t i = 0; i < specs.size(); ++i)
        if (!classify(P, roots[i], rpn.outputs[i].cls, dom)) return false;
    for (size_t k = 0; k < n_totals; ++k) {
        // the scalar arithmetic above the full reduction, then the reduced expression as one value per row
        int found = -1;
        std::function<bool(int)> cls_epi = [&](int id) -> bool {
            PNode& nd = P.nodes[id];
            if (nd.kind == Kind::ALL_REDUCE) {
                if (found >= 0 && found != id) return false;
                if (nd.cls_set && nd.cls != Cls::SCAL) return false;
                found = id;
                nd.cls = Cls::SCAL;
                nd.cls_set = true;
                if (numel_of(P.nodes[nd.args[0]].shape) != dom.R || dom.C == 1) return false;
                return classify(P, nd.args[0], Cls::ROW, dom);
            }
            if (numel_of(nd.shape) != 1) return false;
            if (nd.kind == Kind::SCALAR) { nd.cls = Cls::SCAL; nd.cls_set = true; return true; }
            if (nd.cls_set) return nd.cls == Cls::SCAL;
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
        if (!cls_epi(roots[specs.size() + k]) || found < 0) return false;
        rpn.outputs[specs.size() + k].total_red = found;
    }
    // phases
    std::vector<bool> seen(P.nodes.size(), false);
    for (int r : roots) compute_dep(P, r, seen);
    int nph = 0;
    // (the full reductions of `totals` are no phases of a row: they are folded across workgroups at the end)
    for (size_t id = 0; id < P.nodes.size(); ++id)
        if (seen[id] && is_reduce(P.nodes[id].kind) && !is_all_reduce(P.nodes[id].kind)) nph = std::max(nph, P.nodes[id].phase + 1);
    rpn.n_phases = nph;
    rpn.phase_reduces.assign(nph, {});
    for (size_t id = 0; id < P.nodes.size(); ++id)
        if (seen[id] && is_reduce(P.nodes[id].kind) && !is_all_reduce(P.nodes[id].kind)) rpn.phase_reduces[P.nodes[id].phase].push_back((int)id);
    count_uses(P, roots);

    // launch geometry
    RowParams& rp = rpn.rp;
    rp.VEC = vec4_ok(P, dom) ? 4 : 1;
    static const int ragged_env = env_int("DALI_HIP_ROW_RAGGED", 1);
    if (rp.VEC == 1 && ragged_env && ragged_ok(P, dom)) {
        rp.VEC = 4;
        rp.ragged = true;
        rp.tail = dom.C % rp.VEC != 0;
    }
    // Rows that are not aligned to the vector but all start at the same offset within 16 bytes (contiguous buffers of odd row
    // length): vectors from the row's first 16-byte boundary, from its first 128-byte boundary when the row has 8192 elements or
    // more ([2048,50257] softmax 165 -> 150 us, 163 us with 16-byte boundaries; a wave's unaligned kilobyte touches nine cache
    // lines instead of eight and writes partial lines at both ends).
    static const int peel_env = env_int("DALI_HIP_ROW_PEEL", 1);
    // Long rows whose vectors are aligned but whose length is no whole number of cache lines gain the same way from starting at
    // a 128-byte boundary ([2048,50256]: 156 -> 154 us, [2048,45000]: 142 -> 137 us).
    const bool line_rows = rp.VEC == 4 && !rp.ragged && dom.C >= 8192 && dom.C % 32 != 0;
    // (maps over many long rows as well: `tanh(x + column)` on [2000,50257])
    static const int peel_maps = env_int("DALI_HIP_ROW_PEEL_MAPS", 1);
    const bool long_rows_map = nph == 0 && peel_maps && n_totals == 0 && dom.R >= 1024 && dom.C >= 8192;
    if ((rp.ragged || line_rows) && peel_env && (nph > 0 || long_rows_map) && segments <= 1 && peel_ok(P, dom)) {
        rp.ragged = true;
        rp.peel = true;
        rp.tail = true;
    }
    int64_t CH = dom.C / rp.VEC;
    int n_full = 0, max_el = 4;
    for (const ArrayArg& a : P.arrays)
        if (!a.is_dest && a.cls == Cls::FULL && !a.gather_source) {
            n_full++;
            max_el = std::max(max_el, size_of_dtype(a.buf->dtype));
        }
    int split_S = 1;
    if (nph == 0) {
        rp.cached = false;
        rp.TPR = (int)std::min<int64_t>(256, pow2ceil((int)std::max<int64_t>(1, CH)));
        rp.BT = 256;
        // few long rows (one workgroup per row would leave most of the device idle): a row is cut into S pieces of at
        // least 1024 vectors, as many as bring the grid to about 4096 workgroups
        // operands broadcast along the rows ([1, C] against [R, C]: a bias, per-column statistics): a workgroup walks a band of
        // rows chunk by chunk and keeps those operands, and the reciprocal of a divisor made of them, in registers
        static const int band_env = env_int("DALI_HIP_ROW_BAND", 4);
        bool colvec = false, band_ok = band_env > 1 && rp.VEC == 4 && !rp.tail && rp.TPR == 256 && n_totals == 0 && dom.R >= 2 * band_env;
        for (const ArrayArg& a : P.arrays) {
            if (a.cls == Cls::FULL && !a.is_dest && a.strided && a.strides[0] == 0 && !a.gather_source) colvec = true;
            if (a.gather_source || a.row_index >= 0 || (a.cls == Cls::FULL && a.strided && a.strides[1] != 1)) band_ok = false;
        }
        for (const Output& o : rpn.outputs) band_ok = band_ok && o.cls == Cls::FULL;
        for (const PNode& nd : P.nodes) band_ok = band_ok && nd.kind != Kind::GATHER_FROM_ROWS && nd.kind != Kind::GATHER;
        if (colvec && band_ok) {
            static const int unroll_env = env_int("DALI_HIP_ROW_BAND_UNROLL", 1);
            rp.band = band_env;
            rp.band_unroll = unroll_env >= 1 && band_env % unroll_env == 0 ? unroll_env : 1;
        }
        static const int split_env = env_int("DALI_HIP_ROW_SPLIT", 1);
        if (split_env && rp.band == 0 && n_totals == 0 && rp.TPR == 256 && dom.R < 1024 && CH >= 4096) {
            while (split_S * 2 * dom.R <= 4096 && CH / (split_S * 2) >= 1024) split_S *= 2;
            rp.split = split_S > 1;
        }
    } else {
        // vectors per thread: latency-bound problems (everything in flight at once, one generation
        // of waves) want more threads per row, streaming-size problems more work per thread
        static const int chunks_env = env_int("DALI_HIP_ROW_CHUNKS", 0);
        const bool big = dom.R * dom.C * (int64_t)max_el >= ((int64_t)64 << 20);
        const int chunks_target = chunks_env > 0 ? chunks_env : (!big ? 2 : (nph >= 2 ? 8 : 4));
        static const int tpr_cap = std::max(64, env_int("DALI_HIP_ROW_TPR_MAX", 1024));
        int tpr = pow2ceil((int)std::max<int64_t>(1, (CH + chunks_target - 1) / chunks_target));
        // short rows: never fewer threads per row than the row has vectors (up to a wave), so that a wave's load is one
        // contiguous kilobyte over neighbouring rows; a thread walking several vectors of its own short row makes every
        // load touch 32 bytes of each of 32 cache lines ([1048576, 64]: 279 us against 84 us)
        // (a kernel that only writes per-row results keeps the few-threads form: its reads come through the L1 either way,
        // and it saves the shuffles: [1048576, 64] sum 41 us against 50 us)
        bool writes_rows = false;
        for (const Output& o : rpn.outputs) writes_rows = writes_rows || o.cls == Cls::FULL;
        if (writes_rows) tpr = std::max(tpr, std::min(64, pow2ceil((int)std::max<int64_t>(1, CH))));
        if (rp.tail) tpr = std::max(tpr, rp.peel ? 8 : 4);  // one thread per element outside the whole vectors
        tpr = std::min(tpr, tpr_cap);
        int64_t ept = (CH + tpr - 1) / tpr;
        // every FULL input is held in registers across the phases: bound the footprint
        rp.cached = (int64_t)std::max(1, n_full) * ept * rp.VEC * (max_el / 4) <= 64;
        if (segments > 1) {
            // pieces of rows: one phase, results per row only, streamed (a piece is read once); at least a workgroup's worth of vectors each
            // (or the two phases that one walk takes together, a maximum and the sum of the exponentials relative to it: a piece's
            // results are then those two reductions themselves, its own maximum and its sum relative to that)
            int m_id = -1, s_id = -1, x_id = -1;
            static const int online_env = env_int("DALI_HIP_ROW_ONLINE_SOFTMAX", 1);
            const bool statistics = nph == 2 && online_env && max_then_sum_of_exp(rpn, &m_id, &s_id, &x_id);
            if ((nph != 1 && !statistics) || n_totals != 0 || rp.VEC != 4 || CH / segments < 1024) return false;
            for (const Output& o : rpn.outputs)
                if (o.cls != Cls::ROW || (statistics && o.root != m_id && o.root != s_id)) return false;
            rp.cached = false;
            rp.split = true;
            split_S = segments;
        }
        if (!rp.cached) {
            tpr = 1024;
            ept = 0;
        }
        rp.TPR = tpr;
        rp.EPT = (int)ept;
        // a row wider than a wave owns its whole workgroup (the cross-wave fold is per block)
        rp.BT = tpr > 64 ? tpr : 256;
    }
    rp.RPB = rp.BT / rp.TPR;
    rp.NW = rp.TPR > 64 ? rp.TPR / 64 : 1;
    rp.exact = nph > 0 && rp.cached && !rp.peel && dom.C == (int64_t)rp.TPR * rp.EPT * rp.VEC;
    // A 1024-thread row block fills a CU by itself unless it stays within 64 VGPRs; two resident
    // blocks let one row's loads overlap another row's arithmetic.
    static const int wpe = env_int("DALI_HIP_ROW_WAVES_PER_EU", -1);
    // 1024-thread workgroups: two per CU (8 waves per SIMD, 64 registers per thread) as long as the cached row fits that
    // budget; beyond ~44 cached values per thread the register cap would spill, so one workgroup per CU with twice the
    // registers ([2048,50257] 362 -> 200 us, [1024,65536] 169 -> 115 us; [8192,32000] stays at two)
    int64_t cached_values = rp.cached ? (int64_t)std::max(1, n_full) * rp.EPT * rp.VEC * (max_el / 4) : 0;
    // ... unless the vectors beyond 40 registers' worth fit 64 KiB of LDS: then two workgroups per CU remain possible and
    // one row's exponentials overlap the other's loads
    static const int hybrid_env = env_int("DALI_HIP_ROW_LDS_CACHE", 1);
    // (measured on softmax: [2048,50257] 201 -> 178 us, [2048,45000] 187 -> 155 us, [2048,38000] 134 -> 124 us; 32 values
    // in registers where the rest fits the LDS budget, 36 otherwise; more than 36 spilled under the 64-register cap)
    if (hybrid_env && rp.cached && nph > 0 && rp.BT == 1024 && rp.TPR == 1024 && cached_values > 32 && max_el == 4 && rp.VEC == 4 && n_full >= 1) {
        for (int regs : {32, 36}) {
            const int ept_r = regs / (n_full * rp.VEC);
            const int ept_l = rp.EPT - ept_r;
            if (ept_r >= 1 && ept_l >= 1 && (int64_t)n_full * ept_l * 1024 * rp.VEC * 4 <= (64 << 10)) {
                rp.EPT_L = ept_l;
                cached_values = (int64_t)n_full * ept_r * rp.VEC;
                break;
            }
        }
    }
    rp.waves_per_eu = nph > 0 ? (wpe >= 0 ? wpe : (rp.BT == 1024 ? (cached_values > 44 ? 4 : 8) : 0)) : 0;

    // cross-phase register caching of expensive shared values
    rpn.first_body.assign(P.nodes.size(), -1);
    if (rp.cached && nph > 0) {
        // body roots: phase p -> args of its reduces; output body -> FULL output roots
        std::vector<std::vector<int>> body_roots(nph + 1);
        for (int p = 0; p < nph; ++p)
            for (int id : rpn.phase_reduces[p]) body_roots[p].push_back(P.nodes[id].args[0]);
        for (const Output& o : rpn.outputs)
            if (o.cls == Cls::FULL) body_roots[nph].push_back(o.root);
        int budget = 64 / (max_el / 4) - n_full * rp.EPT * rp.VEC;
        for (int id = (int)P.nodes.size() - 1; id >= 0; --id) {
            PNode& n = P.nodes[id];
            if (n.kind != Kind::ELEMENTWISE || n.cls != Cls::FULL || !contains_expensive(P, id)) continue;
            int bodies = 0, first = -1;
            for (int b = 0; b <= nph; ++b) {
                std::set<int> reach;
                for (int r : body_roots[b]) {
                    if (r == id) reach.insert(id);
                    body_nodes(P, r, reach, true);
                }
                if (reach.count(id)) {
                    bodies++;
                    if (first < 0) first = b;
                }
            }
            if (bodies >= 2 && rp.EPT * rp.VEC * (size_of_dtype(n.dtype) / 4) <= budget) {
                n.kept = true;
                rpn.first_body[id] = first;
                budget -= rp.EPT * rp.VEC * (size_of_dtype(n.dtype) / 4);
            }
        }
    }

    // kernel identity
    std::ostringstream params;
    // Streaming policy: outputs of a kernel that reduces over its rows leave with non-temporal stores (C1 4.6 against
    // 5.9 us, cross-entropy [8192, 32000] 357 against 383 us), outputs of a plain map with ordinary stores (x + bias on
    // [8192, 8192]: 0.88 against 0.72 of the HBM peak); inputs bypass cache allocation once the operands are too large
    // to be found in a cache again (64 MiB).
    static const int nt_l = env_int("DALI_HIP_ROW_NT_LOADS", -1), nt_s = env_int("DALI_HIP_ROW_NT_STORES", -1);
    rp.nt_loads = nt_l >= 0 ? nt_l != 0 : dom.R * dom.C * (int64_t)max_el >= ((int64_t)64 << 20);
    rp.nt_stores = nt_s >= 0 ? nt_s != 0 : rpn.n_phases > 0;
    params << rp.VEC << "," << rp.TPR << "," << rp.EPT << "," << rp.BT << "," << rp.cached << "," << rp.waves_per_eu << ","
           << rp.nt_loads << rp.nt_stores << rp.exact << rp.ragged << rp.tail << rp.peel << "," << rp.EPT_L << (rp.split ? "S" : "") << (!rp.cached && env_int("DALI_HIP_ROW_ONLINE_SOFTMAX", 1) == 0 ? "w" : "") << (rp.band > 1 ? "B" + std::to_string(rp.band) + "u" + std::to_string(rp.band_unroll) : std::string());
    if (n_totals) {
        // one 8-byte slot per workgroup and total in the workspace's 32 MiB of partial results
        const int64_t blocks = (dom.R + rp.RPB - 1) / rp.RPB;
        if (blocks * (int64_t)n_totals * 8 > ((int64_t)32 << 20) || blocks > 2147483647LL) return false;
        params << ",T" << n_totals;
    }
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    std::string sig = signature(P, rpn.outputs);
    uint64_t h = kernel_hash("row", sig, params.str());
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    std::vector<int> shape_ndims = {rp.band > 1 ? 4 : (rp.split ? 3 : 2)};
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = nph == 0 ? "map2d" : "row";
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = rp.BT;
        K->plan.grid_kind = DALI_HIP_GRID_ROWS;
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = rp.split || rp.band > 1 ? 2 : 1;  // split: the grid covers S * R; bands: strips * bands
        K->plan.work_per_block = rp.RPB;
        K->plan.max_blocks = 0;
    }
    std::vector<std::vector<int>> shapes = {{(int)dom.R, (int)dom.C}};
    if (rp.split) shapes[0].insert(shapes[0].begin(), split_S);
    if (rp.band > 1) shapes[0] = {(int)((CH + rp.TPR - 1) / rp.TPR), (int)((dom.R + rp.band - 1) / rp.band), (int)dom.R, (int)dom.C};
    load_and_launch(*K, [&]() { return gen_row_kernel(rpn, L, K->name); }, P, shapes);
    return true;
}

}  // namespace jit

}  // namespace dali
