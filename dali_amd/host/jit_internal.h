// Internal interface of the fused-expression path (planner, program builder, kernel generators, launch): shared by
// the jit_*.cpp files of this directory and by nothing else.
#ifndef DALI_AMD_JIT_INTERNAL_H
#define DALI_AMD_JIT_INTERNAL_H
#include <algorithm>
#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <set>
#include <sstream>
#include <unordered_map>

#include "../../include/dali_hip.h"
#include "expr.h"

namespace dali {

// evaluation switches and the launch recording (jit_launch.cpp)
extern bool g_dry_run;
extern bool g_dry_compile;
extern std::vector<std::string>* g_dry_sources;
extern std::string g_last_source;
extern std::vector<std::function<void()>>* g_recording;
extern std::vector<std::shared_ptr<memory::SynchronizedMemory>>* g_recording_written;
void note_recorded_write(const std::shared_ptr<memory::SynchronizedMemory>& m);

namespace jit {

extern const char* const kCodegenVersion;
// the device support code that precedes every generated kernel (device_prelude.h)
const char* device_prelude();

inline bool is_reduce(Kind k) { return k == Kind::AXIS_REDUCE || k == Kind::ARG_AXIS_REDUCE; }

inline bool is_all_reduce(Kind k) { return k == Kind::ALL_REDUCE || k == Kind::ARG_ALL_REDUCE; }

inline std::vector<int> strides_of(const Expr* b) { return b->strides.empty() ? contiguous_strides(b->shape) : b->strides; }

inline std::string ctype(DType t) { return dtype_to_cpp_name(t); }

inline std::string reducer_struct(const std::string& name) { return name; }  // "reducers::sum" etc. exist in the prelude

// boost-style combine of the reference (dali/utils/hash_utils.h:12-23)
struct Hasher {
    uint64_t value_ = 0;
    template <typename T>
    Hasher& add(const T& element) {
        value_ ^= std::hash<T>()(element) + 0x9e3779b9 + (value_ << 6) + (value_ >> 2);
        return *this;
    }
    uint64_t value() const { return value_; }
};

enum class Cls { FULL, ROW, SCAL };

struct PNode {
    Kind kind;
    DType dtype;
    std::string name;
    std::vector<int> args;
    std::vector<int> shape;
    int array = -1;   // BUFFER: index into Program::arrays
    int scalar = -1;  // SCALAR: index into Program::scalars
    int axis = 0, depth = 0;
    Cls cls = Cls::FULL;
    bool cls_set = false;
    int phase = -1;  // reduce nodes: the phase that computes them
    int dep = 0;     // number of reduce phases that must have finished before this node can be evaluated
    int uses = 0;
    bool kept = false;  // cached in registers across phases
    std::shared_ptr<Expr> src;
};

// how one buffer is presented to the kernel
struct ArrayArg {
    std::shared_ptr<Expr> buf;
    Cls cls = Cls::FULL;
    bool gather_source = false;
    bool is_dest = false;
    int nd = 1;
    bool strided = false;
    std::vector<int> sizes, strides;
    int64_t row_stride = 0, col_stride = 1;
    int row_index = -1;  // FULL presentation of a gather source: array whose per-row value picks the source row
};

struct ScalarArg {
    DType dtype;
    double d;
    float f;
    int i;
    const Expr* src = nullptr;  // the literal's node (the plan cache refills the value from it)
};

struct Program {
    std::vector<PNode> nodes;
    std::vector<ArrayArg> arrays;
    std::vector<ScalarArg> scalars;
    std::map<const Expr*, int> memo;
    std::map<std::string, int> structural;
};

struct Domain {
    int64_t R = 1, C = 1;
    bool flat = false;  // 1-D domain over contiguous operands of any shape
};

struct KernelSpec {
    uint64_t hash = 0;
    std::string name;
    std::string kind;
    std::string source;  // generated lazily
    dali_hip_launch_plan plan;
    std::vector<int32_t> array_ndim, array_strided, array_elsize, scalar_dtype, shape_ndim;
};

// iv layout bookkeeping: position of sizes / strides of each array and of each shape
struct IvLayout {
    std::vector<int> size_pos, stride_pos, shape_pos;
    int total = 0;
};

struct RowParams {
    int VEC = 1, TPR = 64, EPT = 0, BT = 256, RPB = 4, NW = 1;
    int waves_per_eu = 0;  // occupancy hint (0 = compiler default)
    bool cached = true;
    bool nt_loads = false;   // inputs are streamed once: bypass cache allocation
    bool nt_stores = true;   // outputs are not re-read by this kernel: streaming stores
    bool exact = false;      // register-cached rows: C == TPR * EPT * VEC, the chunk guards fall away
    bool ragged = false;     // rows not aligned to the vector: element-aligned vector accesses
    bool tail = false;       // ragged, and C is no multiple of VEC: the rest of a row is handled one element to a thread
    bool peel = false;       // ragged rows that all start at the same offset within 16 bytes: the vectors begin at the first aligned
                             // element of the row, the 0..3 elements in front of it go with the rest behind the last vector
    int EPT_L = 0;           // cached rows: the last EPT_L of the EPT vectors a thread holds live in LDS instead of registers
    bool split = false;      // maps without a reduction over few long rows: every row is cut into S pieces, one workgroup each
    int band_unroll = 1;     // rows of a band whose loads are issued together
    int band = 0;            // maps with operands broadcast along the rows ([1, C]): a workgroup walks `band` rows and keeps those operands
};

// Emits C++ expressions for program nodes inside one loop body, declaring shared
// values once per body.
struct BodyEmitter {
    const Program& P;
    const RowParams& rp;
    std::ostringstream stmts;
    std::set<int> declared;
    bool per_element;  // false: row context (no column variable)
    std::string leaf_suffix;  // "[e][j]" (cached) or "[j]" (streaming)
    int body_index;  // phase number, or number of phases for the output body
    const std::vector<int>* first_body;  // per node: first body that evaluates a kept node
    // Divisions by a row constant: the generator hoists one reciprocal and one range test per divisor out of
    // the element loop and emits the loop twice, `div_mode` 1 with product + FMA correction, 2 with the plain
    // quotient; 0 keeps the self-contained per-element form. `divisors` collects the divisor expressions.
    int div_mode = 0;
    std::vector<std::string>* divisors = nullptr;
    // Band kernels (several rows per workgroup): a divisor that only depends on operands broadcast along the rows is
    // evaluated once per column chunk into hv<k>[j] with its reciprocal hr<k>[j], ahead of the loop over the rows.
    std::vector<int>* band_divisors = nullptr;
    std::function<bool(int)> band_invariant;
    int divisor_index(const std::string& dv) {
        for (size_t k = 0; k < divisors->size(); ++k)
            if ((*divisors)[k] == dv) return (int)k;
        divisors->push_back(dv);
        return (int)divisors->size() - 1;
    }
    static bool simple_token(const std::string& s) {
        if (s.empty()) return false;
        for (char c : s)
            if (!(isalnum((unsigned char)c) || c == '_' || c == '.' || c == '[' || c == ']')) return false;
        return true;
    }

    BodyEmitter(const Program& P_, const RowParams& rp_, bool per_el, int body, const std::vector<int>* fb)
        : P(P_), rp(rp_), per_element(per_el), body_index(body), first_body(fb) {
        leaf_suffix = rp.cached ? (rp.EPT_L > 0 ? "(e, j)" : "[e][j]") : "[j]";
    }

    // true when the node's value is the same for every element of a row (seen through broadcasts)
    bool row_invariant(int id) const {
        const PNode* n = &P.nodes[id];
        while (n->kind == Kind::BROADCAST || n->kind == Kind::EXPAND_DIMS) n = &P.nodes[n->args[0]];
        return n->kind == Kind::SCALAR || (n->cls_set && n->cls != Cls::FULL);
    }

    std::string scalar_ref(const PNode& n) {
        const char* field = n.dtype == DTYPE_FLOAT ? "f" : (n.dtype == DTYPE_DOUBLE ? "d" : "i");
        return "A.s[" + std::to_string(n.scalar) + "]." + field;
    }

    std::string raw(int id) {
        const PNode& n = P.nodes[id];
        switch (n.kind) {
            case Kind::SCALAR:
                return scalar_ref(n);
            case Kind::BUFFER: {
                const ArrayArg& a = P.arrays[n.array];
                if (a.cls == Cls::FULL) return "x" + std::to_string(n.array) + leaf_suffix;
                if (a.cls == Cls::ROW) return "rl" + std::to_string(n.array);
                return "sl" + std::to_string(n.array);
            }
            case Kind::AXIS_REDUCE:
            case Kind::ARG_AXIS_REDUCE:
            case Kind::ALL_REDUCE:
            case Kind::ARG_ALL_REDUCE:
                return "red" + std::to_string(id);
            case Kind::EXPAND_DIMS:
            case Kind::BROADCAST:
                return value(n.args[0]);
            case Kind::ELEMENTWISE: {
                if (band_divisors && n.name == "functor::eltdiv" && n.cls == Cls::FULL && n.args.size() == 2 && n.dtype == DTYPE_FLOAT &&
                    P.nodes[n.args[1]].dtype == DTYPE_FLOAT && band_invariant(n.args[1])) {
                    size_t k = 0;
                    while (k < band_divisors->size() && (*band_divisors)[k] != n.args[1]) ++k;
                    if (k == band_divisors->size()) band_divisors->push_back(n.args[1]);
                    const std::string x = value(n.args[0]), ks = std::to_string(k);
                    if (div_mode == 1) return "dali_div_fast(" + x + ", hv" + ks + "[j], hr" + ks + "[j])";
                    return "(" + x + " / hv" + ks + "[j])";
                }
                if (n.name == "functor::eltdiv" && n.cls == Cls::FULL && n.args.size() == 2 && row_invariant(n.args[1])) {
                    // divisor constant along the row: reciprocal once, product + correction per element
                    const std::string x = value(n.args[0]), dv = value(n.args[1]);
                    if (divisors && n.dtype == DTYPE_FLOAT && P.nodes[n.args[1]].dtype == DTYPE_FLOAT && simple_token(dv)) {
                        const int k = divisor_index(dv);
                        if (div_mode == 1) return "dali_div_fast(" + x + ", " + dv + ", dr" + std::to_string(k) + ")";
                        if (div_mode == 2) return "(" + x + " / " + dv + ")";
                    }
                    return "dali_div_invariant(" + x + ", " + dv + ")";
                }
                std::string s = n.name + "<" + ctype(n.dtype) + ">::Map(";
                for (size_t i = 0; i < n.args.size(); ++i) s += (i ? ", " : "") + value(n.args[i]);
                return s + ")";
            }
            case Kind::GATHER_FROM_ROWS: {
                const ArrayArg& a = P.arrays[n.array];
                std::string t = ctype(n.dtype);
                (void)a;
                return "((const " + t + "*)A.p[" + std::to_string(n.array) + "])[row * g_rs" + std::to_string(n.array) + " + (long)dali_clamp_index(" +
                       value(n.args[1]) + ", g_n" + std::to_string(n.array) + ") * g_cs" + std::to_string(n.array) + "]";
            }
            case Kind::GATHER:
                return "x" + std::to_string(n.array) + leaf_suffix;
            case Kind::ONE_HOT:
                return "dali_one_hot<" + ctype(n.dtype) + ">(" + value(n.args[2]) + ", col, (" + ctype(n.dtype) + ")" + value(n.args[0]) +
                       ", (" + ctype(n.dtype) + ")" + value(n.args[1]) + ")";
            default:
                throw std::runtime_error("internal: node kind not emittable in a fused kernel");
        }
    }

    std::string value(int id) {
        const PNode& n = P.nodes[id];
        bool shareable = n.kind == Kind::ELEMENTWISE || n.kind == Kind::GATHER_FROM_ROWS || n.kind == Kind::ONE_HOT;
        if (!shareable) return raw(id);
        std::string var = "n" + std::to_string(id);
        if (n.kept && rp.cached && per_element) {
            if (declared.count(id)) return var;
            declared.insert(id);
            const std::string slot = "t" + std::to_string(id) + "[e][j]";
            if ((*first_body)[id] == body_index) {
                const std::string r = raw(id);  // may itself append statements (nested kept or shared nodes): before ours
                stmts << "const " << ctype(n.dtype) << " " << var << " = " << r << "; " << slot << " = " << var << ";\n";
            } else {
                stmts << "const " << ctype(n.dtype) << " " << var << " = " << slot << ";\n";
            }
            return var;
        }
        if (n.uses < 2) return raw(id);
        if (declared.count(id)) return var;
        std::string r = raw(id);
        declared.insert(id);
        stmts << "const " << ctype(n.dtype) << " " << var << " = " << r << ";\n";
        return var;
    }
};

struct Output {
    int root;        // program node
    int array;       // dest array index
    OPERATOR_T op;
    Cls cls;
    // row kernel only: the destination is one value for the whole launch, root = [scalar arithmetic over] a full
    // reduction (this node) of a value the kernel holds per row (the mean of the row losses of a cross-entropy)
    int total_red = -1;
};

struct RowPlan {
    Program P;
    Domain dom;
    std::vector<Output> outputs;
    int n_phases = 0;
    std::vector<std::vector<int>> phase_reduces;
    RowParams rp;
    std::vector<int> first_body;
};

struct LoadedKernel {
    uint64_t hash;
    std::string kind;
};

struct Launch {
    KernelSpec* K;
};

// Ensure the module for K is loaded (generating source through `gen` on a miss) and launch it.
// What the outermost planning call launched, for the plan cache: filled by load_and_launch.
struct LaunchCapture {
    int launches = 0;
    KernelSpec* K = nullptr;
    std::vector<ArrayArg> arrays;
    std::vector<ScalarArg> scalars;
    std::vector<std::vector<int>> shapes;
};

struct DestSpec {
    Array dest;
    OPERATOR_T op;
    Array root;
};

// im2col, col2im and the pooling pair (dali/array/op/im2col.cpp, col2im.cpp, conv.cpp:12-212) are index remaps
// bound by memory traffic. Images are dense arrays whose dimensions come in the order of the data format's
// letters; the kernels take extents and element strides as (N, C, H, W), so one source serves every layout.
// At streaming rates a vector instruction slot is worth a few bytes, so index arithmetic is kept off the
// per-element path: it is 32-bit, divisions by extents go through multipliers computed here on the host
// (dali_udiv), per-patch and per-row parts are computed once per wave or workgroup, and layouts whose channels
// are contiguous move four channels per thread.
struct ImageGeom {
    int ext[4];     // N, C, H, W
    int stride[4];  // element strides of a dense array in data_format order, as (N, C, H, W)
};

// Named integers of a kernel's geometry; a divisor brings its multiplier and shift along (see dali_udiv).
struct GeomInts {
    std::vector<std::string> names;
    std::vector<int> values;
    void add(const std::string& name, int v) {
        names.push_back(name);
        values.push_back(v);
    }
    void add_div(const std::string& name, int d) {
        DALI_ASSERT(d >= 1, make_message("internal: divisor ", name, " must be positive (got ", d, ")"));
        int sft = 0;
        while (((int64_t)1 << sft) < d) ++sft;
        const uint64_t m = (((uint64_t)1 << (31 + sft)) + (uint64_t)d - 1) / (uint64_t)d;
        add(name, d);
        add(name + "_M", (int)(uint32_t)m);
        add(name + "_S", sft);
    }
    void add_image(const ImageGeom& g) {
        const char* ext[4] = {"N", "C", "H", "W"};
        const char* str[4] = {"SN", "SC", "SH", "SW"};
        for (int k = 0; k < 4; ++k) add_div(ext[k], g.ext[k]);
        for (int k = 0; k < 4; ++k) add(str[k], g.stride[k]);
    }
};

extern LaunchCapture* g_capture;
extern bool g_capture_compare_only;

// Memo of a graph rewrite, keyed by node identity. It keeps every node it has seen alive: a rewrite may release nodes
// (evaluating an operand in place replaces its node by a buffer), and a node created later at the address of a released
// one would otherwise meet the released node's entry and be replaced by something unrelated.
struct ExprMemo {
    std::map<const Expr*, std::pair<std::shared_ptr<Expr>, Array>> entries;
    const Array* find(const std::shared_ptr<Expr>& e) const {
        auto it = entries.find(e.get());
        return it == entries.end() ? nullptr : &it->second.second;
    }
    void put(const std::shared_ptr<Expr>& e, const Array& out) { entries[e.get()] = std::make_pair(e, out); }
};


// jit_launch.cpp
uint64_t kernel_hash(const std::string& kind, const std::string& sig, const std::string& params);
std::string kernel_name(const std::string& kind, uint64_t hash);
void load_and_launch(KernelSpec& K, const std::function<std::string()>& gen, const Program& P,
                     const std::vector<std::vector<int>>& shapes);

// jit_program.cpp
int64_t numel_of(const std::vector<int>& shape);
std::string array_key(const Expr* b, Cls cls, bool gather);
int add_node(Program& P, const Array& a);
bool collapse_dims(const std::vector<int>& shape, const std::vector<int>& st, int upto, int64_t* stride);
int add_array(Program& P, const std::shared_ptr<Expr>& b, Cls cls, bool gather, const Domain& dom, bool is_dest);
bool classify(Program& P, int id, Cls want, const Domain& dom);
void compute_dep(Program& P, int id, std::vector<bool>& seen);
void body_nodes(const Program& P, int id, std::set<int>& out, bool top);
bool contains_expensive(const Program& P, int id);
void count_uses(Program& P, const std::vector<int>& roots);
int pow2ceil(int v);
std::string signature(const Program& P, const std::vector<Output>& outs);
void fill_plan_arrays(KernelSpec& K, const Program& P, const std::vector<int>& shape_ndims);

// jit_emit.cpp
IvLayout layout_iv(const Program& P, const std::vector<int>& shape_ndims);
std::string kargs_struct(const Program& P, const IvLayout& L);
int env_int(const char* name, int fallback);
std::string op_combine(OPERATOR_T op, const std::string& dst, const std::string& val);
bool expensive_functor(const std::string& name);
void emit_row_prologue(std::ostringstream& ss, const Program& P, const IvLayout& L);
void emit_leaf_load(std::ostringstream& ss, const ArrayArg& a, int i, int VEC, const std::string& dst, const std::string& indent, bool nontemporal,
                    bool ragged = false, const std::string& pointer_prefix = "q");

// jit_row.cpp
// `segments` > 1: the requests are reductions along the rows with one result per row and nothing else; every row is cut into
// that many pieces, each piece goes to a workgroup of its own, and a destination (a view of `dom.R` elements whose stride is
// `segments`: one column of an [R, segments] buffer) receives the pieces' results side by side, for the caller to reduce again.
bool try_row(const std::vector<DestSpec>& specs, const Domain& dom, const std::vector<DestSpec>* totals = nullptr, int segments = 0);

// jit_flat.cpp
bool flat_eligible(const Array& a, int64_t n, std::set<const Expr*>& seen);
bool try_flat(const std::vector<DestSpec>& specs);

// jit_all.cpp
bool has_kind(const Array& a, const std::function<bool(Kind)>& pred, std::set<const Expr*>& seen);
bool has_kind(const Array& a, const std::function<bool(Kind)>& pred);
void find_all_reduces(const Array& a, std::vector<Array>& out, std::set<const Expr*>& seen);
bool try_all(const DestSpec& spec);

// jit_col.cpp
bool col_kept_vector(const std::vector<int>& s, const std::vector<int>& shape);
int col_split_of(const Array& arg);
bool try_col(const DestSpec& spec);

// jit_generic.cpp
bool try_generic(const std::vector<DestSpec>& specs);

// jit_gemm.cpp
void run_gemm(const Array& dst, const Expr* mm, const Expr* mm2, float beta);

// jit_planner.cpp
Array materialize(const Array& a);
Array clean(const Array& a, ExprMemo& memo, bool is_root);
void run_specs_planned(std::vector<DestSpec> specs);

// jit_plan_cache.cpp
void run_specs(std::vector<DestSpec> specs);

// jit_scatter.cpp
ArrayArg manual_arg(const Array& buf, Cls cls, bool is_dest, int nd, const std::vector<int>& sizes, const std::vector<int>& strides);
void scatter_assign(const Array& dest, OPERATOR_T op, const Array& source);

// jit_scan.cpp
Array run_scan(const Array& arg_in, const std::string& reducer, bool inclusive);
Array run_circular_convolution(const Array& x_in, const Array& w_in);

// jit_spatial.cpp
Array dense_buffer(const Array& a);
std::string divmod(const std::string& q, const std::string& r, const std::string& n, const std::string& D);
void launch_special(const char* kind, const std::string& sig, const Program& P, int64_t blocks, const GeomInts& G,
                    const std::function<void(std::ostringstream&)>& body);
Array run_im2col(const Expr& e, const Array& image_in);
Array run_col2im(const Expr& e, const Array& patches_in);
Array run_pool2d(const Expr& e, const Array& x_in);
Array run_pool2d_backward(const Expr& e, const Array& y_in, const Array& dy_in, const Array& x_in);

// jit_transpose.cpp
bool is_transposed_matrix(const Expr* e);
void run_transpose_into(const Array& dest, const Array& src);
bool try_transposed_map(const DestSpec& sp);

// jit_fill.cpp
Array run_fill(const std::shared_ptr<Expr>& e);

}  // namespace jit
}  // namespace dali
#endif
