// Pieces of source text shared by the kernel generators: the argument block of a kernel, the per-row pointer prologue,
// vector loads of a leaf and the combination of a value with its destination (the reference's operator_to_name,
// dali/array/jit/jit.cpp:1144-1160).
#include "jit_internal.h"

namespace dali {
namespace jit {

IvLayout layout_iv(const Program& P, const std::vector<int>& shape_ndims) {
    IvLayout L;
    for (const ArrayArg& a : P.arrays) {
        L.size_pos.push_back(L.total);
        L.total += a.nd;
        if (a.strided) {
            L.stride_pos.push_back(L.total);
            L.total += a.nd;
        } else {
            L.stride_pos.push_back(-1);
        }
    }
    for (int nd : shape_ndims) {
        L.shape_pos.push_back(L.total);
        L.total += nd;
    }
    return L;
}

// The argument block of a generated kernel. The launcher lays it out as one struct (include/dali_hip.h), the kernel
// declares the same bytes as separate parameters: gfx950 preloads the leading parameters of a kernel into scalar
// registers while the wave is being launched (hipRTC runs with amdgpu-kernarg-preload-count), so a wave can form its
// first addresses without waiting for a load of its own arguments. For a kernel that lasts a few microseconds that load
// is 5 to 7% of the launch ([4096,1024] softmax 5.83 -> 5.43 us). DALI_KERNEL_ARGS puts the parameters back into the
// struct the bodies are written against; every index into it is a constant, so it never leaves the registers.
std::string kargs_struct(const Program& P, const IvLayout& L) {
    std::ostringstream ss;
    const int na = (int)P.arrays.size(), ns = std::max<int>(1, (int)P.scalars.size()), ni = std::max(1, L.total);
    ss << "struct KArgs { void* ws; void* p[" << na << "]; dali_slot s[" << ns << "]; int iv[" << ni << "]; };\n";
    ss << "#define DALI_KERNEL_PARAMS void* a_ws";
    for (int i = 0; i < na; ++i) ss << ", void* a_p" << i;
    for (int i = 0; i < ns; ++i) ss << ", unsigned long long a_s" << i;  // a plain integer: aggregates are not preloaded
    for (int i = 0; i < ni; ++i) ss << ", int a_iv" << i;
    ss << "\n#define DALI_KERNEL_ARGS KArgs A; A.ws = a_ws;";
    for (int i = 0; i < na; ++i) ss << " A.p[" << i << "] = a_p" << i << ";";
    for (int i = 0; i < ns; ++i) ss << " A.s[" << i << "] = __builtin_bit_cast(dali_slot, a_s" << i << ");";
    for (int i = 0; i < ni; ++i) ss << " A.iv[" << i << "] = a_iv" << i << ";";
    ss << "\n";
    return ss.str();
}

int env_int(const char* name, int fallback) {
    const char* v = getenv(name);
    return (v && *v) ? atoi(v) : fallback;
}

std::string op_combine(OPERATOR_T op, const std::string& dst, const std::string& val) {
    switch (op) {
        case OPERATOR_T_EQL: return val;
        case OPERATOR_T_ADD: return "(" + dst + " + " + val + ")";
        case OPERATOR_T_SUB: return "(" + dst + " - " + val + ")";
        case OPERATOR_T_MUL: return "(" + dst + " * " + val + ")";
        default: return "(" + dst + " / " + val + ")";
    }
}

bool expensive_functor(const std::string& name) {
    static const char* names[] = {"functor::exp", "functor::log", "functor::tanh", "functor::sigmoid", "functor::power",
                                  "functor::softplus", "functor::softplus_backward", "functor::negative_log",
                                  "functor::safe_entropy_log", "functor::inverse_tanh", "functor::steep_sigmoid",
                                  "functor::eltdiv", "functor::sqrt_f", "functor::rsqrt", "functor::inv",
                                  "functor::binary_cross_entropy", "functor::log_or_zero", "functor::div_grad"};
    for (const char* n : names)
        if (name == n) return true;
    return false;
}

// Declarations of row pointers and per-row values shared by the row and flat templates.
void emit_row_prologue(std::ostringstream& ss, const Program& P, const IvLayout& L) {
    // per-row and scalar input values first: a gathered source's row pointer needs its index value
    for (size_t i = 0; i < P.arrays.size(); ++i) {
        const ArrayArg& a = P.arrays[i];
        std::string t = ctype(a.buf->dtype);
        if (a.gather_source || a.is_dest) continue;
        if (a.cls == Cls::ROW) {
            std::string s = a.strided ? " * (long)A.iv[" + std::to_string(L.stride_pos[i]) + "]" : "";
            ss << "  const " << t << " rl" << i << " = ((const " << t << "*)A.p[" << i << "])[row" << s << "];\n";
        } else if (a.cls == Cls::SCAL) {
            ss << "  const " << t << " sl" << i << " = ((const " << t << "*)A.p[" << i << "])[0];\n";
        }
    }
    for (size_t i = 0; i < P.arrays.size(); ++i) {
        const ArrayArg& a = P.arrays[i];
        std::string t = ctype(a.buf->dtype);
        if (a.gather_source) {
            if (a.strided)
                ss << "  const long g_rs" << i << " = A.iv[" << L.stride_pos[i] << "], g_cs" << i << " = A.iv[" << L.stride_pos[i] + 1 << "];\n";
            else
                ss << "  const long g_rs" << i << " = A.iv[" << L.size_pos[i] + 1 << "], g_cs" << i << " = 1;\n";
            ss << "  const int g_n" << i << " = A.iv[" << L.size_pos[i] + 1 << "]; (void)g_n" << i << ";  // columns of the source: a pick outside them reads the nearest one\n";
        } else if (a.cls == Cls::FULL) {
            std::string rs = a.strided ? "(long)A.iv[" + std::to_string(L.stride_pos[i]) + "]" : "C";
            // a gathered source: the row comes from the index value, held inside the source (the reference reads out of bounds)
            std::string r = a.row_index >= 0 ? "(long)dali_clamp_index(rl" + std::to_string(a.row_index) + ", A.iv[" + std::to_string(L.size_pos[i]) + "])"
                                             : std::string("row");
            ss << "  " << (a.is_dest ? "" : "const ") << t << "* q" << i << " = (" << (a.is_dest ? "" : "const ") << t << "*)A.p[" << i << "] + " << r << " * " << rs << ";\n";
            if (a.strided) ss << "  const long cs" << i << " = A.iv[" << L.stride_pos[i] + 1 << "];\n";
        } else if (a.cls == Cls::ROW) {
            std::string s = a.strided ? " * (long)A.iv[" + std::to_string(L.stride_pos[i]) + "]" : "";
            if (a.is_dest) ss << "  " << t << "* q" << i << " = (" << t << "*)A.p[" << i << "] + row" << s << ";\n";
        } else {
            if (a.is_dest) ss << "  " << t << "* q" << i << " = (" << t << "*)A.p[" << i << "];\n";
        }
    }
}

// load of FULL leaf `i` for chunk `ch` into dst (dst is "x<i>[e]" or "x<i>")
void emit_leaf_load(std::ostringstream& ss, const ArrayArg& a, int i, int VEC, const std::string& dst, const std::string& indent, bool nontemporal,
                    bool ragged, const std::string& pointer_prefix) {
    std::string t = ctype(a.buf->dtype);
    const std::string q = pointer_prefix + std::to_string(i);  // q<i>, or another name where a workgroup walks several rows
    if (VEC > 1 && ragged) {
        ss << indent << "{ const dali_vec<" << t << ", " << VEC << "> tmp = " << (nontemporal ? "dali_loadu_nt<" : "dali_loadu<") << t << ", " << VEC << ">(" << q
           << " + (long)ch * " << VEC << ");\n";
        ss << indent << "  _Pragma(\"unroll\") for (int j = 0; j < " << VEC << "; ++j) " << dst << "[j] = tmp.v[j]; }\n";
    } else if (VEC > 1) {
        ss << indent << "{ dali_vec<" << t << ", " << VEC << "> tmp = " << (nontemporal ? "dali_load_nt<" : "dali_load<") << t << ", " << VEC << ">(" << q
           << " + (long)ch * " << VEC << ");\n";
        ss << indent << "  _Pragma(\"unroll\") for (int j = 0; j < " << VEC << "; ++j) " << dst << "[j] = tmp.v[j]; }\n";
    } else {
        std::string cs = a.strided ? " * cs" + std::to_string(i) : "";
        ss << indent << dst << "[0] = " << q << "[(long)ch" << cs << "];\n";
    }
}

}  // namespace jit

}  // namespace dali
