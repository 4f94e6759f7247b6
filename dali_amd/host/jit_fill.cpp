// Index-valued fills (arange, eye, diag and the like): the value of an element is a function of its position.
#include "jit_internal.h"

namespace dali {
namespace jit {

// arange (dali/array/op/arange.cpp:8-39: start + offset * step, in the operands' own arithmetic) and diag / eye
// (dali/array/op/eye.cpp:29-36: the diagonal value where row == column, else 0) as one thread per element.
Array run_fill(const std::shared_ptr<Expr>& e) {
    Array dest(e->shape, e->dtype);
    const int64_t n = numel_of(e->shape);
    if (n == 0) return dest;
    std::string t = ctype(e->dtype);
    Program P;
    P.arrays.push_back(manual_arg(dest, Cls::FULL, true, 1, {(int)n}, {}));
    std::ostringstream sig, body;
    std::vector<int> shape_ndims = {2};
    std::vector<std::vector<int>> shapes;
    if (e->kind == Kind::ARANGE) {
        for (int k = 0; k < 2; ++k) {
            auto se = e->args[k].expression();
            DALI_ASSERT(se->kind == Kind::SCALAR, "arange takes scalar constants for start and step");
            ScalarArg sa;
            sa.dtype = se->dtype;
            sa.d = se->dvalue;
            sa.f = (float)se->dvalue;
            sa.i = se->ivalue;
            P.scalars.push_back(sa);
        }
        auto field = [&](int k) { return std::string("A.s[") + std::to_string(k) + "]." + (P.scalars[k].dtype == DTYPE_FLOAT ? "f" : (P.scalars[k].dtype == DTYPE_DOUBLE ? "d" : "i")); };
        body << "    out[i] = (T)(" << field(0) << " + (int)i * " << field(1) << ");\n";
        sig << "arange|" << (int)e->dtype << "|" << (int)P.scalars[0].dtype << "|" << (int)P.scalars[1].dtype;
        shapes = {{(int)n, 1}};
    } else {
        Array d = e->args[0];
        const bool scalar_diag = numel_of(d.shape()) == 1;
        if (d.expression()->kind == Kind::SCALAR) {
            // a constant on the diagonal travels as a kernel scalar
            auto se = d.expression();
            ScalarArg sa;
            sa.dtype = se->dtype;
            sa.d = se->dvalue;
            sa.f = (float)se->dvalue;
            sa.i = se->ivalue;
            P.scalars.push_back(sa);
            body << "    const long r = i / cols, c = i % cols;\n    out[i] = r == c ? (T)A.s[0]." << (sa.dtype == DTYPE_FLOAT ? "f" : (sa.dtype == DTYPE_DOUBLE ? "d" : "i"))
                 << " : (T)0;\n";
            sig << "diagc|" << (int)e->dtype << "|" << (int)sa.dtype;
        } else {
            if (!d.is_buffer()) d = materialize(d);
            if (d.dtype() != e->dtype) d = materialize(op::astype(d, e->dtype));
            if (!d.contiguous_memory()) d = d.ascontiguousarray();
            P.arrays.push_back(manual_arg(d, scalar_diag ? Cls::SCAL : Cls::ROW, false, 1, {(int)numel_of(d.shape())}, {}));
            body << "    const long r = i / cols, c = i % cols;\n    out[i] = r == c ? ((const T*)A.p[1])[" << (scalar_diag ? "0" : "c") << "] : (T)0;\n";
            sig << "diag|" << (int)e->dtype << "|" << scalar_diag;
        }
        shapes = {{e->shape[0], e->shape[1]}};
    }
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash("fill", sig.str(), "");
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = "fill";
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = 256;
        K->plan.grid_kind = DALI_HIP_GRID_ELEMS;
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = 2;
        K->plan.work_per_block = 256;
        K->plan.max_blocks = 65536;
    }
    load_and_launch(*K, [&]() {
        std::ostringstream ss;
        ss << device_prelude() << kargs_struct(P, L);
        ss << "extern \"C\" __global__ __launch_bounds__(256) void " << K->name << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n  typedef " << t << " T;\n";
        ss << "  const long rows = A.iv[" << L.shape_pos[0] << "], cols = A.iv[" << L.shape_pos[0] + 1 << "]; (void)rows;\n";
        ss << "  T* out = (T*)A.p[0];\n  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < rows * cols; i += (long)gridDim.x * 256) {\n";
        ss << body.str() << "  }\n}\n";
        return ss.str();
    }, P, shapes);
    return dest;
}

}  // namespace jit

}  // namespace dali
