// Maps whose operands are transposed matrices: tiles go through LDS so that both the reads and the writes are
// coalesced.
#include "jit_internal.h"

namespace dali {
namespace jit {

// A 2-D view whose first index runs along memory (strides [1, ld]: the transpose of a row-major matrix) and that is
// large enough for the layout to matter.
bool is_transposed_matrix(const Expr* e) {
    if (e->kind != Kind::BUFFER || e->shape.size() != 2 || e->strides.size() != 2) return false;
    return e->strides[0] == 1 && e->strides[1] >= e->shape[0] && e->shape[0] >= 32 && e->shape[1] >= 32 && (int64_t)e->shape[0] * e->shape[1] >= (1 << 16);
}

// dest (contiguous [R, C]) = src (a transposed matrix view [R, C]): 64x64 tiles go through LDS, read along the source's
// memory rows and written along the destination's.
void run_transpose_into(const Array& dest, const Array& src) {
    if (try_transposed_map({dest, OPERATOR_T_EQL, op::identity(src)})) return;
    auto se = src.expression();
    const int R = se->shape[0], Cn = se->shape[1], ld = se->strides[1];
    Program P;
    P.arrays.push_back(manual_arg(dest, Cls::FULL, true, 1, {R * Cn}, {}));
    P.arrays.push_back(manual_arg(src, Cls::FULL, false, 2, {R, Cn}, {1, ld}));
    GeomInts G;
    G.add("R", R);
    G.add("CN", Cn);
    G.add("LD", ld);
    G.add_div("TILES_R", (R + 63) / 64);
    const int64_t tiles = (int64_t)((R + 63) / 64) * ((Cn + 63) / 64);
    std::ostringstream sig;
    sig << "transpose|" << (int)se->dtype;
    launch_special("transpose", sig.str(), P, tiles, G, [&](std::ostringstream& ss) {
        ss << "  __shared__ T tile[64][65];\n";
        ss << "  T* out = (T*)A.p[0];\n  const T* in = (const T*)A.p[1];\n";
        ss << "  const unsigned total = (unsigned)TILES_R * (unsigned)((CN + 63) / 64);\n";
        ss << "  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;\n";
        ss << "  for (unsigned b = blockIdx.x; b < total; b += gridDim.x) {\n";
        ss << "    " << divmod("tc", "tr", "b", "TILES_R") << "\n";
        ss << "    const int r0 = tr * 64, c0 = (int)tc * 64;\n";
        ss << "    // the source's memory rows are the view's columns: element (r, c) lives at c * LD + r\n";
        ss << "    _Pragma(\"unroll\") for (int k = 0; k < 16; ++k) {\n      const int c = c0 + ty + 4 * k, r = r0 + tx;\n";
        ss << "      if (c < CN && r < R) tile[ty + 4 * k][tx] = in[(long)c * LD + r];\n    }\n";
        ss << "    __syncthreads();\n";
        ss << "    _Pragma(\"unroll\") for (int k = 0; k < 16; ++k) {\n      const int r = r0 + ty + 4 * k, c = c0 + tx;\n";
        ss << "      if (r < R && c < CN) out[(long)r * CN + c] = tile[tx][ty + 4 * k];\n    }\n";
        ss << "    __syncthreads();\n  }\n}\n";
    });
}

// dest (contiguous [R, C]) op= f(operands), the operands being contiguous [R, C] matrices, transposed views of [C, R]
// matrices, single elements and literals: one launch. The 64x64 tiles of the transposed operands come through LDS (read
// along their memory rows), the other operands and the destination are walked along theirs; writing the transposed
// operands out first costs a read and a write of each more (x.T + 1 on [16384,4096]: 211 us in two launches).
bool try_transposed_map(const DestSpec& sp) {
    if (sp.dest.ndim() != 2 || !sp.dest.is_buffer() || !sp.dest.contiguous_memory() || sp.root.shape() != sp.dest.shape()) return false;
    const std::vector<int> shape = sp.dest.shape();
    const int R = shape[0], Cn = shape[1];
    if ((int64_t)R * Cn >= ((int64_t)1 << 31) || R < 1 || Cn < 1) return false;
    Program P;
    P.arrays.push_back(manual_arg(sp.dest, Cls::FULL, true, 1, {R * Cn}, {}));
    const int root = add_node(P, sp.root);
    std::vector<int> transposed;
    size_t lds_bytes = 0;
    std::function<bool(int)> cls = [&](int id) -> bool {
        PNode& nd = P.nodes[id];
        if (nd.cls_set) return true;
        nd.cls_set = true;
        switch (nd.kind) {
            case Kind::SCALAR: nd.cls = Cls::SCAL; return true;
            case Kind::BUFFER: {
                ArrayArg a;
                a.buf = nd.src;
                if (numel_of(nd.shape) == 1) {
                    a.cls = Cls::SCAL;
                    a.nd = 1;
                    a.sizes = {1};
                    nd.cls = Cls::SCAL;
                } else {
                    if (nd.shape != shape || nd.src->memory.get() == sp.dest.expression()->memory.get()) return false;
                    a.cls = Cls::FULL;
                    nd.cls = Cls::FULL;
                    if (is_transposed_matrix(nd.src.get())) {
                        a.nd = 2;
                        a.sizes = {R, Cn};
                        a.strided = true;
                        a.strides = {1, nd.src->strides[1]};
                        a.row_stride = 1;
                        a.col_stride = nd.src->strides[1];
                    } else if (Array(nd.src).contiguous_memory()) {
                        a.nd = 1;
                        a.sizes = {R * Cn};
                    } else {
                        return false;
                    }
                }
                std::string key = array_key(nd.src.get(), a.cls, false);
                for (size_t i = 1; i < P.arrays.size(); ++i)
                    if (array_key(P.arrays[i].buf.get(), P.arrays[i].cls, false) == key) {
                        P.nodes[id].array = (int)i;
                        return true;
                    }
                P.arrays.push_back(a);
                P.nodes[id].array = (int)P.arrays.size() - 1;
                if (a.strided) {
                    transposed.push_back((int)P.arrays.size() - 1);
                    lds_bytes += (size_t)64 * 65 * size_of_dtype(nd.src->dtype);
                }
                return true;
            }
            case Kind::ELEMENTWISE:
            case Kind::BROADCAST:
            case Kind::EXPAND_DIMS: {
                if (nd.kind != Kind::ELEMENTWISE && numel_of(nd.shape) != 1 && numel_of(P.nodes[nd.args[0]].shape) != 1) return false;
                if (nd.kind == Kind::ELEMENTWISE && numel_of(nd.shape) != 1 && nd.shape != shape) return false;
                nd.cls = numel_of(nd.shape) == 1 ? Cls::SCAL : Cls::FULL;
                std::vector<int> args = nd.args;
                for (int a : args)
                    if (!cls(a)) return false;
                return true;
            }
            default: return false;
        }
    };
    if (!cls(root) || transposed.empty() || lds_bytes > (48 << 10)) return false;
    count_uses(P, {root});
    std::vector<Output> outs(1);
    outs[0].root = root;
    outs[0].array = 0;
    outs[0].op = sp.op;
    outs[0].cls = Cls::FULL;
    GeomInts G;
    G.add("R", R);
    G.add("CN", Cn);
    G.add_div("TILES_R", (R + 63) / 64);
    G.add_div("TILES_C", (Cn + 63) / 64);
    // consecutive workgroups take tiles along the rows of the destination (and of the operands that lie like it): measured
    // better than along its columns when such an operand is read beside the transposed one (x.T * y: 186 -> 163 us)
    static const int order_env = env_int("DALI_HIP_TMAP_ORDER", 1);
    for (int i : transposed) G.add("LD" + std::to_string(i), (int)P.arrays[i].col_stride);
    const int64_t tiles = (int64_t)((R + 63) / 64) * ((Cn + 63) / 64);
    // four-byte elements and extents in whole vectors: 16-byte global accesses on both sides (at element alignment),
    // single LDS words in between (a row pitch of 65 words spreads both the row-wise writes and the column-wise reads
    // over the banks)
    bool vec = R % 4 == 0 && Cn % 4 == 0;
    for (const ArrayArg& a : P.arrays) vec = vec && (a.cls != Cls::FULL || size_of_dtype(a.buf->dtype) == 4);
    std::ostringstream sig;
    sig << "tmap|" << (int)sp.op << "|" << vec << "|" << order_env << "|" << signature(P, outs);
    launch_special("tmap", sig.str(), P, tiles, G, [&](std::ostringstream& ss) {
        RowParams rp;
        rp.cached = false;
        rp.VEC = vec ? 4 : 1;
        for (int i : transposed) ss << "  __shared__ " << ctype(P.arrays[i].buf->dtype) << " tile" << i << "[64][65];\n";
        ss << "  T* out = (T*)A.p[0];\n";
        for (size_t i = 1; i < P.arrays.size(); ++i) {
            const std::string t = ctype(P.arrays[i].buf->dtype);
            if (P.arrays[i].cls == Cls::SCAL) ss << "  const " << t << " sl" << i << " = ((const " << t << "*)A.p[" << i << "])[0];\n";
            else ss << "  const " << t << "* in" << i << " = (const " << t << "*)A.p[" << i << "];\n";
        }
        ss << "  const unsigned total = (unsigned)TILES_R * (unsigned)((CN + 63) / 64);\n";
        std::vector<int> first_body(P.nodes.size(), -1);
        BodyEmitter be(P, rp, true, 0, &first_body);
        const std::string v = be.value(root);
        if (vec) {
            ss << "  constexpr int VEC = 4;\n  const int t16 = threadIdx.x & 15, t4 = (threadIdx.x >> 4) * 1;\n";
            ss << "  for (unsigned b = blockIdx.x; b < total; b += gridDim.x) {\n";
            ss << "    " << (order_env == 1 ? divmod("tr_", "tc_", "b", "TILES_C") + " const int tr = (int)tr_; const unsigned tc = (unsigned)tc_;" : divmod("tc", "tr", "b", "TILES_R")) << "\n";
            ss << "    const int r0 = tr * 64, c0 = (int)tc * 64;\n";
            ss << "    // a transposed operand's memory rows are the view's columns: element (r, c) lives at c * LD + r\n";
            ss << "    _Pragma(\"unroll\") for (int k = 0; k < 4; ++k) {\n      const int lc = t4 + 16 * k, lr = t16 * 4, c = c0 + lc, r = r0 + lr;\n      if (c < CN && r < R) {\n";
            for (int i : transposed) {
                const std::string t = ctype(P.arrays[i].buf->dtype);
                ss << "        { const dali_vec<" << t << ", 4> g = dali_loadu<" << t << ", 4>(in" << i << " + (long)c * LD" << i << " + r);\n";
                ss << "          _Pragma(\"unroll\") for (int j = 0; j < 4; ++j) tile" << i << "[lc][lr + j] = g.v[j]; }\n";
            }
            ss << "      }\n    }\n    __syncthreads();\n";
            ss << "    _Pragma(\"unroll\") for (int k = 0; k < 4; ++k) {\n      const int lr = t4 + 16 * k, lc = t16 * 4, r = r0 + lr, c = c0 + lc;\n      if (r < R && c < CN) {\n";
            ss << "        const long o = (long)r * CN + c, row = r; (void)row;\n";
            for (size_t i = 1; i < P.arrays.size(); ++i) {
                if (P.arrays[i].cls != Cls::FULL) continue;
                const std::string t = ctype(P.arrays[i].buf->dtype);
                if (P.arrays[i].strided)
                    ss << "        " << t << " x" << i << "[4];\n        _Pragma(\"unroll\") for (int j = 0; j < 4; ++j) x" << i << "[j] = tile" << i << "[lc + j][lr];\n";
                else
                    ss << "        const dali_vec<" << t << ", 4> xv" << i << " = dali_loadu<" << t << ", 4>(in" << i << " + o);\n        const " << t << "* x" << i << " = xv" << i
                       << ".v;\n";
            }
            ss << "        dali_vec<T, 4> ov;\n";
            if (sp.op != OPERATOR_T_EQL) ss << "        ov = dali_loadu<T, 4>(out + o);\n";
            ss << "        _Pragma(\"unroll\") for (int j = 0; j < 4; ++j) {\n          const int col = c + j; (void)col;\n";
            ss << be.stmts.str() << "          ov.v[j] = " << op_combine(sp.op, "ov.v[j]", "(T)(" + v + ")") << ";\n        }\n";
            ss << "        dali_storeu<T, 4>(out + o, ov);\n      }\n    }\n";
            ss << "    __syncthreads();\n  }\n}\n";
            return;
        }
        ss << "  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;\n";
        ss << "  for (unsigned b = blockIdx.x; b < total; b += gridDim.x) {\n";
        ss << "    " << (order_env == 1 ? divmod("tr_", "tc_", "b", "TILES_C") + " const int tr = (int)tr_; const unsigned tc = (unsigned)tc_;" : divmod("tc", "tr", "b", "TILES_R")) << "\n";
        ss << "    const int r0 = tr * 64, c0 = (int)tc * 64;\n";
        ss << "    // a transposed operand's memory rows are the view's columns: element (r, c) lives at c * LD + r\n";
        ss << "    _Pragma(\"unroll\") for (int k = 0; k < 16; ++k) {\n      const int c = c0 + ty + 4 * k, r = r0 + tx;\n      if (c < CN && r < R) {\n";
        for (int i : transposed) ss << "        tile" << i << "[ty + 4 * k][tx] = in" << i << "[(long)c * LD" << i << " + r];\n";
        ss << "      }\n    }\n    __syncthreads();\n";
        ss << "    _Pragma(\"unroll\") for (int k = 0; k < 16; ++k) {\n      const int r = r0 + ty + 4 * k, c = c0 + tx;\n      if (r < R && c < CN) {\n";
        ss << "        const long o = (long)r * CN + c, row = r; (void)row;\n        constexpr int j = 0; (void)j;\n        const int col = c; (void)col;\n";
        for (size_t i = 1; i < P.arrays.size(); ++i) {
            if (P.arrays[i].cls != Cls::FULL) continue;
            const std::string t = ctype(P.arrays[i].buf->dtype);
            if (P.arrays[i].strided) ss << "        const " << t << " x" << i << "[1] = { tile" << i << "[tx][ty + 4 * k] };\n";
            else ss << "        const " << t << " x" << i << "[1] = { in" << i << "[o] };\n";
        }
        ss << be.stmts.str() << "        out[o] = " << op_combine(sp.op, "out[o]", "(T)(" + v + ")") << ";\n      }\n    }\n";
        ss << "    __syncthreads();\n  }\n}\n";
    });
    return true;
}

}  // namespace jit

}  // namespace dali
