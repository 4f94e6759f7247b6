// Planner and evaluation driver of the fused-expression path: the counterpart of the reference's JITRunner /
// JITRunnerImpl::run (dali/array/jit/jit.cpp:552-587,1144-1225), redesigned for CDNA4.
//
// Where the reference emits one generic "sequence of assignments" template and leaves the loop structure to the host
// compiler, a GPU needs the reduction structure known up front. A fused subgraph is therefore classified into one of
// four kernel shapes over a collapsed 2-D index domain [R, C]:
//   flat  contiguous elementwise map, 128-bit loads/stores, one tile per block          (jit_flat.cpp)
//   row   reductions over the trailing axis with keepdims broadcast back onto the row,
//         also the strided / broadcasting 2-D elementwise map                            (jit_row.cpp)
//   col   reduction over the leading axis of a row-major matrix, coalesced along the
//         kept axis, two-stage through the library workspace                             (jit_col.cpp)
//   all   full reduction, two-stage through the workspace, optional scalar epilogue      (jit_all.cpp)
// Anything else is split: inner reductions, matrix products and gathers from computed sources are evaluated into
// temporaries first (clean), and what remains is tried against the shapes in turn (run_specs_planned).
#include "jit_internal.h"

namespace dali {
namespace jit {

static Array rebuild(const std::shared_ptr<Expr>& e, const std::vector<Array>& args) {
    // a unit axis inserted into a buffer is a view of that buffer (an evaluated keepdims reduction reads like any other
    // [.., 1, ..] operand)
    if (e->kind == Kind::EXPAND_DIMS && args.size() == 1 && args[0].is_buffer()) return args[0].expand_dims(e->axis);
    auto n = std::make_shared<Expr>(*e);
    n->args = args;
    return Array(n);
}

Array materialize(const Array& a) {
    Array t = a;
    evaluate({t});
    return t;
}

static bool is_plain_matmul(const Array& a) { return a.expression()->kind == Kind::MATMUL; }

// Replace everything a fused kernel cannot contain by evaluated buffers:
// MatMul nodes (and the accumulating pair X.W + H.U), inner full reductions,
// gather sources that are not buffers.
// op::softmax arrives as one node and is written out here. The general form is the reference's expression
// (dali/array/op/softmax.cpp:5-8), which the row kernel fuses into one pass. Two shapes starve that kernel and get their
// statistics (maximum and sum of exponentials per slice) from a pass of their own; what is returned is then the lazy map
// exp(x - maximum) / sum over evaluated buffers, which still fuses with whatever consumes the softmax:
//  - few long rows (one workgroup per row leaves most of the device idle): the rows are read as S times as many shorter
//    ones, each yields its own (maximum, sum), and a small second kernel combines the S pairs of a row;
//  - an axis other than the last (the slices run against memory): when a strip of the reduced axis fits one workgroup's
//    registers (extent up to 2048) the softmax is computed in one pass by a kernel of the library and arrives as a
//    buffer; otherwise the column kernel carries (maximum, sum) pairs, so the data is read once for both instead of once
//    for the maxima and once more for the sums.
// set while a softmax over few long rows evaluates its statistics: try_segmented_reduce then cuts rows into pieces at any size
static bool g_segment_whatever_the_size = false;

static Domain domain_of(const std::vector<int>& shape);

// Maximum M and sum L of exp(x - M) of every row (x's last axis) for rows that are few for their length, where one workgroup
// per row would stream each row through a single compute unit: the rows are cut into pieces that fill the device, and the
// pieces' results are merged by a small second launch. M and L come back evaluated, as [rows, 1]; x comes back as the
// contiguous buffer they were taken from. False (and nothing done) for any other shape.
static bool softmax_statistics_in_pieces(Array* xp, Array* Mp, Array* Lp) {
    static const bool staged_off = env_int("DALI_HIP_SOFTMAX_STAGED", 1) == 0;
    Array& x = *xp;
    const std::vector<int> shape = x.shape();
    if (staged_off || x.dtype() != DTYPE_FLOAT || shape.empty()) return false;
    const int64_t n = numel_of(shape), Cx = shape.back();
    if (n <= 0 || Cx <= 1) return false;
    const int64_t rows = n / Cx;
    auto merged = [&](const Array& m2, const Array& l2) {
        Array M = op::max(m2, {-1}, true);
        Array L = op::sum(op::eltmul(l2, op::exp(op::subtract(m2, M))), {-1}, true);
        evaluate({M, L});
        *Mp = M;
        *Lp = L;
    };
    int S = 1;
    while (rows < 256 && Cx >= 65536 && S * 2 * rows <= 2048 && Cx % (S * 2 * 4) == 0 && Cx / (S * 2) >= 8192) S *= 2;
    if (S >= 4) {
        if (!x.is_buffer()) x = materialize(x);
        if (!x.contiguous_memory()) x = x.ascontiguousarray();
        Array xr = x.reshape({(int)(rows * S), (int)(Cx / S)});
        Array mseg = op::max(xr, {-1}, true);
        Array lseg = op::sum(op::exp(op::subtract(xr, mseg)), {-1}, true);
        evaluate({mseg, lseg});
        merged(mseg.reshape({(int)rows, S}), lseg.reshape({(int)rows, S}));
        return true;
    }
    // the same rows at a length that does not divide that way: the row kernel cuts them into pieces itself (see
    // try_segmented_reduce)
    static const bool pieces_off = env_int("DALI_HIP_SEGMENTED_REDUCE", 1) == 0;
    // (against one launch whose workgroups walk their rows three times: worth it for rows that are few for their
    // length, [2,100003] 22.5 -> 11.1 us, [32,131073] 29.9 -> 14.7 us, but not [64,65537], 13.5 us in one launch; and whenever
    // the rows together are more than the caches keep between the passes)
    const bool few_for_their_length = (double)rows < 75.0 - 3.75e6 / (double)Cx;
    if (pieces_off || !(rows < 256 && Cx >= 65536 && rows * 8 <= 2048 && Cx / 8 >= 8192 && (n * 4 >= ((int64_t)64 << 20) || few_for_their_length)))
        return false;
    if (!x.is_buffer()) x = materialize(x);
    if (!x.contiguous_memory()) x = x.ascontiguousarray();
    Array x2 = x.reshape({(int)rows, (int)Cx});
    // Every piece's maximum and its sum of exponentials relative to that maximum from ONE walk over the rows, then the
    // merge as for equal pieces: two launches and the rows read once ([7,9999999] softmax: 185 -> 152 us). The row kernel
    // says whether it takes the pair.
    static const bool one_walk = env_int("DALI_HIP_ROW_ONLINE_SOFTMAX", 1) != 0;
    int Sp = 1;
    while (Sp * 2 * rows <= 2048 && Cx / (Sp * 2) >= 8192) Sp *= 2;
    if (one_walk && Sp >= 4) {
        Array mx = op::max(x2, {-1}, false);
        Array sm = op::sum(op::exp(op::subtract(x2, mx.expand_dims(1))), {-1}, false);
        Array mseg({(int)rows, Sp}, DTYPE_FLOAT), lseg({(int)rows, Sp}, DTYPE_FLOAT);
        if (try_row({{mseg.pluck_axis(1, 0), OPERATOR_T_EQL, mx}, {lseg.pluck_axis(1, 0), OPERATOR_T_EQL, sm}}, domain_of(x2.shape()), nullptr, Sp)) {
            jit_stats().evals++;
            merged(mseg, lseg);
            return true;
        }
    }
    // otherwise the maxima in pieces, then the sums of the exponentials in pieces (two launches each)
    g_segment_whatever_the_size = true;  // (the rule of the softmax has been applied; the reductions have another)
    try {
        Array M = op::max(x2, {-1}, false);
        evaluate({M});
        Array L = op::sum(op::exp(op::subtract(x2, M.reshape({(int)rows, 1}))), {-1}, false);
        evaluate({L});
        g_segment_whatever_the_size = false;
        *Mp = M.reshape({(int)rows, 1});
        *Lp = L.reshape({(int)rows, 1});
        return true;
    } catch (...) {
        g_segment_whatever_the_size = false;
        throw;
    }
}

static Array expand_softmax(Array x, int axis) {
    static const bool staged_off = env_int("DALI_HIP_SOFTMAX_STAGED", 1) == 0;
    const std::vector<int> shape = x.shape();
    const int nd = (int)shape.size();
    const int64_t n = numel_of(shape), Cx = shape[axis];
    std::vector<int> keep = shape;
    keep[axis] = 1;
    if (!staged_off && x.dtype() == DTYPE_FLOAT && n > 0 && Cx > 1) {
        if (axis == nd - 1) {
            Array M, L;
            if (softmax_statistics_in_pieces(&x, &M, &L)) return op::eltdiv(op::exp(op::subtract(x, M.reshape(keep))), L.reshape(keep));
        } else if (n >= (1 << 16)) {
            int64_t inner = 1, outer = 1;
            for (int d = axis + 1; d < nd; ++d) inner *= shape[d];
            for (int d = 0; d < axis; ++d) outer *= shape[d];
            // a reduced axis short enough for a strip of it to live in one workgroup's registers: one pass, read once and
            // written once ([256,512,512] along axis 1: 142 -> 88 us, 0.76 of the HBM peak)
            static const bool narrow_off = env_int("DALI_HIP_NARROW_MAP", 1) == 0;
            if (!narrow_off && !g_dry_run && nd == 2 && axis == 0 && shape[1] >= 2 && shape[1] <= 48 && n >= (1 << 20)) {
                // along the leading axis of a tall narrow matrix: a strip of 256 columns holds a few ([9999999,7]: 1408 us). Column
                // maxima and column sums go through the grouped forms of such matrices, the exponentials are written out once.
                if (!x.is_buffer()) x = materialize(x);
                if (!x.contiguous_memory()) x = x.ascontiguousarray();
                Array M = op::max(x, {0}, true);
                evaluate({M});
                Array E = materialize(op::exp(op::subtract(x, M)));
                Array L = op::sum(E, {0}, true);
                evaluate({L});
                return op::eltdiv(E, L);
            }
            static const bool one_pass_off = env_int("DALI_HIP_SOFTMAX_AXIS", 1) == 0;
            if (!one_pass_off && !g_dry_run && dali_hip_softmax_axis_supported(outer, (int)Cx, inner)) {
                if (!x.is_buffer()) x = materialize(x);
                if (!x.contiguous_memory()) x = x.ascontiguousarray();
                if (x.offset() % 4 == 0) {
                    Array out(shape, DTYPE_FLOAT);
                    softmax_axis_launch(x, out, outer, (int)Cx, inner);
                    jit_stats().evals++;
                    return out;
                }
            }
            if (inner >= 16) {
                if (!x.is_buffer()) x = materialize(x);
                if (!x.contiguous_memory()) x = x.ascontiguousarray();
                std::vector<int> order, kept_shape;
                for (int d = 0; d < nd; ++d)
                    if (d != axis) { order.push_back(d); kept_shape.push_back(shape[d]); }
                order.push_back(axis);
                auto node = std::make_shared<Expr>();
                node->kind = Kind::AXIS_REDUCE;
                node->name = "reducers::maxsumexp";
                node->args = {x.transpose(order)};
                node->shape = kept_shape;
                node->dtype = DTYPE_FLOAT;
                std::vector<int> stats_shape = kept_shape;
                stats_shape.insert(stats_shape.begin(), 2);
                Array stats(stats_shape, DTYPE_FLOAT);
                if (try_col({stats, OPERATOR_T_EQL, Array(node)})) {
                    jit_stats().evals++;
                    return op::eltdiv(op::exp(op::subtract(x, stats[0].reshape(keep))), stats[1].reshape(keep));
                }
            }
        }
    }
    return op::softmax_naive(x, axis);
}

Array clean(const Array& a, ExprMemo& memo, bool is_root) {
    auto e = a.expression();
    if (const Array* known = memo.find(e)) return *known;
    Array out = a;
    switch (e->kind) {
        case Kind::BUFFER:
        case Kind::SCALAR:
            break;
        case Kind::MATMUL: {
            Array dst(e->shape, e->dtype);
            run_gemm(dst, e.get(), nullptr, 0.0f);
            out = dst;
            break;
        }
        case Kind::ALL_REDUCE:
        case Kind::ARG_ALL_REDUCE: {
            Array arg = clean(e->args[0], memo, false);
            // An argument that holds reductions of its own is evaluated first. Under a root the planner decides: such a
            // full reduction may join the row kernel of the roots evaluated with it, or is split off there.
            if (!is_root && has_kind(arg, [](Kind k) { return is_reduce(k); })) arg = materialize(arg);
            if (arg.expression().get() != e->args[0].expression().get()) out = rebuild(e, {arg});
            break;
        }
        case Kind::ELEMENTWISE: {
            if (e->name == "functor::add" && e->args.size() == 2 && is_plain_matmul(e->args[0]) && is_plain_matmul(e->args[1]) &&
                (e->dtype == DTYPE_FLOAT || e->dtype == DTYPE_DOUBLE) && e->args[0].shape() == e->args[1].shape()) {
                Array dst(e->shape, e->dtype);
                run_gemm(dst, e->args[0].expression().get(), e->args[1].expression().get(), 0.0f);
                out = dst;
                break;
            }
            std::vector<Array> args;
            bool changed = false;
            for (const Array& x : e->args) {
                Array c = clean(x, memo, is_root && x.shape() == e->shape);
                changed = changed || c.expression().get() != x.expression().get();
                args.push_back(c);
            }
            if (changed) out = rebuild(e, args);
            break;
        }
        case Kind::SOFTMAX:
            out = clean(expand_softmax(clean(e->args[0], memo, false), e->axis), memo, is_root);
            break;
        case Kind::AXIS_SCAN: {
            // not chainable (dali/array/op/scan.cpp:38-40): the scan is its own kernel, consumers read its buffer
            Array arg = clean(e->args[0], memo, false);
            out = run_scan(arg, e->name, e->depth != 0);
            break;
        }
        case Kind::ARANGE:
        case Kind::DIAG:
            out = run_fill(e);
            break;
        case Kind::CIRCULAR_CONV: {
            Array x = clean(e->args[0], memo, false), w = clean(e->args[1], memo, false);
            out = run_circular_convolution(x, w);
            break;
        }
        case Kind::IM2COL:
            out = run_im2col(*e, clean(e->args[0], memo, false));
            break;
        case Kind::COL2IM:
            out = run_col2im(*e, clean(e->args[0], memo, false));
            break;
        case Kind::POOL2D:
            out = run_pool2d(*e, clean(e->args[0], memo, false));
            break;
        case Kind::POOL2D_BACKWARD:
            out = run_pool2d_backward(*e, clean(e->args[0], memo, false), clean(e->args[1], memo, false), clean(e->args[2], memo, false));
            break;
        case Kind::GATHER: {
            // source and index are presented as buffers; the gather itself stays lazy only where the row
            // kernel can read through it: a [N, D] node that is the root or sits under same-shape
            // elementwise nodes of the root. Everything else is evaluated through the [N, D] form.
            Array src = clean(e->args[0], memo, false);
            if (src.expression()->kind != Kind::BUFFER) src = materialize(src);
            Array idx = clean(e->args[1], memo, false);
            if (idx.expression()->kind != Kind::BUFFER) idx = materialize(idx);
            const int n_idx = numel_of(idx.shape()), d2 = src.shape()[1];
            const bool two_d = e->shape.size() == 2 && e->shape[0] == n_idx && e->shape[1] == d2;
            if (is_root && two_d) {
                out = rebuild(e, {src, idx});
            } else {
                auto n2 = std::make_shared<Expr>(*e);
                n2->args = {src, idx};
                n2->shape = {n_idx, d2};
                Array g2(n2);
                evaluate({g2});
                out = g2.reshape(e->shape);
            }
            break;
        }
        case Kind::GATHER_FROM_ROWS: {
            Array src = clean(e->args[0], memo, false);
            if (src.expression()->kind != Kind::BUFFER) src = materialize(src);
            Array idx = clean(e->args[1], memo, false);
            if (idx.ndim() == 0) idx = materialize(idx).reshape({1});
            out = rebuild(e, {src, idx});
            break;
        }
        default: {
            std::vector<Array> args;
            bool changed = false;
            for (const Array& x : e->args) {
                Array c = clean(x, memo, false);
                changed = changed || c.expression().get() != x.expression().get();
                args.push_back(c);
            }
            if (changed) out = rebuild(e, args);
            break;
        }
    }
    memo.put(e, out);
    return out;
}

// first reduce node whose argument holds no further reduce
static bool find_innermost_reduce(const Array& a, Array* found, std::set<const Expr*>& seen) {
    auto e = a.expression();
    if (seen.count(e.get())) return false;
    seen.insert(e.get());
    for (const Array& x : e->args)
        if (find_innermost_reduce(x, found, seen)) return true;
    if (is_reduce(e->kind)) {
        *found = a;
        return true;
    }
    return false;
}

static bool find_first_reduce(const Array& a, Array* found, std::set<const Expr*>& seen) {
    auto e = a.expression();
    if (seen.count(e.get())) return false;
    seen.insert(e.get());
    if (is_reduce(e->kind)) {
        *found = a;
        return true;
    }
    for (const Array& x : e->args)
        if (find_first_reduce(x, found, seen)) return true;
    return false;
}

static Array substitute(const Array& a, const Expr* target, const Array& with, ExprMemo& memo) {
    auto e = a.expression();
    if (e.get() == target) return with;
    if (const Array* known = memo.find(e)) return *known;
    std::vector<Array> args;
    bool changed = false;
    for (const Array& x : e->args) {
        Array c = substitute(x, target, with, memo);
        changed = changed || c.expression().get() != x.expression().get();
        args.push_back(c);
    }
    Array out = changed ? rebuild(e, args) : a;
    memo.put(e, out);
    return out;
}

// Evaluating a node turns every handle on it into its buffer, so after an inner reduction has been evaluated the tree
// holds unit axes inserted over a buffer: those become views of the buffer (what `rebuild` makes of them).
static Array fold_expanded_buffers(const Array& a, ExprMemo& memo) {
    auto e = a.expression();
    if (e->kind == Kind::BUFFER || e->kind == Kind::SCALAR) return a;
    if (const Array* known = memo.find(e)) return *known;
    std::vector<Array> args;
    bool changed = false;
    for (const Array& x : e->args) {
        Array c = fold_expanded_buffers(x, memo);
        changed = changed || c.expression().get() != x.expression().get();
        args.push_back(c);
    }
    if (e->kind == Kind::EXPAND_DIMS && args.size() == 1 && args[0].is_buffer()) changed = true;
    Array out = changed ? rebuild(e, args) : a;
    memo.put(e, out);
    return out;
}

static Domain domain_of(const std::vector<int>& shape) {
    Domain d;
    if (shape.empty()) return d;
    d.C = shape.back();
    d.R = numel_of(shape) / std::max<int64_t>(1, d.C);
    if (d.C == 0) d.R = 0;
    return d;
}

// Evaluate one (dest, op, root) after cleaning; splits until a kernel shape fits.
// A plain reduction of a buffer whose shape starves the one-pass kernels is done in two passes over a reshaped view:
//  - few long rows (one workgroup per row leaves most of the device idle): [R, C] is read as [R * S, C / S], reduced
//    along the rows, and the [R, S] partial results are reduced again;
//  - the leading axis of a narrow matrix (a strip of 256 columns per workgroup is mostly empty): [R, C] is read as
//    [R / k, k * C], reduced along the leading axis, and the [k, C] partial results are reduced again.
// Sums come out in a different (still tree-shaped) order; maxima, minima and products of the same values are unchanged.
static bool try_two_stage_reduce(const DestSpec& spec) {
    static const bool off = env_int("DALI_HIP_TWO_STAGE_REDUCE", 1) == 0;
    if (off) return false;
    auto e = spec.root.expression();
    if (e->kind != Kind::AXIS_REDUCE) return false;
    const std::string& red = e->name;
    if (red != "reducers::sum" && red != "reducers::maximum" && red != "reducers::minimum" && red != "reducers::product") return false;
    Array arg = e->args[0];
    if (!arg.is_buffer() && arg.ndim() == 2 && arg.dtype() == e->dtype && arg.expression()->kind == Kind::ELEMENTWISE && arg.shape()[0] >= 2 && arg.shape()[0] <= 64 &&
        numel_of(arg.shape()) >= (1 << 20)) {
        // The leading axis of a tall narrow expression (the column variances inside a standardisation: squares of [N, 7] minus
        // its column means): the fused form walks strips of 256 columns that hold seven ([9999999,7]: 700 us). The expression is
        // written out along memory first, as a map over rows grouped k at a time, and reduced as a buffer: two more passes over
        // the matrix against one that uses a thirtieth of every strip.
        Array matrix = arg.transpose();  // the same node over the operands as they lie in memory
        bool along_memory = matrix.expression()->kind == Kind::ELEMENTWISE;
        std::function<void(const Array&)> look = [&](const Array& a) {
            auto ae = a.expression();
            if (ae->kind == Kind::BUFFER) {
                if (numel_of(ae->shape) == numel_of(matrix.shape()) && !a.contiguous_memory()) along_memory = false;
            } else if (ae->kind == Kind::ELEMENTWISE || ae->kind == Kind::BROADCAST || ae->kind == Kind::EXPAND_DIMS) {
                for (const Array& x : ae->args) look(x);
            } else if (ae->kind != Kind::SCALAR) {
                along_memory = false;
            }
        };
        if (along_memory) look(matrix);
        if (along_memory) {
            Array buf = materialize(matrix);
            run_specs({{spec.dest, spec.op, op::axis_reduce(buf, red, {0}, false)}});
            return true;
        }
    }
    if (!arg.is_buffer() || arg.ndim() < 1 || arg.dtype() != e->dtype) return false;
    const int C_last = arg.shape().back();
    const int64_t n = numel_of(arg.shape());
    if (n == 0 || C_last == 0) return false;
    const int64_t rows = n / C_last;
    if (arg.contiguous_memory()) {
        // few long rows (from the size on at which a second launch pays, see try_segmented_reduce)
        if (rows >= 256 || C_last < (1 << 16)) return false;
        if (C_last < 200000 && n * 4 < ((int64_t)64 << 20)) return false;
        int S = 1;
        while (S * 2 * rows <= 2048 && C_last % (S * 2 * 4) == 0 && C_last / (S * 2) >= 8192) S *= 2;
        if (S < 4) return false;
        Array stage1 = op::axis_reduce(arg.reshape({(int)(rows * S), C_last / S}), red, {1}, false);
        stage1.eval();
        std::vector<int> partial_shape = e->shape;  // the leading dimensions of the argument, then the S partial results
        partial_shape.push_back(S);
        Array root2 = op::axis_reduce(stage1.reshape(partial_shape), red, {(int)partial_shape.size() - 1}, false);
        if (root2.shape() != e->shape) return false;
        run_specs({{spec.dest, spec.op, root2}});
        return true;
    }
    // leading axis of a narrow row-major matrix: the argument is the transposed view [C, R] with strides [1, C]
    if (arg.ndim() != 2) return false;
    const int Cn = arg.shape()[0], R = arg.shape()[1];
    const std::vector<int>& st = arg.strides();
    if (st.size() != 2 || st[0] != 1 || st[1] != Cn || Cn > 1024 || R < 4096) return false;
    // (between 513 and 1024 columns only where the second launch is small beside the first: [50000,1000] 38.0 -> 34.5 us, [65536,1024] 46.7 -> 43.0 us)
    if (Cn > 512 && (int64_t)R * Cn * 4 < ((int64_t)64 << 20)) return false;
    int k = 1;
    while (k * 2 * (int64_t)Cn <= 4096 && R / (k * 2) >= 64) k *= 2;
    if (k < 2) return false;
    Array matrix = arg.transpose();  // [R, C], contiguous
    if (!matrix.contiguous_memory()) return false;
    // rows beyond the last whole group of k (fewer than k, at most 4096 elements) join the k partial rows as they are:
    // [9999999,7] has no divisor to go by, and its sum took 555 us through strips of 256 columns that hold seven
    const int rest = R % k, R0 = R - rest;
    Array partial({k + rest, Cn}, arg.dtype());
    evaluate_into(partial.slice(0, 0, k).reshape({k * Cn}), OPERATOR_T_EQL, op::axis_reduce(matrix.slice(0, 0, R0).reshape({R0 / k, k * Cn}), red, {0}, false));
    if (rest > 0) evaluate_into(partial.slice(0, k, k + rest), OPERATOR_T_EQL, op::identity(matrix.slice(0, R0, R)));
    Array root2 = op::axis_reduce(partial, red, {0}, false);
    if (root2.shape() != e->shape) return false;
    run_specs({{spec.dest, spec.op, root2}});
    return true;
}

// Few long rows that the reshaped view above cannot serve: rows whose length is no multiple of four elements times the
// number of pieces, and the position of the best element (dali/array/op/reducer_operation.cpp:193-228,686-710). The row kernel
// itself cuts every row into S pieces (whole vectors each, the last one with the elements left over), a workgroup per piece,
// and leaves [R, S] partial results. Position: a piece yields its best value and that value's column in the whole row (the
// first one among equals); the first piece that holds the row's best value (an argmax over the S values, first among equals
// again) then names the column, which is the reference's "first index on ties".
static bool try_segmented_reduce(const DestSpec& spec) {
    static const bool off = env_int("DALI_HIP_SEGMENTED_REDUCE", 1) == 0;
    if (off) return false;
    auto e = spec.root.expression();
    const bool position = e->kind == Kind::ARG_AXIS_REDUCE;
    if (e->kind != Kind::AXIS_REDUCE && !position) return false;
    const std::string& red = e->name;
    if (position ? (red != "reducers::maximum" && red != "reducers::minimum")
                 : (red != "reducers::sum" && red != "reducers::maximum" && red != "reducers::minimum" && red != "reducers::product"))
        return false;
    Array arg = e->args[0];
    // a buffer of any rank, or an expression over [R, C] (the exponentials of a softmax's rows: whether it fits the row kernel is
    // the row kernel's to say)
    if (arg.ndim() < 1 || size_of_dtype(arg.dtype()) != 4) return false;
    if (arg.is_buffer() ? !arg.contiguous_memory() : arg.ndim() != 2) return false;
    if (!position && arg.dtype() != e->dtype) return false;
    const int C_last = arg.shape().back();
    const int64_t n = numel_of(arg.shape());
    if (n == 0 || C_last < (1 << 16)) return false;
    const int64_t rows = n / C_last;
    if (rows >= 256) return false;
    // Two or three launches against one: worth it once a row takes a workgroup longer than the extra launches (from about 200000
    // elements on: [4,262145] 8.5 -> 6.1 us, [8,131073] 5.2 -> 6.4 us) or the rows together are more than the caches keep between
    // two uses, where a workgroup streams its row from memory at a fortieth of what the device can ([64,1048577]: 131 -> 41 us).
    if (!g_segment_whatever_the_size && C_last < 200000 && n * 4 < ((int64_t)64 << 20)) return false;
    int S = 1;
    while (S * 2 * rows <= 2048 && C_last / (S * 2) >= 8192) S *= 2;
    if (S < 4) return false;
    const int R = (int)rows;
    Array rows2d = arg.is_buffer() ? arg.reshape({R, C_last}) : arg;
    const Domain dom = domain_of(rows2d.shape());
    std::vector<int> partial_shape = e->shape;  // the leading dimensions of the argument, then the S partial results
    partial_shape.push_back(S);
    Array best({R, S}, arg.dtype());
    if (!position) {
        if (!try_row({{best.pluck_axis(1, 0), OPERATOR_T_EQL, op::axis_reduce(rows2d, red, {1}, false)}}, dom, nullptr, S)) return false;
        Array root2 = op::axis_reduce(best.reshape(partial_shape), red, {(int)partial_shape.size() - 1}, false);
        if (root2.shape() != e->shape) return false;
        run_specs({{spec.dest, spec.op, root2}});
        return true;
    }
    Array where({R, S}, DTYPE_INT32);
    if (!try_row({{best.pluck_axis(1, 0), OPERATOR_T_EQL, op::axis_reduce(rows2d, red, {1}, false)},
                  {where.pluck_axis(1, 0), OPERATOR_T_EQL, op::argument_axis_reduce(rows2d, red, 1)}},
                 dom, nullptr, S))
        return false;
    Array piece = op::argument_axis_reduce(best, red, 1);
    piece.eval();
    Array root2 = op::gather_from_rows(where, piece);
    if (e->shape.size() != 1) root2 = root2.reshape(e->shape);
    run_specs({{spec.dest, spec.op, root2}});
    return true;
}

// A map over a tall matrix whose rows are short and off the vector size, with operands that hold one value per column (a
// bias added to [N, 7] features, columns minus their means): the row kernel would read such rows an element per lane
// ([9999999,7] + [1,7]: 190 us, 0.37 of the HBM peak). k neighbouring rows are read as one row of k * C elements instead, k a
// multiple of four, against the per-column operands repeated k times; the rows past the last whole group go through the
// ordinary form. Operands other than [R, C] matrices along memory, per-column vectors and single values: not taken.
static bool try_narrow_map(const DestSpec& spec) {
    static const bool off = env_int("DALI_HIP_NARROW_MAP", 1) == 0;
    const Array& dest = spec.dest;
    if (off || !dest.is_buffer() || dest.ndim() != 2 || !dest.contiguous_memory()) return false;
    const int R = dest.shape()[0], C = dest.shape()[1];
    if (C % 4 == 0 || C >= 256 || C < 2 || (int64_t)R * C < (1 << 20)) return false;
    const int k = std::max(4, 4 * ((512 / C + 3) / 4));
    if (R / k < 1024) return false;
    const int rest = R % k, R0 = R - rest;
    bool ok = true, per_column = false;
    // pass 0 only looks; pass 1 builds the grouped rows, pass 2 the rows left over
    int pass = 0;
    std::map<const Expr*, Array> tiles, memo;  // per-column operands repeated k times; what a node became in this pass
    auto mapped = [&](const std::vector<int>& shape, std::vector<int>* out) {
        const int64_t n = numel_of(shape);
        if (n == (int64_t)R * C && shape.size() == 2 && shape[0] == R) *out = pass == 2 ? std::vector<int>{rest, C} : std::vector<int>{R0 / k, k * C};
        else if (n == C && (shape == std::vector<int>{C} || shape == std::vector<int>{1, C})) *out = pass == 2 ? std::vector<int>{1, C} : std::vector<int>{1, k * C};
        else return false;
        return true;
    };
    std::function<Array(const Array&)> regroup = [&](const Array& a) -> Array {
        auto e = a.expression();
        if (!ok || e->kind == Kind::SCALAR || numel_of(e->shape) == 1) return a;  // single values are read as they are
        auto known = memo.find(e.get());
        if (known != memo.end()) return known->second;
        Array out = a;
        std::vector<int> shape;
        switch (e->kind) {
            case Kind::BUFFER:
                if (!a.contiguous_memory() || !mapped(e->shape, &shape)) {
                    ok = false;
                } else if (numel_of(e->shape) == C) {
                    per_column = true;
                    if (pass == 1) {
                        auto made = tiles.find(e.get());
                        if (made == tiles.end()) {
                            Array t({1, k * C}, e->dtype);
                            auto b = std::make_shared<Expr>();
                            b->kind = Kind::BROADCAST;
                            b->args = {a.reshape({1, C})};
                            b->shape = {k, C};
                            b->dtype = e->dtype;
                            evaluate_into(t.reshape({k, C}), OPERATOR_T_EQL, op::identity(Array(b)));
                            made = tiles.emplace(e.get(), t).first;
                        }
                        out = made->second;
                    } else if (pass == 2) {
                        out = a.reshape({1, C});
                    }
                } else if (pass == 1) {
                    out = a.slice(0, 0, R0).reshape({R0 / k, k * C});
                } else if (pass == 2) {
                    out = a.slice(0, R0, R);
                }
                break;
            case Kind::EXPAND_DIMS:
                out = regroup(e->args[0]);  // ([C] -> [1, C]: the grouped form is two-dimensional already)
                if (numel_of(e->shape) != C) ok = false;
                break;
            case Kind::BROADCAST:
            case Kind::ELEMENTWISE: {
                if (!mapped(e->shape, &shape)) {
                    ok = false;
                    break;
                }
                std::vector<Array> args;
                for (const Array& x : e->args) args.push_back(regroup(x));
                if (!ok || pass == 0) break;
                if (e->kind == Kind::BROADCAST && args[0].shape() == shape) {
                    out = args[0];
                    break;
                }
                auto n = std::make_shared<Expr>(*e);
                n->args = args;
                n->shape = shape;
                out = Array(n);
                break;
            }
            default: ok = false;
        }
        memo[e.get()] = out;
        return out;
    };
    regroup(spec.root);
    if (!ok || !per_column) return false;
    pass = 1;
    memo.clear();
    Array head = regroup(spec.root);
    if (!ok) return false;
    run_specs({{dest.slice(0, 0, R0).reshape({R0 / k, k * C}), spec.op, head}});
    if (rest > 0) {
        pass = 2;
        memo.clear();
        Array tail = regroup(spec.root);
        if (!ok) throw std::runtime_error("internal: the rows left over by a grouped map could not be planned");
        run_specs({{dest.slice(0, R0, R), spec.op, tail}});
    }
    return true;
}

void run_specs_planned(std::vector<DestSpec> specs) {
    if (specs.size() == 1 && (try_two_stage_reduce(specs[0]) || try_segmented_reduce(specs[0]))) return;
    if (specs.size() == 1) {
        // the same reductions with their reduced axes kept as unit axes (keepdims): unit axes inserted over the reduction,
        // written through a view of the destination without them
        Array base = specs[0].root;
        while (base.expression()->kind == Kind::EXPAND_DIMS) base = base.expression()->args[0];
        const Kind bk = base.expression()->kind;
        if (base.expression().get() != specs[0].root.expression().get() && (bk == Kind::AXIS_REDUCE || bk == Kind::ARG_AXIS_REDUCE) &&
            specs[0].dest.is_buffer() && specs[0].dest.contiguous_memory() && numel_of(specs[0].dest.shape()) == numel_of(base.shape())) {
            DestSpec plain{specs[0].dest.reshape(base.shape()), specs[0].op, base};
            if (try_two_stage_reduce(plain) || try_segmented_reduce(plain)) return;
        }
    }
    // all-reduce roots are planned one by one
    if (specs.size() > 1) {
        bool any_all = false;
        for (auto& s : specs) any_all = any_all || has_kind(s.root, [](Kind k) { return is_all_reduce(k); });
        if (any_all) {
            // Full reductions of per-row values next to requests over the rows themselves (the mean loss beside the
            // gradient and the row losses of a cross-entropy) join the row kernel of the others: one launch.
            std::vector<DestSpec> plain, totals;
            for (auto& s : specs) (has_kind(s.root, [](Kind k) { return is_all_reduce(k); }) ? totals : plain).push_back(s);
            static const bool fuse_totals = env_int("DALI_HIP_ROW_TOTALS", 1) != 0;
            bool row_reduces = !plain.empty();
            for (auto& s : plain) row_reduces = row_reduces && !has_kind(s.root, [](Kind k) { return k == Kind::MATMUL; });
            if (fuse_totals && row_reduces) {
                Array first;
                std::set<const Expr*> seen;
                bool found = false;
                for (auto& s : plain)
                    if (find_first_reduce(s.root, &first, seen)) { found = true; break; }
                if (found) {
                    Domain dom = domain_of(first.expression()->args[0].shape());
                    // (tens of thousands of short rows: a workgroup would live as long as its ticket takes to come back, two memory
                    // round trips for a few microseconds of work, and a second small launch over the per-row values is cheaper:
                    // cross-entropy on [65536,513] 93 -> 51 us, on [100000,1000] 158 -> 142 us)
                    const bool many_short_rows = dom.C < 2048 && dom.R >= 16384;
                    if (!many_short_rows && try_row(plain, dom, &totals)) return;
                }
            }
            if (!plain.empty() && !totals.empty()) {
                // otherwise the others first, together; what they computed is not computed again for the full reductions
                run_specs(plain);
                for (auto& t : totals) {
                    for (auto& p : plain) {
                        ExprMemo memo;
                        t.root = substitute(t.root, p.root.expression().get(), p.dest, memo);
                    }
                    run_specs({t});
                }
                return;
            }
            for (auto& s : specs) run_specs({s});
            return;
        }
    }
    for (int iter = 0; iter < 64; ++iter) {
        if (iter > 0 && specs.size() == 1) {
            ExprMemo fold_memo;
            specs[0].root = fold_expanded_buffers(specs[0].root, fold_memo);
        }
        bool has_all = has_kind(specs[0].root, [](Kind k) { return is_all_reduce(k); });
        if (has_all) {
            if (try_all(specs[0])) return;
            // materialise every full reduction into a 0-d buffer and continue as an elementwise map
            std::vector<Array> reds;
            std::set<const Expr*> seen;
            find_all_reduces(specs[0].root, reds, seen);
            for (const Array& r : reds) {
                Array rr = r;
                Array arg = rr.expression()->args[0];
                if (arg.is_buffer() && !arg.contiguous_memory()) {
                    rr = rebuild(rr.expression(), {arg.ascontiguousarray()});
                } else if (!arg.is_buffer()) {
                    std::set<const Expr*> s2;
                    if (!flat_eligible(arg, numel_of(arg.shape()), s2)) rr = rebuild(rr.expression(), {materialize(arg)});
                }
                Array buf({}, rr.dtype());
                DestSpec ds{buf, OPERATOR_T_EQL, rr};
                if (!try_all(ds)) throw std::runtime_error("internal: full reduction could not be planned");
                ExprMemo memo;
                specs[0].root = substitute(specs[0].root, r.expression().get(), buf, memo);
            }
            continue;
        }
        bool has_red = false;
        for (auto& s : specs) has_red = has_red || has_kind(s.root, [](Kind k) { return is_reduce(k); });
        if (!has_red) {
            if (try_flat(specs)) return;
            if (specs.size() == 1 && !g_dry_run && try_narrow_map(specs[0])) return;
            if (specs.size() == 1) {
                // Large transposed matrices among the operands are first written out along memory by a tiled transpose
                // (both its reads and its writes are coalesced); a map that walked them in place would fetch a cache line
                // per element ([16384,4096]: x.T + 1 took 721 us, a transposed copy takes 90).
                DestSpec& sp = specs[0];
                auto re = sp.root.expression();
                if (re->kind == Kind::ELEMENTWISE && re->name == "functor::identity" && sp.op == OPERATOR_T_EQL && sp.dest.contiguous_memory() &&
                    is_transposed_matrix(re->args[0].expression().get()) && re->args[0].dtype() == sp.dest.dtype() &&
                    re->args[0].shape() == sp.dest.shape()) {
                    run_transpose_into(sp.dest, re->args[0]);
                    return;
                }
                if (try_transposed_map(sp)) return;
                Array found;
                std::function<bool(const Array&)> find = [&](const Array& a) {
                    auto ae = a.expression();
                    if (ae->kind == Kind::BUFFER) {
                        if (is_transposed_matrix(ae.get())) {
                            found = a;
                            return true;
                        }
                        return false;
                    }
                    if (ae->kind == Kind::SCALAR) return false;
                    for (const Array& x : ae->args)
                        if (find(x)) return true;
                    return false;
                };
                if (find(sp.root)) {
                    Array copy(found.shape(), found.dtype());
                    run_transpose_into(copy, found);
                    ExprMemo memo;
                    sp.root = substitute(sp.root, found.expression().get(), copy, memo);
                    continue;
                }
            }
            Domain dom = domain_of(specs[0].dest.shape());
            if (specs[0].dest.ndim() <= 1 && has_kind(specs[0].root, [](Kind k) { return k == Kind::GATHER_FROM_ROWS; })) {
                // one gathered element per row: a single-column domain
                dom.R = numel_of(specs[0].dest.shape());
                dom.C = 1;
            }
            if (try_row(specs, dom)) return;
            if (try_generic(specs)) return;
            if (specs.size() > 1) {
                for (auto& s : specs) run_specs({s});
                return;
            }
            // last resort for layouts the 2-D model cannot express: make strided operands contiguous
            bool changed = false;
            std::function<Array(const Array&)> fix = [&](const Array& x) -> Array {
                auto e = x.expression();
                if (e->kind == Kind::BUFFER) {
                    if (!x.contiguous_memory() && numel_of(e->shape) > 1) {
                        // copy through the row kernel on the buffer's own shape
                        Array c(e->shape, e->dtype);
                        Domain d2 = domain_of(e->shape);
                        std::vector<DestSpec> cp = {{c, OPERATOR_T_EQL, op::identity(x)}};
                        if (!try_row(cp, d2) && !try_generic(cp)) throw std::runtime_error(make_message("unsupported strided layout ", shape_str(e->strides), " for shape ", shape_str(e->shape)));
                        changed = true;
                        return c;
                    }
                    return x;
                }
                std::vector<Array> args;
                bool ch = false;
                for (const Array& y : e->args) {
                    Array c = fix(y);
                    ch = ch || c.expression().get() != y.expression().get();
                    args.push_back(c);
                }
                return ch ? rebuild(e, args) : x;
            };
            specs[0].root = fix(specs[0].root);
            if (changed) continue;
            if (!specs[0].dest.contiguous_memory()) {
                // evaluate into a contiguous temporary, then copy into the strided destination
                Array tmp(specs[0].dest.shape(), specs[0].dest.dtype());
                run_specs({{tmp, OPERATOR_T_EQL, specs[0].root}});
                std::vector<DestSpec> cp = {{specs[0].dest, specs[0].op, op::identity(tmp)}};
                Domain d2 = domain_of(specs[0].dest.shape());
                if (try_row(cp, d2) || try_generic(cp)) return;
            }
            throw std::runtime_error("expression could not be mapped onto a kernel shape (unsupported broadcast or layout)");
        }
        // reductions over the trailing axis
        Array first;
        std::set<const Expr*> seen;
        for (auto& s : specs)
            if (find_first_reduce(s.root, &first, seen)) break;
        Domain dom = domain_of(first.expression()->args[0].shape());
        if (specs.size() == 1) {
            // The argument of a reduction against the layout of its operands (a candidate for the column kernel) may hold
            // small unevaluated operands that are broadcast along the reduced axis (the column means inside a variance):
            // those are evaluated first, so that the column kernel reads them as one value per kept index.
            Array inner;
            std::set<const Expr*> seen_inner;
            if (find_innermost_reduce(specs[0].root, &inner, seen_inner) &&
                (inner.expression()->kind == Kind::AXIS_REDUCE || inner.expression()->kind == Kind::ARG_AXIS_REDUCE)) {
                Array red_arg = inner.expression()->args[0];
                bool against_layout = false, settled = false;
                std::function<void(const Array&)> scan = [&](const Array& a) {
                    auto ae = a.expression();
                    if (ae->kind == Kind::BUFFER && ae->shape.size() >= 2 && ae->shape.back() > 1 && numel_of(ae->shape) > ae->shape.back() &&
                        strides_of(ae.get()).back() != 1)
                        against_layout = true;
                    if (ae->kind != Kind::BUFFER && ae->kind != Kind::SCALAR)
                        for (const Array& x : ae->args) scan(x);
                };
                scan(red_arg);
                std::function<void(const Array&)> settle = [&](const Array& a) {
                    auto ae = a.expression();
                    if (ae->kind == Kind::BUFFER || ae->kind == Kind::SCALAR) return;
                    if (ae->kind == Kind::BROADCAST && !ae->args[0].is_buffer() && numel_of(ae->args[0].shape()) > 1 &&
                        col_kept_vector(ae->args[0].shape(), red_arg.shape()) && !has_kind(ae->args[0], [](Kind k) { return is_reduce(k); })) {
                        materialize(ae->args[0]);
                        settled = true;
                        return;
                    }
                    for (const Array& x : ae->args) settle(x);
                };
                if (against_layout && red_arg.ndim() >= 2) settle(red_arg);
                if (settled) continue;
            }
        }
        if (specs.size() == 1 && try_col(specs[0])) return;
        if (specs.size() == 1) {
            // A reduction along the leading axis of row-major operands under further arithmetic (mean = sum / count, a
            // normalisation by the column maxima): the row kernel would walk the operands against their layout, so
            // the reduction goes through the column kernel on its own and the rest reads its small result.
            Array inner;
            std::set<const Expr*> seen_inner;
            if (find_innermost_reduce(specs[0].root, &inner, seen_inner) && inner.expression().get() != specs[0].root.expression().get() &&
                (inner.expression()->kind == Kind::AXIS_REDUCE || inner.expression()->kind == Kind::ARG_AXIS_REDUCE)) {
                Array red_arg = inner.expression()->args[0];
                bool has_layout = false;  // at least one operand whose reduced axis does not run along memory
                std::function<void(const Array&)> scan = [&](const Array& a) {
                    auto ae = a.expression();
                    if (ae->kind == Kind::BUFFER && ae->shape.size() >= 2 && ae->shape.back() > 1 && numel_of(ae->shape) > ae->shape.back() &&
                        strides_of(ae.get()).back() != 1)
                        has_layout = true;
                    if (ae->kind != Kind::BUFFER && ae->kind != Kind::SCALAR)
                        for (const Array& x : ae->args) scan(x);
                };
                scan(red_arg);
                if (red_arg.ndim() >= 2 && numel_of(red_arg.shape()) > red_arg.shape().back() && has_layout && col_split_of(red_arg) >= 0) {
                    Array buf = materialize(inner);
                    ExprMemo memo;
                    specs[0].root = substitute(specs[0].root, inner.expression().get(), buf, memo);
                    continue;
                }
            }
        }
        if (specs.size() == 1) {
            // Reductions along few long rows under further arithmetic (rows minus their means, rows over their norms, a
            // log-softmax): one launch would give each row to one workgroup, which walks it once per phase through a single
            // compute unit ([7,9999999] minus the row means: 2.5 ms). The reductions are evaluated on their own instead, in pieces of
            // the rows that fill the device, and what is left is a map over the rows that reads their small results.
            static const bool pieces_off = env_int("DALI_HIP_SEGMENTED_REDUCE", 1) == 0;
            // (a result per row only: the rows are walked once either way, and what counts is the rule of a reduction on its own)
            const bool map_over_rows = numel_of(specs[0].dest.shape()) == dom.R * dom.C;
            const bool few_long_rows = dom.R < 256 && dom.C >= 65536 &&
                                       (dom.R * dom.C * 4 >= ((int64_t)64 << 20) ||
                                        (map_over_rows ? dom.C >= 131072 && (double)dom.R < 75.0 - 3.75e6 / (double)dom.C : dom.C >= 200000));
            Array inner;
            std::set<const Expr*> seen_inner;
            if (!pieces_off && few_long_rows && find_innermost_reduce(specs[0].root, &inner, seen_inner) &&
                inner.expression().get() != specs[0].root.expression().get() &&
                (inner.expression()->kind == Kind::AXIS_REDUCE || inner.expression()->kind == Kind::ARG_AXIS_REDUCE) &&
                domain_of(inner.expression()->args[0].shape()).C == dom.C) {
                const bool before = g_segment_whatever_the_size;
                g_segment_whatever_the_size = true;  // (the rule above has been applied; a reduction on its own has another)
                Array buf;
                try {
                    buf = materialize(inner);
                } catch (...) {
                    g_segment_whatever_the_size = before;
                    throw;
                }
                g_segment_whatever_the_size = before;
                ExprMemo memo;
                specs[0].root = substitute(specs[0].root, inner.expression().get(), buf, memo);
                continue;
            }
        }
        if (try_row(specs, dom)) return;
        if (specs.size() > 1) {
            for (auto& s : specs) run_specs({s});
            return;
        }
        // split: evaluate an innermost reduction on its own and substitute the buffer
        Array inner;
        std::set<const Expr*> seen2;
        if (!find_innermost_reduce(specs[0].root, &inner, seen2)) throw std::runtime_error("internal: reduce node vanished");
        Array arg = inner.expression()->args[0];
        bool bare = inner.expression().get() == specs[0].root.expression().get();
        bool arg_is_leaf = arg.is_buffer();
        if (bare && arg_is_leaf) {
            // a lone reduction over a buffer whose layout fits neither template: copy to contiguous
            if (arg.contiguous_memory()) throw std::runtime_error("internal: contiguous reduction was rejected by every kernel shape");
            Array c = arg.ascontiguousarray();
            specs[0].root = rebuild(inner.expression(), {c});
            continue;
        }
        if (!arg_is_leaf && bare) {
            Array c = materialize(arg);
            specs[0].root = rebuild(inner.expression(), {c});
            continue;
        }
        Array buf = materialize(inner);
        ExprMemo memo;
        specs[0].root = substitute(specs[0].root, inner.expression().get(), buf, memo);
    }
    throw std::runtime_error("planner did not converge");
}

}  // namespace jit

bool few_long_rows_softmax_statistics(Array* x, Array* maxima, Array* sums) { return jit::softmax_statistics_in_pieces(x, maxima, sums); }

using namespace jit;

void evaluate(const std::vector<Array>& roots) {
    jit_stats().evals++;
    jit_stats().last_kernel_kinds.clear();
    jit_stats().last_kernel_names.clear();
    g_last_source.clear();
    std::vector<DestSpec> specs;
    ExprMemo memo;
    std::vector<Array> pending;
    for (const Array& r : roots) {
        auto e = r.expression();
        if (e->kind == Kind::BUFFER || e->kind == Kind::SCALAR) continue;
        Array c = clean(r, memo, true);
        if (c.expression()->kind == Kind::BUFFER) {
            // the whole root was a GEMM (or an already evaluated node): adopt its buffer
            r.state_->expr = c.expression();
            continue;
        }
        Array dest(e->shape, e->dtype);
        specs.push_back({dest, OPERATOR_T_EQL, c});
        pending.push_back(r);
    }
    if (specs.empty()) return;
    run_specs(specs);
    // the node becomes its buffer (dali/array/expression/computation.cpp:13-28)
    for (size_t i = 0; i < pending.size(); ++i) pending[i].state_->expr = specs[i].dest.expression();
}

void evaluate_into(const Array& dest, OPERATOR_T op, const Array& source) {
    if (!dest.is_buffer() && (dest.expression()->kind == Kind::GATHER || dest.expression()->kind == Kind::GATHER_FROM_ROWS)) {
        scatter_assign(dest, op, source);
        return;
    }
    DALI_ASSERT(dest.is_buffer(), "assignment destination must be an evaluated buffer");
    jit_stats().evals++;
    jit_stats().last_kernel_kinds.clear();
    jit_stats().last_kernel_names.clear();
    g_last_source.clear();
    Array src = source;
    if (src.dtype() != dest.dtype()) src = op::astype(src, dest.dtype());
    // shape check with broadcasting of single elements (dali/array/jit/jit_utils.cpp:88-105)
    if (src.shape() != dest.shape()) {
        DALI_ASSERT(numel_of(src.shape()) == 1 || numel_of(src.shape()) == numel_of(dest.shape()),
                    make_message("Cannot assign result of shape ", shape_str(src.shape()), " to a location of shape ", shape_str(dest.shape()), "."));
    }
    ExprMemo memo;
    auto se = src.expression();
    // dst (+)= dot(a, b): the GEMM writes (accumulates into) the destination directly
    if (se->kind == Kind::MATMUL && (dest.dtype() == DTYPE_FLOAT || dest.dtype() == DTYPE_DOUBLE) && se->dtype == dest.dtype() && dest.ndim() == 2 &&
        (dest.strides().empty() || dest.strides()[1] == 1) && (op == OPERATOR_T_EQL || op == OPERATOR_T_ADD)) {
        run_gemm(dest, se.get(), nullptr, op == OPERATOR_T_ADD ? 1.0f : 0.0f);
        return;
    }
    Array c = clean(src, memo, true);
    if (c.expression()->kind == Kind::SCALAR || c.expression()->kind == Kind::BUFFER) c = op::identity(c);
    run_specs({{dest, op, c}});
}

// Several assignments dest_i = source_i planned together (one kernel where they fuse): the destinations are buffers or views
// of buffers of their sources' shapes and dtypes.
void evaluate_into_together(const std::vector<Array>& dests, const std::vector<Array>& sources) {
    DALI_ASSERT(dests.size() == sources.size() && !dests.empty(), "evaluate_into_together: one source per destination");
    jit_stats().evals++;
    jit_stats().last_kernel_kinds.clear();
    jit_stats().last_kernel_names.clear();
    g_last_source.clear();
    std::vector<DestSpec> specs;
    ExprMemo memo;
    for (size_t i = 0; i < dests.size(); ++i) {
        DALI_ASSERT(dests[i].is_buffer() && dests[i].shape() == sources[i].shape() && dests[i].dtype() == sources[i].dtype(),
                    "evaluate_into_together: a destination must be an evaluated buffer of its source's shape and dtype");
        Array c = clean(sources[i], memo, true);
        if (c.expression()->kind == Kind::SCALAR || c.expression()->kind == Kind::BUFFER) c = op::identity(c);
        specs.push_back({dests[i], OPERATOR_T_EQL, c});
    }
    run_specs(specs);
}

std::vector<std::string> generate_only(const std::vector<Array>& roots) {
    std::vector<std::string> sources;
    bool prev = g_dry_run;
    g_dry_run = true;
    g_dry_sources = &sources;
    try {
        evaluate(roots);
    } catch (...) {
        g_dry_run = prev;
        g_dry_sources = nullptr;
        throw;
    }
    g_dry_run = prev;
    g_dry_sources = nullptr;
    return sources;
}

}  // namespace dali
