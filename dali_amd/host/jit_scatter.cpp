// Assignment through a gather (dali/array/op/gather.cpp, scatter.cpp): rows addressed by an index vector are
// combined without atomics, by scanning the index vector in LDS for short vectors or by ordering the indices first.
#include "jit_internal.h"

namespace dali {
namespace jit {

// Assignment through a gather: dest[indices[i], :] (op)= values[i, :] for i in input order
// (dali/array/op/gather.cpp:89-97,126-143). The indices are ordered by a stable sort; one workgroup per run of
// equal indices reads the destination row once, applies the run's contributions one after the other in input
// order (the order of the reference's sequential CPU loop) and writes the row once. No atomics, and the result
// does not depend on scheduling.
ArrayArg manual_arg(const Array& buf, Cls cls, bool is_dest, int nd, const std::vector<int>& sizes, const std::vector<int>& strides) {
    ArrayArg a;
    a.buf = buf.expression();
    a.cls = cls;
    a.is_dest = is_dest;
    a.nd = nd;
    a.sizes = sizes;
    a.strided = !strides.empty();
    a.strides = strides;
    return a;
}

static std::string gen_scatter_rows_kernel(const Program& P, const IvLayout& L, OPERATOR_T op, bool scalar_value, int VEC, const std::string& kname) {
    std::string t = ctype(P.arrays[0].buf->dtype);
    std::ostringstream ss;
    ss << device_prelude();
    ss << kargs_struct(P, L);
    // One wave per sorted position, sixteen to a workgroup (a workgroup per position was launch-bound: 65536 positions of
    // 4 KiB rows took 250 us). Only the wave at the head of a run of equal indices works: it reads the destination row once,
    // applies the run's rows of values in input order and writes the row once.
    ss << "extern \"C\" __global__ __launch_bounds__(1024) void " << kname << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n";
    ss << "  constexpr int VEC = " << VEC << ";\n";
    ss << "  const long N = A.iv[" << L.shape_pos[0] << "], D = A.iv[" << L.shape_pos[0] + 1 << "];\n";
    ss << "  const int* sk = (const int*)A.p[1];\n  const int* pm = (const int*)A.p[2];\n";
    ss << "  const int lane = threadIdx.x & 63;\n";
    ss << "  const long p = (long)blockIdx.x * 16 + (long)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));\n  if (p >= N) return;\n";
    ss << "  const int key = sk[p];\n";
    ss << "  if ((unsigned)key >= (unsigned)A.iv[" << L.shape_pos[0] + 2 << "]) return;  // no such destination row: skipped\n";
    ss << "  if (p > 0 && sk[p - 1] == key) return;  // only the head of a run of equal indices works\n";
    ss << "  long q_end = p + 1;\n  while (q_end < N && sk[q_end] == key) ++q_end;\n";
    ss << "  const long drs = A.iv[" << L.stride_pos[0] << "], dcs = A.iv[" << L.stride_pos[0] + 1 << "];\n";
    ss << "  " << t << "* drow = (" << t << "*)A.p[0] + (long)key * drs;\n";
    if (scalar_value) {
        ss << "  const " << t << " sv = ((const " << t << "*)A.p[3])[0];\n";
    } else {
        ss << "  const long vrs = A.iv[" << L.stride_pos[3] << "], vcs = A.iv[" << L.stride_pos[3] + 1 << "];\n";
        ss << "  const " << t << "* vals = (const " << t << "*)A.p[3];\n";
    }
    ss << "  for (long c = (long)lane * VEC; c < D; c += 64 * VEC) {\n";
    if (VEC > 1) {
        ss << "    dali_vec<" << t << ", VEC> acc = dali_load<" << t << ", VEC>(drow + c);\n";
        ss << "    for (long q = p; q < q_end; ++q) {\n";
        if (!scalar_value) ss << "      const dali_vec<" << t << ", VEC> v = dali_load_nt<" << t << ", VEC>(vals + (long)pm[q] * vrs + c);\n";
        ss << "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) acc.v[j] = " << op_combine(op, "acc.v[j]", scalar_value ? "sv" : "v.v[j]") << ";\n";
        ss << "    }\n    dali_store<" << t << ", VEC>(drow + c, acc);\n";
    } else {
        ss << "    " << t << " acc = drow[c * dcs];\n";
        ss << "    for (long q = p; q < q_end; ++q) {\n";
        if (!scalar_value) ss << "      const " << t << " v = vals[(long)pm[q] * vrs + c * vcs];\n";
        ss << "      acc = " << op_combine(op, "acc", scalar_value ? "sv" : "v") << ";\n";
        ss << "    }\n    drow[c * dcs] = acc;\n";
    }
    ss << "  }\n}\n";
    return ss.str();
}

// Assignment through a gather without ordering the indices first, for index vectors that fit the LDS of a workgroup.
// One wave per input position p. A workgroup (16 waves) first copies the whole index vector into LDS. Wave p then looks
// for its index among the positions before p: if it is there, the wave of that earlier position owns the destination row
// and this one is done. Otherwise it loads the destination row, applies its own row of values, keeps scanning the
// positions after p and applies every later row with the same index as it meets it, i.e. in input order, which is the
// order of the reference's sequential loop (dali/array/op/gather.cpp:89-97); then it stores the row once. All waves
// together make N * N comparisons against LDS, which the device does in the shadow of the memory traffic; no index
// ordering pass (and no launch for it) is needed. The values are an expression evaluated where they are used, as in the
// reference's fused scatter kernel (gather.cpp:126-143). Indices outside the destination are skipped.
//
// `sorted`: for index vectors beyond what LDS holds. P.arrays[1] then holds the indices in ascending order (stable) and
// P.arrays[2] the input position of each; the wave of a sorted position works when it heads a run of equal indices, and the
// run's rows of values, still an expression, are evaluated in input order as above.
static std::string gen_scatter_scan_kernel(const Program& P, const IvLayout& L, OPERATOR_T op, int root, int VEC, int KCAP, const std::string& kname, bool sorted) {
    const std::string t = ctype(P.arrays[0].buf->dtype);
    const size_t first_operand = sorted ? 3 : 2;
    const int U = VEC == 4 ? 4 : 16;
    RowParams rp;
    rp.cached = false;
    rp.VEC = VEC;
    std::vector<int> first_body(P.nodes.size(), -1);
    std::ostringstream ss;
    ss << device_prelude();
    ss << kargs_struct(P, L);
    ss << "extern \"C\" __global__ __launch_bounds__(1024) void " << kname << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n";
    ss << "  constexpr int VEC = " << VEC << ", U = " << U << ", KCAP = " << KCAP << ", TILE = 64 * VEC * U;\n";
    ss << "  const int N = A.iv[" << L.shape_pos[0] << "], D = A.iv[" << L.shape_pos[0] + 1 << "], V = A.iv[" << L.shape_pos[0] + 2 << "];\n";
    ss << "  const long C = D; (void)C;\n";
    if (sorted) {
        ss << "  (void)KCAP;\n  const int* sk = (const int*)A.p[1];\n  const int* pm = (const int*)A.p[2];\n";
        ss << "  const int lane = threadIdx.x & 63;\n  const int p = (int)blockIdx.x * 16 + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));\n";
        ss << "  if (p >= N) return;\n  const int key = sk[p];\n  const bool valid = (unsigned)key < (unsigned)V;\n";
        ss << "  if (!valid) return;  // no such destination row: skipped\n  if (p > 0 && sk[p - 1] == key) return;  // only the head of a run of equal indices works\n";
        ss << "  int q_end = p + 1;\n  while (q_end < N && sk[q_end] == key) ++q_end;\n";
    } else {
    ss << "  __shared__ __attribute__((aligned(16))) int lk[KCAP];\n";
    ss << "  const int* keys = (const int*)A.p[1];\n";
    ss << "  const int lane = threadIdx.x & 63;\n  const int p = (int)blockIdx.x * 16 + (int)(threadIdx.x >> 6);\n";
    ss << "  const int key = p < N ? keys[p] : -1;\n  const bool valid = (unsigned)key < (unsigned)V;  // else: no such destination row, skipped\n";
    // this thread's share of the index vector
    ss << "  constexpr int KF = (KCAP + 4095) / 4096;\n  dali_vec<int, 4> kf[KF];\n";
    ss << "  _Pragma(\"unroll\") for (int f = 0; f < KF; ++f) {\n    const int t = (int)threadIdx.x * 4 + f * 4096;\n"
          "    if (t + 3 < N) kf[f] = dali_loadu<int, 4>(keys + t);\n    else { _Pragma(\"unroll\") for (int b = 0; b < 4; ++b) kf[f].v[b] = t + b < N ? keys[t + b] : -1; }\n  }\n";
    }
    for (size_t i = first_operand; i < P.arrays.size(); ++i) {
        const ArrayArg& a = P.arrays[i];
        const std::string ty = ctype(a.buf->dtype);
        if (a.cls == Cls::SCAL) ss << "  const " << ty << " sl" << i << " = ((const " << ty << "*)A.p[" << i << "])[0];\n";
        if (a.cls == Cls::FULL && a.strided) ss << "  const long cs" << i << " = A.iv[" << L.stride_pos[i] + 1 << "];\n";
        if (a.cls == Cls::ROW) ss << "  " << ty << " rl" << i << " = (" << ty << ")0;\n";
        if (a.cls == Cls::FULL) ss << "  " << ty << " x" << i << "[U][VEC];\n";
    }
    ss << "  const long drs = A.iv[" << L.stride_pos[0] << "], dcs = A.iv[" << L.stride_pos[0] + 1 << "]; (void)dcs;\n";
    ss << "  " << t << "* drow = (" << t << "*)A.p[0] + (long)(valid ? key : 0) * drs;\n";
    ss << "  " << t << " acc[U][VEC];\n";
    if (!sorted) {
    ss << "  const dali_vec<int, 4>* lk4 = reinterpret_cast<const dali_vec<int, 4>*>(lk);\n";
    ss << "  const int p_lo = p & ~255;\n  unsigned int m_own = 0;  // this lane's positions after p, in p's own chunk, that repeat the index\n";
    // the index vector goes to LDS; then the ownership test
    ss << "  {\n";
    ss << "      _Pragma(\"unroll\") for (int f = 0; f < KF; ++f) {\n        const int t = (int)threadIdx.x * 4 + f * 4096;\n"
          "        if (t < KCAP) *reinterpret_cast<dali_vec<int, 4>*>(&lk[t]) = kf[f];\n      }\n      __syncthreads();\n      if (!valid) return;\n";
    // Four vector compares per 256 positions: each writes a wave-wide mask, the masks are joined on the scalar unit. The
    // chunk that holds p itself is the only one whose positions have to be told apart (before p: ownership; after p: the
    // first duplicates).
    ss << "      unsigned long long found = 0;\n      _Pragma(\"unroll 4\") for (int base = 0; base < p_lo; base += 256) {\n"
          "        const dali_vec<int, 4> k4 = lk4[(base >> 2) + lane];\n"
          "        found |= __ballot(k4.v[0] == key) | __ballot(k4.v[1] == key) | __ballot(k4.v[2] == key) | __ballot(k4.v[3] == key);\n      }\n"
          "      if (found) return;  // an earlier position holds the same index: its wave works on this row\n";
    ss << "      const int j0 = p_lo + lane * 4;\n      const dali_vec<int, 4> k4 = lk4[(p_lo >> 2) + lane];\n      int before = 0;\n"
          "      _Pragma(\"unroll\") for (int b = 0; b < 4; ++b) { before |= (k4.v[b] == key && j0 + b < p) ? 1 : 0; m_own |= (k4.v[b] == key && j0 + b > p) ? (1u << b) : 0u; }\n"
          "      if (__any(before)) return;\n  }\n";
    }
    ss << "  for (int c0 = 0; c0 < D; c0 += TILE) {\n";
    // loads of row `row` of the value expression's operands
    ss << "    auto fetch = [&](const long row) {\n";
    for (size_t i = first_operand; i < P.arrays.size(); ++i) {
        const ArrayArg& a = P.arrays[i];
        const std::string ty = ctype(a.buf->dtype);
        if (a.cls == Cls::ROW)
            ss << "      rl" << i << " = ((const " << ty << "*)A.p[" << i << "])[row" << (a.strided ? " * (long)A.iv[" + std::to_string(L.stride_pos[i]) + "]" : std::string()) << "];\n";
        else if (a.cls == Cls::FULL)
            ss << "      const " << ty << "* w" << i << " = (const " << ty << "*)A.p[" << i << "] + row * " << (a.strided ? "(long)A.iv[" + std::to_string(L.stride_pos[i]) + "]" : std::string("(long)D")) << ";\n";
    }
    ss << "      _Pragma(\"unroll\") for (int u = 0; u < U; ++u) {\n        const int ch = c0 / VEC + lane + 64 * u;\n        if (ch * VEC < D) {\n";
    for (size_t i = first_operand; i < P.arrays.size(); ++i)
        if (P.arrays[i].cls == Cls::FULL) emit_leaf_load(ss, P.arrays[i], (int)i, VEC, "x" + std::to_string(i) + "[u]", "          ", sorted, false, "w");
    ss << "        }\n      }\n    };\n";
    ss << "    auto combine = [&]() {\n      _Pragma(\"unroll\") for (int u = 0; u < U; ++u) {\n        const int ch = c0 / VEC + lane + 64 * u;\n        if (ch * VEC < D) {\n";
    {
        BodyEmitter be(P, rp, true, 0, &first_body);
        be.leaf_suffix = "[u][j]";
        const std::string v = be.value(root);
        ss << "          _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) {\n            const int col = ch * VEC + j; (void)col;\n" << be.stmts.str();
        ss << "            acc[u][j] = " << op_combine(op, "acc[u][j]", "(" + t + ")(" + v + ")") << ";\n          }\n";
    }
    ss << "        }\n      }\n    };\n";
    ss << "    if (valid) {\n      _Pragma(\"unroll\") for (int u = 0; u < U; ++u) {\n        const int ch = c0 / VEC + lane + 64 * u;\n        if (ch * VEC < D) {\n";
    if (VEC > 1)
        ss << "          const dali_vec<" << t << ", VEC> d4 = dali_load<" << t << ", VEC>(drow + (long)ch * VEC);\n          _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) acc[u][j] = d4.v[j];\n";
    else
        ss << "          acc[u][0] = drow[(long)ch * dcs];\n";
    ss << "        }\n      }\n      fetch(" << (sorted ? "pm[p]" : "p") << ");\n    }\n";
    ss << "    combine();\n";
    if (sorted) {
        ss << "    for (int q = p + 1; q < q_end; ++q) { fetch(pm[q]); combine(); }\n";
    } else {
    ss << "    {\n      unsigned long long any = __ballot(m_own != 0);\n      while (any) {\n        const int l = __builtin_ctzll(any);\n        any &= any - 1;\n"
          "        const unsigned int ml = (unsigned int)__builtin_amdgcn_readlane((int)m_own, l);\n"
          "        for (int b = 0; b < 4; ++b) if ((ml >> b) & 1u) { fetch(p_lo + l * 4 + b); combine(); }\n      }\n    }\n";
    ss << "    _Pragma(\"unroll 4\") for (int base = p_lo + 256; base < N; base += 256) {\n"
          "      const dali_vec<int, 4> k4 = lk4[(base >> 2) + lane];\n"
          "      const unsigned long long a0 = __ballot(k4.v[0] == key), a1 = __ballot(k4.v[1] == key), a2 = __ballot(k4.v[2] == key), a3 = __ballot(k4.v[3] == key);\n"
          "      unsigned long long any = a0 | a1 | a2 | a3;\n"
          "      while (any) {  // rare: the lanes that found this index again, lowest position first\n"
          "        const int l = __builtin_ctzll(any);\n        any &= any - 1;\n"
          "        if ((a0 >> l) & 1ull) { fetch(base + l * 4); combine(); }\n        if ((a1 >> l) & 1ull) { fetch(base + l * 4 + 1); combine(); }\n"
          "        if ((a2 >> l) & 1ull) { fetch(base + l * 4 + 2); combine(); }\n        if ((a3 >> l) & 1ull) { fetch(base + l * 4 + 3); combine(); }\n      }\n    }\n";
    }
    ss << "    _Pragma(\"unroll\") for (int u = 0; u < U; ++u) {\n      const int ch = c0 / VEC + lane + 64 * u;\n      if (ch * VEC < D) {\n";
    if (VEC > 1)
        ss << "        dali_vec<" << t << ", VEC> d4;\n        _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) d4.v[j] = acc[u][j];\n        dali_store<" << t << ", VEC>(drow + (long)ch * VEC, d4);\n";
    else
        ss << "        drow[(long)ch * dcs] = acc[u][0];\n";
    ss << "      }\n    }\n  }\n}\n";
    return ss.str();
}

// dest2d: [V, D] view of the destination buffer; idx_c: contiguous int32 [N] buffer; values: an expression of [N, D] elements
// (or of one element) that a fused kernel can evaluate in place. False when this form does not apply.
// Index vectors beyond 16384 entries are ordered first (a stable sort by the library, on the library stream) and the same
// kernel then walks runs of equal indices instead of scanning LDS; the values stay an expression in both forms.
static void order_indices(const Array& idx_c, int N, int V, const Array& skeys, const Array& perm) {
    if (g_dry_run) return;
    check_hip(dali_hip_argsort_i32((const int32_t*)idx_c.device_ptr(), N, V, (int32_t*)skeys.device_ptr(memory::AM_OVERWRITE),
                                   (int32_t*)perm.device_ptr(memory::AM_OVERWRITE)),
              "index sort for scatter");
    if (g_recording) {
        note_recorded_write(skeys.expression()->memory);
        note_recorded_write(perm.expression()->memory);
        Array k1 = idx_c, k2 = skeys, k3 = perm;
        const int32_t* kp = (const int32_t*)idx_c.device_ptr();
        int32_t* sp = (int32_t*)skeys.device_ptr(memory::AM_MUTABLE);
        int32_t* pp = (int32_t*)perm.device_ptr(memory::AM_MUTABLE);
        g_recording->push_back([=]() {
            (void)k1;
            (void)k2;
            (void)k3;
            check_hip(dali_hip_argsort_i32(kp, N, V, sp, pp), "index sort replay");
        });
    }
}

static bool try_scatter_scan(const Array& dest2d, const Array& idx_c, OPERATOR_T op, const Array& values) {
    static const int scan_max = std::min(16384, env_int("DALI_HIP_SCATTER_SCAN_MAX", 16384));
    static const bool sorted_fused = env_int("DALI_HIP_SCATTER_SORTED_FUSED", 1) != 0;
    const int N = numel_of(idx_c.shape()), D = dest2d.shape()[1], V = dest2d.shape()[0];
    const bool sorted = N > scan_max;
    if ((sorted && !sorted_fused) || has_kind(values, [](Kind k) { return is_reduce(k) || is_all_reduce(k) || k == Kind::GATHER || k == Kind::GATHER_FROM_ROWS; }))
        return false;
    Domain dom;
    dom.R = N;
    dom.C = D;
    Program P;
    auto dst = strides_of(dest2d.expression().get());
    P.arrays.push_back(manual_arg(dest2d, Cls::FULL, true, 2, dest2d.shape(), {dst[0], dst[1]}));
    Array skeys, perm;
    if (sorted) {
        skeys = Array({N}, DTYPE_INT32);
        perm = Array({N}, DTYPE_INT32);
        P.arrays.push_back(manual_arg(skeys, Cls::ROW, false, 1, {N}, {}));
        P.arrays.push_back(manual_arg(perm, Cls::ROW, false, 1, {N}, {}));
    } else {
        P.arrays.push_back(manual_arg(idx_c, Cls::ROW, false, 1, {N}, {}));
    }
    const size_t first_operand = P.arrays.size();
    const bool one_value = numel_of(values.shape()) == 1;
    int root = add_node(P, values);
    if (!classify(P, root, one_value ? Cls::SCAL : Cls::FULL, dom)) return false;
    count_uses(P, {root});
    bool vec = D % 4 == 0 && dst[1] == 1 && dst[0] % 4 == 0 && dest2d.offset() % 4 == 0 && size_of_dtype(dest2d.dtype()) == 4;
    for (size_t i = first_operand; i < P.arrays.size(); ++i) {
        const ArrayArg& a = P.arrays[i];
        if (a.buf->memory.get() == dest2d.expression()->memory.get()) return false;  // values read from the destination: evaluate them first
        if (a.cls == Cls::FULL) vec = vec && a.col_stride == 1 && a.row_stride % 4 == 0 && a.buf->offset % 4 == 0 && size_of_dtype(a.buf->dtype) == 4;
    }
    const int VEC = vec ? 4 : 1;
    int KCAP = 1024;
    while (!sorted && KCAP < N) KCAP *= 2;
    std::vector<Output> outs(1);
    outs[0].root = root;
    outs[0].array = 0;
    outs[0].op = op;
    outs[0].cls = Cls::FULL;
    std::ostringstream params;
    params << (sorted ? "runs1," : "scan6,") << VEC << "," << KCAP;
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash("scatter", signature(P, outs), params.str());
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    std::vector<int> shape_ndims = {3};
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = "scatter";
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = 1024;
        K->plan.grid_kind = DALI_HIP_GRID_ROWS;  // one wave per input position, 16 to a workgroup
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = 1;
        K->plan.work_per_block = 16;
    }
    if (sorted) order_indices(idx_c, N, V, skeys, perm);
    std::vector<std::vector<int>> shapes = {{N, D, V}};
    load_and_launch(*K, [&]() { return gen_scatter_scan_kernel(P, L, op, root, VEC, KCAP, K->name, sorted); }, P, shapes);
    return true;
}

// Column numbers of the k best entries of every row of a dense [rows, cols] matrix, best first
// (dali/array/op/top_k.cpp:96-170). The ordering is a library call on the library stream, not a generated kernel.
static Array topk_rows_impl(const Array& x2d_in, int k, bool largest, bool ties_by_descending_column) {
    Array x2d = dense_buffer(x2d_in);
    const int rows = x2d.shape()[0], cols = x2d.shape()[1];
    Array out({rows, k}, DTYPE_INT32);
    if (rows == 0 || g_dry_run) return out;
    const void* xp = x2d.device_ptr();
    int32_t* op_ = (int32_t*)out.device_ptr(memory::AM_OVERWRITE);
    const int dtype = (int)x2d.dtype();
    check_hip(dali_hip_topk_rows(xp, dtype, rows, cols, k, largest, ties_by_descending_column, op_), "ordering of rows");
    if (g_recording) {
        note_recorded_write(out.expression()->memory);
        Array keep_x = x2d, keep_out = out;
        g_recording->push_back([=]() {
            (void)keep_x;
            (void)keep_out;
            check_hip(dali_hip_topk_rows(xp, dtype, rows, cols, k, largest, ties_by_descending_column, op_), "ordering of rows, replay");
        });
    }
    return out;
}

// dest2d: [V, D] view of the destination buffer; idx: int32 [N] buffer; values: [N, D] buffer or one element
static void run_scatter_rows(const Array& dest2d, const Array& idx, OPERATOR_T op, const Array& values) {
    const int N = numel_of(idx.shape()), D = dest2d.shape()[1], V = dest2d.shape()[0];
    if (N == 0 || D == 0) return;
    const bool scalar_value = numel_of(values.shape()) == 1;
    Array idx_c = idx.contiguous_memory() ? idx : idx.ascontiguousarray();
    // (rows narrower than a wave's 1 KiB gain nothing from the unrolled form: [1000000,128] with 262144 indices 155 against 170 us)
    if ((N <= 16384 || D >= 256) && try_scatter_scan(dest2d, idx_c, op, op::identity(values))) return;
    Array skeys({N}, DTYPE_INT32), perm({N}, DTYPE_INT32);
    order_indices(idx_c, N, V, skeys, perm);
    auto dst = strides_of(dest2d.expression().get());
    Program P;
    P.arrays.push_back(manual_arg(dest2d, Cls::FULL, true, 2, dest2d.shape(), {dst[0], dst[1]}));
    P.arrays.push_back(manual_arg(skeys, Cls::ROW, false, 1, {N}, {}));
    P.arrays.push_back(manual_arg(perm, Cls::ROW, false, 1, {N}, {}));
    bool vec = D % 4 == 0 && dst[1] == 1 && dst[0] % 4 == 0 && dest2d.offset() % 4 == 0;
    if (scalar_value) {
        P.arrays.push_back(manual_arg(values, Cls::SCAL, false, 1, {1}, {}));
    } else {
        auto vst = strides_of(values.expression().get());
        P.arrays.push_back(manual_arg(values, Cls::FULL, false, 2, {N, D}, {vst[0], vst[1]}));
        vec = vec && vst[1] == 1 && vst[0] % 4 == 0 && values.offset() % 4 == 0;
    }
    const int VEC = vec ? 4 : 1;
    std::ostringstream sig;
    sig << "scatter_rows_wave|" << (int)dest2d.dtype() << "|" << (int)op << "|" << scalar_value << "|" << VEC;
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash("scatter", sig.str(), "");
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    std::vector<int> shape_ndims = {3};
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = "scatter";
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = 1024;
        K->plan.grid_kind = DALI_HIP_GRID_ROWS;  // one wave per sorted position, 16 to a workgroup
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = 1;
        K->plan.work_per_block = 16;
    }
    std::vector<std::vector<int>> shapes = {{N, D, V}};
    load_and_launch(*K, [&]() { return gen_scatter_rows_kernel(P, L, op, scalar_value, VEC, K->name); }, P, shapes);
}

// Assignment through gather_from_rows: dest[i, indices[i]] (op)= values[i]; one element per row, so no two
// contributions meet (dali/array/op/gather_from_rows.cpp:41-51,66-78).
static std::string gen_scatter_to_rows_kernel(const Program& P, const IvLayout& L, OPERATOR_T op, bool scalar_value, const std::string& kname) {
    std::string t = ctype(P.arrays[0].buf->dtype);
    std::ostringstream ss;
    ss << device_prelude();
    ss << kargs_struct(P, L);
    ss << "extern \"C\" __global__ __launch_bounds__(256) void " << kname << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n";
    ss << "  const long N = A.iv[" << L.shape_pos[0] << "];\n";
    ss << "  const long drs = A.iv[" << L.stride_pos[0] << "], dcs = A.iv[" << L.stride_pos[0] + 1 << "];\n";
    ss << "  const long is = A.iv[" << L.stride_pos[1] << "];\n";
    if (!scalar_value) ss << "  const long vs = A.iv[" << L.stride_pos[2] << "];\n";
    ss << "  const int cols = A.iv[" << L.shape_pos[0] + 1 << "];\n";
    ss << "  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < N; i += (long)gridDim.x * 256) {\n";
    ss << "    const int pick = ((const int*)A.p[1])[i * is];\n    if ((unsigned)pick >= (unsigned)cols) continue;  // no such column: skipped\n";
    ss << "    " << t << "* d = (" << t << "*)A.p[0] + i * drs + (long)pick * dcs;\n";
    ss << "    const " << t << " v = ((const " << t << "*)A.p[2])[" << (scalar_value ? "0" : "i * vs") << "];\n";
    ss << "    *d = " << op_combine(op, "(*d)", "v") << ";\n  }\n}\n";
    return ss.str();
}

static void run_scatter_to_rows(const Array& dest2d, const Array& idx, OPERATOR_T op, const Array& values) {
    const int N = numel_of(idx.shape());
    if (N == 0) return;
    const bool scalar_value = numel_of(values.shape()) == 1;
    auto dst = strides_of(dest2d.expression().get());
    auto ist = strides_of(idx.expression().get());
    Program P;
    P.arrays.push_back(manual_arg(dest2d, Cls::FULL, true, 2, dest2d.shape(), {dst[0], dst[1]}));
    P.arrays.push_back(manual_arg(idx, Cls::ROW, false, 1, {N}, {ist.empty() ? 1 : ist[0]}));
    if (scalar_value) {
        P.arrays.push_back(manual_arg(values, Cls::SCAL, false, 1, {1}, {}));
    } else {
        auto vst = strides_of(values.expression().get());
        P.arrays.push_back(manual_arg(values, Cls::ROW, false, 1, {N}, {vst.empty() ? 1 : vst[0]}));
    }
    std::ostringstream sig;
    sig << "scatter_to_rows_guarded|" << (int)dest2d.dtype() << "|" << (int)op << "|" << scalar_value;
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash("scatter", sig.str(), "");
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    std::vector<int> shape_ndims = {2};
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = "scatter";
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = 256;
        K->plan.grid_kind = DALI_HIP_GRID_ELEMS;
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = 1;
        K->plan.work_per_block = 256;
        K->plan.max_blocks = 65536;
    }
    std::vector<std::vector<int>> shapes = {{N, dest2d.shape()[1]}};
    load_and_launch(*K, [&]() { return gen_scatter_to_rows_kernel(P, L, op, scalar_value, K->name); }, P, shapes);
}

// dest is a lazy gather / gather_from_rows node over a buffer: write through it
void scatter_assign(const Array& dest, OPERATOR_T op, const Array& source) {
    auto de = dest.expression();
    if (!de->origin.empty()) {
        // The rows of the destination view are not contiguous pieces of memory (strided trailing axes): the rows are
        // scattered into a dense copy taken now, which then goes back into the view. (The reference indexes such a view
        // element by element, dali/array/op/gather.cpp:89-97; here the kernels want [V, D] rows.)
        const Array view = de->origin[0];
        Array dense = view.reshape({view.shape()[0], -1});
        DALI_ASSERT(dense.is_buffer(), "internal: the dense form of a scatter destination is not a buffer");
        Array through = op::gather(dense, de->args[1]);
        scatter_assign(through, op, source);
        evaluate_into(view, OPERATOR_T_EQL, dense.reshape(view.shape()));
        return;
    }
    Array target = de->args[0], idx = de->args[1];
    DALI_ASSERT(target.is_buffer(), "assignment through a gather needs an evaluated buffer as its source (dali/array/op/gather.cpp:126-128)");
    if (!idx.is_buffer()) idx.eval();
    Array values = source;
    if (values.dtype() != dest.dtype()) values = op::astype(values, dest.dtype());
    const int64_t n_dest = numel_of(dest.shape());
    DALI_ASSERT(numel_of(values.shape()) == 1 || numel_of(values.shape()) == n_dest,
                make_message("Cannot assign result of shape ", shape_str(values.shape()), " to a location of shape ", shape_str(dest.shape()), "."));
    if (values.expression()->kind == Kind::SCALAR) values = op::identity(values);  // scalars have no buffer of their own
    if (de->kind == Kind::GATHER && !values.is_buffer()) {
        // the values stay an expression when the scan form of the scatter can evaluate them where they are used
        const int N = numel_of(idx.shape()), D = target.shape()[1];
        ExprMemo memo;
        Array lazy = clean(values, memo, true);
        const bool shaped = numel_of(lazy.shape()) == 1 || (lazy.ndim() == 2 && lazy.shape()[0] == N && lazy.shape()[1] == D);
        if (shaped && !lazy.is_buffer() && lazy.expression()->kind != Kind::SCALAR) {
            jit_stats().evals++;
            jit_stats().last_kernel_kinds.clear();
            jit_stats().last_kernel_names.clear();
            g_last_source.clear();
            Array idx_c = idx.contiguous_memory() ? idx : idx.ascontiguousarray();
            if (try_scatter_scan(target, idx_c, op, lazy)) return;
        }
    }
    values.eval();
    DALI_ASSERT(values.is_buffer(), "internal: scatter values were not evaluated into a buffer");
    if (de->kind == Kind::GATHER) {
        const int N = numel_of(idx.shape()), D = target.shape()[1];
        if (numel_of(values.shape()) != 1) values = values.reshape({N, D});
        run_scatter_rows(target, idx, op, values);
    } else {
        DALI_ASSERT(target.ndim() == 2 && idx.ndim() == 1, "assignment through gather_from_rows is implemented for 2-D sources and 1-D indices");
        if (numel_of(values.shape()) != 1) values = values.reshape({(int)n_dest});
        run_scatter_to_rows(target, idx, op, values);
    }
}

}  // namespace jit

using namespace jit;

Array topk_rows(const Array& x2d, int k, bool largest, bool ties_by_descending_column) {
    return topk_rows_impl(x2d, k, largest, ties_by_descending_column);
}

}  // namespace dali
