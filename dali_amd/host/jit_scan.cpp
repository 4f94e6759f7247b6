// Prefix scans along the trailing axis and the circular convolution (dali/array/op/circular_convolution.cpp).
#include "jit_internal.h"

namespace dali {
namespace jit {

// Running reduction along the trailing axis (dali/array/op/scan.cpp:19-194): inclusive keeps the shape, exclusive
// appends one element (out[0] = init, out[i + 1] = reduce(in[0..i])). A row is scanned by TPR threads in pieces of
// TPR * VEC elements: a thread scans its VEC elements, the wave scans the thread totals with shuffles, waves meet
// through LDS, and the total of the piece is carried to the next one. Everything is combined left to right.
// MODE 0: one row per TPR threads. Few long rows are cut into S segments of SL elements so that the whole chip
// works on them: MODE 1 reduces every segment to its total (one workgroup per segment), MODE 2 scans a segment
// starting from the fold of the totals in front of it.
static std::string gen_scan_kernel(const Program& P, const IvLayout& L, const std::string& reducer, bool inclusive, int VEC, bool vec_store, int TPR,
                            int MODE, const std::string& kname) {
    std::string t = ctype(P.arrays[0].buf->dtype);
    const int BT = 256, RPB = BT / TPR, NW = TPR / 64, EX = inclusive ? 0 : 1;
    const int SRC = MODE == 1 ? 1 : (MODE == 2 ? 1 : 1);
    std::ostringstream ss;
    ss << device_prelude();
    ss << kargs_struct(P, L);
    ss << "extern \"C\" __global__ __launch_bounds__(" << BT << ") void " << kname << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n";
    ss << "  typedef " << reducer << " Rd;\n  typedef " << t << " T;\n";
    ss << "  constexpr int VEC = " << VEC << ", TPR = " << TPR << ", RPB = " << RPB << ", NW = " << NW << ", EX = " << EX << ";\n";
    ss << "  const int tr = threadIdx.x % TPR, rib = threadIdx.x / TPR, lane = threadIdx.x & 63, wv = tr >> 6; (void)rib; (void)wv; (void)lane;\n";
    if (MODE == 0) {
        ss << "  const long R = A.iv[" << L.shape_pos[0] << "], C = A.iv[" << L.shape_pos[0] + 1 << "];\n";
        ss << "  long row = (long)blockIdx.x * RPB + rib;\n  const bool row_ok = row < R;\n  if (!row_ok) row = R - 1;\n";
        ss << "  const long c_begin = 0, c_end = C;\n";
    } else {
        // shape: {R * S, C, S, SL}
        ss << "  const long C = A.iv[" << L.shape_pos[0] + 1 << "], S = A.iv[" << L.shape_pos[0] + 2 << "], SL = A.iv[" << L.shape_pos[0] + 3 << "];\n";
        ss << "  const long row = blockIdx.x / S, seg = blockIdx.x % S;\n  const bool row_ok = true; (void)row_ok;\n";
        ss << "  const long c_begin = seg * SL, c_end = c_begin + SL < C ? c_begin + SL : C;\n";
    }
    ss << "  const T* src = (const T*)A.p[" << SRC << "] + row * (long)A.iv[" << L.stride_pos[SRC] << "];\n";
    if (MODE == 1) {
        // segment total: thread-strided accumulation, then the block fold
        ss << "  T acc = Rd::init<T>();\n";
        ss << "  for (long c0 = c_begin + (long)tr * VEC; c0 < c_end; c0 += TPR * VEC) {\n";
        if (VEC > 1)
            ss << "    if (c0 + VEC <= c_end) {\n      const dali_vec<T, VEC> tmp = dali_load<T, VEC>(src + c0);\n"
                  "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) acc = Rd::step<T>(acc, tmp.v[j]);\n    } else {\n"
                  "      for (int j = 0; j < VEC; ++j) if (c0 + j < c_end) acc = Rd::step<T>(acc, src[c0 + j]);\n    }\n";
        else
            ss << "    acc = Rd::step<T>(acc, src[c0]);\n";
        ss << "  }\n  __shared__ T smr[NW];\n  const T total = dali_block_reduce<Rd, T, NW>(acc, smr);\n";
        ss << "  if (threadIdx.x == 0) ((T*)A.p[0])[row * S + seg] = total;\n}\n";
        return ss.str();
    }
    ss << "  T* dst = (T*)A.p[0] + row * (C + EX);\n";
    if (NW > 1) ss << "  __shared__ T sm[RPB][NW];\n";
    ss << "  T carry = Rd::init<T>();\n";
    if (MODE == 2) {
        ss << "  { const T* totals = (const T*)A.p[2] + row * S;\n    for (long q = 0; q < seg; ++q) carry = Rd::step<T>(carry, totals[q]); }\n";
        ss << "  if (EX && seg == 0 && tr == 0) dst[0] = Rd::init<T>();\n";
    } else {
        ss << "  if (EX && row_ok && tr == 0) dst[0] = carry;\n";
    }
    ss << "  for (long base = c_begin; base < c_end; base += TPR * VEC) {\n";
    ss << "    const long c0 = base + (long)tr * VEC;\n    T v[VEC];\n";
    if (VEC > 1) {
        ss << "    if (c0 + VEC <= c_end) {\n      const dali_vec<T, VEC> tmp = dali_load_nt<T, VEC>(src + c0);\n"
              "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) v[j] = tmp.v[j];\n    } else {\n"
              "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) v[j] = c0 + j < c_end ? src[c0 + j] : Rd::init<T>();\n    }\n";
    } else {
        ss << "    v[0] = c0 < c_end ? src[c0] : Rd::init<T>();\n";
    }
    ss << "    _Pragma(\"unroll\") for (int j = 1; j < VEC; ++j) v[j] = Rd::step<T>(v[j - 1], v[j]);\n";
    if (TPR < 64) {
        // several short rows to a wave: the scan of the thread totals stops at the first lane of every row
        ss << "    T incl = v[VEC - 1];\n    _Pragma(\"unroll\") for (int d = 1; d < TPR; d <<= 1) {\n      const T o = dali_shfl_up<T>(incl, d);\n"
              "      if ((lane & (TPR - 1)) >= d) incl = Rd::step<T>(o, incl);\n    }\n";
        ss << "    T excl = dali_shfl_up<T>(incl, 1);\n    if ((lane & (TPR - 1)) == 0) excl = Rd::init<T>();\n";
    } else {
        ss << "    const T incl = dali_wave_scan<Rd, T>(v[VEC - 1]);\n";
        ss << "    T excl = dali_shfl_up<T>(incl, 1);\n    if (lane == 0) excl = Rd::init<T>();\n";
    }
    ss << "    T off = carry;\n";
    if (NW > 1) {
        ss << "    if (lane == 63) sm[rib][wv] = incl;\n    __syncthreads();\n    T total = Rd::init<T>();\n";
        ss << "    _Pragma(\"unroll\") for (int w = 0; w < NW; ++w) {\n      const T wt = sm[rib][w];\n      if (w < wv) off = Rd::step<T>(off, wt);\n"
              "      total = Rd::step<T>(total, wt);\n    }\n    carry = Rd::step<T>(carry, total);\n    __syncthreads();\n";
    } else if (TPR < 64) {
        ss << "    carry = Rd::step<T>(carry, dali_shfl<T>(incl, lane | (TPR - 1)));\n";
    } else {
        ss << "    carry = Rd::step<T>(carry, dali_shfl<T>(incl, 63));\n";
    }
    ss << "    off = Rd::step<T>(off, excl);\n";
    ss << "    _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) v[j] = Rd::step<T>(off, v[j]);\n";
    ss << "    if (row_ok) {\n";
    if (vec_store) {
        ss << "      if (c0 + VEC <= c_end) {\n        dali_vec<T, VEC> o;\n        _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) o.v[j] = v[j];\n"
              "        dali_store_nt<T, VEC>(dst + c0, o);\n      } else {\n"
              "        _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) if (c0 + j < c_end) dst[c0 + j] = v[j];\n      }\n";
    } else {
        ss << "      _Pragma(\"unroll\") for (int j = 0; j < VEC; ++j) if (c0 + j < c_end) dst[EX + c0 + j] = v[j];\n";
    }
    ss << "    }\n  }\n}\n";
    return ss.str();
}

Array run_scan(const Array& arg_in, const std::string& reducer, bool inclusive) {
    Array arg = arg_in;
    if (!arg.is_buffer()) arg = materialize(arg);
    std::vector<int> in_shape = arg.shape();
    if (in_shape.empty()) in_shape = {1};
    const int C = in_shape.back();
    const int64_t R = C ? numel_of(in_shape) / C : 0;
    std::vector<int> out_shape = in_shape;
    if (!inclusive) out_shape.back() += 1;
    if (arg.shape().empty() && inclusive) out_shape = {};
    Array dest(out_shape, arg.dtype());
    if (R == 0) return dest;
    // rows with unit column stride and one row stride; anything else is copied first
    auto st = strides_of(arg.expression().get());
    int64_t rs = C;
    bool fits = arg.shape().empty() || st.back() == 1 || C == 1;
    if (fits && arg.ndim() > 1) fits = collapse_dims(arg.shape(), st, arg.ndim() - 1, &rs);
    if (!fits) {
        arg = arg.ascontiguousarray();
        rs = C;
    }
    if (R == 1) rs = C;
    const int el = size_of_dtype(arg.dtype());
    const bool vec_load = C % 4 == 0 && rs % 4 == 0 && arg.offset() % 4 == 0 && el <= 8;
    const int VEC = vec_load ? 4 : 1;
    const bool vec_store = vec_load && inclusive;
    // few long rows: cut them into segments, about two thousand workgroups in all (the input is then read twice)
    static const int seg_env = env_int("DALI_HIP_SCAN_SEGMENTS", -1);
    const int piece = 256 * VEC;
    int64_t S = 1;
    if (R < 1024 && C >= 16 * piece) S = std::min<int64_t>((2048 + R - 1) / R, C / (4 * piece));
    if (seg_env >= 0) S = seg_env > 0 ? seg_env : 1;
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    auto launch = [&](int MODE, int TPR, Program& P, const std::vector<int>& shape) {
        std::ostringstream sig;
        sig << "scan|" << reducer << "|" << (int)arg.dtype() << "|" << inclusive << "|" << VEC << "|" << vec_store << "|" << TPR << "|" << MODE;
        uint64_t h = kernel_hash("scan", sig.str(), "");
        std::shared_ptr<KernelSpec>& K = specs_cache[h];
        std::vector<int> shape_ndims = {(int)shape.size()};
        IvLayout L = layout_iv(P, shape_ndims);
        if (!K) {
            K = std::make_shared<KernelSpec>();
            K->hash = h;
            K->kind = "scan";
            K->name = kernel_name(K->kind, h);
            fill_plan_arrays(*K, P, shape_ndims);
            K->plan.block_threads = 256;
            K->plan.grid_kind = DALI_HIP_GRID_ROWS;
            K->plan.work_begin = L.shape_pos[0];
            K->plan.work_count = 1;
            K->plan.work_per_block = 256 / TPR;
        }
        std::vector<std::vector<int>> shapes = {shape};
        load_and_launch(*K, [&]() { return gen_scan_kernel(P, L, reducer, inclusive, VEC, vec_store, TPR, MODE, K->name); }, P, shapes);
    };
    if (S <= 1) {
        Program P;
        P.arrays.push_back(manual_arg(dest, Cls::FULL, true, 2, {(int)R, C + (inclusive ? 0 : 1)}, {}));
        P.arrays.push_back(manual_arg(arg, Cls::FULL, false, 2, {(int)R, C}, {(int)rs, 1}));
        int TPR = (int64_t)C <= 64 * VEC * 4 ? 64 : 256;
        // rows shorter than a wave's vectors: as many threads per row as the row has vectors (four at least), so that a
        // wave scans several rows at once and reads them as one contiguous run ([9999999,7]: 1475 us with a wave per row)
        static const bool short_rows = env_int("DALI_HIP_SCAN_SHORT_ROWS", 1) != 0;
        if (short_rows && (int64_t)C <= 32 * VEC) {
            TPR = 4;
            while (TPR * VEC < C) TPR *= 2;
        }
        launch(0, TPR, P, {(int)R, C});
        return dest;
    }
    int64_t SL = (C + S - 1) / S;
    SL = (SL + piece - 1) / piece * piece;
    S = (C + SL - 1) / SL;
    Array totals({(int)R, (int)S}, arg.dtype());
    {
        Program P;
        P.arrays.push_back(manual_arg(totals, Cls::FULL, true, 2, {(int)R, (int)S}, {}));
        P.arrays.push_back(manual_arg(arg, Cls::FULL, false, 2, {(int)R, C}, {(int)rs, 1}));
        launch(1, 256, P, {(int)(R * S), C, (int)S, (int)SL});
    }
    {
        Program P;
        P.arrays.push_back(manual_arg(dest, Cls::FULL, true, 2, {(int)R, C + (inclusive ? 0 : 1)}, {}));
        P.arrays.push_back(manual_arg(arg, Cls::FULL, false, 2, {(int)R, C}, {(int)rs, 1}));
        P.arrays.push_back(manual_arg(totals, Cls::FULL, false, 2, {(int)R, (int)S}, {}));
        launch(2, 256, P, {(int)(R * S), C, (int)S, (int)SL});
    }
    return dest;
}

// out[r, x] = sum over s of content[r, (x + s) mod n] * weights[r, s] (dali/array/op/circular_convolution.cpp:22-38).
// One workgroup per row keeps the row of both operands in LDS; a thread owns outputs x = tid, tid + 256, ... and
// walks s upwards, so every output is the same left-to-right fp32 sum as the reference's loop. The content reads of
// a wave are consecutive LDS words, the weight is a broadcast.
Array run_circular_convolution(const Array& x_in, const Array& w_in) {
    Array x = x_in, w = w_in;
    if (!x.is_buffer()) x = materialize(x);
    if (!w.is_buffer()) w = materialize(w);
    if (!x.contiguous_memory()) x = x.ascontiguousarray();
    if (!w.contiguous_memory()) w = w.ascontiguousarray();
    Array dest(x.shape(), x.dtype());
    const int n = x.shape().back();
    const int64_t R = n ? numel_of(x.shape()) / n : 0;
    if (R == 0 || n == 0) return dest;
    const int el = size_of_dtype(x.dtype());
    DALI_ASSERT((int64_t)2 * n * el <= 128 * 1024, make_message("circular_convolution: rows of ", n, " elements do not fit the on-chip staging (limit ", 64 * 1024 / el, ")"));
    Program P;
    P.arrays.push_back(manual_arg(dest, Cls::FULL, true, 2, {(int)R, n}, {}));
    P.arrays.push_back(manual_arg(x, Cls::FULL, false, 2, {(int)R, n}, {}));
    P.arrays.push_back(manual_arg(w, Cls::FULL, false, 2, {(int)R, n}, {}));
    std::string t = ctype(x.dtype());
    std::ostringstream sig;
    int CAP = 256;  // LDS capacity of the specialisation, in elements per operand row
    while (CAP < n) CAP *= 2;
    sig << "circconv|" << (int)x.dtype() << "|" << CAP;
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash("circconv", sig.str(), "");
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    std::vector<int> shape_ndims = {2};
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = "circconv";
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = 256;
        K->plan.grid_kind = DALI_HIP_GRID_ROWS;
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = 1;
        K->plan.work_per_block = 1;
    }
    load_and_launch(*K, [&]() {
        std::ostringstream ss;
        ss << device_prelude() << kargs_struct(P, L);
        ss << "extern \"C\" __global__ __launch_bounds__(256) void " << K->name << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n  typedef " << t << " T;\n";
        ss << "  __shared__ T c[" << CAP << "];\n  __shared__ T w[" << CAP << "];\n";
        ss << "  const int n = A.iv[" << L.shape_pos[0] + 1 << "];\n  const long row = blockIdx.x;\n";
        ss << "  const T* cg = (const T*)A.p[1] + row * n;\n  const T* wg = (const T*)A.p[2] + row * n;\n";
        ss << "  for (int i = threadIdx.x; i < n; i += 256) { c[i] = cg[i]; w[i] = wg[i]; }\n  __syncthreads();\n";
        ss << "  T* out = (T*)A.p[0] + row * n;\n";
        ss << "  for (int x = threadIdx.x; x < n; x += 256) {\n    T res = (T)0;\n    int off = x;\n";
        ss << "    for (int s = 0; s < n; ++s) {\n      res += c[off] * w[s];\n      off = off + 1 == n ? 0 : off + 1;\n    }\n    out[x] = res;\n  }\n}\n";
        return ss.str();
    }, P, {{(int)R, n}});
    return dest;
}

}  // namespace jit

}  // namespace dali
