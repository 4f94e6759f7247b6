// Sliding-window kernels (dali/array/op/im2col.cpp, col2im.cpp, spatial_utils.cpp, pool2d): im2col, col2im, pooling
// forward and backward, and the direct NHWC convolution.
#include "jit_internal.h"

namespace dali {
namespace jit {

static ImageGeom image_geom(const std::vector<int>& shape, const std::string& fmt) {
    ImageGeom g;
    const char letters[4] = {'N', 'C', 'H', 'W'};
    std::vector<int> st = contiguous_strides(shape);
    for (int k = 0; k < 4; ++k) {
        const int pos = (int)fmt.find(letters[k]);
        g.ext[k] = shape[pos];
        g.stride[k] = st[pos];
    }
    return g;
}

Array dense_buffer(const Array& a) {
    Array b = a.is_buffer() ? a : materialize(a);
    return b.contiguous_memory() ? b : b.ascontiguousarray();
}

// q = n / D, r = n % D in generated source
std::string divmod(const std::string& q, const std::string& r, const std::string& n, const std::string& D) {
    return "const unsigned " + q + " = dali_udiv(" + n + ", " + D + "_M, " + D + "_S); const int " + r + " = (int)(" + n + " - " + q + " * (unsigned)" + D + ");";
}

// The letters other than N, last to first: the digits of a patch-row index, fastest first
// (dali/array/op/im2col.cpp:76-80 for N in position 0 or 1, where those lines name three different letters).
static std::string row_letters(const std::string& fmt) {
    std::string r;
    for (int p = 3; p >= 0; --p)
        if (fmt[p] != 'N') r.push_back(fmt[p]);
    return r;
}

static const char* row_digit_extent(char letter) { return letter == 'C' ? "C" : (letter == 'H' ? "FH" : "FW"); }

static const char* row_digit_name(char letter) { return letter == 'C' ? "c" : (letter == 'H' ? "kh" : "kw"); }

// Source text: `row` -> c, kh, kw (im2col.cpp:93-110) and back (col2im.cpp:86-94)
static std::string emit_split_row(const std::string& fmt, const std::string& row) {
    std::string l = row_letters(fmt), out;
    out += "      " + divmod("rq1_", row_digit_name(l[0]), "(unsigned)(" + row + ")", row_digit_extent(l[0])) + "\n";
    out += "      " + divmod("rq2_", row_digit_name(l[1]), "rq1_", row_digit_extent(l[1])) + "\n";
    out += std::string("      const int ") + row_digit_name(l[2]) + " = (int)rq2_;\n";
    return out;
}

static std::string emit_join_row(const std::string& fmt) {
    std::string l = row_letters(fmt), expr;
    for (int k = 2; k >= 0; --k) expr = expr.empty() ? row_digit_name(l[k]) : "(" + expr + ") * " + row_digit_extent(l[k]) + " + " + row_digit_name(l[k]);
    return expr;
}

// Element loop of the per-element sliding-window kernels. Workgroups are dealt to the eight XCDs round-robin;
// renumbering them gives every XCD one contiguous band of the index range, so that neighbours which share input rows
// (overlapping windows, the patches over a pixel) find them in the same L2 instead of fetching them once per XCD.
const char* const kBandedElementLoop =
    "  const unsigned nb_ = gridDim.x, vb_ = nb_ % 8u == 0 ? (blockIdx.x % 8u) * (nb_ / 8u) + blockIdx.x / 8u : blockIdx.x;\n"
    "  for (unsigned i = vb_ * 256u + threadIdx.x; i < total; i += nb_ * 256u) {\n";

// One launch of a hand-laid-out kernel: `blocks` workgroups of 256 threads (the kernels stride over blocks, so a
// capped grid still covers the work); the geometry travels as the integers behind the arrays' sizes.
void launch_special(const char* kind, const std::string& sig, const Program& P, int64_t blocks, const GeomInts& G,
                    const std::function<void(std::ostringstream&)>& body) {
    static std::unordered_map<uint64_t, std::shared_ptr<KernelSpec>> specs_cache;
    uint64_t h = kernel_hash(kind, sig, "");
    std::shared_ptr<KernelSpec>& K = specs_cache[h];
    std::vector<int> shape_ndims = {2, (int)G.values.size()};
    IvLayout L = layout_iv(P, shape_ndims);
    if (!K) {
        K = std::make_shared<KernelSpec>();
        K->hash = h;
        K->kind = kind;
        K->name = kernel_name(K->kind, h);
        fill_plan_arrays(*K, P, shape_ndims);
        K->plan.block_threads = 256;
        K->plan.grid_kind = DALI_HIP_GRID_ELEMS;
        K->plan.work_begin = L.shape_pos[0];
        K->plan.work_count = 2;
        K->plan.work_per_block = 256;
        K->plan.max_blocks = 1 << 20;
    }
    const int nblocks = (int)std::min<int64_t>(std::max<int64_t>(blocks, 1), 1 << 20);
    load_and_launch(*K, [&]() {
        std::ostringstream ss;
        ss << device_prelude() << kargs_struct(P, L);
        ss << "extern \"C\" __global__ __launch_bounds__(256) void " << K->name << "(DALI_KERNEL_PARAMS) {\n  DALI_KERNEL_ARGS\n  typedef " << ctype(P.arrays[0].buf->dtype) << " T;\n";
        for (size_t k = 0; k < G.names.size(); ++k) {
            const bool mult = G.names[k].size() > 2 && G.names[k].compare(G.names[k].size() - 2, 2, "_M") == 0;
            ss << "  const " << (mult ? "unsigned " : "int ") << G.names[k] << " = " << (mult ? "(unsigned)" : "") << "A.iv[" << L.shape_pos[1] + k
               << "]; (void)" << G.names[k] << ";\n";
        }
        body(ss);
        return ss.str();
    }, P, {{nblocks, 256}, G.values});
}

// Source text: index `i` of a dense array in `fmt` order whose innermost dimension is taken in groups of VEC
// -> n, c and the two spatial coordinates. `eh` / `ew` name the extents of the H and W positions.
static std::string emit_decompose(const std::string& fmt, const std::string& eh, const std::string& ew, const std::string& nh, const std::string& nw,
                           bool inner_groups) {
    std::ostringstream ss;
    auto ext = [&](int p) { return fmt[p] == 'N' ? std::string("N") : (fmt[p] == 'C' ? std::string("C") : (fmt[p] == 'H' ? eh : ew)); };
    ss << "    " << divmod("dq3_", "q3", "i", inner_groups ? "INNER_GROUPS" : ext(3)) << "\n";
    ss << "    " << divmod("dq2_", "q2", "dq3_", ext(2)) << "\n";
    ss << "    " << divmod("dq1_", "q1", "dq2_", ext(1)) << "\n";
    ss << "    const int q0 = (int)dq1_;\n";
    const char* qn[4] = {"q0", "q1", "q2", "q3"};
    auto coord = [&](char letter) {
        const int p = (int)fmt.find(letter);
        return p == 3 && inner_groups ? std::string("q3 * VEC") : std::string(qn[p]);
    };
    ss << "    const int n = " << coord('N') << ", c = " << coord('C') << ", " << nh << " = " << coord('H') << ", " << nw << " = " << coord('W') << ";\n";
    return ss.str();
}

static bool four_byte_vectors(DType dtype, const Array& a, int inner) { return size_of_dtype(dtype) == 4 && inner % 4 == 0 && a.offset() % 4 == 0; }

// im2col. Two layouts of the same matrix, chosen so that both the gather and the store run along memory:
//  - formats ending in "WC" (NHWC): for a patch and a filter row kh, the filter_w * C values are one contiguous
//    run of the image, and they are consecutive rows (kh, kw, c) of one column. The matrix is stored patch-major
//    ([N*out_h*out_w, filter_h*filter_w*C], returned as its transposed view): one wave copies one patch, whose
//    position is computed once, on the scalar unit.
//  - every other format: row-major [filter_h*filter_w*C, N*out_h*out_w]; a thread owns a column (consecutive
//    columns are consecutive output pixels, i.e. consecutive W) and walks a group of rows, whose decomposition
//    into (c, kh, kw) is the same for the whole workgroup.
Array run_im2col(const Expr& e, const Array& image_in) {
    Array image = dense_buffer(image_in);
    const std::string& fmt = e.data_format;
    ImageGeom g = image_geom(image.shape(), fmt);
    const int fh = e.geom[0], fw = e.geom[1], sth = e.geom[2], stw = e.geom[3], dh = e.geom[4], dw = e.geom[5];
    const int o_h = (g.ext[2] + e.geom[6] + e.geom[8] - (dh * (fh - 1) + 1)) / sth + 1;
    const int o_w = (g.ext[3] + e.geom[7] + e.geom[9] - (dw * (fw - 1) + 1)) / stw + 1;
    const int64_t rows = e.shape[0], cols = e.shape[1];
    DALI_ASSERT(rows == (int64_t)fh * fw * g.ext[1] && cols == (int64_t)g.ext[0] * o_h * o_w, "internal: im2col shape does not match its geometry");
    const bool patch_major = fmt[2] == 'W' && fmt[3] == 'C' && dh == 1 && dw == 1;
    Array store = patch_major ? Array({(int)cols, (int)rows}, e.dtype) : Array({(int)rows, (int)cols}, e.dtype);
    Array result = patch_major ? store.transpose() : store;
    if (rows * cols == 0) return result;
    DALI_ASSERT(rows * cols < ((int64_t)1 << 31), "im2col: the patch matrix must hold fewer than 2^31 elements");
    Program P;
    P.arrays.push_back(manual_arg(store, Cls::FULL, true, 2, store.shape(), {}));
    P.arrays.push_back(manual_arg(image, Cls::FULL, false, 1, {(int)numel_of(image.shape())}, {}));
    GeomInts G;
    G.add_image(g);
    G.add_div("FH", fh);
    G.add_div("FW", fw);
    G.add("STH", sth);
    G.add("STW", stw);
    G.add("DH", dh);
    G.add("DW", dw);
    G.add("PH", e.geom[6]);
    G.add("PW", e.geom[7]);
    G.add_div("OH", o_h);
    G.add_div("OW", o_w);
    if (patch_major) {
        const int VEC = four_byte_vectors(e.dtype, image, g.ext[1]) ? 4 : 1;
        G.add_div("RUN", fw * g.ext[1]);
        std::ostringstream sig;
        sig << "im2col_wc|" << (int)e.dtype << "|" << VEC;
        launch_special("im2col", sig.str(), P, (cols + 3) / 4, G, [&](std::ostringstream& ss) {
            ss << "  constexpr int VEC = " << VEC << ";\n";
            ss << "  T* out = (T*)A.p[0];\n  const T* img = (const T*)A.p[1];\n";
            ss << "  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);\n";
            ss << "  const unsigned cols = (unsigned)(N * OH * OW);\n  const int rows = FH * RUN;\n";
            ss << "  for (unsigned col = blockIdx.x * 4u + wave; col < cols; col += gridDim.x * 4u) {\n";
            ss << "    " << divmod("t1", "ow", "col", "OW") << "\n";
            ss << "    " << divmod("n", "oh", "t1", "OH") << "\n";
            ss << "    const int h0 = oh * STH - PH, w0 = ow * STW - PW;\n";
            ss << "    // a run covers image columns w0 .. w0 + FW - 1 of one image row: element j is valid when that column lies inside the image\n";
            ss << "    const int jlo = w0 < 0 ? -w0 * C : 0, jhi = (W - w0) * C < RUN ? (W - w0) * C : RUN;\n";
            ss << "    T* dst = out + (long)col * rows;\n";
            ss << "    const T* src0 = img + (long)n * SN + (long)w0 * C;\n";
            ss << "    for (int e = lane * VEC; e < rows; e += 64 * VEC) {\n";
            ss << "      " << divmod("kh", "j", "(unsigned)e", "RUN") << "\n";
            ss << "      const int h = h0 + (int)kh;\n";
            ss << "      dali_vec<T, VEC> v;\n";
            ss << "      if (h >= 0 && h < H && j >= jlo && j < jhi) v = dali_load<T, VEC>(src0 + (long)h * SH + j);\n";
            ss << "      else { _Pragma(\"unroll\") for (int k = 0; k < VEC; ++k) v.v[k] = (T)0; }\n";
            ss << "      dali_store_nt<T, VEC>(dst + e, v);\n    }\n  }\n}\n";
        });
    } else {
        const int RB = 16;  // rows per workgroup
        const int64_t col_tiles = (cols + 255) / 256, row_groups = (rows + RB - 1) / RB;
        G.add_div("COL_TILES", (int)col_tiles);
        std::ostringstream sig;
        sig << "im2col_rows|" << (int)e.dtype << "|" << row_letters(fmt);
        launch_special("im2col", sig.str(), P, col_tiles * row_groups, G, [&](std::ostringstream& ss) {
            ss << "  constexpr int RB = " << RB << ";\n";
            ss << "  T* out = (T*)A.p[0];\n  const T* img = (const T*)A.p[1];\n";
            ss << "  const unsigned cols = (unsigned)(N * OH * OW); const int rows = FH * FW * C;\n";
            ss << "  const unsigned total = (unsigned)COL_TILES * (unsigned)((rows + RB - 1) / RB);\n";
            ss << "  for (unsigned b = blockIdx.x; b < total; b += gridDim.x) {\n";
            ss << "    " << divmod("rg", "ct", "b", "COL_TILES") << "\n";
            ss << "    const unsigned col = (unsigned)ct * 256u + threadIdx.x; const int r0 = (int)rg * RB;\n";
            ss << "    if (col >= cols) continue;\n";
            ss << "    " << divmod("t1", "ow", "col", "OW") << "\n";
            ss << "    " << divmod("n", "oh", "t1", "OH") << "\n";
            ss << "    const int h0 = oh * STH - PH, w0 = ow * STW - PW;\n    const T* img_n = img + (long)n * SN;\n";
            ss << "    T* out_c = out + col;\n";
            ss << "    for (int r = r0; r < r0 + RB && r < rows; ++r) {\n" << emit_split_row(fmt, "r");
            ss << "      const int h = h0 + kh * DH, w = w0 + kw * DW;\n";
            ss << "      T v = (T)0;\n      if (h >= 0 && h < H && w >= 0 && w < W) v = img_n[(long)c * SC + (long)h * SH + (long)w * SW];\n";
            ss << "      __builtin_nontemporal_store(v, out_c + (long)r * cols);\n    }\n  }\n}\n";
        });
    }
    return result;
}

// col2im: every image element sums, patch rows outermost, the entries of the patch matrix that im2col would have
// copied it to (col2im.cpp:103-141): the same additions in the same order as the reference's loop. The patch
// matrix is read through its strides, so the patch-major form produced for NHWC needs no copy, and there four
// channels (four consecutive matrix rows, contiguous in that form) travel per thread.
Array run_col2im(const Expr& e, const Array& patches_in) {
    Array patches = patches_in.is_buffer() ? patches_in : materialize(patches_in);
    const std::string& fmt = e.data_format;
    Array dest(e.shape, e.dtype);
    ImageGeom g = image_geom(e.shape, fmt);
    const int fh = e.geom[0], fw = e.geom[1], sth = e.geom[2], stw = e.geom[3];
    const int o_h = (g.ext[2] - fh) / sth + 1, o_w = (g.ext[3] - fw) / stw + 1;
    const int64_t n = numel_of(e.shape);
    if (n == 0) return dest;
    std::vector<int> pst = patches.normalized_strides();
    DALI_ASSERT((int64_t)patches.shape()[0] * patches.shape()[1] < ((int64_t)1 << 31), "col2im: the patch matrix must hold fewer than 2^31 elements");
    const bool channel_vectors = fmt[3] == 'C' && pst[0] == 1 && pst[1] % 4 == 0 && row_letters(fmt)[0] == 'C' && four_byte_vectors(e.dtype, patches, g.ext[1]);
    const int VEC = channel_vectors ? 4 : 1;
    Program P;
    P.arrays.push_back(manual_arg(dest, Cls::FULL, true, 1, {(int)n}, {}));
    P.arrays.push_back(manual_arg(patches, Cls::FULL, false, 2, patches.shape(), {pst[0], pst[1]}));
    GeomInts G;
    G.add_image(g);
    G.add("PH", e.geom[6]);
    G.add("PW", e.geom[7]);
    G.add("OH", o_h);
    G.add("OW", o_w);
    G.add("ORS", pst[0]);
    G.add("OCS", pst[1]);
    G.add_div("INNER_GROUPS", std::max(1, e.shape[3] / VEC));
    // filter, stride and dilation are compile-time: the loops over the covering patches unroll into independent
    // loads (a loop with run-time bounds would wait for each load in turn), and the divisions by them fold
    const int dh = e.geom[4], dw = e.geom[5];
    const int max_ph = (dh * (fh - 1) + sth) / sth, max_pw = (dw * (fw - 1) + stw) / stw;  // ceil(patch extent / stride)
    std::ostringstream sig;
    sig << "col2im|" << (int)e.dtype << "|" << fmt << "|" << VEC << "|" << fh << "," << fw << "," << sth << "," << stw << "," << dh << "," << dw;
    launch_special("col2im", sig.str(), P, (n / VEC + 255) / 256, G, [&](std::ostringstream& ss) {
        ss << "  constexpr int VEC = " << VEC << ", FH = " << fh << ", FW = " << fw << ", STH = " << sth << ", STW = " << stw << ", DH = " << dh
           << ", DW = " << dw << ", MAX_PH = " << max_ph << ", MAX_PW = " << max_pw << ";\n";
        ss << "  T* image = (T*)A.p[0];\n  const T* in = (const T*)A.p[1];\n";
        ss << "  const unsigned total = (unsigned)(N * C) * (unsigned)(H * W) / VEC;\n";
        ss << "  constexpr int patch_h = DH * (FH - 1) + 1, patch_w = DW * (FW - 1) + 1;\n";
        ss << kBandedElementLoop;
        ss << emit_decompose(fmt, "H", "W", "h_", "w_", true);
        ss << "    const int h = h_ + PH, w = w_ + PW;\n";
        ss << "    const int ph_min = h < patch_h ? h % DH : (h - patch_h + STH) / STH;\n";
        ss << "    const int pw_min = w < patch_w ? w % DW : (w - patch_w + STW) / STW;\n";
        ss << "    const int ph_max = (h + STH) / STH < OH ? (h + STH) / STH : OH;\n";
        ss << "    const int pw_max = (w + STW) / STW < OW ? (w + STW) / STW : OW;\n";
        ss << "    dali_vec<T, VEC> res;\n    _Pragma(\"unroll\") for (int k = 0; k < VEC; ++k) res.v[k] = (T)0;\n";
        ss << "    // patches in the reference's order (rows outermost); beyond the range the load goes to the matrix's first element and is not added\n";
        ss << "    _Pragma(\"unroll\") for (int a = 0; a < MAX_PH; ++a) {\n      const int ph = ph_min + a * DH; const bool ph_ok = ph < ph_max;\n";
        ss << "      _Pragma(\"unroll\") for (int b = 0; b < MAX_PW; ++b) {\n        const int pw = pw_min + b * DW; const bool ok = ph_ok && pw < pw_max;\n";
        ss << "        const int kh = (h - ph * STH) / DH, kw = (w - pw * STW) / DW;\n";
        ss << "        const int row = " << emit_join_row(fmt) << ";\n";
        ss << "        const T* src = ok ? in + ((long)row * ORS + (long)((n * OH + ph) * OW + pw) * OCS) : in;\n";
        ss << "        const dali_vec<T, VEC> v = dali_load<T, VEC>(src);\n";
        ss << "        if (ok) { _Pragma(\"unroll\") for (int k = 0; k < VEC; ++k) res.v[k] += v.v[k]; }\n      }\n    }\n";
        ss << "    dali_store<T, VEC>(image + (long)i * VEC, res);\n  }\n}\n";
    });
    return dest;
}

static GeomInts pool_geom(const Expr& e, const ImageGeom& gx, const ImageGeom& gy, int groups) {
    GeomInts G;
    G.add_image(gx);
    G.add("PH", e.geom[4]);
    G.add("PW", e.geom[5]);
    G.add_div("OH", gy.ext[2]);
    G.add_div("OW", gy.ext[3]);
    G.add("YSN", gy.stride[0]);
    G.add("YSC", gy.stride[1]);
    G.add("YSH", gy.stride[2]);
    G.add("YSW", gy.stride[3]);
    G.add_div("INNER_GROUPS", std::max(1, groups));
    return G;
}

static std::string pool_constants(const Expr& e, int VEC) {
    std::ostringstream ss;
    ss << "  constexpr int VEC = " << VEC << ", WH = " << e.geom[0] << ", WW = " << e.geom[1] << ", STH = " << e.geom[2] << ", STW = " << e.geom[3] << ";\n";
    return ss.str();
}

// pool2d: one thread per output element (four channels of it where the channels are contiguous). The window is
// walked columns outermost, as the reference's loop does (conv.cpp:66-89), so an average is the same sequence of
// fp32 additions; window and stride are compile-time, which turns the walk into independent loads at clamped
// coordinates whose values are used only where the window lies inside the image.
Array run_pool2d(const Expr& e, const Array& x_in) {
    Array x = dense_buffer(x_in);
    const std::string& fmt = e.data_format;
    Array dest(e.shape, e.dtype);
    const int64_t n = numel_of(e.shape);
    if (n == 0) return dest;
    ImageGeom gx = image_geom(x.shape(), fmt), gy = image_geom(e.shape, fmt);
    const bool average = e.depth != 0;
    // One output per thread for layouts ending in W: four neighbours along W per thread were tried, but a wave's loads then
    // spread over four times as many cache lines and the kernel ran three times slower.
    const int VEC = fmt[3] == 'C' && four_byte_vectors(e.dtype, x, gx.ext[1]) ? 4 : 1;
    Program P;
    P.arrays.push_back(manual_arg(dest, Cls::FULL, true, 1, {(int)n}, {}));
    P.arrays.push_back(manual_arg(x, Cls::FULL, false, 1, {(int)numel_of(x.shape())}, {}));
    std::ostringstream sig;
    sig << "pool2d|" << (int)e.dtype << "|" << fmt << "|" << average << "|" << VEC << "|" << e.geom[0] << "," << e.geom[1] << "," << e.geom[2] << "," << e.geom[3];
    launch_special("pool2d", sig.str(), P, (n / VEC + 255) / 256, pool_geom(e, gx, gy, e.shape[3] / VEC), [&](std::ostringstream& ss) {
        ss << pool_constants(e, VEC);
        ss << "  T* y = (T*)A.p[0];\n  const T* x = (const T*)A.p[1];\n";
        ss << "  const unsigned total = (unsigned)(N * C) * (unsigned)(OH * OW) / VEC;\n";
        ss << kBandedElementLoop;
        ss << emit_decompose(fmt, "OH", "OW", "oh", "ow", true);
        ss << "    const int h0 = oh * STH - PH;\n";
        ss << "    const int h_start = h0 > 0 ? h0 : 0, h_end = h0 + WH < H ? h0 + WH : H;\n";
        ss << "    const T* xp = x + ((long)n * SN + (long)c * SC);\n";
        ss << "    dali_vec<T, VEC> res;\n";
        const std::string init = average ? "(T)0" : "reducers::lowest<T>()";
        ss << "    const int w0 = ow * STW - PW;\n";
        ss << "    const int w_start = w0 > 0 ? w0 : 0, w_end = w0 + WW < W ? w0 + WW : W;\n";
        ss << "    _Pragma(\"unroll\") for (int k = 0; k < VEC; ++k) res.v[k] = " << init << ";\n";
        ss << "    _Pragma(\"unroll\") for (int a = 0; a < WW; ++a) {\n      const int w = w0 + a; const bool w_ok = w >= 0 && w < W; const int wc = w_ok ? w : w_start;\n";
        ss << "      _Pragma(\"unroll\") for (int b = 0; b < WH; ++b) {\n        const int h = h0 + b; const bool ok = w_ok && h >= 0 && h < H; const int hc = h >= 0 && h < H ? h : h_start;\n";
        ss << "        const dali_vec<T, VEC> v = dali_load<T, VEC>(xp + (hc * SH + wc * SW));\n";
        ss << "        if (ok) { _Pragma(\"unroll\") for (int k = 0; k < VEC; ++k) res.v[k] = " << (average ? "res.v[k] + v.v[k]" : "res.v[k] > v.v[k] ? res.v[k] : v.v[k]") << "; }\n      }\n    }\n";
        if (average) ss << "    _Pragma(\"unroll\") for (int k = 0; k < VEC; ++k) res.v[k] = res.v[k] / ((h_end - h_start) * (w_end - w_start));\n";
        ss << "    dali_store<T, VEC>(y + (long)i * VEC, res);\n  }\n}\n";
    });
    return dest;
}

// pool2d_backward: one thread per input element (or four channels of it), summing over the windows that hold it,
// window rows outermost (conv.cpp:133-172); at most ceil(window / stride) windows per direction, unrolled.
Array run_pool2d_backward(const Expr& e, const Array& y_in, const Array& dy_in, const Array& x_in) {
    Array y = dense_buffer(y_in), dy = dense_buffer(dy_in), x = dense_buffer(x_in);
    const std::string& fmt = e.data_format;
    Array dest(e.shape, e.dtype);
    const int64_t n = numel_of(e.shape);
    if (n == 0) return dest;
    ImageGeom gx = image_geom(x.shape(), fmt), gy = image_geom(y.shape(), fmt);
    const bool average = e.depth != 0;
    const bool channel_vectors = fmt[3] == 'C' && four_byte_vectors(e.dtype, x, gx.ext[1]) && y.offset() % 4 == 0 && dy.offset() % 4 == 0;
    // formats ending in W: a thread takes four neighbours along W, which share everything but their window columns
    const bool along_w = fmt[3] == 'W' && four_byte_vectors(e.dtype, x, gx.ext[3]);
    const int VEC = channel_vectors || along_w ? 4 : 1;
    Program P;
    P.arrays.push_back(manual_arg(dest, Cls::FULL, true, 1, {(int)n}, {}));
    P.arrays.push_back(manual_arg(y, Cls::FULL, false, 1, {(int)numel_of(y.shape())}, {}));
    P.arrays.push_back(manual_arg(dy, Cls::FULL, false, 1, {(int)numel_of(dy.shape())}, {}));
    P.arrays.push_back(manual_arg(x, Cls::FULL, false, 1, {(int)numel_of(x.shape())}, {}));
    std::ostringstream sig;
    sig << "pool2d_backward|" << (int)e.dtype << "|" << fmt << "|" << average << "|" << VEC << along_w << "|" << e.geom[0] << "," << e.geom[1] << "," << e.geom[2] << ","
        << e.geom[3];
    launch_special("pool2d_backward", sig.str(), P, (n / VEC + 255) / 256, pool_geom(e, gx, gy, e.shape[3] / VEC), [&](std::ostringstream& ss) {
        ss << pool_constants(e, VEC);
        ss << "  constexpr int MAX_PH = (WH + STH - 1) / STH, MAX_PW = (WW + STW - 1) / STW;\n";
        ss << "  T* dx = (T*)A.p[0];\n  const T* y = (const T*)A.p[1];\n  const T* dy = (const T*)A.p[2];\n  const T* x = (const T*)A.p[3];\n";
        ss << "  const unsigned total = (unsigned)(N * C) * (unsigned)(H * W) / VEC;\n";
        ss << kBandedElementLoop;
        ss << emit_decompose(fmt, "H", "W", "h", "w", true);
        ss << "    const dali_vec<T, VEC> src = dali_load<T, VEC>(x + (long)i * VEC);\n";
        ss << "    const int ph_start = (h + PH) < WH ? 0 : (h + PH - WH) / STH + 1;\n";
        ss << "    const int ph_end = (h + PH) / STH + 1 < OH ? (h + PH) / STH + 1 : OH;\n";
        ss << "    const long base = (long)n * YSN + (long)c * YSC;\n";
        ss << "    dali_vec<T, VEC> grad;\n    _Pragma(\"unroll\") for (int k = 0; k < VEC; ++k) grad.v[k] = (T)0;\n";
        // one window (ph, pw) adds to element k (all elements when the vector runs along the channels)
        auto add_window = [&](const std::string& k_lo, const std::string& k_hi, const std::string& g, const std::string& yv) {
            if (average) {
                ss << "          int hstart = ph * STH - PH, wstart = pw * STW - PW;\n";
                ss << "          const int hend = hstart + WH < H ? hstart + WH : H, wend = wstart + WW < W ? wstart + WW : W;\n";
                ss << "          hstart = hstart > 0 ? hstart : 0; wstart = wstart > 0 ? wstart : 0;\n";
                ss << "          const int pool_size = (hend - hstart) * (wend - wstart);\n";
                ss << "          if (ok) { _Pragma(\"unroll\") for (int k = " << k_lo << "; k < " << k_hi << "; ++k) grad.v[k] += ((T)1 * " << g << ") / pool_size; }\n";
            } else {
                ss << "          if (ok) { _Pragma(\"unroll\") for (int k = " << k_lo << "; k < " << k_hi << "; ++k) grad.v[k] += (" << yv << " == src.v[k] ? (T)1 : (T)0) * " << g << "; }\n";
            }
        };
        if (along_w) {
            ss << "    _Pragma(\"unroll\") for (int e = 0; e < VEC; ++e) {\n      const int we = w + e;\n";
            ss << "      const int pw_start = (we + PW) < WW ? 0 : (we + PW - WW) / STW + 1;\n";
            ss << "      const int pw_end = (we + PW) / STW + 1 < OW ? (we + PW) / STW + 1 : OW;\n";
            ss << "      _Pragma(\"unroll\") for (int a = 0; a < MAX_PH; ++a) {\n        const int ph = ph_start + a; const bool ph_ok = ph < ph_end;\n";
            ss << "        _Pragma(\"unroll\") for (int b = 0; b < MAX_PW; ++b) {\n          const int pw = pw_start + b; const bool ok = ph_ok && pw < pw_end;\n";
            ss << "          const long q = ok ? base + (ph * YSH + pw * YSW) : 0;  // beyond the range: a valid address, value unused\n";
            ss << "          const T g1 = dy[q];\n";
            if (!average) ss << "          const T y1 = y[q];\n";
            add_window("e", "e + 1", "g1", "y1");
            ss << "        }\n      }\n    }\n";
        } else {
            ss << "    const int pw_start = (w + PW) < WW ? 0 : (w + PW - WW) / STW + 1;\n";
            ss << "    const int pw_end = (w + PW) / STW + 1 < OW ? (w + PW) / STW + 1 : OW;\n";
            ss << "    _Pragma(\"unroll\") for (int a = 0; a < MAX_PH; ++a) {\n      const int ph = ph_start + a; const bool ph_ok = ph < ph_end;\n";
            ss << "      _Pragma(\"unroll\") for (int b = 0; b < MAX_PW; ++b) {\n        const int pw = pw_start + b; const bool ok = ph_ok && pw < pw_end;\n";
            ss << "          const long q = ok ? base + (ph * YSH + pw * YSW) : 0;  // beyond the range: a valid address, value unused\n";
            ss << "          const dali_vec<T, VEC> g = dali_load<T, VEC>(dy + q);\n";
            if (!average) ss << "          const dali_vec<T, VEC> yv = dali_load<T, VEC>(y + q);\n";
            add_window("0", "VEC", "g.v[k]", "yv.v[k]");
            ss << "      }\n    }\n";
        }
        ss << "    dali_store<T, VEC>(dx + (long)i * VEC, grad);\n  }\n}\n";
    });
    return dest;
}

// Stride-1 convolution of a channels-last image without a patch matrix (dali/array/op/conv.cpp:253-272 forms
// im2col + one product). The image is copied once into a zero-padded buffer X[N, Hp, Wp, C]; seen as a matrix of
// pixels with leading dimension C, filter row kh of every patch is the run of filter_w * C values that starts at
// pixel p + kh * Wp, so the convolution is the sum over kh of the products X(shifted by kh * Wp pixels)[., fw * C] .
// F[rows of kh, out]: dali_hip_sgemm_terms with overlapping rows, evaluated at all N * Hp * Wp positions, of which
// the row map stores the out_h x out_w valid ones densely. The patch matrix (filter_h * filter_w times the image) is
// never written or read.
static Array conv2d_nhwc_direct(const Array& x_in, const Array& filters_in, int pad_top, int pad_left, int pad_bottom, int pad_right) {
    Array x = dense_buffer(x_in), f = dense_buffer(filters_in);
    const int N = x.shape()[0], H = x.shape()[1], W = x.shape()[2], C = x.shape()[3];
    const int O = f.shape()[0], fh = f.shape()[1], fw = f.shape()[2];
    const int Hp = H + pad_top + pad_bottom, Wp = W + pad_left + pad_right, oh = Hp - fh + 1, ow = Wp - fw + 1;
    const int64_t pixels = (int64_t)N * Hp * Wp, slack = (int64_t)(fh - 1) * Wp + fw;
    DALI_ASSERT(oh >= 1 && ow >= 1 && (pixels + slack) * C < ((int64_t)1 << 31), "conv2d: image too large for the direct path");
    // the filters as a [filter_h * filter_w * C, out] matrix: the product then reads both operands along their rows
    // (a right operand stored [out][K] costs the kernel a transposing pass through LDS, 211 against 177 us at this size)
    Array ft = f.reshape({O, fh * fw * C}).transpose().ascontiguousarray();
    Array xp({(int)(pixels + slack), C}, DTYPE_FLOAT);
    {
        Program P;
        P.arrays.push_back(manual_arg(xp, Cls::FULL, true, 1, {(int)((pixels + slack) * C)}, {}));
        P.arrays.push_back(manual_arg(x, Cls::FULL, false, 1, {(int)numel_of(x.shape())}, {}));
        GeomInts G;
        G.add("PIXELS", (int)pixels);
        G.add("ALL", (int)(pixels + slack));
        G.add("H", H);
        G.add("W", W);
        G.add("PT", pad_top);
        G.add("PL", pad_left);
        G.add_div("HPWP", Hp * Wp);
        G.add_div("WP", Wp);
        G.add_div("C4", C / 4);
        launch_special("pad", "pad_nhwc|f32", P, ((pixels + slack) * (C / 4) + 255) / 256, G, [&](std::ostringstream& ss) {
            ss << "  T* out = (T*)A.p[0];\n  const T* img = (const T*)A.p[1];\n";
            ss << "  const unsigned total = (unsigned)ALL * (unsigned)C4;\n";
            ss << "  for (unsigned i = blockIdx.x * 256u + threadIdx.x; i < total; i += gridDim.x * 256u) {\n";
            ss << "    " << divmod("p", "c4", "i", "C4") << "\n";
            ss << "    " << divmod("n", "rest", "p", "HPWP") << "\n";
            ss << "    " << divmod("ip", "jp", "(unsigned)rest", "WP") << "\n";
            ss << "    const int h = (int)ip - PT, w = jp - PL;\n";
            ss << "    dali_vec<T, 4> v;\n";
            ss << "    if (p < (unsigned)PIXELS && h >= 0 && h < H && w >= 0 && w < W) v = dali_load<T, 4>(img + ((((long)n * H + h) * W + w) * C4 + c4) * 4);\n";
            ss << "    else { _Pragma(\"unroll\") for (int k = 0; k < 4; ++k) v.v[k] = (T)0; }\n";
            ss << "    dali_store<T, 4>(out + (long)i * 4, v);\n  }\n}\n";
        });
    }
    Array out({N, oh, ow, O}, DTYPE_FLOAT);
    const float* xpp = (const float*)xp.device_ptr();
    const float* fp = (const float*)ft.device_ptr();
    float* op_ = (float*)out.device_ptr(memory::AM_OVERWRITE);
    const int lda = C, ldb = O, M = (int)pixels;
    auto issue = [=]() {
        int K[8];
        const float* As[8];
        const float* Bs[8];
        for (int t = 0; t < fh; ++t) {
            K[t] = fw * C;
            As[t] = xpp + (size_t)t * Wp * C;
            Bs[t] = fp + (size_t)t * fw * C * O;
        }
        const int row_map[4] = {Hp, Wp, oh, ow};
        check_hip(dali_hip_sgemm_terms(fh, 0, 0, M, O, K, As, lda, Bs, ldb, 1.0f, 0.0f, op_, O, row_map), "convolution product");
    };
    jit_stats().gemms_launched++;
    issue();
    if (g_recording) {
        note_recorded_write(out.expression()->memory);
        std::vector<Array> keep = {xp, ft, out};
        g_recording->push_back([=]() {
            (void)keep;
            issue();
        });
    }
    return out;
}

}  // namespace jit

using namespace jit;

Array conv2d_direct_nhwc(const Array& x, const Array& filters, int pad_top, int pad_left, int pad_bottom, int pad_right) {
    return conv2d_nhwc_direct(x, filters, pad_top, pad_left, pad_bottom, pad_right);
}

}  // namespace dali
