// Matrix products and the recurrent steps built on them: operand preparation for dali_hip_sgemm (row-major, optional
// transposition by strides), the accumulating pair X.W + H.U, the fused LSTM step and the persistent recurrent launch.
#include "jit_internal.h"

namespace dali {
namespace jit {

// dali/array/gemm/gemm_utils.cpp:7-21
static void gemm_stride_transpose(const Array& a, bool* transpose, int* ld) {
    if (a.strides().empty()) {
        *transpose = false;
        *ld = a.shape()[1];
        return;
    }
    const auto& st = a.strides();
    if (st[0] == 1) {
        *transpose = true;
        *ld = st[1];
        return;
    }
    if (st[1] == 1) {
        *transpose = false;
        *ld = st[0];
        return;
    }
    throw std::runtime_error(make_message("gemm only supports arrays with a single stride (got strides: ", shape_str(st), ")"));
}

// dali/array/op/dot.cpp:9-16: operand must be contiguous or a plain transpose of a contiguous matrix
static Array gemm_operand(Array a) {
    a.eval();
    if (a.expression()->kind == Kind::SCALAR) throw std::runtime_error("matmul operand cannot be a scalar");
    if (a.contiguous_memory()) return a;
    const auto& st = a.strides();
    if (st.size() == 2 && st[0] == 1 && st[1] >= a.shape()[0]) return a;
    if (st.size() == 2 && st[1] == 1 && st[0] >= a.shape()[1]) return a;
    return a.ascontiguousarray();
}

struct GemmOperands {
    Array lhs, rhs;
    bool lt, rt;
    int lld, rld;
};

static GemmOperands prepare_gemm(const Expr* mm) {
    GemmOperands g;
    g.lhs = gemm_operand(mm->args[0]);
    g.rhs = gemm_operand(mm->args[1]);
    DALI_ASSERT(g.lhs.dtype() == g.rhs.dtype() && (g.lhs.dtype() == DTYPE_FLOAT || g.lhs.dtype() == DTYPE_DOUBLE),
                "op::dot on this backend is implemented for float32 and float64 operands (MFMA GEMM; the reference's integer "
                "product is a scalar CPU loop)");
    gemm_stride_transpose(g.lhs, &g.lt, &g.lld);
    gemm_stride_transpose(g.rhs, &g.rt, &g.rld);
    return g;
}

// dst[n_rows, m] = lhs * rhs through the column-major entry point, argument for
// argument the call of dali/array/gemm/cublas_gemm.cu:153-166.
void run_gemm(const Array& dst, const Expr* mm, const Expr* mm2, float beta) {
    DALI_SCOPE(mm2 ? "gemm_pair" : "gemm");
    GemmOperands g = prepare_gemm(mm);
    int m = g.rhs.shape()[1], n = g.lhs.shape()[0], k = g.rhs.shape()[0];
    jit_stats().gemms_launched++;
    if (!jit_stats().last_kernel_kinds.empty()) jit_stats().last_kernel_kinds += ",";
    jit_stats().last_kernel_kinds += mm2 ? "gemm_pair" : "gemm";
    if (g_dry_run) return;
    int ldc = dst.strides().empty() ? dst.shape()[1] : dst.strides()[0];
    // an overwritten destination that spans its whole allocation needs no migration of what it held (a strided or partial
    // view keeps the elements between and around its rows, so those stay MUTABLE)
    const bool spans = dst.offset() == 0 && dst.contiguous_memory() &&
                       (size_t)numel_of(dst.shape()) * (size_t)size_of_dtype(dst.dtype()) == dst.expression()->memory->bytes();
    memory::AM mode = beta == 0.0f && spans ? memory::AM_OVERWRITE : memory::AM_MUTABLE;
    if (g.lhs.dtype() == DTYPE_DOUBLE) {
        // cublasDgemm's branch (dali/array/gemm/cublas_gemm.cu:167-178); a pair of products is two accumulating calls
        struct Call { int rt, lt, k; const double* rp; int rld; const double* lp; int lld; double beta; };
        std::vector<Call> calls;
        std::vector<GemmOperands> keep = {g};
        calls.push_back({g.rt, g.lt, k, (const double*)g.rhs.device_ptr(), g.rld, (const double*)g.lhs.device_ptr(), g.lld, (double)beta});
        if (mm2) {
            GemmOperands h = prepare_gemm(mm2);
            DALI_ASSERT(h.lhs.dtype() == DTYPE_DOUBLE, "op::dot: the two products of a sum must share a dtype");
            keep.push_back(h);
            calls.push_back({h.rt, h.lt, h.rhs.shape()[0], (const double*)h.rhs.device_ptr(), h.rld, (const double*)h.lhs.device_ptr(), h.lld, 1.0});
        }
        double* dp = (double*)dst.device_ptr(mode);
        auto issue = [=]() {
            for (const Call& c : calls) check_hip(dali_hip_dgemm(c.rt, c.lt, m, n, c.k, 1.0, c.rp, c.rld, c.lp, c.lld, c.beta, dp, ldc), "dgemm");
        };
        issue();
        if (g_recording) {
            note_recorded_write(dst.expression()->memory);
            Array dkeep = dst;
            g_recording->push_back([=]() {
                (void)keep;
                (void)dkeep;
                issue();
            });
        }
        return;
    }
    if (!mm2) {
        const float* rp = (const float*)g.rhs.device_ptr();
        const float* lp = (const float*)g.lhs.device_ptr();
        float* dp = (float*)dst.device_ptr(mode);
        check_hip(dali_hip_sgemm(g.rt, g.lt, m, n, k, 1.0f, rp, g.rld, lp, g.lld, beta, dp, ldc), "sgemm");
        if (g_recording) {
            note_recorded_write(dst.expression()->memory);
            GemmOperands keep = g;
            Array dkeep = dst;
            g_recording->push_back([=]() {
                (void)keep;
                (void)dkeep;
                check_hip(dali_hip_sgemm(g.rt, g.lt, m, n, k, 1.0f, rp, g.rld, lp, g.lld, beta, dp, ldc), "sgemm replay");
            });
        }
    } else {
        GemmOperands h = prepare_gemm(mm2);
        int k2 = h.rhs.shape()[0];
        const float* rp = (const float*)g.rhs.device_ptr();
        const float* lp = (const float*)g.lhs.device_ptr();
        const float* rp2 = (const float*)h.rhs.device_ptr();
        const float* lp2 = (const float*)h.lhs.device_ptr();
        float* dp = (float*)dst.device_ptr(mode);
        check_hip(dali_hip_sgemm_pair(g.rt, g.lt, h.rt, h.lt, m, n, k, k2, 1.0f, rp, g.rld, lp, g.lld, rp2, h.rld, lp2, h.lld, beta, dp, ldc),
                  "sgemm_pair");
        if (g_recording) {
            note_recorded_write(dst.expression()->memory);
            Array dkeep = dst;
            g_recording->push_back([=]() {
                (void)dkeep;
                check_hip(dali_hip_sgemm_pair(g.rt, g.lt, h.rt, h.lt, m, n, k, k2, 1.0f, rp, g.rld, lp, g.lld, rp2, h.rld, lp2, h.lld, beta, dp, ldc),
                          "sgemm_pair replay");
            });
        }
    }
}

}  // namespace jit

using namespace jit;

void lstm_step_fused(const Array& x, const Array& h, const Array& c, const Array& W, const Array& U, const Array& b, const Array& c_new,
                     const Array& h_new) {
    const int Bn = x.shape()[0], In = x.shape()[1], H = h.shape()[1];
    const float* xp = (const float*)x.device_ptr();
    const float* hp = (const float*)h.device_ptr();
    const float* cp = (const float*)c.device_ptr();
    const float* wp = (const float*)W.device_ptr();
    const float* up = (const float*)U.device_ptr();
    const float* bp = (const float*)b.device_ptr();
    float* co = (float*)c_new.device_ptr(memory::AM_OVERWRITE);
    float* ho = (float*)h_new.device_ptr(memory::AM_OVERWRITE);
    jit_stats().gemms_launched++;
    jit_stats().last_kernel_kinds = "lstm_fused";
    check_hip(dali_hip_lstm_step(Bn, In, H, xp, In, hp, H, cp, wp, 4 * H, up, 4 * H, bp, co, ho), "fused lstm step");
    if (g_recording) {
        note_recorded_write(c_new.expression()->memory);
        note_recorded_write(h_new.expression()->memory);
        std::vector<Array> keep = {x, h, c, W, U, b, c_new, h_new};
        g_recording->push_back([=]() {
            (void)keep;
            check_hip(dali_hip_lstm_step(Bn, In, H, xp, In, hp, H, cp, wp, 4 * H, up, 4 * H, bp, co, ho), "fused lstm step replay");
        });
    }
}

// one step at a batch of up to 64 rows: 16-row tiles, one workgroup per compute unit (dali_hip_lstm_step_small)
void lstm_step_small(const Array& x, const Array& h, const Array& c, const Array& W, const Array& U, const Array& b, const Array& c_new,
                     const Array& h_new) {
    const int Bn = x.shape()[0], In = x.shape()[1], H = h.shape()[1];
    const float* xp = (const float*)x.device_ptr();
    const float* hp = (const float*)h.device_ptr();
    const float* cp = (const float*)c.device_ptr();
    const float* wp = (const float*)W.device_ptr();
    const float* up = (const float*)U.device_ptr();
    const float* bp = (const float*)b.device_ptr();
    float* co = (float*)c_new.device_ptr(memory::AM_OVERWRITE);
    float* ho = (float*)h_new.device_ptr(memory::AM_OVERWRITE);
    jit_stats().gemms_launched++;
    jit_stats().last_kernel_kinds = "lstm_small";
    check_hip(dali_hip_lstm_step_small(Bn, In, H, xp, In, hp, H, cp, wp, 4 * H, up, 4 * H, bp, co, ho), "small-batch lstm step");
    if (g_recording) {
        note_recorded_write(c_new.expression()->memory);
        note_recorded_write(h_new.expression()->memory);
        std::vector<Array> keep = {x, h, c, W, U, b, c_new, h_new};
        g_recording->push_back([=]() {
            (void)keep;
            check_hip(dali_hip_lstm_step_small(Bn, In, H, xp, In, hp, H, cp, wp, 4 * H, up, 4 * H, bp, co, ho), "small-batch lstm step replay");
        });
    }
}

// the recurrent half of a whole sequence in one launch (records itself like any other launch)
void lstm_recurrent_persistent(const Array& pre, const Array& U, const Array& h0, const Array& c0, const Array& hs, const Array& c_out) {
    const int T = hs.shape()[0], Bn = hs.shape()[1], H = hs.shape()[2];
    const float* pp = (const float*)pre.device_ptr();
    const float* up = (const float*)U.device_ptr();
    const float* hp = (const float*)h0.device_ptr();
    const float* cp = (const float*)c0.device_ptr();
    float* ho = (float*)hs.device_ptr(memory::AM_OVERWRITE);
    float* co = (float*)c_out.device_ptr(memory::AM_OVERWRITE);
    jit_stats().gemms_launched++;
    jit_stats().last_kernel_kinds = "lstm_persistent";
    check_hip(dali_hip_lstm_recurrent_persistent(T, Bn, H, pp, up, 4 * H, hp, cp, ho, co), "persistent lstm sequence");
    if (g_recording) {
        note_recorded_write(hs.expression()->memory);
        note_recorded_write(c_out.expression()->memory);
        std::vector<Array> keep = {pre, U, h0, c0, hs, c_out};
        g_recording->push_back([=]() {
            (void)keep;
            check_hip(dali_hip_lstm_recurrent_persistent(T, Bn, H, pp, up, 4 * H, hp, cp, ho, co), "persistent lstm sequence replay");
        });
    }
}


// the recurrent half of a whole GRU sequence in one launch
void gru_recurrent_persistent(const Array& pre, const Array& U, const Array& h0, const Array& hs, const Array& scratch) {
    const int T = hs.shape()[0], Bn = hs.shape()[1], H = hs.shape()[2];
    const float* pp = (const float*)pre.device_ptr();
    const float* up = (const float*)U.device_ptr();
    const float* hp = (const float*)h0.device_ptr();
    float* ho = (float*)hs.device_ptr(memory::AM_OVERWRITE);
    float* sp = (float*)scratch.device_ptr(memory::AM_OVERWRITE);
    jit_stats().gemms_launched++;
    jit_stats().last_kernel_kinds = "gru_persistent";
    check_hip(dali_hip_gru_recurrent_persistent(T, Bn, H, pp, up, 3 * H, hp, ho, sp), "persistent gru sequence");
    if (g_recording) {
        note_recorded_write(hs.expression()->memory);
        note_recorded_write(scratch.expression()->memory);
        std::vector<Array> keep = {pre, U, h0, hs, scratch};
        g_recording->push_back([=]() {
            (void)keep;
            check_hip(dali_hip_gru_recurrent_persistent(T, Bn, H, pp, up, 3 * H, hp, ho, sp), "persistent gru sequence replay");
        });
    }
}

void softmax_axis_launch(const Array& x, const Array& out, long long outer, int extent, long long inner) {
    const float* xp = (const float*)x.device_ptr();
    float* op = (float*)out.device_ptr(memory::AM_OVERWRITE);
    jit_stats().kernels_launched++;
    jit_stats().last_kernel_kinds = "softmax_axis";
    check_hip(dali_hip_softmax_axis(xp, op, outer, extent, inner), "softmax along an inner axis");
    if (g_recording) {
        note_recorded_write(out.expression()->memory);
        std::vector<Array> keep = {x, out};
        g_recording->push_back([=]() {
            (void)keep;
            check_hip(dali_hip_softmax_axis(xp, op, outer, extent, inner), "softmax along an inner axis replay");
        });
    }
}

}  // namespace dali
