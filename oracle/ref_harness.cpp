// ref_harness.cpp — thin extern "C" driver around the pieces of the reference
// that compile from their own header files, included FROM WHERE THEY LIE under
// the reference checkout (-I<reference root>): the reducers
// (dali/array/jit/reducer_kernels.h), the view / index arithmetic
// (dali/array/jit/array_view.h) and the scalar reference GEMM
// (dali/array/gemm/reference_gemm.h). TEST INFRASTRUCTURE ONLY: it validates
// oracle/dali_oracle.c and is never linked into the product.
//
// The rest of the reference (the JIT, functor.h, the BLAS call) needs a
// cmake-generated dali/config.h, the empty libcuckoo submodule and a cblas.h this
// image lacks, so it is not built here. The loops below therefore restate the
// generated sequential loops (dali/array/jit/all_reduce_kernel_utils.cpp:105-154,
// 210-223) around the reference's own Reducer::Reduce / SetInitValue and its own
// strided views.
#include <cstddef>
#include <cstdint>

#include "dali/macros.h"
#include "dali/array/jit/array_view.h"
#include "dali/array/jit/reducer_kernels.h"
#include "dali/array/gemm/reference_gemm.h"

namespace {
template <typename Reducer>
void axis_reduce(const float* x, int rows, int cols, int row_stride, int col_stride, float* out) {
    int sizes[2] = {rows, cols}, strides[2] = {row_stride, col_stride};
    auto view = make_strided_view<float, 2>((void*)x, 0, sizes, strides);
    for (int i = 0; i < rows; ++i) {
        Shape<2> query;
        query[0] = i;
        float res;
        Reducer::SetInitValue(res);
        int& i1 = query[1];
        for (i1 = 0; i1 < view.shape()[1]; ++i1) Reducer::Reduce(res, view[query]);
        out[i] = res;
    }
}

template <typename Reducer>
void arg_axis_reduce(const float* x, int rows, int cols, int row_stride, int col_stride, int* out) {
    int sizes[2] = {rows, cols}, strides[2] = {row_stride, col_stride};
    auto view = make_strided_view<float, 2>((void*)x, 0, sizes, strides);
    for (int i = 0; i < rows; ++i) {
        Shape<2> query;
        query[0] = i;
        int idx = 0;
        float res;
        Reducer::SetInitValue(res);
        int& i1 = query[1];
        for (i1 = 0; i1 < view.shape()[1]; ++i1) {
            float tmp = res;
            Reducer::Reduce(res, view[query]);
            if (tmp != res) idx = i1;
        }
        out[i] = idx;
    }
}

template <typename Reducer>
float all_reduce(const float* x, int n) {
    int sizes[1] = {n};
    auto view = make_view<float, 1>((void*)x, 0, sizes);
    float res;
    Reducer::SetInitValue(res);
    for (int i = 0; i < n; ++i) Reducer::Reduce(res, view[Shape<1>(i)]);
    return res;
}
}  // namespace

extern "C" {

// reducer: 0 sum, 1 maximum, 2 minimum, 3 product
int ref_axis_reduce(int reducer, const float* x, int rows, int cols, int row_stride, int col_stride, float* out) {
    switch (reducer) {
        case 0: axis_reduce<reducers::sum>(x, rows, cols, row_stride, col_stride, out); return 0;
        case 1: axis_reduce<reducers::maximum>(x, rows, cols, row_stride, col_stride, out); return 0;
        case 2: axis_reduce<reducers::minimum>(x, rows, cols, row_stride, col_stride, out); return 0;
        case 3: axis_reduce<reducers::product>(x, rows, cols, row_stride, col_stride, out); return 0;
    }
    return -1;
}

int ref_arg_axis_reduce(int reducer, const float* x, int rows, int cols, int row_stride, int col_stride, int* out) {
    switch (reducer) {
        case 1: arg_axis_reduce<reducers::maximum>(x, rows, cols, row_stride, col_stride, out); return 0;
        case 2: arg_axis_reduce<reducers::minimum>(x, rows, cols, row_stride, col_stride, out); return 0;
    }
    return -1;
}

float ref_all_reduce(int reducer, const float* x, int n) {
    switch (reducer) {
        case 0: return all_reduce<reducers::sum>(x, n);
        case 1: return all_reduce<reducers::maximum>(x, n);
        case 2: return all_reduce<reducers::minimum>(x, n);
        default: return all_reduce<reducers::product>(x, n);
    }
}

// index arithmetic of the generated kernels
void ref_index_to_dim3(int index, const int* shape, int* out) {
    Shape<3> s(shape);
    Shape<3> r = index_to_dim(index, s);
    for (int i = 0; i < 3; ++i) out[i] = r[i];
}

int ref_indices_to_offset3(const int* shape, const int* indices) {
    return indices_to_offset(Shape<3>(shape), Shape<3>(indices));
}

// ReferenceGemm as instantiated by igemm (dali/array/gemm/cpu_gemm.cpp:14-20) and,
// for float, the same template: column-major C(m x n) with transpose_c = true.
void ref_gemm_i32(int transpose_a, int transpose_b, int m, int n, int k, const int* a, int lda, const int* b, int ldb,
                  int* c, int ldc) {
    ReferenceGemm<int>(transpose_a, transpose_b, true, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, ldc);
}

void ref_gemm_f32(int transpose_a, int transpose_b, int m, int n, int k, const float* a, int lda, const float* b,
                  int ldb, float* c, int ldc) {
    ReferenceGemm<float>(transpose_a, transpose_b, true, m, n, k, 1.0, a, lda, b, ldb, 0.0, c, ldc);
}

}  // extern "C"
