// Device-side support code prepended to every generated kernel: the scalar
// functors, the reducers and the wave64 / workgroup reduction helpers.
//
// The functors restate the arithmetic contract of the reference's
// dali/array/functor.h (non-CUDA branch, which is what its CPU results come
// from): float arguments use the float libm entry points, `sigmoid` and the other
// functors written with double literals evaluate in double and round once.
// The reducers restate dali/array/jit/reducer_kernels.h:57-169 (init values
// 0 / -FLT_MAX / FLT_MAX / 1; maximum of floats is the device branch's fmaxf).
#ifndef DALI_AMD_DEVICE_PRELUDE_H
#define DALI_AMD_DEVICE_PRELUDE_H

namespace dali {
namespace codegen {

static const char* const kDevicePrelude = R"HIPSRC(
#define DALI_FLT_MAX 3.402823466e+38f
#define DALI_DBL_MAX 1.7976931348623157e+308
#define DALI_INT_MAX 2147483647
#define DALI_INT_MIN (-2147483647 - 1)
#define DI __device__ __forceinline__

union dali_slot { int i; float f; double d; };

template <typename T, int N>
struct alignas(sizeof(T) * N) dali_vec { T v[N]; };

template <typename T, int N>
DI dali_vec<T, N> dali_load(const T* p) { return *reinterpret_cast<const dali_vec<T, N>*>(p); }
template <typename T, int N>
DI void dali_store(T* p, const dali_vec<T, N>& v) { *reinterpret_cast<dali_vec<T, N>*>(p) = v; }
template <typename T, int N>
DI dali_vec<T, N> dali_load_nt(const T* p) {
    dali_vec<T, N> r;
    if constexpr (sizeof(T) * N == 16) {
        typedef int i4 __attribute__((ext_vector_type(4)));
        i4 raw = __builtin_nontemporal_load(reinterpret_cast<const i4*>(p));
        __builtin_memcpy(&r, &raw, 16);
    } else {
        r = *reinterpret_cast<const dali_vec<T, N>*>(p);
    }
    return r;
}
template <typename T, int N>
DI void dali_store_nt(T* p, const dali_vec<T, N>& v) {
    if constexpr (sizeof(T) * N == 16) {
        typedef int i4 __attribute__((ext_vector_type(4)));
        i4 raw;
        __builtin_memcpy(&raw, &v, 16);
        __builtin_nontemporal_store(raw, reinterpret_cast<i4*>(p));
    } else {
        *reinterpret_cast<dali_vec<T, N>*>(p) = v;
    }
}

// The same accesses for addresses aligned to the element only (rows whose length is not a multiple of the
// vector: every row starts at another offset within 16 bytes). Global memory takes multi-dword accesses at any
// dword address, so these are single instructions too.
template <typename T, int N>
struct alignas(sizeof(T)) dali_vecu { T v[N]; };
template <typename T, int N>
DI dali_vec<T, N> dali_loadu(const T* p) {
    const dali_vecu<T, N> u = *reinterpret_cast<const dali_vecu<T, N>*>(p);
    dali_vec<T, N> r;
    __builtin_memcpy(&r, &u, sizeof(r));
    return r;
}
template <typename T, int N>
DI void dali_storeu(T* p, const dali_vec<T, N>& v) {
    dali_vecu<T, N> u;
    __builtin_memcpy(&u, &v, sizeof(u));
    *reinterpret_cast<dali_vecu<T, N>*>(p) = u;
}
template <typename T, int N>
DI dali_vec<T, N> dali_loadu_nt(const T* p) {
    dali_vec<T, N> r;
    if constexpr (sizeof(T) * N == 16) {
        typedef int i4 __attribute__((ext_vector_type(4)));
        typedef i4 i4u __attribute__((aligned(4)));
        i4 raw = __builtin_nontemporal_load(reinterpret_cast<const i4u*>(p));
        __builtin_memcpy(&r, &raw, 16);
    } else {
        r = dali_loadu<T, N>(p);
    }
    return r;
}
template <typename T, int N>
DI void dali_storeu_nt(T* p, const dali_vec<T, N>& v) {
    if constexpr (sizeof(T) * N == 16) {
        typedef int i4 __attribute__((ext_vector_type(4)));
        typedef i4 i4u __attribute__((aligned(4)));
        i4 raw;
        __builtin_memcpy(&raw, &v, 16);
        __builtin_nontemporal_store(raw, reinterpret_cast<i4u*>(p));
    } else {
        dali_storeu<T, N>(p, v);
    }
}

// ------------------------------------------------------------ libm dispatch
// exp for float arguments. 2^(x * log2 e) on the hardware's exp2 unit, with the rounding error of the product put back:
// t = fl(x * c), r = x * c - t exactly (one FMA) plus x times the part of log2 e that c lacks, and 2^(t + r) =
// 2^t * (1 + r ln 2) to first order (|r| < 2^-17). About 1 ulp from the correctly rounded value wherever the result
// is a normal number, which is what libm's expf delivers; results below the normal range come out as zero. Outside
// |t| < 128 (overflow, underflow, infinities, NaN) the exp2 unit's own answer is already the right one and the
// correction (which would be inf * 0 there) is left out. Eleven issue slots against about eighteen for the library
// routine: a row kernel that exponentiates every element is otherwise bound by the vector ALU, not by memory.
DI float dali_expf(float x) {
    const float c = 0x1.715476p+0f, cc = 0x1.4ae0bep-26f;
    const float t = x * c;
    float r = __builtin_fmaf(x, c, -t);
    r = __builtin_fmaf(x, cc, r);
    const float e = __builtin_amdgcn_exp2f(t);
    const float fixed = __builtin_fmaf(e, r * 0x1.62e430p-1f, e);
    return __builtin_fabsf(t) < 128.0f ? fixed : e;
}
DI float  m_exp(float a)  { return dali_expf(a); }
DI double m_exp(double a) { return exp(a); }
DI double m_exp(int a)    { return exp((double)a); }
DI float  m_log(float a)  { return logf(a); }
DI double m_log(double a) { return log(a); }
DI double m_log(int a)    { return log((double)a); }
DI float  m_tanh(float a)  { return tanhf(a); }
DI double m_tanh(double a) { return tanh(a); }
DI double m_tanh(int a)    { return tanh((double)a); }
DI float  m_abs(float a)  { return fabsf(a); }
DI double m_abs(double a) { return fabs(a); }
DI int    m_abs(int a)    { return a < 0 ? -a : a; }
DI float  m_pow(float a, float b)   { return powf(a, b); }
DI double m_pow(double a, double b) { return pow(a, b); }
DI double m_pow(int a, int b)       { return pow((double)a, (double)b); }

namespace functor {
template <typename R> struct square   { DI static R Map(R a) { return a * a; } };
template <typename R> struct cube     { DI static R Map(R a) { return a * a * a; } };
template <typename R> struct fill     { DI static R Map(R a, R filler) { return filler; } };
template <typename R> struct add      { DI static R Map(R a, R b) { return a + b; } };
template <typename R> struct equals   { DI static R Map(R a, R b) { return a == b ? 1 : 0; } };
template <typename R> struct subtract { DI static R Map(R a, R b) { return a - b; } };
template <typename R> struct eltmul   { DI static R Map(R a, R b) { return a * b; } };
template <typename R> struct eltdiv   { DI static R Map(R a, R b) { return a / b; } };
template <typename R> struct sqrt_f   { DI static R Map(R a) { return (R)sqrt((double)a); } };
template <> struct sqrt_f<float>      { DI static float Map(float a) { return sqrtf(a); } };
template <typename R> struct rsqrt    { DI static R Map(R a) { return (R)(1.0 / sqrt((double)a)); } };
template <typename R> struct inv      { DI static R Map(R a) { return ((R)1.0) / a; } };
template <typename R> struct cast     { template <typename O> DI static R Map(O a) { return R(a); } };
template <typename R> struct round    { template <typename O> DI static R Map(O a) { return (R)floor((double)a + 0.5); } };
template <typename R> struct ceil     { template <typename O> DI static R Map(O a) { return (R)::ceil((double)a); } };
template <typename R> struct sigmoid  { DI static R Map(R a) { return (R)(1.0 / (1.0 + (double)m_exp(-a))); } };
template <typename R> struct identity { DI static R Map(R a) { return a; } };
template <typename R> struct log      { DI static R Map(R a) { return (R)m_log(a); } };
template <typename R> struct negative_log { DI static R Map(R a) { return (R)(-m_log(a)); } };
template <typename R> struct safe_entropy_log {
    DI static R Map(R a) {
        R s = a;
        const R lo = (R)1e-6, hi = (R)(1.0 - 1e-6);
        if (s > hi) s = hi;
        if (s < lo) s = lo;
        return (R)m_log(s);
    }
};
template <typename R> struct exp      { DI static R Map(R a) { return (R)m_exp(a); } };
template <typename R> struct isnotanumber { DI static R Map(R a) { return (R)(a != a); } };
template <> struct isnotanumber<int>  { DI static int Map(int a) { return 0; } };
template <typename R> struct isinfinity { DI static R Map(R a) { return (R)(a == a && (a - a) != (a - a)); } };
template <> struct isinfinity<int>    { DI static int Map(int a) { return 0; } };
template <typename R> struct div_grad { DI static R Map(R a, R b) { return a / (b * b); } };
template <typename R> struct dsigmoid { DI static R Map(R a) { return a * (((R)1.0) - a); } };
template <typename R> struct tanh     { DI static R Map(R a) { return (R)m_tanh(a); } };
template <typename R> struct inverse_tanh { DI static R Map(R a) { return (R)((m_log(1 + a) - m_log(1 - a)) * 0.5); } };
template <typename R> struct dtanh    { DI static R Map(R a) { return (R)(1.0 - a * a); } };
template <typename R> struct power    { DI static R Map(R a, R b) { return (R)m_pow(a, b); } };
template <typename R> struct abs      { DI static R Map(R a) { return m_abs(a); } };
template <typename R> struct log_or_zero { DI static R Map(R a) { return a > 0 ? (R)m_log(a) : (R)0; } };
template <typename R> struct sign     { DI static R Map(R x) { return x > 0.0 ? 1.0 : -1.0; } };
template <typename R> struct threshold { DI static R Map(R a, R b) { return a < b ? 1.0 : 0.0; } };
template <typename R> struct max_scalar { DI static R Map(R x, R y) { return x > y ? x : y; } };
template <typename R> struct min_scalar { DI static R Map(R x, R y) { return x < y ? x : y; } };
template <typename R> struct steep_sigmoid { DI static R Map(R x, R g) { return (R)(1.0 / (1.0 + (double)m_exp(-g * x))); } };
template <typename R> struct steep_sigmoid_backward { DI static R Map(R x, R g) { return g * (x - x * x); } };
template <typename R> struct relu     { DI static R Map(R x) { return x > 0.0 ? x : (R)0.0; } };
template <typename R> struct clipped_relu { DI static R Map(R x, R c) { return x > 0.0 ? (x > c ? c : x) : (R)0.0; } };
template <typename R> struct relu_backward { DI static R Map(R x) { return x > 0.0 ? 1.0 : 0.0; } };
template <typename R> struct clipped_relu_backward { DI static R Map(R x, R c) { return x > 0.0 ? (x > c ? 0.0 : 1.0) : 0.0; } };
template <typename R> struct clip {
    DI static R Map(R x, R c) { return x > c ? c : (x < -c ? -c : x); }
};
template <typename R> struct lessthanequal { DI static R Map(R x, R u) { return x <= u ? 1 : 0; } };
template <typename R> struct greaterthanequal { DI static R Map(R x, R l) { return x >= l ? 1 : 0; } };
template <typename R> struct binary_cross_entropy {
    DI static R Map(R x, R t) {
        R d1 = t * (R)m_log(x);
        R d0 = (R)((1.0 - t) * m_log(1. - (double)x));
        return -(d1 + d0);
    }
};
template <typename R> struct binary_cross_entropy_grad {
    DI static R Map(R x, R t) {
        R num = t - x;
        R den = (R)(x * (x - 1.0));
        return num / den;
    }
};
template <typename R> struct softplus {
    DI static R Map(R x) { return x > 20.0 ? x : (R)m_log((R)1.0 + (R)m_exp(x)); }
};
template <typename R> struct softplus_backward {
    DI static R Map(R x) { return x > 20.0 ? (R)1.0 : (R)((R)m_exp(x) / ((R)1.0 + (R)m_exp(x))); }
};
template <typename R> struct prelu { DI static R Map(R x, R w) { return x > 0 ? x : w * x; } };
template <typename R> struct prelu_backward_weights { DI static R Map(R x, R g) { return x > 0 ? (R)0 : x * g; } };
template <typename R> struct prelu_backward_inputs { DI static R Map(R x, R w) { return x > 0 ? (R)1.0 : w; } };
}  // namespace functor

// x / s for a divisor that is the same for every element a thread handles (a row value
// or a scalar): one true reciprocal per row, then per element a product and one FMA
// correction step, which yields the correctly rounded quotient except in rare last-place
// cases. Divisors whose reciprocal is not a normal number take the plain division.
DI float dali_div_invariant(float x, float s) {
    const float a = __builtin_fabsf(s);
    if (a > 1e-30f && a < 1e30f) {
        const float r = 1.0f / s;
        const float q = x * r;
        const float e = __builtin_fmaf(-q, s, x);
        return __builtin_fmaf(e, r, q);
    }
    return x / s;
}
// The same with the reciprocal and the range test hoisted out of the element loop by the kernel generator.
DI bool dali_div_ok(float s) {
    const float a = __builtin_fabsf(s);
    return a > 1e-30f && a < 1e30f;
}
DI float dali_div_fast(float x, float s, float r) {
    const float q = x * r;
    const float e = __builtin_fmaf(-q, s, x);
    return __builtin_fmaf(e, r, q);
}
DI double dali_div_invariant(double x, double s) { return x / s; }
DI int dali_div_invariant(int x, int s) { return x / s; }

// n / d for 0 <= n < 2^31 and a divisor d >= 1 that the host knows at launch. With 2^(s-1) < d <= 2^s the host
// passes m = ceil(2^(31+s) / d), which fits 32 bits. Then n * m / 2^(31+s) = n / d + n * e / (d * 2^(31+s)) with
// 0 <= e < d <= 2^s, and the second term is below 1 / d, the distance from n / d to the next integer, so the
// floor of the product is floor(n / d).
DI unsigned dali_udiv(unsigned n, unsigned m, int s) { return (unsigned)(((unsigned long long)n * m) >> (31 + s)); }

// one_hot element. The reference evaluates on*is_on + (1.0 - is_on)*off with is_on in T and
// the rest in double (dali/array/op/one_hot.cpp:38-46). With is_on in {0, 1} that is
// on + 0*off when the index matches and on*0 + off otherwise, and both forms round to
// the same T as the double evaluation (the products are exact zeros or NaN), so the
// select below is bit-identical, including inf / NaN propagation.
// index into an axis of n entries, held inside it: what a gather reads for an index outside its source
DI int dali_clamp_index(int i, int n) { return i < 0 ? 0 : (i >= n ? n - 1 : i); }

template <typename T>
DI T dali_one_hot(int index, int column, T on, T off) {
    return index == column ? (T)(on + (T)0 * off) : (T)(on * (T)0 + off);
}

// ------------------------------------------------------------------ reducers
namespace reducers {
struct sum {
    template <typename T> DI static T init() { return (T)0; }
    template <typename T> DI static T step(T d, T s) { return d + s; }
    template <typename T> DI static bool better(T cand, T cur) { return false; }
};
struct product {
    template <typename T> DI static T init() { return (T)1; }
    template <typename T> DI static T step(T d, T s) { return d * s; }
    template <typename T> DI static bool better(T cand, T cur) { return false; }
};
template <typename T> DI T lowest();
template <> DI float lowest<float>() { return -DALI_FLT_MAX; }
template <> DI double lowest<double>() { return -DALI_DBL_MAX; }
template <> DI int lowest<int>() { return DALI_INT_MIN; }
template <typename T> DI T highest();
template <> DI float highest<float>() { return DALI_FLT_MAX; }
template <> DI double highest<double>() { return DALI_DBL_MAX; }
template <> DI int highest<int>() { return DALI_INT_MAX; }
// float and double: fmax / fmin, one instruction each, which is also what the reference's device code calls
// (dali/array/jit/reducer_kernels.h:92-98,127-131 under __CUDACC__); on numbers it equals the host form
// `dst > src ? dst : src`, the two differ only in which operand survives a NaN.
DI float dali_max(float d, float s) { return __builtin_fmaxf(d, s); }
DI double dali_max(double d, double s) { return __builtin_fmax(d, s); }
DI int dali_max(int d, int s) { return d > s ? d : s; }
DI float dali_min(float d, float s) { return __builtin_fminf(d, s); }
DI double dali_min(double d, double s) { return __builtin_fmin(d, s); }
DI int dali_min(int d, int s) { return d < s ? d : s; }
struct maximum {
    template <typename T> DI static T init() { return lowest<T>(); }
    template <typename T> DI static T step(T d, T s) { return dali_max(d, s); }
    template <typename T> DI static bool better(T cand, T cur) { return cand > cur; }
};
struct minimum {
    template <typename T> DI static T init() { return highest<T>(); }
    template <typename T> DI static T step(T d, T s) { return dali_min(d, s); }
    template <typename T> DI static bool better(T cand, T cur) { return cand < cur; }
};
// Running (maximum, sum of exp(x - maximum)) of a softmax, for reductions against the memory layout where the values
// cannot stay in registers between a max pass and a sum pass: one pass over the data yields both. Feeding a value
// costs one exp (of minus the distance between the value and the running maximum; one of the two terms keeps the
// factor exp(0)); two partial results combine the same way. A fresh accumulator is (-FLT_MAX, 0).
struct dali_ms { float m, l; };
struct maxsumexp {
    template <typename T> DI static dali_ms init() { dali_ms r; r.m = -DALI_FLT_MAX; r.l = 0.0f; return r; }
    DI static dali_ms feed(dali_ms a, float x) {
        const float d = x - a.m;
        const float e = dali_expf(-__builtin_fabsf(d));
        dali_ms r;
        r.m = __builtin_fmaxf(a.m, x);
        r.l = d > 0.0f ? a.l * e + 1.0f : a.l + e;
        return r;
    }
    // N values at once: their maximum first, then one exp per value against the new running maximum and one to carry
    // the old sum over; the N exponentials are added among themselves before they meet the running sum.
    template <int N> DI static dali_ms feed_n(dali_ms a, const float* x) {
        float bm = x[0];
#pragma unroll
        for (int u = 1; u < N; ++u) bm = __builtin_fmaxf(bm, x[u]);
        dali_ms r;
        r.m = __builtin_fmaxf(a.m, bm);
        float s = 0.0f;
#pragma unroll
        for (int u = 0; u < N; ++u) s += dali_expf(x[u] - r.m);
        r.l = a.l * dali_expf(a.m - r.m) + s;
        return r;
    }
    template <typename T> DI static dali_ms step(dali_ms a, dali_ms b) {
        const float d = b.m - a.m;
        const float e = dali_expf(-__builtin_fabsf(d));
        dali_ms r;
        r.m = __builtin_fmaxf(a.m, b.m);
        r.l = d > 0.0f ? a.l * e + b.l : a.l + b.l * e;
        return r;
    }
};
}  // namespace reducers
using reducers::dali_ms;

// ------------------------------------------------- cross-workgroup hand-off
// Agent-scope relaxed atomics: the store is written through to the coherence point
// shared by all XCDs, the load does not return a stale line of the local L2.
template <typename T> DI void dali_publish(T* p, T v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
template <typename T> DI T dali_observe(const T* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
DI void dali_publish(dali_ms* p, dali_ms v) {
    __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
DI dali_ms dali_observe(const dali_ms* p) {
    return __builtin_bit_cast(dali_ms, __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
// Waits until this thread's earlier stores are acknowledged by memory; also a compiler barrier for memory operations.
DI void dali_stores_acknowledged() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }
// Waits until this thread's earlier stores are acknowledged by memory, then draws a ticket. The wait is written as an asm
// statement that clobbers memory: the compiler may then move neither the published stores behind it nor the ticket (or the
// loads of the fold that follows it) in front of it.
DI unsigned int dali_take_ticket(unsigned int* counter) {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    const unsigned int ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("" ::: "memory");
    return ticket;
}

// Whether workgroup b is the last of n to arrive. One counter takes an arrival every 12 ns or so, whoever asks: tens of
// thousands of workgroups of a short kernel would queue for it (65536 rows of 513 in one launch: 200 us, of which 130 us
// waiting for tickets). From 1024 workgroups on they arrive in 64 groups with a counter each, counters[1 + group], and the
// last of a group, which sets its counter back to zero, draws from counters[0] for the group. Every arrival has had its
// earlier stores acknowledged, so what all of them published is in memory when the last one is told so. counters[0] is left
// at n (or 64) for the caller to set back.
DI bool dali_last_arrival(unsigned int* counters, unsigned int b, unsigned int n) {
    constexpr unsigned int kGroups = 64;
    if (n < 1024) return dali_take_ticket(&counters[0]) == n - 1;
    const unsigned int group = b % kGroups, members = (n - group + kGroups - 1) / kGroups;
    if (dali_take_ticket(&counters[1 + group]) != members - 1) return false;
    dali_publish(&counters[1 + group], 0u);
    return dali_take_ticket(&counters[0]) == kGroups - 1;
}

// --------------------------------------------------------- cross-lane helpers
template <typename T> DI T dali_shfl_xor(T v, int mask) { return __shfl_xor(v, mask, 64); }
template <> DI double dali_shfl_xor<double>(double v, int mask) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __shfl_xor(lo, mask, 64);
    hi = __shfl_xor(hi, mask, 64);
    return __hiloint2double(hi, lo);
}

template <typename T> DI T dali_shfl_up(T v, int delta) { return __shfl_up(v, delta, 64); }
template <> DI double dali_shfl_up<double>(double v, int delta) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __shfl_up(lo, delta, 64);
    hi = __shfl_up(hi, delta, 64);
    return __hiloint2double(hi, lo);
}
template <typename T> DI T dali_shfl(T v, int lane) { return __shfl(v, lane, 64); }
template <> DI double dali_shfl<double>(double v, int lane) {
    int lo = __double2loint(v), hi = __double2hiint(v);
    lo = __shfl(lo, lane, 64);
    hi = __shfl(hi, lane, 64);
    return __hiloint2double(hi, lo);
}
// Inclusive scan over the 64 lanes of a wave: lane l ends with step(v_0, ..., v_l), combined left to right.
template <typename R, typename T>
DI T dali_wave_scan(T v) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const T o = dali_shfl_up<T>(v, d);
        if (lane >= d) v = R::template step<T>(o, v);
    }
    return v;
}

// A lane's value as another lane holds it, moved by the data-parallel-primitive path of the vector ALU (a few
// cycles) instead of through the LDS crossbar that __shfl uses (a round trip of its own per step). CTRL: 0xB1 / 0x4E
// swap neighbours / pairs inside a quad, 0x141 / 0x140 mirror a half row / a row of 16 lanes, 0x142 / 0x143 hand
// lane 15 of every row to the next row / lane 31 to the upper half; ROW_MASK picks the rows of 16 lanes that receive
// (the others keep their value).
template <int CTRL, int ROW_MASK>
DI int dali_dpp_word(int v) { return __builtin_amdgcn_update_dpp(v, v, CTRL, ROW_MASK, 0xF, false); }
template <typename T, int CTRL, int ROW_MASK>
DI T dali_dpp(T v) {
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, dali_dpp_word<CTRL, ROW_MASK>(__builtin_bit_cast(int, v)));
    } else {
        static_assert(sizeof(T) == 8, "4- or 8-byte values");
        long long w = __builtin_bit_cast(long long, v);
        const int lo = dali_dpp_word<CTRL, ROW_MASK>((int)w), hi = dali_dpp_word<CTRL, ROW_MASK>((int)(w >> 32));
        return __builtin_bit_cast(T, ((long long)hi << 32) | (unsigned int)lo);
    }
}
template <typename T>
DI T dali_readlane(T v, int lane) {
    if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
    } else {
        long long w = __builtin_bit_cast(long long, v);
        const int lo = __builtin_amdgcn_readlane((int)w, lane), hi = __builtin_amdgcn_readlane((int)(w >> 32), lane);
        return __builtin_bit_cast(T, ((long long)hi << 32) | (unsigned int)lo);
    }
}

// Reduce over aligned groups of WIDTH lanes (WIDTH a power of two <= 64); every
// lane of the group ends with the group's result. Groups of up to 16 lanes stay inside a row of the data-parallel
// path (exchange inside quads, then mirrored halves: after every step the lanes that have met hold the same value);
// 32 lanes add one exchange through the crossbar; a whole wave adds two row hand-offs, which leave the result in
// lane 63, and reads that lane for everybody (a scalar from there on).
template <typename R, typename T, int WIDTH>
DI T dali_group_reduce(T v) {
    if constexpr (WIDTH >= 2) v = R::template step<T>(v, dali_dpp<T, 0xB1, 0xF>(v));
    if constexpr (WIDTH >= 4) v = R::template step<T>(v, dali_dpp<T, 0x4E, 0xF>(v));
    if constexpr (WIDTH >= 8) v = R::template step<T>(v, dali_dpp<T, 0x141, 0xF>(v));
    if constexpr (WIDTH >= 16) v = R::template step<T>(v, dali_dpp<T, 0x140, 0xF>(v));
    if constexpr (WIDTH == 32) v = R::template step<T>(v, dali_shfl_xor<T>(v, 16));
    if constexpr (WIDTH == 64) {
        v = R::template step<T>(v, dali_dpp<T, 0x142, 0xA>(v));
        v = R::template step<T>(v, dali_dpp<T, 0x143, 0xC>(v));
        v = dali_readlane<T>(v, 63);
    }
    return v;
}

// (value, index) variant: a candidate wins when its value is strictly better, or
// equal with a lower index, which reproduces "first index on ties" of a sequential scan.
template <typename R, typename T, int WIDTH>
DI void dali_group_arg_reduce(T& v, int& idx) {
#pragma unroll
    for (int m = WIDTH / 2; m >= 1; m >>= 1) {
        T ov = dali_shfl_xor<T>(v, m);
        int oi = __shfl_xor(idx, m, 64);
        if (R::template better<T>(ov, v) || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
}

// Reduce over the NW waves of a workgroup through LDS. `sm` must hold NW values
// and be private to this call site (no barrier is needed before reusing other
// slots). Every thread returns the workgroup's result, combined in wave order.
template <typename R, typename T, int NW>
DI T dali_block_reduce(T v, T* sm) {
    v = dali_group_reduce<R, T, 64>(v);
    if constexpr (NW == 1) return v;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) sm[wave] = v;
    __syncthreads();
    T r = sm[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) r = R::template step<T>(r, sm[w]);
    return r;
}

template <typename R, typename T, int NW>
DI void dali_block_arg_reduce(T& v, int& idx, T* smv, int* smi) {
    dali_group_arg_reduce<R, T, 64>(v, idx);
    if constexpr (NW == 1) return;
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { smv[wave] = v; smi[wave] = idx; }
    __syncthreads();
    T r = smv[0];
    int ri = smi[0];
#pragma unroll
    for (int w = 1; w < NW; ++w) {
        T ov = smv[w];
        int oi = smi[w];
        if (R::template better<T>(ov, r) || (ov == r && oi < ri)) { r = ov; ri = oi; }
    }
    v = r;
    idx = ri;
}
)HIPSRC";

}  // namespace codegen
}  // namespace dali

#endif
