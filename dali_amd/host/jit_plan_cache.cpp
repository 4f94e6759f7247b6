// The plan cache: a request that repeats (same expression structure, dtypes, shapes classes and layouts) skips
// classification and code generation and re-binds the arrays of the cached launches.
#include "jit_internal.h"

namespace dali {
namespace jit {

// Planning an expression (classification, kernel parameters, the structural signature and its hash) costs more
// host time than a small kernel runs. The outcome only depends on the structure of the request: node kinds,
// functors, dtypes, shapes, the layout of every buffer and which buffers share memory. That structure is written
// out as a word list by one walk; an outermost planning call that ended in exactly one kernel launch is stored
// under it, and the next request with the same words skips the planner: the stored argument layout is refilled
// with this request's buffers and literal values. Requests that the planner splits into several launches are not
// stored. Entries are compared word for word, so two structures never share a plan by accident.
struct PlanWalk {
    std::vector<uint64_t> words;
    std::vector<const Expr*> seen;
    std::vector<const void*> memories;
    std::vector<int> first_offsets;
    std::vector<std::shared_ptr<Expr>> buffers;  // in visiting order, destinations first
    std::vector<const Expr*> literals;

    void put(uint64_t v) { words.push_back(v); }
    void put_ints(const std::vector<int>& v) {
        put(v.size());
        for (int x : v) put((uint64_t)(uint32_t)x);
    }
    void visit(const Array& a) {
        const std::shared_ptr<Expr> ep = a.expression();
        const Expr* e = ep.get();
        for (size_t k = 0; k < seen.size(); ++k)
            if (seen[k] == e) {
                put(0xB000000000000000ull | k);  // a node met before: shared subexpression
                return;
            }
        seen.push_back(e);
        put(((uint64_t)e->kind) | ((uint64_t)e->dtype << 8) | ((uint64_t)(uint32_t)e->axis << 16));
        put((uint64_t)(uint32_t)e->depth);
        put(std::hash<std::string>()(e->name));
        put(std::hash<std::string>()(e->data_format));
        put_ints(e->geom);
        put_ints(e->shape);
        if (e->kind == Kind::BUFFER) {
            // which of the request's allocations (in-place and shared operands plan differently), the alignment class
            // of the view, and for a further view of an allocation its distance from the first one
            size_t m = 0;
            while (m < memories.size() && memories[m] != e->memory.get()) ++m;
            const bool first_view = m == memories.size();
            if (first_view) {
                memories.push_back(e->memory.get());
                first_offsets.push_back(e->offset);
            }
            put(m);
            put((uint64_t)(uint32_t)(e->offset % 16));
            put(first_view ? 0xF000000000000000ull : (uint64_t)(uint32_t)(e->offset - first_offsets[m]));
            put_ints(e->strides);
            buffers.push_back(ep);
        } else if (e->kind == Kind::SCALAR) {
            literals.push_back(e);
        } else {
            put(e->args.size());
            for (const Array& x : e->args) visit(x);
        }
    }
};

struct CachedPlan {
    std::vector<uint64_t> words;
    KernelSpec* K = nullptr;
    std::vector<ArrayArg> arrays;      // layouts as planned; `buf` is refilled per request and dropped after the launch
    std::vector<ScalarArg> scalars;
    std::vector<std::vector<int>> shapes;
    std::vector<int> array_source;     // index into PlanWalk::buffers
    std::vector<int> scalar_source;    // index into PlanWalk::literals
};

static std::unordered_map<uint64_t, std::vector<CachedPlan>>& plan_cache() {
    static std::unordered_map<uint64_t, std::vector<CachedPlan>> c;
    return c;
}

static uint64_t fold_words(const std::vector<uint64_t>& w) {
    uint64_t h = 0x9E3779B97F4A7C15ull;
    for (uint64_t v : w) {
        h = (h ^ v) * 0xFF51AFD7ED558CCDull;
        h ^= h >> 29;
    }
    return h;
}

static bool same_view(const Expr* a, const Expr* b) {
    return a->memory.get() == b->memory.get() && a->offset == b->offset && a->dtype == b->dtype && a->shape == b->shape && a->strides == b->strides;
}

void run_specs(std::vector<DestSpec> specs) {
    static const bool cache_off = env_int("DALI_HIP_PLAN_CACHE", 1) == 0;
    static const bool cache_check = env_int("DALI_HIP_PLAN_CACHE_CHECK", 0) != 0;
    static int depth = 0;
    if (depth > 0 || cache_off || g_dry_run || g_capture) {
        run_specs_planned(std::move(specs));
        return;
    }
    struct Depth {
        Depth() { ++depth; }
        ~Depth() { --depth; }
    } guard;
    PlanWalk walk;
    for (const DestSpec& sp : specs) {
        walk.put(0xD000000000000000ull | (uint64_t)sp.op);
        walk.visit(sp.dest);
    }
    for (const DestSpec& sp : specs) walk.visit(sp.root);
    const uint64_t key = fold_words(walk.words);
    std::vector<CachedPlan>& bucket = plan_cache()[key];
    CachedPlan* hit = nullptr;
    for (CachedPlan& c : bucket)
        if (c.words == walk.words) hit = &c;
    JitStats& st = jit_stats();
    if (hit) {
        if (cache_check) {
            // run the planner beside the stored plan: it must arrive at the same kernel and argument layout
            LaunchCapture cap;
            g_capture = &cap;
            g_capture_compare_only = true;
            try {
                run_specs_planned(specs);
            } catch (...) {
                g_capture = nullptr;
                g_capture_compare_only = false;
                throw;
            }
            g_capture = nullptr;
            g_capture_compare_only = false;
            bool same = cap.launches == 1 && cap.K == hit->K && cap.shapes == hit->shapes && cap.arrays.size() == hit->arrays.size() &&
                        cap.scalars.size() == hit->scalars.size();
            for (size_t i = 0; same && i < cap.arrays.size(); ++i) {
                const ArrayArg &x = cap.arrays[i], &y = hit->arrays[i];
                same = x.nd == y.nd && x.strided == y.strided && x.sizes == y.sizes && x.strides == y.strides && x.is_dest == y.is_dest &&
                       same_view(x.buf.get(), walk.buffers[hit->array_source[i]].get());
            }
            for (size_t j = 0; same && j < cap.scalars.size(); ++j) same = cap.scalars[j].src == walk.literals[hit->scalar_source[j]];
            if (!same) throw std::runtime_error("plan cache: the stored plan differs from what the planner builds for this request");
        }
        for (size_t i = 0; i < hit->arrays.size(); ++i) hit->arrays[i].buf = walk.buffers[hit->array_source[i]];
        for (size_t j = 0; j < hit->scalars.size(); ++j) {
            const Expr* lit = walk.literals[hit->scalar_source[j]];
            hit->scalars[j].d = lit->dvalue;
            hit->scalars[j].f = (float)lit->dvalue;
            hit->scalars[j].i = lit->ivalue;
        }
        Program P;
        P.arrays.swap(hit->arrays);
        P.scalars.swap(hit->scalars);
        try {
            load_and_launch(*hit->K, []() -> std::string { throw std::runtime_error("plan cache: the stored kernel is no longer loaded"); }, P, hit->shapes);
        } catch (...) {
            bucket.clear();
            throw;
        }
        hit->arrays.swap(P.arrays);
        hit->scalars.swap(P.scalars);
        for (ArrayArg& a : hit->arrays) a.buf.reset();  // the cache must not keep a request's memory alive
        st.plan_cache_hits++;
        return;
    }
    // miss: plan as usual, remembering what was launched
    const uint64_t kernels0 = st.kernels_launched, gemms0 = st.gemms_launched, evals0 = st.evals;
    LaunchCapture cap;
    g_capture = &cap;
    try {
        run_specs_planned(specs);
    } catch (...) {
        g_capture = nullptr;
        throw;
    }
    g_capture = nullptr;
    if (cap.launches != 1 || st.kernels_launched - kernels0 != 1 || st.gemms_launched != gemms0 || st.evals != evals0) return;
    CachedPlan plan;
    plan.K = cap.K;
    plan.shapes = cap.shapes;
    for (const ArrayArg& a : cap.arrays) {
        int src = -1;
        for (size_t k = 0; k < walk.buffers.size() && src < 0; ++k)
            if (walk.buffers[k].get() == a.buf.get() || same_view(walk.buffers[k].get(), a.buf.get())) src = (int)k;
        if (src < 0) return;  // the planner made this operand itself (a temporary or a reshaped view)
        plan.array_source.push_back(src);
        plan.arrays.push_back(a);
        plan.arrays.back().buf.reset();
    }
    for (const ScalarArg& sc : cap.scalars) {
        int src = -1;
        for (size_t k = 0; k < walk.literals.size() && src < 0; ++k)
            if (walk.literals[k] == sc.src) src = (int)k;
        if (src < 0) return;
        plan.scalar_source.push_back(src);
        plan.scalars.push_back(sc);
    }
    plan.words = std::move(walk.words);
    static size_t stored = 0;
    if (stored >= 16384) {  // a bound on what a long-running process can accumulate: start over
        plan_cache().clear();
        stored = 0;
        plan_cache()[key].push_back(std::move(plan));
    } else if (bucket.size() < 8) {
        bucket.push_back(std::move(plan));
    }
    ++stored;
    st.plan_cache_stored++;
}

}  // namespace jit

}  // namespace dali
