// Shared state of the fused-expression path and the one place where a generated kernel meets the device library: the
// identity (hash and entry-point name) of a kernel, the hand-over of its source to dali_hip_module_load on a miss, the
// six argument arrays of a launch (dali/array/jit/jit.cpp:1209-1223) and the recording of launches for replay.
#include "jit_internal.h"
#include "device_prelude.h"

namespace dali {
namespace jit {

const char* device_prelude() { return codegen::kDevicePrelude; }

// Bump when generated code changes meaning, so stale on-disk code objects are not reused.
const char* const kCodegenVersion = "dali-hip-codegen-38";

static std::unordered_map<uint64_t, bool>& loaded_hashes() {
    static std::unordered_map<uint64_t, bool> m;
    return m;
}

// The identity of a generated kernel, also the name of its code object on disk: besides the structure of the request it
// covers everything else that shapes the code (the generator's version, the device support code prepended to every kernel
// and the compiler options), so an edit to any of those cannot meet a stale code object.
uint64_t kernel_hash(const std::string& kind, const std::string& sig, const std::string& params) {
    static const uint64_t toolchain = Hasher().add(std::string(device_prelude())).add(std::string(dali_hip_rtc_options())).value();
    return Hasher().add(std::string(kCodegenVersion)).add(toolchain).add(kind).add(sig).add(params).value();
}

// entry-point name: shape + hash, so that a profile tells the generated kernels apart
std::string kernel_name(const std::string& kind, uint64_t hash) {
    char buf[64];
    snprintf(buf, sizeof(buf), "dali_%s_%016llx", kind.c_str(), (unsigned long long)hash);
    return buf;
}

LaunchCapture* g_capture = nullptr;

bool g_capture_compare_only = false;  // checking mode: the planner runs beside a cached plan and must not launch

void load_and_launch(KernelSpec& K, const std::function<std::string()>& gen, const Program& P,
                     const std::vector<std::vector<int>>& shapes) {
    if (g_capture) {
        g_capture->launches++;
        g_capture->K = &K;
        g_capture->arrays = P.arrays;
        g_capture->scalars = P.scalars;
        g_capture->shapes = shapes;
        if (g_capture_compare_only) return;
    }
    DALI_SCOPE("JIT[" + K.kind + ":" + K.name + "]");
    JitStats& st = jit_stats();
    static const bool trace_plan = getenv("DALI_HIP_TRACE_PLAN") != nullptr;  // one line per planned launch on stderr
    if (trace_plan) fprintf(stderr, "[dali-hip plan] %s\n", K.name.c_str());
    if (!st.last_kernel_kinds.empty()) st.last_kernel_kinds += ",";
    st.last_kernel_kinds += K.kind;
    if (!st.last_kernel_names.empty()) st.last_kernel_names += ",";
    st.last_kernel_names += K.name;
    bool need_source = g_dry_run || !loaded_hashes().count(K.hash);
    if (g_dry_run) {
        std::string src = gen();
        g_last_source += src;
        if (g_dry_sources) g_dry_sources->push_back(src);
        if (g_dry_compile) {
            size_t sz = 0;
            check_hip(dali_hip_compile_only(src.c_str(), &sz), "hipRTC compile of generated kernel");
        }
        st.plans_built++;
        return;
    }
    if (need_source) {
        DALI_SCOPE("get_function");
        int cached = 0;
        if (dali_hip_module_is_loaded(K.hash)) {
            cached = 2;
        } else {
            std::string src = gen();
            g_last_source += src;
            st.plans_built++;
            std::unique_ptr<Scope> compilation;
            if (Scope::has_observers()) compilation.reset(new Scope(std::make_shared<std::string>("compilation")));
            check_hip(dali_hip_module_load(K.hash, src.c_str(), K.name.c_str(), &K.plan, &cached), "JIT module load");
        }
        loaded_hashes()[K.hash] = true;
    }
    // six argument arrays (dali/array/jit/jit.cpp:1209-1223)
    size_t na = P.arrays.size();
    std::vector<void*> data(na);
    std::vector<int> offsets(na);
    std::vector<const int*> sizes(na), strides(na);
    for (size_t i = 0; i < na; ++i) {
        const ArrayArg& a = P.arrays[i];
        memory::AM mode = a.is_dest ? memory::AM_MUTABLE : memory::AM_READONLY;
        data[i] = a.buf->memory->data(memory::DEVICE_T_GPU, mode);
        offsets[i] = a.buf->offset;
        sizes[i] = a.sizes.data();
        strides[i] = a.strided ? a.strides.data() : nullptr;
    }
    std::vector<const void*> scalars(P.scalars.size());
    for (size_t j = 0; j < P.scalars.size(); ++j) {
        const ScalarArg& s = P.scalars[j];
        scalars[j] = s.dtype == DTYPE_FLOAT ? (const void*)&s.f : (s.dtype == DTYPE_DOUBLE ? (const void*)&s.d : (const void*)&s.i);
    }
    std::vector<const int*> shp(shapes.size());
    for (size_t k = 0; k < shapes.size(); ++k) shp[k] = shapes[k].data();
    check_hip(dali_hip_launch(K.hash, data.data(), offsets.data(), sizes.data(), strides.data(), scalars.data(), shp.data()),
              "kernel launch");
    st.kernels_launched++;
    if (g_recording) {
        for (const ArrayArg& a : P.arrays)
            if (a.is_dest) note_recorded_write(a.buf->memory);
        uint64_t hash = K.hash;
        auto arrays = std::make_shared<std::vector<ArrayArg>>(P.arrays);
        auto scal = std::make_shared<std::vector<ScalarArg>>(P.scalars);
        auto shapes_copy = std::make_shared<std::vector<std::vector<int>>>(shapes);
        auto data_copy = std::make_shared<std::vector<void*>>(data);
        auto offsets_copy = std::make_shared<std::vector<int>>(offsets);
        g_recording->push_back([hash, arrays, scal, shapes_copy, data_copy, offsets_copy]() {
            size_t n = arrays->size();
            std::vector<const int*> sz(n), sd(n);
            for (size_t i = 0; i < n; ++i) {
                sz[i] = (*arrays)[i].sizes.data();
                sd[i] = (*arrays)[i].strided ? (*arrays)[i].strides.data() : nullptr;
            }
            std::vector<const void*> sc(scal->size());
            for (size_t j = 0; j < scal->size(); ++j) {
                const ScalarArg& s = (*scal)[j];
                sc[j] = s.dtype == DTYPE_FLOAT ? (const void*)&s.f : (s.dtype == DTYPE_DOUBLE ? (const void*)&s.d : (const void*)&s.i);
            }
            std::vector<const int*> sh(shapes_copy->size());
            for (size_t k = 0; k < shapes_copy->size(); ++k) sh[k] = (*shapes_copy)[k].data();
            check_hip(dali_hip_launch(hash, data_copy->data(), offsets_copy->data(), sz.data(), sd.data(), sc.data(), sh.data()),
                      "kernel replay");
        });
    }
}

// dest access: a destination that is fully overwritten does not need its old contents migrated
static void mark_dest_modes(Program& P, const std::vector<Output>& outs) {
    (void)P;
    (void)outs;
}

}  // namespace jit

using namespace jit;

bool g_dry_run = false;

bool g_dry_compile = false;

std::vector<std::string>* g_dry_sources = nullptr;

void set_dry_run(bool on) { g_dry_run = on; }

void set_dry_compile(bool on) { g_dry_compile = on; }

bool dry_run() { return g_dry_run; }

JitStats& jit_stats() {
    static JitStats s;
    return s;
}

std::string g_last_source;

const std::string& last_generated_source() { return g_last_source; }

// Launch recording: while a recording is open every kernel / GEMM launch is also
// stored as a closure (owning copies of its argument arrays and of the buffers it
// touches) so that a steady-state loop can re-issue exactly the same device work
// without rebuilding and re-planning the expression.
std::vector<std::function<void()>>* g_recording = nullptr;

// memories the recorded launches write: a replay bypasses the access-mode calls of a
// normal evaluation, so their host copies must be declared stale by the replayer
std::vector<std::shared_ptr<memory::SynchronizedMemory>>* g_recording_written = nullptr;

void set_recording(std::vector<std::function<void()>>* rec, std::vector<std::shared_ptr<memory::SynchronizedMemory>>* written) {
    g_recording = rec;
    g_recording_written = written;
}

void note_recorded_write(const std::shared_ptr<memory::SynchronizedMemory>& m) {
    if (!g_recording_written) return;
    for (auto& w : *g_recording_written)
        if (w == m) return;
    g_recording_written->push_back(m);
}

}  // namespace dali
