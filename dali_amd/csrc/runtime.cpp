// Device, memory, code-object cache and launcher of the C ABI declared in
// include/dali_hip.h. Host code only; compiled with hipcc for the HIP headers.
//
// One process drives one MI355X: a single non-blocking stream orders every
// launch and copy, a size-keyed bank recycles device blocks, and one persistent
// workspace holds the partial results and self-resetting counters of the
// two-stage reduction kernels.
#include "runtime.h"

#include <hip/hiprtc.h>
#include <dirent.h>
#include <sys/stat.h>
#include <sys/types.h>
#include <unistd.h>

#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace dali_hip {

static thread_local std::string g_last_error;

int fail(const char* fmt, ...) {
    char buf[4096];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return DALI_HIP_ERROR;
}

int fail_str(const std::string& s) {
    g_last_error = s;
    return DALI_HIP_ERROR;
}

struct Runtime {
    std::mutex mu;
    bool ready = false;
    int device = -1;
    hipStream_t stream = nullptr;
    // migrations that should not stall the compute stream run here (created on first use, default priority)
    hipStream_t copy_stream = nullptr;
    hipEvent_t order_event = nullptr;
    std::string arch = "gfx950";
    // workspace: [counters | partials]
    char* ws = nullptr;
    // bank: size class -> parked blocks. Blocks up to kSlabBlockMax are carved out of large slabs (a driver
    // allocation costs tens to hundreds of microseconds whatever its size); larger ones are driver allocations
    std::unordered_map<size_t, std::vector<void*>> bank;
    size_t bank_parked = 0, bank_live = 0;
    std::vector<char*> slabs;
    size_t slab_used = 0;  // bytes handed out from the newest slab
    // modules
    struct Module {
        hipModule_t module = nullptr;
        hipFunction_t fn = nullptr;
        dali_hip_launch_plan plan;
        std::vector<int32_t> array_ndim, array_strided, array_elsize, scalar_dtype, shape_ndim;
        size_t karg_bytes = 0;
        int n_iv = 0;
    };
    std::unordered_map<uint64_t, Module> modules;
    std::unordered_map<uint64_t, bool> recompiled_once;
    // code objects loaded ahead of their first use by dali_hip_cache_warm (no launch plan yet)
    std::unordered_map<uint64_t, hipModule_t> preloaded;
    std::string cache_dir;
    uint64_t n_compiled = 0, n_disk = 0, n_launch = 0;
};

static Runtime& rt() {
    static Runtime r;
    return r;
}

hipStream_t stream() { return rt().stream; }
char* workspace() { return rt().ws; }
int bound_device() { return rt().ready ? rt().device : -1; }

int ensure_init() {
    if (rt().ready) return DALI_HIP_OK;
    return dali_hip_init(0);
}

static std::string default_cache_dir() {
    const char* env = getenv("DALI_HIP_CACHE_DIR");
    if (env && *env) return env;
    const char* home = getenv("HOME");
    std::string base = (home && *home) ? home : "/tmp";
    return base + "/.dali/cache_hip";
}

static void mkdir_p(const std::string& path) {
    std::string cur;
    for (size_t i = 0; i < path.size(); ++i) {
        cur.push_back(path[i]);
        if (path[i] == '/' || i + 1 == path.size()) {
            if (cur != "/") mkdir(cur.c_str(), 0755);
        }
    }
}

static std::string hash_hex(uint64_t h) {
    char buf[32];
    snprintf(buf, sizeof(buf), "%016llx", (unsigned long long)h);
    return buf;
}

static bool env_true(const char* name) {
    const char* v = getenv(name);
    if (!v) return false;
    std::string s(v);
    return s == "true" || s == "1" || s == "TRUE" || s == "True";
}

// Options every generated kernel is compiled with (besides the target). No fast-math and no contraction: the CPU path
// this is checked against is built without either (dali/utils/compiler.cpp:137-145). The leading kernel parameters (up
// to the 14 scalar registers the hardware offers) arrive preloaded with the wave instead of through a load at its start.
static const char* const kRtcOptions[] = {"-O3", "-ffp-contract=off", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                                          "-mllvm", "-amdgpu-kernarg-preload-count=14"};

// hipRTC: source -> gfx code object
static int rtc_compile(const std::string& arch, const char* src, std::vector<char>* code, std::string* log) {
    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, src, "dali_jit.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) return fail("hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
    std::string arch_opt = "--offload-arch=" + arch;
    std::vector<const char*> opts = {arch_opt.c_str()};
    for (const char* o : kRtcOptions) opts.push_back(o);
    r = hiprtcCompileProgram(prog, (int)opts.size(), opts.data());
    size_t log_size = 0;
    hiprtcGetProgramLogSize(prog, &log_size);
    if (log_size > 1) {
        log->resize(log_size);
        hiprtcGetProgramLog(prog, &(*log)[0]);
    }
    if (r != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&prog);
        return fail("hipRTC compile failed (%s):\n%s", hiprtcGetErrorString(r), log->c_str());
    }
    size_t code_size = 0;
    hiprtcGetCodeSize(prog, &code_size);
    code->resize(code_size);
    hiprtcGetCode(prog, code->data());
    hiprtcDestroyProgram(&prog);
    return DALI_HIP_OK;
}

hipError_t reserve_dynamic_lds(const void* kernel, size_t bytes) {
    static std::mutex m;
    static std::unordered_map<const void*, size_t> reserved;
    std::lock_guard<std::mutex> lock(m);
    auto it = reserved.find(kernel);
    if (it != reserved.end() && it->second >= bytes) return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e == hipSuccess) reserved[kernel] = bytes;
    return e;
}

}  // namespace dali_hip

using namespace dali_hip;

#define HIP_TRY(expr)                                                                      \
    do {                                                                                   \
        hipError_t e__ = (expr);                                                           \
        if (e__ != hipSuccess) return fail("%s failed: %s", #expr, hipGetErrorString(e__)); \
    } while (0)

extern "C" {

const char* dali_hip_last_error(void) { return g_last_error.c_str(); }

int dali_hip_device_count(int* count) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        return fail("hipGetDeviceCount failed: %s", hipGetErrorString(e));
    }
    *count = n;
    return DALI_HIP_OK;
}

int dali_hip_init(int device) {
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (r.ready && r.device == device) return DALI_HIP_OK;
    if (r.ready) return fail("dali_hip_init: already bound to device %d", r.device);
    int n = 0;
    HIP_TRY(hipGetDeviceCount(&n));
    if (device < 0 || device >= n) return fail("dali_hip_init: no device %d (have %d)", device, n);
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    std::string arch = prop.gcnArchName;
    size_t colon = arch.find(':');
    if (colon != std::string::npos) arch = arch.substr(0, colon);
    r.arch = arch;
    HIP_TRY(hipStreamCreateWithFlags(&r.stream, hipStreamNonBlocking));
    HIP_TRY(hipMalloc((void**)&r.ws, kWorkspaceBytes));
    HIP_TRY(hipMemsetAsync(r.ws, 0, kWorkspaceBytes, r.stream));
    HIP_TRY(hipStreamSynchronize(r.stream));
    if (sort_scratch_init(device)) return DALI_HIP_ERROR;
    r.device = device;
    r.ready = true;
    return DALI_HIP_OK;
}

int dali_hip_device_name(int device, char* name, size_t name_len, char* arch, size_t arch_len) {
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (name && name_len) snprintf(name, name_len, "%s", prop.name);
    if (arch && arch_len) snprintf(arch, arch_len, "%s", prop.gcnArchName);
    return DALI_HIP_OK;
}

int dali_hip_mem_info(size_t* free_bytes, size_t* total_bytes) {
    if (ensure_init()) return DALI_HIP_ERROR;
    HIP_TRY(hipMemGetInfo(free_bytes, total_bytes));
    return DALI_HIP_OK;
}

// after the stream has drained: did a persistent kernel abandon a grid barrier?
static int check_persistent_status() {
    if (persistent_status_take())
        return fail("a persistent kernel gave up waiting at a grid barrier (its workgroups were not all resident in time); its outputs are undefined");
    return DALI_HIP_OK;
}

int dali_hip_sync(void) {
    if (ensure_init()) return DALI_HIP_ERROR;
    HIP_TRY(hipStreamSynchronize(rt().stream));
    return check_persistent_status();
}

void* dali_hip_stream(void) {
    if (ensure_init()) return nullptr;
    return (void*)rt().stream;
}

// true while the library stream records into a graph: what would be baked into the graph and then reused or released
// behind its back (bank blocks, driver allocations) or is known to misbehave in a replayed graph (memset nodes) is refused
static bool stream_is_capturing() {
    Runtime& r = rt();
    if (!r.ready) return false;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(r.stream, &cs) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return cs != hipStreamCaptureStatusNone;
}

int dali_hip_malloc(void** ptr, size_t bytes) {
    if (ensure_init()) return DALI_HIP_ERROR;
    *ptr = nullptr;
    if (stream_is_capturing()) return fail("dali_hip_malloc: not allowed while the library stream is being captured");
    if (bytes == 0) bytes = 4;
    HIP_TRY(hipMalloc(ptr, bytes));
    return DALI_HIP_OK;
}

int dali_hip_free(void* ptr) {
    if (!ptr) return DALI_HIP_OK;
    if (ensure_init()) return DALI_HIP_ERROR;
    // a block may still be read by queued kernels
    HIP_TRY(hipStreamSynchronize(rt().stream));
    HIP_TRY(hipFree(ptr));
    return DALI_HIP_OK;
}

// Size class of a request: four classes per power of two above 256 bytes (at most 25% slack), so that
// requests of nearly equal size share parked blocks.
static size_t bank_class(size_t bytes) {
    if (bytes <= 256) return 256;
    size_t p = 256;
    while (p * 2 < bytes) p *= 2;  // p < bytes <= 2p
    const size_t step = p / 4;
    return p + (bytes - p + step - 1) / step * step;
}

constexpr size_t kSlabBytes = (size_t)64 << 20;
constexpr size_t kSlabBlockMax = (size_t)2 << 20;

int dali_hip_bank_allocate(void** ptr, size_t bytes) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (stream_is_capturing())
        return fail("dali_hip_bank_allocate: not allowed while the library stream is being captured (the block's address would be part of the "
                    "graph while the bank hands the block to others)");
    Runtime& r = rt();
    bytes = bank_class(bytes);
    {
        std::lock_guard<std::mutex> lock(r.mu);
        auto it = r.bank.find(bytes);
        if (it != r.bank.end() && !it->second.empty()) {
            *ptr = it->second.back();
            it->second.pop_back();
            r.bank_parked -= bytes;
            r.bank_live += bytes;
            return DALI_HIP_OK;
        }
        if (bytes <= kSlabBlockMax) {
            if (r.slabs.empty() || r.slab_used + bytes > kSlabBytes) {
                void* slab = nullptr;
                hipError_t se = hipMalloc(&slab, kSlabBytes);
                if (se != hipSuccess) {
                    (void)hipGetLastError();
                    slab = nullptr;  // fall through to a plain allocation of the block
                } else {
                    r.slabs.push_back((char*)slab);
                    r.slab_used = 0;
                }
            }
            if (!r.slabs.empty() && r.slab_used + bytes <= kSlabBytes) {
                *ptr = r.slabs.back() + r.slab_used;
                r.slab_used += bytes;  // classes are multiples of 64 bytes above 256: blocks stay 256-byte aligned
                r.slab_used = (r.slab_used + 255) / 256 * 256;
                r.bank_live += bytes;
                return DALI_HIP_OK;
            }
        }
    }
    *ptr = nullptr;
    hipError_t e = hipMalloc(ptr, bytes);
    if (e == hipErrorOutOfMemory) {
        // give parked blocks back to the driver and retry once
        (void)hipGetLastError();
        dali_hip_bank_clear();
        e = hipMalloc(ptr, bytes);
    }
    if (e != hipSuccess) return fail("hipMalloc(%zu bytes) failed: %s", bytes, hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(r.mu);
    r.bank_live += bytes;
    return DALI_HIP_OK;
}

int dali_hip_bank_deposit(void* ptr, size_t bytes) {
    if (!ptr) return DALI_HIP_OK;
    Runtime& r = rt();
    bytes = bank_class(bytes);
    std::lock_guard<std::mutex> lock(r.mu);
    // Same-stream ordering makes immediate reuse safe: a later kernel that
    // receives this block runs after every kernel already queued on it.
    r.bank[bytes].push_back(ptr);
    r.bank_parked += bytes;
    r.bank_live = r.bank_live >= bytes ? r.bank_live - bytes : 0;
    return DALI_HIP_OK;
}

int dali_hip_bank_clear(void) {
    Runtime& r = rt();
    if (!r.ready) return DALI_HIP_OK;
    HIP_TRY(hipStreamSynchronize(r.stream));
    std::lock_guard<std::mutex> lock(r.mu);
    // parked driver allocations go back to the driver; blocks carved from slabs stay parked (a slab is only
    // released as a whole, at process end)
    size_t kept = 0;
    for (auto it = r.bank.begin(); it != r.bank.end();) {
        if (it->first > kSlabBlockMax) {
            for (void* p : it->second) (void)hipFree(p);
            it = r.bank.erase(it);
        } else {
            kept += it->first * it->second.size();
            ++it;
        }
    }
    r.bank_parked = kept;
    return DALI_HIP_OK;
}

int dali_hip_bank_stats(size_t* parked_bytes, size_t* live_bytes) {
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (parked_bytes) *parked_bytes = r.bank_parked;
    if (live_bytes) *live_bytes = r.bank_live;
    return DALI_HIP_OK;
}

int dali_hip_memset_async(void* ptr, int value, size_t bytes) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (bytes == 0) return DALI_HIP_OK;
    if (stream_is_capturing()) return fail("dali_hip_memset_async: not allowed while the library stream is being captured (fill with a kernel instead)");
    HIP_TRY(hipMemsetAsync(ptr, value, bytes, rt().stream));
    return DALI_HIP_OK;
}

int dali_hip_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (bytes == 0) return DALI_HIP_OK;
    HIP_TRY(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, rt().stream));
    HIP_TRY(hipStreamSynchronize(rt().stream));
    return DALI_HIP_OK;
}

int dali_hip_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (bytes == 0) return DALI_HIP_OK;
    HIP_TRY(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, rt().stream));
    HIP_TRY(hipStreamSynchronize(rt().stream));
    return check_persistent_status();
}

int dali_hip_memcpy_d2d(void* dst_device, const void* src_device, size_t bytes) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (bytes == 0) return DALI_HIP_OK;
    HIP_TRY(hipMemcpyAsync(dst_device, src_device, bytes, hipMemcpyDeviceToDevice, rt().stream));
    return DALI_HIP_OK;
}

int dali_hip_host_alloc(void** ptr, size_t bytes) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (!ptr) return fail("dali_hip_host_alloc: ptr is NULL");
    HIP_TRY(hipHostMalloc(ptr, bytes ? bytes : 4, hipHostMallocDefault));
    return DALI_HIP_OK;
}

int dali_hip_host_free(void* ptr) {
    if (!ptr) return DALI_HIP_OK;
    HIP_TRY(hipHostFree(ptr));
    return DALI_HIP_OK;
}

// The copy stream starts a migration only after the work already issued on the compute stream (which may
// still read or write the device block), and tells the caller's event when the bytes have arrived.
static int async_copy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind, void* done_event, const char* what) {
    if (ensure_init()) return DALI_HIP_ERROR;
    Runtime& r = rt();
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    HIP_TRY(hipStreamIsCapturing(r.stream, &cs));
    if (cs != hipStreamCaptureStatusNone) return fail("%s: not allowed while the library stream is being captured", what);
    {
        std::lock_guard<std::mutex> lock(r.mu);
        if (!r.copy_stream) {
            HIP_TRY(hipStreamCreateWithFlags(&r.copy_stream, hipStreamNonBlocking));
            HIP_TRY(hipEventCreateWithFlags(&r.order_event, hipEventDisableTiming));
        }
    }
    HIP_TRY(hipEventRecord(r.order_event, r.stream));
    HIP_TRY(hipStreamWaitEvent(r.copy_stream, r.order_event, 0));
    if (bytes) HIP_TRY(hipMemcpyAsync(dst, src, bytes, kind, r.copy_stream));
    if (done_event) HIP_TRY(hipEventRecord((hipEvent_t)done_event, r.copy_stream));
    return DALI_HIP_OK;
}

int dali_hip_memcpy_h2d_async(void* dst_device, const void* src_pinned, size_t bytes, void* done_event) {
    return async_copy(dst_device, src_pinned, bytes, hipMemcpyHostToDevice, done_event, "dali_hip_memcpy_h2d_async");
}

int dali_hip_memcpy_d2h_async(void* dst_pinned, const void* src_device, size_t bytes, void* done_event) {
    return async_copy(dst_pinned, src_device, bytes, hipMemcpyDeviceToHost, done_event, "dali_hip_memcpy_d2h_async");
}

int dali_hip_stream_wait_event(void* event) {
    if (ensure_init()) return DALI_HIP_ERROR;
    if (!event) return fail("dali_hip_stream_wait_event: event is NULL");
    HIP_TRY(hipStreamWaitEvent(rt().stream, (hipEvent_t)event, 0));
    return DALI_HIP_OK;
}

int dali_hip_event_synchronize(void* event) {
    if (!event) return fail("dali_hip_event_synchronize: event is NULL");
    HIP_TRY(hipEventSynchronize((hipEvent_t)event));
    return DALI_HIP_OK;
}

int dali_hip_event_query(void* event, int* done) {
    if (!event || !done) return fail("dali_hip_event_query: NULL argument");
    hipError_t e = hipEventQuery((hipEvent_t)event);
    if (e != hipSuccess && e != hipErrorNotReady) return fail("dali_hip_event_query: %s", hipGetErrorString(e));
    *done = e == hipSuccess ? 1 : 0;
    return DALI_HIP_OK;
}

int dali_hip_set_cache_dir(const char* path) {
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    r.cache_dir = path ? path : "";
    return DALI_HIP_OK;
}

const char* dali_hip_rtc_options(void) {
    static const std::string joined = [] {
        std::string s;
        for (const char* o : kRtcOptions) s += std::string(o) + " ";
        return s;
    }();
    return joined.c_str();
}

int dali_hip_compile_only(const char* hip_source, size_t* code_size) {
    std::vector<char> code;
    std::string log;
    if (rtc_compile("gfx950", hip_source, &code, &log)) return DALI_HIP_ERROR;
    if (code_size) *code_size = code.size();
    return DALI_HIP_OK;
}

int dali_hip_jit_stats(uint64_t* compiled, uint64_t* disk_hits, uint64_t* launches) {
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (compiled) *compiled = r.n_compiled;
    if (disk_hits) *disk_hits = r.n_disk;
    if (launches) *launches = r.n_launch;
    return DALI_HIP_OK;
}

int dali_hip_cache_warm(int* loaded) {
    if (ensure_init()) return DALI_HIP_ERROR;
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (r.cache_dir.empty()) r.cache_dir = default_cache_dir();
    const std::string suffix = "-" + r.arch + ".hsaco";
    int n = 0;
    DIR* d = opendir(r.cache_dir.c_str());
    if (d) {
        while (struct dirent* ent = readdir(d)) {
            const std::string name = ent->d_name;
            if (name.size() != 16 + suffix.size() || name.compare(16, suffix.size(), suffix) != 0) continue;
            char* end = nullptr;
            const uint64_t hash = strtoull(name.substr(0, 16).c_str(), &end, 16);
            if (!end || *end != 0 || r.modules.count(hash) || r.preloaded.count(hash)) continue;
            std::ifstream in(r.cache_dir + "/" + name, std::ios::binary);
            std::vector<char> code((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
            hipModule_t mod = nullptr;
            if (code.empty() || hipModuleLoadData(&mod, code.data()) != hipSuccess) {
                (void)hipGetLastError();  // a stale or foreign file is rebuilt from source at its first use
                continue;
            }
            r.preloaded[hash] = mod;
            ++n;
        }
        closedir(d);
    }
    if (loaded) *loaded = n;
    return DALI_HIP_OK;
}

int dali_hip_module_is_loaded(uint64_t hash) {
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    return r.modules.count(hash) ? 1 : 0;
}

int dali_hip_module_load(uint64_t hash, const char* hip_source, const char* kernel_name,
                         const dali_hip_launch_plan* plan, int* was_cached) {
    if (ensure_init()) return DALI_HIP_ERROR;
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    bool force = env_true("DALI_JIT_ALWAYS_RECOMPILE") && !r.recompiled_once[hash];
    if (!force && r.modules.count(hash)) {
        if (was_cached) *was_cached = 2;
        return DALI_HIP_OK;
    }
    if (!plan || !kernel_name) return fail("dali_hip_module_load: plan and kernel_name are required");
    if (plan->n_arrays < 1 || plan->n_arrays > 64 || plan->n_scalars < 0 || plan->n_scalars > 64 ||
        plan->n_shapes < 0 || plan->n_shapes > 64)
        return fail("dali_hip_module_load: bad plan counts (%d arrays, %d scalars, %d shapes)", plan->n_arrays,
                    plan->n_scalars, plan->n_shapes);
    if (plan->block_threads < 64 || plan->block_threads > 1024 || plan->block_threads % 64)
        return fail("dali_hip_module_load: block_threads %d must be a multiple of 64 in [64,1024]",
                    plan->block_threads);

    if (r.cache_dir.empty()) r.cache_dir = default_cache_dir();
    std::string path = r.cache_dir + "/" + hash_hex(hash) + "-" + r.arch + ".hsaco";
    std::vector<char> code;
    int cached = 0;
    if (!force && r.preloaded.count(hash)) {
        cached = 1;
    } else if (!force) {
        std::ifstream in(path, std::ios::binary);
        if (in) {
            code.assign(std::istreambuf_iterator<char>(in), std::istreambuf_iterator<char>());
            if (!code.empty()) cached = 1;
        }
    }
    if (!cached) {
        if (!hip_source) return fail("dali_hip_module_load: no cached code object for %s and no source given", hash_hex(hash).c_str());
        std::string log;
        if (rtc_compile(r.arch, hip_source, &code, &log)) return DALI_HIP_ERROR;
        mkdir_p(r.cache_dir);
        // write-then-rename so a concurrent process never maps half a file
        std::string tmp = path + ".tmp" + std::to_string((long)getpid());
        {
            std::ofstream out(tmp, std::ios::binary);
            out.write(code.data(), (std::streamsize)code.size());
        }
        if (rename(tmp.c_str(), path.c_str()) != 0) unlink(tmp.c_str());
        if (env_true("DALI_HIP_KEEP_SOURCE")) {
            std::ofstream src(r.cache_dir + "/" + hash_hex(hash) + ".hip");
            src << hip_source;
        }
        r.n_compiled++;
        r.recompiled_once[hash] = true;
    } else {
        r.n_disk++;
    }

    Runtime::Module m;
    hipError_t e = hipSuccess;
    auto pre = r.preloaded.find(hash);
    if (cached && pre != r.preloaded.end()) {
        m.module = pre->second;
        r.preloaded.erase(pre);
    } else {
        e = hipModuleLoadData(&m.module, code.data());
    }
    if (e != hipSuccess && cached && hip_source) {
        // stale or foreign file: rebuild from source
        (void)hipGetLastError();
        std::string log;
        if (rtc_compile(r.arch, hip_source, &code, &log)) return DALI_HIP_ERROR;
        std::ofstream out(path, std::ios::binary);
        out.write(code.data(), (std::streamsize)code.size());
        r.n_compiled++;
        cached = 0;
        e = hipModuleLoadData(&m.module, code.data());
    }
    if (e != hipSuccess) return fail("hipModuleLoadData failed: %s", hipGetErrorString(e));
    e = hipModuleGetFunction(&m.fn, m.module, kernel_name);
    if (e != hipSuccess && cached && hip_source) {
        // a cached object without this entry point (written by another build): drop it and rebuild from source
        (void)hipGetLastError();
        (void)hipModuleUnload(m.module);
        m.module = nullptr;
        std::string log;
        if (rtc_compile(r.arch, hip_source, &code, &log)) return DALI_HIP_ERROR;
        std::ofstream out(path, std::ios::binary);
        out.write(code.data(), (std::streamsize)code.size());
        r.n_compiled++;
        cached = 0;
        e = hipModuleLoadData(&m.module, code.data());
        if (e != hipSuccess) return fail("hipModuleLoadData failed: %s", hipGetErrorString(e));
        e = hipModuleGetFunction(&m.fn, m.module, kernel_name);
    }
    if (e != hipSuccess) {
        if (m.module) (void)hipModuleUnload(m.module);
        return fail("hipModuleGetFunction(%s) failed: %s", kernel_name, hipGetErrorString(e));
    }

    m.plan = *plan;
    m.array_ndim.assign(plan->array_ndim, plan->array_ndim + plan->n_arrays);
    m.array_strided.assign(plan->array_strided, plan->array_strided + plan->n_arrays);
    m.array_elsize.assign(plan->array_elsize, plan->array_elsize + plan->n_arrays);
    if (plan->n_scalars) m.scalar_dtype.assign(plan->scalar_dtype, plan->scalar_dtype + plan->n_scalars);
    if (plan->n_shapes) m.shape_ndim.assign(plan->shape_ndim, plan->shape_ndim + plan->n_shapes);
    int n_iv = 0;
    for (int i = 0; i < plan->n_arrays; ++i) {
        if (m.array_ndim[i] < 1 || m.array_ndim[i] > 8) return fail("dali_hip_module_load: array %d has ndim %d", i, m.array_ndim[i]);
        n_iv += m.array_ndim[i] * (m.array_strided[i] ? 2 : 1);
    }
    for (int k = 0; k < plan->n_shapes; ++k) n_iv += m.shape_ndim[k];
    m.n_iv = n_iv;
    int n_slots = plan->n_scalars > 0 ? plan->n_scalars : 1;
    m.karg_bytes = 8 + 8 * (size_t)plan->n_arrays + 8 * (size_t)n_slots + 4 * (size_t)(n_iv > 0 ? n_iv : 1);
    m.karg_bytes = (m.karg_bytes + 7) & ~(size_t)7;
    if (m.karg_bytes > 4000) return fail("dali_hip_module_load: kernel argument block of %zu bytes is too large", m.karg_bytes);
    auto old = r.modules.find(hash);
    if (old != r.modules.end()) {
        (void)hipStreamSynchronize(r.stream);
        (void)hipModuleUnload(old->second.module);
        r.modules.erase(old);
    }
    r.modules.emplace(hash, std::move(m));
    if (was_cached) *was_cached = cached;
    return DALI_HIP_OK;
}

int dali_hip_launch(uint64_t hash, void** array_data, const int* offsets, const int** sizes,
                    const int** strides, const void** scalar_arguments, const int** shapes) {
    Runtime& r = rt();
    if (!r.ready) return fail("dali_hip_launch: library not initialised");
    Runtime::Module* m;
    {
        std::lock_guard<std::mutex> lock(r.mu);
        auto it = r.modules.find(hash);
        if (it == r.modules.end()) return fail("dali_hip_launch: no module loaded for hash %s", hash_hex(hash).c_str());
        m = &it->second;
        r.n_launch++;
    }
    const dali_hip_launch_plan& P = m->plan;
    alignas(8) char buf[4096];
    char* w = buf;
    void* ws = r.ws;
    memcpy(w, &ws, 8);
    w += 8;
    for (int i = 0; i < P.n_arrays; ++i) {
        if (!array_data[i]) return fail("dali_hip_launch: array_data[%d] is NULL", i);
        char* p = (char*)array_data[i] + (int64_t)offsets[i] * (int64_t)m->array_elsize[i];
        memcpy(w, &p, 8);
        w += 8;
    }
    int n_slots = P.n_scalars > 0 ? P.n_scalars : 1;
    for (int j = 0; j < n_slots; ++j) {
        uint64_t slot = 0;
        if (j < P.n_scalars) {
            if (!scalar_arguments || !scalar_arguments[j]) return fail("dali_hip_launch: scalar_arguments[%d] is NULL", j);
            int bytes = m->scalar_dtype[j] == DALI_HIP_DOUBLE ? 8 : 4;
            memcpy(&slot, scalar_arguments[j], bytes);
        }
        memcpy(w, &slot, 8);
        w += 8;
    }
    int32_t* iv = (int32_t*)w;
    int n = 0;
    for (int i = 0; i < P.n_arrays; ++i) {
        int nd = m->array_ndim[i];
        for (int d = 0; d < nd; ++d) {
            int v = sizes[i][d];
            if (v < 0) return fail("dali_hip_launch: sizes[%d][%d] = %d is negative", i, d, v);
            iv[n++] = v;
        }
        if (m->array_strided[i]) {
            if (!strides || !strides[i]) return fail("dali_hip_launch: strides[%d] missing for a strided array", i);
            for (int d = 0; d < nd; ++d) iv[n++] = strides[i][d];
        }
    }
    for (int k = 0; k < P.n_shapes; ++k)
        for (int d = 0; d < m->shape_ndim[k]; ++d) iv[n++] = shapes[k][d];

    auto extent = [&](int begin, int count) -> int64_t {
        int64_t e = 1;
        for (int t = 0; t < count; ++t) e *= (int64_t)iv[begin + t];
        return e;
    };
    if (P.work_begin < 0 || P.work_begin + P.work_count > m->n_iv) return fail("dali_hip_launch: plan extent out of range");
    int64_t work = extent(P.work_begin, P.work_count);
    if (work <= 0) return DALI_HIP_OK;  // empty arrays: nothing to do
    int64_t per = P.work_per_block > 0 ? P.work_per_block : 1;
    int64_t gx = (work + per - 1) / per;
    if (P.grid_kind != DALI_HIP_GRID_COLS && P.max_blocks > 0 && gx > P.max_blocks) gx = P.max_blocks;
    int64_t gy = 1;
    if (P.grid_kind == DALI_HIP_GRID_COLS) {
        if (P.work2_begin < 0 || P.work2_begin >= m->n_iv) return fail("dali_hip_launch: plan reduced extent out of range");
        int64_t red = iv[P.work2_begin];
        if (red <= 0) return DALI_HIP_OK;
        int64_t per2 = P.work2_per_block > 0 ? P.work2_per_block : 1;
        gy = (red + per2 - 1) / per2;
        if (P.max_blocks2 > 0 && gy > P.max_blocks2) gy = P.max_blocks2;
        // every column strip needs its block, so the bound on the whole grid is met by the y split alone
        if (P.max_blocks > 0 && gx * gy > P.max_blocks) gy = P.max_blocks / gx > 0 ? P.max_blocks / gx : 1;
        // rows of partials are padded to whole column strips
        int64_t cap = (int64_t)kWorkspacePartialBytes / (gx * per * (int64_t)(P.ws_elsize > 0 ? P.ws_elsize : 4));
        if (cap < 1) cap = 1;
        if (gy > cap) gy = cap;
        // more strips than tickets: no split of the reduced rows (the kernel then finishes each strip by itself and
        // touches neither tickets nor partial results)
        if (gx > (int64_t)kWorkspaceCounters) gy = 1;
    } else if (P.grid_kind == DALI_HIP_GRID_ALL) {
        int64_t cap = (int64_t)kWorkspacePartialBytes / (int64_t)(P.ws_elsize > 0 ? P.ws_elsize : 4);
        if (gx > cap) gx = cap;
    }
    if (gx > 2147483647LL || gy > 65535) return fail("dali_hip_launch: grid %lld x %lld too large", (long long)gx, (long long)gy);
    size_t karg = m->karg_bytes;
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, buf, HIP_LAUNCH_PARAM_BUFFER_SIZE, &karg, HIP_LAUNCH_PARAM_END};
    hipError_t e = hipModuleLaunchKernel(m->fn, (unsigned)gx, (unsigned)gy, 1, (unsigned)P.block_threads, 1, 1, 0,
                                         r.stream, nullptr, extra);
    if (e != hipSuccess) return fail("hipModuleLaunchKernel failed: %s", hipGetErrorString(e));
    return DALI_HIP_OK;
}

int dali_hip_capture_begin(void) {
    if (ensure_init()) return DALI_HIP_ERROR;
    HIP_TRY(hipStreamBeginCapture(rt().stream, hipStreamCaptureModeThreadLocal));
    return DALI_HIP_OK;
}

int dali_hip_capture_end(void** graph_exec) {
    hipGraph_t graph = nullptr;
    HIP_TRY(hipStreamEndCapture(rt().stream, &graph));
    if (!graph) return fail("dali_hip_capture_end: nothing was captured");
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return fail("hipGraphInstantiate failed: %s", hipGetErrorString(e));
    *graph_exec = (void*)exec;
    return DALI_HIP_OK;
}

int dali_hip_graph_launch(void* graph_exec) {
    HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph_exec, rt().stream));
    return DALI_HIP_OK;
}

int dali_hip_graph_destroy(void* graph_exec) {
    if (!graph_exec) return DALI_HIP_OK;
    HIP_TRY(hipStreamSynchronize(rt().stream));
    HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return DALI_HIP_OK;
}

int dali_hip_event_create(void** event) {
    if (ensure_init()) return DALI_HIP_ERROR;
    hipEvent_t ev;
    HIP_TRY(hipEventCreate(&ev));
    *event = (void*)ev;
    return DALI_HIP_OK;
}

int dali_hip_event_record(void* event) {
    HIP_TRY(hipEventRecord((hipEvent_t)event, rt().stream));
    return DALI_HIP_OK;
}

int dali_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
    HIP_TRY(hipEventSynchronize((hipEvent_t)stop));
    HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return DALI_HIP_OK;
}

int dali_hip_event_destroy(void* event) {
    HIP_TRY(hipEventDestroy((hipEvent_t)event));
    return DALI_HIP_OK;
}

}  // extern "C"
