#include "core.h"

#include <dlfcn.h>
#include <glob.h>
#include <hip/hip_runtime_api.h>
#include <stdlib.h>

#include <algorithm>
#include <mutex>

namespace tq {

std::string format(const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    return buf;
}

void raise(int code, const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    throw Error(code, buf);
}

const char* dtype_name(int dt) { return dt == F32 ? "float32" : dt == BF16 ? "bfloat16" : dt == I32 ? "int32" : "?"; }

std::string Tensor::describe() const {
    std::string s = dtype_name(dtype);
    s += " [";
    for (int i = 0; i < ndim; ++i) s += format(i ? ", %lld" : "%lld", (long long)shape[i]);
    return s + "]";
}

// ---- device ----------------------------------------------------------------------------------
static thread_local bool g_null_device = false;
bool null_device() { return g_null_device; }
void set_null_device(bool on) { g_null_device = on; }

void hip_check(int status, const char* what) {
    if (status != hipSuccess) raise(TQE_ERR_DEVICE, "%s: %s", what, hipGetErrorString((hipError_t)status));
}

void* device_malloc(size_t bytes) {
    void* p = nullptr;
    if (g_null_device) {
        p = calloc(1, bytes ? bytes : 1);
        if (!p) raise(TQE_ERR_DEVICE, "out of host memory (%zu bytes)", bytes);
        return p;
    }
    const hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) raise(TQE_ERR_DEVICE, "cannot allocate %zu bytes of device memory: %s", bytes, hipGetErrorString(e));
    return p;
}

void device_free(void* p, bool null) {
    if (!p) return;
    if (null) { free(p); return; }
    (void)hipFree(p);
}

void copy_to_device(void* dst, const void* src, size_t bytes, hipStream_t stream) {
    if (!bytes) return;
    if (g_null_device) { memcpy(dst, src, bytes); return; }
    hip_check(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream), "copy to the device");
}

void copy_to_host(void* dst, const void* src, size_t bytes, hipStream_t stream) {
    if (g_null_device) { if (bytes) memcpy(dst, src, bytes); return; }
    if (bytes) hip_check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, stream), "copy to the host");
    hip_check(hipStreamSynchronize(stream), "waiting for the device");
}

void copy_on_device(void* dst, const void* src, size_t bytes, hipStream_t stream) {
    if (!bytes) return;
    if (g_null_device) { memmove(dst, src, bytes); return; }
    hip_check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, stream), "copy on the device");
}

void zero_device(void* dst, size_t bytes, hipStream_t stream) {
    if (!bytes) return;
    if (g_null_device) { memset(dst, 0, bytes); return; }
    hip_check(hipMemsetAsync(dst, 0, bytes, stream), "clearing device memory");
}

void stream_synchronize(hipStream_t stream) {
    if (g_null_device) return;
    hip_check(hipStreamSynchronize(stream), "waiting for the device");
}

int compute_units() {
    if (g_null_device) return 0;
    static int n = -1;
    if (n < 0) {
        int dev = 0, v = 0;
        n = (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess) ? v : 0;
    }
    return n;
}

void device_synchronize() {
    if (g_null_device) return;
    hip_check(hipDeviceSynchronize(), "waiting for the device");
}

// ---- workspace -------------------------------------------------------------------------------
static size_t round_up(size_t n, size_t to) { return (n + to - 1) / to * to; }

void Workspace::reserve(size_t bytes) {
    Arena& a = arenas_[current_];
    a.chunks.clear();
    a.chunks.emplace_back();
    a.chunks.back().mem.allocate(round_up(std::max<size_t>(bytes, 256), 256));
    a.at = a.held = 0;
}

void Workspace::reserve_like(const Workspace& measured, size_t more_for_the_step) {
    for (int i = 0; i < N_ARENAS; ++i) {
        const size_t need = measured.arenas_[i].high + (i == STEP ? more_for_the_step : 0);
        Arena& a = arenas_[i];
        a.chunks.clear();
        a.at = a.held = 0;
        if (need == 0) continue;
        a.chunks.emplace_back();
        a.chunks.back().mem.allocate(round_up(need, 256));
    }
}

size_t Workspace::capacity() const {
    size_t n = 0;
    for (const Arena& a : arenas_)
        for (const Chunk& c : a.chunks) n += c.mem.bytes();
    return n;
}

size_t Workspace::high_water() const {
    size_t n = 0;
    for (const Arena& a : arenas_) n += a.high;
    return n;
}

void Workspace::reset(hipStream_t stream) {
    bool waited = false;
    for (Arena& a : arenas_) {
        if (a.chunks.size() > 1 && !fixed_) {
            // what the arena needed at most, in one piece: first let the last step finish
            if (!waited) stream_synchronize(stream);
            waited = true;
            const size_t want = a.high + a.high / 8;
            a.chunks.clear();
            a.chunks.emplace_back();
            a.chunks.back().mem.allocate(round_up(std::max<size_t>(want, 256), 256));
        }
        for (Chunk& c : a.chunks) c.used = 0;
        a.at = a.held = a.high = 0;
    }
    current_ = STEP;
}

void Workspace::rewind(int arena) {
    Arena& a = arenas_[arena];
    for (Chunk& c : a.chunks) c.used = 0;
    a.at = a.held = 0;
}

int Workspace::arena_of(const void* p) const {
    for (int i = 0; i < N_ARENAS; ++i)
        for (const Chunk& c : arenas_[i].chunks)
            if (p >= c.mem.data() && p < (const char*)c.mem.data() + c.mem.bytes()) return i;
    return -1;
}

void* Workspace::alloc_in(int arena, size_t bytes) {
    Arena& a = arenas_[arena];
    bytes = round_up(std::max<size_t>(bytes, 1), 256);
    while (a.at < a.chunks.size() && a.chunks[a.at].used + bytes > a.chunks[a.at].mem.bytes()) ++a.at;
    if (a.at >= a.chunks.size()) {
        if (fixed_)
            raise(TQE_ERR_DEVICE, "a captured step's workspace of %zu bytes is too small (%zu more asked for)", capacity(), bytes);
        size_t have = 0;
        for (const Chunk& c : a.chunks) have += c.mem.bytes();
        a.chunks.emplace_back();
        a.chunks.back().mem.allocate(std::max(bytes, std::max<size_t>(have / 2, (size_t)4 << 20)));
        a.at = a.chunks.size() - 1;
    }
    Chunk& c = a.chunks[a.at];
    void* p = (char*)c.mem.data() + c.used;
    c.used += bytes;
    a.held += bytes;
    a.high = std::max(a.high, a.held);
    return p;
}

// ---- staging ---------------------------------------------------------------------------------
Staging::Staging(int depth) : slots_((size_t)depth) {}

Staging::~Staging() {
    for (Slot& s : slots_) {
        if (s.event) { (void)hipEventSynchronize(s.event); (void)hipEventDestroy(s.event); }
        if (s.host) (void)hipHostFree(s.host);
    }
}

void Staging::upload(void* dst, const void* src, size_t n_bytes, hipStream_t stream) {
    if (!n_bytes) return;
    if (g_null_device) { memcpy(dst, src, n_bytes); return; }
    Slot& s = slots_[(size_t)turn_];
    turn_ = (turn_ + 1) % (int)slots_.size();
    if (s.busy) { hip_check(hipEventSynchronize(s.event), "waiting for an upload"); s.busy = false; }
    if (s.cap < n_bytes) {
        if (s.host) hip_check(hipHostFree(s.host), "freeing pinned memory");
        s.cap = std::max<size_t>(16384, 2 * n_bytes);
        s.host = nullptr;
        hip_check(hipHostMalloc(&s.host, s.cap, hipHostMallocDefault), "allocating pinned memory");
    }
    if (!s.event) hip_check(hipEventCreateWithFlags(&s.event, hipEventDisableTiming), "creating an event");
    memcpy(s.host, src, n_bytes);
    hip_check(hipMemcpyAsync(dst, s.host, n_bytes, hipMemcpyHostToDevice, stream), "uploading a step's arrays");
    hip_check(hipEventRecord(s.event, stream), "recording an event");
    s.busy = true;
}

// ---- the kernel library ------------------------------------------------------------------------
static std::mutex g_kernel_mutex;
static std::string g_kernel_path;
static void* g_kernel_handle = nullptr;

static const char* (*g_kernel_builder)(void) = nullptr;

void set_kernel_builder(const char* (*builder)(void)) {
    std::lock_guard<std::mutex> lock(g_kernel_mutex);
    g_kernel_builder = builder;
}

void set_kernel_library(const std::string& path) {
    std::lock_guard<std::mutex> lock(g_kernel_mutex);
    if (g_kernel_handle && path != g_kernel_path) { dlclose(g_kernel_handle); g_kernel_handle = nullptr; }
    g_kernel_path = path;
}

static std::string find_kernel_library() {
    if (const char* env = getenv("TQ_KERNEL_LIBRARY")) return env;
    // beside this library: csrc/libtqkernels_<hash of its sources>.so
    Dl_info info;
    if (dladdr((void*)&find_kernel_library, &info) && info.dli_fname) {
        std::string dir = info.dli_fname;
        const size_t slash = dir.rfind('/');
        dir = slash == std::string::npos ? "." : dir.substr(0, slash);
        glob_t g;
        std::string found;
        if (glob((dir + "/libtqkernels_*.so").c_str(), 0, nullptr, &g) == 0) {
            if (g.gl_pathc > 0) found = g.gl_pathv[g.gl_pathc - 1];
            globfree(&g);
        }
        if (!found.empty()) return found;
    }
    return "";
}

std::string kernel_library_path() {
    std::lock_guard<std::mutex> lock(g_kernel_mutex);
    if (g_kernel_path.empty()) g_kernel_path = find_kernel_library();
    return g_kernel_path;
}

void* kernel_symbol(const char* name) {
    std::lock_guard<std::mutex> lock(g_kernel_mutex);
    if (!g_kernel_handle) {
        if (g_kernel_path.empty()) g_kernel_path = find_kernel_library();
        if (g_kernel_path.empty() && g_kernel_builder) {
            // the program that loaded this library knows how to build the kernels (the Python package compiles them)
            const char* built = g_kernel_builder();
            if (built && *built) g_kernel_path = built;
        }
        if (g_kernel_path.empty())
            throw Error(TQE_ERR_DEVICE, "the HIP kernel library is not built: no libtqkernels_*.so beside the engine library "
                                        "(build it with tq_kv_amd/csrc/build.py, or name it in TQ_KERNEL_LIBRARY)");
        g_kernel_handle = dlopen(g_kernel_path.c_str(), RTLD_NOW | RTLD_LOCAL);
        if (!g_kernel_handle) throw Error(TQE_ERR_DEVICE, format("cannot load the HIP kernel library %s: %s", g_kernel_path.c_str(), dlerror()));
        // the two libraries index the same cache pages and share one list of entry points: both must say so
        typedef int (*Query)(void);
        Query page = (Query)dlsym(g_kernel_handle, "tqk_page_size"), abi = (Query)dlsym(g_kernel_handle, "tqk_abi_version");
        const int page_size = page ? page() : -1, abi_version = abi ? abi() : -1;
        if (page_size != TQE_PAGE || abi_version != TQE_KERNEL_ABI) {
            dlclose(g_kernel_handle);
            g_kernel_handle = nullptr;
            throw Error(TQE_ERR_DEVICE, format("the kernel library %s does not fit this engine library: its cache pages hold %d positions (here %d), "
                                               "its interface is version %d (here %d); build both from the same sources",
                                               g_kernel_path.c_str(), page_size, TQE_PAGE, abi_version, TQE_KERNEL_ABI));
        }
    }
    void* sym = dlsym(g_kernel_handle, name);
    if (!sym) throw Error(TQE_ERR_DEVICE, format("the kernel library %s has no entry point %s (built from other sources?)", g_kernel_path.c_str(), name));
    return sym;
}

void raise_kernel_error(const char* what) {
    static KernelFn<const char*()> last("tqk_last_error");
    const char* msg = last.raw();
    const char* short_name = strncmp(what, "tqk_", 4) ? what : what + 4;
    throw Error(TQE_ERR_KERNEL, format("%s: %s", short_name, msg ? msg : "failed"));
}

}  // namespace tq
