// What every file of the engine shares: errors that carry a status code of the C boundary,
// a view of a tensor in device (or host) memory, memory that is owned, the workspace of a
// step, pinned staging for small uploads, and the table of kernel entry points.
#pragma once
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../tq_engine.h"

typedef struct ihipStream_t* hipStream_t;
typedef struct ihipEvent_t* hipEvent_t;

namespace tq {

// ---- errors --------------------------------------------------------------------------------
struct Error : std::runtime_error {
    int code;
    std::string detail;          // optional JSON with the findings (weight errors)
    Error(int code_, const std::string& msg, std::string detail_ = "") : std::runtime_error(msg), code(code_), detail(std::move(detail_)) {}
};

std::string format(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
[[noreturn]] void raise(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// ---- tensors -------------------------------------------------------------------------------
enum DType { F32 = 0, BF16 = 1, I32 = 2 };
inline size_t dtype_size(int dt) { return dt == BF16 ? 2 : 4; }
const char* dtype_name(int dt);

// A view: the memory belongs to someone else (a Buffer, the workspace, the caller).
struct Tensor {
    void* data = nullptr;
    int dtype = F32;
    int ndim = 0;
    int64_t shape[6] = {0, 0, 0, 0, 0, 0};

    Tensor() {}
    Tensor(void* d, int dt, std::initializer_list<int64_t> dims) : data(d), dtype(dt) {
        for (int64_t v : dims) shape[ndim++] = v;
    }
    bool defined() const { return ndim > 0; }
    int64_t numel() const {
        int64_t n = 1;
        for (int i = 0; i < ndim; ++i) n *= shape[i];
        return ndim ? n : 0;
    }
    size_t bytes() const { return (size_t)numel() * dtype_size(dtype); }
    int64_t rows() const { return shape[0]; }
    int64_t cols() const { return ndim > 1 ? numel() / (shape[0] ? shape[0] : 1) : 1; }
    size_t row_bytes() const { return (size_t)cols() * dtype_size(dtype); }
    // rows a .. b of the first dimension
    Tensor slice(int64_t a, int64_t b) const {
        Tensor t = *this;
        t.data = (char*)data + (size_t)a * row_bytes();
        t.shape[0] = b - a;
        return t;
    }
    std::string describe() const;
};

// ---- device memory ---------------------------------------------------------------------------
// Where memory lives and how kernels are reached.  "hip": the GPU.  "null": host memory and
// kernel calls that do nothing, for running the engine's host logic without a GPU (under
// sanitizers); nothing it computes means anything.
bool null_device();
void set_null_device(bool on);                  // for the calling thread
struct DeviceScope {                            // the device of an object, for the length of a call into it
    bool before;
    explicit DeviceScope(bool on_gpu) : before(null_device()) { set_null_device(!on_gpu); }
    ~DeviceScope() { set_null_device(before); }
};

void* device_malloc(size_t bytes);
void device_free(void* p, bool null);
void copy_to_device(void* dst, const void* src, size_t bytes, hipStream_t stream);           // host (pageable or pinned) -> device
void copy_to_host(void* dst, const void* src, size_t bytes, hipStream_t stream);             // returns after the copy has landed
void copy_on_device(void* dst, const void* src, size_t bytes, hipStream_t stream);
void zero_device(void* dst, size_t bytes, hipStream_t stream);                               // not inside a captured graph
void stream_synchronize(hipStream_t stream);
void device_synchronize();
int compute_units();                  // of the current device (0 on the null device)
void hip_check(int status, const char* what);

class Buffer {
public:
    Buffer() {}
    explicit Buffer(size_t bytes) { allocate(bytes); }
    ~Buffer() { release(); }
    Buffer(const Buffer&) = delete;
    Buffer& operator=(const Buffer&) = delete;
    Buffer(Buffer&& o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_), null_(o.null_) { o.ptr_ = nullptr; o.bytes_ = 0; }
    Buffer& operator=(Buffer&& o) noexcept {
        if (this != &o) { release(); ptr_ = o.ptr_; bytes_ = o.bytes_; null_ = o.null_; o.ptr_ = nullptr; o.bytes_ = 0; }
        return *this;
    }
    void allocate(size_t bytes) { release(); bytes_ = bytes; null_ = null_device(); ptr_ = bytes ? device_malloc(bytes) : nullptr; }
    void release() { if (ptr_) device_free(ptr_, null_); ptr_ = nullptr; bytes_ = 0; }
    void* data() const { return ptr_; }
    size_t bytes() const { return bytes_; }
private:
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
    bool null_ = false;
};

// The scratch memory of one step: handed out front to back, all of it given back when the
// next step starts.  A growing workspace adds a chunk to an arena that runs out and, at the
// next reset, makes one chunk of what that arena needed (after the stream has drained); a fixed
// one (what a captured graph's kernels point into) refuses instead.
class Workspace {
public:
    // Three arenas, each a bump allocator: what lives for the whole step (STEP), and two that the
    // layers of a model use in turn, so that the temporaries of a layer go into the memory that the
    // layer before the last one has left: a step needs the memory of two layers, not of all, and
    // its kernels meet the same addresses layer after layer.
    enum { STEP = 0, N_ARENAS = 3 };
    explicit Workspace(bool fixed = false) : fixed_(fixed) {}
    void reserve(size_t bytes);                  // the current arena: one chunk of at least so many bytes (drops what it has)
    void reserve_like(const Workspace& measured, size_t more_for_the_step);     // every arena: what `measured` needed since its reset
    void reset(hipStream_t stream);              // a new step: every arena is empty, the current one is STEP
    void* alloc(size_t bytes) { return alloc_in(current_, bytes); }
    void* alloc_for_step(size_t bytes) { return alloc_in(STEP, bytes); }
    Tensor tensor(int dtype, std::initializer_list<int64_t> dims) {
        Tensor t(nullptr, dtype, dims);
        t.data = alloc(t.bytes());
        return t;
    }
    void use(int arena) { current_ = arena; }
    void rewind(int arena);                      // what the arena holds is no longer needed
    int arena_of(const void* p) const;           // the arena whose memory p points into, or -1
    size_t high_water() const;                   // the most that was held at once since the last reset
    size_t capacity() const;
private:
    struct Chunk { Buffer mem; size_t used = 0; };
    struct Arena { std::vector<Chunk> chunks; size_t at = 0, held = 0, high = 0; };
    void* alloc_in(int arena, size_t bytes);
    Arena arenas_[N_ARENAS];
    int current_ = STEP;
    bool fixed_;
};

// Pinned host buffers for small uploads, used in turn; a buffer is written again only after
// the copy that last read it has finished.
class Staging {
public:
    explicit Staging(int depth = 4);
    ~Staging();
    Staging(const Staging&) = delete;
    Staging& operator=(const Staging&) = delete;
    // copies n_bytes from host memory to dst on the device without waiting for the device
    void upload(void* dst, const void* src, size_t n_bytes, hipStream_t stream);
private:
    struct Slot { void* host = nullptr; size_t cap = 0; hipEvent_t event = nullptr; bool busy = false; };
    std::vector<Slot> slots_;
    int turn_ = 0;
};

// ---- kernels ---------------------------------------------------------------------------------
// The kernel library is a shared object of its own (built by hipcc); it is opened at the first
// use and its entry points are looked up by name.
void set_kernel_library(const std::string& path);
void set_kernel_builder(const char* (*builder)(void));       // asked for the library's path when none is found
std::string kernel_library_path();
void* kernel_symbol(const char* name);             // raises if the library or the symbol is missing
[[noreturn]] void raise_kernel_error(const char* what);

template <typename Fn> struct KernelFn;
template <typename R, typename... A> struct KernelFn<R(A...)> {
    const char* name;
    R (*fn)(A...) = nullptr;
    explicit KernelFn(const char* n) : name(n) {}
    R raw(A... a) {
        if (!fn) fn = (R (*)(A...))kernel_symbol(name);
        return fn(a...);
    }
};
// An entry point that returns a status: 0 or an error with the library's message.  With the
// null device nothing is called.
template <typename... A> struct Kernel {
    KernelFn<int(A...)> k;
    explicit Kernel(const char* n) : k(n) {}
    void operator()(A... a) {
        if (null_device()) return;
        if (k.raw(a...) != 0) raise_kernel_error(k.name);
    }
};

}  // namespace tq
