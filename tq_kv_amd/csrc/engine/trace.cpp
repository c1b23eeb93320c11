#include "trace.h"

#include <dlfcn.h>
#include <stdio.h>
#include <stdlib.h>

namespace tq {
namespace {
bool g_on = false, g_tried = false;
TracePush g_push = nullptr, g_user_push = nullptr;
TracePop g_pop = nullptr, g_user_pop = nullptr;

bool load() {
    if (g_user_push && g_user_pop) return true;
    if (g_tried) return g_push != nullptr;
    g_tried = true;
    const char* names[] = {"librocprofiler-sdk-roctx.so", "/opt/rocm/lib/librocprofiler-sdk-roctx.so", "libroctx64.so"};
    for (const char* name : names) {
        void* lib = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
        if (!lib) continue;
        g_push = (TracePush)dlsym(lib, "roctxRangePushA");
        g_pop = (TracePop)dlsym(lib, "roctxRangePop");
        if (g_push && g_pop) return true;
        g_push = nullptr;
        g_pop = nullptr;
    }
    fprintf(stderr, "[tq_kv_amd tracing] no ROCTx library found: ranges stay off\n");
    return false;
}

struct EnvInit {
    EnvInit() {
        const char* e = getenv("TQ_TRACE");
        if (e && *e && !(e[0] == '0' && !e[1])) trace_enable(true);
    }
} g_env_init;
}  // namespace

bool trace_enable(bool on) {
    g_on = on && load();
    return g_on;
}

bool trace_enabled() { return g_on; }

void trace_set_sink(TracePush push, TracePop pop) {
    g_user_push = push;
    g_user_pop = pop;
    if (!push || !pop) g_on = g_on && g_push != nullptr;
}

Span::Span(const char* name) : pop_(nullptr) {
    if (!g_on) return;
    const bool user = g_user_push && g_user_pop;
    (user ? g_user_push : g_push)(name);
    pop_ = user ? g_user_pop : g_pop;
}

Span::~Span() {
    if (pop_) pop_();
}

}  // namespace tq
