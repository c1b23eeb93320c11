// Named ranges around the parts of a step, after the reference's tracing spans ("model", "attn",
// "attn-mlp", "rms-norm", "output": src/models/turbo_generic.rs:36, :1920-1922, :1932-1933,
// entered around the work at :43, :1957-1985).  The reference installs no subscriber, so its
// spans never show; these show in a profiler's marker trace once switched on and cost one test
// of a flag otherwise.  The ranges go to ROCm's ROCTx library (roctxRangePushA / roctxRangePop),
// or to whatever pair of functions the caller installs (a test's recorder).
#pragma once

namespace tq {

typedef int (*TracePush)(const char* name);
typedef int (*TracePop)(void);

bool trace_enable(bool on);                     // returns whether ranges are on now (off if no library is found)
bool trace_enabled();
void trace_set_sink(TracePush push, TracePop pop);      // nullptrs: back to ROCTx

class Span {
public:
    explicit Span(const char* name);
    ~Span();
    Span(const Span&) = delete;
    Span& operator=(const Span&) = delete;
private:
    TracePop pop_;
};

}  // namespace tq
