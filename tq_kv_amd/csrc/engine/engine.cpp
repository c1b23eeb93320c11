#include "engine.h"

#include <hip/hip_runtime_api.h>

#include "kernels.h"
#include "trace.h"

namespace tq {

void prime_graph_launches() {
    static bool primed = false;
    if (primed || null_device()) return;
    primed = true;
    hipStream_t s = nullptr;
    hip_check(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "creating a stream");
    Buffer buf(64 * sizeof(float));
    zero_device(buf.data(), buf.bytes(), s);
    K::finish_logits((float*)buf.data(), 1, 64, nullptr, 1.0f, 0.0f, s);
    stream_synchronize(s);
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hip_check(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal), "beginning a capture");
    K::finish_logits((float*)buf.data(), 1, 64, nullptr, 1.0f, 0.0f, s);
    hip_check(hipStreamEndCapture(s, &graph), "ending a capture");
    hip_check(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "instantiating a graph");
    // launched where steps will be launched by a caller that names no stream: the default stream
    hip_check(hipGraphLaunch(exec, nullptr), "launching a graph");
    stream_synchronize(nullptr);
    (void)hipGraphExecDestroy(exec);
    (void)hipGraphDestroy(graph);
    (void)hipStreamDestroy(s);
}

Engine::Engine(std::shared_ptr<Model> m, long long max_tokens_, int max_slots, bool use_graphs_)
    : model(std::move(m)), max_tokens(max_tokens_), staging_(4) {
    if (!model->loaded) raise(TQE_ERR_STATE, "the model has no weights yet");
    cache.reset(new CacheStore(model->needs, model->cache_of, max_tokens, max_slots, model->dtype));
    // Steps of one token per sequence are captured as HIP graphs and replayed: the step is some
    // hundred short kernels, and launching them one by one from the host would cost more than
    // running them.  Only if every part says its forward can be captured.
    use_graphs = use_graphs_ && model->on_gpu && model->graph_safe;
    if (use_graphs) {
        prime_graph_launches();
        hip_check(hipStreamCreateWithFlags(&capture_stream_, hipStreamNonBlocking), "creating a stream");
    }
}

void Engine::release_graph(Graph& g) {
    if (g.exec) (void)hipGraphExecDestroy(g.exec);
    g.exec = nullptr;
}

Engine::~Engine() {
    if (model->on_gpu) (void)hipDeviceSynchronize();
    for (Graph& g : graphs_) release_graph(g);
    if (capture_stream_) (void)hipStreamDestroy(capture_stream_);
}

const float* Engine::step(int n_seqs, const int32_t* slots, const int32_t* n_new, const int32_t* tokens, const int32_t* want_counts,
                          const int32_t* want_idx, const int32_t* device_tokens, float* logits_out, hipStream_t stream) {
    if (n_seqs < 1 || !slots || !n_new || !want_counts) raise(TQE_ERR_STEP, "a step needs at least one sequence");
    if (device_tokens)
        for (int i = 0; i < n_seqs; ++i)
            if (n_new[i] != 1) raise(TQE_ERR_STEP, "tokens on the device stand for one token per sequence");
    if (!device_tokens && !tokens) raise(TQE_ERR_ARGUMENT, "a step needs its tokens, on the host or on the device");
    // the bookkeeping checks the rest: slots held and named once, no empty prompt, tokens inside the
    // vocabulary (where the host knows them), no sequence beyond the model's positions
    int status = tqe_check_step(cache->book, n_seqs, slots, n_new, device_tokens ? nullptr : tokens, (int)model->spec.vocab_size,
                                (int)std::min<int64_t>(model->spec.max_positions, INT32_MAX));
    if (status != TQE_OK) throw Error(status, tqe_last_error());
    for (int i = 0; i < n_seqs; ++i)
        if (want_counts[i] < 0) raise(TQE_ERR_ARGUMENT, "sequence %d of the step wants %d places", i, want_counts[i]);
    Span span("step");
    cache->reserve(n_seqs, slots, n_new);
    std::vector<int32_t> starts((size_t)n_seqs), placeholder;
    bool all_one = true;
    for (int i = 0; i < n_seqs; ++i) {
        starts[(size_t)i] = cache->length(slots[i]);
        all_one = all_one && n_new[i] == 1;
    }
    if (!tokens) { placeholder.assign((size_t)n_seqs, 0); tokens = placeholder.data(); }
    const float* logits = nullptr;
    try {
    StepContext ctx;
    ctx.stream = stream;
    ctx.staging = &staging_;
    ctx.act_dtype = model->dtype;
    if (use_graphs && all_one && n_seqs <= mid_max_rows()) {
        logits = graphed_step(ctx, n_seqs, slots, starts.data(), n_new, tokens, want_counts, want_idx, device_tokens, logits_out, stream);
    } else {
        ws_.reset(stream);
        ctx.ws = &ws_;
        ctx.plan(cache->book, n_seqs, slots, starts.data(), n_new, tokens, want_counts, want_idx, 1);
        ctx.upload();
        if (device_tokens) copy_on_device((void*)ctx.dev.tokens, device_tokens, (size_t)n_seqs * sizeof(int32_t), stream);
        logits = (const float*)model->forward(ctx, *cache, logits_out).data;
        last_n_want_ = ctx.n_want;
    }
    } catch (...) {
        // the reservation goes back: the sequences keep the lengths and the pages they had
        (void)tqe_cache_trim(cache->book, n_seqs, slots);
        throw;
    }
    cache->commit(n_seqs, slots, n_new);
    return logits;
}

// A step of one token per sequence through a captured graph.  The graph reads the step's arrays
// (tokens, positions, page tables) from one device buffer that is overwritten before every replay;
// its kernels take every size from those arrays or from the shapes the graph was captured for.
const float* Engine::graphed_step(StepContext& probe, int n_seqs, const int32_t* slots, const int32_t* starts, const int32_t* n_new,
                                  const int32_t* tokens, const int32_t* want_counts, const int32_t* want_idx, const int32_t* device_tokens,
                                  float* logits_out, hipStream_t stream) {
    probe.plan(cache->book, n_seqs, slots, starts, n_new, tokens, want_counts, want_idx, GRAPH_WIDTH_STEP);
    last_n_want_ = probe.n_want;
    const StepShape shape = probe.shape();
    auto it = graphs_.begin();
    for (; it != graphs_.end(); ++it)
        if (!(it->shape < shape) && !(shape < it->shape)) break;
    const size_t logits_bytes = (size_t)probe.n_want * (size_t)model->spec.vocab_size * sizeof(float);
    if (it == graphs_.end()) {
        // this step's work, eagerly, which also warms everything up; then the same step captured
        ws_.reset(stream);
        probe.ws = &ws_;
        probe.upload();
        if (device_tokens) copy_on_device((void*)probe.dev.tokens, device_tokens, (size_t)n_seqs * sizeof(int32_t), stream);
        const float* logits = (const float*)model->forward(probe, *cache, logits_out).data;
        device_synchronize();
        if ((int)graphs_.size() >= MAX_GRAPHS) {
            release_graph(graphs_.front());
            graphs_.pop_front();
        }
        graphs_.emplace_back();
        Graph& g = graphs_.back();
        try {
            g.shape = shape;
            g.flat.allocate(probe.flat_count * sizeof(int32_t));
            g.ws.reserve_like(ws_, logits_bytes + (size_t)(1 << 16));      // the eager run's logits may have gone to the caller's memory
            g.ctx.stream = capture_stream_;
            g.ctx.staging = &staging_;
            g.ctx.act_dtype = model->dtype;
            g.ctx.ws = &g.ws;
            g.ctx.plan(cache->book, n_seqs, slots, starts, n_new, tokens, want_counts, want_idx, GRAPH_WIDTH_STEP);
            // the arrays the graph reads: this step's, so that the captured run is a valid one
            g.ctx.stream = stream;             // the upload belongs to the caller's stream
            g.ctx.upload((int32_t*)g.flat.data());
            if (device_tokens) copy_on_device((void*)g.ctx.dev.tokens, device_tokens, (size_t)n_seqs * sizeof(int32_t), stream);
            stream_synchronize(stream);
            g.ctx.stream = capture_stream_;
            g.ctx.capturing = true;
            hipGraph_t graph = nullptr;
            hip_check(hipStreamBeginCapture(capture_stream_, hipStreamCaptureModeThreadLocal), "beginning a capture");
            try {
                g.logits = model->forward(g.ctx, *cache, nullptr);
            } catch (...) {
                (void)hipStreamEndCapture(capture_stream_, &graph);
                if (graph) (void)hipGraphDestroy(graph);
                throw;
            }
            hip_check(hipStreamEndCapture(capture_stream_, &graph), "ending a capture");
            const hipError_t e = hipGraphInstantiate(&g.exec, graph, nullptr, nullptr, 0);
            (void)hipGraphDestroy(graph);
            hip_check(e, "instantiating a graph");
        } catch (...) {
            graphs_.pop_back();
            throw;
        }
        return logits;
    }
    graphs_.splice(graphs_.end(), graphs_, it);          // most recently used last
    Graph& g = graphs_.back();
    staging_.upload(g.flat.data(), probe.packed.data(), probe.flat_count * sizeof(int32_t), stream);
    if (device_tokens) copy_on_device((void*)g.ctx.dev.tokens, device_tokens, (size_t)n_seqs * sizeof(int32_t), stream);
    hip_check(hipGraphLaunch(g.exec, stream), "launching a captured step");
    if (logits_out) {
        copy_on_device(logits_out, g.logits.data, logits_bytes, stream);
        return logits_out;
    }
    return (const float*)g.logits.data;
}

}  // namespace tq
