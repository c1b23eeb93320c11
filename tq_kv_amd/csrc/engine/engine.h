// The engine: a model, its cache, and the one step function everything above uses.
//
// The reference's step is forward(tokens, index_pos) for one sequence with the last row's logits
// (src/models/turbo_generic.rs:1950-1987) and its per-request state is one position counter
// (src/engine.rs:117, :322-324).  Here a step takes a batch of sequences with unequal numbers of
// new tokens (whole prompts, or one token each, or anything between), runs exactly those tokens
// against what the cache holds, and returns the logits at the wanted places.
#pragma once
#include <list>

#include "model.h"

typedef struct hipGraphExec* hipGraphExec_t;

namespace tq {

class Engine {
public:
    // max_tokens: positions live sequences may hold together, each sequence counted up to whole
    // pages.  max_slots: most live sequences.
    Engine(std::shared_ptr<Model> model, long long max_tokens, int max_slots, bool use_graphs);
    ~Engine();
    Engine(const Engine&) = delete;
    Engine& operator=(const Engine&) = delete;

    std::shared_ptr<Model> model;
    std::unique_ptr<CacheStore> cache;
    long long max_tokens;
    bool use_graphs;

    int open(hipStream_t stream) { return cache->acquire(stream); }
    void close(int slot) { cache->release(slot); }

    // One step.  Sequence i lives in slots[i] and brings n_new[i] tokens (tokens: all of them, one
    // sequence after the other, on the host; device_tokens: for a step of one token per sequence
    // whose tokens were chosen on the device, int32 [n_seqs] there, and `tokens` may be null);
    // want_counts[i] of its places are wanted, want_idx lists them.  The logits [wanted, vocab]
    // go to logits_out (device memory) if given; otherwise they stay in memory of the engine's that
    // the next step writes again.  Returns where they are.
    const float* step(int n_seqs, const int32_t* slots, const int32_t* n_new, const int32_t* tokens, const int32_t* want_counts,
                      const int32_t* want_idx, const int32_t* device_tokens, float* logits_out, hipStream_t stream);
    int n_graphs() const { return (int)graphs_.size(); }
    int last_n_want() const { return last_n_want_; }

    static const int GRAPH_WIDTH_STEP = 8;      // page-table widths of graphed steps grow in steps of 8 pages
    static const int MAX_GRAPHS = 32;

private:
    struct Graph {
        StepShape shape;
        hipGraphExec_t exec = nullptr;
        Buffer flat;                    // the step's arrays, overwritten before every replay
        Workspace ws{true};             // what the captured kernels point into
        StepContext ctx;
        Tensor logits;
    };
    const float* graphed_step(StepContext& probe, int n_seqs, const int32_t* slots, const int32_t* starts, const int32_t* n_new,
                              const int32_t* tokens, const int32_t* want_counts, const int32_t* want_idx, const int32_t* device_tokens,
                              float* logits_out, hipStream_t stream);
    void release_graph(Graph& g);
    Workspace ws_;
    Staging staging_;
    std::list<Graph> graphs_;            // least recently used first
    hipStream_t capture_stream_ = nullptr;
    int last_n_want_ = 0;
};

// The first launch of a captured graph in a process leaves the device slower for about a quarter of
// a second (measured at the Qwen2.5-7B sizes: every kernel of a decoding step then takes 5 to 10 %
// longer, whichever graph is launched).  A graph of one small kernel, launched once when the first
// engine is made, moves that quarter of a second to where no request waits for it.
void prime_graph_launches();

}  // namespace tq
