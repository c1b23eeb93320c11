// Sampling on the device and the generation loop above the step function.
//
// One request in the reference (src/engine.rs:364-438): the prompt whole, a first draw, then while
// fewer than max_tokens tokens have been emitted: stop if the drawn token is a stop token (it is
// not emitted), emit it, feed it, draw the next.  Here many requests run as batches that start
// together: their prompts in one step, then one token each per step; a request that ends leaves
// the batch and gives its slot back at once, the others go on unchanged; when a batch is done the
// next one starts, until every request has been served.
//
// The loop only decides; it computes nothing.  It is written against two small interfaces, an
// engine (open, close, step) and a sampler (sample; optionally draw / pick / read without
// waiting), so that it can be driven by stand-ins without a GPU.  The decisions themselves (which
// requests run together, how prompts are cut into steps, what becomes of a drawn token) are
// tqe_plan_batches, tqe_prompt_steps and tqe_batch_*.
#pragma once
#include <functional>

#include "engine.h"

namespace tq {

// Generation parameters with the reference's names and defaults (GenerationParams,
// src/engine.rs:29-49; the flags of `tq chat`, src/main.rs:56-69).
struct GenerationParams {
    int max_tokens = 512;
    float temperature = 0.7f;        // <= 0 is greedy (src/engine.rs:353-354)
    float top_p = 0.9f;
    int top_k = 40;                  // 0 switches it off
    float repeat_penalty = 1.1f;     // 1.0 switches it off (src/engine.rs:403)
    uint64_t seed = 0;
    bool greedy() const { return temperature <= 0.0f; }
    void validate() const;
};

// The uniform number of one draw: a function of (seed, request, step) and nothing else, so that
// what a request draws does not depend on which other requests share its batch.
float draw_uniform(uint64_t seed, uint64_t request, uint64_t step);

// ---- what the loop needs of an engine and of a sampler -----------------------------------------
struct StepItem {
    int slot;
    const int32_t* tokens;
    int n_tokens;
    bool want_last;                 // the logits of its last token are wanted
};

class LoopEngine {
public:
    virtual ~LoopEngine() {}
    virtual int open() = 0;
    virtual void close(int slot) = 0;
    // returns the logits of the wanted places (whatever the sampler understands by that)
    virtual const float* step(const std::vector<StepItem>& items, const int32_t* device_tokens) = 0;
    virtual long long max_tokens() const = 0;
    virtual long long max_positions() const = 0;
    virtual int max_slots() const = 0;
    virtual bool holds_pages() const { return true; }
    virtual bool takes_device_tokens() const { return false; }
};

// Tokens that have been chosen and may still be on their way to the host.
class Draw {
public:
    virtual ~Draw() {}
    virtual std::vector<int32_t> read() = 0;        // waits for this draw alone
};

class LoopSampler {
public:
    virtual ~LoopSampler() {}
    // rows: for each row of the logits the request's index in the batch; waits for the tokens
    virtual std::vector<int32_t> sample(const float* logits, const std::vector<int>& rows) = 0;
    // optional: start a draw without waiting, and name tokens of a draw on the device
    virtual bool runs_ahead() const { return false; }
    virtual std::unique_ptr<Draw> draw(const float* logits, const std::vector<int>& rows) { (void)logits; (void)rows; return nullptr; }
    virtual const int32_t* pick(Draw& draw, const std::vector<int>& places) { (void)draw; (void)places; return nullptr; }
};

using SamplerFactory = std::function<std::unique_ptr<LoopSampler>(const GenerationParams&, const std::vector<int>& request_ids)>;
using OnTokens = std::function<void(int n, const int32_t* requests, const int32_t* tokens)>;

// prompts: token ids of every request.  Returns for each the emitted token ids.  eos: stop tokens.
// max_step_tokens: most tokens one step runs; a batch's prompts are fed in as many steps as that
// takes, which bounds the step's working memory.
std::vector<std::vector<int32_t>> generate(LoopEngine& engine, const std::vector<std::vector<int32_t>>& prompts, const GenerationParams& params,
                                           const std::vector<int32_t>& eos, const OnTokens& on_tokens, int max_batch,
                                           const SamplerFactory& make_sampler, int max_step_tokens);

// ---- the real ones -------------------------------------------------------------------------------
class EngineForLoop : public LoopEngine {
public:
    EngineForLoop(Engine& e, hipStream_t stream) : e_(e), stream_(stream) {}
    int open() override { return e_.open(stream_); }
    void close(int slot) override { e_.close(slot); }
    const float* step(const std::vector<StepItem>& items, const int32_t* device_tokens) override;
    long long max_tokens() const override { return e_.max_tokens; }
    long long max_positions() const override { return e_.model->spec.max_positions; }
    int max_slots() const override { return e_.cache->max_slots; }
    bool holds_pages() const override { return e_.cache->holds_pages; }
    bool takes_device_tokens() const override { return true; }
private:
    Engine& e_;
    hipStream_t stream_;
};

// Choosing next tokens on the device for the live requests of a batch.  The reference samples one
// request on the host (src/engine.rs:353-373, 403-423): repeat penalty over the generated tokens
// (not on the first draw, when none exist), then argmax if temperature <= 0, else top-k then top-p
// at the temperature.  Here the same steps run as kernels on the rows of the step's logits; the
// history of generated tokens lives on the device and is appended to by a kernel.
class DeviceSampler : public LoopSampler {
public:
    DeviceSampler(const GenerationParams& params, const std::vector<int>& request_ids, int vocab, hipStream_t stream);
    ~DeviceSampler();
    std::vector<int32_t> sample(const float* logits, const std::vector<int>& rows) override;
    bool runs_ahead() const override { return true; }
    std::unique_ptr<Draw> draw(const float* logits, const std::vector<int>& rows) override;
    const int32_t* pick(Draw& draw, const std::vector<int>& places) override;
    static const int READ_AHEAD = 4;        // draws that may be unread at a time
private:
    GenerationParams p_;
    std::vector<int> request_ids_;
    std::vector<uint64_t> steps_;
    int vocab_;
    hipStream_t stream_;
    bool use_penalty_;
    Buffer hist_, hist_times_, hist_len_;
    int hist_cap_ = 0;
    // device buffers used in turn: one set per draw and one per pick, more sets than draws can be under way
    static const int RING = READ_AHEAD + 2;
    Buffer out_[RING], row_req_[RING], uniforms_[RING], pick_idx_[RING], picked_[RING], scratch_;
    size_t scratch_bytes_ = 0;
    void* landing_ = nullptr;               // pinned: READ_AHEAD rows of n tokens
    hipEvent_t events_[READ_AHEAD];
    int turn_ = 0, draw_turn_ = 0, pick_turn_ = 0;
    Staging staging_;
    bool null_ = false;
    friend class DeviceDraw;
};

}  // namespace tq
